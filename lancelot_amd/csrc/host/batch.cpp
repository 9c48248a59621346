// Batched evaluation for callers that hold many small independent ciphertexts (Lancelot's have three or four limbs:
// one of them neither fills the GPU nor amortises a kernel launch).  Not in the reference, which evaluates one
// ciphertext per call; every item goes through the same arithmetic as the single-ciphertext functions, so its limbs
// equal theirs.
#include <cmath>
#include <stdexcept>

#include "cahel.h"

using cahel::check_status;
using cahel::DeviceBuffer;

// For every (i, j) of `pairs`: acc = sum over chunks of (clients[j][c] - clients[i][c])^2, relinearised and rescaled,
// then for every round acc += sum over the round's steps of rot(acc, step) (hoisted), as
// GPU_compute_pair_distance does per pair (lancelot-main-GPU/utils/byzantine_fl.py:173-321) -- here with one
// launch per stage for all pairs.  scale > 0 overrides the scale after the rescale (the reference's set_scale).
// drop_levels > 0 switches the rescaled ciphertexts down by that many further limbs without scaling
// (mod_switch_to_next) before the slot sum, whose key switches then run over fewer limbs.
std::vector<CAHELGPUCiphertext> pair_square_distances(
    const CAHELGPUContext &context, const std::vector<std::vector<const CAHELGPUCiphertext *>> &clients,
    const std::vector<std::pair<std::size_t, std::size_t>> &pairs, const CAHELGPURelinKey &rlk,
    const CAHELGPUGaloisKey &glk, const std::vector<std::vector<int>> &rounds, double scale, std::size_t drop_levels) {
    if (context.scheme() != cahel::scheme_type::ckks) throw std::logic_error("unsupported scheme");
    if (clients.empty() || clients[0].empty()) throw std::invalid_argument("no ciphertexts");
    if (pairs.empty()) return {};
    if (pairs.size() > 16384) throw std::invalid_argument("too many pairs");
    const CAHELGPUCiphertext &first = *clients[0][0];
    const std::size_t chunks = clients[0].size();
    for (const auto &client : clients) {
        if (client.size() != chunks) throw std::invalid_argument("clients differ in their number of chunks");
        for (const CAHELGPUCiphertext *ct : client) {
            if (!ct || ct->size() != 2 || !ct->is_ntt_form()) throw std::invalid_argument("encrypted is not valid");
            if (ct->parms_id() != first.parms_id() || ct->chain_index() != first.chain_index())
                throw std::invalid_argument("encrypted parameter mismatch");
            if (ct->scale() != first.scale()) throw std::invalid_argument("scale mismatch");
        }
    }
    for (const auto &pr : pairs)
        if (pr.first >= clients.size() || pr.second >= clients.size()) throw std::invalid_argument("pair out of range");
    if (rlk.parms_id() != context.key_parms_id() || glk.parms_id() != context.key_parms_id())
        throw std::invalid_argument("keys are not valid for encryption parameters");
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    const std::size_t chain = first.chain_index();
    if (chain == 0) throw std::invalid_argument("key switching needs a data-level ciphertext");
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");

    he_context *h = context.handle();
    he_stream st = context.stream();
    const std::size_t n = context.poly_degree(), K = context.size_p();
    const uint32_t L = (uint32_t)first.coeff_modulus_size(), items = (uint32_t)pairs.size();

    // (1) squared differences, summed over the chunks, as size-3 ciphertexts (lazy relinearisation)
    std::vector<const uint64_t *> table;
    table.reserve((std::size_t)items * chunks * 2);
    for (const auto &pr : pairs)
        for (std::size_t c = 0; c < chunks; c++) {
            table.push_back(clients[pr.second][c]->data());
            table.push_back(clients[pr.first][c]->data());
        }
    DeviceBuffer d_table(table.size());
    check_status(he_memcpy_h2d(d_table.get(), table.data(), table.size() * sizeof(uint64_t), st), "upload");
    DeviceBuffer d01((std::size_t)items * 2 * L * n), d2((std::size_t)items * L * n);
    check_status(he_pair_square_sum(h, L, items, (uint32_t)chunks, reinterpret_cast<const uint64_t *const *>(d_table.get()),
                                    d01.get(), d2.get(), st),
                 "he_pair_square_sum");

    // (2) relinearise + rescale
    auto rl = rlk.key_ptrs();
    if (rl.size() < (L + K - 1) / K) throw std::invalid_argument("key_poly_num != 2");
    DeviceBuffer ws(he_keyswitch_batch_workspace_words(h, L, items));
    DeviceBuffer acc((std::size_t)items * 2 * (L - 1) * n);
    check_status(he_keyswitch_rescale_batch(h, L, items, d2.get(), L, rl.data(), d01.get(), acc.get(), 0, ws.get(), st),
                 "he_keyswitch_rescale_batch");
    double out_scale = first.scale() * first.scale() / static_cast<double>(context.key_modulus()[L - 1].value());
    if (scale > 0) out_scale = scale;

    // (2b) optional: drop limbs without scaling, the leading limbs of every polynomial move to a denser batch
    uint32_t L1 = L - 1;
    std::size_t out_chain = chain + 1;
    if (drop_levels) {
        if (drop_levels >= L1) throw std::invalid_argument("end of modulus switching chain reached");
        const uint32_t L2 = L1 - (uint32_t)drop_levels;
        DeviceBuffer dense((std::size_t)items * 2 * L2 * n);
        check_status(he_memcpy2d_d2d(dense.get(), (std::size_t)L2 * n * sizeof(uint64_t), acc.get(),
                                     (std::size_t)L1 * n * sizeof(uint64_t), (std::size_t)L2 * n * sizeof(uint64_t),
                                     (std::size_t)items * 2, st),
                     "he_memcpy2d_d2d");
        acc = std::move(dense);
        L1 = L2;
        out_chain += drop_levels;
    }

    // (3) the slot sum, one hoisted round at a time: acc += sum_s rot(acc, s)
    const std::size_t beta = (L1 + K - 1) / K;
    DeviceBuffer next(rounds.empty() ? 0 : (std::size_t)items * 2 * L1 * n);
    for (const auto &steps : rounds) {
        if (steps.empty()) throw std::invalid_argument("steps cannot be empty");
        std::vector<const uint64_t *> ptrs;
        std::vector<uint32_t> elts;
        for (int s : steps) {
            const long idx = context.find_galois_elt(context.get_elt_from_step(s));
            if (idx < 0 || (std::size_t)idx >= glk.relin_keys_.size())
                throw std::logic_error("Galois key not present in hoisting");
            auto key = glk.relin_keys_[(std::size_t)idx].key_ptrs();
            if (key.size() < beta) throw std::invalid_argument("key_poly_num must be 2 in hoisting");
            ptrs.insert(ptrs.end(), key.begin(), key.begin() + beta);
            elts.push_back(context.galois_elts()[(std::size_t)idx]);
        }
        check_status(he_hoisted_rotations_batch(h, L1, items, acc.get(), ptrs.data(), elts.data(), (uint32_t)elts.size(), 1,
                                                next.get(), ws.get(), st),
                     "he_hoisted_rotations_batch");
        std::swap(acc, next);
    }

    // (4) one ciphertext object per pair, each a slice of the batch (no copies)
    std::vector<CAHELGPUCiphertext> out(items);
    const std::size_t words = 2 * (std::size_t)L1 * n;
    auto shared = std::make_shared<DeviceBuffer>(std::move(acc));
    for (uint32_t k = 0; k < items; k++) {
        CAHELGPUCiphertext &ct = out[k];
        ct.adopt(DeviceBuffer::slice(shared, k * words, words));
        ct.size_ = 2;
        ct.coeff_modulus_size_ = L1;
        ct.poly_modulus_degree_ = n;
        ct.chain_index_ = out_chain;
        ct.parms_id_ = context.parms_id_at(out_chain);
        ct.scale_ = out_scale;
        ct.is_ntt_form_ = true;
        ct.is_asymmetric_ = first.is_asymmetric_;
    }
    return out;
}
