// Keys, encryption and decryption.  Order of operations follows cahel-main/src/secretkey.cu
// (gen_secretkey :254-282, encrypt_zero_symmetric :451-515, generate_one_kswitch_key :328-372, gen_relinkey
// :374-396, create_galois_keys :398-442, encrypt_zero_asymmetric :47-117 and its ModDown :126-170,
// ckks_decrypt :594-654).  Randomness comes from the context's seeded ChaCha20 streams, one stream id per
// sampled polynomial, handed out in the order the polynomials are drawn.
#include <cmath>
#include <string>

#include "cahel.h"

using namespace cahel;

namespace {

void sample(const CAHELGPUContext &c, int kind, uint64_t *out, uint32_t limbs, uint32_t split, uint32_t tail) {
    check_status(he_sample(c.handle(), kind, c.prng_key(), c.next_stream(), out, limbs, 0, split, tail, c.gauss_cdt(),
                           c.gauss_cdt_len(), c.stream()),
                 "he_sample");
}

// limb layout of a polynomial at chain_index: chain 0 = all of Q u P, otherwise the first L limbs of Q
struct Layout {
    uint32_t limbs, split, tail;
};

Layout layout_of(const CAHELGPUContext &c, std::size_t chain_index) {
    const uint32_t limbs = (uint32_t)c.limbs_at(chain_index);
    return Layout{limbs, limbs, 0};
}

}  // namespace

CAHELGPURelinKey::CAHELGPURelinKey(const CAHELGPUContext &context) {
    if (context.size_p()) pk_num_ = context.size_q() / context.size_p();  // include/secretkey.h:141-144
}

std::vector<const uint64_t *> CAHELGPURelinKey::key_ptrs() const {
    std::vector<const uint64_t *> p;
    for (auto &k : public_keys_) p.push_back(k.pk_.data());
    return p;
}

CAHELGPUSecretKey::CAHELGPUSecretKey(const EncryptionParameters &params) {
    poly_modulus_degree_ = params.poly_modulus_degree();
    coeff_modulus_size_ = params.coeff_modulus().size();
}

void CAHELGPUSecretKey::gen_secretkey(const CAHELGPUContext &context) {
    const std::size_t n = context.poly_degree(), qp = context.size_qp();
    poly_modulus_degree_ = n;
    coeff_modulus_size_ = qp;
    sk_powers_.allocate(qp * n);
    sample(context, 0, sk_powers_.get(), (uint32_t)qp, (uint32_t)qp, 0);
    check_status(he_ntt_forward(context.handle(), sk_powers_.get(), 1, (uint32_t)qp, (uint32_t)qp, 0, (uint32_t)qp, 0,
                                context.stream()),
                 "he_ntt_forward");
    sk_max_power_ = 1;
    gen_flag_ = true;
}

void CAHELGPUSecretKey::compute_secret_key_array(const CAHELGPUContext &context, std::size_t max_power) {
    if (!gen_flag_) throw std::logic_error("cannot generate relinearization keys for unspecified secret key");
    if (max_power <= 1 || max_power <= sk_max_power_) return;
    const std::size_t n = poly_modulus_degree_, qp = coeff_modulus_size_, poly = qp * n;
    DeviceBuffer grown(max_power * poly);
    check_status(he_memcpy_d2d(grown.get(), sk_powers_.get(), sk_max_power_ * poly * sizeof(uint64_t), context.stream()),
                 "copy");
    for (std::size_t p = sk_max_power_; p < max_power; p++)
        check_status(he_multiply(context.handle(), grown.get() + (p - 1) * poly, grown.get(), grown.get() + p * poly, 1,
                                 (uint32_t)qp, 0, context.stream()),
                     "he_multiply");
    sk_powers_ = std::move(grown);
    sk_max_power_ = max_power;
}

void CAHELGPUSecretKey::encrypt_zero_symmetric(const CAHELGPUContext &context, CAHELGPUCiphertext &cipher,
                                               std::size_t chain_index) const {
    if (!gen_flag_) throw std::logic_error("secret key has not been generated");
    const std::size_t n = context.poly_degree();
    const Layout lay = layout_of(context, chain_index);
    cipher.resize(context, chain_index, 2);
    cipher.is_ntt_form() = true;
    cipher.scale() = 1.0;
    uint64_t *c0 = cipher.data(), *c1 = c0 + (std::size_t)lay.limbs * n;
    DeviceBuffer e((std::size_t)lay.limbs * n);
    sample(context, 1, e.get(), lay.limbs, lay.split, lay.tail);
    check_status(he_ntt_forward(context.handle(), e.get(), 1, lay.limbs, lay.limbs, 0, lay.split, lay.tail, context.stream()),
                 "he_ntt_forward");
    sample(context, 2, c1, lay.limbs, lay.split, lay.tail);
    // c0 = -(a s + e)
    check_status(he_multiply_add(context.handle(), c1, sk_powers_.get(), e.get(), c0, 1, lay.limbs, 0, 1, context.stream()),
                 "he_multiply_add");
}

void CAHELGPUSecretKey::gen_publickey(const CAHELGPUContext &context, CAHELGPUPublicKey &pk, bool) const {
    encrypt_zero_symmetric(context, pk.pk_, 0);
    pk.pk_.parms_id() = context.key_parms_id();
    pk.gen_flag_ = true;
}

void CAHELGPUSecretKey::generate_one_kswitch_key(const CAHELGPUContext &context, const uint64_t *new_key,
                                                 CAHELGPURelinKey &relin_key) const {
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    const std::size_t n = context.poly_degree(), alpha = context.size_p();
    const std::size_t dnum = context.size_q() / alpha;
    relin_key.pk_num_ = dnum;
    relin_key.public_keys_.clear();
    relin_key.public_keys_.resize(dnum);
    for (std::size_t d = 0; d < dnum; d++) gen_publickey(context, relin_key.public_keys_[d], false);
    for (std::size_t d = 0; d < dnum; d++) {
        uint64_t *b = relin_key.public_keys_[d].pk_.data() + d * alpha * n;  // c0, limbs of digit d
        check_status(he_add_p_multiple(context.handle(), b, new_key + d * alpha * n, b, (uint32_t)(d * alpha),
                                       (uint32_t)alpha, context.stream()),
                     "he_add_p_multiple");
    }
    // shared ownership of the digits' blocks: a deferred relinearisation keeps them alive (relinearize_inplace)
    for (auto &pk : relin_key.public_keys_) pk.pk_.data_.make_shared();
    relin_key.gen_flag_ = true;
    relin_key.parms_id_ = context.key_parms_id();
}

void CAHELGPUSecretKey::gen_relinkey(const CAHELGPUContext &context, CAHELGPURelinKey &relin_key, bool) {
    if (!gen_flag_) throw std::logic_error("cannot generate relinearization keys for unspecified secret key");
    compute_secret_key_array(context, 2);
    const uint64_t *sk_square = sk_powers_.get() + coeff_modulus_size_ * poly_modulus_degree_;
    generate_one_kswitch_key(context, sk_square, relin_key);
}

void CAHELGPUSecretKey::create_galois_keys(const CAHELGPUContext &context, CAHELGPUGaloisKey &galois_keys, bool) const {
    if (!gen_flag_) throw std::logic_error("cannot generate relinearization keys for unspecified secret key");
    const auto &elts = context.galois_elts();
    const std::size_t qp = context.size_qp(), n = context.poly_degree();
    DeviceBuffer rotated(qp * n);
    galois_keys.relin_key_num_ = elts.size();
    galois_keys.relin_keys_.clear();
    galois_keys.relin_keys_.resize(elts.size());
    for (std::size_t i = 0; i < elts.size(); i++) {
        check_status(he_galois_ntt(context.handle(), sk_powers_.get(), rotated.get(), (uint32_t)qp, elts[i], context.stream()),
                     "he_galois_ntt");
        generate_one_kswitch_key(context, rotated.get(), galois_keys.relin_keys_[i]);
    }
    galois_keys.parms_id_ = context.key_parms_id();
    galois_keys.gen_flag_ = true;
}

void CAHELGPUSecretKey::encrypt_symmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                          CAHELGPUCiphertext &cipher, bool) const {
    if (!plain.is_ntt_form()) throw std::invalid_argument("CKKS plain must be in NTT form");
    encrypt_zero_symmetric(context, cipher, plain.chain_index());
    const uint32_t limbs = (uint32_t)context.limbs_at(plain.chain_index());
    check_status(he_add(context.handle(), cipher.data(), plain.data(), cipher.data(), 1, limbs, 0, context.stream()), "he_add");
    cipher.scale() = plain.scale();
}

void CAHELGPUPublicKey::encrypt_asymmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                           CAHELGPUCiphertext &cipher, bool) const {
    if (!gen_flag_) throw std::logic_error("public key has not been generated");
    if (!plain.is_ntt_form()) throw std::invalid_argument("CKKS plain must be in NTT form");
    const std::size_t chain = plain.chain_index();
    const std::size_t n = context.poly_degree(), Q = context.size_q(), K = context.size_p(), QP = Q + K;
    he_context *h = context.handle();
    he_stream st = context.stream();
    if (chain == 0 || K == 0) {
        // key level (or a context without special primes): c_i = u pk_i + e_i, no modulus switch
        const uint32_t limbs = (uint32_t)context.limbs_at(chain);
        cipher.resize(context, chain, 2);
        DeviceBuffer u((std::size_t)limbs * n);
        sample(context, 0, u.get(), limbs, limbs, 0);
        check_status(he_ntt_forward(h, u.get(), 1, limbs, limbs, 0, limbs, 0, st), "he_ntt_forward");
        for (int i = 0; i < 2; i++) {
            uint64_t *ci = cipher.data() + (std::size_t)i * limbs * n;
            sample(context, 1, ci, limbs, limbs, 0);
            check_status(he_ntt_forward(h, ci, 1, limbs, limbs, 0, limbs, 0, st), "he_ntt_forward");
            check_status(he_multiply_add(h, u.get(), pk_.data() + (std::size_t)i * QP * n, ci, ci, 1, limbs, 0, 0, st),
                         "he_multiply_add");
        }
        check_status(he_add(h, cipher.data(), plain.data(), cipher.data(), 1, limbs, 0, st), "he_add");
    } else {
        // encrypt over Ql u P, then divide by P (ModDown) onto the L limbs of the plaintext's level: the batched
        // pipeline with one item (u, e0, e1 from the next three stream ids; the plaintext lies in polynomial 0 and the
        // division adds onto it)
        const uint32_t L = (uint32_t)context.limbs_at(chain);
        cipher.resize(context, chain, 2);
        check_status(he_memcpy_d2d(cipher.data(), plain.data(), (std::size_t)L * n * sizeof(uint64_t), st), "copy");
        DeviceBuffer ws(he_encrypt_batch_workspace_words(h, L, 1));
        check_status(he_encrypt_batch(h, L, 1, pk_.data(), context.prng_key(), context.next_stream(3), cipher.data(),
                                      ws.get(), st),
                     "he_encrypt_batch");
    }
    cipher.is_ntt_form() = true;
    cipher.is_asymmetric() = true;
    cipher.scale() = plain.scale();
}

void CAHELGPUSecretKey::decrypt(const CAHELGPUContext &context, const CAHELGPUCiphertext &cipher, CAHELGPUPlaintext &plain) {
    if (!gen_flag_) throw std::logic_error("secret key has not been generated");
    if (!cipher.is_ntt_form()) throw std::invalid_argument("encrypted must be in NTT form");
    if (cipher.size() < 2) throw std::invalid_argument("encrypted is not valid");
    const std::size_t n = context.poly_degree();
    const uint32_t limbs = (uint32_t)cipher.coeff_modulus_size();
    const std::size_t poly = (std::size_t)limbs * n, sk_poly = coeff_modulus_size_ * poly_modulus_degree_;
    const std::size_t needed = cipher.size() - 1;
    if (needed > sk_max_power_) compute_secret_key_array(context, needed);
    he_context *h = context.handle();
    he_stream st = context.stream();
    plain.resize(limbs, n);
    // c0 + c1 s (+ c2 s^2 ...): the first product reads c0 directly
    for (std::size_t i = 1; i <= needed; i++)
        check_status(he_multiply_add(h, cipher.data() + i * poly, sk_powers_.get() + (i - 1) * sk_poly,
                                     i == 1 ? cipher.data() : plain.data(), plain.data(), 1, limbs, 0, 0, st),
                     "he_multiply_add");
    if (noise_flooding_) {
        DeviceBuffer noise(poly);
        sample(context, 3, noise.get(), limbs, limbs, 0);
        check_status(he_ntt_forward(h, noise.get(), 1, limbs, limbs, 0, limbs, 0, st), "he_ntt_forward");
        check_status(he_add(h, plain.data(), noise.get(), plain.data(), 1, limbs, 0, st), "he_add");
    }
    plain.chain_index() = cipher.chain_index();
    plain.scale() = cipher.scale();
    plain.parms_id() = cipher.parms_id();
    plain.is_ntt_form_ = true;
}

std::vector<double> CAHELGPUSecretKey::decrypt_decode_many(const CAHELGPUContext &context,
                                                           const std::vector<const CAHELGPUCiphertext *> &ciphers,
                                                           std::size_t slots, std::size_t count) {
    if (!gen_flag_) throw std::logic_error("secret key has not been generated");
    if (ciphers.empty()) return {};
    if (ciphers.size() > 16384) throw std::invalid_argument("too many ciphertexts");
    const CAHELGPUCiphertext &first = *ciphers[0];
    for (const CAHELGPUCiphertext *ct : ciphers) {
        if (!ct || ct->size() != 2 || !ct->is_ntt_form()) throw std::invalid_argument("encrypted is not valid");
        if (ct->parms_id() != first.parms_id() || ct->chain_index() != first.chain_index() || ct->scale() != first.scale())
            throw std::invalid_argument("encrypted parameter mismatch");
    }
    const std::size_t n = context.poly_degree();
    const uint32_t limbs = (uint32_t)first.coeff_modulus_size(), items = (uint32_t)ciphers.size();
    if (slots < 2 || (slots & (slots - 1)) || slots > n / 2 || count == 0 || count > slots)
        throw std::invalid_argument("slot count out of range");
    const int total_bits = context.total_coeff_modulus_bit_count(first.chain_index());
    if (first.scale() <= 0 || (static_cast<int>(std::log2(first.scale())) >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    he_context *h = context.handle();
    he_stream st = context.stream();
    std::vector<const uint64_t *> table;
    for (const CAHELGPUCiphertext *ct : ciphers) table.push_back(ct->data());
    DeviceBuffer d_table(items);
    check_status(he_memcpy_h2d(d_table.get(), table.data(), table.size() * sizeof(uint64_t), st), "upload");
    DeviceBuffer noise;
    if (noise_flooding_) {
        // one flooding-noise polynomial per ciphertext, the stream ids that `items` calls of decrypt would draw
        noise.allocate((std::size_t)items * limbs * n);
        check_status(he_sample_batch(h, 3, context.prng_key(), context.next_stream(items), noise.get(), limbs, 0, limbs, 0,
                                     context.gauss_cdt(), context.gauss_cdt_len(), items, st),
                     "he_sample_batch");
        check_status(he_ntt_forward(h, noise.get(), items, limbs, limbs, 0, limbs, 0, st), "he_ntt_forward");
    }
    DeviceBuffer ws(he_decrypt_decode_batch_workspace_words(h, limbs, (uint32_t)slots, items));
    DeviceBuffer out(2 * (std::size_t)items * count);
    check_status(he_decrypt_decode_batch(h, reinterpret_cast<const uint64_t *const *>(d_table.get()), items, limbs,
                                         sk_powers_.get(), noise.get(), (uint32_t)slots, first.scale(), (uint32_t)count,
                                         reinterpret_cast<double *>(out.get()), ws.get(), st),
                 "he_decrypt_decode_batch");
    std::vector<double> v(2 * (std::size_t)items * count);
    check_status(he_memcpy_d2h(v.data(), out.get(), v.size() * sizeof(double), st), "download");
    std::vector<double> re((std::size_t)items * count);
    for (std::size_t i = 0; i < re.size(); i++) re[i] = v[2 * i];
    return re;
}
