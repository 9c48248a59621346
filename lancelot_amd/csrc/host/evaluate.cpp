// Evaluator: bookkeeping (chain index, scale, size, NTT form) and the order of device operations for the
// CKKS functions of cahel-main/include/evaluate.h / src/evaluate.cu: add/sub/negate (:15-284), multiply and
// square (:357-501, :1433-1483), plain operations (:1600-1784), relinearize (:2019-2056), rescale and
// modulus switching (:2058-2362), rotations, conjugation and hoisting (:2364-2702); key switching follows
// src/eval_key_switch.cu:80-216.  Error types and messages are the reference's.
#include <algorithm>
#include <cmath>

#include "cahel.h"

using namespace cahel;

namespace {

void require_ckks(const CAHELGPUContext &context) {
    if (context.scheme() != scheme_type::ckks) throw std::logic_error("unsupported scheme");
}

void check_same(const CAHELGPUCiphertext &a, const CAHELGPUCiphertext &b, bool need_same_size) {
    if (a.chain_index() != b.chain_index()) throw std::invalid_argument("encrypted1 and encrypted2 parameter mismatch");
    if (a.is_ntt_form() != b.is_ntt_form()) throw std::invalid_argument("NTT form mismatch");
    if (a.scale() != b.scale()) throw std::invalid_argument("scale mismatch");
    if (need_same_size && a.size() != b.size()) throw std::invalid_argument("poly number mismatch");
}

bool scale_within_bounds(const CAHELGPUContext &context, double scale, std::size_t chain_index) {
    const int bound = context.total_coeff_modulus_bit_count(chain_index);
    return !(scale <= 0 || (static_cast<int>(std::log2(scale)) >= bound));
}

}  // namespace

void negate_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted) {
    check_status(he_negate(context.handle(), encrypted.data(), encrypted.data(), (uint32_t)encrypted.size(),
                           (uint32_t)encrypted.coeff_modulus_size(), 0, context.stream()),
                 "he_negate");
}

void negate(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination) {
    if (&encrypted != &destination) destination = encrypted;
    negate_inplace(context, destination);
}

void add_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2) {
    check_same(encrypted1, encrypted2, true);
    check_status(he_add(context.handle(), encrypted1.data(), encrypted2.data(), encrypted1.data(),
                        (uint32_t)encrypted1.size(), (uint32_t)encrypted1.coeff_modulus_size(), 0, context.stream()),
                 "he_add");
}

void add(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
         CAHELGPUCiphertext &destination) {
    if (&encrypted2 == &destination) {
        add_inplace(context, destination, encrypted1);
    } else {
        if (&encrypted1 != &destination) destination = encrypted1;
        add_inplace(context, destination, encrypted2);
    }
}

void add_many(const CAHELGPUContext &context, const std::vector<CAHELGPUCiphertext> &encrypteds,
              CAHELGPUCiphertext &destination) {
    if (encrypteds.empty()) throw std::invalid_argument("encrypteds cannot be empty");
    for (auto &e : encrypteds)
        if (&e == &destination) throw std::invalid_argument("encrypteds must be different from destination");
    destination = encrypteds[0];
    for (std::size_t i = 1; i < encrypteds.size(); i++) add_inplace(context, destination, encrypteds[i]);
}

void sub_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
                 const bool &negate) {
    check_same(encrypted1, encrypted2, true);
    const uint32_t polys = (uint32_t)encrypted1.size(), limbs = (uint32_t)encrypted1.coeff_modulus_size();
    // negate: encrypted1 <- encrypted2 - encrypted1 (the aliasing case of sub(), include/evaluate.h:52-61)
    if (negate)
        check_status(he_sub(context.handle(), encrypted2.data(), encrypted1.data(), encrypted1.data(), polys, limbs, 0,
                            context.stream()),
                     "he_sub");
    else
        check_status(he_sub(context.handle(), encrypted1.data(), encrypted2.data(), encrypted1.data(), polys, limbs, 0,
                            context.stream()),
                     "he_sub");
}

void sub(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
         CAHELGPUCiphertext &destination) {
    if (&encrypted2 == &destination) {
        sub_inplace(context, destination, encrypted1, true);
    } else {
        if (&encrypted1 != &destination) destination = encrypted1;
        sub_inplace(context, destination, encrypted2, false);
    }
}

static void check_plain(const CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain, bool need_scale) {
    if (!encrypted.is_ntt_form() || !plain.is_ntt_form()) throw std::invalid_argument("NTT form mismatch");
    if (encrypted.chain_index() != plain.chain_index()) throw std::invalid_argument("encrypted and plain parameter mismatch");
    if (need_scale && encrypted.scale() != plain.scale()) throw std::invalid_argument("scale mismatch");
}

void add_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain) {
    check_plain(encrypted, plain, true);
    check_status(he_add(context.handle(), encrypted.data(), plain.data(), encrypted.data(), 1,
                        (uint32_t)encrypted.coeff_modulus_size(), 0, context.stream()),
                 "he_add");
}

void add_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
               CAHELGPUCiphertext &destination) {
    if (&encrypted != &destination) destination = encrypted;
    add_plain_inplace(context, destination, plain);
}

void sub_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain) {
    check_plain(encrypted, plain, true);
    check_status(he_sub(context.handle(), encrypted.data(), plain.data(), encrypted.data(), 1,
                        (uint32_t)encrypted.coeff_modulus_size(), 0, context.stream()),
                 "he_sub");
}

void sub_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
               CAHELGPUCiphertext &destination) {
    if (&encrypted != &destination) destination = encrypted;
    sub_plain_inplace(context, destination, plain);
}

void multiply_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain) {
    check_plain(encrypted, plain, false);
    const std::size_t n = context.poly_degree();
    const uint32_t limbs = (uint32_t)encrypted.coeff_modulus_size();
    for (std::size_t i = 0; i < encrypted.size(); i++) {
        uint64_t *ci = encrypted.data() + i * limbs * n;
        check_status(he_multiply(context.handle(), ci, plain.data(), ci, 1, limbs, 0, context.stream()), "he_multiply");
    }
    encrypted.scale() *= plain.scale();
    if (!scale_within_bounds(context, encrypted.scale(), encrypted.chain_index()))
        throw std::invalid_argument("scale out of bounds");
}

void multiply_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
                    CAHELGPUCiphertext &destination) {
    if (&encrypted != &destination) destination = encrypted;
    multiply_plain_inplace(context, destination, plain);
}

// destination = encrypted1 * encrypted2 as a size-3 ciphertext; destination may be either operand.  The product is
// written into a fresh block, so neither an in-place call nor a distinct destination costs a device copy.
static void multiply_into(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1,
                          const CAHELGPUCiphertext &encrypted2, CAHELGPUCiphertext &destination) {
    require_ckks(context);
    if (encrypted1.parms_id() != encrypted2.parms_id()) throw std::invalid_argument("encrypted1 and encrypted2 parameter mismatch");
    check_same(encrypted1, encrypted2, true);
    if (!(encrypted1.is_ntt_form() && encrypted2.is_ntt_form()))
        throw std::invalid_argument("encrypted1 or encrypted2 must be in NTT form");
    const std::size_t size1 = encrypted1.size(), size2 = encrypted2.size();
    if (size1 < 2 || size2 < 2) throw std::invalid_argument("ciphertext size must be at least 2");
    // the reference takes operands of any size (src/evaluate.cu:474-488: tensor_prod_mxn_rns_poly); here up to 16
    // polynomials each (he_tensor_mxn)
    if (size1 > 16 || size2 > 16) throw std::invalid_argument("ciphertext multiplication takes operands of at most 16 polynomials");
    const std::size_t dest_size = size1 + size2 - 1;
    const uint32_t L = (uint32_t)encrypted1.coeff_modulus_size();
    const std::size_t chain = encrypted1.chain_index(), n = encrypted1.poly_modulus_degree();
    const double scale = encrypted1.scale() * encrypted2.scale();
    DeviceBuffer product(dest_size * (std::size_t)L * n);
    if (dest_size != 3)
        check_status(he_tensor_mxn(context.handle(), encrypted1.data(), (uint32_t)size1, encrypted2.data(), (uint32_t)size2,
                                   product.get(), L, context.stream()),
                     "he_tensor_mxn");
    else if (&encrypted1 == &encrypted2)
        check_status(he_tensor_square(context.handle(), encrypted1.data(), product.get(), L, context.stream()),
                     "he_tensor_square");
    else
        check_status(he_tensor(context.handle(), encrypted1.data(), encrypted2.data(), product.get(), L, context.stream()),
                     "he_tensor");
    const bool asym = encrypted1.is_asymmetric_;
    const auto id = encrypted1.parms_id();
    destination.prng_seed_ = encrypted1.prng_seed_;   // the reference's `destination = encrypted1` carries it along
    destination.adopt(std::move(product));
    destination.size_ = dest_size;
    destination.coeff_modulus_size_ = L;
    destination.poly_modulus_degree_ = n;
    destination.chain_index() = chain;
    destination.parms_id() = id;
    destination.is_ntt_form() = true;
    destination.is_asymmetric_ = asym;
    destination.scale() = scale;
    if (!scale_within_bounds(context, scale, chain)) throw std::invalid_argument("scale out of bounds");
}

void multiply_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2) {
    multiply_into(context, encrypted1, encrypted2, encrypted1);
}

void multiply(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
              CAHELGPUCiphertext &destination) {
    multiply_into(context, encrypted1, encrypted2, destination);
}

void multiply_and_relin_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1,
                                const CAHELGPUCiphertext &encrypted2, const CAHELGPURelinKey &relin_keys) {
    multiply_inplace(context, encrypted1, encrypted2);
    relinearize_inplace(context, encrypted1, relin_keys);
}

void multiply_many(const CAHELGPUContext &, std::vector<CAHELGPUCiphertext> &, CAHELGPURelinKey &, CAHELGPUCiphertext &) {
    throw std::logic_error("unsupported scheme");  // BFV only in the reference (src/evaluate.cu:305-306)
}

// a size-3 operand goes through the general tensor product, as in the reference (src/evaluate.cu:531-545)
void square_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted) {
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("encrypted must be in NTT form");
    multiply_into(context, encrypted, encrypted, encrypted);
}

void square(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination) {
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("encrypted must be in NTT form");
    multiply_into(context, encrypted, encrypted, destination);
}

void exponentiate_inplace(const CAHELGPUContext &, CAHELGPUCiphertext &, uint64_t, CAHELGPURelinKey &) {
    throw std::logic_error("unsupported scheme");  // reaches multiply_many in the reference
}

void exponentiate(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, uint64_t exponent,
                  CAHELGPUCiphertext &destination, CAHELGPURelinKey &relin_key) {
    if (&encrypted != &destination) destination = encrypted;
    exponentiate_inplace(context, destination, exponent, relin_key);
}

// ct[0..1] += KeySwitch(c2) (src/eval_key_switch.cu:80-216)
void switch_key_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const uint64_t *c2,
                        const CAHELGPURelinKey &relin_keys, bool, uint32_t galois_elt) {
    if (relin_keys.parms_id() != context.key_parms_id())
        throw std::invalid_argument("relin_keys is not valid for encryption parameters");
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    if (encrypted.chain_index() == 0) throw std::invalid_argument("key switching needs a data-level ciphertext");
    const uint32_t L = (uint32_t)encrypted.coeff_modulus_size();
    auto ptrs = relin_keys.key_ptrs();
    const std::size_t beta = (L + context.size_p() - 1) / context.size_p();
    if (ptrs.size() < beta) throw std::invalid_argument("key_poly_num != 2");
    DeviceBuffer ws(he_keyswitch_workspace_words(context.handle(), L));
    check_status(he_keyswitch(context.handle(), L, c2, ptrs.data(), encrypted.data(), galois_elt, ws.get(), context.stream()),
                 "he_keyswitch");
}

// The key switch itself is deferred when the key's blocks can be kept alive (keys made by gen_relinkey or load):
// callers run rescale_to_next_inplace right after (lancelot-main-GPU/utils/byzantine_fl.py:254-256), and that call
// then does both in one device call (he_keyswitch_rescale, the same limbs); any other use of the ciphertext runs the
// switch first (CAHELGPUCiphertext::settle).  Every check is made here, as in the reference.
void relinearize_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPURelinKey &relin_keys) {
    if (encrypted.size() != 3) throw std::invalid_argument("destination_size must be 3");
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("CKKS encrypted must be in NTT form");
    const std::size_t poly = encrypted.coeff_modulus_size() * encrypted.poly_modulus_degree();
    const uint32_t L = (uint32_t)encrypted.coeff_modulus_size();
    const std::size_t beta = context.size_p() ? (L + context.size_p() - 1) / context.size_p() : 0;
    bool defer = relin_keys.parms_id() == context.key_parms_id() && context.using_keyswitching() &&
                 encrypted.chain_index() != 0 && relin_keys.public_keys_.size() >= beta;
    for (std::size_t d = 0; defer && d < beta; d++) defer = static_cast<bool>(relin_keys.public_keys_[d].pk_.data_.owner());
    if (!defer) {
        // (also every argument error: switch_key_inplace throws it)
        switch_key_inplace(context, encrypted, encrypted.data() + 2 * poly, relin_keys, true);
        encrypted.resize(2, encrypted.coeff_modulus_size(), encrypted.poly_modulus_degree());
        return;
    }
    (void)encrypted.data();   // (a size-3 ciphertext has nothing deferred; this keeps the invariant in one place)
    auto pending = std::make_shared<PendingKeySwitch>();
    pending->handle = context.handle();
    pending->limbs = L;
    for (std::size_t d = 0; d < beta; d++) {
        const DeviceBuffer &block = relin_keys.public_keys_[d].pk_.data_;
        pending->key_ptrs.push_back(block.get());
        pending->key_owners.push_back(block.owner());
    }
    encrypted.size_ = 2;
    encrypted.pending_ = std::move(pending);
}

// relinearize_inplace followed by rescale_to_next_inplace in one device call (he_keyswitch_rescale): the same limbs,
// one forward transform less.  Not in the reference; its callers run the two back to back
// (lancelot-main-GPU/utils/byzantine_fl.py:254-256).
void relinearize_rescale_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted,
                                 const CAHELGPURelinKey &relin_keys) {
    require_ckks(context);
    if (encrypted.size() != 3) throw std::invalid_argument("destination_size must be 3");
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("CKKS encrypted must be in NTT form");
    if (relin_keys.parms_id() != context.key_parms_id())
        throw std::invalid_argument("relin_keys is not valid for encryption parameters");
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    const std::size_t chain = encrypted.chain_index();
    if (chain == 0) throw std::invalid_argument("key switching needs a data-level ciphertext");
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");
    const std::size_t n = context.poly_degree();
    const uint32_t L = (uint32_t)encrypted.coeff_modulus_size();
    auto ptrs = relin_keys.key_ptrs();
    const std::size_t beta = (L + context.size_p() - 1) / context.size_p();
    if (ptrs.size() < beta) throw std::invalid_argument("key_poly_num != 2");
    DeviceBuffer ws(he_keyswitch_workspace_words(context.handle(), L)), out(2 * (std::size_t)(L - 1) * n);
    check_status(he_keyswitch_rescale(context.handle(), L, encrypted.data() + 2 * (std::size_t)L * n, ptrs.data(),
                                      encrypted.data(), out.get(), 0, ws.get(), context.stream()),
                 "he_keyswitch_rescale");
    const double scale = encrypted.scale() / static_cast<double>(context.key_modulus()[L - 1].value());
    encrypted.adopt(std::move(out));
    encrypted.size_ = 2;
    encrypted.coeff_modulus_size_ = L - 1;
    encrypted.poly_modulus_degree_ = n;
    encrypted.chain_index() = chain + 1;
    encrypted.parms_id() = context.parms_id_at(chain + 1);
    encrypted.scale() = scale;
}

// multiply + relinearize_inplace + rescale_to_next_inplace of two size-2 ciphertexts in one device call
// (he_multiply_relin_rescale): the same limbs as the three calls, with the tensor product formed inside the first
// pass of the key switch.  Not in the reference, whose callers run the three back to back (src/evaluate.cu:447-501,
// src/eval_key_switch.cu:80-216, src/evaluate.cu:2058-2085).
void multiply_relin_rescale(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1,
                            const CAHELGPUCiphertext &encrypted2, const CAHELGPURelinKey &relin_keys,
                            CAHELGPUCiphertext &destination) {
    require_ckks(context);
    if (encrypted1.parms_id() != encrypted2.parms_id()) throw std::invalid_argument("encrypted1 and encrypted2 parameter mismatch");
    check_same(encrypted1, encrypted2, true);
    if (!(encrypted1.is_ntt_form() && encrypted2.is_ntt_form()))
        throw std::invalid_argument("encrypted1 or encrypted2 must be in NTT form");
    if (encrypted1.size() != 2 || encrypted2.size() != 2)
        throw std::invalid_argument("multiply_relin_rescale takes size-2 operands");
    if (relin_keys.parms_id() != context.key_parms_id())
        throw std::invalid_argument("relin_keys is not valid for encryption parameters");
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    const std::size_t chain = encrypted1.chain_index();
    if (chain == 0) throw std::invalid_argument("key switching needs a data-level ciphertext");
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");
    const double product_scale = encrypted1.scale() * encrypted2.scale();
    if (!scale_within_bounds(context, product_scale, chain)) throw std::invalid_argument("scale out of bounds");
    const std::size_t n = context.poly_degree();
    const uint32_t L = (uint32_t)encrypted1.coeff_modulus_size();
    auto ptrs = relin_keys.key_ptrs();
    const std::size_t beta = (L + context.size_p() - 1) / context.size_p();
    if (ptrs.size() < beta) throw std::invalid_argument("key_poly_num != 2");
    DeviceBuffer ws(he_multiply_relin_rescale_workspace_words(context.handle(), L)), out(2 * (std::size_t)(L - 1) * n);
    check_status(he_multiply_relin_rescale(context.handle(), L, encrypted1.data(), encrypted2.data(), ptrs.data(), out.get(),
                                           ws.get(), context.stream()),
                 "he_multiply_relin_rescale");
    destination.is_ntt_form() = true;
    destination.is_asymmetric_ = encrypted1.is_asymmetric_;
    destination.prng_seed_ = encrypted1.prng_seed_;
    destination.adopt(std::move(out));
    destination.size_ = 2;
    destination.coeff_modulus_size_ = L - 1;
    destination.poly_modulus_degree_ = n;
    destination.chain_index() = chain + 1;
    destination.parms_id() = context.parms_id_at(chain + 1);
    destination.scale() = product_scale / static_cast<double>(context.key_modulus()[L - 1].value());
}

void relinearize(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination,
                 const CAHELGPURelinKey &relin_keys) {
    if (&encrypted != &destination) destination = encrypted;
    relinearize_inplace(context, destination, relin_keys);
}

// ---- modulus switching ----
void mod_switch_to_next(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUPlaintext &destination) {
    if (!plain.is_ntt_form()) throw std::invalid_argument("plain is not in NTT form");
    const std::size_t chain = plain.chain_index();
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");
    const std::size_t next = chain + 1, next_limbs = context.limbs_at(next), n = context.poly_degree();
    if (!scale_within_bounds(context, plain.scale(), next)) throw std::invalid_argument("scale out of bounds");
    // dropping the last limb of a single polynomial keeps the leading words in place
    DeviceBuffer fresh(next_limbs * n);
    check_status(he_memcpy_d2d(fresh.get(), plain.data(), next_limbs * n * sizeof(uint64_t), context.stream()), "copy");
    const double scale = plain.scale();
    destination.data_ = std::move(fresh);
    destination.coeff_modulus_size_ = next_limbs;
    destination.poly_modulus_degree_ = n;
    destination.chain_index() = next;
    destination.scale() = scale;
    destination.parms_id() = context.parms_id_at(next);
    destination.is_ntt_form_ = true;
}

void mod_switch_to_next_inplace(const CAHELGPUContext &context, CAHELGPUPlaintext &plain) {
    mod_switch_to_next(context, plain, plain);
}

void mod_switch_to_inplace(const CAHELGPUContext &context, CAHELGPUPlaintext &plain, std::size_t chain_index) {
    if (chain_index >= context.chain_size()) throw std::invalid_argument("chain index out of range");
    if (plain.chain_index() > chain_index) throw std::invalid_argument("cannot switch to higher level modulus");
    while (plain.chain_index() != chain_index) mod_switch_to_next_inplace(context, plain);
}

void mod_switch_to(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUPlaintext &destination,
                   std::size_t chain_index) {
    if (&plain != &destination) destination = plain;
    mod_switch_to_inplace(context, destination, chain_index);
}

void mod_switch_to_next(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                        CAHELGPUCiphertext &destination) {
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("CKKS encrypted must be in NTT form");
    const std::size_t chain = encrypted.chain_index();
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");
    const std::size_t next = chain + 1, n = context.poly_degree();
    const std::size_t limbs = encrypted.coeff_modulus_size(), next_limbs = context.limbs_at(next), size = encrypted.size();
    if (!scale_within_bounds(context, encrypted.scale(), next)) throw std::invalid_argument("scale out of bounds");
    DeviceBuffer fresh(size * next_limbs * n);
    for (std::size_t i = 0; i < size; i++)
        check_status(he_memcpy_d2d(fresh.get() + i * next_limbs * n, encrypted.data() + i * limbs * n,
                                   next_limbs * n * sizeof(uint64_t), context.stream()),
                     "copy");
    const double scale = encrypted.scale();
    const bool asym = encrypted.is_asymmetric_;
    destination.adopt(std::move(fresh));
    destination.size_ = size;
    destination.coeff_modulus_size_ = next_limbs;
    destination.poly_modulus_degree_ = n;
    destination.chain_index() = next;
    destination.parms_id() = context.parms_id_at(next);
    destination.scale() = scale;
    destination.is_ntt_form() = true;
    destination.is_asymmetric_ = asym;
}

void mod_switch_to_next_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted) {
    mod_switch_to_next(context, encrypted, encrypted);
}

void mod_switch_to_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t chain_index) {
    if (chain_index >= context.chain_size()) throw std::invalid_argument("chain index out of range");
    if (encrypted.chain_index() > chain_index) throw std::invalid_argument("cannot switch to higher level modulus");
    while (encrypted.chain_index() != chain_index) mod_switch_to_next_inplace(context, encrypted);
}

void mod_switch_to(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination,
                   std::size_t chain_index) {
    if (&encrypted != &destination) destination = encrypted;
    mod_switch_to_inplace(context, destination, chain_index);
}

void rescale_to_next(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination) {
    require_ckks(context);
    if (!encrypted.is_ntt_form()) throw std::invalid_argument("CKKS encrypted must be in NTT form");
    const std::size_t chain = encrypted.chain_index();
    if (chain == 0) throw std::invalid_argument("cannot rescale a key-level ciphertext");
    if (chain == context.max_chain_index()) throw std::invalid_argument("end of modulus switching chain reached");
    const std::size_t n = context.poly_degree(), size = encrypted.size();
    const uint32_t L = (uint32_t)encrypted.coeff_modulus_size();
    DeviceBuffer out(size * (L - 1) * n);
    if (const std::shared_ptr<PendingKeySwitch> pending = encrypted.pending_) {
        // a relinearisation is still due: both in one call, from the three polynomials that the block still holds
        const uint64_t *raw = encrypted.data_.get();
        DeviceBuffer ws(he_keyswitch_workspace_words(context.handle(), L));
        check_status(he_keyswitch_rescale(context.handle(), L, raw + 2 * (std::size_t)L * n, pending->key_ptrs.data(), raw,
                                          out.get(), 0, ws.get(), context.stream()),
                     "he_keyswitch_rescale");
    } else {
        DeviceBuffer ws(size * n);
        check_status(he_rescale(context.handle(), encrypted.data(), out.get(), (uint32_t)size, L, ws.get(), context.stream()),
                     "he_rescale");
    }
    const double scale = encrypted.scale() / static_cast<double>(context.key_modulus()[L - 1].value());
    const bool asym = encrypted.is_asymmetric_;
    destination.adopt(std::move(out));
    destination.size_ = size;
    destination.coeff_modulus_size_ = L - 1;
    destination.poly_modulus_degree_ = n;
    destination.chain_index() = chain + 1;
    destination.parms_id() = context.parms_id_at(chain + 1);
    destination.scale() = scale;
    destination.is_ntt_form() = true;
    destination.is_asymmetric_ = asym;
}

void rescale_to_next_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted) {
    rescale_to_next(context, encrypted, encrypted);
}

// ---- rotations ----
// destination = rotation of encrypted by the element at galois_elt_index; the two may be the same object.
// (sigma(c0), 0) + KeySwitch(sigma(c1)) is one device call that writes a fresh buffer, so a distinct destination
// costs no copy of the input.
static void apply_galois_into(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                              std::size_t galois_elt_index, const CAHELGPUGaloisKey &galois_keys,
                              CAHELGPUCiphertext &destination) {
    if (galois_keys.parms_id() != context.key_parms_id())
        throw std::invalid_argument("galois_keys is not valid for encryption parameters");
    if (encrypted.size() > 2) throw std::invalid_argument("encrypted size must be 2");
    if (galois_elt_index >= galois_keys.relin_keys_.size() || galois_elt_index >= context.galois_elts().size())
        throw std::invalid_argument("Galois key not present");
    const uint32_t elt = context.galois_elts()[galois_elt_index];
    const std::size_t n = context.poly_degree();
    const uint32_t L = (uint32_t)encrypted.coeff_modulus_size();
    const std::size_t poly = (std::size_t)L * n;
    const CAHELGPURelinKey &key = galois_keys.relin_keys_[galois_elt_index];
    if (key.parms_id() != context.key_parms_id())
        throw std::invalid_argument("relin_keys is not valid for encryption parameters");
    if (!context.using_keyswitching()) throw std::logic_error("keyswitching is not supported by the context");
    if (encrypted.chain_index() == 0) throw std::invalid_argument("key switching needs a data-level ciphertext");
    auto ptrs = key.key_ptrs();
    const std::size_t beta = (L + context.size_p() - 1) / context.size_p();
    if (ptrs.size() < beta) throw std::invalid_argument("key_poly_num != 2");
    DeviceBuffer rotated(2 * poly), ws(he_keyswitch_workspace_words(context.handle(), L));
    check_status(he_rotate(context.handle(), L, encrypted.data(), ptrs.data(), rotated.get(), elt, ws.get(),
                           context.stream()),
                 "he_rotate");
    if (&encrypted != &destination) {
        destination.size_ = encrypted.size_;
        destination.coeff_modulus_size_ = encrypted.coeff_modulus_size_;
        destination.poly_modulus_degree_ = encrypted.poly_modulus_degree_;
        destination.chain_index_ = encrypted.chain_index_;
        destination.parms_id_ = encrypted.parms_id_;
        destination.scale_ = encrypted.scale_;
        destination.is_ntt_form_ = encrypted.is_ntt_form_;
        destination.is_asymmetric_ = encrypted.is_asymmetric_;
    }
    destination.adopt(std::move(rotated));
}

void apply_galois_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t galois_elt_index,
                          const CAHELGPUGaloisKey &galois_keys) {
    apply_galois_into(context, encrypted, galois_elt_index, galois_keys, encrypted);
}

void apply_galois(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t galois_elt_index,
                  const CAHELGPUGaloisKey &galois_keys, CAHELGPUCiphertext &destination) {
    apply_galois_into(context, encrypted, galois_elt_index, galois_keys, destination);
}

// destination = encrypted rotated by `step`
static void rotate_internal(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, int step,
                            const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &destination) {
    if (galois_key.parms_id() != context.key_parms_id())
        throw std::invalid_argument("galois_keys is not valid for encryption parameters");
    if (step == 0) {
        if (&encrypted != &destination) destination = encrypted;
        return;
    }
    const std::size_t coeff_count = context.poly_degree();
    const long idx = context.find_galois_elt(context.get_elt_from_step(step));
    if (idx >= 0) {
        apply_galois_into(context, encrypted, (std::size_t)idx, galois_key, destination);
        return;
    }
    // no key for this step: split it into signed powers of two (src/evaluate.cu:2395-2408)
    const std::vector<int> parts = naf(step);
    if (parts.size() == 1) throw std::invalid_argument("Galois key not present");
    const CAHELGPUCiphertext *src = &encrypted;
    for (int part : parts) {
        if (static_cast<std::size_t>(std::abs(part)) == (coeff_count >> 1)) continue;
        rotate_internal(context, *src, part, galois_key, destination);
        src = &destination;
    }
    if (src == &encrypted && &encrypted != &destination) destination = encrypted;
}

static void conjugate_internal(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                               const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &destination) {
    if (galois_key.parms_id() != context.key_parms_id())
        throw std::invalid_argument("galois_keys is not valid for encryption parameters");
    // the reference uses element index 0, which holds 2N-1 in the default element list (src/evaluate.cu:2690-2702)
    const long idx = context.find_galois_elt((uint32_t)(2 * context.poly_degree() - 1));
    if (idx < 0) throw std::invalid_argument("Galois key not present");
    apply_galois_into(context, encrypted, (std::size_t)idx, galois_key, destination);
}

void rotate_rows_inplace(const CAHELGPUContext &, CAHELGPUCiphertext &, int, const CAHELGPUGaloisKey &) {
    throw std::logic_error("unsupported scheme");  // BFV/BGV only (include/evaluate.h:501-509)
}

void rotate_rows(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int steps,
                 const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &) {
    rotate_rows_inplace(context, encrypted, steps, galois_key);
}

void rotate_columns_inplace(const CAHELGPUContext &, CAHELGPUCiphertext &, const CAHELGPUGaloisKey &) {
    throw std::logic_error("unsupported scheme");  // BFV/BGV only (include/evaluate.h:527-535)
}

void rotate_columns(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUGaloisKey &galois_key,
                    CAHELGPUCiphertext &) {
    rotate_columns_inplace(context, encrypted, galois_key);
}

void rotate_vector_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int step,
                           const CAHELGPUGaloisKey &galois_key) {
    require_ckks(context);
    rotate_internal(context, encrypted, step, galois_key, encrypted);
}

void rotate_vector(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int step,
                   const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &destination) {
    require_ckks(context);
    rotate_internal(context, encrypted, step, galois_key, destination);
}

void complex_conjugate_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted,
                               const CAHELGPUGaloisKey &galois_key) {
    require_ckks(context);
    conjugate_internal(context, encrypted, galois_key, encrypted);
}

void complex_conjugate(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUGaloisKey &galois_key,
                       CAHELGPUCiphertext &destination) {
    require_ckks(context);
    conjugate_internal(context, encrypted, galois_key, destination);
}

// sum over steps of rot(ct, step) with one ModUp of c1 and one ModDown pair (src/evaluate.cu:2412-2629)
static void hoisting_into(const CAHELGPUContext &context, const CAHELGPUCiphertext &ct, const CAHELGPUGaloisKey &glk,
                          const std::vector<int> &steps, CAHELGPUCiphertext &destination) {
    if (ct.size() > 2) throw std::invalid_argument("ciphertext size must be 2");
    if (steps.empty()) throw std::invalid_argument("steps cannot be empty");
    if (glk.parms_id() != context.key_parms_id())
        throw std::invalid_argument("galois_keys is not valid for encryption parameters");
    if (!context.using_keyswitching() || ct.chain_index() == 0)
        throw std::logic_error("keyswitching is not supported by the context");
    he_context *h = context.handle();
    he_stream st = context.stream();
    const std::size_t n = context.poly_degree(), K = context.size_p();
    const uint32_t L = (uint32_t)ct.coeff_modulus_size();
    const std::size_t poly = (std::size_t)L * n, beta = (L + K - 1) / K;
    std::vector<std::size_t> idxs;
    for (int s : steps) {
        const long idx = context.find_galois_elt(context.get_elt_from_step(s));
        if (idx < 0 || (std::size_t)idx >= glk.relin_keys_.size()) throw std::logic_error("Galois key not present in hoisting");
        idxs.push_back((std::size_t)idx);
    }
    // every step's key pointers, step-major, and its Galois element
    std::vector<const uint64_t *> ptrs;
    std::vector<uint32_t> elts;
    for (std::size_t idx : idxs) {
        auto key = glk.relin_keys_[idx].key_ptrs();
        if (key.size() < beta) throw std::invalid_argument("key_poly_num must be 2 in hoisting");
        ptrs.insert(ptrs.end(), key.begin(), key.begin() + beta);
        elts.push_back(context.galois_elts()[idx]);
    }
    // new c0 = sum sigma(c0) + ModDown(acc_0), new c1 = ModDown(acc_1): one device call into a fresh buffer
    DeviceBuffer sum(2 * poly), ws(he_keyswitch_workspace_words(h, L));
    check_status(he_hoisted_rotations(h, L, ct.data(), ptrs.data(), elts.data(), (uint32_t)elts.size(), sum.get(),
                                      ws.get(), st),
                 "he_hoisted_rotations");
    if (&ct != &destination) {
        destination.size_ = ct.size_;
        destination.coeff_modulus_size_ = ct.coeff_modulus_size_;
        destination.poly_modulus_degree_ = ct.poly_modulus_degree_;
        destination.chain_index_ = ct.chain_index_;
        destination.parms_id_ = ct.parms_id_;
        destination.scale_ = ct.scale_;
        destination.is_ntt_form_ = ct.is_ntt_form_;
        destination.is_asymmetric_ = ct.is_asymmetric_;
    }
    destination.adopt(std::move(sum));
}

void hoisting_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &ct, const CAHELGPUGaloisKey &glk,
                      const std::vector<int> &steps) {
    hoisting_into(context, ct, glk, steps, ct);
}

CAHELGPUCiphertext hoisting(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                            const CAHELGPUGaloisKey &glk, const std::vector<int> &steps) {
    CAHELGPUCiphertext destination;
    hoisting_into(context, encrypted, glk, steps, destination);
    return destination;
}
