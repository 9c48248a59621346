// Host-side API of the CKKS engine: the SEAL-style objects and free evaluator functions that CAHEL exposes
// (cahel-main/include/cahel.h:1-12 -> gpucontext.h, ciphertext.h, plaintext.h, secretkey.h, ckks.h,
// evaluate.h), re-implemented for MI355X.  This layer is plain C++17: it owns parameters, bookkeeping and
// the order of operations, and reaches the GPU only through the C-ABI of include/cahel_hip.h.
//
// Only the CKKS scheme is implemented; BFV/BGV entry points exist (the Python binding exports their
// names) and throw std::logic_error("unsupported scheme") the way the reference does for the scheme it
// is not running (src/evaluate.cu:305-306, include/evaluate.h:501-535).
#pragma once
#include <array>
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <iosfwd>
#include <memory>
#include <stdexcept>
#include <utility>
#include <vector>

#include "cahel_hip.h"
#include "hostmath.h"

namespace cahel {

enum class scheme_type : std::uint8_t { none = 0, bgv = 1, bfv = 2, ckks = 3 };
enum class mul_tech_type : std::uint8_t { none = 0, behz = 1, hps = 2, hps_overq = 3, hps_overq_leveled = 4 };
enum class sec_level_type : int { none = 0, tc128 = 128, tc192 = 192, tc256 = 256 };

// 256-bit BLAKE2b digest of the parameter words (include/util/hash.h:22-37)
using parms_id_type = std::array<std::uint64_t, 4>;
constexpr parms_id_type parms_id_zero{{0, 0, 0, 0}};
// The words the reference hashes (include/util/encryptionparams.h:337-379): scheme, degree, special modulus
// count, every key modulus, the first `limbs` coefficient moduli, the plain modulus (0 for CKKS).
parms_id_type compute_parms_id(scheme_type scheme, std::size_t poly_modulus_degree, std::size_t special_modulus_size,
                               const std::vector<std::uint64_t> &key_modulus, std::size_t limbs);

// include/util/encryptionparams.h:40-149
class EncryptionParameters {
public:
    explicit EncryptionParameters(scheme_type scheme = scheme_type::none) : scheme_(scheme) {}
    void set_mul_tech(mul_tech_type mul_tech);
    void set_poly_modulus_degree(std::size_t poly_modulus_degree);
    void set_special_modulus_size(std::size_t special_modulus_size);
    void set_galois_elts(const std::vector<uint32_t> &galois_elts) { galois_elts_ = galois_elts; }
    void set_coeff_modulus(const std::vector<Modulus> &coeff_modulus);

    scheme_type scheme() const { return scheme_; }
    mul_tech_type mul_tech() const { return mul_tech_; }
    std::size_t poly_modulus_degree() const { return poly_modulus_degree_; }
    std::size_t special_modulus_size() const { return special_modulus_size_; }
    const std::vector<Modulus> &coeff_modulus() const { return coeff_modulus_; }
    const std::vector<Modulus> &key_modulus() const { return coeff_modulus_; }
    const std::vector<uint32_t> &galois_elts() const { return galois_elts_; }
    // identifier of the key level (all moduli), as include/util/encryptionparams.h:315-317 returns it
    parms_id_type parms_id() const;
    // include/util/encryptionparams.h:302-308, 381-474: scheme u8 | degree u64 | count u64 | moduli u64... | plain
    // modulus u64 (0); the special modulus count and the Galois elements are not part of the record
    void save(std::ostream &stream) const;
    void load(std::istream &stream);

private:
    scheme_type scheme_;
    mul_tech_type mul_tech_ = mul_tech_type::none;
    std::size_t poly_modulus_degree_ = 0;
    std::size_t special_modulus_size_ = 1;  // include/util/encryptionparams.h:484
    std::vector<Modulus> coeff_modulus_;
    std::vector<uint32_t> galois_elts_;
};

void check_status(int status, const char *what);  // throws std::logic_error on a non-zero C-ABI status

// RAII device allocation from a process-wide size-bucketed pool (the role of cahel::util::Pointer<T> over
// MemoryPoolST, include/mempool.cuh:183-280): freed blocks are kept and reused so that the evaluator does
// not hit the allocator (and its implicit device synchronisation) on every operation.
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(std::size_t words) { allocate(words); }
    DeviceBuffer(const DeviceBuffer &o);
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), words_(o.words_), lane_(o.lane_), parent_(std::move(o.parent_)) {
        o.ptr_ = nullptr;
        o.words_ = 0;
    }
    DeviceBuffer &operator=(const DeviceBuffer &o);
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept;
    ~DeviceBuffer() { release(); }
    void allocate(std::size_t words);
    void release();
    // becomes a copy of the first `words` words of `src`; keeps its own block when that is large enough
    void assign(const DeviceBuffer &src, std::size_t words);
    // `words` words of `parent` from word `offset` on, without a copy: the slice keeps the parent's block alive and
    // returns nothing to the pool itself (batched evaluations hand out their results this way); a copy of a slice
    // is an ordinary buffer of its own
    static DeviceBuffer slice(std::shared_ptr<DeviceBuffer> parent, std::size_t offset, std::size_t words);
    // Turns the buffer into the only slice of a shared owner of its block, so that others can keep the block alive
    // past this object (owner()); the words stay where they are.  Not safe against concurrent use of this object.
    void make_shared();
    // the shared owner of the block, or null for a plain buffer
    const std::shared_ptr<DeviceBuffer> &owner() const { return parent_; }
    uint64_t *get() const { return ptr_; }
    std::size_t words() const { return words_; }
    static void trim_pool();  // return every cached block to the driver

private:
    uint64_t *ptr_ = nullptr;
    std::size_t words_ = 0;
    int lane_ = 0;  // the lane whose stream orders the reuse of this block
    std::shared_ptr<DeviceBuffer> parent_;  // set for a slice: the owner of the block that ptr_ points into
};

// Lanes (not in the reference, which runs everything on the legacy default stream): lane 0 is the null stream,
// lanes 1 .. lane_count() are non-blocking streams.  Every evaluator, encoder and key function enqueues on the
// current lane, and temporaries are recycled per lane, so independent ciphertext pipelines given different lanes
// overlap on the GPU.  An object produced on one lane may be used on another only after synchronize_lanes(); it
// may be dropped there (its storage returns to the producing lane after the dropping lane has drained).
he_stream current_stream();
int current_lane();
int lane_count();
void set_lane(int lane);
void synchronize_lanes();

}  // namespace cahel

// Step -> Galois element with generator 5 (include/galois.cuh:158-195): step 0 -> 2N-1 (conjugation),
// negative step s -> 5^(N/2 - |s|).
std::vector<uint32_t> get_elts_from_steps(const std::vector<int> &steps, std::size_t coeff_count);

// include/gpucontext.h:24-225.  Owns the CPU-side parameter chain and the device tables.
class CAHELGPUContext {
public:
    CAHELGPUContext(const cahel::EncryptionParameters &params, bool expand_mod_chain = true,
                    cahel::sec_level_type sec_level = cahel::sec_level_type::tc128);
    ~CAHELGPUContext();
    CAHELGPUContext(const CAHELGPUContext &) = delete;
    CAHELGPUContext &operator=(const CAHELGPUContext &) = delete;

    cahel::scheme_type scheme() const { return params_.scheme(); }
    std::size_t poly_degree() const { return n_; }
    int log_n() const { return log_n_; }
    std::size_t size_q() const { return size_q_; }
    std::size_t size_p() const { return size_p_; }
    std::size_t size_qp() const { return size_q_ + size_p_; }
    const std::vector<cahel::Modulus> &key_modulus() const { return params_.coeff_modulus(); }
    // chain index 0 = key level (Q u P); c >= 1 -> size_q - c + 1 limbs (src/context.cu:380-402)
    std::size_t chain_size() const { return chain_limbs_.size(); }
    std::size_t limbs_at(std::size_t chain_index) const;
    std::size_t get_first_index() const { return chain_limbs_.size() > 1 ? 1 : 0; }
    std::size_t max_chain_index() const { return chain_limbs_.size() - 1; }
    cahel::parms_id_type parms_id_at(std::size_t chain_index) const;
    cahel::parms_id_type key_parms_id() const { return parms_id_at(0); }
    int total_coeff_modulus_bit_count(std::size_t chain_index) const;
    bool using_keyswitching() const { return size_p_ > 0 && chain_limbs_.size() > 1; }

    const std::vector<uint32_t> &galois_elts() const { return galois_elts_; }
    uint32_t get_elt_from_step(int step) const;
    // index into galois_elts() or -1
    long find_galois_elt(uint32_t elt) const;

    he_context *handle() const { return he_; }
    he_stream stream() const { return cahel::current_stream(); }

    // Seeded randomness: every sampled polynomial takes the next stream id of the context's ChaCha20 key.
    // The default key comes from /dev/urandom (include/prng.cuh:12-23); set_seed makes runs reproducible.
    void set_seed(uint64_t seed);
    const uint32_t *prng_key() const { return prng_key_; }
    uint64_t next_stream(uint64_t count = 1) const { return prng_stream_.fetch_add(count, std::memory_order_relaxed); }
    const uint64_t *gauss_cdt() const { return gauss_cdt_.get(); }
    uint32_t gauss_cdt_len() const { return gauss_cdt_len_; }

    // host copies of the level tables (kept for introspection by tests)
    struct LevelHost {
        std::vector<uint64_t> part_hat_inv, digit_mats, qlast_inv;
        std::vector<uint32_t> digit_mat_off;
        uint32_t beta = 0;
    };
    const LevelHost &level_host(std::size_t L) const { return level_host_.at(L); }
    const std::vector<uint64_t> &psi_host() const { return psi_host_; }
    const std::vector<uint64_t> &ipsi_host() const { return ipsi_host_; }

private:
    void build_tables();
    cahel::EncryptionParameters params_;
    std::size_t n_ = 0, size_q_ = 0, size_p_ = 0;
    int log_n_ = 0;
    std::vector<std::size_t> chain_limbs_;
    std::vector<cahel::parms_id_type> parms_ids_;
    std::vector<uint32_t> galois_elts_;
    he_context *he_ = nullptr;
    uint32_t prng_key_[8];
    mutable std::atomic<uint64_t> prng_stream_{0};
    cahel::DeviceBuffer gauss_cdt_;
    uint32_t gauss_cdt_len_ = 0;
    std::vector<LevelHost> level_host_;
    std::vector<uint64_t> psi_host_, ipsi_host_;
};

// include/plaintext.h: CKKS plaintext = one polynomial over the limbs of its chain index, NTT form.
class CAHELGPUPlaintext {
public:
    CAHELGPUPlaintext() = default;
    explicit CAHELGPUPlaintext(const CAHELGPUContext &) {}
    void resize(std::size_t coeff_modulus_size, std::size_t poly_modulus_degree);
    uint64_t *data() const { return data_.get(); }
    std::size_t &chain_index() { return chain_index_; }
    std::size_t chain_index() const { return chain_index_; }
    double &scale() { return scale_; }
    double scale() const { return scale_; }
    bool is_ntt_form() const { return is_ntt_form_; }
    std::size_t coeff_modulus_size() const { return coeff_modulus_size_; }
    std::size_t poly_modulus_degree() const { return poly_modulus_degree_; }
    cahel::parms_id_type &parms_id() { return parms_id_; }
    cahel::parms_id_type parms_id() const { return parms_id_; }
    // the reference's byte layout (include/plaintext.h:109-200); load checks the header against the context
    void save(std::ostream &stream) const;
    void load(const CAHELGPUContext &context, std::istream &stream);

    cahel::DeviceBuffer data_;
    std::size_t chain_index_ = 0, coeff_modulus_size_ = 0, poly_modulus_degree_ = 0;
    double scale_ = 1.0;
    bool is_ntt_form_ = true;
    cahel::parms_id_type parms_id_ = cahel::parms_id_zero;
};

// A relinearize_inplace that has not run yet: the ciphertext still holds the three polynomials of the product and
// counts as two.  rescale_to_next consumes it together with the rescale in one device call (ModDown and the rescale
// then share one inverse and one forward transform); every other use of the ciphertext's data runs the key switch
// first, so nothing outside this layer can tell the difference except by the clock.
struct PendingKeySwitch {
    he_context *handle = nullptr;
    uint32_t limbs = 0;                                          // L of the level the product lives at
    std::vector<const uint64_t *> key_ptrs;                      // the relinearisation key's digits
    std::vector<std::shared_ptr<cahel::DeviceBuffer>> key_owners;  // keep those blocks alive until the switch has run
};

// include/ciphertext.h: size_ polynomials, layout [poly][limb][coeff].
class CAHELGPUCiphertext {
public:
    CAHELGPUCiphertext() = default;
    explicit CAHELGPUCiphertext(const CAHELGPUContext &) {}
    // copies move size() polynomials; the buffer behind data() may be larger than that (resize keeps a block that is
    // large enough, so that relinearize_inplace's 3 -> 2 polynomials and a later growth back cost no device copy)
    CAHELGPUCiphertext(const CAHELGPUCiphertext &o) { *this = o; }
    CAHELGPUCiphertext &operator=(const CAHELGPUCiphertext &o);
    CAHELGPUCiphertext(CAHELGPUCiphertext &&) noexcept = default;
    CAHELGPUCiphertext &operator=(CAHELGPUCiphertext &&) noexcept = default;
    // keeps the leading min(old, new) words (include/ciphertext.h:303-333)
    void resize(const CAHELGPUContext &context, std::size_t chain_index, std::size_t size);
    void resize(std::size_t size, std::size_t coeff_modulus_size, std::size_t poly_modulus_degree);
    uint64_t *data() const {
        if (pending_) settle();
        return data_.get();
    }
    // runs a deferred relinearisation (on the current lane); a no-op otherwise
    void settle() const;
    bool has_pending_key_switch() const { return static_cast<bool>(pending_); }
    // takes over a freshly computed block (whatever was deferred on the old one is dropped with it)
    void adopt(cahel::DeviceBuffer &&block) {
        pending_.reset();
        data_ = std::move(block);
    }
    std::size_t size() const { return size_; }
    std::size_t &chain_index() { return chain_index_; }
    std::size_t chain_index() const { return chain_index_; }
    double &scale() { return scale_; }
    double scale() const { return scale_; }
    void set_scale(double scale) { scale_ = scale; }
    bool &is_ntt_form() { return is_ntt_form_; }
    bool is_ntt_form() const { return is_ntt_form_; }
    bool &is_asymmetric() { return is_asymmetric_; }
    std::size_t coeff_modulus_size() const { return coeff_modulus_size_; }
    std::size_t poly_modulus_degree() const { return poly_modulus_degree_; }
    cahel::parms_id_type &parms_id() { return parms_id_; }
    cahel::parms_id_type parms_id() const { return parms_id_; }
    // the reference's byte layout (include/ciphertext.h:174-290); load checks the header against the context
    void save(std::ostream &stream) const;
    void load(const CAHELGPUContext &context, std::istream &stream);

    cahel::DeviceBuffer data_;
    std::size_t size_ = 0, chain_index_ = 0, coeff_modulus_size_ = 0, poly_modulus_degree_ = 0;
    double scale_ = 1.0;
    bool is_ntt_form_ = true, is_asymmetric_ = false;
    cahel::parms_id_type parms_id_ = cahel::parms_id_zero;
    // the 64 seed bytes that close a ciphertext record (the reference keeps them on the device and fills them only
    // when asked to save the seed, include/ciphertext.h:31, 205-213); kept here so that a record survives a round trip
    std::array<std::uint8_t, 64> prng_seed_{};
    // set by relinearize_inplace when it defers its key switch; data_ then holds size_ + 1 polynomials
    mutable std::shared_ptr<PendingKeySwitch> pending_;
};

// include/secretkey.h:20-108: a key-level ciphertext (-(a s + e), a)
class CAHELGPUPublicKey {
public:
    CAHELGPUPublicKey() = default;
    explicit CAHELGPUPublicKey(const CAHELGPUContext &) {}
    void encrypt_asymmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUCiphertext &cipher,
                            bool save_seed = false) const;
    CAHELGPUCiphertext encrypt_asymmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                          bool save_seed = false) const {
        CAHELGPUCiphertext cipher(context);
        encrypt_asymmetric(context, plain, cipher, save_seed);
        return cipher;
    }
    void save(std::ostream &stream) const;  // include/secretkey.h:53-59: the pair as a ciphertext record
    void load(const CAHELGPUContext &context, std::istream &stream);
    CAHELGPUCiphertext pk_;
    bool gen_flag_ = false;
};

// include/secretkey.h:113-268: dnum = size_q / size_p key-level pairs, one per digit
class CAHELGPURelinKey {
public:
    CAHELGPURelinKey() = default;
    explicit CAHELGPURelinKey(const CAHELGPUContext &context);
    cahel::parms_id_type parms_id() const { return parms_id_; }
    std::vector<const uint64_t *> key_ptrs() const;
    void save(std::ostream &stream) const;  // include/secretkey.h:212-256
    void load(const CAHELGPUContext &context, std::istream &stream);
    std::vector<CAHELGPUPublicKey> public_keys_;
    std::size_t pk_num_ = 0;
    bool gen_flag_ = false;
    cahel::parms_id_type parms_id_ = cahel::parms_id_zero;
};

// include/secretkey.h:270-410: one switching key per Galois element of the context
class CAHELGPUGaloisKey {
public:
    CAHELGPUGaloisKey() = default;
    explicit CAHELGPUGaloisKey(const CAHELGPUContext &) {}
    cahel::parms_id_type parms_id() const { return parms_id_; }
    void save(std::ostream &stream) const;  // include/secretkey.h:354-398
    void load(const CAHELGPUContext &context, std::istream &stream);
    std::vector<CAHELGPURelinKey> relin_keys_;
    std::size_t relin_key_num_ = 0;
    bool gen_flag_ = false;
    cahel::parms_id_type parms_id_ = cahel::parms_id_zero;
};

// include/secretkey.h:412-659
class CAHELGPUSecretKey {
public:
    explicit CAHELGPUSecretKey(const cahel::EncryptionParameters &params);
    void gen_secretkey(const CAHELGPUContext &context);
    void gen_publickey(const CAHELGPUContext &context, CAHELGPUPublicKey &pk, bool save_seed = true) const;
    void gen_relinkey(const CAHELGPUContext &context, CAHELGPURelinKey &relin_key, bool save_seed = false);
    void create_galois_keys(const CAHELGPUContext &context, CAHELGPUGaloisKey &galois_key, bool save_seed = false) const;
    void encrypt_symmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUCiphertext &cipher,
                           bool save_seed = false) const;
    CAHELGPUCiphertext encrypt_symmetric(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                         bool save_seed) const {
        CAHELGPUCiphertext cipher(context);
        encrypt_symmetric(context, plain, cipher, save_seed);
        return cipher;
    }
    void decrypt(const CAHELGPUContext &context, const CAHELGPUCiphertext &cipher, CAHELGPUPlaintext &plain);
    CAHELGPUPlaintext decrypt(const CAHELGPUContext &context, const CAHELGPUCiphertext &cipher) {
        CAHELGPUPlaintext plain(context);
        decrypt(context, cipher, plain);
        return plain;
    }
    // Decryption adds discrete-Gaussian noise (sigma = 5.574611952644673) as the reference does
    // (src/secretkey.cu:632-649); tests that compare limbs switch it off.
    void set_noise_flooding(bool on) { noise_flooding_ = on; }
    // Real parts of the first `count` slots of every ciphertext, [items][count] row-major: decrypt + decode of all of
    // them with one launch per stage (not in the reference).  All ciphertexts: size 2, one level, one scale;
    // `slots` = the encoder's slot count.
    std::vector<double> decrypt_decode_many(const CAHELGPUContext &context,
                                            const std::vector<const CAHELGPUCiphertext *> &ciphers, std::size_t slots,
                                            std::size_t count);
    const uint64_t *secret_key_array() const { return sk_powers_.get(); }

private:
    void encrypt_zero_symmetric(const CAHELGPUContext &context, CAHELGPUCiphertext &cipher, std::size_t chain_index) const;
    void generate_one_kswitch_key(const CAHELGPUContext &context, const uint64_t *new_key, CAHELGPURelinKey &relin_key) const;
    void compute_secret_key_array(const CAHELGPUContext &context, std::size_t max_power);
    cahel::DeviceBuffer sk_powers_;  // [max_power][QP][N] NTT form
    std::size_t sk_max_power_ = 0;
    std::size_t coeff_modulus_size_ = 0, poly_modulus_degree_ = 0;
    bool gen_flag_ = false;
    bool noise_flooding_ = true;
};

// include/ckks.h: canonical-embedding encoder over the orbit 5^j mod 2N
class CAHELGPUCKKSEncoder {
public:
    explicit CAHELGPUCKKSEncoder(const CAHELGPUContext &context);
    std::size_t slot_count() const { return slots_; }
    void reset_sparse_slots() { sparse_slots_ = 0; }
    std::size_t first_chain_index() const { return first_chain_index_; }
    // slot count of a message of `count` values: the first message fixes it for the lifetime of the encoder
    // (src/ckks.cu:131-142)
    std::size_t message_slots(std::size_t count);
    // Encode and encrypt `items` real vectors (row k at values + k * value_stride, `count` values each) at the
    // encoder's first chain index with one launch per stage; the ciphertexts equal those of encode +
    // encrypt_asymmetric called item by item (same randomness).  Not in the reference.
    std::vector<CAHELGPUCiphertext> encode_encrypt_many(const CAHELGPUContext &context, const CAHELGPUPublicKey &pk,
                                                        const double *values, std::size_t items, std::size_t count,
                                                        std::size_t value_stride, double scale);
    void encode(const CAHELGPUContext &context, const std::vector<double> &values, std::size_t chain_index, double scale,
                CAHELGPUPlaintext &destination);
    void encode(const CAHELGPUContext &context, const std::vector<double> &values, double scale,
                CAHELGPUPlaintext &destination) {
        encode(context, values, first_chain_index_, scale, destination);
    }
    void encode_complex(const CAHELGPUContext &context, const double *re, const double *im, std::size_t count,
                        std::size_t chain_index, double scale, CAHELGPUPlaintext &destination);
    CAHELGPUPlaintext encode(const CAHELGPUContext &context, const std::vector<double> &values, double scale) {
        CAHELGPUPlaintext destination(context);
        encode(context, values, scale, destination);
        return destination;
    }
    CAHELGPUPlaintext encode(const CAHELGPUContext &context, const std::vector<double> &values, std::size_t chain_index,
                             double scale) {
        CAHELGPUPlaintext destination(context);
        encode(context, values, chain_index, scale, destination);
        return destination;
    }
    void decode(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, std::vector<double> &destination);
    // real parts of the first `count` slots only (0: all): the transform runs in full, the download is `count` values
    void decode_values(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, std::size_t count,
                       std::vector<double> &interleaved);
    void decode_prefix(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, std::size_t count,
                       std::vector<double> &destination);
    void decode_complex(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, std::vector<double> &re,
                        std::vector<double> &im);
    std::vector<double> decode(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain) {
        std::vector<double> out;
        decode(context, plain, out);
        return out;
    }

private:
    std::size_t slots_ = 0, sparse_slots_ = 0;
    std::size_t first_chain_index_ = 1;  // include/ckks.h:325
};

// ---- evaluator: include/evaluate.h:15-600 ----
void negate_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted);
void negate(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination);
void add_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2);
void add(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
         CAHELGPUCiphertext &destination);
void add_many(const CAHELGPUContext &context, const std::vector<CAHELGPUCiphertext> &encrypteds,
              CAHELGPUCiphertext &destination);
void sub_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
                 const bool &negate = false);
void sub(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
         CAHELGPUCiphertext &destination);
void add_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain);
void add_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
               CAHELGPUCiphertext &destination);
void sub_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain);
void sub_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
               CAHELGPUCiphertext &destination);
void multiply_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2);
void multiply(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1, const CAHELGPUCiphertext &encrypted2,
              CAHELGPUCiphertext &destination);
void multiply_and_relin_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted1,
                                const CAHELGPUCiphertext &encrypted2, const CAHELGPURelinKey &relin_keys);
void multiply_plain_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain);
void multiply_plain(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUPlaintext &plain,
                    CAHELGPUCiphertext &destination);
void multiply_many(const CAHELGPUContext &context, std::vector<CAHELGPUCiphertext> &encrypteds,
                   CAHELGPURelinKey &relin_key, CAHELGPUCiphertext &destination);
void square_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted);
void square(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination);
void exponentiate_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, uint64_t exponent,
                          CAHELGPURelinKey &relin_key);
void exponentiate(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, uint64_t exponent,
                  CAHELGPUCiphertext &destination, CAHELGPURelinKey &relin_key);
void relinearize_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPURelinKey &relin_keys);
// Batched squared distances of ciphertext pairs (batch.cpp); not in the reference
std::vector<CAHELGPUCiphertext> pair_square_distances(
    const CAHELGPUContext &context, const std::vector<std::vector<const CAHELGPUCiphertext *>> &clients,
    const std::vector<std::pair<std::size_t, std::size_t>> &pairs, const CAHELGPURelinKey &rlk,
    const CAHELGPUGaloisKey &glk, const std::vector<std::vector<int>> &rounds, double scale, std::size_t drop_levels = 0);
void relinearize_rescale_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted,
                                 const CAHELGPURelinKey &relin_keys);
void multiply_relin_rescale(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted1,
                            const CAHELGPUCiphertext &encrypted2, const CAHELGPURelinKey &relin_keys,
                            CAHELGPUCiphertext &destination);  // this build's addition
void relinearize(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination,
                 const CAHELGPURelinKey &relin_keys);
void mod_switch_to_next_inplace(const CAHELGPUContext &context, CAHELGPUPlaintext &plain);
void mod_switch_to_next(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUPlaintext &destination);
void mod_switch_to_inplace(const CAHELGPUContext &context, CAHELGPUPlaintext &plain, std::size_t chain_index);
void mod_switch_to(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain, CAHELGPUPlaintext &destination,
                   std::size_t chain_index);
void mod_switch_to_next(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                        CAHELGPUCiphertext &destination);
void mod_switch_to_next_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted);
void mod_switch_to_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t chain_index);
void mod_switch_to(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination,
                   std::size_t chain_index);
void rescale_to_next(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted, CAHELGPUCiphertext &destination);
void rescale_to_next_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted);
void switch_key_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const uint64_t *c2,
                        const CAHELGPURelinKey &relin_keys, bool is_relin = false, uint32_t galois_elt = 0);
void apply_galois_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t galois_elt_index,
                          const CAHELGPUGaloisKey &galois_keys);
void apply_galois(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, std::size_t galois_elt_index,
                  const CAHELGPUGaloisKey &galois_keys, CAHELGPUCiphertext &destination);
void rotate_rows_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int steps,
                         const CAHELGPUGaloisKey &galois_key);
void rotate_rows(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int steps,
                 const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &destination);
void rotate_columns_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUGaloisKey &galois_key);
void rotate_columns(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUGaloisKey &galois_key,
                    CAHELGPUCiphertext &destination);
void rotate_vector_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int step,
                           const CAHELGPUGaloisKey &galois_key);
void rotate_vector(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, int step,
                   const CAHELGPUGaloisKey &galois_key, CAHELGPUCiphertext &destination);
void hoisting_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &ct, const CAHELGPUGaloisKey &glk,
                      const std::vector<int> &steps);
CAHELGPUCiphertext hoisting(const CAHELGPUContext &context, const CAHELGPUCiphertext &encrypted,
                            const CAHELGPUGaloisKey &glk, const std::vector<int> &steps);
void complex_conjugate_inplace(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted,
                               const CAHELGPUGaloisKey &galois_key);
void complex_conjugate(const CAHELGPUContext &context, CAHELGPUCiphertext &encrypted, const CAHELGPUGaloisKey &galois_key,
                       CAHELGPUCiphertext &destination);
