// Parameters, device buffers and the context: host precompute of every table the kernels read.
// Follows cahel-main/include/gpucontext.h:53-136 (what is uploaded), src/context.cu:128-403 (validation and the
// modulus-switching chain), src/util/ntt.cu:32-80 (psi tables) and src/util/rns.cu:433-556 (hybrid
// key-switching constants); the arithmetic is restated with 128-bit integers instead of multi-word helpers.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <random>
#include <string>

#include "cahel.h"

namespace cahel {

void check_status(int status, const char *what) {
    if (status != HE_OK) throw std::logic_error(std::string(what) + ": " + he_error_string(status));
}

// ---------------------------------------------------------------------------------------------------
// EncryptionParameters
// ---------------------------------------------------------------------------------------------------
void EncryptionParameters::set_mul_tech(mul_tech_type mul_tech) {
    if (scheme_ != scheme_type::bfv) throw std::invalid_argument("mul_tech selection is only supported for BFV");
    if (mul_tech == mul_tech_type::none) throw std::invalid_argument("unsupported multiplication technique for BFV");
    mul_tech_ = mul_tech;
}

void EncryptionParameters::set_poly_modulus_degree(std::size_t poly_modulus_degree) {
    if (scheme_ == scheme_type::none && poly_modulus_degree)
        throw std::logic_error("poly_modulus_degree is not supported for this scheme");
    poly_modulus_degree_ = poly_modulus_degree;
}

void EncryptionParameters::set_special_modulus_size(std::size_t special_modulus_size) {
    if (scheme_ == scheme_type::none && special_modulus_size)
        throw std::logic_error("special_modulus_size is not supported for this scheme");
    special_modulus_size_ = special_modulus_size;
}

void EncryptionParameters::set_coeff_modulus(const std::vector<Modulus> &coeff_modulus) {
    if (scheme_ == scheme_type::none) {
        if (!coeff_modulus.empty()) throw std::logic_error("coeff_modulus is not supported for this scheme");
    } else if (coeff_modulus.size() > 64 || coeff_modulus.size() < 1) {
        throw std::invalid_argument("coeff_modulus is invalid");
    }
    coeff_modulus_ = coeff_modulus;
}

parms_id_type compute_parms_id(scheme_type scheme, std::size_t poly_modulus_degree, std::size_t special_modulus_size,
                               const std::vector<uint64_t> &key_modulus, std::size_t limbs) {
    if (limbs > key_modulus.size()) throw std::invalid_argument("more limbs than key moduli");
    std::vector<uint64_t> words{(uint64_t)scheme, (uint64_t)poly_modulus_degree, (uint64_t)special_modulus_size};
    words.insert(words.end(), key_modulus.begin(), key_modulus.end());
    words.insert(words.end(), key_modulus.begin(), key_modulus.begin() + (std::ptrdiff_t)limbs);
    words.push_back(0);  // plain modulus: one zero word outside BFV / BGV
    parms_id_type id;
    blake2b(id.data(), sizeof(id), words.data(), words.size() * sizeof(uint64_t));
    if (id == parms_id_zero) throw std::logic_error("parms_id cannot be zero");
    return id;
}

parms_id_type EncryptionParameters::parms_id() const {
    std::vector<uint64_t> mods;
    for (const auto &m : coeff_modulus_) mods.push_back(m.value());
    return compute_parms_id(scheme_, poly_modulus_degree_, special_modulus_size_, mods, mods.size());
}

// ---------------------------------------------------------------------------------------------------
// device memory pool
// ---------------------------------------------------------------------------------------------------
namespace {

// Lanes: lane 0 is the null stream (what the reference uses for everything); lanes 1 .. kMaxLanes are
// non-blocking streams created on first use.  Work of different lanes may overlap on the GPU.
constexpr int kMaxLanes = 8;
thread_local int g_lane = 0;  // every host thread has its own current lane
he_stream g_lane_streams[kMaxLanes + 1] = {};
std::mutex g_lane_mu;

struct Pool {
    std::mutex mu;
    // (lane, bytes) -> block.  A block returns to the lane that took it, so that reuse is ordered by that lane's
    // stream however the owning object travelled.
    std::multimap<std::pair<int, std::size_t>, void *> free_blocks;
    ~Pool() {
        // the HIP runtime may already be gone at static destruction; leave the blocks to process exit
    }
    void *take(std::size_t bytes, int lane) {
        {
            std::lock_guard<std::mutex> g(mu);
            auto it = free_blocks.find({lane, bytes});
            if (it != free_blocks.end()) {
                void *p = it->second;
                free_blocks.erase(it);
                return p;
            }
        }
        void *p = nullptr;
        int rc = he_malloc(&p, bytes);
        if (rc != HE_OK) {
            trim();
            rc = he_malloc(&p, bytes);
        }
        check_status(rc, "device allocation failed");
        return p;
    }
    void give(void *p, std::size_t bytes, int lane) {
        std::lock_guard<std::mutex> g(mu);
        free_blocks.emplace(std::make_pair(lane, bytes), p);
    }
    void trim() {
        std::lock_guard<std::mutex> g(mu);
        for (auto &kv : free_blocks) he_free(kv.second);
        free_blocks.clear();
    }
};

Pool &pool() {
    static Pool *p = new Pool;  // intentionally leaked: outlives every static DeviceBuffer
    return *p;
}

}  // namespace

void DeviceBuffer::allocate(std::size_t words) {
    release();
    if (words == 0) return;
    lane_ = g_lane;
    ptr_ = static_cast<uint64_t *>(pool().take(words * sizeof(uint64_t), lane_));
    words_ = words;
}

void DeviceBuffer::release() {
    // A block goes back to the lane that took it.  Dropped from another lane, it may still be read by work that
    // the dropping thread has enqueued there: wait for that lane before the owner's lane can reuse the block.
    if (ptr_ && g_lane != lane_) (void)he_stream_synchronize(g_lane_streams[g_lane]);
    if (ptr_ && !parent_) pool().give(ptr_, words_ * sizeof(uint64_t), lane_);
    parent_.reset();  // the last slice to go releases the parent's block (same rule, in the parent's destructor)
    ptr_ = nullptr;
    words_ = 0;
}

DeviceBuffer DeviceBuffer::slice(std::shared_ptr<DeviceBuffer> parent, std::size_t offset, std::size_t words) {
    if (!parent || offset + words > parent->words_) throw std::logic_error("DeviceBuffer::slice: out of range");
    DeviceBuffer v;
    v.ptr_ = parent->ptr_ + offset;
    v.words_ = words;
    v.lane_ = parent->lane_;
    v.parent_ = std::move(parent);
    return v;
}

void DeviceBuffer::make_shared() {
    if (!ptr_ || parent_) return;
    auto owner = std::make_shared<DeviceBuffer>();
    owner->ptr_ = ptr_;
    owner->words_ = words_;
    owner->lane_ = lane_;
    parent_ = std::move(owner);
}

DeviceBuffer::DeviceBuffer(const DeviceBuffer &o) {
    allocate(o.words_);
    if (words_) check_status(he_memcpy_d2d(ptr_, o.ptr_, words_ * sizeof(uint64_t), current_stream()), "device copy failed");
}

DeviceBuffer &DeviceBuffer::operator=(const DeviceBuffer &o) {
    if (this == &o) return *this;
    if (words_ != o.words_) allocate(o.words_);
    if (words_) check_status(he_memcpy_d2d(ptr_, o.ptr_, words_ * sizeof(uint64_t), current_stream()), "device copy failed");
    return *this;
}

void DeviceBuffer::assign(const DeviceBuffer &src, std::size_t words) {
    if (this == &src) return;
    if (words > src.words_) throw std::logic_error("DeviceBuffer::assign: source too small");
    if (words_ < words || !ptr_) allocate(words);
    if (words) check_status(he_memcpy_d2d(ptr_, src.ptr_, words * sizeof(uint64_t), current_stream()), "device copy failed");
}

DeviceBuffer &DeviceBuffer::operator=(DeviceBuffer &&o) noexcept {
    if (this != &o) {
        release();
        ptr_ = o.ptr_;
        words_ = o.words_;
        lane_ = o.lane_;
        parent_ = std::move(o.parent_);
        o.ptr_ = nullptr;
        o.words_ = 0;
    }
    return *this;
}

void DeviceBuffer::trim_pool() { pool().trim(); }

he_stream current_stream() { return g_lane_streams[g_lane]; }

int current_lane() { return g_lane; }

int lane_count() { return kMaxLanes; }

void set_lane(int lane) {
    if (lane < 0 || lane > kMaxLanes) throw std::invalid_argument("lane out of range");
    if (lane > 0) {
        std::lock_guard<std::mutex> g(g_lane_mu);
        if (!g_lane_streams[lane]) check_status(he_stream_create(&g_lane_streams[lane]), "stream creation failed");
    }
    g_lane = lane;
}

void synchronize_lanes() {
    for (int i = 0; i <= kMaxLanes; i++)
        if (i == 0 || g_lane_streams[i]) check_status(he_stream_synchronize(g_lane_streams[i]), "synchronisation failed");
}

}  // namespace cahel

using namespace cahel;

// ---------------------------------------------------------------------------------------------------
// Galois elements
// ---------------------------------------------------------------------------------------------------
static uint32_t elt_from_step(int step, std::size_t coeff_count) {
    const uint32_t n = (uint32_t)coeff_count;
    const uint64_t m = 2ull * n;
    if (step == 0) return (uint32_t)(m - 1);
    const bool sign = step < 0;
    const uint32_t pos = (uint32_t)std::abs(step);
    if (pos >= (n >> 1)) throw std::invalid_argument("step count too large");
    uint32_t k = sign ? (n >> 1) - pos : pos;
    uint64_t elt = 1;
    while (k--) elt = (elt * 5) & (m - 1);
    return (uint32_t)elt;
}

std::vector<uint32_t> get_elts_from_steps(const std::vector<int> &steps, std::size_t coeff_count) {
    std::vector<uint32_t> out;
    for (int s : steps) out.push_back(elt_from_step(s, coeff_count));
    return out;
}

// ---------------------------------------------------------------------------------------------------
// containers
// ---------------------------------------------------------------------------------------------------
void CAHELGPUPlaintext::resize(std::size_t coeff_modulus_size, std::size_t poly_modulus_degree) {
    const std::size_t words = coeff_modulus_size * poly_modulus_degree;
    if (words != data_.words()) data_.allocate(words);
    coeff_modulus_size_ = coeff_modulus_size;
    poly_modulus_degree_ = poly_modulus_degree;
}

CAHELGPUCiphertext &CAHELGPUCiphertext::operator=(const CAHELGPUCiphertext &o) {
    if (this == &o) return *this;
    o.settle();
    pending_.reset();
    data_.assign(o.data_, o.size_ * o.coeff_modulus_size_ * o.poly_modulus_degree_);
    size_ = o.size_;
    chain_index_ = o.chain_index_;
    coeff_modulus_size_ = o.coeff_modulus_size_;
    poly_modulus_degree_ = o.poly_modulus_degree_;
    scale_ = o.scale_;
    is_ntt_form_ = o.is_ntt_form_;
    is_asymmetric_ = o.is_asymmetric_;
    parms_id_ = o.parms_id_;
    prng_seed_ = o.prng_seed_;
    return *this;
}

void CAHELGPUCiphertext::settle() const {
    if (!pending_) return;
    // (two host threads may read one ciphertext; only one of them runs the switch)
    static std::mutex mu;
    std::lock_guard<std::mutex> g(mu);
    if (!pending_) return;
    const PendingKeySwitch &p = *pending_;
    const std::size_t poly = (std::size_t)p.limbs * poly_modulus_degree_;
    DeviceBuffer ws(he_keyswitch_workspace_words(p.handle, p.limbs));
    check_status(he_keyswitch(p.handle, p.limbs, data_.get() + 2 * poly, p.key_ptrs.data(), data_.get(), 0, ws.get(),
                              current_stream()),
                 "he_keyswitch");
    pending_.reset();
}

void CAHELGPUCiphertext::resize(std::size_t size, std::size_t coeff_modulus_size, std::size_t poly_modulus_degree) {
    settle();
    const std::size_t old_words = size_ * coeff_modulus_size_ * poly_modulus_degree_;
    const std::size_t new_words = size * coeff_modulus_size * poly_modulus_degree;
    // a block that is large enough stays: the leading words are the ones to keep anyway
    if (new_words > data_.words() || !data_.get()) {
        DeviceBuffer fresh(new_words);
        const std::size_t keep = old_words < new_words ? old_words : new_words;
        if (keep && data_.get())
            check_status(he_memcpy_d2d(fresh.get(), data_.get(), keep * sizeof(uint64_t), current_stream()), "device copy failed");
        data_ = std::move(fresh);
    }
    size_ = size;
    coeff_modulus_size_ = coeff_modulus_size;
    poly_modulus_degree_ = poly_modulus_degree;
}

void CAHELGPUCiphertext::resize(const CAHELGPUContext &context, std::size_t chain_index, std::size_t size) {
    resize(size, context.limbs_at(chain_index), context.poly_degree());
    chain_index_ = chain_index;
    parms_id_ = context.parms_id_at(chain_index);
}

// ---------------------------------------------------------------------------------------------------
// context
// ---------------------------------------------------------------------------------------------------
static void chacha_key_from_seed(uint64_t seed, uint32_t key[8]) {
    uint64_t z = seed;
    for (int i = 0; i < 4; i++) {
        z += 0x9E3779B97F4A7C15ull;
        uint64_t x = z;
        x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
        x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
        x ^= x >> 31;
        key[2 * i] = (uint32_t)x;
        key[2 * i + 1] = (uint32_t)(x >> 32);
    }
}

// cdt[i] = floor(2^63 P(|X| <= i)) of the discrete Gaussian with the decryption-flooding sigma of the
// reference (src/secretkey.cu:633), truncated at 12 sigma; double precision, fixed operation order.
static std::vector<uint64_t> gauss_cdt_table(double sigma) {
    const int bound = (int)std::ceil(12 * sigma);
    std::vector<double> w(bound + 1);
    for (int x = 0; x <= bound; x++) w[x] = std::exp(-((double)x * x) / (2.0 * sigma * sigma));
    double total = w[0];
    for (int x = 1; x <= bound; x++) total += 2.0 * w[x];
    std::vector<uint64_t> out(bound + 1);
    double acc = 0.0;
    const uint64_t top = ((uint64_t)1 << 63) - 1;
    for (int x = 0; x <= bound; x++) {
        acc += x == 0 ? w[x] : 2.0 * w[x];
        const double frac = acc / total;
        uint64_t v = frac < 1.0 ? (uint64_t)(frac * 9223372036854775808.0) : top;
        out[x] = v < top ? v : top;
    }
    return out;
}

CAHELGPUContext::CAHELGPUContext(const EncryptionParameters &params, bool expand_mod_chain, sec_level_type sec_level)
    : params_(params) {
    if (params.scheme() != scheme_type::ckks)
        throw std::invalid_argument("unsupported scheme: this engine implements CKKS");
    n_ = params.poly_modulus_degree();
    log_n_ = power_of_two(n_);
    if (log_n_ < 0) throw std::invalid_argument("invalid poly_modulus_degree");
    if (log_n_ < 9 || log_n_ > 17) throw std::invalid_argument("poly_modulus_degree must be between 2^9 and 2^17");
    const auto &mods = params.coeff_modulus();
    if (mods.empty() || mods.size() > 64) throw std::invalid_argument("parameter generate failed");
    std::size_t size_qp = mods.size();
    size_p_ = size_qp == 1 ? 0 : params.special_modulus_size();
    if (size_p_ >= size_qp) throw std::invalid_argument("special modulus size must be smaller than the modulus count");
    size_q_ = size_qp - size_p_;
    if (size_p_ && size_q_ % size_p_)
        throw std::invalid_argument("coeff modulus count (without special primes) must be a multiple of the special modulus size");
    int total_bits = 0;
    {
        std::vector<uint64_t> vals;
        for (auto &m : mods) {
            if (m.value() >> 60 || m.value() < 2) throw std::invalid_argument("parameter generate failed");
            vals.push_back(m.value());
        }
        for (std::size_t i = 0; i < vals.size(); i++)
            for (std::size_t j = i + 1; j < vals.size(); j++)
                if (vals[i] == vals[j]) throw std::invalid_argument("coeff_modulus must consist of distinct primes");
        total_bits = BigUInt::product(vals).bit_count();
    }
    if (sec_level != sec_level_type::none && total_bits > CoeffModulus::MaxBitCount(n_, (int)sec_level))
        throw std::invalid_argument("invalid parameters_insecure");

    chain_limbs_.push_back(size_qp);
    if (size_qp > 1) {
        const std::size_t levels = expand_mod_chain ? size_q_ : 1;
        for (std::size_t i = 0; i < levels; i++) chain_limbs_.push_back(size_q_ - i);
    }
    {
        // src/context.cu:352-401: the key level hashes all moduli, data level c the first size_q - c + 1 of them;
        // a single-modulus chain has no special modulus
        std::vector<uint64_t> vals;
        for (auto &m : mods) vals.push_back(m.value());
        for (std::size_t limbs : chain_limbs_)
            parms_ids_.push_back(compute_parms_id(params.scheme(), n_, size_p_, vals, limbs));
    }
    galois_elts_ = params.galois_elts();
    if (galois_elts_.empty()) {
        // include/galois.cuh / src/galois.cu:109-133: conjugation, then 5^(2^i) and 5^-(2^i)
        const uint32_t m = (uint32_t)(2 * n_);
        galois_elts_.push_back(m - 1);
        uint64_t pos = 5, neg = invert_mod(5, m);
        for (int i = 0; i < log_n_ - 1; i++) {
            galois_elts_.push_back((uint32_t)pos);
            pos = (pos * pos) & (m - 1);
            galois_elts_.push_back((uint32_t)neg);
            neg = (neg * neg) & (m - 1);
        }
    }
    for (uint32_t e : galois_elts_)
        if (!(e & 1) || e >= 2 * n_) throw std::invalid_argument("Galois element is not valid");

    std::random_device rd("/dev/urandom");
    for (auto &k : prng_key_) k = rd();
    build_tables();
}

CAHELGPUContext::~CAHELGPUContext() { he_context_destroy(he_); }

void CAHELGPUContext::set_seed(uint64_t seed) {
    chacha_key_from_seed(seed, prng_key_);
    prng_stream_ = 0;
}

std::size_t CAHELGPUContext::limbs_at(std::size_t chain_index) const {
    if (chain_index >= chain_limbs_.size()) throw std::invalid_argument("chain index out of range");
    return chain_limbs_[chain_index];
}

parms_id_type CAHELGPUContext::parms_id_at(std::size_t chain_index) const {
    if (chain_index >= parms_ids_.size()) throw std::invalid_argument("chain index out of range");
    return parms_ids_[chain_index];
}

int CAHELGPUContext::total_coeff_modulus_bit_count(std::size_t chain_index) const {
    std::vector<uint64_t> vals;
    const auto &mods = params_.coeff_modulus();
    for (std::size_t i = 0; i < limbs_at(chain_index); i++) vals.push_back(mods[i].value());
    return BigUInt::product(vals).bit_count();
}

uint32_t CAHELGPUContext::get_elt_from_step(int step) const { return elt_from_step(step, n_); }

long CAHELGPUContext::find_galois_elt(uint32_t elt) const {
    for (std::size_t i = 0; i < galois_elts_.size(); i++)
        if (galois_elts_[i] == elt) return (long)i;
    return -1;
}

static void push_shoup(std::vector<uint64_t> &v, uint64_t w, uint64_t q) {
    v.push_back(w);
    v.push_back(shoup_quotient(w, q));
}

void CAHELGPUContext::build_tables() {
    const auto &mods = params_.coeff_modulus();
    const std::size_t qp = mods.size(), n = n_;
    std::vector<uint64_t> moduli(qp), barrett(2 * qp);
    psi_host_.assign(2 * qp * n, 0);
    ipsi_host_.assign(2 * qp * n, 0);
    for (std::size_t t = 0; t < qp; t++) {
        const uint64_t q = mods[t].value();
        moduli[t] = q;
        barrett[2 * t] = mods[t].const_ratio()[0];
        barrett[2 * t + 1] = mods[t].const_ratio()[1];
        uint64_t root;
        if (!try_minimal_primitive_root(2 * n, q, root))
            throw std::invalid_argument("invalid modulus in try_minimal_primitive_root");
        const uint64_t inv_root = invert_mod(root, q);
        const uint64_t half = invert_mod(2, q);
        uint64_t *psi = psi_host_.data() + 2 * t * n, *ipsi = ipsi_host_.data() + 2 * t * n;
        uint64_t p = 1, ip = half;
        for (std::size_t i = 0; i < n; i++) {
            const std::size_t r = reverse_bits((uint32_t)i, log_n_);
            psi[2 * r] = p;
            psi[2 * r + 1] = shoup_quotient(p, q);
            ipsi[2 * r] = ip;
            ipsi[2 * r + 1] = shoup_quotient(ip, q);
            p = mul_mod(p, root, q);
            ip = mul_mod(ip, inv_root, q);
        }
        // entry 0 of the inverse table holds psi^-1 / 2 (src/util/ntt.cu:71); no butterfly reads it
        ipsi[0] = mul_mod(inv_root, half, q);
        ipsi[1] = shoup_quotient(ipsi[0], q);
    }
    he_context_desc d;
    std::memset(&d, 0, sizeof(d));
    d.log_n = (uint32_t)log_n_;
    d.size_q = (uint32_t)size_q_;
    d.size_p = (uint32_t)size_p_;
    d.moduli = moduli.data();
    d.barrett = barrett.data();
    d.psi = psi_host_.data();
    d.ipsi_div2 = ipsi_host_.data();
    std::vector<uint64_t> p_mod_q, pinv_mod_q, phat_inv, phat_mod_q;
    const std::size_t Q = size_q_, K = size_p_;
    if (K) {
        for (std::size_t i = 0; i < Q; i++) {
            const uint64_t q = moduli[i];
            uint64_t pm = 1;
            for (std::size_t k = 0; k < K; k++) pm = mul_mod(pm, moduli[Q + k] % q, q);
            push_shoup(p_mod_q, pm, q);
            push_shoup(pinv_mod_q, invert_mod(pm, q), q);
        }
        for (std::size_t k = 0; k < K; k++) {
            const uint64_t pk = moduli[Q + k];
            uint64_t hat = 1;
            for (std::size_t k2 = 0; k2 < K; k2++)
                if (k2 != k) hat = mul_mod(hat, moduli[Q + k2] % pk, pk);
            push_shoup(phat_inv, invert_mod(hat, pk), pk);
        }
        phat_mod_q.resize(Q * K);
        for (std::size_t j = 0; j < Q; j++)
            for (std::size_t k = 0; k < K; k++) {
                uint64_t hat = 1;
                for (std::size_t k2 = 0; k2 < K; k2++)
                    if (k2 != k) hat = mul_mod(hat, moduli[Q + k2] % moduli[j], moduli[j]);
                phat_mod_q[j * K + k] = hat;
            }
        d.p_mod_q = p_mod_q.data();
        d.pinv_mod_q = pinv_mod_q.data();
        d.phat_inv_mod_p = phat_inv.data();
        d.phat_mod_q = phat_mod_q.data();
    }
    check_status(he_context_create(&d, &he_), "he_context_create");

    level_host_.resize(Q + 1);
    for (std::size_t L = 1; L <= Q; L++) {
        LevelHost &lh = level_host_[L];
        he_level_desc ld;
        std::memset(&ld, 0, sizeof(ld));
        ld.L = (uint32_t)L;
        for (std::size_t j = 0; j + 1 < L; j++) push_shoup(lh.qlast_inv, invert_mod(moduli[L - 1] % moduli[j], moduli[j]), moduli[j]);
        ld.qlast_inv = lh.qlast_inv.data();
        if (K) {
            lh.beta = (uint32_t)((L + K - 1) / K);
            ld.beta = lh.beta;
            for (uint32_t dg = 0; dg < lh.beta; dg++) {
                const std::size_t start = dg * K, size = (start + K <= L) ? K : L - start;
                for (std::size_t i = start; i < start + size; i++) {
                    const uint64_t q = moduli[i];
                    uint64_t hat = 1;
                    for (std::size_t i2 = start; i2 < start + size; i2++)
                        if (i2 != i) hat = mul_mod(hat, moduli[i2] % q, q);
                    push_shoup(lh.part_hat_inv, invert_mod(hat, q), q);
                }
                lh.digit_mat_off.push_back((uint32_t)lh.digit_mats.size());
                for (std::size_t t = 0; t < L + K; t++) {
                    if (t >= start && t < start + size) continue;
                    const uint64_t m = moduli[t < L ? t : Q + (t - L)];
                    for (std::size_t i = start; i < start + size; i++) {
                        uint64_t hat = 1;
                        for (std::size_t i2 = start; i2 < start + size; i2++)
                            if (i2 != i) hat = mul_mod(hat, moduli[i2] % m, m);
                        lh.digit_mats.push_back(hat);
                    }
                }
            }
            ld.part_hat_inv = lh.part_hat_inv.data();
            ld.digit_mats = lh.digit_mats.data();
            ld.digit_mat_off = lh.digit_mat_off.data();
        }
        check_status(he_context_set_level(he_, &ld), "he_context_set_level");
    }
    auto cdt = gauss_cdt_table(5.574611952644673);
    gauss_cdt_len_ = (uint32_t)cdt.size();
    gauss_cdt_.allocate(cdt.size());
    check_status(he_memcpy_h2d(gauss_cdt_.get(), cdt.data(), cdt.size() * sizeof(uint64_t), nullptr), "upload");
}
