#include "hostmath.h"

#include <algorithm>
#include <cmath>
#include <map>
#include <stdexcept>

namespace cahel {

uint64_t pow_mod(uint64_t base, uint64_t exp, uint64_t q) {
    uint64_t result = 1 % q;
    base %= q;
    while (exp) {
        if (exp & 1) result = mul_mod(result, base, q);
        base = mul_mod(base, base, q);
        exp >>= 1;
    }
    return result;
}

bool try_invert_mod(uint64_t a, uint64_t q, uint64_t &result) {
    if (q < 2) return false;
    // extended Euclid on signed 128-bit cofactors
    __int128 t0 = 0, t1 = 1;
    uint64_t r0 = q, r1 = a % q;
    while (r1) {
        uint64_t quo = r0 / r1;
        uint64_t r2 = r0 - quo * r1;
        __int128 t2 = t0 - (__int128)quo * t1;
        r0 = r1; r1 = r2; t0 = t1; t1 = t2;
    }
    if (r0 != 1) return false;
    if (t0 < 0) t0 += q;
    result = (uint64_t)t0;
    return true;
}

uint64_t invert_mod(uint64_t a, uint64_t q) {
    uint64_t r;
    if (!try_invert_mod(a, q, r)) throw std::invalid_argument("value is not invertible modulo the modulus");
    return r;
}

int significant_bits(uint64_t v) { return v ? 64 - __builtin_clzll(v) : 0; }

uint32_t reverse_bits(uint32_t x, int bits) {
    if (bits == 0) return 0;
    uint32_t r = 0;
    for (int i = 0; i < bits; i++) r |= ((x >> i) & 1u) << (bits - 1 - i);
    return r;
}

bool is_prime(uint64_t v) {
    if (v < 2) return false;
    static const uint64_t bases[] = {2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37};
    for (uint64_t p : bases) {
        if (v % p == 0) return v == p;
    }
    uint64_t d = v - 1;
    int r = 0;
    while (!(d & 1)) { d >>= 1; r++; }
    // these twelve bases decide primality for every 64-bit integer
    for (uint64_t a : bases) {
        uint64_t x = pow_mod(a, d, v);
        if (x == 1 || x == v - 1) continue;
        bool composite = true;
        for (int i = 1; i < r; i++) {
            x = mul_mod(x, x, v);
            if (x == v - 1) { composite = false; break; }
        }
        if (composite) return false;
    }
    return true;
}

std::vector<uint64_t> get_primes(size_t ntt_size, int bit_size, size_t count) {
    if (bit_size < 2 || bit_size > 61) throw std::invalid_argument("bit_size is invalid");
    const uint64_t factor = 2 * (uint64_t)ntt_size;
    uint64_t value = (uint64_t)1 << bit_size;
    if (value <= factor) throw std::logic_error("failed to find enough qualifying primes");
    value = value - factor + 1;
    const uint64_t lower = (uint64_t)1 << (bit_size - 1);
    std::vector<uint64_t> out;
    while (count > 0 && value > lower) {
        if (is_prime(value)) { out.push_back(value); count--; }
        if (value < factor) break;
        value -= factor;
    }
    if (count > 0) throw std::logic_error("failed to find enough qualifying primes");
    return out;
}

bool is_primitive_root(uint64_t root, uint64_t degree, uint64_t q) {
    if (root == 0) return false;
    return pow_mod(root, degree >> 1, q) == q - 1;
}

bool try_minimal_primitive_root(uint64_t degree, uint64_t q, uint64_t &root) {
    if (degree < 2 || (q - 1) % degree) return false;
    const uint64_t quotient = (q - 1) / degree;
    uint64_t r = 0;
    bool found = false;
    for (uint64_t x = 2; x < 2 + 4096 && x < q; x++) {
        r = pow_mod(x, quotient, q);
        if (is_primitive_root(r, degree, q)) { found = true; break; }
    }
    if (!found) return false;
    // every primitive root is an odd power of r; walk them all and keep the smallest
    const uint64_t sq = mul_mod(r, r, q);
    uint64_t best = r, cur = r;
    for (uint64_t i = 0; i < degree / 2; i++) {
        if (cur < best) best = cur;
        cur = mul_mod(cur, sq, q);
    }
    root = best;
    return true;
}

std::vector<int> naf(int value) {
    std::vector<int> res;
    const bool sign = value < 0;
    unsigned v = (unsigned)std::abs(value);
    for (int i = 0; v; i++) {
        int zi = (v & 1u) ? 2 - (int)(v & 3u) : 0;
        v = (unsigned)((int)v - zi) >> 1;
        if (zi) res.push_back((sign ? -zi : zi) * (1 << i));
    }
    return res;
}

void Modulus::set_value(uint64_t value) {
    if (value == 0) {
        value_ = 0; ratio_[0] = ratio_[1] = 0; bit_count_ = 0; prime_ = false;
        return;
    }
    if ((value >> 61) != 0 || value == 1) throw std::invalid_argument("value can be at most 61-bit and cannot be 1");
    value_ = value;
    bit_count_ = significant_bits(value);
    // floor(2^128 / value) by two rounds of 128/64 division
    const u128 hi_part = (~(u128)0) / value;          // floor((2^128 - 1) / value)
    const u128 rem = (~(u128)0) - hi_part * value;    // (2^128 - 1) mod value
    const u128 ratio = hi_part + ((rem + 1 == value) ? 1 : 0);
    ratio_[0] = (uint64_t)ratio;
    ratio_[1] = (uint64_t)(ratio >> 64);
    prime_ = cahel::is_prime(value);
}

int CoeffModulus::MaxBitCount(size_t n, int sec) {
    static const std::map<size_t, int> t128 = {{1024, 27}, {2048, 54}, {4096, 109}, {8192, 218}, {16384, 438},
                                               {32768, 881}, {65536, 1777}, {131072, 3576}};
    static const std::map<size_t, int> t192 = {{1024, 19}, {2048, 37}, {4096, 75}, {8192, 151}, {16384, 304},
                                               {32768, 611}, {65536, 1229}, {131072, 2469}};
    static const std::map<size_t, int> t256 = {{1024, 14}, {2048, 29}, {4096, 58}, {8192, 118}, {16384, 237},
                                               {32768, 476}, {65536, 955}, {131072, 1918}};
    const std::map<size_t, int> *t = sec == 128 ? &t128 : sec == 192 ? &t192 : sec == 256 ? &t256 : nullptr;
    if (!t) return 0;
    auto it = t->find(n);
    return it == t->end() ? 0 : it->second;
}

std::vector<Modulus> CoeffModulus::Create(size_t n, std::vector<int> bit_sizes) {
    if (n < 2 || n > 131072 || power_of_two(n) < 0) throw std::invalid_argument("poly_modulus_degree is invalid");
    if (bit_sizes.size() > 64) throw std::invalid_argument("bit_sizes is invalid");
    for (int b : bit_sizes)
        if (b > 60 || b < 2) throw std::invalid_argument("bit_sizes is invalid");
    std::map<int, size_t> counts;
    for (int b : bit_sizes) counts[b]++;
    std::map<int, std::vector<uint64_t>> primes;
    std::map<int, size_t> next;
    for (auto &kv : counts) primes[kv.first] = get_primes(n, kv.first, kv.second);
    std::vector<Modulus> out;
    for (int b : bit_sizes) out.emplace_back(primes[b][next[b]++]);
    return out;
}

// ---- BigUInt ----
void BigUInt::trim() {
    while (!w_.empty() && w_.back() == 0) w_.pop_back();
}

BigUInt BigUInt::product(const std::vector<uint64_t> &factors) {
    BigUInt r(1);
    for (uint64_t f : factors) r.mul_u64(f);
    return r;
}

void BigUInt::mul_u64(uint64_t m) {
    uint64_t carry = 0;
    for (auto &w : w_) {
        u128 p = (u128)w * m + carry;
        w = (uint64_t)p;
        carry = (uint64_t)(p >> 64);
    }
    if (carry) w_.push_back(carry);
    trim();
}

void BigUInt::add_mul_u64(const BigUInt &a, uint64_t m) {
    if (w_.size() < a.w_.size() + 1) w_.resize(a.w_.size() + 1, 0);
    uint64_t carry = 0;
    size_t i = 0;
    for (; i < a.w_.size(); i++) {
        u128 p = (u128)a.w_[i] * m + w_[i] + carry;
        w_[i] = (uint64_t)p;
        carry = (uint64_t)(p >> 64);
    }
    for (; carry; i++) {
        if (i == w_.size()) w_.push_back(0);
        u128 p = (u128)w_[i] + carry;
        w_[i] = (uint64_t)p;
        carry = (uint64_t)(p >> 64);
    }
    trim();
}

void BigUInt::add(const BigUInt &a) { add_mul_u64(a, 1); }

void BigUInt::sub(const BigUInt &a) {
    uint64_t borrow = 0;
    for (size_t i = 0; i < w_.size(); i++) {
        uint64_t s = i < a.w_.size() ? a.w_[i] : 0;
        u128 d = (u128)w_[i] - s - borrow;
        w_[i] = (uint64_t)d;
        borrow = (uint64_t)(d >> 64) ? 1 : 0;
    }
    trim();
}

int BigUInt::compare(const BigUInt &a) const {
    if (w_.size() != a.w_.size()) return w_.size() < a.w_.size() ? -1 : 1;
    for (size_t i = w_.size(); i-- > 0;)
        if (w_[i] != a.w_[i]) return w_[i] < a.w_[i] ? -1 : 1;
    return 0;
}

void BigUInt::shift_right1() {
    uint64_t carry = 0;
    for (size_t i = w_.size(); i-- > 0;) {
        uint64_t next = w_[i] & 1;
        w_[i] = (w_[i] >> 1) | (carry << 63);
        carry = next;
    }
    trim();
}

uint64_t BigUInt::mod_u64(uint64_t q) const {
    u128 r = 0;
    for (size_t i = w_.size(); i-- > 0;) r = ((r << 64) | w_[i]) % q;
    return (uint64_t)r;
}

int BigUInt::bit_count() const { return w_.empty() ? 0 : (int)(64 * (w_.size() - 1)) + significant_bits(w_.back()); }

double BigUInt::to_double() const {
    double r = 0.0;
    for (size_t i = w_.size(); i-- > 0;) r = r * 18446744073709551616.0 + (double)w_[i];
    return r;
}

void BigUInt::reduce_small(const BigUInt &m) {
    while (compare(m) >= 0) sub(m);
}

// ---------------------------------------------------------------------------------------------------
// BLAKE2b, RFC 7693 section 3: 12 rounds of the mixing function G over a 16-word working vector, message
// words chosen by the SIGMA schedule, little-endian words throughout.
// ---------------------------------------------------------------------------------------------------
namespace {

constexpr uint64_t kBlakeIv[8] = {0x6a09e667f3bcc908ull, 0xbb67ae8584caa73bull, 0x3c6ef372fe94f82bull,
                                  0xa54ff53a5f1d36f1ull, 0x510e527fade682d1ull, 0x9b05688c2b3e6c1full,
                                  0x1f83d9abfb41bd6bull, 0x5be0cd19137e2179ull};

constexpr uint8_t kBlakeSigma[10][16] = {
    {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3},
    {11, 8, 12, 0, 5, 2, 15, 13, 10, 14, 3, 6, 7, 1, 9, 4}, {7, 9, 3, 1, 13, 12, 11, 14, 2, 6, 5, 10, 4, 0, 15, 8},
    {9, 0, 5, 7, 2, 4, 10, 15, 14, 1, 11, 12, 6, 8, 3, 13}, {2, 12, 6, 10, 0, 11, 8, 3, 4, 13, 7, 5, 15, 14, 1, 9},
    {12, 5, 1, 15, 14, 13, 4, 10, 0, 7, 6, 3, 9, 2, 8, 11}, {13, 11, 7, 14, 12, 1, 3, 9, 5, 0, 15, 4, 8, 6, 2, 10},
    {6, 15, 14, 9, 11, 3, 0, 8, 12, 2, 13, 7, 1, 4, 10, 5}, {10, 2, 8, 4, 7, 6, 1, 5, 15, 11, 9, 14, 3, 12, 13, 0}};

inline uint64_t rotr64(uint64_t v, int r) { return (v >> r) | (v << (64 - r)); }

// one 128-byte block; t = bytes hashed so far including this block (below 2^64 here), last = final block
void blake_compress(uint64_t h[8], const uint8_t block[128], uint64_t t, bool last) {
    uint64_t m[16], v[16];
    for (int i = 0; i < 16; i++) {
        uint64_t w = 0;
        for (int b = 7; b >= 0; b--) w = (w << 8) | block[8 * i + b];
        m[i] = w;
    }
    for (int i = 0; i < 8; i++) {
        v[i] = h[i];
        v[i + 8] = kBlakeIv[i];
    }
    v[12] ^= t;
    if (last) v[14] = ~v[14];
    auto g = [&](int a, int b, int c, int d, uint64_t x, uint64_t y) {
        v[a] = v[a] + v[b] + x;
        v[d] = rotr64(v[d] ^ v[a], 32);
        v[c] = v[c] + v[d];
        v[b] = rotr64(v[b] ^ v[c], 24);
        v[a] = v[a] + v[b] + y;
        v[d] = rotr64(v[d] ^ v[a], 16);
        v[c] = v[c] + v[d];
        v[b] = rotr64(v[b] ^ v[c], 63);
    };
    for (int r = 0; r < 12; r++) {
        const uint8_t *s = kBlakeSigma[r % 10];
        g(0, 4, 8, 12, m[s[0]], m[s[1]]);
        g(1, 5, 9, 13, m[s[2]], m[s[3]]);
        g(2, 6, 10, 14, m[s[4]], m[s[5]]);
        g(3, 7, 11, 15, m[s[6]], m[s[7]]);
        g(0, 5, 10, 15, m[s[8]], m[s[9]]);
        g(1, 6, 11, 12, m[s[10]], m[s[11]]);
        g(2, 7, 8, 13, m[s[12]], m[s[13]]);
        g(3, 4, 9, 14, m[s[14]], m[s[15]]);
    }
    for (int i = 0; i < 8; i++) h[i] ^= v[i] ^ v[i + 8];
}

}  // namespace

void blake2b(void *out, size_t out_len, const void *in, size_t in_len) {
    if (!out || out_len == 0 || out_len > 64 || (!in && in_len)) throw std::invalid_argument("blake2b: invalid argument");
    uint64_t h[8];
    for (int i = 0; i < 8; i++) h[i] = kBlakeIv[i];
    h[0] ^= 0x01010000ull ^ (uint64_t)out_len;  // parameter block: digest length, no key, fanout = depth = 1
    const uint8_t *src = static_cast<const uint8_t *>(in);
    uint64_t done = 0;
    // every block but the last (the last one is padded with zeros and may be empty only for an empty message)
    while (in_len - done > 128) {
        done += 128;
        blake_compress(h, src + done - 128, done, false);
    }
    uint8_t tail[128] = {0};
    for (size_t i = 0; i < in_len - done; i++) tail[i] = src[done + i];
    blake_compress(h, tail, in_len, true);
    uint8_t *dst = static_cast<uint8_t *>(out);
    for (size_t i = 0; i < out_len; i++) dst[i] = (uint8_t)(h[i / 8] >> (8 * (i % 8)));
}

}  // namespace cahel
