// Host-side number theory for the CKKS parameter tables: primes, roots of unity, modular inverses,
// Barrett / Shoup constants, a small unsigned big integer for CRT composition.
//
// Plain C++17, no device code.  Behaviour follows cahel-main/src/modulus.cu (Modulus, CoeffModulus::Create
// :93-133), src/util/numth.cu (is_prime :131-207, get_primes :209-235, try_minimal_primitive_root :311-333,
// naf in include/util/numth.h:18) and include/util/uintarithsmallmod.h:158-180 (Shoup operand).
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

namespace cahel {

using u128 = unsigned __int128;

inline uint64_t mul_mod(uint64_t a, uint64_t b, uint64_t q) { return (uint64_t)((u128)a * b % q); }
uint64_t pow_mod(uint64_t base, uint64_t exp, uint64_t q);
// returns false when gcd(a, q) != 1
bool try_invert_mod(uint64_t a, uint64_t q, uint64_t &result);
uint64_t invert_mod(uint64_t a, uint64_t q);  // throws std::invalid_argument if not invertible

inline uint64_t shoup_quotient(uint64_t w, uint64_t q) { return (uint64_t)(((u128)w << 64) / q); }

int significant_bits(uint64_t v);
inline int power_of_two(uint64_t v) { return (v && !(v & (v - 1))) ? significant_bits(v) - 1 : -1; }
uint32_t reverse_bits(uint32_t x, int bits);

bool is_prime(uint64_t v);
// the `count` largest primes of the form 2^bit_size - k * 2 * ntt_size + 1, descending
std::vector<uint64_t> get_primes(size_t ntt_size, int bit_size, size_t count);
bool is_primitive_root(uint64_t root, uint64_t degree, uint64_t q);
// smallest primitive degree-th root of unity mod q (degree a power of two); false if none exists
bool try_minimal_primitive_root(uint64_t degree, uint64_t q, uint64_t &root);
// non-adjacent form: signed powers of two summing to value, least significant first
std::vector<int> naf(int value);

// BLAKE2b (RFC 7693), unkeyed, digest of 1..64 bytes: the hash behind the parameter identifiers
// (cahel-main/include/util/hash.h:30-37 calls blake2b with a 32-byte digest).
void blake2b(void *out, size_t out_len, const void *in, size_t in_len);

// A modulus below 2^61 with its 128-bit Barrett ratio floor(2^128 / value).
class Modulus {
public:
    Modulus() = default;
    Modulus(uint64_t value) { set_value(value); }  // NOLINT: implicit by design (Python: modulus(int))
    uint64_t value() const { return value_; }
    int bit_count() const { return bit_count_; }
    const uint64_t *const_ratio() const { return ratio_; }
    bool is_zero() const { return value_ == 0; }
    bool is_prime() const { return prime_; }
    bool operator==(const Modulus &o) const { return value_ == o.value_; }
    bool operator!=(const Modulus &o) const { return value_ != o.value_; }

private:
    void set_value(uint64_t value);
    uint64_t value_ = 0;
    uint64_t ratio_[2] = {0, 0};
    int bit_count_ = 0;
    bool prime_ = false;
};

struct CoeffModulus {
    // Upper bound on the total coefficient-modulus bit count for a security level
    // (include/util/hestdparms.h); 0 for an unknown degree.
    static int MaxBitCount(size_t poly_modulus_degree, int sec_level_bits);
    static std::vector<Modulus> Create(size_t poly_modulus_degree, std::vector<int> bit_sizes);
};

// Little-endian unsigned big integer, just enough for CRT composition and bit counts.
class BigUInt {
public:
    BigUInt() = default;
    explicit BigUInt(uint64_t v) : w_{v} { trim(); }
    static BigUInt product(const std::vector<uint64_t> &factors);
    void mul_u64(uint64_t m);
    void add_mul_u64(const BigUInt &a, uint64_t m);  // *this += a * m
    void add(const BigUInt &a);
    void sub(const BigUInt &a);                      // requires *this >= a
    int compare(const BigUInt &a) const;
    void shift_right1();
    uint64_t mod_u64(uint64_t q) const;
    int bit_count() const;
    double to_double() const;
    bool is_zero() const { return w_.empty(); }
    size_t words() const { return w_.size(); }
    // *this mod m by repeated subtraction; requires *this < count * m for a small count
    void reduce_small(const BigUInt &m);

private:
    void trim();
    std::vector<uint64_t> w_;
};

}  // namespace cahel
