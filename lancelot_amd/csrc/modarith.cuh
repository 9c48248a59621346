// Device-side 64-bit modular arithmetic for gfx950 (wave64, VALU integer multiplies).
//
// All routines work on residues of primes below 2^61.  "lazy" values live in [0, 2q) or [0, 4q) and
// never leave a kernel: every store to HBM that a caller can observe is the canonical residue, which
// is what makes limb-for-limb comparison with the CPU checker meaningful.
//
// Semantics follow cahel-main/include/uintmodmath.cuh (Shoup :226-245, Barrett :112-218) and
// cahel-main/src/ntt/butterfly.cuh:10-43 (Harvey butterflies); the code is written for the CDNA4
// integer pipeline (64x64 products are assembled from v_mad_u64_u32 by the compiler).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace he {

struct Shoup {
    uint64_t w;   // operand in [0, q)
    uint64_t wq;  // floor(w * 2^64 / q)
};

__device__ __forceinline__ uint64_t mulhi64(uint64_t a, uint64_t b) { return __umul64hi(a, b); }

// x * w mod q up to one subtraction of q: result in [0, 2q).  x may be any 64-bit value.
__device__ __forceinline__ uint64_t mul_shoup_lazy(uint64_t x, Shoup s, uint64_t q) {
    uint64_t hi = mulhi64(x, s.wq);
    return x * s.w - hi * q;
}

__device__ __forceinline__ uint64_t mul_shoup(uint64_t x, Shoup s, uint64_t q) {
    uint64_t r = mul_shoup_lazy(x, s, q);
    return r >= q ? r - q : r;
}

__device__ __forceinline__ uint64_t add_mod(uint64_t a, uint64_t b, uint64_t q) {
    uint64_t s = a + b;
    return s >= q ? s - q : s;
}

__device__ __forceinline__ uint64_t sub_mod(uint64_t a, uint64_t b, uint64_t q) {
    return a >= b ? a - b : a + q - b;
}

__device__ __forceinline__ uint64_t neg_mod(uint64_t a, uint64_t q) { return a ? q - a : 0; }

// 128-bit value (hi:lo) mod q with ratio = floor(2^128 / q) = (r1:r0), q < 2^62.  r1 = floor(2^64 / q), so
// w = 2^64 mod q = 2^64 - r1 q, and r0 = floor(2^128 / q) - r1 2^64 = floor(w 2^64 / q) is the Shoup quotient of w:
// hi w - floor(hi r0 / 2^64) q lies in [0, 2q) for every hi below 2^64, and lo - floor(lo r1 / 2^64) q in [0, 2q).
// Two high and three low 64-bit products (w comes from scalar operands) where the plain Barrett reduction of the
// 128-bit value takes four and four.
__device__ __forceinline__ uint64_t barrett128(uint64_t lo, uint64_t hi, uint64_t q, uint64_t r0, uint64_t r1) {
    const uint64_t w = 0 - r1 * q;
    const uint64_t a = hi * w - mulhi64(hi, r0) * q;
    const uint64_t b = lo - mulhi64(lo, r1) * q;
    const uint64_t q2 = q << 1;
    uint64_t r = a + b;
    r = r >= q2 ? r - q2 : r;
    return r >= q ? r - q : r;
}

__device__ __forceinline__ uint64_t mul_mod(uint64_t a, uint64_t b, uint64_t q, uint64_t r0, uint64_t r1) {
    return barrett128(a * b, mulhi64(a, b), q, r0, r1);
}

// 64-bit value mod q with r1 = floor(2^64 / q).
__device__ __forceinline__ uint64_t barrett64(uint64_t x, uint64_t q, uint64_t r1) {
    uint64_t r = x - mulhi64(r1, x) * q;
    return r >= q ? r - q : r;
}

struct U128 {
    uint64_t lo, hi;
};

__device__ __forceinline__ void mac128(U128 &acc, uint64_t a, uint64_t b) {
    uint64_t lo = a * b;
    uint64_t hi = mulhi64(a, b);
    acc.lo += lo;
    acc.hi += hi + (acc.lo < lo);
}

// Lazy sum of products of residues below 2^61 with few carries.  The factors are split at bit 30
// (a = a1 2^30 + a0 with a0 < 2^30, a1 < 2^31); the four partial products of a term go, by weight, into three
// 64-bit words (ll: a0 b0 < 2^60, mid: a1 b0 + a0 b1 < 2^62, hh: a1 b1 < 2^62), each a 32 x 32 + 64 multiply-add with
// no carry out.  Four terms fit (4 * 2^62 = 2^64) before the words have to be relieved (spill3), eight when the
// residues are below 2^60 (a1 < 2^30: mid < 2^61, hh < 2^60), so a product costs 4 multiply-adds and a few
// additions instead of a 64 x 64 -> 128 product (6 multiplies) and a carry chain.  (Measured on gfx950: every
// 32-bit multiply, v_mad_u64_u32 included, issues at the rate of an FP64 fused multiply-add, half the rate of a
// 32-bit addition.)
struct Split30 {
    uint32_t lo, hi;
};

__device__ __forceinline__ Split30 split30(uint64_t a) { return Split30{(uint32_t)a & 0x3fffffffu, (uint32_t)(a >> 30)}; }

struct Lazy3 {
    uint64_t ll, mid, hh;
};

// One term for two sums that share the factor a (the two key polynomials of an inner product): eight
// v_mad_u64_u32 (32 x 32 + 64 -> 64; the carry out goes to a scalar pair that nobody reads, the sums stay below
// 2^64).  Written out because the compiler emits a multiply with a zero addend followed by a 64-bit add for
// `acc += (uint64_t)a * b`, and one statement because it separates inline-assembly statements by s_nop.
__device__ __forceinline__ void mac3x2(Lazy3 &s, Lazy3 &t, Split30 a, Split30 b, Split30 c) {
    uint64_t carry;
    asm("v_mad_u64_u32 %0, %6, %7, %9, %0\n\t"
        "v_mad_u64_u32 %1, %6, %8, %9, %1\n\t"
        "v_mad_u64_u32 %2, %6, %8, %10, %2\n\t"
        "v_mad_u64_u32 %3, %6, %7, %11, %3\n\t"
        "v_mad_u64_u32 %4, %6, %8, %11, %4\n\t"
        "v_mad_u64_u32 %5, %6, %8, %12, %5\n\t"
        "v_mad_u64_u32 %1, %6, %7, %10, %1\n\t"
        "v_mad_u64_u32 %4, %6, %7, %12, %4"
        : "+v"(s.ll), "+v"(s.mid), "+v"(s.hh), "+v"(t.ll), "+v"(t.mid), "+v"(t.hh), "=&s"(carry)
        : "v"(a.lo), "v"(a.hi), "v"(b.lo), "v"(b.hi), "v"(c.lo), "v"(c.hi));
}

// The upper halves of the three words move into three counters of weight 2^32 (two additions and a move per word:
// no carries between the words), which leaves room for the next four (eight) terms; total3 puts the six words
// together at the end.  Up to 64 terms (the counters stay below 2^37).
__device__ __forceinline__ void spill3(Lazy3 &h, Lazy3 &s) {
    h.ll += s.ll >> 32;
    s.ll &= 0xffffffffu;
    h.mid += s.mid >> 32;
    s.mid &= 0xffffffffu;
    h.hh += s.hh >> 32;
    s.hh &= 0xffffffffu;
}

__device__ __forceinline__ U128 total3(const Lazy3 &h, const Lazy3 &s) {
    typedef unsigned __int128 u128;
    const u128 t = ((u128)s.ll + ((u128)h.ll << 32)) + (((u128)s.mid + ((u128)h.mid << 32)) << 30) +
                   (((u128)s.hh + ((u128)h.hh << 32)) << 60);
    return U128{(uint64_t)t, (uint64_t)(t >> 64)};
}

// The butterflies' view of a modulus: q, 2q and their negatives modulo 2^64.  With the negatives at hand a Shoup
// product is y w + hi (2^64 - q) and a conditional subtraction is x + (2^64 - 2q) followed by a select on the sign, i.e.
// 64-bit additions (one instruction each) where subtractions would be borrow chains through VCC, which on this GPU need
// two idle issue slots between producer and consumer.  The negatives pass through an empty asm statement so that the
// compiler does not fold them back into subtractions: 37 -> 31 instructions per butterfly.
struct IntMod {
    uint64_t q, q2, nq, nq2;
};

// (q is the same in every lane of a wave: a workgroup works on one limb; read from lane 0 so that the constants are
// scalars wherever the compiler cannot see that)
__device__ __forceinline__ IntMod int_mod(uint64_t q_any_lane) {
    const uint32_t q_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(q_any_lane >> 32));
    const uint32_t q_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)q_any_lane);   // (the builtin returns int)
    const uint64_t q = ((uint64_t)q_hi << 32) | q_lo;
    // (as 32-bit scalars)
    uint32_t a0 = (uint32_t)(0 - q), a1 = (uint32_t)((0 - q) >> 32);
    uint32_t b0 = (uint32_t)(0 - (q << 1)), b1 = (uint32_t)((0 - (q << 1)) >> 32);
    asm volatile("" : "+s"(a0), "+s"(a1), "+s"(b0), "+s"(b1));
    return IntMod{q, q << 1, ((uint64_t)a1 << 32) | a0, ((uint64_t)b1 << 32) | b0};
}

// y w mod q up to one subtraction of q, in [0, 2q), for any 64-bit y
__device__ __forceinline__ uint64_t mul_shoup_lazy(uint64_t y, Shoup s, const IntMod &m) {
    return y * s.w + mulhi64(y, s.wq) * m.nq;
}

// v - 2q if that is not negative, else v (v below 2^63)
__device__ __forceinline__ uint64_t reduce_once_2q(uint64_t v, const IntMod &m) {
    const uint64_t d = v + m.nq2;
    return (int64_t)d < 0 ? v : d;
}

// Cooley-Tukey butterfly, inputs in [0, 4q), outputs in [0, 4q).
__device__ __forceinline__ void ct_butterfly(uint64_t &x, uint64_t &y, Shoup tw, const IntMod &m) {
    const uint64_t t = mul_shoup_lazy(y, tw, m);
    const uint64_t xr = reduce_once_2q(x, m);
    y = (xr + m.q2) - t;
    x = xr + t;
}

// Gentleman-Sande butterfly with the division by two folded in (the inverse twiddles are stored
// pre-halved), inputs in [0, 2q), outputs in [0, 2q).
__device__ __forceinline__ void gs_butterfly(uint64_t &x, uint64_t &y, Shoup tw, const IntMod &m) {
    const uint64_t d = x + m.q2 - y;
    uint64_t s = reduce_once_2q(x + y, m);
    s += (d & 1) ? m.q : 0;
    x = s >> 1;
    y = mul_shoup_lazy(d, tw, m);
}

__device__ __forceinline__ uint64_t reduce_4q(uint64_t v, uint64_t q) {
    uint64_t q2 = q << 1;
    v = v >= q2 ? v - q2 : v;
    return v >= q ? v - q : v;
}

__device__ __forceinline__ uint64_t reduce_2q(uint64_t v, uint64_t q) { return v >= q ? v - q : v; }

__device__ __forceinline__ Shoup load_shoup(const uint64_t *table, size_t idx) {
    const ulonglong2 v = reinterpret_cast<const ulonglong2 *>(table)[idx];
    return Shoup{v.x, v.y};
}

// NTT-domain automorphism X -> X^elt as a gather: out[i] = in[pi(i)],
// pi(i) = bitrev(((elt * (2 bitrev(i) + 1)) >> 1) mod N)   (table of cahel-main/include/galois.cuh:45-57, on the fly)
__device__ __forceinline__ uint32_t galois_index(uint32_t i, uint32_t elt, uint32_t log_n) {
    const uint32_t r = __brev(i) >> (32 - log_n);
    const uint32_t raw = (uint32_t)(((uint64_t)elt * (2 * r + 1)) >> 1) & ((1u << log_n) - 1);
    return __brev(raw) >> (32 - log_n);
}

// R = 2^LOGR point decimation-in-time block: LOGR consecutive forward stages on register values.
// v[j] are the elements whose index differs in the LOGR bits that these stages pair, most significant
// first; idx = 2^s0 + (group number at the first stage s0); twiddle of local stage l, sub-block b is
// table[(idx << l) + b].
template <int LOGR>
__device__ __forceinline__ void ct_block(uint64_t *v, const uint64_t *table, uint32_t idx, uint64_t q) {
    constexpr int R = 1 << LOGR;
    const IntMod m = int_mod(q);
#pragma unroll
    for (int l = 0; l < LOGR; l++) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            Shoup tw = load_shoup(table, ((size_t)idx << l) + b);
#pragma unroll
            for (int j = 0; j < half; j++) ct_butterfly(v[2 * b * half + j], v[2 * b * half + j + half], tw, m);
        }
    }
}

// The mirror image: the same LOGR stages in inverse order with Gentleman-Sande butterflies.
template <int LOGR>
__device__ __forceinline__ void gs_block(uint64_t *v, const uint64_t *table, uint32_t idx, uint64_t q) {
    constexpr int R = 1 << LOGR;
    const IntMod m = int_mod(q);
#pragma unroll
    for (int l = LOGR - 1; l >= 0; l--) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            Shoup tw = load_shoup(table, ((size_t)idx << l) + b);
#pragma unroll
            for (int j = 0; j < half; j++) gs_butterfly(v[2 * b * half + j], v[2 * b * half + j + half], tw, m);
        }
    }
}

}  // namespace he

// ---------------------------------------------------------------------------------------------------
// FP64 modular arithmetic for primes below 2^50.
//
// v_fma_f64 / v_mul_f64 / v_add_f64 run at full rate on CDNA4, so a modular product costs six
// operations instead of the ~20 of a 64-bit Shoup product.  Every value is an integer held exactly
// in a double; residues are signed and lazy (|v| < 2^53).  All steps below are exact integer
// computations, so the canonical result equals the integer path's bit for bit.
//
//   x * w = h + l exactly (h = fl(x w), l = fma(x, w, -h)); k = rint(x * winv), winv ~ w/q with
//   relative error at most 2^-52, differs from x w / q by at most 1/2 + 1.5 |x| 2^-52; h - k q and
//   (h - k q) + l are integers below 2^53 in magnitude, hence exact; the result is congruent to x w
//   with |r| <= (1/2 + 1.5 |x| 2^-52) q, i.e. (1/2 + 0.375 b) q for |x| <= b q, q < 2^50.
// ---------------------------------------------------------------------------------------------------
namespace he {

struct FpMod {
    double q, qinv;
};

struct FpTw {
    double w, winv;
};

// canonical residue (< 2^52) <-> exact double, through the exponent-bias trick
__device__ __forceinline__ double fp_from_u64(uint64_t x) {
    return __longlong_as_double((long long)(x | 0x4330000000000000ull)) - 4503599627370496.0;
}

__device__ __forceinline__ uint64_t fp_to_u64(double c) {  // 0 <= c < 2^52, integer
    return (uint64_t)__double_as_longlong(c + 4503599627370496.0) & 0x000FFFFFFFFFFFFFull;
}

__device__ __forceinline__ double fp_mulmod(double x, FpTw t, FpMod m) {
    const double k = __builtin_rint(x * t.winv);
    const double h = x * t.w;
    const double l = __builtin_fma(x, t.w, -h);
    return __builtin_fma(-k, m.q, h) + l;
}

// centred representative, |result| <= (1/2 + 2^-49) q for |v| < 2^53
__device__ __forceinline__ double fp_reduce(double v, FpMod m) {
    const double k = __builtin_rint(v * m.qinv);
    return __builtin_fma(-k, m.q, v);
}

// canonical residue in [0, q) as an exact double
__device__ __forceinline__ double fp_canonical(double v, FpMod m) {
    const double c = fp_reduce(v, m);
    return c < 0.0 ? c + m.q : c;
}

// Twiddle tables hold w only (8 bytes per entry: the tables are as large as the data they transform, so
// their size is HBM traffic); the quotient estimate w * fl(1/q) has relative error 2^-52, which with the
// rounding of x * winv puts k within 1/2 + 1.5 |x| 2^-52 of x w / q.
__device__ __forceinline__ FpTw load_fptw(const double *table, size_t idx, FpMod m) {
    const double w = table[idx];
    return FpTw{w, w * m.qinv};
}

// Forward block on lazy signed doubles.  REDUCE_FIRST = 1 brings every input back to |v| <= q/2; from there
// (or from canonical inputs) the bound grows by 1.375 b + 0.5 per stage: 5.3 q after four stages, 7.1 q from
// canonical inputs, always below 8 q < 2^53.
// REDUCE_FIRST = 2 reduces only the inputs that the first stage adds and subtracts; those that it multiplies go into
// the modular product as they are (its result is at most (1/2 + 0.375 b) 2^50 for an input of b 2^50).  In units of
// 2^50, for every q below 2^50: the first stage ends at 1 + 0.375 b and each later one at 1.375 b' + 0.5, which
// is 5.92 after three stages from inputs of 4, 7.28 after three more, 5.63 after two more: for a chain of blocks of
// at most 3, 3 and 2 stages whose first inputs are at most 4 x 2^50, and whose consumer reduces first.
template <int LOGR, int REDUCE_FIRST>
__device__ __forceinline__ void fp_ct_block(double *v, const double *table, uint32_t idx, FpMod m) {
    constexpr int R = 1 << LOGR;
    static_assert(REDUCE_FIRST != 2 || LOGR <= 3, "bounds of the partial reduction are derived for blocks of at most 3 stages");
    if (REDUCE_FIRST) {
#pragma unroll
        for (int j = 0; j < (REDUCE_FIRST == 2 ? R / 2 : R); j++) v[j] = fp_reduce(v[j], m);
    }
#pragma unroll
    for (int l = 0; l < LOGR; l++) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            const FpTw tw = load_fptw(table, ((size_t)idx << l) + b, m);
#pragma unroll
            for (int j = 0; j < half; j++) {
                const double x = v[2 * b * half + j];
                const double t = fp_mulmod(v[2 * b * half + j + half], tw, m);
                v[2 * b * half + j] = x + t;
                v[2 * b * half + j + half] = x - t;
            }
        }
    }
}

// Inverse block (no halving: the factor 1/N is applied once at the end of the transform).  Sums double
// per stage, so in blocks of four or five stages the sum outputs are reduced again after every second stage (not
// after the last); outputs stay at or below 5 q (8 q from canonical inputs without REDUCE_FIRST), which is below 2^53.
template <int LOGR, bool REDUCE_FIRST>
__device__ __forceinline__ void fp_gs_block(double *v, const double *table, uint32_t idx, FpMod m) {
    constexpr int R = 1 << LOGR;
    if (REDUCE_FIRST) {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = fp_reduce(v[j], m);
    }
#pragma unroll
    for (int l = LOGR - 1; l >= 0; l--) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            const FpTw tw = load_fptw(table, ((size_t)idx << l) + b, m);
#pragma unroll
            for (int j = 0; j < half; j++) {
                const double x = v[2 * b * half + j], y = v[2 * b * half + j + half];
                v[2 * b * half + j] = x + y;
                v[2 * b * half + j + half] = fp_mulmod(x - y, tw, m);
            }
        }
        if (LOGR >= 4 && l > 0 && ((LOGR - l) & 1) == 0) {
#pragma unroll
            for (int b = 0; b < (1 << l); b++)
#pragma unroll
                for (int j = 0; j < half; j++) v[2 * b * half + j] = fp_reduce(v[2 * b * half + j], m);
        }
    }
}

// The same blocks with the 2^LOGR - 1 twiddles already in registers (tw[2^l - 1 + b] for stage l, sub-block b):
// a workgroup that transforms several limbs of one modulus loads them once.
template <int LOGR>
__device__ __forceinline__ void fp_load_block_tw(double *tw, const double *table, uint32_t idx) {
#pragma unroll
    for (int l = 0; l < LOGR; l++)
#pragma unroll
        for (int b = 0; b < (1 << l); b++) tw[(1 << l) - 1 + b] = table[((size_t)idx << l) + b];
}

template <int LOGR, bool REDUCE_FIRST>
__device__ __forceinline__ void fp_ct_block_tw(double *v, const double *tw, FpMod m) {
    constexpr int R = 1 << LOGR;
    if (REDUCE_FIRST) {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = fp_reduce(v[j], m);
    }
#pragma unroll
    for (int l = 0; l < LOGR; l++) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            double w = tw[(1 << l) - 1 + b];
            asm volatile("" : "+v"(w));  // keeps w * qinv out of the caller's loop-invariant registers
            const FpTw t{w, w * m.qinv};
#pragma unroll
            for (int j = 0; j < half; j++) {
                const double x = v[2 * b * half + j];
                const double p = fp_mulmod(v[2 * b * half + j + half], t, m);
                v[2 * b * half + j] = x + p;
                v[2 * b * half + j + half] = x - p;
            }
        }
    }
}

template <int LOGR, bool REDUCE_FIRST>
__device__ __forceinline__ void fp_gs_block_tw(double *v, const double *tw, FpMod m) {
    constexpr int R = 1 << LOGR;
    if (REDUCE_FIRST) {
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = fp_reduce(v[j], m);
    }
#pragma unroll
    for (int l = LOGR - 1; l >= 0; l--) {
        const int half = R >> (l + 1);
#pragma unroll
        for (int b = 0; b < (1 << l); b++) {
            double w = tw[(1 << l) - 1 + b];
            asm volatile("" : "+v"(w));  // keeps w * qinv out of the caller's loop-invariant registers
            const FpTw t{w, w * m.qinv};
#pragma unroll
            for (int j = 0; j < half; j++) {
                const double x = v[2 * b * half + j], y = v[2 * b * half + j + half];
                v[2 * b * half + j] = x + y;
                v[2 * b * half + j + half] = fp_mulmod(x - y, t, m);
            }
        }
        if (LOGR >= 4 && l > 0 && ((LOGR - l) & 1) == 0) {
#pragma unroll
            for (int b = 0; b < (1 << l); b++)
#pragma unroll
                for (int j = 0; j < half; j++) v[2 * b * half + j] = fp_reduce(v[2 * b * half + j], m);
        }
    }
}

}  // namespace he
