// Streaming RNS kernels for gfx950: elementwise polynomial arithmetic, tensor product, NTT-domain Galois
// gather, base conversion (the modular matrix-vector product of ModUp / ModDown), the key-switch inner
// product, and the seeded samplers.  All of them are HBM-bound streams over [limb][coeff] arrays: one
// coefficient per lane, 256 consecutive coefficients per workgroup, so every access is a full-width
// coalesced row segment.
//
// What they compute follows cahel-main/src/polymath.cu (add :40, sub :108, multiply :160, mad :227/:349,
// tensor :531-612), src/galois.cu:20-30 + include/galois.cuh:45-57, src/rns_bconv.cu:587-623 and :166-198
// (base conversion, uncorrected sum, one reduction), src/eval_key_switch.cu:13-76 (inner product) and
// src/prng.cu:143-242 (distributions of the samplers).
#include <cstdlib>
#include <cstring>

#include "kernels.h"
#include "modarith.cuh"

namespace he {

namespace {

constexpr int kThreads = 256;

struct EwArgs {
    const uint64_t *a, *b, *c;
    uint64_t *out;
    const uint64_t *moduli, *barrett;
    LimbMap map;
    uint32_t log_n;
    int op;
};

// grid: (N / 256, limbs, polys)
__global__ __launch_bounds__(kThreads) void elementwise_kernel(EwArgs p) {
    const uint32_t limb = blockIdx.y;
    const uint32_t table = map_table(p.map, limb);
    const uint64_t q = p.moduli[table];
    const size_t idx = (((size_t)blockIdx.z * p.map.limbs + limb) << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    uint64_t r;
    switch (p.op) {
        case EW_ADD: r = add_mod(p.a[idx], p.b[idx], q); break;
        case EW_SUB: r = sub_mod(p.a[idx], p.b[idx], q); break;
        case EW_NEG: r = neg_mod(p.a[idx], q); break;
        case EW_MUL: r = mul_mod(p.a[idx], p.b[idx], q, p.barrett[2 * table], p.barrett[2 * table + 1]); break;
        default: {
            r = add_mod(mul_mod(p.a[idx], p.b[idx], q, p.barrett[2 * table], p.barrett[2 * table + 1]), p.c[idx], q);
            if (p.op == EW_MUL_ADD_NEG) r = neg_mod(r, q);
        }
    }
    p.out[idx] = r;
}

// grid: (N / 256, limbs): out = a + b * w[first + limb]
__global__ __launch_bounds__(kThreads) void scalar_mul_add_kernel(const uint64_t *a, const uint64_t *b, uint64_t *out,
                                                                  const uint64_t *moduli, const uint64_t *w,
                                                                  uint32_t first, uint32_t log_n) {
    const uint32_t table = first + blockIdx.y;
    const uint64_t q = moduli[table];
    const size_t idx = ((size_t)blockIdx.y << log_n) + blockIdx.x * kThreads + threadIdx.x;
    out[idx] = add_mod(a[idx], mul_shoup(b[idx], load_shoup(w, table), q), q);
}

// grid: (N / 256, limbs): residue of a rounded real coefficient
// blockIdx.z = item: coefficient vectors N apart, outputs out_item_stride words apart
__global__ __launch_bounds__(kThreads) void decompose_real_kernel(const double *coeffs, uint64_t *out,
                                                                  const uint64_t *moduli, const uint64_t *barrett,
                                                                  uint32_t first, uint32_t log_n, size_t out_item_stride) {
    const uint32_t table = first + blockIdx.y;
    const uint64_t q = moduli[table];
    const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
    const double c = coeffs[((size_t)blockIdx.z << log_n) + i];
    const uint64_t r = barrett64((uint64_t)fabs(c), q, barrett[2 * table + 1]);
    out[blockIdx.z * out_item_stride + ((size_t)blockIdx.y << log_n) + i] = c < 0 ? neg_mod(r, q) : r;
}

// grid: (N / 256, L + K, items).  wide[item][i][t] += u[item][t] * pk[i][table(t)] for both polynomials of the public
// key: the products of an encryption over Ql u P
__global__ __launch_bounds__(kThreads) void encrypt_fma_kernel(const uint64_t *u, const uint64_t *pk, uint64_t *wide,
                                                               const uint64_t *moduli, const uint64_t *barrett,
                                                               uint32_t L, uint32_t K, uint32_t size_q, uint32_t log_n) {
    const uint32_t t = blockIdx.y, LK = L + K;
    const uint32_t table = t < L ? t : size_q + (t - L);
    const uint64_t q = moduli[table], r0 = barrett[2 * table], r1 = barrett[2 * table + 1];
    const uint32_t j = blockIdx.x * kThreads + threadIdx.x;
    const uint64_t uv = u[(((size_t)blockIdx.z * LK + t) << log_n) + j];
    const size_t key_poly = (size_t)(size_q + K) << log_n;
    const uint64_t *k = pk + ((size_t)table << log_n) + j;
    uint64_t *w = wide + (((size_t)blockIdx.z * 2 * LK + t) << log_n) + j;
    const size_t wpoly = (size_t)LK << log_n;
    w[0] = add_mod(w[0], mul_mod(uv, k[0], q, r0, r1), q);
    w[wpoly] = add_mod(w[wpoly], mul_mod(uv, k[key_poly], q, r0, r1), q);
}

struct TensorArgs {
    const uint64_t *ct1, *ct2;
    uint64_t *out;
    const uint64_t *moduli, *barrett;
    uint32_t L, log_n;
    uint64_t *out2;                           // d2 (out + 2 polynomials for a dense size-3 result)
    size_t in_item_stride, out_item_stride, out2_item_stride;   // blockIdx.z = item (words between items)
};

// grid: (N / 256, L).  Reads the four input limbs once, writes the three outputs: (d0, d1, d2) =
// (a0 b0, a0 b1 + a1 b0, a1 b1); out may alias ct1 (every index is read before it is written).
template <bool SQUARE>
__global__ __launch_bounds__(kThreads) void tensor_kernel(TensorArgs p) {
    const uint32_t limb = blockIdx.y;
    const uint64_t q = p.moduli[limb], r0 = p.barrett[2 * limb], r1 = p.barrett[2 * limb + 1];
    const size_t poly = (size_t)p.L << p.log_n;
    const size_t idx = ((size_t)limb << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    const uint64_t *ct1 = p.ct1 + blockIdx.z * p.in_item_stride, *ct2 = p.ct2 + blockIdx.z * p.in_item_stride;
    uint64_t *out = p.out + blockIdx.z * p.out_item_stride, *out2 = p.out2 + blockIdx.z * p.out2_item_stride;
    const uint64_t a0 = ct1[idx], a1 = ct1[idx + poly];
    uint64_t d0, d1, d2;
    if (SQUARE) {
        d0 = mul_mod(a0, a0, q, r0, r1);
        d2 = mul_mod(a1, a1, q, r0, r1);
        uint64_t m = mul_mod(a0, a1, q, r0, r1);
        d1 = add_mod(m, m, q);
    } else {
        const uint64_t b0 = ct2[idx], b1 = ct2[idx + poly];
        d0 = mul_mod(a0, b0, q, r0, r1);
        d2 = mul_mod(a1, b1, q, r0, r1);
        // Karatsuba: (a0 + a1)(b0 + b1) - d0 - d2; the sums stay below 2^62
        uint64_t m = mul_mod(a0 + a1, b0 + b1, q, r0, r1);
        d1 = sub_mod(sub_mod(m, d0, q), d2, q);
    }
    out[idx] = d0;
    out[idx + poly] = d1;
    out2[idx] = d2;
}

// The same in exact FP64 arithmetic (every prime below 2^50): about 60 instructions per coefficient instead of
// about 260, the same canonical residues.
template <bool SQUARE>
__global__ __launch_bounds__(kThreads) void tensor_fp_kernel(TensorArgs p, const double *fp_consts) {
    const uint32_t limb = blockIdx.y;
    const FpMod m{fp_consts[4 * limb], fp_consts[4 * limb + 1]};
    const size_t poly = (size_t)p.L << p.log_n;
    const size_t idx = ((size_t)limb << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    const uint64_t *ct1 = p.ct1 + blockIdx.z * p.in_item_stride, *ct2 = p.ct2 + blockIdx.z * p.in_item_stride;
    uint64_t *out = p.out + blockIdx.z * p.out_item_stride, *out2 = p.out2 + blockIdx.z * p.out2_item_stride;
    const double a0 = fp_from_u64(ct1[idx]), a1 = fp_from_u64(ct1[idx + poly]);
    double d0, d1, d2;
    if (SQUARE) {
        d0 = fp_canonical(fp_mulmod(a0, FpTw{a0, a0 * m.qinv}, m), m);
        d2 = fp_canonical(fp_mulmod(a1, FpTw{a1, a1 * m.qinv}, m), m);
        const double mm = fp_mulmod(a0, FpTw{a1, a1 * m.qinv}, m);
        d1 = fp_canonical(mm + mm, m);
    } else {
        const double b0 = fp_from_u64(ct2[idx]), b1 = fp_from_u64(ct2[idx + poly]);
        d0 = fp_canonical(fp_mulmod(a0, FpTw{b0, b0 * m.qinv}, m), m);
        d2 = fp_canonical(fp_mulmod(a1, FpTw{b1, b1 * m.qinv}, m), m);
        const double sb = b0 + b1;
        const double mm = fp_mulmod(a0 + a1, FpTw{sb, sb * m.qinv}, m);
        d1 = fp_canonical(mm - d0 - d2, m);
    }
    out[idx] = fp_to_u64(d0);
    out[idx + poly] = fp_to_u64(d1);
    out2[idx] = fp_to_u64(d2);
}

// General tensor product: grid (N / 256, L); ct1 [S1][L][N], ct2 [S2][L][N] -> out [S1 + S2 - 1][L][N],
// out_j = sum over a + b = j of ct1_a * ct2_b with the products summed in 128 bits and reduced once (at most three
// products of 61-bit factors).  Sizes are template parameters: the operands stay in registers, nothing is allocated
// on the device.  out may be ct1's buffer: every coefficient is read before it is written.
template <int S1, int S2>
__global__ __launch_bounds__(kThreads) void tensor_mxn_kernel(TensorArgs p) {
    const uint32_t limb = blockIdx.y;
    const uint64_t q = p.moduli[limb], r0 = p.barrett[2 * limb], r1 = p.barrett[2 * limb + 1];
    const size_t poly = (size_t)p.L << p.log_n;
    const size_t idx = ((size_t)limb << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    uint64_t c1[S1], c2[S2], o[S1 + S2 - 1];
#pragma unroll
    for (int a = 0; a < S1; a++) c1[a] = p.ct1[idx + poly * a];
#pragma unroll
    for (int b = 0; b < S2; b++) c2[b] = p.ct2[idx + poly * b];
#pragma unroll
    for (int j = 0; j < S1 + S2 - 1; j++) {
        U128 acc{0, 0};
#pragma unroll
        for (int a = 0; a < S1; a++)
            if (j - a >= 0 && j - a < S2) mac128(acc, c1[a], c2[j - a]);
        o[j] = barrett128(acc.lo, acc.hi, q, r0, r1);
    }
#pragma unroll
    for (int j = 0; j < S1 + S2 - 1; j++) p.out[idx + poly * j] = o[j];
}

// The same product for operands of any size (run-time sizes, up to 16 polynomials each): nothing is kept in registers,
// the operands are read where they are needed (a coefficient's S1 + S2 words stay in the first-level cache), at most
// 16 products of 61-bit factors are summed in 128 bits per output.  Outputs are formed from the last to the first, so
// that out may be ct1's buffer: output j overwrites word j of ct1, which only the outputs from j on read.
__global__ __launch_bounds__(kThreads) void tensor_any_kernel(TensorArgs p, uint32_t s1, uint32_t s2) {
    const uint32_t limb = blockIdx.y;
    const uint64_t q = p.moduli[limb], r0 = p.barrett[2 * limb], r1 = p.barrett[2 * limb + 1];
    const size_t poly = (size_t)p.L << p.log_n;
    const size_t idx = ((size_t)limb << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    for (uint32_t j = s1 + s2 - 1; j-- > 0;) {
        const uint32_t a_first = j >= s2 ? j - (s2 - 1) : 0, a_last = j < s1 ? j : s1 - 1;
        U128 acc{0, 0};
        for (uint32_t a = a_first; a <= a_last; a++) mac128(acc, p.ct1[idx + poly * a], p.ct2[idx + poly * (j - a)]);
        p.out[idx + poly * j] = barrett128(acc.lo, acc.hi, q, r0, r1);
    }
}

// grid: (N / 256, limbs, items).  out[item][limb] = c0 + c1 * s (+ noise[item][limb]) for the ciphertext cts[item]
__global__ __launch_bounds__(kThreads) void decrypt_gather_kernel(const uint64_t *const *cts, const uint64_t *sk,
                                                                  const uint64_t *noise, uint64_t *out,
                                                                  const uint64_t *moduli, const uint64_t *barrett,
                                                                  uint32_t limbs, uint32_t log_n) {
    const uint32_t limb = blockIdx.y;
    const uint64_t q = moduli[limb], r0 = barrett[2 * limb], r1 = barrett[2 * limb + 1];
    const size_t idx = ((size_t)limb << log_n) + blockIdx.x * kThreads + threadIdx.x;
    const size_t poly = (size_t)limbs << log_n;
    const uint64_t *ct = cts[blockIdx.z];
    uint64_t v = add_mod(ct[idx], mul_mod(ct[idx + poly], sk[idx], q, r0, r1), q);
    const size_t o = (size_t)blockIdx.z * poly + idx;
    if (noise) v = add_mod(v, noise[o], q);
    out[o] = v;
}

struct PairSquareArgs {
    const uint64_t *const *pairs;   // device array [items][chunks][2] of ciphertext pointers, each [2][L][N]
    uint64_t *out01, *out2;         // [items][2][L][N] (d0, d1) and [items][L][N] (d2)
    const uint64_t *moduli, *barrett;
    uint32_t L, log_n, chunks;
};

// grid: (N / 256, L, items).  (d0, d1 | d2)[item] = sum over chunks of (a - b)^2 as a size-3 ciphertext, for the pair
// (a, b) of every chunk: the subtraction, the tensor square and the accumulation of the lazily relinearised
// squared distance in one pass over the inputs.  d2, the key-switch input, goes to a buffer of its own so that
// (d0, d1) is a dense batch of size-2 ciphertexts.
__global__ __launch_bounds__(kThreads) void pair_square_sum_kernel(PairSquareArgs p) {
    const uint32_t limb = blockIdx.y;
    const uint64_t q = p.moduli[limb], r0 = p.barrett[2 * limb], r1 = p.barrett[2 * limb + 1];
    const size_t poly = (size_t)p.L << p.log_n;
    const size_t idx = ((size_t)limb << p.log_n) + blockIdx.x * kThreads + threadIdx.x;
    const uint64_t *const *pair = p.pairs + (size_t)blockIdx.z * p.chunks * 2;
    uint64_t d0 = 0, d1 = 0, d2 = 0;
    for (uint32_t c = 0; c < p.chunks; c++) {
        const uint64_t *a = pair[2 * c], *b = pair[2 * c + 1];
        const uint64_t x0 = sub_mod(a[idx], b[idx], q), x1 = sub_mod(a[idx + poly], b[idx + poly], q);
        d0 = add_mod(d0, mul_mod(x0, x0, q, r0, r1), q);
        d2 = add_mod(d2, mul_mod(x1, x1, q, r0, r1), q);
        const uint64_t m = mul_mod(x0, x1, q, r0, r1);
        d1 = add_mod(d1, add_mod(m, m, q), q);
    }
    uint64_t *out = p.out01 + (size_t)blockIdx.z * 2 * poly;
    out[idx] = d0;
    out[idx + poly] = d1;
    p.out2[(size_t)blockIdx.z * poly + idx] = d2;
}

// grid: (N / 256, total limbs)
__global__ __launch_bounds__(kThreads) void galois_kernel(const uint64_t *in, uint64_t *out, uint32_t elt,
                                                          uint32_t log_n) {
    const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
    const size_t base = (size_t)blockIdx.y << log_n;
    out[base + i] = in[base + galois_index(i, elt, log_n)];
}

// Base conversion of one digit: thread = one coefficient x kRows output limbs.
constexpr int kRows = 4;

struct BconvKArgs {
    BconvArgs a;
    const uint64_t *moduli, *barrett;
    uint32_t log_n;
};

template <int NIN>
__global__ __launch_bounds__(kThreads) void bconv_kernel(BconvKArgs p) {
    const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const uint32_t n_in = NIN > 0 ? NIN : p.a.n_in;
    uint64_t x[NIN > 0 ? NIN : 1];
    if (NIN > 0) {
#pragma unroll
        for (int i = 0; i < NIN; i++) x[i] = p.a.x[((size_t)i << p.log_n) + j];
    }
    for (uint32_t rr = 0; rr < kRows; rr++) {
        const uint32_t row = blockIdx.y * kRows + rr;
        if (row >= p.a.n_out) return;
        const uint64_t *m = p.a.mat + (size_t)row * n_in;
        U128 acc{0, 0};
        if (NIN > 0) {
#pragma unroll
            for (int i = 0; i < NIN; i++) mac128(acc, x[i], m[i]);
        } else {
            for (uint32_t i = 0; i < n_in; i++) mac128(acc, p.a.x[((size_t)i << p.log_n) + j], m[i]);
        }
        const uint32_t t = p.a.out_table[row];
        p.a.out[((size_t)p.a.out_limb[row] << p.log_n) + j] =
            barrett128(acc.lo, acc.hi, p.moduli[t], p.barrett[2 * t], p.barrett[2 * t + 1]);
    }
}

// output limbs per thread in the batched base conversion: the inputs are re-read once per row group

constexpr int kBatchIn = 8;

struct BconvBatchK {
    BconvBatch b;
    const uint64_t *moduli, *barrett;
    uint32_t log_n, compute_groups, rows_per;
};

// grid: (N / 256, compute groups + copy groups, units); thread = one coefficient x kBatchRows output limbs
__global__ __launch_bounds__(kThreads) void bconv_batched_kernel(BconvBatchK p) {
    const uint32_t item = blockIdx.z / p.b.n_units;
    const BconvDesc d = p.b.descs[blockIdx.z - item * p.b.n_units];
    const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
    uint64_t *out = p.b.out_base + item * p.b.out_item_stride + d.out_off;
    if (blockIdx.y >= p.compute_groups) {
        // limbs that pass through unchanged
        const uint64_t *from = p.b.copy_base + item * p.b.copy_item_stride;
        const uint32_t first = (blockIdx.y - p.compute_groups) * p.rows_per;
        for (uint32_t r = first; r < first + p.rows_per && r < d.copy_count; r++) {
            const size_t idx = ((size_t)(d.copy_first + r) << p.log_n) + j;
            out[idx] = from[idx];
        }
        return;
    }
    const uint32_t row0 = blockIdx.y * p.rows_per;
    if (row0 >= d.n_out) return;
    const uint64_t *x = p.b.x_base + item * p.b.x_item_stride + d.x_off;
    uint64_t xv[kBatchIn];
#pragma unroll
    for (int i = 0; i < kBatchIn; i++) xv[i] = (uint32_t)i < d.n_in ? x[((size_t)i << p.log_n) + j] : 0;
    const uint64_t *mat = p.b.mat_base + d.mat_off;
    for (uint32_t row = row0; row < row0 + p.rows_per && row < d.n_out; row++) {
        const uint64_t *m = mat + (size_t)row * d.n_in;
        const uint32_t t = p.b.out_table[d.map_off + row];
        uint64_t r;
        if (d.n_in == 1 && m[0] == 1) {
            // a digit of one limb (one special prime): Q_d / q_i = 1, the conversion is a plain reduction
            r = barrett64(xv[0], p.moduli[t], p.barrett[2 * t + 1]);
        } else {
            U128 acc{0, 0};
#pragma unroll
            for (int i = 0; i < kBatchIn; i++)
                if ((uint32_t)i < d.n_in) mac128(acc, xv[i], m[i]);
            r = barrett128(acc.lo, acc.hi, p.moduli[t], p.barrett[2 * t], p.barrett[2 * t + 1]);
        }
        out[((size_t)p.b.out_limb[d.map_off + row] << p.log_n) + j] = r;
    }
}

// FP64 variant: every product is reduced on the fly to |r| <= 0.75 m, so the sum of up to 8 terms stays an
// exact integer below 6 m < 2^53; one canonicalisation per output.
__global__ __launch_bounds__(kThreads) void bconv_batched_fp_kernel(BconvBatchK p) {
    const uint32_t item = blockIdx.z / p.b.n_units;
    const BconvDesc d = p.b.descs[blockIdx.z - item * p.b.n_units];
    const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
    uint64_t *out = p.b.out_base + item * p.b.out_item_stride + d.out_off;
    if (blockIdx.y >= p.compute_groups) {
        const uint64_t *from = p.b.copy_base + item * p.b.copy_item_stride;
        const uint32_t first = (blockIdx.y - p.compute_groups) * p.rows_per;
        for (uint32_t r = first; r < first + p.rows_per && r < d.copy_count; r++) {
            const size_t idx = ((size_t)(d.copy_first + r) << p.log_n) + j;
            out[idx] = from[idx];
        }
        return;
    }
    const uint32_t row0 = blockIdx.y * p.rows_per;
    if (row0 >= d.n_out) return;
    const uint64_t *x = p.b.x_base + item * p.b.x_item_stride + d.x_off;
    double xv[kBatchIn];
#pragma unroll
    for (int i = 0; i < kBatchIn; i++) xv[i] = (uint32_t)i < d.n_in ? fp_from_u64(x[((size_t)i << p.log_n) + j]) : 0.0;
    const double *mat = p.b.mat_fp + 2 * d.mat_off;
    for (uint32_t row = row0; row < row0 + p.rows_per && row < d.n_out; row++) {
        const double *m = mat + 2 * (size_t)row * d.n_in;
        const uint32_t t = p.b.out_table[d.map_off + row];
        const FpMod mod{p.b.fp_consts[4 * t], p.b.fp_consts[4 * t + 1]};
        double acc = 0.0;
#pragma unroll
        for (int i = 0; i < kBatchIn; i++)
            if ((uint32_t)i < d.n_in) acc += fp_mulmod(xv[i], FpTw{m[2 * i], m[2 * i + 1]}, mod);
        out[((size_t)p.b.out_limb[d.map_off + row] << p.log_n) + j] = fp_to_u64(fp_canonical(acc, mod));
    }
}

struct InnerArgs {
    const uint64_t *y;
    uint64_t *out;
    const uint64_t *moduli, *barrett;
    EvkPtrs evk;
    uint32_t L, K, size_q, beta, log_n, galois_elt;
    int accumulate;
    const uint64_t *fold_ct, *fold_w;
    size_t y_item_stride, out_item_stride, fold_item_stride;   // blockIdx.z = item (words between items)
    const uint64_t *add_c0, *p_mod_q;
    uint32_t add_elt;
    const uint64_t *own;            // optional: the key-switch input [L][N]; a digit's own limbs are read from it (their
    size_t own_item_stride;         // slots in y were left unwritten), items own_item_stride words apart
    uint32_t own_elt;               // != 0: the key-switch input is sigma(own), gathered here (X -> X^own_elt)
};

// grid: (N / 256, L + K, items).  Streams beta digit limbs of y and 2 beta key limbs, writes (or accumulates) the
// two output limbs.  The products are summed in 128 bits and reduced once (beta <= 64 products of
// 61-bit factors cannot overflow).
__global__ __launch_bounds__(kThreads) void inner_product_kernel(InnerArgs p) {
    const uint32_t t = blockIdx.y;
    const uint32_t LK = p.L + p.K;
    const uint32_t table = t < p.L ? t : p.size_q + (t - p.L);
    const uint32_t j = blockIdx.x * kThreads + threadIdx.x;
    const uint32_t src = p.galois_elt ? galois_index(j, p.galois_elt, p.log_n) : j;
    const size_t key_off = ((size_t)table << p.log_n) + j;
    const size_t key_poly = (size_t)(p.size_q + p.K) << p.log_n;
    // (the argument struct stays untouched: a modified copy would move its pointer table to scratch memory)
    const uint64_t *y = p.y + blockIdx.z * p.y_item_stride;
    uint64_t *out = p.out + blockIdx.z * p.out_item_stride;
    const uint64_t *own = p.own ? p.own + blockIdx.z * p.own_item_stride + ((size_t)t << p.log_n) : nullptr;
    const uint32_t own_d = (own && t < p.L) ? t / p.K : 0xffffffffu;
    const uint32_t own_src = p.own_elt ? galois_index(j, p.own_elt, p.log_n) : src;
    U128 a0{0, 0}, a1{0, 0};
    for (uint32_t d = 0; d < p.beta; d++) {
        const uint64_t v = d == own_d ? own[own_src] : y[(((size_t)d * LK + t) << p.log_n) + src];
        const uint64_t *k = p.evk.p[d];
        mac128(a0, v, k[key_off]);
        mac128(a1, v, k[key_off + key_poly]);
    }
    const uint64_t q = p.moduli[table], r0 = p.barrett[2 * table], r1 = p.barrett[2 * table + 1];
    uint64_t o0 = barrett128(a0.lo, a0.hi, q, r0, r1);
    uint64_t o1 = barrett128(a1.lo, a1.hi, q, r0, r1);
    const size_t o = ((size_t)t << p.log_n) + j;
    const size_t opoly = (size_t)LK << p.log_n;
    if (p.accumulate) {
        o0 = add_mod(o0, out[o], q);
        o1 = add_mod(o1, out[o + opoly], q);
    }
    if (p.add_c0 && t < p.L) {
        // a rotation: polynomial 0 gains P sigma(c0), which ModDown's division by P turns into sigma(c0)
        const uint32_t g = p.add_elt ? galois_index(j, p.add_elt, p.log_n) : j;
        o0 = add_mod(o0, mul_shoup(p.add_c0[((size_t)t << p.log_n) + g], load_shoup(p.p_mod_q, t), q), q);
    }
    if (p.fold_ct && t == p.L - 1) {
        const Shoup w = load_shoup(p.fold_w, 0);
        const size_t cpoly = (size_t)p.L << p.log_n;
        const uint64_t *fold = p.fold_ct + blockIdx.z * p.fold_item_stride;
        o0 = add_mod(mul_shoup(o0, w, q), fold[o], q);
        o1 = add_mod(mul_shoup(o1, w, q), fold[o + cpoly], q);
    }
    out[o] = o0;
    out[o + opoly] = o1;
}

struct HoistArgs {
    const uint64_t *y, *c0;
    uint64_t *out, *c0_out;
    const uint64_t *moduli, *barrett;
    EvkPtrs evk;                    // [step * beta + digit]
    uint32_t elts[kMaxDigits];      // Galois element of every step
    uint32_t n_steps, L, K, size_q, beta, log_n;
    int accumulate, with_self;
    uint32_t items;
    size_t ct_item_stride;          // words between the ciphertexts of consecutive items (blockIdx.z), in and out
    const double *fp_consts;        // [tables][4] of the FP64 back end
    uint64_t fp_mask;               // bit t: the products of table t (a prime below 2^50) are formed in FP64
    int own_from_ct;                // a digit's own limbs are read from c1 of the input (c0 + L limbs), not from y
    uint32_t rows, groups;          // grid: N / 256 blocks x rows x groups of items, as one dimension
    int xcd_map;                    // workgroup order that keeps the sharers of a key block on one XCD
};

// Hoisted rotations in one launch: grid (N / 256, (L + K) + L [+ L], ceil(items / I)); a thread serves the same
// coefficient of I consecutive items, so that a key word is loaded once for all of them.
// rows t < L + K:  out[p][t] = sum_s sum_d sigma_s(y_d)[t] * evk_{s,d}[p][t]  (n_steps * beta <= 64 products, summed
//                  lazily as partial products of factors split at bit 30, see Lazy3, and reduced once); the automorphism is the
//                  gather index of the load of y.  The kernel is bound by instruction issue (its multiply-adds).
// rows L + K + t:  c0_out[t] = sum_s sigma_s(c0)[t]  (+ c0[t] with_self)
// rows L + K + L + t (with_self only): c1 is copied to the output, so that the ModDown that follows adds onto
//                  the input ciphertext: ct_out = ct_in + sum_s rot_s(ct_in)
// LOCAL: every step's Galois element is 1 modulo 2^(log_n - 7) (steps that are multiples of N / 512), so the
// automorphism permutes inside each aligned block of 256 NTT-order words: a workgroup stages its block of every item
// and digit in LDS once (I * beta <= kHoistLocalTiles) and gathers from there, instead of one global gather per step.
constexpr int kHoistLocalTiles = 16;
template <int I, bool LOCAL>
__global__ __launch_bounds__(kThreads) void hoist_inner_kernel(HoistArgs p) {
    __shared__ uint64_t ybuf[LOCAL ? kHoistLocalTiles * kThreads : 1];
    const uint32_t LK = p.L + p.K;
    // Workgroup -> (block of 256 coefficients bx, row by, group of items bz).  The workgroups that share key words
    // (same block and row, every group) get linear ids 8 apart and consecutive in that sequence: the hardware deals
    // consecutive ids round-robin to the 8 XCDs, so they run on one XCD at about the same time and all but the first
    // find the keys in that XCD's L2 (p.xcd_map; otherwise the plain order).
    uint32_t bx, by, bz;
    {
        const uint32_t nb = (1u << p.log_n) / kThreads, id = blockIdx.x;
        if (p.xcd_map) {
            // xcd_map 2 (gathers from memory, N >= 2^15): an XCD also takes the 16 blocks of an aligned 4,096-word
            // stretch of one row one after the other, so that the words which the steps' gathers bring into its L2 (a
            // step of 8 k permutes inside such stretches) are found there by the neighbouring workgroups; the stretches
            // of every row are dealt to the XCDs in turn, heavy rows first everywhere
            const uint32_t s = id >> 3;
            uint32_t pair = (s / p.groups) * 8 + (id & 7);
            if (p.xcd_map == 2) {
                const uint32_t q = s / p.groups, u = (q >> 4) * 8 + (id & 7), stretches = nb >> 4;
                pair = (u / stretches) * nb + (u % stretches) * 16 + (q & 15);
            }
            bz = s % p.groups;
            bx = pair % nb;
            by = pair / nb;
        } else {
            bx = id % nb;
            by = (id / nb) % p.rows;
            bz = id / (nb * p.rows);
        }
    }
    const uint32_t j = bx * kThreads + threadIdx.x;
    const uint32_t item0 = bz * I;
    const uint32_t count = p.items - item0 < (uint32_t)I ? p.items - item0 : (uint32_t)I;
    // (the argument struct stays untouched: a modified copy would move its tables to scratch memory)
    if (by >= LK) {
        const size_t o = ((size_t)(by - LK) << p.log_n) + j;
        if (by >= LK + p.L) {
            if (!p.accumulate)
                for (uint32_t it = 0; it < count; it++)
                    p.c0_out[(item0 + it) * p.ct_item_stride + o] = p.c0[(item0 + it) * p.ct_item_stride + o];
            return;
        }
        // the gathers of a step are independent of the running sums: one index per step for all items, and the
        // loads of several steps in flight (a loop of one dependent load after the other ran longer than the rows
        // that multiply)
        const uint32_t t = by - LK;
        const uint64_t q = p.moduli[t];
        const uint64_t *in = p.c0 + item0 * p.ct_item_stride + ((size_t)t << p.log_n);
        uint64_t *c0_out = p.c0_out + item0 * p.ct_item_stride + o;
        uint64_t acc[I];
#pragma unroll
        for (int it = 0; it < I; it++)
            acc[it] = (uint32_t)it >= count ? 0 : p.accumulate ? c0_out[it * p.ct_item_stride] : p.with_self ? in[it * p.ct_item_stride + j] : 0;
#pragma unroll 4
        for (uint32_t s = 0; s < p.n_steps; s++) {
            const uint32_t g = galois_index(j, p.elts[s], p.log_n);
            uint64_t w[I];
#pragma unroll
            for (int it = 0; it < I; it++) w[it] = (uint32_t)it < count ? in[it * p.ct_item_stride + g] : 0;
#pragma unroll
            for (int it = 0; it < I; it++) acc[it] = add_mod(acc[it], w[it], q);
        }
#pragma unroll
        for (int it = 0; it < I; it++)
            if ((uint32_t)it < count) c0_out[it * p.ct_item_stride] = acc[it];
        return;
    }
    const uint32_t t = by;
    const size_t y_item = (size_t)p.beta * LK << p.log_n;
    const uint64_t *y = p.y + item0 * y_item + ((size_t)t << p.log_n);
    const uint32_t table = t < p.L ? t : p.size_q + (t - p.L);
    const size_t key_off = ((size_t)table << p.log_n) + j;
    const size_t key_poly = (size_t)(p.size_q + p.K) << p.log_n;
    const size_t digit = (size_t)LK << p.log_n;
    // the digit that owns limb t: its "lifted" limb is the input's c1 itself
    const uint32_t own = (p.own_from_ct && t < p.L) ? t / p.K : 0xffffffffu;
    const uint64_t *c1 = p.c0 + item0 * p.ct_item_stride + ((size_t)(p.L + t) << p.log_n);
    auto word = [&](uint32_t d, int it, uint32_t at) {
        return d == own ? c1[it * p.ct_item_stride + at] : y[it * y_item + d * digit + at];
    };
    const uint32_t n_terms = p.n_steps * p.beta;
    if (LOCAL) {
        for (uint32_t d = 0; d < p.beta; d++)
#pragma unroll
            for (int it = 0; it < I; it++)
                ybuf[(it * p.beta + d) * kThreads + threadIdx.x] = (uint32_t)it < count ? word(d, it, j) : 0;
        __syncthreads();
    }
    // term e = step e / beta, digit e mod beta; the operands of term e + 1 are requested before term e is
    // multiplied, so that a wave does not wait for memory once per term
    // (the gather index belongs to the step: it is formed for a step's first digit and kept for the others; the last
    // iteration's repeated request is for the term just served)
    uint32_t src = 0;
    auto fetch = [&](uint32_t e, uint64_t &k0, uint64_t &k1, uint64_t(&v)[I]) {
        const uint32_t st = e / p.beta, d = e - st * p.beta;
        if (d == 0 || e == 0) src = galois_index(j, p.elts[st], p.log_n);
        const uint64_t *k = p.evk.p[e];
        k0 = k[key_off];
        k1 = k[key_off + key_poly];
#pragma unroll
        for (int it = 0; it < I; it++)
            v[it] = LOCAL ? ybuf[(it * p.beta + d) * kThreads + (src & (kThreads - 1))]
                          : ((uint32_t)it < count ? word(d, it, src) : 0);
    };
    uint64_t k0, k1, v[I];
    fetch(0, k0, k1, v);
    const size_t o = ((size_t)t << p.log_n) + j;
    const size_t opoly = (size_t)LK << p.log_n;
    if (table < 64 && ((p.fp_mask >> table) & 1)) {
        // a prime below 2^50: the sum of the products as an exact pair (hi, lo) before any reduction, four FP64
        // operations per product.  hi runs in [2^B, 2^(B+1)), where doubles are the multiples of 2^(B-52): the fused
        // multiply-add t = fl(x w + hi) rounds the exact sum to such a multiple, t - hi is exact, x w - (t - hi) is the
        // rounding error, an integer of at most 2^(B-53) in magnitude that the second fused multiply-add returns
        // exactly.  B = 103 takes 8 products below 2^100 between two folds (8 errors sum exactly, <= 2^53); when
        // n_terms q^2 <= 2^100 a smaller B takes all of them (at most 64) in one go.
        const FpMod m{p.fp_consts[4 * table], p.fp_consts[4 * table + 1]};
        const uint32_t qbits = 64 - __builtin_clzll(p.moduli[table]);              // q < 2^qbits
        const uint32_t tbits = 32 - __builtin_clz(n_terms);                        // n_terms < 2^tbits
        const bool one_go = 2 * qbits + tbits <= 100;
        const uint32_t B = !one_go ? 103 : 2 * qbits + tbits < 60 ? 60 : 2 * qbits + tbits;   // (any B up to 100 serves small primes)
        const uint32_t period = one_go ? n_terms : 8;
        const double base = __hiloint2double((int)((1023 + B) << 20), 0);
        const double down = __hiloint2double((int)((1023 + 52 - B) << 20), 0);     // 2^-(B-52)
        const double cB = fp_reduce(__hiloint2double((int)((1023 + B - 52) << 20), 0), m);
        const FpTw wB{cB, cB * m.qinv};
        double hi0[I], lo0[I], hi1[I], lo1[I], f0[I], f1[I];
#pragma unroll
        for (int it = 0; it < I; it++) {
            hi0[it] = hi1[it] = base;
            lo0[it] = lo1[it] = f0[it] = f1[it] = 0.0;
        }
        // (hi - 2^B) / 2^(B-52) is an integer below 2^52; times 2^(B-52) mod q it is congruent to the high part, and the
        // modular product takes it as it is (result at most 2.5 q in magnitude)
        auto fold = [&]() {
#pragma unroll
            for (int it = 0; it < I; it++) {
                f0[it] = fp_reduce(f0[it] + fp_mulmod((hi0[it] - base) * down, wB, m) + fp_reduce(lo0[it], m), m);
                f1[it] = fp_reduce(f1[it] + fp_mulmod((hi1[it] - base) * down, wB, m) + fp_reduce(lo1[it], m), m);
                hi0[it] = hi1[it] = base;
                lo0[it] = lo1[it] = 0.0;
            }
        };
        uint32_t pending = 0;
        for (uint32_t e = 0; e < n_terms; e++) {
            uint64_t nk0, nk1, nv[I];
            fetch(e + 1 < n_terms ? e + 1 : e, nk0, nk1, nv);
            asm volatile("" ::: "memory");       // (a compiler barrier: without it the loads, whose values are first used in the
            __builtin_amdgcn_sched_barrier(0);   //  next iteration, sink to the end of this one and every term waits for its operands)
            const double w0 = fp_from_u64(k0), w1 = fp_from_u64(k1);
#pragma unroll
            for (int it = 0; it < I; it++) {
                const double x = fp_from_u64(v[it]);
                const double t0 = __builtin_fma(x, w0, hi0[it]), t1 = __builtin_fma(x, w1, hi1[it]);
                lo0[it] += __builtin_fma(x, w0, -(t0 - hi0[it]));
                lo1[it] += __builtin_fma(x, w1, -(t1 - hi1[it]));
                hi0[it] = t0;
                hi1[it] = t1;
            }
            if (++pending == period) {
                fold();
                pending = 0;
            }
            k0 = nk0;
            k1 = nk1;
#pragma unroll
            for (int it = 0; it < I; it++) v[it] = nv[it];
        }
        if (pending) fold();
#pragma unroll
        for (int it = 0; it < I; it++) {
            if ((uint32_t)it >= count) break;
            uint64_t *out = p.out + (item0 + it) * ((size_t)2 * LK << p.log_n);
            double o0 = f0[it], o1 = f1[it];
            if (p.accumulate) {
                o0 += fp_from_u64(out[o]);
                o1 += fp_from_u64(out[o + opoly]);
            }
            out[o] = fp_to_u64(fp_canonical(o0, m));
            out[o + opoly] = fp_to_u64(fp_canonical(o1, m));
        }
        return;
    }
    Lazy3 s0[I], s1[I], h0[I], h1[I];
    // the words are relieved every 8 terms for a prime below 2^60, every 4 otherwise (see Lazy3)
    const uint32_t spill_mask = (p.moduli[table] >> 60) ? 3u : 7u;
#pragma unroll
    for (int it = 0; it < I; it++) s0[it] = s1[it] = h0[it] = h1[it] = Lazy3{0, 0, 0};
    for (uint32_t e = 0; e < n_terms; e++) {
        uint64_t nk0, nk1, nv[I];
        fetch(e + 1 < n_terms ? e + 1 : e, nk0, nk1, nv);
        asm volatile("" ::: "memory");       // (a compiler barrier: without it the loads, whose values are first used in the
            __builtin_amdgcn_sched_barrier(0);   //  next iteration, sink to the end of this one and every term waits for its operands)
        const Split30 ks0 = split30(k0), ks1 = split30(k1);
#pragma unroll
        for (int it = 0; it < I; it++) {
            mac3x2(s0[it], s1[it], split30(v[it]), ks0, ks1);
        }
        if ((e & spill_mask) == spill_mask) {
#pragma unroll
            for (int it = 0; it < I; it++) {
                spill3(h0[it], s0[it]);
                spill3(h1[it], s1[it]);
            }
        }
        k0 = nk0;
        k1 = nk1;
#pragma unroll
        for (int it = 0; it < I; it++) v[it] = nv[it];
    }
    const uint64_t q = p.moduli[table], r0 = p.barrett[2 * table], r1 = p.barrett[2 * table + 1];
#pragma unroll
    for (int it = 0; it < I; it++) {
        if ((uint32_t)it >= count) break;
        uint64_t *out = p.out + (item0 + it) * ((size_t)2 * LK << p.log_n);
        const U128 a0 = total3(h0[it], s0[it]), a1 = total3(h1[it], s1[it]);
        uint64_t o0 = barrett128(a0.lo, a0.hi, q, r0, r1);
        uint64_t o1 = barrett128(a1.lo, a1.hi, q, r0, r1);
        if (p.accumulate) {
            o0 = add_mod(o0, out[o], q);
            o1 = add_mod(o1, out[o + opoly], q);
        }
        out[o] = o0;
        out[o + opoly] = o1;
    }
}

// ---------------------------------------------------------------------------------------------------
// samplers: ChaCha20 block function (RFC 8439 section 2.3), 64-bit block counter in words 12-13,
// 64-bit stream id in words 14-15
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t rotl32(uint32_t v, int c) { return (v << c) | (v >> (32 - c)); }

#define HE_QR(a, b, c, d) \
    a += b; d ^= a; d = rotl32(d, 16); \
    c += d; b ^= c; b = rotl32(b, 12); \
    a += b; d ^= a; d = rotl32(d, 8);  \
    c += d; b ^= c; b = rotl32(b, 7);

__device__ void chacha20_block(const ChaChaKey &key, uint64_t counter, uint64_t stream, uint32_t *out) {
    uint32_t s[16] = {0x61707865u, 0x3320646eu, 0x79622d32u, 0x6b206574u,
                      key.k[0], key.k[1], key.k[2], key.k[3], key.k[4], key.k[5], key.k[6], key.k[7],
                      (uint32_t)counter, (uint32_t)(counter >> 32), (uint32_t)stream, (uint32_t)(stream >> 32)};
    uint32_t x[16];
#pragma unroll
    for (int i = 0; i < 16; i++) x[i] = s[i];
    for (int i = 0; i < 10; i++) {
        HE_QR(x[0], x[4], x[8], x[12]) HE_QR(x[1], x[5], x[9], x[13]) HE_QR(x[2], x[6], x[10], x[14]) HE_QR(x[3], x[7], x[11], x[15])
        HE_QR(x[0], x[5], x[10], x[15]) HE_QR(x[1], x[6], x[11], x[12]) HE_QR(x[2], x[7], x[8], x[13]) HE_QR(x[3], x[4], x[9], x[14])
    }
#pragma unroll
    for (int i = 0; i < 16; i++) out[i] = x[i] + s[i];
}

struct SampleArgs {
    uint64_t *out;
    const uint64_t *moduli, *barrett;
    const uint64_t *cdt;
    ChaChaKey key;
    uint64_t stream;
    LimbMap map;
    uint32_t log_n, cdt_len;
    int kind;
    uint32_t stream_stride;
    size_t out_item_stride;
};

// ternary / error / gauss: one thread = one ChaCha block = 16 (ternary) or 8 coefficients, the same
// signed value written to every limb.  uniform: one thread = one block = 4 residues of one limb.
// KIND is a template parameter so that the loops over the block's words unroll and the words stay in registers (with
// a run-time count the array lived in scratch memory); a thread's 16 or 8 consecutive output words leave as 16-byte
// stores.
template <int KIND>
__device__ __forceinline__ void sample_signed(const SampleArgs &p, uint32_t b, uint64_t stream, uint64_t *out);

template <int KIND>
__global__ __launch_bounds__(kThreads) void sample_kernel(SampleArgs p) {
    const uint32_t n = 1u << p.log_n;
    const uint32_t b = blockIdx.x * kThreads + threadIdx.x;
    // blockIdx.y = item: its own stream id, its own polynomial
    const uint64_t stream = p.stream + (uint64_t)blockIdx.y * p.stream_stride;
    uint64_t *out = p.out + blockIdx.y * p.out_item_stride;
    uint32_t w[16];
    if (KIND == SAMPLE_UNIFORM) {
        const uint32_t per_limb = n / 4;
        if (b >= per_limb * p.map.limbs) return;
        const uint32_t limb = b / per_limb, blk = b % per_limb;
        const uint32_t table = map_table(p.map, limb);
        const uint64_t q = p.moduli[table], r0 = p.barrett[2 * table], r1 = p.barrett[2 * table + 1];
        chacha20_block(p.key, b, stream, w);
        uint64_t r[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            uint64_t lo = ((uint64_t)w[4 * e + 1] << 32) | w[4 * e];
            uint64_t hi = ((uint64_t)w[4 * e + 3] << 32) | w[4 * e + 2];
            r[e] = barrett128(lo, hi, q, r0, r1);
        }
        ulonglong2 *dst = reinterpret_cast<ulonglong2 *>(out + ((size_t)limb << p.log_n) + 4 * blk);
        dst[0] = ulonglong2{r[0], r[1]};
        dst[1] = ulonglong2{r[2], r[3]};
        return;
    }
    sample_signed<KIND>(p, b, stream, out);
}

// ternary / error / gauss coefficients of ChaCha block b of `stream`, the same signed value to every limb of `out`
template <int KIND>
__device__ __forceinline__ void sample_signed(const SampleArgs &p, uint32_t b, uint64_t stream, uint64_t *out) {
    const uint32_t n = 1u << p.log_n;
    uint32_t w[16];
    constexpr int per_block = KIND == SAMPLE_TERNARY ? 16 : 8;
    if (b >= n / per_block) return;
    chacha20_block(p.key, b, stream, w);
    int v[per_block];
#pragma unroll
    for (int e = 0; e < per_block; e++) {
        if (KIND == SAMPLE_TERNARY) {
            v[e] = (int)(((uint64_t)w[e] * 3) >> 32) - 1;
        } else if (KIND == SAMPLE_ERROR) {
            v[e] = __popc(w[2 * e] & 0x1FFFFFu) - __popc(w[2 * e + 1] & 0x1FFFFFu);
        } else {
            uint64_t u = ((uint64_t)w[2 * e + 1] << 32) | w[2 * e];
            const bool neg = u >> 63;
            u &= 0x7FFFFFFFFFFFFFFFull;
            uint32_t mag = 0;
            while (mag < p.cdt_len && u >= p.cdt[mag]) mag++;
            v[e] = neg ? -(int)mag : (int)mag;
        }
    }
    for (uint32_t limb = 0; limb < p.map.limbs; limb++) {
        const uint64_t q = p.moduli[map_table(p.map, limb)];
        ulonglong2 *dst = reinterpret_cast<ulonglong2 *>(out + ((size_t)limb << p.log_n) + (size_t)per_block * b);
#pragma unroll
        for (int e = 0; e < per_block; e += 2)
            dst[e / 2] = ulonglong2{v[e] < 0 ? q - (uint64_t)(-v[e]) : (uint64_t)v[e],
                                    v[e + 1] < 0 ? q - (uint64_t)(-v[e + 1]) : (uint64_t)v[e + 1]};
    }
}

// The three polynomials of `items` public-key encryptions in one launch: out holds [items] ternary polynomials u and
// behind them [items][2] error polynomials (e0, e1), all out_item_stride words apart; item k draws u, e0, e1 from the
// streams p.stream + 3 k, + 1, + 2.  blockIdx.y = polynomial, blockIdx.z = 0.
__global__ __launch_bounds__(kThreads) void sample_encrypt_kernel(SampleArgs p, uint32_t items) {
    const uint32_t b = blockIdx.x * kThreads + threadIdx.x, y = blockIdx.y;
    uint64_t *out = p.out + y * p.out_item_stride;
    if (y < items) {
        sample_signed<SAMPLE_TERNARY>(p, b, p.stream + 3 * (uint64_t)y, out);
    } else {
        const uint32_t e = y - items;
        sample_signed<SAMPLE_ERROR>(p, b, p.stream + 3 * (uint64_t)(e >> 1) + 1 + (e & 1), out);
    }
}

}  // namespace

hipError_t launch_elementwise(const Tables &t, int op, const uint64_t *a, const uint64_t *b, const uint64_t *c,
                              uint64_t *out, uint32_t n_polys, LimbMap map, hipStream_t s) {
    if (n_polys == 0 || map.limbs == 0) return hipSuccess;
    EwArgs p{a, b, c, out, t.moduli, t.barrett, map, t.log_n, op};
    hipLaunchKernelGGL(elementwise_kernel, dim3((1u << t.log_n) / kThreads, map.limbs, n_polys), dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_scalar_mul_add(const Tables &t, const uint64_t *a, const uint64_t *b, uint64_t *out,
                                 const uint64_t *w, uint32_t first, uint32_t limbs, hipStream_t s) {
    if (limbs == 0) return hipSuccess;
    hipLaunchKernelGGL(scalar_mul_add_kernel, dim3((1u << t.log_n) / kThreads, limbs), dim3(kThreads), 0, s, a, b, out,
                       t.moduli, w, first, t.log_n);
    return hipGetLastError();
}

hipError_t launch_decompose_real(const Tables &t, const double *coeffs, uint64_t *out, uint32_t limbs, uint32_t first,
                                 uint32_t items, size_t out_item_stride, hipStream_t s) {
    if (limbs == 0 || items == 0) return hipSuccess;
    if (items > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(decompose_real_kernel, dim3((1u << t.log_n) / kThreads, limbs, items), dim3(kThreads), 0, s, coeffs,
                       out, t.moduli, t.barrett, first, t.log_n, out_item_stride);
    return hipGetLastError();
}

hipError_t launch_encrypt_fma(const Tables &t, const uint64_t *u, const uint64_t *pk, uint64_t *wide, uint32_t L,
                              uint32_t K, uint32_t size_q, uint32_t items, hipStream_t s) {
    if (items == 0 || items > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(encrypt_fma_kernel, dim3((1u << t.log_n) / kThreads, L + K, items), dim3(kThreads), 0, s, u, pk, wide,
                       t.moduli, t.barrett, L, K, size_q, t.log_n);
    return hipGetLastError();
}

hipError_t launch_tensor(const Tables &t, const uint64_t *ct1, const uint64_t *ct2, uint64_t *out, uint32_t L,
                         bool square, hipStream_t s, const double *fp_consts, uint32_t items, uint64_t *out2) {
    if (items == 0 || items > 65535 || (items > 1 && !out2)) return hipErrorInvalidValue;
    const size_t poly = (size_t)L << t.log_n;
    TensorArgs p{ct1, ct2, out, t.moduli, t.barrett, L, t.log_n, out2 ? out2 : out + 2 * poly, 2 * poly, 2 * poly, poly};
    dim3 grid((1u << t.log_n) / kThreads, L, items);
    if (fp_consts && square)
        hipLaunchKernelGGL(tensor_fp_kernel<true>, grid, dim3(kThreads), 0, s, p, fp_consts);
    else if (fp_consts)
        hipLaunchKernelGGL(tensor_fp_kernel<false>, grid, dim3(kThreads), 0, s, p, fp_consts);
    else if (square)
        hipLaunchKernelGGL(tensor_kernel<true>, grid, dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL(tensor_kernel<false>, grid, dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_tensor_mxn(const Tables &t, const uint64_t *ct1, uint32_t s1, const uint64_t *ct2, uint32_t s2,
                             uint64_t *out, uint32_t L, hipStream_t s) {
    const size_t poly = (size_t)L << t.log_n;
    TensorArgs p{ct1, ct2, out, t.moduli, t.barrett, L, t.log_n, out, 0, 0, poly};
    dim3 grid((1u << t.log_n) / kThreads, L);
#define HE_CASE(A, B) \
    if (s1 == A && s2 == B) hipLaunchKernelGGL((tensor_mxn_kernel<A, B>), grid, dim3(kThreads), 0, s, p); else
    HE_CASE(1, 1) HE_CASE(1, 2) HE_CASE(1, 3) HE_CASE(2, 1) HE_CASE(2, 2) HE_CASE(2, 3) HE_CASE(3, 1) HE_CASE(3, 2)
    HE_CASE(3, 3) {
        if (s1 == 0 || s2 == 0 || s1 > 16 || s2 > 16) return hipErrorInvalidValue;
        hipLaunchKernelGGL(tensor_any_kernel, grid, dim3(kThreads), 0, s, p, s1, s2);
    }
#undef HE_CASE
    return hipGetLastError();
}

hipError_t launch_pair_square_sum(const Tables &t, const uint64_t *const *pairs, uint64_t *out01, uint64_t *out2,
                                  uint32_t L, uint32_t items, uint32_t chunks, hipStream_t s) {
    if (items == 0 || items > 65535 || chunks == 0 || L == 0) return hipErrorInvalidValue;
    PairSquareArgs p{pairs, out01, out2, t.moduli, t.barrett, L, t.log_n, chunks};
    hipLaunchKernelGGL(pair_square_sum_kernel, dim3((1u << t.log_n) / kThreads, L, items), dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_decrypt_gather(const Tables &t, const uint64_t *const *cts, const uint64_t *sk, const uint64_t *noise,
                                 uint64_t *out, uint32_t limbs, uint32_t items, hipStream_t s) {
    if (items == 0 || items > 65535 || limbs == 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(decrypt_gather_kernel, dim3((1u << t.log_n) / kThreads, limbs, items), dim3(kThreads), 0, s, cts, sk,
                       noise, out, t.moduli, t.barrett, limbs, t.log_n);
    return hipGetLastError();
}

hipError_t launch_galois(const Tables &t, const uint64_t *in, uint64_t *out, uint32_t total_limbs, uint32_t elt,
                         hipStream_t s) {
    if (total_limbs == 0) return hipSuccess;
    hipLaunchKernelGGL(galois_kernel, dim3((1u << t.log_n) / kThreads, total_limbs), dim3(kThreads), 0, s, in, out, elt,
                       t.log_n);
    return hipGetLastError();
}

hipError_t launch_bconv(const Tables &t, const BconvArgs &a, hipStream_t s) {
    if (a.n_out == 0) return hipSuccess;
    BconvKArgs p{a, t.moduli, t.barrett, t.log_n};
    dim3 grid((1u << t.log_n) / kThreads, (a.n_out + kRows - 1) / kRows);
    switch (a.n_in) {
#define HE_CASE(NIN) \
    case NIN: hipLaunchKernelGGL(bconv_kernel<NIN>, grid, dim3(kThreads), 0, s, p); break;
        HE_CASE(1) HE_CASE(2) HE_CASE(3) HE_CASE(4) HE_CASE(5) HE_CASE(6) HE_CASE(7) HE_CASE(8)
#undef HE_CASE
        default: hipLaunchKernelGGL(bconv_kernel<0>, grid, dim3(kThreads), 0, s, p);
    }
    return hipGetLastError();
}

hipError_t launch_bconv_batched(const Tables &t, const BconvBatch &b, const Tuning &tune, hipStream_t s) {
    if (b.n_units == 0) return hipSuccess;
    const uint32_t target = tune.bconv_rows >= 1 && tune.bconv_rows <= 64 ? tune.bconv_rows : 6;
    const uint32_t cg = (b.max_rows + target - 1) / target;
    const uint32_t rows_per = (b.max_rows + cg - 1) / cg;
    const uint32_t kg = (b.max_copy + rows_per - 1) / rows_per;
    BconvBatchK p{b, t.moduli, t.barrett, t.log_n, cg, rows_per};
    const uint32_t items = b.items ? b.items : 1;
    if ((uint64_t)b.n_units * items > 65535) return hipErrorInvalidValue;
    const dim3 grid((1u << t.log_n) / kThreads, cg + kg, b.n_units * items);
    if (b.mat_fp)
        hipLaunchKernelGGL(bconv_batched_fp_kernel, grid, dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL(bconv_batched_kernel, grid, dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_inner_product(const Tables &t, const uint64_t *y, const EvkPtrs &evk, uint64_t *out, uint32_t L,
                                uint32_t K, uint32_t size_q, uint32_t beta, uint32_t galois_elt, bool accumulate,
                                const uint64_t *fold_ct, const uint64_t *fold_w, uint32_t items, size_t fold_item_stride,
                                hipStream_t s, const uint64_t *add_c0, uint32_t add_elt, const uint64_t *p_mod_q,
                                const uint64_t *own, size_t own_item_stride, uint32_t own_elt) {
    const size_t n = (size_t)1 << t.log_n;
    InnerArgs p{y, out, t.moduli, t.barrett, evk, L, K, size_q, beta, t.log_n, galois_elt, accumulate ? 1 : 0,
                fold_ct, fold_w, (size_t)beta * (L + K) * n, 2 * (size_t)(L + K) * n, fold_item_stride,
                add_c0, p_mod_q, add_elt, own, own_item_stride, own_elt};
    if (items == 0 || items > 65535 || (add_c0 && (items != 1 || !p_mod_q))) return hipErrorInvalidValue;
    hipLaunchKernelGGL(inner_product_kernel, dim3((1u << t.log_n) / kThreads, L + K, items), dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

struct InnerFpArgs {
    const uint64_t *y, *own;
    uint64_t *out;
    const double *fp_consts;
    EvkPtrs evk;
    uint32_t L, K, size_q, beta, log_n, items;
    const uint64_t *fold_ct, *fold_w;
    size_t y_item_stride, own_item_stride, out_item_stride, fold_item_stride;
};

// The inner product of a batch on the FP64 back end (every prime below 2^50).  grid: (N / 512, L + K, groups of I
// items); a thread holds two coefficients of I items.  A key word is loaded and converted once and multiplies all I
// items, so the 2 beta key limbs are read once per group instead of once per item; a digit's own limbs are read from
// the key switch's input (own, NTT form) rather than from a copy inside y.  Terms stay below 0.875 q, eight of them
// fit between two reductions; the stores are canonical, hence equal to the integer kernel's.
template <int I>
__global__ __launch_bounds__(kThreads) void inner_product_fp_kernel(InnerFpArgs p) {
    const uint32_t t = blockIdx.y;
    const uint32_t LK = p.L + p.K;
    const uint32_t table = t < p.L ? t : p.size_q + (t - p.L);
    const FpMod m{p.fp_consts[4 * table], p.fp_consts[4 * table + 1]};
    const size_t j = 2 * ((size_t)blockIdx.x * kThreads + threadIdx.x);
    const size_t key_off = ((size_t)table << p.log_n) + j;
    const size_t key_poly = (size_t)(p.size_q + p.K) << p.log_n;
    const uint32_t item0 = blockIdx.z * I;
    const uint32_t own_digit = t < p.L ? t / p.K : 0xffffffffu;
    double acc[I][4];
#pragma unroll
    for (int i = 0; i < I; i++) acc[i][0] = acc[i][1] = acc[i][2] = acc[i][3] = 0.0;
    for (uint32_t d = 0; d < p.beta; d++) {
        const uint64_t *k = p.evk.p[d];
        const ulonglong2 k0 = *reinterpret_cast<const ulonglong2 *>(k + key_off);
        const ulonglong2 k1 = *reinterpret_cast<const ulonglong2 *>(k + key_off + key_poly);
        const double w00 = fp_from_u64(k0.x), w01 = fp_from_u64(k0.y), w10 = fp_from_u64(k1.x), w11 = fp_from_u64(k1.y);
        const FpTw t00{w00, w00 * m.qinv}, t01{w01, w01 * m.qinv}, t10{w10, w10 * m.qinv}, t11{w11, w11 * m.qinv};
        const bool is_own = d == own_digit;
        const uint64_t *src = is_own ? p.own + ((size_t)t << p.log_n) + j : p.y + (((size_t)d * LK + t) << p.log_n) + j;
        const size_t stride = is_own ? p.own_item_stride : p.y_item_stride;
#pragma unroll
        for (int i = 0; i < I; i++) {
            const uint32_t item = item0 + i < p.items ? item0 + i : p.items - 1;
            const ulonglong2 v = *reinterpret_cast<const ulonglong2 *>(src + item * stride);
            const double y0 = fp_from_u64(v.x), y1 = fp_from_u64(v.y);
            acc[i][0] += fp_mulmod(y0, t00, m);
            acc[i][1] += fp_mulmod(y1, t01, m);
            acc[i][2] += fp_mulmod(y0, t10, m);
            acc[i][3] += fp_mulmod(y1, t11, m);
        }
        if ((d & 7) == 7) {
#pragma unroll
            for (int i = 0; i < I; i++)
                for (int c = 0; c < 4; c++) acc[i][c] = fp_reduce(acc[i][c], m);
        }
    }
    const size_t o = ((size_t)t << p.log_n) + j;
    const size_t opoly = (size_t)LK << p.log_n;
    const bool fold = p.fold_ct && t == p.L - 1;
    const double wd = fold ? fp_from_u64(p.fold_w[0]) : 0.0;
    const FpTw fw{wd, wd * m.qinv};
#pragma unroll
    for (int i = 0; i < I; i++) {
        if (item0 + i >= p.items) break;
        double r[4];
        for (int c = 0; c < 4; c++) r[c] = fp_canonical(acc[i][c], m);
        if (fold) {
            const uint64_t *f = p.fold_ct + (item0 + i) * p.fold_item_stride + o;
            const ulonglong2 f0 = *reinterpret_cast<const ulonglong2 *>(f);
            const ulonglong2 f1 = *reinterpret_cast<const ulonglong2 *>(f + ((size_t)p.L << p.log_n));
            r[0] = fp_canonical(fp_mulmod(r[0], fw, m) + fp_from_u64(f0.x), m);
            r[1] = fp_canonical(fp_mulmod(r[1], fw, m) + fp_from_u64(f0.y), m);
            r[2] = fp_canonical(fp_mulmod(r[2], fw, m) + fp_from_u64(f1.x), m);
            r[3] = fp_canonical(fp_mulmod(r[3], fw, m) + fp_from_u64(f1.y), m);
        }
        uint64_t *out = p.out + (item0 + i) * p.out_item_stride + o;
        *reinterpret_cast<ulonglong2 *>(out) = ulonglong2{fp_to_u64(r[0]), fp_to_u64(r[1])};
        *reinterpret_cast<ulonglong2 *>(out + opoly) = ulonglong2{fp_to_u64(r[2]), fp_to_u64(r[3])};
    }
}

hipError_t launch_inner_product_fp(const Tables &t, const double *fp_consts, const uint64_t *y, const uint64_t *own,
                                   size_t own_item_stride, const EvkPtrs &evk, uint64_t *out, uint32_t L, uint32_t K,
                                   uint32_t size_q, uint32_t beta, const uint64_t *fold_ct, const uint64_t *fold_w,
                                   uint32_t items, size_t fold_item_stride, hipStream_t s) {
    const size_t n = (size_t)1 << t.log_n;
    if (items == 0 || n < 2 * kThreads || !fp_consts || !own) return hipErrorInvalidValue;
    InnerFpArgs p{y, own, out, fp_consts, evk, L, K, size_q, beta, t.log_n, items, fold_ct, fold_w,
                  (size_t)beta * (L + K) * n, own_item_stride, 2 * (size_t)(L + K) * n, fold_item_stride};
    auto grid = [&](uint32_t per) { return dim3((uint32_t)(n / (2 * kThreads)), L + K, (items + per - 1) / per); };
    if ((items + 7) / 8 > 65535) return hipErrorInvalidValue;
    if (items >= 7)
        hipLaunchKernelGGL(inner_product_fp_kernel<8>, grid(8), dim3(kThreads), 0, s, p);
    else if (items >= 3)
        hipLaunchKernelGGL(inner_product_fp_kernel<4>, grid(4), dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL(inner_product_fp_kernel<2>, grid(2), dim3(kThreads), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_hoist_inner(const Tables &t, const Tuning &tune, const uint64_t *y, const uint64_t *c0, const uint64_t *const *evk,
                              const uint32_t *elts, uint32_t n_steps, uint64_t *out, uint64_t *c0_out, uint32_t L,
                              uint32_t K, uint32_t size_q, uint32_t beta, bool accumulate, bool with_self, uint32_t items,
                              size_t ct_item_stride, hipStream_t s, const double *fp_consts, uint64_t fp_mask,
                              bool own_from_ct) {
    if (n_steps == 0 || n_steps * beta > (uint32_t)kMaxDigits || items == 0 || items > 65535) return hipErrorInvalidValue;
    HoistArgs p;
    memset(&p, 0, sizeof(p));
    p.y = y;
    p.c0 = c0;
    p.out = out;
    p.c0_out = c0_out;
    p.moduli = t.moduli;
    p.barrett = t.barrett;
    for (uint32_t i = 0; i < n_steps * beta; i++) p.evk.p[i] = evk[i];
    for (uint32_t i = 0; i < n_steps; i++) p.elts[i] = elts[i];
    p.n_steps = n_steps;
    p.L = L;
    p.K = K;
    p.size_q = size_q;
    p.beta = beta;
    p.log_n = t.log_n;
    p.accumulate = accumulate ? 1 : 0;
    p.with_self = with_self ? 1 : 0;
    p.ct_item_stride = ct_item_stride;
    p.items = items;
    p.fp_consts = fp_consts;
    p.fp_mask = fp_consts ? fp_mask : 0;
    p.own_from_ct = own_from_ct ? 1 : 0;
    const uint32_t rows = (L + K) + (with_self ? 2 : 1) * L;
    const uint32_t nb = (1u << t.log_n) / kThreads;
    p.rows = rows;
    // every automorphism of the launch stays inside the aligned 256-word blocks of the NTT order
    bool local = t.log_n >= 8 && beta * 4 <= (uint32_t)kHoistLocalTiles;
    for (uint32_t i = 0; i < n_steps && local; i++) local = t.log_n < 9 || ((elts[i] - 1) & ((1u << (t.log_n - 7)) - 1)) == 0;
    const bool no_local = tune.hoist_no_local, no_xcd = tune.hoist_no_xcd, no_contig = tune.hoist_no_contig;
    if (no_local) local = false;
    // ... or inside the aligned stretches of 4,096 words (steps that are multiples of N / 8192)
    bool stretch_local = t.log_n >= 12;
    for (uint32_t i = 0; i < n_steps && stretch_local; i++) stretch_local = ((elts[i] - 1) & ((1u << (t.log_n - 11)) - 1)) == 0;
    const bool p_xcd_ok = !no_xcd && (nb * rows) % 8 == 0;
    auto launch = [&](auto kernel, uint32_t per) {
        p.groups = (items + per - 1) / per;
        p.xcd_map = p_xcd_ok && p.groups > 1 ? (local || no_contig || !stretch_local || nb < 128 || (nb >> 4) % 8 != 0 ? 1 : 2) : 0;
        hipLaunchKernelGGL(kernel, dim3(nb * rows * p.groups), dim3(kThreads), 0, s, p);
    };
#define HE_HOIST(I) \
    if (local) launch(hoist_inner_kernel<I, true>, I); \
    else launch(hoist_inner_kernel<I, false>, I)
    // (more items per thread read the keys less often but need more registers: 5, 6 and 8 items at 3, 2 and 2 waves per
    // SIMD measured 6 %, 5 to 20 % and 20 % slower than 4 items at 4 waves)
    // With the keys shared through L2, gathers from memory are served better by twice the waves (2 items per thread:
    // 452 against 498 us for 15 steps of 45 items at N = 2^16); the block-local form keeps 4 (389 against 500 us).
    if (items >= 4 && (local || !p_xcd_ok)) {
        HE_HOIST(4);
    } else if (items >= 2) {
        HE_HOIST(2);
    } else {
        HE_HOIST(1);
    }
#undef HE_HOIST
    return hipGetLastError();
}

hipError_t launch_sample(const Tables &t, int kind, ChaChaKey key, uint64_t stream_id, uint64_t *out, LimbMap map,
                         const uint64_t *cdt, uint32_t cdt_len, uint32_t items, uint32_t stream_stride,
                         size_t out_item_stride, hipStream_t s) {
    if (items == 0 || items > 65535) return hipErrorInvalidValue;
    const uint32_t n = 1u << t.log_n;
    uint32_t blocks = kind == SAMPLE_UNIFORM ? (n / 4) * map.limbs : (kind == SAMPLE_TERNARY ? n / 16 : n / 8);
    // (a thread's words leave as 16-byte stores)
    if ((reinterpret_cast<uintptr_t>(out) & 15) || (out_item_stride & 1)) return hipErrorInvalidValue;
    SampleArgs p{out, t.moduli, t.barrett, cdt, key, stream_id, map, t.log_n, cdt_len, kind, stream_stride, out_item_stride};
    const dim3 grid((blocks + kThreads - 1) / kThreads, items);
    switch (kind) {
        case SAMPLE_UNIFORM: hipLaunchKernelGGL(sample_kernel<SAMPLE_UNIFORM>, grid, dim3(kThreads), 0, s, p); break;
        case SAMPLE_TERNARY: hipLaunchKernelGGL(sample_kernel<SAMPLE_TERNARY>, grid, dim3(kThreads), 0, s, p); break;
        case SAMPLE_ERROR: hipLaunchKernelGGL(sample_kernel<SAMPLE_ERROR>, grid, dim3(kThreads), 0, s, p); break;
        case SAMPLE_GAUSS: hipLaunchKernelGGL(sample_kernel<SAMPLE_GAUSS>, grid, dim3(kThreads), 0, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_sample_encrypt(const Tables &t, ChaChaKey key, uint64_t stream_id, uint64_t *out, LimbMap map,
                                 uint32_t items, size_t poly_stride, hipStream_t s) {
    if (items == 0 || 3 * (uint64_t)items > 65535) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(out) & 15) || (poly_stride & 1)) return hipErrorInvalidValue;
    const uint32_t n = 1u << t.log_n;
    SampleArgs p{out, t.moduli, t.barrett, nullptr, key, stream_id, map, t.log_n, 0, SAMPLE_ERROR, 0, poly_stride};
    // (a ChaCha block yields 16 ternary or 8 error coefficients: the grid covers the error polynomials, the surplus
    // threads of the ternary ones leave at once)
    const dim3 grid((n / 8 + kThreads - 1) / kThreads, 3 * items);
    hipLaunchKernelGGL(sample_encrypt_kernel, grid, dim3(kThreads), 0, s, p, items);
    return hipGetLastError();
}

}  // namespace he
