/*
 * CPU restatement of the CKKS integer hot path of CAHEL (reference tree: cahel-main/).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU library is compared against; it is
 * loaded by tests/, by the smoke check and by the benchmark's cpu_baseline leg.  The product never
 * links, imports or calls it.
 *
 * Every function names the reference lines it follows.  All residues are uint64_t in [0, q) on
 * entry and on exit (the reference's kernels also only ever store canonical residues:
 * src/ntt/fntt_2d.cu:231-241, include/uintmodmath.cuh:154,232-233), so each function is fixed by
 * the mathematical value it returns; tests/test_oracle_*.py pin those values against Python
 * big-integer closed forms and the reference's own known-answer tests.
 *
 * Layout conventions (reference: include/ciphertext.h:303-333): a polynomial over k limbs is
 * k*N words, limb-major, coefficient index fastest.  "table index" of limb t of a Ql u P buffer
 * is t for t < L and size_Q + (t - L) otherwise (src/ntt/ntt_modup.cu:404-406).
 *
 * Pinning status: every function below is pinned (see tests/test_oracle_*.py) except the
 * samplers' use inside encryption/decryption noise, which the reference seeds from /dev/urandom
 * (include/prng.cuh:12-23) and OpenFHE (src/secretkey.cu:632-649): parity unpinned there, the
 * generator itself is pinned by the RFC 8439 ChaCha20 block test vector.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

typedef unsigned __int128 u128;

typedef struct {
    uint32_t logn;          /* N = 1 << logn */
    uint32_t size_q;        /* number of Q limbs at the key level */
    uint32_t size_p;        /* number of special limbs (alpha) */
    uint32_t reserved;
    const uint64_t *mod;    /* [size_q + size_p] */
    const uint64_t *ratio;  /* [size_q + size_p][2]  floor(2^128 / q): low word, high word */
    const uint64_t *tw;     /* [size_qp][N] psi^bitrev(i)                    (src/util/ntt.cu:46-56) */
    const uint64_t *twq;    /* [size_qp][N] floor(tw * 2^64 / q) */
    const uint64_t *itw;    /* [size_qp][N] psi^-bitrev(i) / 2               (src/util/ntt.cu:58-71) */
    const uint64_t *itwq;   /* [size_qp][N] floor(itw * 2^64 / q) */
} orc_params;

/* --------------------------------------------------------------------------------------------
 * scalar modular arithmetic -- include/uintmodmath.cuh
 * ------------------------------------------------------------------------------------------ */

/* floor(w * 2^64 / q): the Shoup quotient of include/util/uintarithsmallmod.h:158-180 */
uint64_t orc_shoup_quotient(uint64_t w, uint64_t q) { return (uint64_t)(((u128)w << 64) / q); }

/* include/uintmodmath.cuh:236-245  multiply_and_reduce_shoup_lazy: result in [0, 2q) */
static inline uint64_t mul_shoup_lazy(uint64_t x, uint64_t w, uint64_t wq, uint64_t q) {
    uint64_t hi = (uint64_t)(((u128)x * wq) >> 64);
    return x * w - hi * q;
}

/* include/uintmodmath.cuh:226-233  multiply_and_reduce_shoup */
uint64_t orc_mul_shoup(uint64_t x, uint64_t w, uint64_t wq, uint64_t q) {
    uint64_t r = mul_shoup_lazy(x, w, wq, q);
    return r >= q ? r - q : r;
}

/* include/uintmodmath.cuh:112-156  barrett_reduce_uint128_uint64 (the carry chain of the PTX block) */
static inline uint64_t barrett128(u128 x, uint64_t q, const uint64_t *ratio) {
    uint64_t lo = (uint64_t)x, hi = (uint64_t)(x >> 64);
    uint64_t carry = (uint64_t)(((u128)lo * ratio[0]) >> 64);
    u128 r1 = (u128)lo * ratio[1] + carry;
    uint64_t tmp = (uint64_t)r1;
    uint64_t quo = (uint64_t)(r1 >> 64);
    u128 r2 = (u128)hi * ratio[0] + tmp;
    quo += (uint64_t)(r2 >> 64);
    quo += hi * ratio[1];
    uint64_t r = lo - quo * q;
    return r >= q ? r - q : r;
}

uint64_t orc_barrett128(uint64_t lo, uint64_t hi, uint64_t q, const uint64_t *ratio) {
    return barrett128(((u128)hi << 64) | lo, q, ratio);
}

/* include/uintmodmath.cuh:164-173  barrett_reduce_uint64_uint64, ratio_hi = floor(2^64 / q) */
static inline uint64_t barrett64(uint64_t x, uint64_t q, uint64_t ratio_hi) {
    uint64_t s = (uint64_t)(((u128)ratio_hi * x) >> 64);
    uint64_t r = x - s * q;
    return r >= q ? r - q : r;
}

uint64_t orc_barrett64(uint64_t x, uint64_t q, uint64_t ratio_hi) { return barrett64(x, q, ratio_hi); }

/* include/uintmodmath.cuh:182-218  multiply_and_barrett_reduce_uint64 */
static inline uint64_t mulmod(uint64_t a, uint64_t b, uint64_t q, const uint64_t *ratio) {
    return barrett128((u128)a * b, q, ratio);
}

uint64_t orc_mulmod(uint64_t a, uint64_t b, uint64_t q, const uint64_t *ratio) { return mulmod(a, b, q, ratio); }

static inline uint64_t addmod(uint64_t a, uint64_t b, uint64_t q) {
    uint64_t s = a + b;
    return s >= q ? s - q : s;
}

static inline uint64_t submod(uint64_t a, uint64_t b, uint64_t q) { return a >= b ? a - b : a + q - b; }

/* out[i] = start * base^i mod q, i < count (helper for building psi tables; src/util/ntt.cu:46-71
 * walks the same power sequences with start = 1 and start = 1/2) */
void orc_power_table(uint64_t *out, uint64_t start, uint64_t base, uint64_t q, size_t count) {
    uint64_t p = start % q;
    for (size_t i = 0; i < count; i++) {
        out[i] = p;
        p = (uint64_t)(((u128)p * base) % q);
    }
}

void orc_shoup_table(uint64_t *out, const uint64_t *w, uint64_t q, size_t count) {
    for (size_t i = 0; i < count; i++) out[i] = orc_shoup_quotient(w[i], q);
}

/* --------------------------------------------------------------------------------------------
 * negacyclic NTT -- src/ntt/butterfly.cuh, src/ntt/ntt_1d.cu (loop structure), output order and
 * range as src/ntt/fntt_2d.cu:231-241 / src/ntt/intt_2d.cu
 * ------------------------------------------------------------------------------------------ */

/* src/ntt/butterfly.cuh:10-20 (Harvey lazy Cooley-Tukey butterfly), loop of src/ntt/ntt_1d.cu:38-73 */
void orc_ntt_fwd(uint64_t *a, uint32_t logn, uint64_t q, const uint64_t *tw, const uint64_t *twq) {
    size_t n = (size_t)1 << logn;
    uint64_t q2 = 2 * q;
    for (size_t m = 1, t = n >> 1; m < n; m <<= 1, t >>= 1) {
        for (size_t k = 0; k < m; k++) {
            uint64_t w = tw[m + k], wq = twq[m + k];
            uint64_t *x = a + 2 * k * t, *y = x + t;
            for (size_t j = 0; j < t; j++) {
                uint64_t ty = mul_shoup_lazy(y[j], w, wq, q);
                uint64_t xv = x[j];
                if (xv >= q2) xv -= q2;
                y[j] = xv + q2 - ty;
                x[j] = xv + ty;
            }
        }
    }
    for (size_t i = 0; i < n; i++) {
        uint64_t v = a[i];
        if (v >= q2) v -= q2;
        if (v >= q) v -= q;
        a[i] = v;
    }
}

/* src/ntt/butterfly.cuh:29-43 (Gentleman-Sande butterfly with the halving folded in), loop of
 * src/ntt/ntt_1d.cu:129-170.  itw holds psi^-bitrev(i) / 2, so no final multiply by 1/N. */
void orc_ntt_inv(uint64_t *a, uint32_t logn, uint64_t q, const uint64_t *itw, const uint64_t *itwq) {
    size_t n = (size_t)1 << logn;
    uint64_t q2 = 2 * q;
    for (size_t m = n >> 1, t = 1; m >= 1; m >>= 1, t <<= 1) {
        for (size_t k = 0; k < m; k++) {
            uint64_t w = itw[m + k], wq = itwq[m + k];
            uint64_t *x = a + 2 * k * t, *y = x + t;
            for (size_t j = 0; j < t; j++) {
                uint64_t tt = x[j] + q2 - y[j];
                uint64_t s = x[j] + y[j];
                if (s >= q2) s -= q2;
                if (tt & 1) s += q;
                x[j] = s >> 1;
                y[j] = mul_shoup_lazy(tt, w, wq, q);
            }
        }
    }
    for (size_t i = 0; i < n; i++)
        if (a[i] >= q) a[i] -= q;
}

/* batched forms of src/ntt/fntt_2d.cu:872-910 / src/ntt/intt_2d.cu:693-771: limb i of data uses
 * table tidx[i] */
void orc_ntt_fwd_limbs(const orc_params *p, uint64_t *data, uint32_t nlimbs, const uint32_t *tidx) {
    size_t n = (size_t)1 << p->logn;
#pragma omp parallel for schedule(dynamic)
    for (uint32_t i = 0; i < nlimbs; i++) {
        uint32_t t = tidx[i];
        orc_ntt_fwd(data + (size_t)i * n, p->logn, p->mod[t], p->tw + (size_t)t * n, p->twq + (size_t)t * n);
    }
}

void orc_ntt_inv_limbs(const orc_params *p, uint64_t *data, uint32_t nlimbs, const uint32_t *tidx) {
    size_t n = (size_t)1 << p->logn;
#pragma omp parallel for schedule(dynamic)
    for (uint32_t i = 0; i < nlimbs; i++) {
        uint32_t t = tidx[i];
        orc_ntt_inv(data + (size_t)i * n, p->logn, p->mod[t], p->itw + (size_t)t * n, p->itwq + (size_t)t * n);
    }
}

/* --------------------------------------------------------------------------------------------
 * elementwise kernels -- src/polymath.cu
 * ------------------------------------------------------------------------------------------ */

static inline uint32_t table_index(const orc_params *p, uint32_t L, uint32_t t) {
    return t < L ? t : p->size_q + (t - L);
}

/* op: 0 add (polymath.cu:40), 1 sub (:108), 2 multiply (:160); nlimbs limbs, limb i uses modulus i */
void orc_elementwise(const orc_params *p, int op, const uint64_t *a, const uint64_t *b, uint64_t *out,
                     uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
#pragma omp parallel for
    for (uint32_t l = 0; l < nlimbs; l++) {
        uint64_t q = p->mod[l];
        const uint64_t *r = p->ratio + 2 * (size_t)l;
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) {
            if (op == 0) out[i] = addmod(a[i], b[i], q);
            else if (op == 1) out[i] = submod(a[i], b[i], q);
            else out[i] = mulmod(a[i], b[i], q, r);
        }
    }
}

/* src/polymath.cu:16  negate_rns_poly */
void orc_negate(const orc_params *p, const uint64_t *a, uint64_t *out, uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (uint32_t l = 0; l < nlimbs; l++)
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) out[i] = a[i] ? p->mod[l] - a[i] : 0;
}

/* src/polymath.cu:227 multiply_and_add_rns_poly: out = a*b + c; with negate != 0,
 * :349 multiply_and_add_negate_rns_poly: out = -(a*b + c) */
void orc_mul_add(const orc_params *p, const uint64_t *a, const uint64_t *b, const uint64_t *c, uint64_t *out,
                 uint32_t nlimbs, int negate) {
    size_t n = (size_t)1 << p->logn;
#pragma omp parallel for
    for (uint32_t l = 0; l < nlimbs; l++) {
        uint64_t q = p->mod[l];
        const uint64_t *r = p->ratio + 2 * (size_t)l;
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) {
            uint64_t v = addmod(mulmod(a[i], b[i], q, r), c[i], q);
            out[i] = negate ? (v ? q - v : 0) : v;
        }
    }
}

/* src/polymath.cu:531-566  tensor_prod_2x2_rns_poly: ct1 = (a0,a1), ct2 = (b0,b1), each [2][L][N];
 * out = (d0,d1,d2) [3][L][N] with d1 by the Karatsuba form */
void orc_tensor_2x2(const orc_params *p, const uint64_t *ct1, const uint64_t *ct2, uint64_t *out, uint32_t L) {
    size_t n = (size_t)1 << p->logn, poly = (size_t)L * n;
#pragma omp parallel for
    for (uint32_t l = 0; l < L; l++) {
        uint64_t q = p->mod[l];
        const uint64_t *r = p->ratio + 2 * (size_t)l;
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) {
            uint64_t a0 = ct1[i], a1 = ct1[i + poly], b0 = ct2[i], b1 = ct2[i + poly];
            uint64_t d0 = mulmod(a0, b0, q, r);
            uint64_t d2 = mulmod(a1, b1, q, r);
            uint64_t d1 = mulmod(a0 + a1, b0 + b1, q, r);
            d1 = d1 + 2 * q - d0 - d2;
            if (d1 >= q) d1 -= q;
            if (d1 >= q) d1 -= q;
            out[i] = d0;
            out[i + poly] = d1;
            out[i + 2 * poly] = d2;
        }
    }
}

/* src/polymath.cu:568-612  tensor_square_2x2_rns_poly */
void orc_tensor_square(const orc_params *p, const uint64_t *ct, uint64_t *out, uint32_t L) {
    size_t n = (size_t)1 << p->logn, poly = (size_t)L * n;
#pragma omp parallel for
    for (uint32_t l = 0; l < L; l++) {
        uint64_t q = p->mod[l];
        const uint64_t *r = p->ratio + 2 * (size_t)l;
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) {
            uint64_t c0 = ct[i], c1 = ct[i + poly];
            uint64_t d0 = mulmod(c0, c0, q, r);
            uint64_t d1 = barrett128(((u128)c0 * c1) << 1, q, r);
            uint64_t d2 = mulmod(c1, c1, q, r);
            out[i] = d0;
            out[i + poly] = d1;
            out[i + 2 * poly] = d2;
        }
    }
}

/* src/polymath.cu:614-672  tensor_prod_mxn_rns_poly: out_j = sum over a + b = j of ct1_a * ct2_b, the products
 * summed in 128 bits and reduced once.  ct1 [s1][L][N], ct2 [s2][L][N], out [s1 + s2 - 1][L][N]; out may be ct1's
 * buffer when that has room (every coefficient is read before it is written, as in the reference). */
void orc_tensor_mxn(const orc_params *p, const uint64_t *ct1, uint32_t s1, const uint64_t *ct2, uint32_t s2,
                    uint64_t *out, uint32_t L) {
    size_t n = (size_t)1 << p->logn, poly = (size_t)L * n;
    uint32_t res = s1 + s2 - 1;
#pragma omp parallel for
    for (uint32_t l = 0; l < L; l++) {
        uint64_t q = p->mod[l];
        const uint64_t *r = p->ratio + 2 * (size_t)l;
        for (size_t i = (size_t)l * n; i < (size_t)(l + 1) * n; i++) {
            uint64_t c1[16], c2[16], o[32];
            for (uint32_t a = 0; a < s1; a++) c1[a] = ct1[i + poly * a];
            for (uint32_t b = 0; b < s2; b++) c2[b] = ct2[i + poly * b];
            for (uint32_t j = 0; j < res; j++) {
                uint32_t last1 = j < s1 - 1 ? j : s1 - 1, first2 = j < s2 - 1 ? j : s2 - 1, first1 = j - first2;
                u128 acc = 0;
                for (uint32_t k = 0; k + first1 <= last1; k++) acc += (u128)c1[first1 + k] * c2[first2 - k];
                o[j] = barrett128(acc, q, r);
            }
            for (uint32_t j = 0; j < res; j++) out[i + poly * j] = o[j];
        }
    }
}

/* src/galois.cu:20-30  apply_galois_ntt_permutation: out[limb][i] = in[limb][table[i]] */
void orc_galois_ntt(const orc_params *p, const uint64_t *in, uint64_t *out, const uint32_t *table,
                    uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (uint32_t l = 0; l < nlimbs; l++)
        for (size_t i = 0; i < n; i++) out[(size_t)l * n + i] = in[(size_t)l * n + table[i]];
}

/* include/galois.cuh:45-57  NTT-domain permutation table of Galois element elt */
static uint32_t reverse_bits(uint32_t x, uint32_t bits) {
    uint32_t r = 0;
    for (uint32_t i = 0; i < bits; i++) r |= ((x >> i) & 1u) << (bits - 1 - i);
    return r;
}

void orc_galois_table(uint32_t logn, uint32_t elt, uint32_t *table) {
    uint32_t n = 1u << logn;
    for (uint32_t i = n; i < 2 * n; i++) {
        uint32_t rev = reverse_bits(i, logn + 1);
        uint64_t raw = ((uint64_t)elt * rev) >> 1;
        raw &= (uint64_t)(n - 1);
        table[i - n] = reverse_bits((uint32_t)raw, logn);
    }
}

/* --------------------------------------------------------------------------------------------
 * rescale -- src/rns.cu:507-570  divide_and_round_q_last_ntt
 *   in: [npoly][L][N] NTT form, out: [npoly][L-1][N];  out_j = (c_j - NTT_j(INTT(c_last) mod q_j)) / q_last.
 *   No (q_last-1)/2 rounding offset is applied (the reference's comment at :496 is not implemented).
 * ------------------------------------------------------------------------------------------ */
void orc_rescale(const orc_params *p, const uint64_t *in, uint64_t *out, uint32_t npoly, uint32_t L,
                 const uint64_t *qlast_inv /* [L-1] */, uint64_t *scratch /* N */) {
    size_t n = (size_t)1 << p->logn;
    uint32_t last = L - 1;
    for (uint32_t pi = 0; pi < npoly; pi++) {
        const uint64_t *ci = in + (size_t)pi * L * n;
        uint64_t *co = out + (size_t)pi * last * n;
        memcpy(scratch, ci + (size_t)last * n, n * sizeof(uint64_t));
        orc_ntt_inv(scratch, p->logn, p->mod[last], p->itw + (size_t)last * n, p->itwq + (size_t)last * n);
#pragma omp parallel for
        for (uint32_t j = 0; j < last; j++) {
            uint64_t q = p->mod[j];
            uint64_t *o = co + (size_t)j * n;
            for (size_t i = 0; i < n; i++) o[i] = barrett64(scratch[i], q, p->ratio[2 * j + 1]);
            orc_ntt_fwd(o, p->logn, q, p->tw + (size_t)j * n, p->twq + (size_t)j * n);
            uint64_t w = qlast_inv[j], wq = orc_shoup_quotient(w, q);
            for (size_t i = 0; i < n; i++) o[i] = orc_mul_shoup(submod(ci[(size_t)j * n + i], o[i], q), w, wq, q);
        }
    }
}

/* --------------------------------------------------------------------------------------------
 * hybrid key switching
 * ------------------------------------------------------------------------------------------ */

/* src/rns_bconv.cu:668-792  DRNSTool::modup.
 *   c:      [L][N] NTT form
 *   out:    [beta][L+K][N] NTT form
 *   hatinv: [L]  (Q_d / q_i)^-1 mod q_i for the digit d containing limb i  (src/util/rns.cu:526-551)
 *   mats:   digit d's matrix starts at mats[mat_off[d]], row-major [L+K-size_d][size_d], rows over the
 *           limbs of Ql u P outside the digit in order, entry (Q_d / q_i) mod m_t  (src/util/rns.cu:374-392)
 *   The conversion is the uncorrected sum (no overflow term), accumulated in 128 bits and reduced
 *   once (src/rns_bconv.cu:587-623, include/rns_bconv.cuh:191-209). */
void orc_modup(const orc_params *p, uint32_t L, const uint64_t *c, uint64_t *out, const uint64_t *hatinv,
               const uint64_t *mats, const uint32_t *mat_off, uint64_t *scratch /* L*N */) {
    size_t n = (size_t)1 << p->logn;
    uint32_t K = p->size_p, alpha = K, LK = L + K;
    uint32_t beta = (L + alpha - 1) / alpha;
    /* INTT with the multiply by hatinv folded into the store (src/ntt/ntt_modup.cu:200-290) */
    memcpy(scratch, c, (size_t)L * n * sizeof(uint64_t));
#pragma omp parallel for
    for (uint32_t i = 0; i < L; i++) {
        uint64_t q = p->mod[i], *s = scratch + (size_t)i * n;
        orc_ntt_inv(s, p->logn, q, p->itw + (size_t)i * n, p->itwq + (size_t)i * n);
        uint64_t w = hatinv[i], wq = orc_shoup_quotient(w, q);
        for (size_t j = 0; j < n; j++) s[j] = orc_mul_shoup(s[j], w, wq, q);
    }
    for (uint32_t d = 0; d < beta; d++) {
        uint32_t start = d * alpha, size = (start + alpha <= L) ? alpha : L - start;
        uint64_t *od = out + (size_t)d * LK * n;
        const uint64_t *mat = mats + mat_off[d];
#pragma omp parallel for
        for (uint32_t t = 0; t < LK; t++) {
            uint64_t *o = od + (size_t)t * n;
            if (t >= start && t < start + size) { /* src/rns_bconv.cu:554-560: own limbs stay in NTT form */
                memcpy(o, c + (size_t)t * n, n * sizeof(uint64_t));
                continue;
            }
            uint32_t row = t < start ? t : t - size;
            uint32_t ti = table_index(p, L, t);
            uint64_t m = p->mod[ti];
            const uint64_t *r = p->ratio + 2 * (size_t)ti;
            for (size_t j = 0; j < n; j++) {
                u128 acc = 0;
                for (uint32_t i = 0; i < size; i++)
                    acc += (u128)scratch[(size_t)(start + i) * n + j] * mat[(size_t)row * size + i];
                o[j] = barrett128(acc, m, r);
            }
            orc_ntt_fwd(o, p->logn, m, p->tw + (size_t)ti * n, p->twq + (size_t)ti * n);
        }
    }
}

/* src/eval_key_switch.cu:13-76  key_switch_inner_prod_c2_and_evk.
 *   y:    [beta][L+K][N];  evk[d]: [2][size_q+size_p][N];  out: [2][L+K][N]
 *   128-bit accumulation over the beta digits, one Barrett reduction per output. */
void orc_inner_prod(const orc_params *p, uint32_t L, uint32_t beta, const uint64_t *y, const uint64_t *const *evk,
                    uint64_t *out) {
    size_t n = (size_t)1 << p->logn;
    uint32_t K = p->size_p, LK = L + K, QP = p->size_q + p->size_p;
#pragma omp parallel for
    for (uint32_t t = 0; t < LK; t++) {
        uint32_t ti = table_index(p, L, t);
        uint64_t m = p->mod[ti];
        const uint64_t *r = p->ratio + 2 * (size_t)ti;
        for (size_t j = 0; j < n; j++) {
            u128 a0 = 0, a1 = 0;
            for (uint32_t d = 0; d < beta; d++) {
                uint64_t v = y[((size_t)d * LK + t) * n + j];
                a0 += (u128)v * evk[d][(size_t)ti * n + j];
                a1 += (u128)v * evk[d][((size_t)QP + ti) * n + j];
            }
            out[(size_t)t * n + j] = barrett128(a0, m, r);
            out[((size_t)LK + t) * n + j] = barrett128(a1, m, r);
        }
    }
}

/* src/rns_bconv.cu:965-1053  DRNSTool::moddown_from_NTT (and :871-944 moddown, same mathematics).
 *   cx:       [L+K][N] NTT form (read only)
 *   out:      [L][N]   = (cx_j - NTT_j(delta_j)) * P^-1 mod q_j     (src/ntt/ntt_moddown.cu:244-252)
 *   phat_inv: [K] (P/p_k)^-1 mod p_k; mat: [L][K] (P/p_k) mod q_j; pinv: [L] P^-1 mod q_j
 *   delta_j = sum_k [INTT(cx_{L+k}) * phat_inv_k]_{p_k} * mat[j][k] mod q_j  (src/rns_bconv.cu:249-274) */
void orc_moddown(const orc_params *p, uint32_t L, const uint64_t *cx, uint64_t *out, const uint64_t *phat_inv,
                 const uint64_t *mat, const uint64_t *pinv, uint64_t *scratch /* K*N */) {
    size_t n = (size_t)1 << p->logn;
    uint32_t K = p->size_p;
#pragma omp parallel for
    for (uint32_t k = 0; k < K; k++) {
        uint32_t ti = p->size_q + k;
        uint64_t q = p->mod[ti], *s = scratch + (size_t)k * n;
        memcpy(s, cx + (size_t)(L + k) * n, n * sizeof(uint64_t));
        orc_ntt_inv(s, p->logn, q, p->itw + (size_t)ti * n, p->itwq + (size_t)ti * n);
        uint64_t w = phat_inv[k], wq = orc_shoup_quotient(w, q);
        for (size_t j = 0; j < n; j++) s[j] = orc_mul_shoup(s[j], w, wq, q);
    }
#pragma omp parallel for
    for (uint32_t j = 0; j < L; j++) {
        uint64_t q = p->mod[j];
        const uint64_t *r = p->ratio + 2 * (size_t)j;
        uint64_t *o = out + (size_t)j * n;
        for (size_t i = 0; i < n; i++) {
            u128 acc = 0;
            for (uint32_t k = 0; k < K; k++) acc += (u128)scratch[(size_t)k * n + i] * mat[(size_t)j * K + k];
            o[i] = barrett128(acc, q, r);
        }
        orc_ntt_fwd(o, p->logn, q, p->tw + (size_t)j * n, p->twq + (size_t)j * n);
        uint64_t w = pinv[j], wq = orc_shoup_quotient(w, q);
        for (size_t i = 0; i < n; i++) /* include/uintmodmath.cuh:248-259 sub_negate_const_mult */
            o[i] = orc_mul_shoup(submod(cx[(size_t)j * n + i], o[i], q), w, wq, q);
    }
}

/* src/polymath.cu:320-338  multiply_temp_mod_and_add_rns_poly (key generation): on the limbs of
 * digit d, evk_d.b += [P mod q_i] * s'.   key: [2][QP][N] of digit d, sprime: [QP][N] */
void orc_evk_add_ps(const orc_params *p, uint32_t d, uint64_t *key, const uint64_t *sprime, const uint64_t *p_mod_q) {
    size_t n = (size_t)1 << p->logn;
    uint32_t alpha = p->size_p;
    for (uint32_t i = d * alpha; i < (d + 1) * alpha && i < p->size_q; i++) {
        uint64_t q = p->mod[i];
        uint64_t w = p_mod_q[i], wq = orc_shoup_quotient(w, q);
        for (size_t j = (size_t)i * n; j < (size_t)(i + 1) * n; j++)
            key[j] = addmod(key[j], orc_mul_shoup(sprime[j], w, wq, q), q);
    }
}

/* --------------------------------------------------------------------------------------------
 * samplers.  The reference draws from Salsa20 keyed from /dev/urandom (src/prng.cu:143-242,
 * include/prng.cuh:12-23), which cannot be reproduced; the build uses the ChaCha20 block function
 * (RFC 8439 section 2.3) keyed by a 256-bit seed, with the 64-bit block counter in state words
 * 12-13 and a 64-bit stream id in words 14-15, and keeps the reference's distributions:
 *   ternary: uniform on {-1,0,1}, the same value on every limb        (src/prng.cu:143-174)
 *   error:   centred binomial, 21 bits minus 21 bits, same on every limb (src/prng.cu:219-242)
 *   uniform: uniform residue per limb                                  (src/prng.cu:176-206)
 * ------------------------------------------------------------------------------------------ */
#define ROTL32(v, c) (((v) << (c)) | ((v) >> (32 - (c))))
#define QR(a, b, c, d)                                                                                      \
    a += b; d ^= a; d = ROTL32(d, 16);                                                                      \
    c += d; b ^= c; b = ROTL32(b, 12);                                                                      \
    a += b; d ^= a; d = ROTL32(d, 8);                                                                       \
    c += d; b ^= c; b = ROTL32(b, 7);

void orc_chacha20_block(const uint32_t key[8], uint64_t counter, uint64_t stream, uint32_t out[16]) {
    uint32_t s[16] = {0x61707865u, 0x3320646eu, 0x79622d32u, 0x6b206574u};
    for (int i = 0; i < 8; i++) s[4 + i] = key[i];
    s[12] = (uint32_t)counter;
    s[13] = (uint32_t)(counter >> 32);
    s[14] = (uint32_t)stream;
    s[15] = (uint32_t)(stream >> 32);
    uint32_t x[16];
    memcpy(x, s, sizeof(x));
    for (int i = 0; i < 10; i++) {
        QR(x[0], x[4], x[8], x[12]) QR(x[1], x[5], x[9], x[13]) QR(x[2], x[6], x[10], x[14]) QR(x[3], x[7], x[11], x[15])
        QR(x[0], x[5], x[10], x[15]) QR(x[1], x[6], x[11], x[12]) QR(x[2], x[7], x[8], x[13]) QR(x[3], x[4], x[9], x[14])
    }
    for (int i = 0; i < 16; i++) out[i] = x[i] + s[i];
}

/* one block -> 16 coefficients; word w -> floor(3w / 2^32) - 1 */
void orc_sample_ternary(const orc_params *p, const uint32_t key[8], uint64_t stream, uint64_t *out, uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (size_t b = 0; b < (n + 15) / 16; b++) {
        uint32_t w[16];
        orc_chacha20_block(key, b, stream, w);
        for (size_t e = 0; e < 16 && 16 * b + e < n; e++) {
            uint32_t v = (uint32_t)(((uint64_t)w[e] * 3) >> 32); /* 0,1,2 -> -1,0,1 */
            for (uint32_t l = 0; l < nlimbs; l++)
                out[(size_t)l * n + 16 * b + e] = v == 0 ? p->mod[l] - 1 : v - 1;
        }
    }
}

/* one block -> 8 coefficients; popcount(21 bits) - popcount(21 bits) */
void orc_sample_error(const orc_params *p, const uint32_t key[8], uint64_t stream, uint64_t *out, uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (size_t b = 0; b < (n + 7) / 8; b++) {
        uint32_t w[16];
        orc_chacha20_block(key, b, stream, w);
        for (size_t e = 0; e < 8 && 8 * b + e < n; e++) {
            int v = __builtin_popcount(w[2 * e] & 0x1FFFFFu) - __builtin_popcount(w[2 * e + 1] & 0x1FFFFFu);
            for (uint32_t l = 0; l < nlimbs; l++)
                out[(size_t)l * n + 8 * b + e] = v < 0 ? p->mod[l] - (uint64_t)(-v) : (uint64_t)v;
        }
    }
}

/* one block -> 4 residues of one limb; 128 random bits reduced mod q.  Block counter runs over the
 * whole [nlimbs][N] array so that every limb gets independent values. */
void orc_sample_uniform(const orc_params *p, const uint32_t key[8], uint64_t stream, uint64_t *out, uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (uint32_t l = 0; l < nlimbs; l++) {
        uint64_t q = p->mod[l];
        for (size_t b = 0; b < n / 4; b++) {
            uint32_t w[16];
            orc_chacha20_block(key, (uint64_t)l * (n / 4) + b, stream, w);
            for (size_t e = 0; e < 4; e++) {
                u128 v = ((u128)w[4 * e + 3] << 96) | ((u128)w[4 * e + 2] << 64) | ((u128)w[4 * e + 1] << 32) | w[4 * e];
                out[(size_t)l * n + 4 * b + e] = (uint64_t)(v % q);
            }
        }
    }
}

/* Discrete Gaussian by inversion against a cumulative table (decryption noise flooding; the
 * reference takes it from OpenFHE's generator with sigma = 5.574611952644673, src/secretkey.cu:632-649).
 * cdt[i] = floor(2^63 * P(|X| <= i)), i < cdt_len; one block -> 8 coefficients: word 2e+1:2e gives a
 * 63-bit uniform for the magnitude and one sign bit. */
void orc_sample_gauss(const orc_params *p, const uint32_t key[8], uint64_t stream, uint64_t *out, uint32_t nlimbs,
                      const uint64_t *cdt, uint32_t cdt_len) {
    size_t n = (size_t)1 << p->logn;
    for (size_t b = 0; b < (n + 7) / 8; b++) {
        uint32_t w[16];
        orc_chacha20_block(key, b, stream, w);
        for (size_t e = 0; e < 8 && 8 * b + e < n; e++) {
            uint64_t u = ((uint64_t)w[2 * e + 1] << 32) | w[2 * e];
            int neg = (int)(u >> 63);
            u &= 0x7FFFFFFFFFFFFFFFull;
            uint32_t mag = 0;
            while (mag < cdt_len && u >= cdt[mag]) mag++;
            for (uint32_t l = 0; l < nlimbs; l++)
                out[(size_t)l * n + 8 * b + e] = (neg && mag) ? p->mod[l] - mag : mag;
        }
    }
}

/* --------------------------------------------------------------------------------------------
 * encoder support -- src/rns_base.cu:121-156 (decompose_array_uint64): rounded real coefficient
 * -> residue per limb; coefficient i*gap <- round(re[i]), N/2 + i*gap <- round(im[i])
 * ------------------------------------------------------------------------------------------ */
void orc_decompose_coeffs(const orc_params *p, const double *coeffs /* N, already rounded */, uint64_t *out,
                          uint32_t nlimbs) {
    size_t n = (size_t)1 << p->logn;
    for (uint32_t l = 0; l < nlimbs; l++) {
        uint64_t q = p->mod[l];
        for (size_t i = 0; i < n; i++) {
            double c = coeffs[i];
            uint64_t a = (uint64_t)(c < 0 ? -c : c);
            uint64_t r = barrett64(a, q, p->ratio[2 * l + 1]);
            out[(size_t)l * n + i] = (c < 0 && r) ? q - r : r;
        }
    }
}
