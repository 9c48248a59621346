// Internal interface between the C-ABI layer (capi.hip) and the kernel translation units.
// Nothing here is visible to callers of the shared library; see include/cahel_hip.h for that.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace he {

// Launch choices that the context fixes once, when it is created (the device's size and the environment switches
// that select bit-identical alternates): the launchers read nothing from the environment themselves.
struct Tuning {
    uint32_t cus = 256;              // compute units of the context's device
    uint32_t fuse_rows_forced = 0;   // CAHEL_HIP_FUSE_ROWS: output limbs per workgroup of bconv_rows_fp_kernel, 0 = chosen per launch
    uint32_t bconv_rows = 6;         // CAHEL_HIP_BCONV_ROWS: output rows per workgroup of the batched base conversion
    bool hoist_no_local = false;     // CAHEL_HIP_NO_LOCAL_HOIST=1
    bool hoist_no_xcd = false;       // CAHEL_HIP_NO_XCD_MAP=1
    bool hoist_no_contig = false;    // CAHEL_HIP_NO_XCD_CONTIG=1
    bool no_matrix_bconv = false;    // CAHEL_HIP_NO_MATRIX_BCONV=1: the fused base conversion stays on the FP64 vector units
    bool no_source_intt = false;     // CAHEL_HIP_NO_SOURCE_INTT=1: K = 1, small launches: the inverse rows pass of a reduced
                                     // source limb stays a launch of its own
};

// One limb-sized NTT job given explicitly: which limb of the buffer, which modulus table.
struct LimbJob {
    uint32_t data_limb;
    uint32_t table;
};

// Consecutive jobs of an explicit list that share a modulus table: the blocks pass of the NTT gives each
// group to one set of workgroups so that the table is read once.
struct LimbGroup {
    uint32_t first;
    uint32_t count;
};

// How limb i (0 <= i < limbs) of every polynomial maps to a modulus table:
//   table(i) = first + i             for i < split
//   table(i) = tail_first + i - split  otherwise
// (the second branch is the "special primes after the first L data primes" layout of a Ql u P buffer).
struct LimbMap {
    uint32_t limbs;
    uint32_t first;
    uint32_t split;
    uint32_t tail_first;
};

__host__ __device__ inline uint32_t map_table(const LimbMap &m, uint32_t i) {
    return i < m.split ? m.first + i : m.tail_first + (i - m.split);
}

inline LimbMap plain_map(uint32_t limbs, uint32_t first = 0) { return LimbMap{limbs, first, limbs, 0}; }

// Prologue of the first forward pass / epilogue of the last pass of either direction.
enum : int {
    NTT_PLAIN = 0,
    // forward prologue: input value = pro_src[poly][coeff] mod q (one source limb broadcast to every limb)
    NTT_PRO_BROADCAST_REDUCE = 1,
    // forward epilogue: dst = (epi_a - v) * w mod q
    NTT_EPI_SUB_MUL = 2,
    // forward epilogue: dst = epi_b + (epi_a - v) * w mod q
    NTT_EPI_SUB_MUL_ADD = 3,
    // inverse epilogue: out = v * w mod q
    NTT_EPI_MUL = 4,
    // forward epilogue: dst = ((epi_a * pro_w + epi_b) - v) * w mod q
    NTT_EPI_FMA_SUB_MUL = 6,
    // forward prologue of the merged ModDown + rescale: with r = pro_src - pro_src2 * pro_w[pro_last] mod q_last
    // (the coefficients of the last limb of the ModDown result), input value = in * pro_w + (r mod q)
    NTT_PRO_MODDOWN_RESCALE = 7,
    // forward prologue: input value = source limb mod q by integer Barrett reduction (the source may be any 64-bit
    // residue, also where the limb itself runs on the FP64 back end).  Map mode: the source of polynomial p is
    // pro_src + p * pro_poly_stride * N.  List mode: the source of job (data_limb, table) of item i is limb
    // data_limb / pro_lk of pro_src + i * pro_item_stride: the base conversion of digits of one limb each (K = 1),
    // whose matrix is all ones, done where the forward transform of the converted limb reads its input
    NTT_PRO_SOURCE_REDUCE = 8,
    // the same with the source limb still in the middle of its inverse transform: pro_src holds the words that the
    // inverse blocks pass left (launch_ntt_inverse with rows_skipped), and the forward rows pass first runs the inverse
    // rows pass on its tile of the source (the two passes work on the same rows x columns tile), without the round trip
    // of the coefficients through memory and without a launch.  Every job repeats its source's inverse rows pass, so
    // this is for launches of a few limbs, which are bound by the latency of one workgroup (ntt_source_intt_ok).
    // Source of a job as for NTT_PRO_SOURCE_REDUCE; its prime is table data_limb / pro_lk in list mode, pro_src_table
    // in map mode; bit t of pro_src_fp_mask says whether the blocks pass of table t ran on the FP64 back end.  The
    // inverse transform's scaling must be N^-1 alone (digits of one limb each).
    NTT_PRO_SOURCE_INTT_REDUCE = 9,
};

struct NttArgs {
    const uint64_t *in;   // limb (poly, i) at in + (poly * in_poly_stride + i) * N
    uint64_t *out;
    uint32_t in_poly_stride;
    uint32_t out_poly_stride;
    const uint64_t *tw;       // [tables][N][2] (operand, Shoup quotient)
    const double *tw_fp;      // [tables][N] twiddles as exact doubles for the FP64 back end (primes below 2^50)
    const double *fp_consts;  // [tables][4]: q, 1/q, N^-1 mod q, (N^-1 mod q)/q
    uint64_t fp_mask;         // bit t: table t has a prime below 2^50 (read by the mixed back end only)
    int one_pass;             // N <= 2^14, FP64 back end, plain transforms: one kernel with the limb resident in LDS
    const uint64_t *moduli;   // [tables]
    const uint64_t *barrett;  // [tables][2]
    const LimbJob *jobs;      // explicit list (then in/out limbs are absolute, no prologue/epilogue)
    uint32_t n_jobs;
    const LimbGroup *groups;  // partition of `jobs` into runs with one table each (required with `jobs`)
    uint32_t n_groups;
    uint32_t items;           // list mode: the whole list is applied to `items` buffers (0 = 1) ...
    size_t item_stride;       // ... that lie item_stride words apart
    uint32_t batch, n_polys;  // filled in by the launcher
    uint32_t unit_filter;     // blocks pass of a mixed launch run as two kernels (filled in by the launcher): 1 = only the
                              // units whose prime is below 2^50, 2 = only the others, 0 = every unit
    uint32_t log_n;
    LimbMap map;
    int pro_mode;
    int epi_mode;
    const uint64_t *pro_src;  // [poly][pro_poly_stride limbs], the first limb of each poly is the source
    uint32_t pro_poly_stride;
    size_t pro_item_stride;   // NTT_PRO_SOURCE_REDUCE in list mode: words between the sources of consecutive items
    uint32_t pro_lk;          // ... and limbs per digit of the list's buffer (L + K)
    uint32_t pro_src_table;   // NTT_PRO_SOURCE_INTT_REDUCE in map mode: table of the source limb
    uint64_t pro_src_fp_mask; // NTT_PRO_SOURCE_INTT_REDUCE: tables whose inverse blocks pass left FP64 lazy words
    const uint64_t *pro_itw;  // ... and the inverse transform's twiddle tables (laid out like tw and tw_fp)
    const double *pro_itw_fp;
    const uint64_t *epi_a;    // limb (poly, i) like `out`, with its own poly stride
    uint32_t epi_a_poly_stride;
    const uint64_t *epi_b;
    uint32_t epi_b_poly_stride;
    uint32_t epi_b_mask;      // NTT_EPI_SUB_MUL_ADD: bit (poly mod 32) set = that polynomial has an addend
    uint32_t in_galois;       // inverse transform, map mode: the input is sigma(in), gathered by the blocks pass
    const uint64_t *pro_w;    // [limbs][2] Shoup constants of the scaling prologue / epilogue, indexed like w
    const uint64_t *pro_src2; // NTT_PRO_MODDOWN_RESCALE: second source, limb (poly) at pro_src2 + poly * pro2_poly_stride * N
    uint32_t pro2_poly_stride;
    uint32_t pro_last;        // NTT_PRO_MODDOWN_RESCALE: table (and index into pro_w) of the limb that is dropped
    int pro_k1;               // NTT_PRO_MODDOWN_RESCALE with one special prime: the P -> Q conversion is the reduction of
                              // that prime's coefficients, so pro_src2 is the special limb itself (any residue below 2^61)
                              // and both delta_j and delta_last are its Barrett reductions; `in` is not read
    const uint64_t *w;        // [limbs][2] Shoup constants indexed by limb i of the map
    uint64_t *epi_dst;        // destination of the forward epilogues
    uint32_t epi_dst_poly_stride;
};

// Forward transform: phase 1 (strided rows) then phase 2 (contiguous 256-blocks).  `a.in`/`a.out` and the
// prologue describe phase 1's input; phase 2 runs in place on a.out unless an epilogue redirects it.
// backend: NTT_BACKEND_INT, NTT_BACKEND_FP (every table the launch touches must then hold a prime below 2^50) or
// NTT_BACKEND_MIXED (every workgroup picks the FP64 back end when its limb's bit of fp_mask is set, the integer
// one otherwise: for chains that mix primes below and above 2^50, tables below 64 only).
enum : int { NTT_BACKEND_INT = 0, NTT_BACKEND_FP = 1, NTT_BACKEND_MIXED = 2 };
// rows_done: the rows pass has run already (launch_bconv_rows), only the blocks pass is launched.
hipError_t launch_ntt_forward(const NttArgs &a, uint32_t n_polys, int backend, hipStream_t s, bool rows_done = false);
// Inverse transform: phase A (contiguous blocks, reads a.in writes a.out) then phase B (rows, in place on
// a.out, epilogue NTT_EPI_MUL optional).
// blocks_done: the blocks pass has run already (launch_tensor_intt_blocks left its lazy words in a.out), only the
// rows pass is launched.
// rows_skipped: only the blocks pass is launched; a forward transform with NTT_PRO_SOURCE_INTT_REDUCE finishes it.
hipError_t launch_ntt_inverse(const NttArgs &a, uint32_t n_polys, int backend, hipStream_t s, bool blocks_done = false,
                              bool rows_skipped = false);
// whether a forward launch of n_jobs limbs may take NTT_PRO_SOURCE_INTT_REDUCE (2^15 <= N <= 2^16, a launch small
// enough to run on quarter tiles, every table below 64)
bool ntt_source_intt_ok(uint32_t log_n, uint32_t n_jobs, uint32_t n_tables);

// Tensor product of two size-2 ciphertexts fused with the blocks pass of the inverse transform of its third polynomial
// (FP64 back end; every prime of the L limbs below 2^50).  `a`: inverse base arguments with map = the L data limbs
// and out = where the lazy words of INTT(d2) go ([L][N]); finish with launch_ntt_inverse(a, 1, FP, s, true).
struct TensorFuse {
    const uint64_t *ct1, *ct2;   // [2][L][N]
    uint64_t *d01;               // [2][L][N]: d0, d1
    uint64_t *d2;                // [L][N]: d2 in NTT form
    uint32_t L;
    int square;                  // ct2 is ignored, (d0, d1, d2) = (a0^2, 2 a0 a1, a1^2)
};
hipError_t launch_tensor_intt_blocks(NttArgs a, const TensorFuse &x, hipStream_t s);

struct Tables {
    const uint64_t *moduli;
    const uint64_t *barrett;
    uint32_t log_n;
};

// elementwise family, limb i of every poly uses table map_table(map, i)
enum : int { EW_ADD = 0, EW_SUB = 1, EW_MUL = 2, EW_NEG = 3, EW_MUL_ADD = 4, EW_MUL_ADD_NEG = 5 };
hipError_t launch_elementwise(const Tables &t, int op, const uint64_t *a, const uint64_t *b, const uint64_t *c,
                              uint64_t *out, uint32_t n_polys, LimbMap map, hipStream_t s);
// out = a + b * w[limb] on limbs first .. first+limbs-1 (pointers already offset to limb `first`)
hipError_t launch_scalar_mul_add(const Tables &t, const uint64_t *a, const uint64_t *b, uint64_t *out,
                                 const uint64_t *w, uint32_t first, uint32_t limbs, hipStream_t s);
// fp_consts != nullptr: exact FP64 arithmetic (every prime of limbs 0 .. L-1 below 2^50; [tables][4] as in NttArgs)
// items > 1: that many dense inputs [items][2][L][N] -> (d0, d1) in out [items][2][L][N], d2 in out2 [items][L][N]
hipError_t launch_tensor(const Tables &t, const uint64_t *ct1, const uint64_t *ct2, uint64_t *out, uint32_t L,
                         bool square, hipStream_t s, const double *fp_consts = nullptr, uint32_t items = 1,
                         uint64_t *out2 = nullptr);
// ct1 [s1][L][N] x ct2 [s2][L][N] -> out [s1 + s2 - 1][L][N], 1 <= s1, s2 <= 3
hipError_t launch_tensor_mxn(const Tables &t, const uint64_t *ct1, uint32_t s1, const uint64_t *ct2, uint32_t s2,
                             uint64_t *out, uint32_t L, hipStream_t s);
// (out01 [items][2][L][N], out2 [items][L][N]) = sum over chunks of (a - b)^2 for the pairs of ciphertexts in the
// device pointer table pairs [items][chunks][2]
hipError_t launch_pair_square_sum(const Tables &t, const uint64_t *const *pairs, uint64_t *out01, uint64_t *out2,
                                  uint32_t L, uint32_t items, uint32_t chunks, hipStream_t s);
hipError_t launch_galois(const Tables &t, const uint64_t *in, uint64_t *out, uint32_t total_limbs, uint32_t elt,
                         hipStream_t s);

// out[(row_limb(t))][j] = sum_i x[i][j] * mat[row][i] mod m: base conversion of one digit.
//   x: [n_in][N] scaled residues; rows: n_out output limbs, output limb r is written to
//   out + out_limb[r] * N and reduced by table out_table[r] (both small device arrays).
struct BconvArgs {
    const uint64_t *x;
    uint64_t *out;
    const uint64_t *mat;         // [n_out][n_in]
    const uint32_t *out_limb;    // [n_out]
    const uint32_t *out_table;   // [n_out]
    uint32_t n_in, n_out;
};
hipError_t launch_bconv(const Tables &t, const BconvArgs &a, hipStream_t s);

// Batched form: every unit (a ModUp digit or a ModDown polynomial) in one launch, together with the limbs
// that are copied unchanged (a digit's own limbs keep their NTT form).  Requires n_in <= 8.
struct BconvDesc {
    uint64_t x_off;      // words from x_base to this unit's first input limb
    uint64_t out_off;    // words from out_base to limb 0 of this unit's output buffer
    uint64_t mat_off;    // words from mat_base to this unit's row-major [n_out][n_in] matrix
    uint32_t map_off;    // offset into out_limb / out_table
    uint32_t n_in, n_out;
    uint32_t copy_first, copy_count;  // limbs copied from copy_base (same limb index in the unit's output)
    uint32_t mx_off;     // first record of this unit in BconvRows::mx_tab (one record per four output rows)
};
struct BconvBatch {
    const uint64_t *x_base;
    uint64_t *out_base;
    const uint64_t *copy_base;
    const uint64_t *mat_base;
    const uint32_t *out_limb;
    const uint32_t *out_table;
    const BconvDesc *descs;  // device memory
    uint32_t n_units, max_rows, max_copy;
    // the same units applied to `items` inputs (0 = 1): item k reads x_base + k * x_item_stride (and copy_base + k *
    // copy_item_stride) and writes out_base + k * out_item_stride (strides in words)
    // FP64 back end (all primes involved below 2^50): the matrix as (M, M/m) pairs at the same offsets * 2,
    // per-table constants as in NttArgs::fp_consts; null selects the integer kernel
    const double *mat_fp;
    const double *fp_consts;
    uint32_t items;
    size_t x_item_stride, out_item_stride, copy_item_stride;
};
hipError_t launch_bconv_batched(const Tables &t, const BconvBatch &b, const Tuning &tune, hipStream_t s);

// Base conversion fused with the rows pass of the forward transform of its output limbs (FP64 back end, N >= 2^12,
// n_in <= 8): the units of a BconvBatch, with the results left as the lazy words that the blocks pass continues on.
struct BconvRows {
    const uint64_t *x_base;
    uint64_t *out_base;
    const uint64_t *copy_base;   // limbs copied unchanged (descs' copy_first / copy_count), or nullptr
    const double *mat_fp;        // (M, M/m) pairs at 2 * mat_off
    const uint32_t *out_limb;
    const uint32_t *out_table;
    const BconvDesc *descs;      // device memory
    uint32_t n_units, max_rows, max_copy;
    uint32_t items;              // 0 = 1
    size_t x_item_stride, out_item_stride, copy_item_stride;
    // merged ModDown + rescale: the last row of every unit's matrix is the limb that is dropped; the other output
    // limbs receive sum_i x_i M[j][i] + ((t - sum_i x_i M[last][i] mod q_last) mod q_j), t = the limb before x
    int mdr;
    // The unit's matrices for the int8 matrix cores (N = 2^16), or nullptr.  M_ij = M[r][i] 2^(8 j) mod q_r in eight
    // digits of 7 bits: sum_i x_i M[r][i] = sum over the bytes x_ij of x_i of x_ij M_ij (mod q_r), a 64-term product per
    // digit with the bytes as they lie in memory.  One record of kMxRecord 16-byte words per group of four output rows:
    // [half h = digits 4 h .. 4 h + 3][lane]: the lane's 16 bytes of the A operand (row 4 rr + e of the instruction is
    // digit 4 h + e of output row rr; k = 8 limb + byte), then 8 doubles: for each row rr the constant
    // 128 x sum_e 2^(7 e) x (sum of the row of digit e) mod q_r that the sums lack (the bytes enter as x - 128), and a zero.
    const void *mx_tab;
    // mdr: the record of the dropped limb's row, alone and repeated in the four row slots of its record (every lane then
    // holds the row's sums for its coefficient).  Byte 7 of input limb i is free (the residues are below 2^50): the kernel
    // stores byte i of r = (t - sum_i x_i M[last][i]) mod q_last there, and the records of mx_tab multiply it by the
    // digits of 2^(8 i) mod q_r.
    const void *mx_last;
};
constexpr uint32_t kMxRecord = 144;
// `a` supplies the FP64 twiddles and constants of a forward transform (base_args)
hipError_t launch_bconv_rows(const NttArgs &a, const BconvRows &b, const Tuning &tune, hipStream_t s);

constexpr int kMaxDigits = 64;
struct EvkPtrs {
    const uint64_t *p[kMaxDigits];
};
// (2, L+K, N) <- sum_d y_d * evk_d ; galois_elt != 0 applies the NTT-domain automorphism to y on load.
// items inputs (y and out dense, fold_ct fold_item_stride words apart) in one launch.
// fold_ct / fold_w as in KsFuseArgs (nullptr: plain inner product).
// add_c0 / add_elt / p_mod_q as in KsFuseArgs (add_elt = 0: add_c0 is added as it is; items must be 1).
// own: the key switch's input in NTT form, from which a digit's own limbs are read instead of from y; own_elt != 0:
// that input is sigma(own), X -> X^own_elt, gathered on load.
hipError_t launch_inner_product(const Tables &t, const uint64_t *y, const EvkPtrs &evk, uint64_t *out, uint32_t L,
                                uint32_t K, uint32_t size_q, uint32_t beta, uint32_t galois_elt, bool accumulate,
                                const uint64_t *fold_ct, const uint64_t *fold_w, uint32_t items, size_t fold_item_stride,
                                hipStream_t s, const uint64_t *add_c0 = nullptr, uint32_t add_elt = 0,
                                const uint64_t *p_mod_q = nullptr, const uint64_t *own = nullptr, size_t own_item_stride = 0,
                                uint32_t own_elt = 0);

// The same product for a batch on the FP64 back end (every prime below 2^50, N >= 512): key words are loaded once
// per group of up to 8 items, and a digit's own limbs come from own (the key switch's input in NTT form, items
// own_item_stride words apart) instead of a copy inside y, whose own-limb slots are not read.
hipError_t launch_inner_product_fp(const Tables &t, const double *fp_consts, const uint64_t *y, const uint64_t *own,
                                   size_t own_item_stride, const EvkPtrs &evk, uint64_t *out, uint32_t L, uint32_t K,
                                   uint32_t size_q, uint32_t beta, const uint64_t *fold_ct, const uint64_t *fold_w,
                                   uint32_t items, size_t fold_item_stride, hipStream_t s);

// Hoisted rotations: out (2, L+K, N) (+)= sum over steps of the inner product of sigma_s(y) with the step's key, and
// c0_out (L, N) (+)= sum_s sigma_s(c0).  with_self: c0_out also receives c0 itself and the L limbs after it a copy
// of the L limbs after c0 (c1), so that ModDown can add onto the input ciphertext.  items: that many inputs,
// y and out dense, the ciphertexts ct_item_stride words apart.  evk: n_steps * beta HOST-side device pointers, step-major; n_steps * beta <=
// kMaxDigits per launch.  fp_consts / fp_mask: rows whose table has its bit set (a prime below 2^50) form their
// products in exact FP64 arithmetic; the results are the same canonical residues.  own_from_ct: y holds no copy of the
// digits' own limbs (ModUp skipped it); they are read from c1 of the input ciphertext, which follows c0's L limbs.
hipError_t launch_hoist_inner(const Tables &t, const Tuning &tune, const uint64_t *y, const uint64_t *c0, const uint64_t *const *evk,
                              const uint32_t *elts, uint32_t n_steps, uint64_t *out, uint64_t *c0_out, uint32_t L,
                              uint32_t K, uint32_t size_q, uint32_t beta, bool accumulate, bool with_self, uint32_t items,
                              size_t ct_item_stride, hipStream_t s, const double *fp_consts = nullptr, uint64_t fp_mask = 0,
                              bool own_from_ct = false);

// Forward NTT of ModUp's converted limbs fused with the key-switch inner product (FP64 back end only).
// `a` describes the converted limbs as launch_ntt_forward's job list does (a.out = the beta x (L+K) x N digit
// buffer, whose own-digit limbs are never touched); the blocks pass multiplies every transformed tile by the
// matching key tile and accumulates over the digits, so the transformed limbs are never written:
//   out[k][t] = sum_d y_d[t] * evk_d[k][t],  y_d[t] = own[t] for the limbs t of digit d itself.
struct KsFuseArgs {
    EvkPtrs evk;          // per digit: [2][size_qp][N], NTT form
    const uint64_t *own;  // the key-switch input c, [L][N], NTT form
    uint32_t own_galois;  // != 0: the input is sigma(own), gathered while it is read
    // optional (a rotation): out[0][t] += P * sigma(add_c0)[t] on the data limbs, with the same sigma; the ModDown that
    // follows divides by P, so the rotated c0 arrives in the result without a pass of its own
    const uint64_t *add_c0;   // [L][N], NTT form
    const uint64_t *p_mod_q;  // [size_q][2] Shoup pairs of P mod q_i
    uint64_t *out;        // [2][L+K][N]
    uint32_t L, K, size_q, size_qp, beta;
    // optional: limb L-1 of the result becomes out * fold_w + fold_ct[k][L-1] (what the merged ModDown + rescale
    // transforms back to coefficients); fold_ct = nullptr leaves the inner product as it is
    const uint64_t *fold_ct;  // [2][L][N]
    const uint64_t *fold_w;   // Shoup pair of P^-1 mod q_{L-1}
    // items > 1: that many inputs in one launch (no Galois element, no add_c0); item i's own limbs, output and fold_ct
    // lie i * own_item_stride, i * 2 (L+K) N and i * fold_item_stride words further on, its lazy digits
    // i * NttArgs::item_stride.  The workgroups of one (limb, tile) for all items are placed on one XCD next to each
    // other, so that the key tile is read from memory by the first and from that XCD's L2 by the others.
    uint32_t items;
    size_t own_item_stride, fold_item_stride;
};
hipError_t launch_ntt_forward_inner(const NttArgs &a, const KsFuseArgs &x, hipStream_t s, bool rows_done = false);

hipError_t launch_decompose_real(const Tables &t, const double *coeffs, uint64_t *out, uint32_t limbs, uint32_t first,
                                 uint32_t items, size_t out_item_stride, hipStream_t s);

// samplers (ChaCha20 block function keyed by key[8]; distributions as in the CPU checker)
enum : int { SAMPLE_TERNARY = 0, SAMPLE_ERROR = 1, SAMPLE_UNIFORM = 2, SAMPLE_GAUSS = 3 };
struct ChaChaKey {
    uint32_t k[8];
};
// items polynomials in one launch: item k draws from stream_id + k * stream_stride and lands k * out_item_stride words on
hipError_t launch_sample(const Tables &t, int kind, ChaChaKey key, uint64_t stream_id, uint64_t *out, LimbMap map,
                         const uint64_t *cdt, uint32_t cdt_len, uint32_t items, uint32_t stream_stride,
                         size_t out_item_stride, hipStream_t s);
// u, e0, e1 of `items` public-key encryptions in one launch: out = [items] ternary polynomials, then [items][2]
// error polynomials, poly_stride words apart; item k draws from the streams stream_id + 3 k, + 1, + 2
hipError_t launch_sample_encrypt(const Tables &t, ChaChaKey key, uint64_t stream_id, uint64_t *out, LimbMap map,
                                 uint32_t items, size_t poly_stride, hipStream_t s);
// wide [items][2][L+K][N] += u [items][L+K][N] * pk [2][size_q+K][N] (both polynomials of the public key)
hipError_t launch_encrypt_fma(const Tables &t, const uint64_t *u, const uint64_t *pk, uint64_t *wide, uint32_t L,
                              uint32_t K, uint32_t size_q, uint32_t items, hipStream_t s);

// CKKS encoder tables: 5^j mod 2N for j < N/2 and e^{2 pi i k / 2N} for k <= 2N.
struct FftTables {
    const uint32_t *rot_group;
    const double2 *ksi;
    uint32_t log_n;
};
// values (count <= slots, zero padded) -> rounded real coefficients [N]; *max_bits receives the bit pattern of the
// largest |coefficient| (a non-negative double).  v: scratch of `slots` complex values.  With `out` the coefficients
// leave as residues of the first `limbs` primes of `tab` instead (out [items][limbs][N], items out_item_stride words
// apart) and coeffs is not written.
hipError_t launch_ckks_encode(const FftTables &t, const double *re, const double *im, uint32_t count, uint32_t slots,
                              double scale, double2 *v, double *coeffs, uint64_t *max_bits, uint32_t items,
                              size_t value_stride, hipStream_t s, const Tables *tab = nullptr, uint64_t *out = nullptr,
                              uint32_t limbs = 0, size_t out_item_stride = 0);
// res: [limbs][N] coefficient-form residues of the first `limbs` primes -> v: `slots` complex values.
// garner_inv[i * stride + j] = q_j^-1 mod q_i for j < i.
// items: that many dense plaintexts res [items][limbs][N] -> v [items][slots].
hipError_t launch_ckks_decode(const FftTables &t, const Tables &tab, const uint64_t *res, uint32_t limbs,
                              uint32_t slots, double scale, const uint64_t *garner_inv, uint32_t garner_stride,
                              double2 *v, uint32_t items, hipStream_t s);
// out [items][count] = the first `count` values of every v [items][slots]
hipError_t launch_take_slots(const double2 *v, uint32_t slots, uint32_t items, uint32_t count, double2 *out, hipStream_t s);
// out [items][limbs][N] = c0 + c1 * s (+ noise [items][limbs][N]) for the size-2 ciphertexts [2][limbs][N] named by the
// device pointer table cts [items]; s holds the secret key's first `limbs` limbs
hipError_t launch_decrypt_gather(const Tables &t, const uint64_t *const *cts, const uint64_t *sk, const uint64_t *noise,
                                 uint64_t *out, uint32_t limbs, uint32_t items, hipStream_t s);

}  // namespace he
