/*
 * cahel_hip.h -- C-ABI of the MI355X (gfx950) CKKS kernel library, libcahel_hip.so.
 *
 * This is the device boundary of the engine: the C++ host layer (context, encoder, keys, evaluator,
 * pyCAHEL binding) calls only these functions and never includes a HIP header.  Each entry point
 * replaces one device routine of the reference (cited per function, paths relative to cahel-main/).
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t value when the HIP runtime failed, or a
 *     negative HE_E_* code for invalid arguments; nothing throws across this boundary
 *   - all polynomial pointers are DEVICE pointers to uint64_t residues in [0, q), layout
 *     [poly][limb][coeff] with the coefficient index fastest (include/ciphertext.h:303-333); outputs
 *     are always canonical residues, and inputs (ciphertexts, keys, plaintexts) must be: a word of q or more
 *     (every q is below 2^61) gives undefined limbs, not an error
 *   - pointers need the 8-byte alignment of their words; buffers that hipMalloc / he_malloc return, and limbs
 *     inside them, are 16-byte aligned, which the kernels use where they can (he_sample requires it)
 *   - "L" is the number of data limbs of the level, K = size_p special limbs; limb t of a Ql u P buffer
 *     uses modulus table t for t < L and size_q + (t - L) otherwise (src/ntt/ntt_modup.cu:404-406)
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); calls are asynchronous on it
 *   - the caller owns every buffer, including the workspaces whose sizes the *_workspace_words functions
 *     return; the library allocates device memory only in he_context_create / he_context_set_level /
 *     he_malloc
 */
#ifndef CAHEL_HIP_H
#define CAHEL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HE_OK 0
#define HE_E_INVALID_ARGUMENT (-1)
#define HE_E_UNSUPPORTED (-2)
#define HE_E_LEVEL_NOT_SET (-3)
#define HE_E_OUT_OF_MEMORY (-4)

typedef struct he_context he_context;
typedef void *he_stream;

/* Human-readable text for a status code returned by any function below. */
const char *he_error_string(int status);

/* ---- device memory and streams: what cahel::util::Pointer<T> / MemoryPoolST give the reference's host
 *      code (include/mempool.cuh:183-280) and its cudaMemcpy/cudaMemset calls ---- */
int he_device_count(int *count);
int he_malloc(void **dev_ptr, size_t bytes);
int he_free(void *dev_ptr);
int he_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, he_stream stream);
/* Page-locked host memory and an upload from it that does not wait: the copy is ordered on `stream` like a kernel, and
 * the caller keeps the source unchanged until the stream has passed it (cudaMallocHost / cudaMemcpyAsync in the
 * reference's terms; src/ckks.cu:143-152 uploads the values of every encoding with a blocking copy). */
int he_host_malloc(void **host_ptr, size_t bytes);
int he_host_free(void *host_ptr);
int he_memcpy_h2d_async(void *dst_dev, const void *src_pinned, size_t bytes, he_stream stream);
int he_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, he_stream stream);
int he_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes, he_stream stream);
/* `rows` runs of `width` bytes, the runs src_pitch bytes apart in the source and dst_pitch bytes apart in the
 * destination (the leading limbs of every polynomial of a batch: a modulus switch that drops limbs without scaling,
 * mod_switch_drop_to_next, src/evaluate.cu:2253-2305, for many polynomials at once). */
int he_memcpy2d_d2d(void *dst_dev, size_t dst_pitch, const void *src_dev, size_t src_pitch, size_t width, size_t rows,
                    he_stream stream);
int he_memset_zero(void *dst_dev, size_t bytes, he_stream stream);
int he_stream_create(he_stream *stream);
int he_stream_destroy(he_stream stream);
int he_stream_synchronize(he_stream stream);

/* Events for timing work on a stream (the role of CUDATimer, include/util.cuh:66-157). */
typedef void *he_event;
int he_event_create(he_event *event);
int he_event_destroy(he_event event);
int he_event_record(he_event event, he_stream stream);
int he_event_synchronize(he_event event);
/* Work enqueued on `stream` after this call starts only when `event` (recorded on another stream) has completed. */
int he_stream_wait_event(he_stream stream, he_event event);
int he_event_elapsed_ms(he_event start, he_event stop, float *ms);

/* ---- parameter tables ---- */

/* Host-side description of one parameter set; replaces the uploads of CAHELGPUContext's constructor
 * (include/gpucontext.h:53-136: DNTTTable, DModulus) and the level-independent part of DRNSTool::init
 * (src/rns.cu:9-67).  All arrays are HOST pointers, copied during he_context_create. */
typedef struct {
    uint32_t log_n;               /* N = 2^log_n, 9 <= log_n <= 17 */
    uint32_t size_q;              /* Q limbs at the key level */
    uint32_t size_p;              /* special limbs (alpha); may be 0 when no key switching is used */
    uint32_t reserved;
    const uint64_t *moduli;       /* [size_q + size_p] q_0..q_{Q-1}, p_0..p_{K-1}, each < 2^61 */
    const uint64_t *barrett;      /* [size_qp][2] floor(2^128 / m): low word, high word */
    const uint64_t *psi;          /* [size_qp][N][2] (psi^bitrev(i), Shoup quotient); src/util/ntt.cu:46-56 */
    const uint64_t *ipsi_div2;    /* [size_qp][N][2] (psi^-bitrev(i) / 2, Shoup quotient); src/util/ntt.cu:58-71 */
    const uint64_t *p_mod_q;      /* [size_q][2] (P mod q_i, Shoup quotient)            src/util/rns.cu:497-508 */
    const uint64_t *pinv_mod_q;   /* [size_q][2] (P^-1 mod q_i, Shoup quotient) */
    const uint64_t *phat_inv_mod_p; /* [size_p][2] ((P/p_k)^-1 mod p_k, Shoup quotient)  src/util/rns.cu:218-270 */
    const uint64_t *phat_mod_q;   /* [size_q][size_p] (P/p_k) mod q_j                    src/util/rns.cu:374-392 */
} he_context_desc;

/* Tables of the data level with L limbs: the hybrid section of RNSTool (src/util/rns.cu:514-551) and
 * inv_q_last_mod_q (:483-488). */
typedef struct {
    uint32_t L;
    uint32_t beta;                   /* ceil(L / size_p) digits */
    const uint64_t *part_hat_inv;    /* [L][2] ((Q_d/q_i)^-1 mod q_i, Shoup quotient), d = digit of limb i */
    const uint64_t *digit_mats;      /* digit d: row-major [L + K - size_d][size_d], (Q_d/q_i) mod m_t over the
                                        limbs t of Ql u P outside the digit, in order */
    const uint32_t *digit_mat_off;   /* [beta] word offset of digit d's matrix in digit_mats */
    const uint64_t *qlast_inv;       /* [L-1][2] (q_{L-1}^-1 mod q_j, Shoup quotient) */
} he_level_desc;

int he_context_create(const he_context_desc *desc, he_context **out);
int he_context_set_level(he_context *ctx, const he_level_desc *level);
int he_context_destroy(he_context *ctx);

/* ---- NTT ---- */

/* Batched forward negacyclic NTT in place.  data: [n_polys][poly_stride_limbs][N]; the first `limbs` limbs
 * of every polynomial are transformed; limb i uses table first_table + i for i < split and
 * tail_table + (i - split) for i >= split (pass split = limbs for a plain range).
 * Replaces nwt_2d_radix8_forward_inplace (src/ntt/fntt_2d.cu:872-910) and its _include_special_mod
 * variant (src/ntt/ntt_modup.cu:591-643). */
int he_ntt_forward(const he_context *ctx, uint64_t *data, uint32_t n_polys, uint32_t poly_stride_limbs,
                   uint32_t limbs, uint32_t first_table, uint32_t split, uint32_t tail_table, he_stream stream);

/* Batched inverse NTT in place (includes the factor 1/N).  Replaces nwt_2d_radix8_backward_inplace
 * (src/ntt/intt_2d.cu:693-771) and _include_special_mod (:773-815). */
int he_ntt_inverse(const he_context *ctx, uint64_t *data, uint32_t n_polys, uint32_t poly_stride_limbs,
                   uint32_t limbs, uint32_t first_table, uint32_t split, uint32_t tail_table, he_stream stream);

/* ---- elementwise polynomial arithmetic (src/polymath.cu:16-180, 227, 349) ----
 * a, b, c, out: [n_polys][limbs][N], limb i mod q_{first_table + i}; out may alias any input. */
int he_add(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
           uint32_t limbs, uint32_t first_table, he_stream stream);
int he_sub(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
           uint32_t limbs, uint32_t first_table, he_stream stream);
int he_negate(const he_context *ctx, const uint64_t *a, uint64_t *out, uint32_t n_polys, uint32_t limbs,
              uint32_t first_table, he_stream stream);
int he_multiply(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
                uint32_t limbs, uint32_t first_table, he_stream stream);
/* out = a*b + c, or -(a*b + c) when negate != 0 */
int he_multiply_add(const he_context *ctx, const uint64_t *a, const uint64_t *b, const uint64_t *c, uint64_t *out,
                    uint32_t n_polys, uint32_t limbs, uint32_t first_table, int negate, he_stream stream);

/* out = a + b * P mod q_i on limbs [first_limb, first_limb + limbs) of Q (a, b, out point at limb first_limb):
 * the key-generation step that plants [P]_{q_i} s' on one digit of a switching key.
 * Replaces multiply_temp_mod_and_add_rns_poly (src/polymath.cu:320-338). */
int he_add_p_multiple(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t first_limb,
                      uint32_t limbs, he_stream stream);

/* (c0,c1) x (c0',c1') -> (d0,d1,d2): ct1, ct2 [2][L][N], out [3][L][N] (out may alias ct1 if it has room).
 * Replaces tensor_prod_2x2_rns_poly (src/polymath.cu:531-566). */
int he_tensor(const he_context *ctx, const uint64_t *ct1, const uint64_t *ct2, uint64_t *out, uint32_t L,
              he_stream stream);
/* Squaring variant; replaces tensor_square_2x2_rns_poly (src/polymath.cu:568-612). */
int he_tensor_square(const he_context *ctx, const uint64_t *ct, uint64_t *out, uint32_t L, he_stream stream);

/* General tensor product of a size-`size1` and a size-`size2` ciphertext (1 <= sizes <= 16): ct1 [size1][L][N],
 * ct2 [size2][L][N] -> out [size1 + size2 - 1][L][N], out_j = sum over a + b = j of ct1_a * ct2_b (dyadic products,
 * summed in 128 bits, one reduction).  out may be ct1's buffer when that has room for the result; it must not
 * overlap ct2 otherwise.  Sizes up to 3 x 3 keep their operands in registers; larger ones read them where they are
 * needed.  Sizes above 16 return HE_E_UNSUPPORTED (the reference allocates its operands per thread with device-side
 * new[] and accepts any size).
 * Replaces tensor_prod_mxn_rns_poly (src/polymath.cu:614-672). */
int he_tensor_mxn(const he_context *ctx, const uint64_t *ct1, uint32_t size1, const uint64_t *ct2, uint32_t size2,
                  uint64_t *out, uint32_t L, he_stream stream);

/* NTT-domain Galois automorphism X -> X^galois_elt of `total_limbs` limbs (any moduli): out[l][i] =
 * in[l][pi(i)]; in and out must not overlap.  Replaces CAHELGPUGaloisTool::apply_galois_ntt
 * (src/galois.cu:20-30, table of include/galois.cuh:45-57, computed on the fly here). */
int he_galois_ntt(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t total_limbs,
                  uint32_t galois_elt, he_stream stream);

/* ---- rescale ---- */

/* in [n_polys][L][N] -> out [n_polys][L-1][N], out_j = (in_j - NTT_j(INTT(in_{L-1}) mod q_j)) / q_{L-1}.
 * workspace: n_polys * N words.  in and out must not overlap.
 * Replaces DRNSTool::divide_and_round_q_last_ntt (src/rns.cu:544-570). */
int he_rescale(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t n_polys, uint32_t L,
               uint64_t *workspace, he_stream stream);

/* he_rescale without a workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc): the coefficient form of the dropped limb goes to a
 * buffer that is part of the library's device image (4 * 65536 words = 2 MiB on every GPU the library runs on,
 * held until the process ends), so the call allocates nothing and passes nothing but inputs and outputs.
 * Limit: n_polys <= 4 (and n_polys * N <= 4 * 65536 words); beyond it the call returns HE_E_UNSUPPORTED and
 * launches nothing.  Same limbs as he_rescale.  All calls on one GPU share the buffer, on every stream: calls
 * that overlap in time on one GPU race; calls issued to one stream are ordered and safe.  Nothing in the buffer
 * has to start at zero (every word read is written earlier in the same call).
 * No counterpart in the reference, whose rescale takes its temporaries from a memory pool. */
int he_rescale_static(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t n_polys, uint32_t L,
                      he_stream stream);

/* ---- hybrid key switching ---- */

/* c [L][N] (NTT) -> out [beta][L+K][N] (NTT).  workspace: L * N words.
 * Replaces DRNSTool::modup (src/rns_bconv.cu:668-792). */
int he_modup(const he_context *ctx, uint32_t L, const uint64_t *c, uint64_t *out, uint64_t *workspace,
             he_stream stream);

/* y [beta][L+K][N], evk: HOST array of beta DEVICE pointers, each [2][size_q+size_p][N] -> out [2][L+K][N].
 * galois_elt != 0 applies X -> X^galois_elt to y while loading (the hoisting form, src/evaluate.cu:2492-2497);
 * accumulate != 0 adds onto out instead of overwriting it (:2571-2576).
 * Replaces key_switch_inner_prod_c2_and_evk (src/eval_key_switch.cu:13-76). */
int he_ks_inner_product(const he_context *ctx, uint32_t L, const uint64_t *y, const uint64_t *const *evk,
                        uint64_t *out, uint32_t galois_elt, int accumulate, he_stream stream);

/* cx [n_polys][L+K][N] (NTT) -> out [n_polys][L][N]: out_j = (cx_j - NTT_j(delta)) * P^-1 mod q_j; with
 * accumulate != 0 the result is added onto out (the add_to_ct step of src/eval_key_switch.cu:193-215).
 * cx's special limbs are overwritten.  workspace: n_polys * L * N words.
 * Replaces DRNSTool::moddown_from_NTT (src/rns_bconv.cu:965-1053) and moddown (:871-944). */
int he_moddown(const he_context *ctx, uint32_t L, uint64_t *cx, uint64_t *out, uint32_t n_polys, int accumulate,
               uint64_t *workspace, he_stream stream);

/* Words of workspace he_keyswitch and he_keyswitch_rescale need at level L:
 * beta*(L+K)*N + 2*(L+K)*N + 2*L*N + 2*N. */
size_t he_keyswitch_workspace_words(const he_context *ctx, uint32_t L);

/* ct[0..1] += KeySwitch(c): c [L][N], ct [2][L][N], evk as in he_ks_inner_product.  galois_elt != 0 switches
 * sigma(c) instead of c (the permutation is fused into the first pass).
 * Replaces switch_key_inplace (src/eval_key_switch.cu:80-216). */
int he_keyswitch(const he_context *ctx, uint32_t L, const uint64_t *c, const uint64_t *const *evk, uint64_t *ct,
                 uint32_t galois_elt, uint64_t *workspace, he_stream stream);

/* ct_out [2][L][N] = (sigma(c0), 0) + KeySwitch(sigma(c1)) for ct_in = (c0, c1) and sigma = X -> X^galois_elt: one
 * keyed rotation.  ct_in and ct_out must not overlap.  workspace as for he_keyswitch.
 * Replaces apply_galois_inplace (src/evaluate.cu:2631-2702): two apply_galois_ntt gathers, a memset and
 * switch_key_inplace. */
int he_rotate(const he_context *ctx, uint32_t L, const uint64_t *ct_in, const uint64_t *const *evk, uint64_t *ct_out,
              uint32_t galois_elt, uint64_t *workspace, he_stream stream);

/* ct_out [2][L][N] = sum over the n_steps Galois elements of the rotation of ct_in = (c0, c1), with ONE ModUp of c1
 * and ONE ModDown pair (hoisting): ct_out = (sum_s sigma_s(c0), 0) + ModDown(sum_s <sigma_s(ModUp(c1)), evk_s>).
 * evk: HOST array of n_steps * beta device pointers, step-major (evk[s * beta + d] = digit d of the key of
 * galois_elts[s], each as in he_ks_inner_product); galois_elts: HOST array of n_steps odd elements below 2N.
 * All steps of up to 64 / beta keys run in one launch.  ct_in and ct_out must not overlap; workspace as for
 * he_keyswitch.  Replaces hoisting_inplace (src/evaluate.cu:2412-2629: per step 1 + beta gathers, an inner product
 * and three additions). */
int he_hoisted_rotations(const he_context *ctx, uint32_t L, const uint64_t *ct_in, const uint64_t *const *evk,
                         const uint32_t *galois_elts, uint32_t n_steps, uint64_t *ct_out, uint64_t *workspace,
                         he_stream stream);

/* The batched forms below run the same kernels over `items` independent inputs in one launch each; Lancelot's
 * ciphertexts have three or four limbs, and one of them neither fills the GPU nor amortises a launch.  They have
 * no counterpart in the reference, which evaluates one ciphertext per call; the limbs they produce are those of
 * `items` separate calls.  workspace: he_keyswitch_batch_workspace_words(ctx, L, items) words. */
size_t he_keyswitch_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items);

/* he_hoisted_rotations over ct_in [items][2][L][N] -> ct_out [items][2][L][N]; add_input != 0 adds the input
 * ciphertext as well: ct_out = ct_in + sum_s rot_s(ct_in), one round of a rotate-and-sum
 * (lancelot-main-GPU/utils/byzantine_fl.py:252-300 does it as hoisting + add_inplace). */
int he_hoisted_rotations_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *ct_in,
                               const uint64_t *const *evk, const uint32_t *galois_elts, uint32_t n_steps, int add_input,
                               uint64_t *ct_out, uint64_t *workspace, he_stream stream);

/* he_keyswitch_rescale over `items` inputs: item k switches c + k * c_item_stride * N (stride in limbs, so that the
 * third polynomial of dense size-3 ciphertexts is c = base + 2 L N, stride 3 L), adds onto ct [items][2][L][N] and
 * writes out [items][2][L-1][N].  galois_elt must be 0 when items > 1. */
int he_keyswitch_rescale_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *c,
                               uint32_t c_item_stride, const uint64_t *const *evk, const uint64_t *ct, uint64_t *out,
                               uint32_t galois_elt, uint64_t *workspace, he_stream stream);

/* (out01 [items][2][L][N], out2 [items][L][N]) = sum over chunks of (a - b)^2 (size-3 tensor square: d0, d1 and d2)
 * for the ciphertext pairs named by the DEVICE pointer table d_pairs [items][chunks][2] (each entry a [2][L][N]
 * ciphertext): the sub, square_inplace and add_inplace loop of GPU_compute_pair_distance
 * (byzantine_fl.py:201-246, lazy relinearisation) in one pass.  d2 is the input of he_keyswitch_rescale_batch
 * (c = out2, c_item_stride = L) and (d0, d1) its ct. */
int he_pair_square_sum(const he_context *ctx, uint32_t L, uint32_t items, uint32_t chunks,
                       const uint64_t *const *d_pairs, uint64_t *out01, uint64_t *out2, he_stream stream);

/* out [2][L-1][N] = rescale(ct + KeySwitch(c)): he_keyswitch followed by he_rescale with the same limbs, in one
 * pass less over the data (ModDown and the rescale share one inverse and one forward transform: the NTT is linear).
 * ct [2][L][N] is only read.  workspace as for he_keyswitch.
 * Replaces the sequence switch_key_inplace (src/eval_key_switch.cu:80-216) + rescale_to_next
 * (src/evaluate.cu:2058-2085) that relinearize_inplace + rescale_to_next_inplace run back to back. */
int he_keyswitch_rescale(const he_context *ctx, uint32_t L, const uint64_t *c, const uint64_t *const *evk,
                         const uint64_t *ct, uint64_t *out, uint32_t galois_elt, uint64_t *workspace,
                         he_stream stream);

/* out [2][L-1][N] = rescale(relinearize(ct1 * ct2)) for two size-2 ciphertexts ct1, ct2 [2][L][N] (ct2 == ct1
 * squares): he_tensor, he_keyswitch and he_rescale with the same limbs in one call; when every prime of the level
 * is below 2^50 the tensor product is formed by the first pass of the key switch's inverse transform (its third
 * polynomial is never read back).  workspace: he_multiply_relin_rescale_workspace_words words.
 * Replaces the sequence multiply (src/evaluate.cu:447-501: tensor_prod_2x2_rns_poly), relinearize_inplace
 * (src/eval_key_switch.cu:80-216) and rescale_to_next (src/evaluate.cu:2058-2085). */
size_t he_multiply_relin_rescale_workspace_words(const he_context *ctx, uint32_t L);
int he_multiply_relin_rescale(const he_context *ctx, uint32_t L, const uint64_t *ct1, const uint64_t *ct2,
                              const uint64_t *const *evk, uint64_t *out, uint64_t *workspace, he_stream stream);

/* he_multiply_relin_rescale over `items` independent products with one launch per stage: ct1, ct2 [items][2][L][N]
 * -> out [items][2][L-1][N] (ct2 == ct1 squares every item), all with the same relinearisation key.  The limbs are
 * those of `items` separate calls.  Contexts with more than 8 special primes are not served (HE_E_UNSUPPORTED: the
 * batched base conversion holds at most 8 input limbs per thread); call he_multiply_relin_rescale per item there.
 * No counterpart in the reference, which multiplies one pair per call.
 * workspace: he_multiply_relin_rescale_batch_workspace_words words. */
size_t he_multiply_relin_rescale_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items);
int he_multiply_relin_rescale_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *ct1,
                                    const uint64_t *ct2, const uint64_t *const *evk, uint64_t *out, uint64_t *workspace,
                                    he_stream stream);

/* ---- encoder support ----
 * coeffs: DEVICE array of N doubles holding integers (already rounded, |c| < 2^63); out [limbs][N]:
 * out[l][i] = c_i mod q_{first_table + l} (negative values wrap to q - |c| mod q).
 * Replaces decompose_array_uint64 (src/rns_base.cu:121-156). */
int he_decompose_real(const he_context *ctx, const double *coeffs, uint64_t *out, uint32_t limbs,
                      uint32_t first_table, he_stream stream);

/* CKKS encode on the device: `count` <= `slots` values (DEVICE arrays re, im; im may be NULL), zero padded to
 * `slots` (a power of two, 2 <= slots <= N/2) -> inverse special FFT over the orbit 5^j mod 2N -> times
 * scale / slots -> rounded to integers -> residues of the first `limbs` primes -> NTT form in out [limbs][N].
 * workspace: DEVICE, he_ckks_workspace_words(ctx, limbs) words; after the call word 0 of the workspace holds, as
 * a double, the largest |coefficient| (the caller compares it with the modulus size, as src/ckks.cu:163-181 does).
 * Replaces CAHELGPUCKKSEncoder::encode_internal (src/ckks.cu:104-209), special_fft_backward (src/fft.cu:350-453)
 * and decompose_array (src/rns_base.cu:306-323). */
int he_ckks_encode(const he_context *ctx, const double *re, const double *im, uint32_t count, uint32_t slots,
                   double scale, uint32_t limbs, uint64_t *out, uint64_t *workspace, he_stream stream);

/* CKKS decode on the device: plain [limbs][N] (NTT form, first `limbs` primes) -> inverse NTT -> CRT
 * composition centred around zero, as doubles divided by `scale` -> forward special FFT.
 * out: DEVICE, 2 * slots doubles, value i = (out[2 i], out[2 i + 1]).  workspace as above.
 * Replaces CAHELGPUCKKSEncoder::decode_internal (src/ckks.cu:292-465), special_fft_forward (src/fft.cu:350-453)
 * and compose_array (src/rns_base.cu:325-459). */
int he_ckks_decode(const he_context *ctx, const uint64_t *plain, uint32_t limbs, uint32_t slots, double scale,
                   double *out, uint64_t *workspace, he_stream stream);

size_t he_ckks_workspace_words(const he_context *ctx, uint32_t limbs);

/* he_ckks_encode over `items` messages with one launch per stage: message k is re + k * value_stride (and im likewise,
 * or NULL), plaintext k is written to out + k * out_poly_stride * N ([limbs][N], NTT form; a stride of 2 * limbs puts
 * it into polynomial 0 of a dense batch of ciphertexts).  The largest |coefficient| of message k is left as a double
 * in workspace[k].  workspace: he_ckks_encode_batch_workspace_words words.  No counterpart in the reference. */
size_t he_ckks_encode_batch_workspace_words(const he_context *ctx, uint32_t items);
int he_ckks_encode_batch(const he_context *ctx, const double *re, const double *im, uint32_t count, uint32_t slots,
                         double scale, uint32_t limbs, uint32_t items, size_t value_stride, uint64_t *out,
                         uint32_t out_poly_stride, uint64_t *workspace, he_stream stream);

/* Public-key encryption of `items` plaintexts with one launch per stage: cts [items][2][L][N] holds plaintext k in
 * polynomial 0 of ciphertext k on entry and ciphertext k on return: (u pk_0 + e_0, u pk_1 + e_1) over Ql u P, divided
 * by P, plus the plaintext.  pk: [2][size_q + size_p][N] at the key level.  Item k draws u, e_0, e_1 from the
 * ChaCha20 streams stream_id + 3 k, + 1, + 2 (what `items` encryptions in a row draw).  Replaces, per item,
 * encrypt_asymmetric (src/secretkey.cu:179-246: encrypt_zero_asymmetric at the key level, DRNSTool::moddown, add).
 * workspace: he_encrypt_batch_workspace_words words. */
size_t he_encrypt_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items);
int he_encrypt_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *pk, const uint32_t key[8],
                     uint64_t stream_id, uint64_t *cts, uint64_t *workspace, he_stream stream);

/* Decryption and decoding of `items` size-2 ciphertexts in one launch per stage: for the ciphertexts [2][limbs][N]
 * named by the DEVICE pointer table d_cts, m = c0 + c1 s (+ noise [items][limbs][N] in NTT form, or NULL), inverse
 * NTT, CRT composition and the special FFT; the first `count` complex slots of every item are written to
 * out [items][count] (re, im).  sk: the secret key in NTT form (its first `limbs` limbs are read).
 * Replaces, per item, ckks_decrypt (src/secretkey.cu:594-654) followed by decode_internal (src/ckks.cu:292-465).
 * workspace: he_decrypt_decode_batch_workspace_words words. */
size_t he_decrypt_decode_batch_workspace_words(const he_context *ctx, uint32_t limbs, uint32_t slots, uint32_t items);
int he_decrypt_decode_batch(const he_context *ctx, const uint64_t *const *d_cts, uint32_t items, uint32_t limbs,
                            const uint64_t *sk, const uint64_t *noise, uint32_t slots, double scale, uint32_t count,
                            double *out, uint64_t *workspace, he_stream stream);

/* ---- samplers (replace sample_ternary_poly / sample_error_poly / sample_uniform_poly, src/prng.cu:143-242,
 *      and the OpenFHE Gaussian of src/secretkey.cu:632-649) ----
 * ChaCha20 block function keyed by key[8]; `stream_id` selects an independent stream.  out: [limbs][N], 16-byte
 * aligned (HE_E_INVALID_ARGUMENT otherwise: the words leave as 16-byte stores),
 * limb i mod table first_table+i (i < split) / tail_table + i - split.
 * kind: 0 ternary {-1,0,1}; 1 centred binomial (21 - 21 bits); 2 uniform residues; 3 discrete Gaussian by
 * the cumulative table cdt[cdt_len] (DEVICE pointer, cdt[i] = floor(2^63 P(|X| <= i))). */
int he_sample(const he_context *ctx, int kind, const uint32_t key[8], uint64_t stream_id, uint64_t *out,
              uint32_t limbs, uint32_t first_table, uint32_t split, uint32_t tail_table, const uint64_t *cdt,
              uint32_t cdt_len, he_stream stream);

/* `items` polynomials in one launch: item k draws from stream_id + k (what `items` calls with consecutive stream ids
 * would give) and is written limbs * N words after item k - 1.  No counterpart in the reference. */
int he_sample_batch(const he_context *ctx, int kind, const uint32_t key[8], uint64_t stream_id, uint64_t *out,
                    uint32_t limbs, uint32_t first_table, uint32_t split, uint32_t tail_table, const uint64_t *cdt,
                    uint32_t cdt_len, uint32_t items, he_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* CAHEL_HIP_H */
