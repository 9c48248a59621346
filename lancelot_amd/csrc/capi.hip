// C-ABI of libcahel_hip.so (declared in include/cahel_hip.h): parameter tables on the device and the
// orchestration of the kernels in ntt.hip / rns.hip into the operations of the CKKS hot path.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/cahel_hip.h"
#include "kernels.h"

using namespace he;

namespace {

struct Digit {
    uint32_t start = 0, size = 0, n_out = 0;
    uint32_t *d_out_limb = nullptr;   // [n_out] limb of Ql u P each matrix row writes
    uint32_t *d_out_table = nullptr;  // [n_out] modulus table of that limb
    size_t mat_off = 0;
};

struct Level {
    bool set = false;
    uint32_t L = 0, beta = 0;
    uint64_t *d_part_hat_inv = nullptr;  // [L][2]
    uint64_t *d_mats = nullptr;
    uint64_t *d_qlast_inv = nullptr;     // [L-1][2]
    uint64_t *d_mdr_w = nullptr;         // [1+K][2]: 1 mod q_{L-1}, then (P/p_k)^-1 mod p_k (merged ModDown + rescale)
    std::vector<Digit> digits;
    LimbJob *d_modup_jobs = nullptr;     // NTT jobs over the converted limbs of all digits
    uint32_t n_modup_jobs = 0;
    LimbGroup *d_modup_groups = nullptr; // runs of those jobs that share a modulus table
    uint32_t n_modup_groups = 0;
    LimbGroup *d_modup_singles = nullptr; // every job a group of its own (n_modup_jobs of them): for launches so small
                                          // that a workgroup which takes a run of limbs in turn is what they wait for
    // batched base conversion (all digits of ModUp / all polynomials of ModDown in one launch)
    BconvDesc *d_modup_descs = nullptr, *d_moddown_descs = nullptr;
    uint32_t *d_modup_limb = nullptr, *d_modup_table = nullptr;
    uint32_t modup_max_rows = 0, modup_max_copy = 0;
    bool batched = false;
    double *d_mats_fp = nullptr;         // (M, M/m) pairs of the digit matrices, when every prime is below 2^50
    int32_t *d_mx_up = nullptr;          // the same matrices as 7-bit digits for the int8 matrix cores (N = 2^16)
};

}  // namespace

// Scratch of he_rescale_static: the coefficient form of the dropped limb of up to kStaticPolys polynomials at
// N <= 2^16 (2 MiB).  Every GPU the library runs on holds its own copy until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress: kernels and copies get the per-device address kept in
// g_static_ptr.
constexpr uint32_t kStaticPolys = 4;
constexpr size_t kStaticWords = (size_t)kStaticPolys << 16;
static __device__ __align__(256) uint64_t scratch[kStaticWords];

namespace {

constexpr int kMaxDevices = 64;
uint64_t *g_static_ptr[kMaxDevices];
std::mutex g_static_mutex;

// Address of `scratch` on the current device, resolved once per device with that device current.
int static_scratch(uint64_t **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HE_E_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        uint64_t *p = nullptr;
        e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return HE_E_UNSUPPORTED;
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return HE_OK;
}

}  // namespace

struct he_context {
    uint32_t log_n = 0, size_q = 0, size_p = 0, size_qp = 0;
    int device = 0;
    uint64_t *d_moduli = nullptr, *d_barrett = nullptr, *d_psi = nullptr, *d_ipsi = nullptr;
    uint64_t *d_p_mod_q = nullptr, *d_pinv_mod_q = nullptr, *d_phat_inv = nullptr, *d_phat_mod_q = nullptr;
    uint32_t *d_iota = nullptr;  // 0, 1, 2, ...: row -> limb/table map of the P -> Ql conversion
    std::vector<uint64_t> h_phat_inv;    // host copy of d_phat_inv
    double *d_psi_fp = nullptr, *d_ipsi_fp = nullptr, *d_fp_consts = nullptr;  // FP64 back end tables
    double *d_phat_mod_q_fp = nullptr;   // (M, M/q_j) pairs of the P -> Ql matrix
    double *d_phat_pinv_fp = nullptr;    // the same matrix times P^-1 mod q_j (merged ModDown + rescale, fused kernel)
    bool fuse_rows = true;       // environment CAHEL_HIP_NO_FUSED_BCONV=1: conversion kernel, then the rows pass
    bool fuse_tensor = true;     // environment CAHEL_HIP_NO_FUSED_TENSOR=1: he_multiply_relin_rescale as tensor kernel + key switch
    bool single_limb_digits = false;  // K = 1 (environment CAHEL_HIP_NO_REDUCE_IN_NTT=1: keep the conversion kernels)
    bool batch_fused_inner = true;  // environment CAHEL_HIP_NO_BATCH_FUSED_KS=1: a batch's inner product as a kernel of its own
    uint32_t *d_rot_group = nullptr;     // encoder: 5^j mod 2N
    double2 *d_ksi = nullptr;            // encoder: e^{2 pi i k / 2N}, k <= 2N
    uint64_t *d_garner_inv = nullptr;    // decoder: [size_q][size_q], q_j^-1 mod q_i for j < i
    std::vector<uint64_t> h_moduli;
    std::vector<uint8_t> fp_ok;  // per table: prime below 2^50
    bool use_fp = true;          // environment CAHEL_HIP_NO_FP64=1 forces the integer back end
    bool fuse_inner = true;      // environment CAHEL_HIP_NO_FUSED_KS=1: separate NTT and inner-product kernels
    uint64_t fp_mask = 0;        // bit t: table t has a prime below 2^50
    bool mixed_ok = false;       // mixed launches allowed (at most 64 tables; CAHEL_HIP_NO_MIXED=1 switches them off)
    int one_pass = 1;            // environment CAHEL_HIP_NO_ONE_PASS=1: plain transforms at N <= 2^14 as rows pass + blocks pass;
                                 // CAHEL_HIP_FORCE_ONE_PASS=1: the whole-limb kernel also where two launches are faster
    Tuning tune;                 // the device's size and the switches that the launchers would otherwise read per launch
    std::vector<Level> levels;   // indexed by L
    std::vector<void *> owned;

    int32_t *d_mx_down = nullptr, *d_mx_last = nullptr;   // the P -> Ql matrix (times P^-1) for the int8 matrix cores
    Tables tables() const { return Tables{d_moduli, d_barrett, log_n}; }
    size_t n() const { return (size_t)1 << log_n; }
};

namespace {

#define HE_HIP(expr)                          \
    do {                                      \
        hipError_t _e = (expr);               \
        if (_e != hipSuccess) return (int)_e; \
    } while (0)

// One record of BconvRows::mx_tab: up to four rows of a conversion matrix with at most 8 columns as 7-bit digits of
// M[r][i] 2^(8 j) mod q_r, laid out as the A operands of v_mfma_i32_16x16x64_i8, and the constant that undoes the shift of
// the input bytes by 128.  entry(rr, i) / modulus(rr): row rr of the record (rr < rows).  term = +1 / -1: byte 7 of limb i
// carries byte i of a number that is added / subtracted (digits of +-2^(8 i) mod q_r there), see BconvRows::mx_last.
template <typename Entry, typename Modulus>
void mx_record(std::vector<int32_t> &tab, uint32_t rows, uint32_t n_in, int term, Entry entry, Modulus modulus) {
    const size_t base = tab.size();
    tab.resize(base + 4 * kMxRecord, 0);
    int8_t *amat = reinterpret_cast<int8_t *>(tab.data() + base);
    double offs[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint64_t m8[64];
    for (uint32_t rr = 0; rr < 4 && rr < rows; rr++) {
        const uint64_t q = modulus(rr);
        for (uint32_t i = 0; i < 8; i++) {
            uint64_t v = i < n_in ? entry(rr, i) % q : 0;
            for (uint32_t j = 0; j < 7; j++) {
                m8[8 * i + j] = v;
                v = (uint64_t)(((unsigned __int128)v << 8) % q);
            }
            const uint64_t pw = (uint64_t)((((unsigned __int128)1) << (8 * i)) % q);
            m8[8 * i + 7] = (term == 0 || i == 7) ? 0 : term > 0 ? pw : (q - pw) % q;
        }
        for (uint32_t h = 0; h < 2; h++)
            for (uint32_t e = 0; e < 4; e++) {
                // row 4 rr + e of the instruction: lanes 16 kg + (4 rr + e) supply k = 16 kg .. 16 kg + 15
                int64_t sum = 0;
                for (uint32_t k = 0; k < 64; k++) {
                    const int8_t digit = (int8_t)((m8[k] >> (7 * (4 * h + e))) & 127);
                    amat[((size_t)h * 64 + 16 * (k / 16) + 4 * rr + e) * 16 + k % 16] = digit;
                    sum += digit;
                }
                offs[2 * rr + h] += (double)((128 * sum) << (7 * e));
            }
    }
    // one constant per row: (offset of the high group x 2^28 + offset of the low group) mod q
    for (uint32_t rr = 0; rr < 4 && rr < rows; rr++) {
        const uint64_t q = modulus(rr);
        const unsigned __int128 v = ((unsigned __int128)(uint64_t)offs[2 * rr + 1] << 28) + (uint64_t)offs[2 * rr];
        offs[2 * rr] = (double)(uint64_t)(v % q);
        offs[2 * rr + 1] = 0.0;
    }
    memcpy(tab.data() + base + 4 * 128, offs, sizeof(offs));
}

template <typename T>
int upload(he_context *ctx, T **dst, const T *src, size_t count) {
    if (count == 0) {
        *dst = nullptr;
        return HE_OK;
    }
    void *p = nullptr;
    HE_HIP(hipMalloc(&p, count * sizeof(T)));
    ctx->owned.push_back(p);
    HE_HIP(hipMemcpy(p, src, count * sizeof(T), hipMemcpyHostToDevice));
    *dst = static_cast<T *>(p);
    return HE_OK;
}

inline hipStream_t S(he_stream s) { return static_cast<hipStream_t>(s); }

inline uint32_t table_of(const he_context *ctx, uint32_t L, uint32_t t) { return t < L ? t : ctx->size_q + (t - L); }

const Level *level_of(const he_context *ctx, uint32_t L) {
    if (L == 0 || L >= ctx->levels.size() || !ctx->levels[L].set) return nullptr;
    return &ctx->levels[L];
}

NttArgs base_args(const he_context *ctx, bool forward) {
    NttArgs a;
    memset(&a, 0, sizeof(a));
    a.tw = forward ? ctx->d_psi : ctx->d_ipsi;
    a.tw_fp = forward ? ctx->d_psi_fp : ctx->d_ipsi_fp;
    a.fp_consts = ctx->d_fp_consts;
    a.moduli = ctx->d_moduli;
    a.barrett = ctx->d_barrett;
    a.log_n = ctx->log_n;
    a.epi_b_mask = 0xffffffffu;
    a.fp_mask = ctx->fp_mask;
    a.one_pass = ctx->one_pass;
    return a;
}

// Back end of a launch over the tables of a map: FP64 when every prime is below 2^50, integer when none is (or the
// FP64 back end is switched off), else the mixed kernels, in which every workgroup follows its own limb's prime.
// `also`: a further table whose residues the launch reads (the source limb of a prologue); when its prime is not
// below 2^50 the FP64 code cannot take it in and the whole launch stays on the integer back end.
int backend_for(const he_context *ctx, const LimbMap &m, int also = -1) {
    if (!ctx->use_fp || (also >= 0 && !ctx->fp_ok[(size_t)also])) return NTT_BACKEND_INT;
    uint32_t capable = 0;
    for (uint32_t i = 0; i < m.limbs; i++) capable += ctx->fp_ok[map_table(m, i)] != 0;
    if (capable == m.limbs) return NTT_BACKEND_FP;
    return capable && ctx->mixed_ok ? NTT_BACKEND_MIXED : NTT_BACKEND_INT;
}

// the same over the converted limbs of a ModUp at level L (every table of Ql u P takes part)
int backend_for_level(const he_context *ctx, uint32_t L) {
    if (!ctx->use_fp) return NTT_BACKEND_INT;
    uint32_t capable = 0;
    for (uint32_t t = 0; t < L + ctx->size_p; t++) capable += ctx->fp_ok[table_of(ctx, L, t)] != 0;
    if (capable == L + ctx->size_p) return NTT_BACKEND_FP;
    return capable && ctx->mixed_ok ? NTT_BACKEND_MIXED : NTT_BACKEND_INT;
}

// tables whose limbs a launch of this back end transforms in FP64
uint64_t fp_mask_of(const he_context *ctx, int backend) {
    return backend == NTT_BACKEND_INT ? 0 : (backend == NTT_BACKEND_FP ? ~(uint64_t)0 : ctx->fp_mask);
}

// A forward transform that reduces single-limb sources (K = 1) finishes those sources' inverse transform itself when
// the launch is small (NTT_PRO_SOURCE_INTT_REDUCE): the inverse launch then stops after its blocks pass.
// Environment CAHEL_HIP_NO_SOURCE_INTT=1 keeps the two rows passes apart.
bool source_intt_ok(const he_context *ctx, uint32_t n_jobs) {
    return !ctx->tune.no_source_intt && ntt_source_intt_ok(ctx->log_n, n_jobs, ctx->size_qp);
}

void set_source_intt(const he_context *ctx, NttArgs &fwd, int inverse_backend) {
    fwd.pro_mode = NTT_PRO_SOURCE_INTT_REDUCE;
    fwd.pro_src_fp_mask = fp_mask_of(ctx, inverse_backend);
    fwd.pro_itw = ctx->d_ipsi;
    fwd.pro_itw_fp = ctx->d_ipsi_fp;
}

// the FP64 back end applies when every table of the launch has a prime below 2^50
bool fp_for(const he_context *ctx, const LimbMap &m) {
    if (!ctx->use_fp) return false;
    for (uint32_t i = 0; i < m.limbs; i++)
        if (!ctx->fp_ok[map_table(m, i)]) return false;
    return true;
}

bool fp_for_level(const he_context *ctx, uint32_t L) {
    if (!ctx->use_fp) return false;
    for (uint32_t t = 0; t < L + ctx->size_p; t++)
        if (!ctx->fp_ok[table_of(ctx, L, t)]) return false;
    return true;
}

// base conversion fused with the rows pass of the forward transform that follows it (launch_bconv_rows)
bool fuse_rows_ok(const he_context *ctx, const Level *lv, uint32_t L) {
    return ctx->fuse_rows && lv && lv->batched && ctx->log_n >= 12 && ctx->log_n <= 16 && fp_for_level(ctx, L);
}

int check_map(const he_context *ctx, uint32_t limbs, uint32_t first, uint32_t split, uint32_t tail) {
    if (split > limbs) return HE_E_INVALID_ARGUMENT;
    if (first + split > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    if (limbs > split && tail + (limbs - split) > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    return HE_OK;
}

}  // namespace

extern "C" {

const char *he_error_string(int status) {
    switch (status) {
        case HE_OK: return "success";
        case HE_E_INVALID_ARGUMENT: return "invalid argument";
        case HE_E_UNSUPPORTED: return "unsupported parameter";
        case HE_E_LEVEL_NOT_SET: return "tables of this level were not provided (he_context_set_level)";
        case HE_E_OUT_OF_MEMORY: return "out of host memory";
        default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown error";
    }
}

int he_device_count(int *count) {
    if (!count) return HE_E_INVALID_ARGUMENT;
    HE_HIP(hipGetDeviceCount(count));
    return HE_OK;
}

int he_malloc(void **dev_ptr, size_t bytes) {
    if (!dev_ptr) return HE_E_INVALID_ARGUMENT;
    *dev_ptr = nullptr;
    if (bytes == 0) return HE_OK;
    HE_HIP(hipMalloc(dev_ptr, bytes));
    return HE_OK;
}

int he_free(void *dev_ptr) {
    if (dev_ptr) HE_HIP(hipFree(dev_ptr));
    return HE_OK;
}

int he_memcpy_h2d(void *dst, const void *src, size_t bytes, he_stream s) {
    if (bytes == 0) return HE_OK;
    HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, S(s)));
    HE_HIP(hipStreamSynchronize(S(s)));  // the host buffer may be pageable and reused by the caller
    return HE_OK;
}

int he_host_malloc(void **host_ptr, size_t bytes) {
    if (!host_ptr || bytes == 0) return HE_E_INVALID_ARGUMENT;
    *host_ptr = nullptr;
    HE_HIP(hipHostMalloc(host_ptr, bytes, hipHostMallocDefault));
    return HE_OK;
}

int he_host_free(void *host_ptr) {
    if (host_ptr) HE_HIP(hipHostFree(host_ptr));
    return HE_OK;
}

int he_memcpy_h2d_async(void *dst, const void *src, size_t bytes, he_stream s) {
    if (bytes == 0) return HE_OK;
    if (!dst || !src) return HE_E_INVALID_ARGUMENT;
    HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, S(s)));
    return HE_OK;
}

int he_memcpy_d2h(void *dst, const void *src, size_t bytes, he_stream s) {
    if (bytes == 0) return HE_OK;
    HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, S(s)));
    HE_HIP(hipStreamSynchronize(S(s)));
    return HE_OK;
}

int he_memcpy_d2d(void *dst, const void *src, size_t bytes, he_stream s) {
    if (bytes == 0) return HE_OK;
    HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, S(s)));
    return HE_OK;
}

int he_memcpy2d_d2d(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t width, size_t rows,
                    he_stream s) {
    if (width == 0 || rows == 0) return HE_OK;
    if (!dst || !src || dst_pitch < width || src_pitch < width) return HE_E_INVALID_ARGUMENT;
    HE_HIP(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width, rows, hipMemcpyDeviceToDevice, S(s)));
    return HE_OK;
}

int he_memset_zero(void *dst, size_t bytes, he_stream s) {
    if (bytes == 0) return HE_OK;
    HE_HIP(hipMemsetAsync(dst, 0, bytes, S(s)));
    return HE_OK;
}

int he_stream_create(he_stream *s) {
    if (!s) return HE_E_INVALID_ARGUMENT;
    hipStream_t st;
    HE_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    *s = st;
    return HE_OK;
}

int he_stream_destroy(he_stream s) {
    if (s) HE_HIP(hipStreamDestroy(S(s)));
    return HE_OK;
}

int he_stream_synchronize(he_stream s) {
    HE_HIP(hipStreamSynchronize(S(s)));
    return HE_OK;
}

int he_event_create(he_event *e) {
    if (!e) return HE_E_INVALID_ARGUMENT;
    hipEvent_t ev;
    HE_HIP(hipEventCreate(&ev));
    *e = ev;
    return HE_OK;
}

int he_event_destroy(he_event e) {
    if (e) HE_HIP(hipEventDestroy(static_cast<hipEvent_t>(e)));
    return HE_OK;
}

int he_event_record(he_event e, he_stream s) {
    HE_HIP(hipEventRecord(static_cast<hipEvent_t>(e), S(s)));
    return HE_OK;
}

int he_stream_wait_event(he_stream s, he_event e) {
    if (!e) return HE_E_INVALID_ARGUMENT;
    HE_HIP(hipStreamWaitEvent(S(s), static_cast<hipEvent_t>(e), 0));
    return HE_OK;
}

int he_event_synchronize(he_event e) {
    HE_HIP(hipEventSynchronize(static_cast<hipEvent_t>(e)));
    return HE_OK;
}

int he_event_elapsed_ms(he_event start, he_event stop, float *ms) {
    if (!ms) return HE_E_INVALID_ARGUMENT;
    HE_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return HE_OK;
}

int he_context_create(const he_context_desc *d, he_context **out) {
    if (!d || !out || !d->moduli || !d->barrett || !d->psi || !d->ipsi_div2) return HE_E_INVALID_ARGUMENT;
    if (d->log_n < 9 || d->log_n > 17) return HE_E_UNSUPPORTED;
    if (d->size_q == 0 || d->size_q + d->size_p > 256) return HE_E_INVALID_ARGUMENT;
    if (d->size_p && (!d->p_mod_q || !d->pinv_mod_q || !d->phat_inv_mod_p || !d->phat_mod_q)) return HE_E_INVALID_ARGUMENT;
    for (uint32_t i = 0; i < d->size_q + d->size_p; i++)
        if (d->moduli[i] < 2 || (d->moduli[i] >> 61)) return HE_E_UNSUPPORTED;
    he_context *ctx = new (std::nothrow) he_context;
    if (!ctx) return HE_E_OUT_OF_MEMORY;
    ctx->log_n = d->log_n;
    ctx->size_q = d->size_q;
    ctx->size_p = d->size_p;
    ctx->size_qp = d->size_q + d->size_p;
    ctx->levels.resize(ctx->size_q + 1);
    ctx->h_moduli.assign(d->moduli, d->moduli + ctx->size_qp);
    const size_t n = ctx->n(), qp = ctx->size_qp;
    int rc = hipGetDevice(&ctx->device);
    if (!rc) {
        // he_rescale_static's scratch on this device: resolved here, so that the entry point itself only looks it up
        uint64_t *unused = nullptr;
        rc = static_scratch(&unused);
    }
    if (!rc) rc = upload(ctx, &ctx->d_moduli, d->moduli, qp);
    if (!rc) rc = upload(ctx, &ctx->d_barrett, d->barrett, 2 * qp);
    if (!rc) rc = upload(ctx, &ctx->d_psi, d->psi, 2 * qp * n);
    if (!rc) rc = upload(ctx, &ctx->d_ipsi, d->ipsi_div2, 2 * qp * n);
    if (!rc && d->size_p) {
        rc = upload(ctx, &ctx->d_p_mod_q, d->p_mod_q, 2 * (size_t)d->size_q);
        if (!rc) rc = upload(ctx, &ctx->d_pinv_mod_q, d->pinv_mod_q, 2 * (size_t)d->size_q);
        if (!rc) rc = upload(ctx, &ctx->d_phat_inv, d->phat_inv_mod_p, 2 * (size_t)d->size_p);
        ctx->h_phat_inv.assign(d->phat_inv_mod_p, d->phat_inv_mod_p + 2 * (size_t)d->size_p);
        if (!rc) rc = upload(ctx, &ctx->d_phat_mod_q, d->phat_mod_q, (size_t)d->size_q * d->size_p);
    }
    if (!rc) {
        // encoder tables (cahel-main/src/ckks.cu:34-102): rotation group and the 2N-th roots of unity
        const size_t m = 2 * n;
        std::vector<uint32_t> rot(n / 2);
        uint32_t pos = 1;
        for (size_t i = 0; i < n / 2; i++) {
            rot[i] = pos;
            pos = (uint32_t)(((uint64_t)pos * 5) & (m - 1));
        }
        std::vector<double2> ksi(m + 1);
        const double pi = 3.14159265358979323846264338327950288;
        for (size_t k = 0; k <= m; k++) {
            const double angle = 2.0 * pi * (double)k / (double)m;
            ksi[k] = double2{std::cos(angle), std::sin(angle)};
        }
        // Garner constants of the data primes
        const size_t sq = d->size_q;
        std::vector<uint64_t> ginv(sq * sq, 0);
        for (size_t i = 0; i < sq; i++)
            for (size_t j = 0; j < i; j++) {
                const uint64_t qi = d->moduli[i];
                unsigned __int128 base = d->moduli[j] % qi, acc = 1;
                for (uint64_t e = qi - 2; e; e >>= 1) {  // q_i is prime: a^(q_i - 2) = a^-1
                    if (e & 1) acc = acc * base % qi;
                    base = base * base % qi;
                }
                ginv[i * sq + j] = (uint64_t)acc;
            }
        rc = upload(ctx, &ctx->d_rot_group, rot.data(), rot.size());
        if (!rc) rc = upload(ctx, &ctx->d_ksi, ksi.data(), ksi.size());
        if (!rc) rc = upload(ctx, &ctx->d_garner_inv, ginv.data(), ginv.size());
    }
    if (!rc) {
        // FP64 back end: twiddles as doubles (inverse ones un-halved), per-table constants
        const char *env = getenv("CAHEL_HIP_NO_FP64");
        ctx->use_fp = !(env && env[0] == '1');
        const char *nf = getenv("CAHEL_HIP_NO_FUSED_KS");
        ctx->fuse_inner = !(nf && nf[0] == '1');
        const char *nx = getenv("CAHEL_HIP_NO_MIXED");
        ctx->mixed_ok = qp <= 64 && !(nx && nx[0] == '1');
        const char *no1 = getenv("CAHEL_HIP_NO_ONE_PASS"), *f1 = getenv("CAHEL_HIP_FORCE_ONE_PASS");
        ctx->one_pass = (no1 && no1[0] == '1') ? 0 : ((f1 && f1[0] == '1') ? 2 : 1);
        const char *nb = getenv("CAHEL_HIP_NO_FUSED_BCONV");
        ctx->fuse_rows = !(nb && nb[0] == '1');
        const char *nt = getenv("CAHEL_HIP_NO_FUSED_TENSOR");
        ctx->fuse_tensor = !(nt && nt[0] == '1');
        const char *nr = getenv("CAHEL_HIP_NO_REDUCE_IN_NTT");
        ctx->single_limb_digits = ctx->size_p == 1 && !(nr && nr[0] == '1');
        const char *nbf = getenv("CAHEL_HIP_NO_BATCH_FUSED_KS");
        ctx->batch_fused_inner = !(nbf && nbf[0] == '1');
        auto env_on = [](const char *name) { const char *e = getenv(name); return e && e[0] == '1'; };
        auto env_count = [](const char *name, int lo, int hi, int otherwise) {
            const char *e = getenv(name);
            const int v = e ? atoi(e) : otherwise;
            return (uint32_t)(v >= lo && v <= hi ? v : otherwise);
        };
        ctx->tune.hoist_no_local = env_on("CAHEL_HIP_NO_LOCAL_HOIST");
        ctx->tune.hoist_no_xcd = env_on("CAHEL_HIP_NO_XCD_MAP");
        ctx->tune.hoist_no_contig = env_on("CAHEL_HIP_NO_XCD_CONTIG");
        ctx->tune.no_matrix_bconv = env_on("CAHEL_HIP_NO_MATRIX_BCONV");
        ctx->tune.no_source_intt = env_on("CAHEL_HIP_NO_SOURCE_INTT");
        ctx->tune.fuse_rows_forced = env_count("CAHEL_HIP_FUSE_ROWS", 1, 24, 0);
        ctx->tune.bconv_rows = env_count("CAHEL_HIP_BCONV_ROWS", 1, 64, 6);
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device) == hipSuccess && cus > 0)
            ctx->tune.cus = (uint32_t)cus;
        ctx->fp_ok.assign(qp, 0);
        std::vector<double> psi_fp(qp * n, 0.0), ipsi_fp(qp * n, 0.0), consts(4 * qp, 0.0);
        for (size_t t = 0; t < qp; t++) {
            const uint64_t q = d->moduli[t];
            if (q >> 50) continue;
            ctx->fp_ok[t] = 1;
            if (t < 64) ctx->fp_mask |= 1ull << t;
            const double qd = (double)q;
            for (size_t i = 0; i < n; i++) {
                const uint64_t w = d->psi[2 * (t * n + i)];
                uint64_t iw = 2 * d->ipsi_div2[2 * (t * n + i)];
                if (iw >= q) iw -= q;
                psi_fp[t * n + i] = (double)w;
                ipsi_fp[t * n + i] = (double)iw;
            }
            const uint64_t ninv = q - (q - 1) / n;  // q = 1 mod 2N, so N * (q - (q-1)/N) = 1 mod q
            consts[4 * t] = qd;
            consts[4 * t + 1] = 1.0 / qd;
            consts[4 * t + 2] = (double)ninv;
            consts[4 * t + 3] = (double)ninv / qd;
        }
        if (d->size_p) {
            // (16 doubles of padding: the fused conversion kernel fetches 8 pairs per row whatever the row's length)
            std::vector<double> pfp(2 * (size_t)d->size_q * d->size_p + 16, 0.0);
            for (size_t jq = 0; jq < d->size_q; jq++)
                for (size_t k = 0; k < d->size_p; k++) {
                    pfp[2 * (jq * d->size_p + k)] = (double)d->phat_mod_q[jq * d->size_p + k];
                    pfp[2 * (jq * d->size_p + k) + 1] = (double)d->phat_mod_q[jq * d->size_p + k] / (double)d->moduli[jq];
                }
            rc = upload(ctx, &ctx->d_phat_mod_q_fp, pfp.data(), pfp.size());
            // (P / p_k) P^-1 mod q_j: delta_j P^-1 straight from the conversion
            for (size_t jq = 0; jq < d->size_q; jq++)
                for (size_t k = 0; k < d->size_p; k++) {
                    const uint64_t q = d->moduli[jq];
                    const uint64_t v = (uint64_t)((unsigned __int128)d->phat_mod_q[jq * d->size_p + k] * d->pinv_mod_q[2 * jq] % q);
                    pfp[2 * (jq * d->size_p + k)] = (double)v;
                    pfp[2 * (jq * d->size_p + k) + 1] = (double)v / (double)q;
                }
            if (!rc) rc = upload(ctx, &ctx->d_phat_pinv_fp, pfp.data(), pfp.size());
            if (!rc && d->log_n == 16 && d->size_p <= 8) {
                // the same matrix for the int8 matrix cores: rows in groups of four with the bytes of the rescale term,
                // and every row alone (the row of the limb that a level drops)
                std::vector<int32_t> grp, single;
                auto entry = [&](size_t jq, uint32_t k) {
                    return (uint64_t)((unsigned __int128)d->phat_mod_q[jq * d->size_p + k] * d->pinv_mod_q[2 * jq] % d->moduli[jq]);
                };
                for (uint32_t r0 = 0; r0 < d->size_q; r0 += 4)
                    mx_record(grp, d->size_q - r0, d->size_p, 1, [&](uint32_t rr, uint32_t k) { return entry(r0 + rr, k); },
                              [&](uint32_t rr) { return d->moduli[r0 + rr]; });
                for (uint32_t r = 0; r < d->size_q; r++)
                    mx_record(single, 4, d->size_p, 0, [&](uint32_t, uint32_t k) { return entry(r, k); },
                              [&](uint32_t) { return d->moduli[r]; });
                rc = upload(ctx, &ctx->d_mx_down, grp.data(), grp.size());
                if (!rc) rc = upload(ctx, &ctx->d_mx_last, single.data(), single.size());
            }
        }
        if (!rc) rc = upload(ctx, &ctx->d_psi_fp, psi_fp.data(), psi_fp.size());
        if (!rc) rc = upload(ctx, &ctx->d_ipsi_fp, ipsi_fp.data(), ipsi_fp.size());
        if (!rc) rc = upload(ctx, &ctx->d_fp_consts, consts.data(), consts.size());
    }
    if (!rc) {
        std::vector<uint32_t> iota(qp);
        for (uint32_t i = 0; i < qp; i++) iota[i] = i;
        rc = upload(ctx, &ctx->d_iota, iota.data(), qp);
    }
    if (rc) {
        he_context_destroy(ctx);
        return rc;
    }
    *out = ctx;
    return HE_OK;
}

int he_context_set_level(he_context *ctx, const he_level_desc *d) {
    if (!ctx || !d || d->L == 0 || d->L > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    Level &lv = ctx->levels[d->L];
    if (lv.set) return HE_OK;
    const uint32_t L = d->L, K = ctx->size_p;
    lv.L = L;
    int rc = HE_OK;
    if (L > 1) {
        if (!d->qlast_inv) return HE_E_INVALID_ARGUMENT;
        rc = upload(ctx, &lv.d_qlast_inv, d->qlast_inv, 2 * (size_t)(L - 1));
        if (!rc && K) {
            std::vector<uint64_t> w(2 * (size_t)(K + 1));
            w[0] = 1;
            w[1] = (uint64_t)((((unsigned __int128)1) << 64) / ctx->h_moduli[L - 1]);
            std::copy(ctx->h_phat_inv.begin(), ctx->h_phat_inv.end(), w.begin() + 2);
            rc = upload(ctx, &lv.d_mdr_w, w.data(), w.size());
        }
        if (rc) return rc;
    }
    if (K) {
        const uint32_t beta = (L + K - 1) / K;
        if (d->beta != beta || beta > (uint32_t)kMaxDigits || !d->part_hat_inv || !d->digit_mats || !d->digit_mat_off)
            return HE_E_INVALID_ARGUMENT;
        lv.beta = beta;
        rc = upload(ctx, &lv.d_part_hat_inv, d->part_hat_inv, 2 * (size_t)L);
        if (rc) return rc;
        size_t mat_words = 0;
        std::vector<LimbJob> jobs;
        lv.digits.resize(beta);
        for (uint32_t dg = 0; dg < beta; dg++) {
            Digit &g = lv.digits[dg];
            g.start = dg * K;
            g.size = (g.start + K <= L) ? K : L - g.start;
            g.n_out = L + K - g.size;
            g.mat_off = d->digit_mat_off[dg];
            mat_words = g.mat_off + (size_t)g.n_out * g.size;
            std::vector<uint32_t> limb(g.n_out), table(g.n_out);
            for (uint32_t r = 0; r < g.n_out; r++) {
                limb[r] = r < g.start ? r : r + g.size;
                table[r] = table_of(ctx, L, limb[r]);
                jobs.push_back(LimbJob{dg * (L + K) + limb[r], table[r]});
            }
            rc = upload(ctx, &g.d_out_limb, limb.data(), g.n_out);
            if (!rc) rc = upload(ctx, &g.d_out_table, table.data(), g.n_out);
            if (rc) return rc;
        }
        rc = upload(ctx, &lv.d_mats, d->digit_mats, mat_words);
        if (rc) return rc;
        if (K <= 8) {
            const size_t n = ctx->n();
            std::vector<BconvDesc> up(beta), down(4);
            std::vector<uint32_t> limb_all, table_all;
            for (uint32_t dg = 0; dg < beta; dg++) {
                const Digit &g = lv.digits[dg];
                BconvDesc &bd = up[dg];
                memset(&bd, 0, sizeof(bd));
                bd.x_off = (uint64_t)g.start * n;
                bd.out_off = (uint64_t)dg * (L + K) * n;
                bd.mat_off = g.mat_off;
                bd.map_off = (uint32_t)limb_all.size();
                bd.n_in = g.size;
                bd.n_out = g.n_out;
                bd.copy_first = g.start;
                bd.copy_count = g.size;
                for (uint32_t r = 0; r < g.n_out; r++) {
                    const uint32_t lim = r < g.start ? r : r + g.size;
                    limb_all.push_back(lim);
                    table_all.push_back(table_of(ctx, L, lim));
                }
                lv.modup_max_rows = std::max(lv.modup_max_rows, g.n_out);
                lv.modup_max_copy = std::max(lv.modup_max_copy, g.size);
            }
            for (uint32_t p = 0; p < 4; p++) {
                BconvDesc &bd = down[p];
                memset(&bd, 0, sizeof(bd));
                bd.x_off = ((uint64_t)p * (L + K) + L) * n;
                bd.out_off = (uint64_t)p * L * n;
                bd.n_in = K;
                bd.n_out = L;
            }
            rc = upload(ctx, &lv.d_moddown_descs, down.data(), down.size());
            if (!rc) rc = upload(ctx, &lv.d_modup_limb, limb_all.data(), limb_all.size());
            if (!rc) rc = upload(ctx, &lv.d_modup_table, table_all.data(), table_all.size());
            if (rc) return rc;
            lv.batched = true;
            if (fp_for_level(ctx, L)) {
                std::vector<double> mfp(2 * mat_words + 16, 0.0);   // padded as the P -> Ql matrix is
                for (uint32_t dg = 0; dg < beta; dg++) {
                    const Digit &g = lv.digits[dg];
                    for (uint32_t r = 0; r < g.n_out; r++) {
                        const uint32_t lim = r < g.start ? r : r + g.size;
                        const double m = (double)ctx->h_moduli[table_of(ctx, L, lim)];
                        for (uint32_t i = 0; i < g.size; i++) {
                            const size_t idx = g.mat_off + (size_t)r * g.size + i;
                            mfp[2 * idx] = (double)d->digit_mats[idx];
                            mfp[2 * idx + 1] = (double)d->digit_mats[idx] / m;
                        }
                    }
                }
                rc = upload(ctx, &lv.d_mats_fp, mfp.data(), mfp.size());
                if (rc) return rc;
                if (ctx->log_n == 16) {
                    // the digit matrices for the int8 matrix cores (BconvRows::mx_tab), one record per four output rows
                    std::vector<int32_t> tab;
                    for (uint32_t dg = 0; dg < beta; dg++) {
                        const Digit &g = lv.digits[dg];
                        up[dg].mx_off = (uint32_t)(tab.size() / (4 * kMxRecord));
                        for (uint32_t r0 = 0; r0 < g.n_out; r0 += 4)
                            mx_record(tab, g.n_out - r0, g.size, 0,
                                      [&](uint32_t rr, uint32_t i) { return d->digit_mats[g.mat_off + (size_t)(r0 + rr) * g.size + i]; },
                                      [&](uint32_t rr) {
                                          const uint32_t r = r0 + rr;
                                          return ctx->h_moduli[table_of(ctx, L, r < g.start ? r : r + g.size)];
                                      });
                    }
                    rc = upload(ctx, &lv.d_mx_up, tab.data(), tab.size());
                    if (rc) return rc;
                }
            }
            rc = upload(ctx, &lv.d_modup_descs, up.data(), up.size());
            if (rc) return rc;
        }
        // limbs with the same modulus sit together so that one set of workgroups can share the twiddle table
        std::stable_sort(jobs.begin(), jobs.end(), [](const LimbJob &x, const LimbJob &y) { return x.table < y.table; });
        std::vector<LimbGroup> groups;
        for (uint32_t j = 0; j < jobs.size(); j++) {
            if (groups.empty() || jobs[groups.back().first].table != jobs[j].table || groups.back().count == 4)
                groups.push_back(LimbGroup{j, 0});
            groups.back().count++;
        }
        lv.n_modup_jobs = (uint32_t)jobs.size();
        lv.n_modup_groups = (uint32_t)groups.size();
        rc = upload(ctx, &lv.d_modup_jobs, jobs.data(), jobs.size());
        if (!rc) rc = upload(ctx, &lv.d_modup_groups, groups.data(), groups.size());
        std::vector<LimbGroup> singles;
        for (uint32_t j = 0; j < jobs.size(); j++) singles.push_back(LimbGroup{j, 1});
        if (!rc) rc = upload(ctx, &lv.d_modup_singles, singles.data(), singles.size());
        if (rc) return rc;
    }
    lv.set = true;
    return HE_OK;
}

int he_context_destroy(he_context *ctx) {
    if (!ctx) return HE_OK;
    for (void *p : ctx->owned) (void)hipFree(p);
    delete ctx;
    return HE_OK;
}

int he_ntt_forward(const he_context *ctx, uint64_t *data, uint32_t n_polys, uint32_t poly_stride, uint32_t limbs,
                   uint32_t first, uint32_t split, uint32_t tail, he_stream s) {
    if (!ctx || !data || limbs > poly_stride) return HE_E_INVALID_ARGUMENT;
    if (int rc = check_map(ctx, limbs, first, split, tail)) return rc;
    NttArgs a = base_args(ctx, true);
    a.in = data;
    a.out = data;
    a.in_poly_stride = a.out_poly_stride = poly_stride;
    a.map = LimbMap{limbs, first, split, tail};
    HE_HIP(launch_ntt_forward(a, n_polys, backend_for(ctx, a.map), S(s)));
    return HE_OK;
}

int he_ntt_inverse(const he_context *ctx, uint64_t *data, uint32_t n_polys, uint32_t poly_stride, uint32_t limbs,
                   uint32_t first, uint32_t split, uint32_t tail, he_stream s) {
    if (!ctx || !data || limbs > poly_stride) return HE_E_INVALID_ARGUMENT;
    if (int rc = check_map(ctx, limbs, first, split, tail)) return rc;
    NttArgs a = base_args(ctx, false);
    a.in = data;
    a.out = data;
    a.in_poly_stride = a.out_poly_stride = poly_stride;
    a.map = LimbMap{limbs, first, split, tail};
    HE_HIP(launch_ntt_inverse(a, n_polys, backend_for(ctx, a.map), S(s)));
    return HE_OK;
}

static int elementwise(const he_context *ctx, int op, const uint64_t *a, const uint64_t *b, const uint64_t *c,
                       uint64_t *out, uint32_t n_polys, uint32_t limbs, uint32_t first, he_stream s) {
    if (!ctx || !a || !out || (op != EW_NEG && !b)) return HE_E_INVALID_ARGUMENT;
    if (first + limbs > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_elementwise(ctx->tables(), op, a, b, c, out, n_polys, plain_map(limbs, first), S(s)));
    return HE_OK;
}

int he_add(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
           uint32_t limbs, uint32_t first, he_stream s) {
    return elementwise(ctx, EW_ADD, a, b, nullptr, out, n_polys, limbs, first, s);
}

int he_sub(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
           uint32_t limbs, uint32_t first, he_stream s) {
    return elementwise(ctx, EW_SUB, a, b, nullptr, out, n_polys, limbs, first, s);
}

int he_negate(const he_context *ctx, const uint64_t *a, uint64_t *out, uint32_t n_polys, uint32_t limbs,
              uint32_t first, he_stream s) {
    return elementwise(ctx, EW_NEG, a, nullptr, nullptr, out, n_polys, limbs, first, s);
}

int he_multiply(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t n_polys,
                uint32_t limbs, uint32_t first, he_stream s) {
    return elementwise(ctx, EW_MUL, a, b, nullptr, out, n_polys, limbs, first, s);
}

int he_multiply_add(const he_context *ctx, const uint64_t *a, const uint64_t *b, const uint64_t *c, uint64_t *out,
                    uint32_t n_polys, uint32_t limbs, uint32_t first, int negate, he_stream s) {
    if (!c) return HE_E_INVALID_ARGUMENT;
    return elementwise(ctx, negate ? EW_MUL_ADD_NEG : EW_MUL_ADD, a, b, c, out, n_polys, limbs, first, s);
}

int he_add_p_multiple(const he_context *ctx, const uint64_t *a, const uint64_t *b, uint64_t *out, uint32_t first_limb,
                      uint32_t limbs, he_stream s) {
    if (!ctx || !a || !b || !out || ctx->size_p == 0 || first_limb + limbs > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_scalar_mul_add(ctx->tables(), a, b, out, ctx->d_p_mod_q, first_limb, limbs, S(s)));
    return HE_OK;
}

int he_tensor(const he_context *ctx, const uint64_t *ct1, const uint64_t *ct2, uint64_t *out, uint32_t L,
              he_stream s) {
    if (!ctx || !ct1 || !ct2 || !out || L == 0 || L > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_tensor(ctx->tables(), ct1, ct2, out, L, false, S(s),
                         L <= ctx->size_q && fp_for(ctx, plain_map(L)) ? ctx->d_fp_consts : nullptr));
    return HE_OK;
}

int he_tensor_square(const he_context *ctx, const uint64_t *ct, uint64_t *out, uint32_t L, he_stream s) {
    if (!ctx || !ct || !out || L == 0 || L > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_tensor(ctx->tables(), ct, ct, out, L, true, S(s),
                         L <= ctx->size_q && fp_for(ctx, plain_map(L)) ? ctx->d_fp_consts : nullptr));
    return HE_OK;
}

int he_tensor_mxn(const he_context *ctx, const uint64_t *ct1, uint32_t size1, const uint64_t *ct2, uint32_t size2,
                  uint64_t *out, uint32_t L, he_stream s) {
    if (!ctx || !ct1 || !ct2 || !out || L == 0 || L > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    if (size1 == 0 || size2 == 0) return HE_E_INVALID_ARGUMENT;
    if (size1 > 16 || size2 > 16) return HE_E_UNSUPPORTED;
    HE_HIP(launch_tensor_mxn(ctx->tables(), ct1, size1, ct2, size2, out, L, S(s)));
    return HE_OK;
}

int he_pair_square_sum(const he_context *ctx, uint32_t L, uint32_t items, uint32_t chunks,
                       const uint64_t *const *d_pairs, uint64_t *out01, uint64_t *out2, he_stream s) {
    if (!ctx || !d_pairs || !out01 || !out2 || L == 0 || L > ctx->size_q || items == 0 || items > 16384 || chunks == 0)
        return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_pair_square_sum(ctx->tables(), d_pairs, out01, out2, L, items, chunks, S(s)));
    return HE_OK;
}

int he_galois_ntt(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t total_limbs, uint32_t elt,
                  he_stream s) {
    if (!ctx || !in || !out || in == out || !(elt & 1) || elt >= (2u << ctx->log_n)) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_galois(ctx->tables(), in, out, total_limbs, elt, S(s)));
    return HE_OK;
}

int he_rescale(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t n_polys, uint32_t L,
               uint64_t *ws, he_stream s) {
    if (!ctx || !in || !out || !ws || L < 2 || L > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    const size_t n = ctx->n();
    // last limb -> coefficient form, one limb per poly in the workspace
    NttArgs inv = base_args(ctx, false);
    inv.in = in + (size_t)(L - 1) * n;
    inv.in_poly_stride = L;
    inv.out = ws;
    inv.out_poly_stride = 1;
    inv.map = plain_map(1, L - 1);
    HE_HIP(launch_ntt_inverse(inv, n_polys, backend_for(ctx, inv.map), S(s)));
    // every remaining limb: NTT_j(ws mod q_j), then (in_j - that) / q_last
    NttArgs fwd = base_args(ctx, true);
    fwd.pro_mode = NTT_PRO_BROADCAST_REDUCE;
    fwd.pro_src = ws;
    fwd.pro_poly_stride = 1;
    fwd.out = out;
    fwd.out_poly_stride = L - 1;
    fwd.map = plain_map(L - 1, 0);
    fwd.epi_mode = NTT_EPI_SUB_MUL;
    fwd.epi_a = in;
    fwd.epi_a_poly_stride = L;
    fwd.w = lv->d_qlast_inv;
    fwd.epi_dst = out;
    fwd.epi_dst_poly_stride = L - 1;
    // the broadcast source is a residue of q_{L-1}: the FP64 back end needs it below 2^50 as well
    HE_HIP(launch_ntt_forward(fwd, n_polys, backend_for(ctx, fwd.map, (int)L - 1), S(s)));
    return HE_OK;
}

int he_rescale_static(const he_context *ctx, const uint64_t *in, uint64_t *out, uint32_t n_polys, uint32_t L,
                      he_stream s) {
    if (!ctx || n_polys == 0) return HE_E_INVALID_ARGUMENT;
    if (n_polys > kStaticPolys || (size_t)n_polys * ctx->n() > kStaticWords) return HE_E_UNSUPPORTED;
    uint64_t *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    // the scratch needs no clearing: the inverse transform writes every word of it that the forward one reads
    return he_rescale(ctx, in, out, n_polys, L, ws, s);
}

}  // extern "C"

namespace {

// ModUp of `items` polynomials: item k reads c + k * c_item_stride * N (stride in limbs), writes out [k][beta][L+K][N];
// ws holds items * L limbs
// in_galois != 0 (one item, skip_own): the input is sigma(c), X -> X^in_galois, gathered by the inverse blocks pass
int modup_impl(const he_context *ctx, uint32_t L, const uint64_t *c, uint32_t c_item_stride, uint32_t items,
               uint64_t *out, uint64_t *ws, he_stream s, bool skip_own = false, uint32_t in_galois = 0) {
    if (!ctx || !c || !out || !ws || ctx->size_p == 0 || items == 0 || c_item_stride < L) return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    if (items > 1 && !lv->batched) return HE_E_UNSUPPORTED;
    const size_t n = ctx->n();
    const uint32_t LK = L + ctx->size_p;
    // coefficient form scaled by (Q_d / q_i)^-1, out of place into the workspace
    NttArgs inv = base_args(ctx, false);
    inv.in = c;
    inv.out = ws;
    inv.in_poly_stride = c_item_stride;
    inv.out_poly_stride = L;
    inv.map = plain_map(L, 0);
    inv.epi_mode = NTT_EPI_MUL;
    inv.w = lv->d_part_hat_inv;
    // skip_own (batched levels only): the consumer reads a digit's own limbs from c, their slots in out stay unwritten
    if (skip_own && !lv->batched) return HE_E_INVALID_ARGUMENT;
    if (in_galois && (items != 1 || !skip_own)) return HE_E_INVALID_ARGUMENT;   // (own limbs are copied from c as it is)
    inv.in_galois = in_galois;
    const bool fused = fuse_rows_ok(ctx, lv, L);
    // digits of one limb each (K = 1): (Q_d / q_d)^-1 and the conversion matrix are all ones, so the conversion is the
    // reduction of the digit's coefficients modulo each other prime, which the forward transform does where it reads
    // its input; only the digits' own limbs are copied
    const bool reduce_in_ntt = ctx->single_limb_digits && !fused;
    // ... and a small launch finishes the inverse transform there as well
    const int inv_backend = backend_for(ctx, inv.map);
    const bool source_intt = reduce_in_ntt && source_intt_ok(ctx, lv->n_modup_jobs * items);
    HE_HIP(launch_ntt_inverse(inv, items, inv_backend, S(s), false, source_intt));
    const uint32_t copy_rows = skip_own ? 0 : lv->modup_max_copy;
    if (reduce_in_ntt) {
        for (uint32_t d = 0; d < lv->beta && !skip_own; d++)
            HE_HIP(hipMemcpy2DAsync(out + ((size_t)d * LK + d) * n, (size_t)lv->beta * LK * n * sizeof(uint64_t),
                                    c + (size_t)d * n, (size_t)c_item_stride * n * sizeof(uint64_t), n * sizeof(uint64_t),
                                    items, hipMemcpyDeviceToDevice, S(s)));
    } else if (fused) {
        BconvRows b{ws, out, c, lv->d_mats_fp, lv->d_modup_limb, lv->d_modup_table, lv->d_modup_descs,
                    lv->beta, lv->modup_max_rows, copy_rows,
                    items, (size_t)L * n, (size_t)lv->beta * LK * n, (size_t)c_item_stride * n, 0, lv->d_mx_up};
        HE_HIP(launch_bconv_rows(base_args(ctx, true), b, ctx->tune, S(s)));
    } else if (lv->batched) {
        BconvBatch b{ws, out, c, lv->d_mats, lv->d_modup_limb, lv->d_modup_table, lv->d_modup_descs,
                     lv->beta, lv->modup_max_rows, copy_rows, lv->d_mats_fp, ctx->d_fp_consts,
                     items, (size_t)L * n, (size_t)lv->beta * LK * n, (size_t)c_item_stride * n};
        HE_HIP(launch_bconv_batched(ctx->tables(), b, ctx->tune, S(s)));
    }
    for (uint32_t d = 0; d < lv->beta && !lv->batched && !reduce_in_ntt; d++) {
        const Digit &g = lv->digits[d];
        uint64_t *od = out + (size_t)d * LK * n;
        // the digit's own limbs keep their NTT form
        HE_HIP(hipMemcpyAsync(od + (size_t)g.start * n, c + (size_t)g.start * n, (size_t)g.size * n * sizeof(uint64_t),
                              hipMemcpyDeviceToDevice, S(s)));
        BconvArgs b{ws + (size_t)g.start * n, od, lv->d_mats + g.mat_off, g.d_out_limb, g.d_out_table, g.size, g.n_out};
        HE_HIP(launch_bconv(ctx->tables(), b, S(s)));
    }
    NttArgs fwd = base_args(ctx, true);
    fwd.in = out;
    fwd.out = out;
    fwd.jobs = lv->d_modup_jobs;
    fwd.n_jobs = lv->n_modup_jobs;
    // (a launch of at most 1024 workgroups of the smallest tile: one limb per workgroup)
    const bool singles = (uint64_t)lv->n_modup_jobs * items * (n >> 10) <= 1024;
    fwd.groups = singles ? lv->d_modup_singles : lv->d_modup_groups;
    fwd.n_groups = singles ? lv->n_modup_jobs : lv->n_modup_groups;
    fwd.items = items;
    fwd.item_stride = (size_t)lv->beta * LK * n;
    if (reduce_in_ntt) {
        fwd.pro_mode = NTT_PRO_SOURCE_REDUCE;
        fwd.pro_src = ws;
        fwd.pro_item_stride = (size_t)L * n;
        fwd.pro_lk = LK;
        if (source_intt) set_source_intt(ctx, fwd, inv_backend);
    }
    HE_HIP(launch_ntt_forward(fwd, 1, backend_for_level(ctx, L), S(s), fused));
    return HE_OK;
}

}  // namespace

extern "C" {

int he_modup(const he_context *ctx, uint32_t L, const uint64_t *c, uint64_t *out, uint64_t *ws, he_stream s) {
    return modup_impl(ctx, L, c, L, 1, out, ws, s);
}

int he_ks_inner_product(const he_context *ctx, uint32_t L, const uint64_t *y, const uint64_t *const *evk,
                        uint64_t *out, uint32_t galois_elt, int accumulate, he_stream s) {
    if (!ctx || !y || !evk || !out || ctx->size_p == 0 || L == 0 || L > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    if (galois_elt && (!(galois_elt & 1) || galois_elt >= (2u << ctx->log_n))) return HE_E_INVALID_ARGUMENT;
    const uint32_t beta = (L + ctx->size_p - 1) / ctx->size_p;
    if (beta > (uint32_t)kMaxDigits) return HE_E_UNSUPPORTED;
    EvkPtrs ptrs;
    memset(&ptrs, 0, sizeof(ptrs));
    for (uint32_t d = 0; d < beta; d++) {
        if (!evk[d]) return HE_E_INVALID_ARGUMENT;
        ptrs.p[d] = evk[d];
    }
    HE_HIP(launch_inner_product(ctx->tables(), y, ptrs, out, L, ctx->size_p, ctx->size_q, beta, galois_elt,
                                accumulate != 0, nullptr, nullptr, 1, 0, S(s)));
    return HE_OK;
}

}  // extern "C"

namespace {

// add_mask: which polynomials of `out` are added onto (bit p set) instead of overwritten
int moddown_impl(const he_context *ctx, uint32_t L, uint64_t *cx, uint64_t *out, uint32_t n_polys, uint32_t add_mask,
                 uint64_t *ws, he_stream s) {
    if (!ctx || !cx || !out || !ws || ctx->size_p == 0 || L == 0 || L > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    const int accumulate = add_mask != 0;
    const size_t n = ctx->n();
    const uint32_t K = ctx->size_p, LK = L + K;
    // special limbs -> coefficient form, scaled by (P / p_k)^-1, in place
    NttArgs inv = base_args(ctx, false);
    inv.in = cx + (size_t)L * n;
    inv.out = cx + (size_t)L * n;
    inv.in_poly_stride = inv.out_poly_stride = LK;
    inv.map = plain_map(K, ctx->size_q);
    inv.epi_mode = NTT_EPI_MUL;
    inv.w = ctx->d_phat_inv;
    const Level *lv = level_of(ctx, L);
    // the conversion tables describe up to 4 polynomials; more of them go as items of 2 (ciphertexts)
    const bool batched = lv && lv->batched && (n_polys <= 4 || n_polys % 2 == 0);
    const bool fused = batched && fuse_rows_ok(ctx, lv, L);
    // one special prime: (P / p)^-1 and the conversion matrix are ones, the conversion is the reduction of the special
    // limb's coefficients modulo each q_j, done where the forward transform reads its input
    const bool reduce_in_ntt = ctx->single_limb_digits && !fused;
    // ... and a small launch finishes the special limb's inverse transform there as well
    const int inv_backend = backend_for(ctx, inv.map);
    const bool source_intt = reduce_in_ntt && source_intt_ok(ctx, n_polys * L);
    HE_HIP(launch_ntt_inverse(inv, n_polys, inv_backend, S(s), false, source_intt));
    if (reduce_in_ntt) {
    } else if (batched) {
        const uint32_t units = n_polys <= 4 ? n_polys : 2, items = n_polys / units;
        if (fused) {
            BconvRows b{cx, ws, nullptr, ctx->d_phat_mod_q_fp, ctx->d_iota, ctx->d_iota, lv->d_moddown_descs, units, L, 0,
                        items, (size_t)units * LK * n, (size_t)units * L * n, 0, 0};
            HE_HIP(launch_bconv_rows(base_args(ctx, true), b, ctx->tune, S(s)));
        } else {
            BconvBatch b{cx, ws, nullptr, ctx->d_phat_mod_q, ctx->d_iota, ctx->d_iota, lv->d_moddown_descs, units, L, 0,
                         fp_for_level(ctx, L) ? ctx->d_phat_mod_q_fp : nullptr, ctx->d_fp_consts,
                         items, (size_t)units * LK * n, (size_t)units * L * n, 0};
            HE_HIP(launch_bconv_batched(ctx->tables(), b, ctx->tune, S(s)));
        }
    }
    for (uint32_t p = 0; p < n_polys && !batched && !reduce_in_ntt; p++) {
        BconvArgs b{cx + ((size_t)p * LK + L) * n, ws + (size_t)p * L * n, ctx->d_phat_mod_q, ctx->d_iota, ctx->d_iota, K, L};
        HE_HIP(launch_bconv(ctx->tables(), b, S(s)));
    }
    NttArgs fwd = base_args(ctx, true);
    fwd.in = ws;
    fwd.out = ws;
    fwd.in_poly_stride = fwd.out_poly_stride = L;
    fwd.map = plain_map(L, 0);
    fwd.epi_mode = accumulate ? NTT_EPI_SUB_MUL_ADD : NTT_EPI_SUB_MUL;
    fwd.epi_a = cx;
    fwd.epi_a_poly_stride = LK;
    fwd.epi_b = out;
    fwd.epi_b_poly_stride = L;
    fwd.epi_b_mask = add_mask;
    fwd.w = ctx->d_pinv_mod_q;
    fwd.epi_dst = out;
    fwd.epi_dst_poly_stride = L;
    if (reduce_in_ntt) {
        fwd.pro_mode = NTT_PRO_SOURCE_REDUCE;
        fwd.pro_src = cx + (size_t)L * n;
        fwd.pro_poly_stride = LK;
        if (source_intt) {
            set_source_intt(ctx, fwd, inv_backend);
            fwd.pro_src_table = ctx->size_q;
        }
    }
    HE_HIP(launch_ntt_forward(fwd, n_polys, backend_for(ctx, fwd.map), S(s), fused));
    return HE_OK;
}

}  // namespace

extern "C" {

int he_moddown(const he_context *ctx, uint32_t L, uint64_t *cx, uint64_t *out, uint32_t n_polys, int accumulate,
               uint64_t *ws, he_stream s) {
    return moddown_impl(ctx, L, cx, out, n_polys, accumulate ? 0xffffffffu : 0u, ws, s);
}

size_t he_keyswitch_workspace_words(const he_context *ctx, uint32_t L) {
    if (!ctx || ctx->size_p == 0 || L == 0 || L > ctx->size_q) return 0;
    const size_t n = ctx->n(), K = ctx->size_p, LK = L + K;
    const size_t beta = (L + K - 1) / K;
    // digits | inner product | ModDown scratch | last limb of both polynomials (he_keyswitch_rescale)
    return beta * LK * n + 2 * LK * n + 2 * (size_t)L * n + 2 * n;
}

size_t he_keyswitch_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items) {
    return (size_t)items * he_keyswitch_workspace_words(ctx, L);
}

}  // extern "C"

namespace {

// Workspace of a key switch over `items` inputs: y [items][beta][L+K][N] | cx [items][2][L+K][N] | tmp [items][2][L][N]
struct KsWorkspace {
    uint64_t *y, *cx, *tmp;
};

KsWorkspace ks_workspace(const he_context *ctx, const Level *lv, uint32_t L, uint32_t items, uint64_t *ws) {
    const size_t n = ctx->n(), LK = L + ctx->size_p;
    KsWorkspace w;
    w.y = ws;
    w.cx = w.y + (size_t)items * lv->beta * LK * n;
    w.tmp = w.cx + (size_t)items * 2 * LK * n;
    return w;
}

// ModUp and inner product of a key switch over `items` inputs (item k at c + k * c_item_stride * N): ws -> cx.
// fold_ct != nullptr: limb L-1 of cx becomes cx * P^-1 + fold_ct (see KsFuseArgs); fold_ct holds [items][2][L][N].
// add_c0 != nullptr (a rotation, items = 1): polynomial 0 of cx gains P sigma(add_c0) on its data limbs, sigma =
// X -> X^galois_elt, so that the ModDown of cx yields sigma(add_c0) + KeySwitch(sigma(c)) with no pass for sigma.
int ks_accumulate(const he_context *ctx, const Level *lv, uint32_t L, const uint64_t *c, uint32_t c_item_stride,
                  uint32_t items, const uint64_t *const *evk, uint32_t galois_elt, const uint64_t *fold_ct, uint64_t *ws,
                  he_stream s, const uint64_t *add_c0 = nullptr, const TensorFuse *tin = nullptr) {
    if (items == 0 || (items > 1 && (galois_elt || add_c0))) return HE_E_INVALID_ARGUMENT;
    const uint64_t *fold_w = fold_ct ? ctx->d_pinv_mod_q + 2 * (size_t)(L - 1) : nullptr;
    const size_t n = ctx->n();
    const KsWorkspace w = ks_workspace(ctx, lv, L, items, ws);
    uint64_t *y = w.y, *cx = w.cx, *tmp = w.tmp;
    const uint64_t *src = c;
    const bool fused_inner = ctx->fuse_inner && lv->batched && fp_for_level(ctx, L) &&
                             (items == 1 || (ctx->batch_fused_inner && !tin));
    // levels whose inner product reads a digit's own limbs from the input gather sigma(c) where they read c (the
    // inverse blocks pass and the inner product); the others stage it
    const bool gather = galois_elt && !fused_inner && lv->batched && items == 1;
    if (galois_elt && !fused_inner && !gather) {
        // sigma(c) is staged in the second half of the ModDown workspace, which ModUp leaves alone and ModDown
        // only touches after the inner product has read it
        uint64_t *staged = tmp + (size_t)L * n;
        if (int rc = he_galois_ntt(ctx, c, staged, L, galois_elt, s)) return rc;
        src = staged;
    }
    if (fused_inner) {
        // ModUp without the copy of a digit's own limbs, then the forward NTT fused with the inner product: the
        // transformed digits are never written (216 limb transfers less at L = 24, K = 8)
        // (a batch: the items are the polynomials of the inverse transform and the items of everything after it)
        NttArgs inv = base_args(ctx, false);
        inv.in = src;
        inv.out = tmp;
        inv.in_poly_stride = items == 1 ? L : c_item_stride;
        inv.out_poly_stride = L;
        inv.map = plain_map(L, 0);
        inv.epi_mode = NTT_EPI_MUL;
        inv.w = lv->d_part_hat_inv;
        inv.in_galois = galois_elt;
        // tin: c is the third polynomial of a tensor product that has not been formed yet; the blocks pass forms it
        if (tin) HE_HIP(launch_tensor_intt_blocks(inv, *tin, S(s)));
        HE_HIP(launch_ntt_inverse(inv, items, NTT_BACKEND_FP, S(s), tin != nullptr));
        NttArgs fwd = base_args(ctx, true);
        fwd.in = y;
        fwd.out = y;
        fwd.jobs = lv->d_modup_jobs;
        fwd.n_jobs = lv->n_modup_jobs;
        fwd.groups = lv->d_modup_groups;
        fwd.n_groups = lv->n_modup_groups;
        fwd.items = items;
        fwd.item_stride = (size_t)lv->beta * (L + ctx->size_p) * n;
        const bool rows_done = fuse_rows_ok(ctx, lv, L);
        if (rows_done) {
            BconvRows b{tmp, y, nullptr, lv->d_mats_fp, lv->d_modup_limb, lv->d_modup_table, lv->d_modup_descs,
                        lv->beta, lv->modup_max_rows, 0, items, (size_t)L * n, fwd.item_stride, 0, 0, lv->d_mx_up};
            HE_HIP(launch_bconv_rows(fwd, b, ctx->tune, S(s)));
        } else {
            BconvBatch b{tmp, y, src, lv->d_mats, lv->d_modup_limb, lv->d_modup_table, lv->d_modup_descs,
                         lv->beta, lv->modup_max_rows, 0, lv->d_mats_fp, ctx->d_fp_consts, items, (size_t)L * n,
                         fwd.item_stride, 0};
            HE_HIP(launch_bconv_batched(ctx->tables(), b, ctx->tune, S(s)));
        }
        KsFuseArgs x;
        memset(&x, 0, sizeof(x));
        for (uint32_t d = 0; d < lv->beta; d++) {
            if (!evk[d]) return HE_E_INVALID_ARGUMENT;
            x.evk.p[d] = evk[d];
        }
        x.own = src;
        x.own_galois = galois_elt;
        x.add_c0 = add_c0;
        x.p_mod_q = ctx->d_p_mod_q;
        x.out = cx;
        x.L = L;
        x.K = ctx->size_p;
        x.size_q = ctx->size_q;
        x.size_qp = ctx->size_qp;
        x.beta = lv->beta;
        x.fold_ct = fold_ct;
        x.fold_w = fold_w;
        x.items = items;
        x.own_item_stride = (size_t)c_item_stride * n;
        x.fold_item_stride = 2 * (size_t)L * n;
        HE_HIP(launch_ntt_forward_inner(fwd, x, S(s), rows_done));
    } else {
        // a batch on the FP64 back end shares each key word among the items of a group and reads a digit's own limbs
        // where they are
        // (its kernel moves two words per access: operands that are only 8-byte aligned take the integer kernel)
        auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
        bool fp_batch = items > 1 && lv->batched && fp_for_level(ctx, L) && n >= 512 && !galois_elt && !add_c0 &&
                        aligned16(src) && aligned16(cx) && aligned16(y) && aligned16(fold_ct);
        for (uint32_t d = 0; d < lv->beta && fp_batch; d++) fp_batch = aligned16(evk[d]);
        if (tin) return HE_E_INVALID_ARGUMENT;
        // (batched levels: neither kernel needs the copy of a digit's own limbs into y)
        const bool skip_own = fp_batch || lv->batched;
        const uint32_t src_stride = (galois_elt && !gather) ? L : c_item_stride;
        if (int rc = modup_impl(ctx, L, src, src_stride, items, y, tmp, s, skip_own, gather ? galois_elt : 0)) return rc;
        EvkPtrs ptrs;
        memset(&ptrs, 0, sizeof(ptrs));
        for (uint32_t d = 0; d < lv->beta; d++) {
            if (!evk[d]) return HE_E_INVALID_ARGUMENT;
            ptrs.p[d] = evk[d];
        }
        if (fp_batch) {
            HE_HIP(launch_inner_product_fp(ctx->tables(), ctx->d_fp_consts, y, src, (size_t)c_item_stride * n, ptrs, cx, L,
                                           ctx->size_p, ctx->size_q, lv->beta, fold_ct, fold_w, items, 2 * (size_t)L * n,
                                           S(s)));
            return HE_OK;
        }
        HE_HIP(launch_inner_product(ctx->tables(), y, ptrs, cx, L, ctx->size_p, ctx->size_q, lv->beta, 0, false,
                                    fold_ct, fold_w, items, 2 * (size_t)L * n, S(s), add_c0, galois_elt, ctx->d_p_mod_q,
                                    skip_own ? src : nullptr, (size_t)src_stride * n, gather ? galois_elt : 0));
    }
    return HE_OK;
}

}  // namespace

extern "C" {

int he_keyswitch(const he_context *ctx, uint32_t L, const uint64_t *c, const uint64_t *const *evk, uint64_t *ct,
                 uint32_t galois_elt, uint64_t *ws, he_stream s) {
    if (!ctx || !c || !evk || !ct || !ws || ctx->size_p == 0) return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    const KsWorkspace w = ks_workspace(ctx, lv, L, 1, ws);
    if (int rc = ks_accumulate(ctx, lv, L, c, L, 1, evk, galois_elt, nullptr, ws, s)) return rc;
    return he_moddown(ctx, L, w.cx, ct, 2, 1, w.tmp, s);
}

int he_rotate(const he_context *ctx, uint32_t L, const uint64_t *ct_in, const uint64_t *const *evk, uint64_t *ct_out,
              uint32_t galois_elt, uint64_t *ws, he_stream s) {
    if (!ctx || !ct_in || !evk || !ct_out || !ws || ctx->size_p == 0 || ct_in == ct_out) return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    const size_t n = ctx->n();
    const KsWorkspace w = ks_workspace(ctx, lv, L, 1, ws);
    if (!(galois_elt & 1) || galois_elt >= (2u << ctx->log_n)) return HE_E_INVALID_ARGUMENT;
    // the automorphism is never a pass of its own: sigma(c1) is gathered where the key switch reads its input,
    // sigma(c0) where the inner product adds P sigma(c0) to its first polynomial
    if (int rc = ks_accumulate(ctx, lv, L, ct_in + (size_t)L * n, L, 1, evk, galois_elt, nullptr, ws, s, ct_in)) return rc;
    // out0 = sigma(c0) + ks0 (the inner product carries P sigma(c0)), out1 = ks1
    return moddown_impl(ctx, L, w.cx, ct_out, 2, 0u, w.tmp, s);
}

int he_hoisted_rotations_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *ct_in,
                               const uint64_t *const *evk, const uint32_t *galois_elts, uint32_t n_steps, int add_input,
                               uint64_t *ct_out, uint64_t *ws, he_stream s) {
    if (!ctx || !ct_in || !evk || !galois_elts || !ct_out || !ws || ctx->size_p == 0 || n_steps == 0 || items == 0 ||
        items > 16384 || ct_in == ct_out)
        return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    if (lv->beta > (uint32_t)kMaxDigits) return HE_E_UNSUPPORTED;
    for (uint32_t i = 0; i < n_steps; i++) {
        if (!(galois_elts[i] & 1) || galois_elts[i] >= (2u << ctx->log_n)) return HE_E_INVALID_ARGUMENT;
        for (uint32_t d = 0; d < lv->beta; d++)
            if (!evk[(size_t)i * lv->beta + d]) return HE_E_INVALID_ARGUMENT;
    }
    const size_t n = ctx->n();
    const KsWorkspace w = ks_workspace(ctx, lv, L, items, ws);
    // (the digits' own limbs are not copied into y: the kernel reads them from c1 where they are)
    const bool skip_own = lv->batched;
    if (int rc = modup_impl(ctx, L, ct_in + (size_t)L * n, 2 * L, items, w.y, w.tmp, s, skip_own)) return rc;
    // as many steps per launch as the 128-bit accumulator and the pointer table allow
    const uint32_t per_launch = (uint32_t)kMaxDigits / lv->beta;
    for (uint32_t first = 0; first < n_steps; first += per_launch) {
        const uint32_t count = n_steps - first < per_launch ? n_steps - first : per_launch;
        HE_HIP(launch_hoist_inner(ctx->tables(), ctx->tune, w.y, ct_in, evk + (size_t)first * lv->beta, galois_elts + first, count,
                                  w.cx, ct_out, L, ctx->size_p, ctx->size_q, lv->beta, first != 0, add_input != 0, items,
                                  2 * (size_t)L * n, S(s), ctx->use_fp ? ctx->d_fp_consts : nullptr, ctx->fp_mask, skip_own));
    }
    // out0 = [c0 +] sum sigma(c0) + ModDown(cx0), out1 = [c1 +] ModDown(cx1)
    return moddown_impl(ctx, L, w.cx, ct_out, 2 * items, add_input ? 0xffffffffu : 0x55555555u, w.tmp, s);
}

int he_hoisted_rotations(const he_context *ctx, uint32_t L, const uint64_t *ct_in, const uint64_t *const *evk,
                         const uint32_t *galois_elts, uint32_t n_steps, uint64_t *ct_out, uint64_t *ws, he_stream s) {
    return he_hoisted_rotations_batch(ctx, L, 1, ct_in, evk, galois_elts, n_steps, 0, ct_out, ws, s);
}

}  // extern "C"

namespace {

// the fused tensor + key switch of he_multiply_relin_rescale applies: one input, FP64 back end, fused inner product
bool tensor_fusion_ok(const he_context *ctx, const Level *lv, uint32_t L) {
    return lv && ctx->fuse_tensor && ctx->fuse_inner && lv->batched && fp_for_level(ctx, L);
}

int ksr_impl(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *c, uint32_t c_item_stride,
             const uint64_t *const *evk, const uint64_t *ct, uint64_t *out, uint32_t galois_elt, uint64_t *ws, he_stream s,
             const TensorFuse *tin) {
    if (!ctx || !c || !evk || !ct || !out || !ws || ctx->size_p == 0 || L < 2 || items == 0 || items > 16384 ||
        c_item_stride < L)
        return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    if (items > 1 && !lv->batched) return HE_E_UNSUPPORTED;
    const size_t n = ctx->n();
    const uint32_t K = ctx->size_p, LK = L + K, polys = 2 * items;
    const KsWorkspace w = ks_workspace(ctx, lv, L, items, ws);
    uint64_t *cx = w.cx, *delta = w.tmp;           // [items][2][L+K][N], [items][2][L][N]
    // With c' = (cx - NTT(delta)) P^-1 + ct the ModDown result and t = INTT(cx_{L-1} P^-1 + ct_{L-1}), linearity of
    // the transform gives INTT(c'_{L-1}) = t - delta_{L-1} P^-1 and
    //   rescale(c')_j = ((cx_j P^-1 + ct_j) - NTT_j(delta_j P^-1 + [INTT(c'_{L-1})]_{q_j})) q_last^-1,
    // so ModDown and rescale share one inverse and one forward transform.  Every step is exact modular arithmetic:
    // the limbs equal he_keyswitch followed by he_rescale.
    // (1) inner product; limb L-1 of cx leaves as cx_{L-1} P^-1 + ct_{L-1}
    if (int rc = ks_accumulate(ctx, lv, L, c, c_item_stride, items, evk, galois_elt, ct, ws, s, nullptr, tin)) return rc;
    // (2) limb L-1 and the special limbs -> coefficient form, the latter scaled by (P / p_k)^-1
    NttArgs inv = base_args(ctx, false);
    inv.in = cx + (size_t)(L - 1) * n;
    inv.out = cx + (size_t)(L - 1) * n;
    inv.in_poly_stride = inv.out_poly_stride = LK;
    inv.map = LimbMap{K + 1, L - 1, 1, ctx->size_q};
    inv.epi_mode = NTT_EPI_MUL;
    inv.w = lv->d_mdr_w;
    HE_HIP(launch_ntt_inverse(inv, polys, backend_for(ctx, inv.map), S(s)));
    // (3) delta = P -> Ql conversion of the special limbs
    const bool fused = fuse_rows_ok(ctx, lv, L);
    // one special prime: the conversion is the reduction of its coefficients modulo every q_j, which the prologue of (4)
    // does where it reads them (no conversion kernel, no delta in memory before the transform)
    const bool k1 = ctx->single_limb_digits && !fused;
    if (k1) {
    } else if (fused) {
        // with the prologue of (4) and the rows pass of its transform
        BconvRows b{cx, delta, nullptr, ctx->d_phat_pinv_fp, ctx->d_iota, ctx->d_iota, lv->d_moddown_descs, 2, L, 0,
                    items, 2 * (size_t)LK * n, 2 * (size_t)L * n, 0, 1, ctx->d_mx_down,
                    ctx->d_mx_last ? ctx->d_mx_last + (size_t)(L - 1) * 4 * kMxRecord : nullptr};
        HE_HIP(launch_bconv_rows(base_args(ctx, true), b, ctx->tune, S(s)));
    } else if (lv->batched) {
        BconvBatch b{cx, delta, nullptr, ctx->d_phat_mod_q, ctx->d_iota, ctx->d_iota, lv->d_moddown_descs, 2, L, 0,
                     fp_for_level(ctx, L) ? ctx->d_phat_mod_q_fp : nullptr, ctx->d_fp_consts,
                     items, 2 * (size_t)LK * n, 2 * (size_t)L * n, 0};
        HE_HIP(launch_bconv_batched(ctx->tables(), b, ctx->tune, S(s)));
    } else {
        for (uint32_t p = 0; p < 2; p++) {
            BconvArgs b{cx + ((size_t)p * LK + L) * n, delta + (size_t)p * L * n, ctx->d_phat_mod_q, ctx->d_iota,
                        ctx->d_iota, K, L};
            HE_HIP(launch_bconv(ctx->tables(), b, S(s)));
        }
    }
    // (4) the merged forward transform over the limbs that stay
    NttArgs fwd = base_args(ctx, true);
    fwd.in = fwd.out = delta;
    fwd.in_poly_stride = fwd.out_poly_stride = L;
    fwd.map = plain_map(L - 1, 0);
    fwd.pro_mode = NTT_PRO_MODDOWN_RESCALE;
    fwd.pro_src = cx + (size_t)(L - 1) * n;
    fwd.pro_poly_stride = LK;
    fwd.pro_src2 = delta + (size_t)(L - 1) * n;
    fwd.pro2_poly_stride = L;
    fwd.pro_w = ctx->d_pinv_mod_q;
    fwd.pro_last = L - 1;
    if (k1) {
        fwd.pro_src2 = cx + (size_t)L * n;
        fwd.pro2_poly_stride = LK;
        fwd.pro_k1 = 1;
    }
    fwd.epi_mode = NTT_EPI_FMA_SUB_MUL;
    fwd.epi_a = cx;
    fwd.epi_a_poly_stride = LK;
    fwd.epi_b = ct;
    fwd.epi_b_poly_stride = L;
    fwd.w = lv->d_qlast_inv;
    fwd.epi_dst = out;
    fwd.epi_dst_poly_stride = L - 1;
    HE_HIP(launch_ntt_forward(fwd, polys, backend_for(ctx, fwd.map, (int)L - 1), S(s), fused));
    return HE_OK;
}

}  // namespace

extern "C" {

int he_keyswitch_rescale_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *c,
                               uint32_t c_item_stride, const uint64_t *const *evk, const uint64_t *ct, uint64_t *out,
                               uint32_t galois_elt, uint64_t *ws, he_stream s) {
    return ksr_impl(ctx, L, items, c, c_item_stride, evk, ct, out, galois_elt, ws, s, nullptr);
}

size_t he_multiply_relin_rescale_workspace_words(const he_context *ctx, uint32_t L) {
    const size_t ks = he_keyswitch_workspace_words(ctx, L);
    return ks ? ks + 3 * (size_t)L * ctx->n() : 0;
}

int he_multiply_relin_rescale(const he_context *ctx, uint32_t L, const uint64_t *ct1, const uint64_t *ct2,
                              const uint64_t *const *evk, uint64_t *out, uint64_t *ws, he_stream s) {
    if (!ctx || !ct1 || !ct2 || !evk || !out || !ws || ctx->size_p == 0 || L < 2 || L > ctx->size_q)
        return HE_E_INVALID_ARGUMENT;
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    const size_t n = ctx->n();
    uint64_t *d01 = ws + he_keyswitch_workspace_words(ctx, L), *d2 = d01 + 2 * (size_t)L * n;
    if (tensor_fusion_ok(ctx, lv, L)) {
        const TensorFuse tin{ct1, ct2, d01, d2, L, ct1 == ct2 ? 1 : 0};
        return ksr_impl(ctx, L, 1, d2, L, evk, d01, out, 0, ws, s, &tin);
    }
    // (d0, d1 | d2) are contiguous: the layout of he_tensor's output
    if (int rc = ct1 == ct2 ? he_tensor_square(ctx, ct1, d01, L, s) : he_tensor(ctx, ct1, ct2, d01, L, s)) return rc;
    return ksr_impl(ctx, L, 1, d2, L, evk, d01, out, 0, ws, s, nullptr);
}

size_t he_multiply_relin_rescale_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items) {
    const size_t ks = he_keyswitch_workspace_words(ctx, L);
    return ks ? (size_t)items * (ks + 3 * (size_t)L * ctx->n()) : 0;
}

int he_multiply_relin_rescale_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *ct1,
                                    const uint64_t *ct2, const uint64_t *const *evk, uint64_t *out, uint64_t *ws,
                                    he_stream s) {
    if (!ctx || !ct1 || !ct2 || !evk || !out || !ws || ctx->size_p == 0 || L < 2 || L > ctx->size_q || items == 0 ||
        items > 16384)
        return HE_E_INVALID_ARGUMENT;
    if (items == 1) return he_multiply_relin_rescale(ctx, L, ct1, ct2, evk, out, ws, s);
    const Level *lv = level_of(ctx, L);
    if (!lv) return HE_E_LEVEL_NOT_SET;
    if (!lv->batched) return HE_E_UNSUPPORTED;
    const size_t n = ctx->n();
    // [items] key-switch workspaces | (d0, d1) [items][2][L][N] | d2 [items][L][N]
    uint64_t *d01 = ws + (size_t)items * he_keyswitch_workspace_words(ctx, L), *d2 = d01 + (size_t)items * 2 * L * n;
    // (a tensor product formed inside the key switch's first pass, as the single call does it, measures slower here:
    // with many items in one launch the plain tensor kernel streams at a higher rate than the fused one computes)
    HE_HIP(launch_tensor(ctx->tables(), ct1, ct2, d01, L, ct1 == ct2, S(s),
                         fp_for(ctx, plain_map(L)) ? ctx->d_fp_consts : nullptr, items, d2));
    return ksr_impl(ctx, L, items, d2, L, evk, d01, out, 0, ws, s, nullptr);
}

int he_keyswitch_rescale(const he_context *ctx, uint32_t L, const uint64_t *c, const uint64_t *const *evk,
                         const uint64_t *ct, uint64_t *out, uint32_t galois_elt, uint64_t *ws, he_stream s) {
    return he_keyswitch_rescale_batch(ctx, L, 1, c, L, evk, ct, out, galois_elt, ws, s);
}

int he_decompose_real(const he_context *ctx, const double *coeffs, uint64_t *out, uint32_t limbs, uint32_t first,
                      he_stream s) {
    if (!ctx || !coeffs || !out || first + limbs > ctx->size_qp) return HE_E_INVALID_ARGUMENT;
    HE_HIP(launch_decompose_real(ctx->tables(), coeffs, out, limbs, first, 1, 0, S(s)));
    return HE_OK;
}

size_t he_ckks_workspace_words(const he_context *ctx, uint32_t limbs) {
    if (!ctx) return 0;
    const size_t n = ctx->n();
    // encode: [8 words, the first holds the maximum] [N words: complex scratch]
    // decode: [limbs * N words: coefficient-form copy]
    const size_t enc = 8 + n, dec = (size_t)limbs * n;
    return enc > dec ? enc : dec;
}

size_t he_ckks_encode_batch_workspace_words(const he_context *ctx, uint32_t items) {
    if (!ctx) return 0;
    // [items words rounded up to 8: the maxima] [items][N words: complex scratch]
    return (((size_t)items + 7) & ~(size_t)7) + (size_t)items * ctx->n();
}

int he_ckks_encode_batch(const he_context *ctx, const double *re, const double *im, uint32_t count, uint32_t slots,
                         double scale, uint32_t limbs, uint32_t items, size_t value_stride, uint64_t *out,
                         uint32_t out_poly_stride, uint64_t *ws, he_stream s) {
    if (!ctx || !re || !out || !ws || limbs == 0 || limbs > ctx->size_qp || items == 0 || items > 16384 ||
        out_poly_stride < limbs)
        return HE_E_INVALID_ARGUMENT;
    if (slots < 2 || (slots & (slots - 1)) || slots > ctx->n() / 2 || count > slots || !(scale > 0) ||
        (items > 1 && value_stride < count))
        return HE_E_INVALID_ARGUMENT;
    const size_t n = ctx->n();
    const size_t head = ((size_t)items + 7) & ~(size_t)7;
    double2 *v = reinterpret_cast<double2 *>(ws + head);
    const FftTables ft{ctx->d_rot_group, ctx->d_ksi, ctx->log_n};
    // (the complex scratch of an item is `slots` values = at most N words: the items are packed `slots` apart)
    // (the rounding kernel writes the residues itself: the coefficients never exist as an array of doubles)
    const Tables tab = ctx->tables();
    HE_HIP(launch_ckks_encode(ft, re, im, count, slots, scale, v, nullptr, ws, items, value_stride, S(s), &tab, out, limbs,
                              (size_t)out_poly_stride * n));
    return he_ntt_forward(ctx, out, items, out_poly_stride, limbs, 0, limbs, 0, s);
}

int he_ckks_encode(const he_context *ctx, const double *re, const double *im, uint32_t count, uint32_t slots,
                   double scale, uint32_t limbs, uint64_t *out, uint64_t *ws, he_stream s) {
    // one item: the maximum in ws[0], then the scratch (the layout of he_ckks_workspace_words)
    return he_ckks_encode_batch(ctx, re, im, count, slots, scale, limbs, 1, 0, out, limbs, ws, s);
}

size_t he_encrypt_batch_workspace_words(const he_context *ctx, uint32_t L, uint32_t items) {
    if (!ctx || L == 0 || L > ctx->size_q) return 0;
    const size_t n = ctx->n(), LK = L + ctx->size_p;
    // u [items][L+K][N] | wide [items][2][L+K][N] | ModDown scratch [items][2][L][N]
    return (size_t)items * (3 * LK + 2 * L) * n;
}

int he_encrypt_batch(const he_context *ctx, uint32_t L, uint32_t items, const uint64_t *pk, const uint32_t key[8],
                     uint64_t stream_id, uint64_t *cts, uint64_t *ws, he_stream s) {
    if (!ctx || !pk || !key || !cts || !ws || ctx->size_p == 0 || L == 0 || L > ctx->size_q || items == 0 || items > 8192)
        return HE_E_INVALID_ARGUMENT;
    const size_t n = ctx->n();
    const uint32_t K = ctx->size_p, Q = ctx->size_q, LK = L + K;
    uint64_t *u = ws, *wide = u + (size_t)items * LK * n, *tmp = wide + (size_t)items * 2 * LK * n;
    ChaChaKey k;
    memcpy(k.k, key, sizeof(k.k));
    const LimbMap map{LK, 0, L, Q};
    // item k draws u, e0, e1 from the stream ids stream_id + 3 k, + 1, + 2: what `items` encryptions in a row draw
    // (one launch: u and wide lie one after the other, 3 * items polynomials LK * N words apart)
    HE_HIP(launch_sample_encrypt(ctx->tables(), k, stream_id, u, map, items, (size_t)LK * n, S(s)));
    // u and wide lie one after the other: 3 * items polynomials of the same limbs
    if (int rc = he_ntt_forward(ctx, u, 3 * items, LK, LK, 0, L, Q, s)) return rc;
    HE_HIP(launch_encrypt_fma(ctx->tables(), u, pk, wide, L, K, Q, items, S(s)));
    // divide by P; polynomial 0 of every ciphertext already holds the plaintext and is added onto
    return moddown_impl(ctx, L, wide, cts, 2 * items, 0x55555555u, tmp, s);
}

int he_ckks_decode(const he_context *ctx, const uint64_t *plain, uint32_t limbs, uint32_t slots, double scale,
                   double *out, uint64_t *ws, he_stream s) {
    if (!ctx || !plain || !out || !ws || limbs == 0 || limbs > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    if (slots < 2 || (slots & (slots - 1)) || slots > ctx->n() / 2 || !(scale > 0)) return HE_E_INVALID_ARGUMENT;
    const size_t n = ctx->n();
    HE_HIP(hipMemcpyAsync(ws, plain, (size_t)limbs * n * sizeof(uint64_t), hipMemcpyDeviceToDevice, S(s)));
    if (int rc = he_ntt_inverse(ctx, ws, 1, limbs, limbs, 0, limbs, 0, s)) return rc;
    const FftTables ft{ctx->d_rot_group, ctx->d_ksi, ctx->log_n};
    HE_HIP(launch_ckks_decode(ft, ctx->tables(), ws, limbs, slots, scale, ctx->d_garner_inv, ctx->size_q,
                              reinterpret_cast<double2 *>(out), 1, S(s)));
    return HE_OK;
}

size_t he_decrypt_decode_batch_workspace_words(const he_context *ctx, uint32_t limbs, uint32_t slots, uint32_t items) {
    if (!ctx) return 0;
    // [items][limbs][N] plaintexts | [items][slots] complex values
    return (size_t)items * limbs * ctx->n() + 2 * (size_t)items * slots;
}

int he_decrypt_decode_batch(const he_context *ctx, const uint64_t *const *d_cts, uint32_t items, uint32_t limbs,
                            const uint64_t *sk, const uint64_t *noise, uint32_t slots, double scale, uint32_t count,
                            double *out, uint64_t *ws, he_stream s) {
    if (!ctx || !d_cts || !sk || !out || !ws || items == 0 || items > 16384 || limbs == 0 || limbs > ctx->size_q)
        return HE_E_INVALID_ARGUMENT;
    if (slots < 2 || (slots & (slots - 1)) || slots > ctx->n() / 2 || !(scale > 0) || count == 0 || count > slots)
        return HE_E_INVALID_ARGUMENT;
    const size_t n = ctx->n();
    uint64_t *plain = ws;
    double2 *v = reinterpret_cast<double2 *>(ws + (size_t)items * limbs * n);
    HE_HIP(launch_decrypt_gather(ctx->tables(), d_cts, sk, noise, plain, limbs, items, S(s)));
    if (int rc = he_ntt_inverse(ctx, plain, items, limbs, limbs, 0, limbs, 0, s)) return rc;
    const FftTables ft{ctx->d_rot_group, ctx->d_ksi, ctx->log_n};
    HE_HIP(launch_ckks_decode(ft, ctx->tables(), plain, limbs, slots, scale, ctx->d_garner_inv, ctx->size_q, v, items, S(s)));
    HE_HIP(launch_take_slots(v, slots, items, count, reinterpret_cast<double2 *>(out), S(s)));
    return HE_OK;
}

static int sample_impl(const he_context *ctx, int kind, const uint32_t key[8], uint64_t stream_id, uint64_t *out,
                       uint32_t limbs, uint32_t first, uint32_t split, uint32_t tail, const uint64_t *cdt,
                       uint32_t cdt_len, uint32_t items, he_stream s) {
    if (!ctx || !key || !out || kind < 0 || kind > 3 || (kind == SAMPLE_GAUSS && (!cdt || !cdt_len)) || items == 0 ||
        items > 16384 || (reinterpret_cast<uintptr_t>(out) & 15))
        return HE_E_INVALID_ARGUMENT;
    if (int rc = check_map(ctx, limbs, first, split, tail)) return rc;
    ChaChaKey k;
    memcpy(k.k, key, sizeof(k.k));
    HE_HIP(launch_sample(ctx->tables(), kind, k, stream_id, out, LimbMap{limbs, first, split, tail}, cdt, cdt_len, items,
                         1, (size_t)limbs * ctx->n(), S(s)));
    return HE_OK;
}

int he_sample(const he_context *ctx, int kind, const uint32_t key[8], uint64_t stream_id, uint64_t *out,
              uint32_t limbs, uint32_t first, uint32_t split, uint32_t tail, const uint64_t *cdt, uint32_t cdt_len,
              he_stream s) {
    return sample_impl(ctx, kind, key, stream_id, out, limbs, first, split, tail, cdt, cdt_len, 1, s);
}

int he_sample_batch(const he_context *ctx, int kind, const uint32_t key[8], uint64_t stream_id, uint64_t *out,
                    uint32_t limbs, uint32_t first, uint32_t split, uint32_t tail, const uint64_t *cdt, uint32_t cdt_len,
                    uint32_t items, he_stream s) {
    return sample_impl(ctx, kind, key, stream_id, out, limbs, first, split, tail, cdt, cdt_len, items, s);
}

}  // extern "C"
