// Host-memory stand-in for the C-ABI entry points that the host layer's table construction, record parsing and
// containers call (he_malloc .. he_context_destroy, and he_keyswitch for a deferred relinearisation), so that those
// CPU code paths can run under AddressSanitizer and UndefinedBehaviorSanitizer without a GPU.  Test infrastructure: "device" memory is malloc'ed host memory, copies
// are memcpy, a context is an opaque token.  Nothing here computes.
#include <cstdlib>
#include <cstring>

#include "cahel_hip.h"

struct he_context {
    uint32_t log_n, size_q, size_p;
};

extern "C" {

const char *he_error_string(int status) { return status == 0 ? "success" : "mock device error"; }

int he_malloc(void **dev_ptr, size_t bytes) {
    if (!dev_ptr) return HE_E_INVALID_ARGUMENT;
    *dev_ptr = bytes ? std::malloc(bytes) : nullptr;
    return (bytes && !*dev_ptr) ? HE_E_OUT_OF_MEMORY : HE_OK;
}

int he_free(void *dev_ptr) {
    std::free(dev_ptr);
    return HE_OK;
}

int he_memcpy_h2d(void *dst, const void *src, size_t bytes, he_stream) {
    if (bytes) std::memcpy(dst, src, bytes);
    return HE_OK;
}

int he_memcpy_d2h(void *dst, const void *src, size_t bytes, he_stream) {
    if (bytes) std::memcpy(dst, src, bytes);
    return HE_OK;
}

int he_memcpy_d2d(void *dst, const void *src, size_t bytes, he_stream) {
    if (bytes) std::memmove(dst, src, bytes);
    return HE_OK;
}

int he_stream_create(he_stream *stream) {
    if (!stream) return HE_E_INVALID_ARGUMENT;
    *stream = nullptr;
    return HE_OK;
}

int he_stream_synchronize(he_stream) { return HE_OK; }

int he_context_create(const he_context_desc *d, he_context **out) {
    if (!d || !out || !d->moduli || !d->barrett || !d->psi || !d->ipsi_div2) return HE_E_INVALID_ARGUMENT;
    if (d->log_n < 9 || d->log_n > 16) return HE_E_UNSUPPORTED;
    // touch every table the real library would upload, so that a short array shows up as a sanitizer report
    const size_t n = (size_t)1 << d->log_n, qp = (size_t)d->size_q + d->size_p;
    volatile uint64_t sink = 0;
    for (size_t i = 0; i < qp; i++) sink += d->moduli[i] + d->barrett[2 * i + 1];
    sink += d->psi[2 * qp * n - 1] + d->ipsi_div2[2 * qp * n - 1];
    if (d->size_p)
        sink += d->p_mod_q[2 * d->size_q - 1] + d->pinv_mod_q[2 * d->size_q - 1] + d->phat_inv_mod_p[2 * d->size_p - 1] +
                d->phat_mod_q[(size_t)d->size_q * d->size_p - 1];
    (void)sink;
    *out = new he_context{d->log_n, d->size_q, d->size_p};
    return HE_OK;
}

int he_context_set_level(he_context *ctx, const he_level_desc *d) {
    if (!ctx || !d || d->L == 0 || d->L > ctx->size_q) return HE_E_INVALID_ARGUMENT;
    volatile uint64_t sink = 0;
    if (d->L > 1) sink += d->qlast_inv[2 * (d->L - 1) - 1];
    if (ctx->size_p) {
        sink += d->part_hat_inv[2 * d->L - 1];
        const uint32_t K = ctx->size_p, beta = d->beta;
        for (uint32_t g = 0; g < beta; g++) {
            const uint32_t start = g * K, size = start + K <= d->L ? K : d->L - start, n_out = d->L + K - size;
            sink += d->digit_mats[d->digit_mat_off[g] + (size_t)n_out * size - 1];
        }
    }
    (void)sink;
    return HE_OK;
}

int he_context_destroy(he_context *ctx) {
    delete ctx;
    return HE_OK;
}

size_t he_keyswitch_workspace_words(const he_context *ctx, uint32_t L) { return ctx ? (size_t)L << ctx->log_n : 0; }

// Touches what the real call reads and writes (every word of c, of the beta key digits and of ct, and the
// workspace), so that a stale pointer shows up as a sanitizer report; marks ct so that the caller can tell it ran.
int he_keyswitch(const he_context *ctx, uint32_t L, const uint64_t *c, const uint64_t *const *evk, uint64_t *ct,
                 uint32_t, uint64_t *workspace, he_stream) {
    if (!ctx || !c || !evk || !ct || !workspace || L == 0 || L > ctx->size_q || ctx->size_p == 0) return HE_E_INVALID_ARGUMENT;
    const size_t n = (size_t)1 << ctx->log_n, qp = (size_t)ctx->size_q + ctx->size_p;
    const uint32_t beta = (L + ctx->size_p - 1) / ctx->size_p;
    uint64_t sum = 0;
    for (size_t i = 0; i < (size_t)L * n; i++) sum += c[i];
    for (uint32_t d = 0; d < beta; d++)
        for (size_t i = 0; i < 2 * qp * n; i += 97) sum += evk[d][i];
    for (size_t i = 0; i < (size_t)L * n; i++) workspace[i] = sum;
    for (size_t i = 0; i < 2 * (size_t)L * n; i++) ct[i] += 1;
    return HE_OK;
}

}  // extern "C"
