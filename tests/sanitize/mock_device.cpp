// Host-memory stand-in for the eleven C-ABI entry points that the host layer's table construction and record
// parsing call (he_malloc .. he_context_destroy), so that those CPU code paths can run under AddressSanitizer and
// UndefinedBehaviorSanitizer without a GPU.  Test infrastructure: "device" memory is malloc'ed host memory, copies
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

}  // extern "C"
