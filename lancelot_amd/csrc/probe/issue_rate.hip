// Issue-rate probe for the VALU roofline: the FP64 back end spends its time in v_fma_f64 / v_mul_f64 / v_add_f64 /
// v_rndne_f64, all of which issue at the rate this kernel measures (8 independent fused multiply-add chains per
// lane, enough waves to fill every SIMD).  bench.py prices the instruction counts of the step's kernels against it.
// Built as a library of its own (libcahel_probe.so, include/cahel_probe.h): measurement support, not part of the
// engine's C-ABI.
#include <hip/hip_runtime.h>

#include "../../../include/cahel_probe.h"

namespace {

__global__ __launch_bounds__(256) void fp64_issue_probe_kernel(double *sink, double a, double b, uint32_t iters) {
    double v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = a + threadIdx.x + i;
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++)
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = __builtin_fma(v[i], a, b);
    }
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < 8; i++) s += v[i];
    if (s == 12345.678) sink[0] = s;   // never true: keeps the chains alive
}

// The other instruction kinds that the kernels' bounds are argued with: 32-bit integer multiplies (the integer back
// end's Shoup and Barrett arithmetic, the lazy sums of the hoisting kernel), a plain 32-bit addition for scale, and the
// FP64 matrix instruction alone and interleaved with vector multiply-adds (do the two pipes run side by side?).
typedef double probe_d4 __attribute__((ext_vector_type(4)));

template <int KIND>
__global__ __launch_bounds__(256) void issue_probe_kernel(uint64_t *sink, uint32_t a, uint32_t b, uint32_t iters) {
    uint64_t acc[8];
    uint32_t u[8];
    double f[8];
    probe_d4 m[4];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc[i] = threadIdx.x + i;
        u[i] = threadIdx.x + i;
        f[i] = threadIdx.x + i;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) m[i] = probe_d4{0.0, 0.0, 0.0, 0.0};
    const double fa = 1.0000001 + a * 1e-12, fb = b * 1e-9;
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++) {
            if (KIND == HE_PROBE_MFMA_F64 || KIND == HE_PROBE_MFMA_F64_WITH_FMA) {
                // 1 matrix instruction = 16 x 16 x 4 = 1,024 multiply-adds = 16 vector instructions of 64 lanes
                if ((r & 1) == 0) m[(r >> 1) & 3] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa, fb, m[(r >> 1) & 3], 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (KIND == HE_PROBE_MAD_U64_U32) {
                    uint64_t carry;
                    asm volatile("v_mad_u64_u32 %0, %1, %2, %3, %0" : "+v"(acc[i]), "=&s"(carry) : "v"(a), "v"(b));
                }
                if (KIND == HE_PROBE_MUL_LO_U32) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(u[i]) : "v"(a));
                if (KIND == HE_PROBE_ADD_U32) asm volatile("v_add_u32 %0, %0, %1" : "+v"(u[i]) : "v"(a));
                if (KIND == HE_PROBE_FMA_F64 || KIND == HE_PROBE_MFMA_F64_WITH_FMA) f[i] = __builtin_fma(f[i], fa, fb);
            }
        }
    }
    uint64_t s = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) s += acc[i] + u[i] + (uint64_t)f[i];
#pragma unroll
    for (int i = 0; i < 4; i++) s += (uint64_t)(m[i].x + m[i].y + m[i].z + m[i].w);
    if (s == 0x123456789abcdefull) sink[0] = s;   // never true: keeps the chains alive
}

template <int KIND>
void launch_issue_probe(uint32_t blocks, uint64_t *sink, uint32_t iters, hipStream_t s) {
    hipLaunchKernelGGL(issue_probe_kernel<KIND>, dim3(blocks), dim3(256), 0, s, sink, 3u, 5u, iters);
}

void launch_issue_probe_kind(uint32_t kind, uint32_t blocks, uint64_t *sink, uint32_t iters, hipStream_t s) {
    switch (kind) {
        case HE_PROBE_FMA_F64: launch_issue_probe<HE_PROBE_FMA_F64>(blocks, sink, iters, s); break;
        case HE_PROBE_MAD_U64_U32: launch_issue_probe<HE_PROBE_MAD_U64_U32>(blocks, sink, iters, s); break;
        case HE_PROBE_MUL_LO_U32: launch_issue_probe<HE_PROBE_MUL_LO_U32>(blocks, sink, iters, s); break;
        case HE_PROBE_ADD_U32: launch_issue_probe<HE_PROBE_ADD_U32>(blocks, sink, iters, s); break;
        case HE_PROBE_MFMA_F64: launch_issue_probe<HE_PROBE_MFMA_F64>(blocks, sink, iters, s); break;
        default: launch_issue_probe<HE_PROBE_MFMA_F64_WITH_FMA>(blocks, sink, iters, s); break;
    }
}

}  // namespace

extern "C" int he_probe_issue_rate(uint32_t kind, uint32_t blocks, uint32_t iters, double *lane_ops_per_second, void *stream) {
    if (!lane_ops_per_second || blocks == 0 || iters == 0 || blocks > 65535 || kind > HE_PROBE_MFMA_F64_WITH_FMA)
        return HE_E_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    uint64_t *sink = nullptr;
    hipError_t e = hipMalloc(&sink, 64);
    if (e != hipSuccess) return (int)e;
    e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        launch_issue_probe_kind(kind, blocks, sink, 16u, s);   // warm-up
        e = hipEventRecord(e0, s);
    }
    if (e == hipSuccess) {
        launch_issue_probe_kind(kind, blocks, sink, iters, s);
        e = hipEventRecord(e1, s);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (e != hipSuccess) return (int)e;
    // per lane and iteration: 64 vector operations; the matrix kinds add 4 instructions of 1,024 multiply-adds per wave,
    // i.e. 64 per lane (alone: those only)
    const double per_lane = kind == HE_PROBE_MFMA_F64 ? 64.0 : kind == HE_PROBE_MFMA_F64_WITH_FMA ? 128.0 : 64.0;
    *lane_ops_per_second = (double)blocks * 256.0 * iters * per_lane / ((double)ms * 1e-3);
    return HE_OK;
}

extern "C" int he_probe_fp64_issue_rate(uint32_t blocks, uint32_t iters, double *lane_ops_per_second, void *stream) {
    if (!lane_ops_per_second || blocks == 0 || iters == 0 || blocks > 65535) return HE_E_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    double *sink = nullptr;
    hipError_t e = hipMalloc(&sink, 64);
    if (e != hipSuccess) return (int)e;
    e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(fp64_issue_probe_kernel, dim3(blocks), dim3(256), 0, s, sink, 1.0000001, 1e-9, 16u);  // warm-up
        e = hipEventRecord(e0, s);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(fp64_issue_probe_kernel, dim3(blocks), dim3(256), 0, s, sink, 1.0000001, 1e-9, iters);
        e = hipEventRecord(e1, s);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (e != hipSuccess) return (int)e;
    *lane_ops_per_second = (double)blocks * 256.0 * iters * 64.0 / ((double)ms * 1e-3);
    return HE_OK;
}
