// Issue-rate probe for the VALU roofline: the FP64 back end spends its time in v_fma_f64 / v_mul_f64 / v_add_f64 /
// v_rndne_f64, all of which issue at the rate this kernel measures (8 independent fused multiply-add chains per
// lane, enough waves to fill every SIMD).  bench.py prices the instruction counts of the step's kernels against it.
#include <hip/hip_runtime.h>

#include "../../include/cahel_hip.h"

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

}  // namespace

extern "C" int he_probe_fp64_issue_rate(uint32_t blocks, uint32_t iters, double *lane_ops_per_second, he_stream stream) {
    if (!lane_ops_per_second || blocks == 0 || iters == 0 || blocks > 65535) return HE_E_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0, e1;
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
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (e != hipSuccess) return (int)e;
    *lane_ops_per_second = (double)blocks * 256.0 * iters * 64.0 / ((double)ms * 1e-3);
    return HE_OK;
}
