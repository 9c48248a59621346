// Batched negacyclic NTT / inverse NTT over RNS limbs for gfx950.
//
// Mathematics (what the CPU checker and the reference compute; cahel-main/src/ntt/fntt_2d.cu:8-246,
// src/ntt/intt_2d.cu:8-198, src/ntt/butterfly.cuh): forward = log2(N) Cooley-Tukey stages m = 1, 2, ..., N/2
// with twiddle psi^bitrev(m+k) for group k, output in bit-reversed order, canonical residues; inverse =
// the Gentleman-Sande stages in the opposite order including the factor 1/N.
//
// Decomposition for the GPU: N = R x 256.  A limb is an R x 256 row-major matrix.
//   rows pass   : the first log2(R) stages pair elements that are whole rows apart.  A workgroup owns a
//                 tile of R rows x C columns (4096 elements, 32 KiB) in LDS; global accesses run along the
//                 columns (C consecutive words per row).
//   blocks pass : the last 8 stages stay inside one row (256 consecutive words).  A workgroup owns 16
//                 rows (4096 consecutive words).
// Inside a pass each thread takes 2^r elements from LDS into registers, runs r stages on them (r <= 4,
// radix-16) and writes them back; 8 stages cost two LDS round trips.  LDS indices are skewed by one word
// per 16 so that both the stride-16 and the stride-256 gathers of a wave hit distinct banks.
// The forward transform runs rows pass then blocks pass, the inverse the other way round.
//
// Two arithmetic back ends share this skeleton:
//   integer : 64-bit Shoup/Harvey butterflies, any prime below 2^61 (~35 VALU instructions per butterfly);
//             inverse twiddles are pre-halved so that 1/N comes for free
//   FP64    : exact integer arithmetic in doubles for primes below 2^50 (8 full-rate operations per
//             butterfly, see modarith.cuh); values between the two passes are lazy signed doubles stored
//             in the same 8-byte words; the factor 1/N is folded into the last multiplication
// A launch uses the FP64 back end when every limb it touches has a prime below 2^50.
#include "kernels.h"
#include "modarith.cuh"

namespace he {

namespace {

constexpr int kThreads = 256;
constexpr int kTileLog = 12;
constexpr uint32_t kTile = 1u << kTileLog;
constexpr uint32_t kLdsWords = kTile + (kTile >> 4);

__device__ __forceinline__ uint32_t skew(uint32_t e) { return e + (e >> 4); }

// Workgroups are dealt round-robin to the 8 XCDs; give every XCD a contiguous range of logical ids so
// that the tiles of one limb (which share a twiddle table) meet in one L2.
__device__ __forceinline__ uint32_t logical_block() {
    uint32_t b = blockIdx.x, n = gridDim.x;
    if (n % 8 == 0) return (b % 8) * (n / 8) + b / 8;
    return b;
}

struct Job {
    const uint64_t *in;
    uint64_t *out;
    uint32_t table;
    uint32_t poly;
    uint32_t limb;
};

__device__ __forceinline__ Job decode_job(const NttArgs &a, uint32_t job) {
    Job j;
    const size_t n = (size_t)1 << a.log_n;
    if (a.jobs) {
        LimbJob lj = a.jobs[job];
        j.in = a.in + (size_t)lj.data_limb * n;
        j.out = a.out + (size_t)lj.data_limb * n;
        j.table = lj.table;
        j.poly = 0;
        j.limb = 0;
    } else {
        j.poly = job / a.map.limbs;
        j.limb = job % a.map.limbs;
        j.in = a.in ? a.in + ((size_t)j.poly * a.in_poly_stride + j.limb) * n : nullptr;
        j.out = a.out + ((size_t)j.poly * a.out_poly_stride + j.limb) * n;
        j.table = map_table(a.map, j.limb);
    }
    return j;
}

// Per-limb constants of one back end.
struct IntCtx {
    uint64_t q;
    const uint64_t *tw;
};

struct FpCtx {
    FpMod m;
    const double *tw;
};

__device__ __forceinline__ IntCtx int_ctx(const NttArgs &a, uint32_t table) {
    return IntCtx{a.moduli[table], a.tw + ((size_t)table << (a.log_n + 1))};
}

__device__ __forceinline__ FpCtx fp_ctx(const NttArgs &a, uint32_t table) {
    const double *c = a.fp_consts + 4 * (size_t)table;
    return FpCtx{FpMod{c[0], c[1]}, a.tw_fp + ((size_t)table << a.log_n)};
}

// r stages on a tile held in LDS.  Tile index bits: [upper][mid: r bits][lower: low_bits]; the 2^r
// elements of a group differ in `mid`.  idx_base + upper is the twiddle index of the group's first stage.
template <int LOGR, bool FWD>
__device__ __forceinline__ void tile_pass(uint64_t *lds, uint32_t tile_elems, uint32_t low_bits, uint32_t idx_base,
                                          IntCtx c) {
    constexpr int R = 1 << LOGR;
    const uint32_t groups = tile_elems >> LOGR;
    const uint32_t low_mask = (1u << low_bits) - 1;
    for (uint32_t g = threadIdx.x; g < groups; g += kThreads) {
        const uint32_t upper = g >> low_bits;
        const uint32_t base = (upper << (low_bits + LOGR)) | (g & low_mask);
        uint64_t v[R];
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lds[skew(base + ((uint32_t)j << low_bits))];
        if (FWD)
            ct_block<LOGR>(v, c.tw, idx_base + upper, c.q);
        else
            gs_block<LOGR>(v, c.tw, idx_base + upper, c.q);
#pragma unroll
        for (int j = 0; j < R; j++) lds[skew(base + ((uint32_t)j << low_bits))] = v[j];
    }
}

template <int LOGR, bool FWD, bool REDUCE_FIRST>
__device__ __forceinline__ void tile_pass_fp(uint64_t *lds, uint32_t tile_elems, uint32_t low_bits, uint32_t idx_base,
                                             FpCtx c) {
    constexpr int R = 1 << LOGR;
    double *ld = reinterpret_cast<double *>(lds);
    const uint32_t groups = tile_elems >> LOGR;
    const uint32_t low_mask = (1u << low_bits) - 1;
    for (uint32_t g = threadIdx.x; g < groups; g += kThreads) {
        const uint32_t upper = g >> low_bits;
        const uint32_t base = (upper << (low_bits + LOGR)) | (g & low_mask);
        double v[R];
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = ld[skew(base + ((uint32_t)j << low_bits))];
        if (FWD)
            fp_ct_block<LOGR, REDUCE_FIRST>(v, c.tw, idx_base + upper, c.m);
        else
            fp_gs_block<LOGR, REDUCE_FIRST>(v, c.tw, idx_base + upper, c.m);
#pragma unroll
        for (int j = 0; j < R; j++) ld[skew(base + ((uint32_t)j << low_bits))] = v[j];
    }
}

template <int LD>
struct Split {
    static constexpr int p0 = LD >= 7 ? 4 : (LD >= 5 ? 3 : LD);
    static constexpr int p1 = LD - p0;
};

template <int LD>
__device__ __forceinline__ constexpr int log_cols() {
    return (kTileLog - LD) < 8 ? (kTileLog - LD) : 8;
}

// (N^-1 [* w]) as an FP twiddle for the last multiplication of the inverse transform
__device__ __forceinline__ FpTw inverse_scale(const NttArgs &a, const Job &job, FpMod m) {
    const double *c = a.fp_consts + 4 * (size_t)job.table;
    FpTw ninv{c[2], c[3]};
    if (a.epi_mode != NTT_EPI_MUL) return ninv;
    const double w = fp_canonical(fp_mulmod(fp_from_u64(a.w[2 * job.limb]), ninv, m), m);
    return FpTw{w, w * m.qinv};
}

// ---------------------------------------------------------------------------------------------------
// rows pass: stages 0 .. LD-1 (forward) over an R = 2^LD rows x 256 matrix
// ---------------------------------------------------------------------------------------------------
template <int LD, bool FWD, bool FP>
__global__ __launch_bounds__(kThreads) void ntt_rows_kernel(NttArgs a) {
    __shared__ uint64_t lds[kLdsWords];
    constexpr int LOGC = log_cols<LD>();
    constexpr uint32_t C = 1u << LOGC;
    constexpr uint32_t tile_elems = 1u << (LD + LOGC);
    constexpr uint32_t tiles_per_limb = 256u >> LOGC;
    constexpr int p0 = Split<LD>::p0, p1 = Split<LD>::p1;

    const uint32_t lb = logical_block();
    const Job job = decode_job(a, lb / tiles_per_limb);
    const uint32_t col0 = (lb % tiles_per_limb) << LOGC;
    double *ld = reinterpret_cast<double *>(lds);

    if (FP) {
        const FpCtx c = fp_ctx(a, job.table);
        if (FWD) {
            // input: canonical residues (or one broadcast source limb); output: lazy signed doubles
            const uint64_t *src =
                a.pro_mode == NTT_PRO_BROADCAST_REDUCE ? a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n) : job.in;
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                ld[skew(e)] = fp_from_u64(src[(size_t)row * 256 + col0 + col]);
            }
            __syncthreads();
            // a broadcast source may exceed this limb's prime: reduce first in that case
            if (a.pro_mode == NTT_PRO_BROADCAST_REDUCE)
                tile_pass_fp<p0, true, true>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
            else
                tile_pass_fp<p0, true, false>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
            __syncthreads();
            if (p1 > 0) {
                tile_pass_fp<(p1 > 0 ? p1 : 1), true, true>(lds, tile_elems, LOGC, 1u << p0, c);
                __syncthreads();
            }
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = lds[skew(e)];
            }
        } else {
            // input: lazy signed doubles from the blocks pass; output: canonical residues
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                lds[skew(e)] = job.in[(size_t)row * 256 + col0 + col];
            }
            __syncthreads();
            if (p1 > 0) {
                tile_pass_fp<(p1 > 0 ? p1 : 1), false, true>(lds, tile_elems, LOGC, 1u << p0, c);
                __syncthreads();
            }
            tile_pass_fp<p0, false, true>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
            __syncthreads();
            const FpTw scale = inverse_scale(a, job, c.m);
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = fp_to_u64(fp_canonical(fp_mulmod(ld[skew(e)], scale, c.m), c.m));
            }
        }
        return;
    }

    const IntCtx c = int_ctx(a, job.table);
    const uint64_t q = c.q;
    if (FWD && a.pro_mode == NTT_PRO_BROADCAST_REDUCE) {
        const uint64_t r1 = a.barrett[2 * job.table + 1];
        const uint64_t *src = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
            uint32_t row = e >> LOGC, col = e & (C - 1);
            lds[skew(e)] = barrett64(src[(size_t)row * 256 + col0 + col], q, r1);
        }
    } else {
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
            uint32_t row = e >> LOGC, col = e & (C - 1);
            lds[skew(e)] = job.in[(size_t)row * 256 + col0 + col];
        }
    }
    __syncthreads();

    if (FWD) {
        tile_pass<p0, true>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
        __syncthreads();
        if (p1 > 0) {
            tile_pass<(p1 > 0 ? p1 : 1), true>(lds, tile_elems, LOGC, 1u << p0, c);
            __syncthreads();
        }
        // lazy values in [0, 4q) go to the blocks pass
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
            uint32_t row = e >> LOGC, col = e & (C - 1);
            job.out[(size_t)row * 256 + col0 + col] = lds[skew(e)];
        }
    } else {
        if (p1 > 0) {
            tile_pass<(p1 > 0 ? p1 : 1), false>(lds, tile_elems, LOGC, 1u << p0, c);
            __syncthreads();
        }
        tile_pass<p0, false>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
        __syncthreads();
        if (a.epi_mode == NTT_EPI_MUL) {
            const Shoup w = load_shoup(a.w, job.limb);
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = mul_shoup(lds[skew(e)], w, q);
            }
        } else {
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = reduce_2q(lds[skew(e)], q);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// blocks pass: the 8 stages that stay inside 256 consecutive words
// ---------------------------------------------------------------------------------------------------
template <bool FWD, bool FP>
__global__ __launch_bounds__(kThreads) void ntt_blocks_kernel(NttArgs a) {
    __shared__ uint64_t lds[kLdsWords];
    const uint32_t lr = a.log_n - 8;                       // log2(number of 256-blocks per limb)
    const uint32_t log_b = lr < 4 ? lr : 4;                // blocks per tile = 2^log_b
    const uint32_t tile_elems = 256u << log_b;
    const uint32_t tiles_per_limb = 1u << (lr - log_b);

    const uint32_t lb = logical_block();
    const Job job = decode_job(a, lb / tiles_per_limb);
    const uint32_t tile = lb % tiles_per_limb;
    const size_t off = (size_t)tile * tile_elems;
    const uint32_t blk0 = tile << log_b;                   // first 256-block of this tile within the limb
    const size_t n = (size_t)1 << a.log_n;
    double *ld = reinterpret_cast<double *>(lds);

    const uint64_t *src = FWD ? job.out : job.in;  // the forward blocks pass continues on the rows pass's output
    if (FP && !FWD) {
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) ld[skew(e)] = fp_from_u64(src[off + e]);
    } else {
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) lds[skew(e)] = src[off + e];
    }
    __syncthreads();

    const bool epi = a.epi_mode == NTT_EPI_SUB_MUL || a.epi_mode == NTT_EPI_SUB_MUL_ADD;
    const uint64_t *minuend = epi ? a.epi_a + ((size_t)job.poly * a.epi_a_poly_stride + job.limb) * n + off : nullptr;
    const uint64_t *addend =
        a.epi_mode == NTT_EPI_SUB_MUL_ADD ? a.epi_b + ((size_t)job.poly * a.epi_b_poly_stride + job.limb) * n + off : nullptr;
    uint64_t *dst = epi ? a.epi_dst + ((size_t)job.poly * a.epi_dst_poly_stride + job.limb) * n + off : job.out + off;
    // the epilogue operands are fetched now so that their latency hides behind the butterflies
    constexpr int kPer = kTile / kThreads;
    uint64_t pre_a[kPer], pre_b[kPer];
    if (FWD && epi) {
#pragma unroll
        for (int i = 0; i < kPer; i++) {
            const uint32_t e = threadIdx.x + i * kThreads;
            pre_a[i] = e < tile_elems ? minuend[e] : 0;
            pre_b[i] = (addend && e < tile_elems) ? addend[e] : 0;
        }
    }

    if (FP) {
        const FpCtx c = fp_ctx(a, job.table);
        if (FWD) {
            tile_pass_fp<4, true, true>(lds, tile_elems, 4, (1u << lr) + blk0, c);
            __syncthreads();
            tile_pass_fp<4, true, true>(lds, tile_elems, 0, (1u << (lr + 4)) + (blk0 << 4), c);
            __syncthreads();
            if (epi) {
                const double wd = fp_from_u64(a.w[2 * job.limb]);
                const FpTw w{wd, wd * c.m.qinv};
#pragma unroll
                for (int i = 0; i < kPer; i++) {
                    const uint32_t e = threadIdx.x + i * kThreads;
                    if (e < tile_elems) {
                        const double v = fp_canonical(ld[skew(e)], c.m);
                        double r = fp_mulmod(fp_from_u64(pre_a[i]) - v, w, c.m);
                        if (addend) r += fp_from_u64(pre_b[i]);
                        dst[e] = fp_to_u64(fp_canonical(r, c.m));
                    }
                }
            } else {
                for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads)
                    dst[e] = fp_to_u64(fp_canonical(ld[skew(e)], c.m));
            }
        } else {
            tile_pass_fp<4, false, false>(lds, tile_elems, 0, (1u << (lr + 4)) + (blk0 << 4), c);
            __syncthreads();
            tile_pass_fp<4, false, true>(lds, tile_elems, 4, (1u << lr) + blk0, c);
            __syncthreads();
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) job.out[off + e] = lds[skew(e)];
        }
        return;
    }

    const IntCtx c = int_ctx(a, job.table);
    const uint64_t q = c.q;
    if (FWD) {
        tile_pass<4, true>(lds, tile_elems, 4, (1u << lr) + blk0, c);
        __syncthreads();
        tile_pass<4, true>(lds, tile_elems, 0, (1u << (lr + 4)) + (blk0 << 4), c);
        __syncthreads();
        if (epi) {
            const Shoup w = load_shoup(a.w, job.limb);
#pragma unroll
            for (int i = 0; i < kPer; i++) {
                const uint32_t e = threadIdx.x + i * kThreads;
                if (e < tile_elems) {
                    uint64_t v = reduce_4q(lds[skew(e)], q);
                    uint64_t r = mul_shoup(sub_mod(pre_a[i], v, q), w, q);
                    if (addend) r = add_mod(r, pre_b[i], q);
                    dst[e] = r;
                }
            }
        } else {
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) dst[e] = reduce_4q(lds[skew(e)], q);
        }
    } else {
        tile_pass<4, false>(lds, tile_elems, 0, (1u << (lr + 4)) + (blk0 << 4), c);
        __syncthreads();
        tile_pass<4, false>(lds, tile_elems, 4, (1u << lr) + blk0, c);
        __syncthreads();
        // lazy values in [0, 2q) go to the rows pass
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kThreads) job.out[off + e] = lds[skew(e)];
    }
}

template <bool FWD, bool FP>
hipError_t launch_rows(const NttArgs &a, uint32_t n_jobs, hipStream_t s) {
    const int ld = (int)a.log_n - 8;
    auto grid = [&](int ldv) {
        int logc = (kTileLog - ldv) < 8 ? (kTileLog - ldv) : 8;
        return dim3(n_jobs * (256u >> logc));
    };
    switch (ld) {
#define HE_CASE(LD)                                                                          \
    case LD:                                                                                 \
        hipLaunchKernelGGL((ntt_rows_kernel<LD, FWD, FP>), grid(LD), dim3(kThreads), 0, s, a); \
        break;
        HE_CASE(1) HE_CASE(2) HE_CASE(3) HE_CASE(4) HE_CASE(5) HE_CASE(6) HE_CASE(7) HE_CASE(8)
#undef HE_CASE
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <bool FWD, bool FP>
hipError_t launch_blocks(const NttArgs &a, uint32_t n_jobs, hipStream_t s) {
    const uint32_t lr = a.log_n - 8;
    const uint32_t log_b = lr < 4 ? lr : 4;
    hipLaunchKernelGGL((ntt_blocks_kernel<FWD, FP>), dim3(n_jobs << (lr - log_b)), dim3(kThreads), 0, s, a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_ntt_forward(const NttArgs &a, uint32_t n_polys, bool fp, hipStream_t s) {
    if (a.log_n < 9 || a.log_n > 16) return hipErrorInvalidValue;
    const uint32_t n_jobs = a.jobs ? a.n_jobs : n_polys * a.map.limbs;
    if (n_jobs == 0) return hipSuccess;
    hipError_t e = fp ? launch_rows<true, true>(a, n_jobs, s) : launch_rows<true, false>(a, n_jobs, s);
    if (e != hipSuccess) return e;
    return fp ? launch_blocks<true, true>(a, n_jobs, s) : launch_blocks<true, false>(a, n_jobs, s);
}

hipError_t launch_ntt_inverse(const NttArgs &a, uint32_t n_polys, bool fp, hipStream_t s) {
    if (a.log_n < 9 || a.log_n > 16) return hipErrorInvalidValue;
    const uint32_t n_jobs = a.jobs ? a.n_jobs : n_polys * a.map.limbs;
    if (n_jobs == 0) return hipSuccess;
    hipError_t e = fp ? launch_blocks<false, true>(a, n_jobs, s) : launch_blocks<false, false>(a, n_jobs, s);
    if (e != hipSuccess) return e;
    NttArgs rows = a;
    rows.in = a.out;  // the rows pass continues in place on the output buffer
    rows.in_poly_stride = a.out_poly_stride;
    return fp ? launch_rows<false, true>(rows, n_jobs, s) : launch_rows<false, false>(rows, n_jobs, s);
}

}  // namespace he
