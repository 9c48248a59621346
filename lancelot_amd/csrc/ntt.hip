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
// Inside a pass each thread takes 2^r elements into registers, runs r stages on them (r <= 4, radix-16) and
// hands them on; the stages of a pass form two such register blocks.  In the blocks pass both blocks take
// their elements from LDS and write them back.  In the rows pass (N >= 2^12) the outer block works on the
// words that a coalesced access of the tile gives the thread anyway, straight from or to global memory, and
// only the exchange between the two blocks goes through LDS (rows_direct below).  LDS indices are skewed by
// one word per 16 so that both the stride-16 and the stride-256 gathers of a wave hit distinct banks.
// The forward transform runs rows pass then blocks pass, the inverse the other way round.
//
// Two arithmetic back ends share this skeleton:
//   integer : 64-bit Shoup/Harvey butterflies, any prime below 2^61 (~35 VALU instructions per butterfly);
//             inverse twiddles are pre-halved so that 1/N comes for free
//   FP64    : exact integer arithmetic in doubles for primes below 2^50 (8 full-rate operations per
//             butterfly, see modarith.cuh); values between the two passes are lazy signed doubles stored
//             in the same 8-byte words; the factor 1/N is folded into the last multiplication
// A launch uses the FP64 back end when every limb it touches has a prime below 2^50, the integer one when none
// has, and otherwise the mixed instantiations, in which every workgroup follows its own limb's prime.
#include <cstdlib>
#include <type_traits>

#include "kernels.h"
#include "modarith.cuh"

namespace he {

namespace {

constexpr int kThreads = 256;
constexpr int kTileLog = 12;
constexpr uint32_t kTile = 1u << kTileLog;
constexpr uint32_t kLdsWords = kTile + (kTile >> 4);

__device__ __forceinline__ uint32_t skew(uint32_t e) { return e + (e >> 4); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load and
// store of the wave, which would serialise a prefetch issued before it with the butterflies after it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

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
    const uint64_t *src;   // NTT_PRO_SOURCE_[INTT_]REDUCE (rows pass only): the limb that is reduced into this one
    uint32_t src_table;    // NTT_PRO_SOURCE_INTT_REDUCE: its prime
};

__device__ __forceinline__ Job decode_job(const NttArgs &a, uint32_t job) {
    Job j;
    const size_t n = (size_t)1 << a.log_n;
    if (a.jobs) {
        // job = item * n_jobs + entry of the list
        const uint32_t item = job / a.n_jobs;
        LimbJob lj = a.jobs[job - item * a.n_jobs];
        j.in = a.in + item * a.item_stride + (size_t)lj.data_limb * n;
        j.out = a.out + item * a.item_stride + (size_t)lj.data_limb * n;
        j.table = lj.table;
        j.poly = 0;
        j.limb = 0;
        const bool sourced = a.pro_mode == NTT_PRO_SOURCE_REDUCE || a.pro_mode == NTT_PRO_SOURCE_INTT_REDUCE;
        j.src_table = sourced ? lj.data_limb / a.pro_lk : 0;
        j.src = sourced ? a.pro_src + item * a.pro_item_stride + (size_t)j.src_table * n : nullptr;
    } else {
        j.poly = job / a.map.limbs;
        j.limb = job % a.map.limbs;
        j.in = a.in ? a.in + ((size_t)j.poly * a.in_poly_stride + j.limb) * n : nullptr;
        j.out = a.out + ((size_t)j.poly * a.out_poly_stride + j.limb) * n;
        j.table = map_table(a.map, j.limb);
        j.src = a.pro_src + ((size_t)j.poly * a.pro_poly_stride << a.log_n);
        j.src_table = a.pro_src_table;
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
    for (uint32_t g = threadIdx.x; g < groups; g += blockDim.x) {
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
                                             FpCtx c, uint32_t first = threadIdx.x, uint32_t stride = blockDim.x) {
    constexpr int R = 1 << LOGR;
    double *ld = reinterpret_cast<double *>(lds);
    const uint32_t groups = tile_elems >> LOGR;
    const uint32_t low_mask = (1u << low_bits) - 1;
    for (uint32_t g = first; g < groups; g += stride) {
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

// TL = log2(words per tile): 12, or 10 when a launch has too few limbs to give every CU a 4096-word tile
template <int LD, int TL>
__device__ __forceinline__ constexpr int log_cols() {
    return (TL - LD) < 8 ? (TL - LD) : 8;
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
// rows pass with 16 words per thread (N >= 2^12: a tile of 2^LD rows x C columns is 16 T words for its T threads).
// The stages split into an outer block of p0 and an inner block of p1 = LD - p0 stages.  The words of a thread's
// outer groups are t, t + T, ..., t + 15 T in tile order, i.e. what a coalesced load of the tile hands to thread t
// anyway, so the outer block runs on registers straight from (forward) or to (inverse) global memory and the
// tile crosses LDS once, between the blocks, instead of three times (no LDS at all when p1 = 0): the pass is
// bound by the latency of one workgroup, and two of its three LDS round trips and barriers go away.  Same
// arithmetic, same words.
//   outer: register i is tile word t + T i; group k of 16 >> p0 holds registers k + (16 >> p0) j; twiddle index 1
//   inner: group k of 16 >> p1 is group g = t + T k of the tile: registers k 2^p1 + j are the tile words
//          ((g / C) << (LOGC + p1)) + g mod C + j C; twiddle index 2^p0 + g / C
// Tile word e lives at row e / C, column col0 + e mod C of the limb's (N / 256) x 256 view.
// ---------------------------------------------------------------------------------------------------
// SRC_INTT (forward, NTT_PRO_SOURCE_INTT_REDUCE): the inverse rows pass of the source limb's tile runs first, on the
// same registers: its last block leaves the coefficient of tile word t + T i in register i, which is where the forward
// pass's first block takes its input from.
template <int LD, bool FWD, int BE, int LOGC, bool SRC_INTT = false>
__device__ __forceinline__ void rows_direct(const NttArgs &a, const Job &job, uint32_t col0, uint64_t *lds) {
    constexpr int p0 = Split<LD>::p0, p1 = Split<LD>::p1;
    constexpr int R0 = 1 << p0, R1 = 1 << p1, NG0 = 16 >> p0, NG1 = 16 >> p1;
    constexpr uint32_t C = 1u << LOGC, T = 1u << (LD + LOGC - 4);
    const uint32_t t = threadIdx.x, col = t & (C - 1);
    double *ld = reinterpret_cast<double *>(lds);
    // tile word, global offset and LDS slot of register i in the outer and in the inner layout (folded to a few
    // shifts and adds where they are used; tables of them would have to stay live across both back ends)
    auto e_far = [&](int i) { return t + T * (uint32_t)i; };
    auto e_near = [&](int i) {
        const uint32_t upper = (t + T * (uint32_t)(i >> p1)) >> LOGC;
        return (upper << (LOGC + p1)) + col + ((uint32_t)(i & (R1 - 1)) << LOGC);
    };
    auto glob = [&](uint32_t e) { return (size_t)(e >> LOGC) * 256 + col0 + col; };
    auto idx_near = [&](int k) { return (1u << p0) + ((t + T * (uint32_t)k) >> LOGC); };
    // the outer / inner block on every group of the 16 registers
    auto outer = [&](auto *v, auto block) {
#pragma unroll
        for (int k = 0; k < NG0; k++) {
            std::remove_reference_t<decltype(v[0])> w[R0];
#pragma unroll
            for (int j = 0; j < R0; j++) w[j] = v[k + NG0 * j];
            block(w, 1u);
#pragma unroll
            for (int j = 0; j < R0; j++) v[k + NG0 * j] = w[j];
        }
    };
    auto inner = [&](auto *v, auto block) {
#pragma unroll
        for (int k = 0; k < NG1; k++) block(v + k * R1, idx_near(k));
    };
    // canonical coefficients of the source limb at the tile words t + T i
    uint64_t s[SRC_INTT ? 16 : 1];
    if constexpr (SRC_INTT) {
        const uint32_t st = job.src_table;
        // (the tables of the inverse transform lie behind the forward ones: a.tw / a.tw_fp are the forward launch's)
        if ((a.pro_src_fp_mask >> st) & 1) {
            const FpMod m = fp_ctx(a, st).m;
            const double *itw = a.pro_itw_fp + ((size_t)st << a.log_n);
            double v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = __longlong_as_double((long long)job.src[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))]);
            if (p1 > 0) {
                inner(v, [&](double *w, uint32_t idx) { fp_gs_block<(p1 > 0 ? p1 : 1), true>(w, itw, idx, m); });
#pragma unroll
                for (int j = 0; j < 16; j++) ld[skew(e_near(j))] = v[j];
                __syncthreads();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = ld[skew(e_far(j))];
            }
            outer(v, [&](double *w, uint32_t idx) { fp_gs_block<p0, true>(w, itw, idx, m); });
            const double *cc = a.fp_consts + 4 * (size_t)st;
            const FpTw ninv{cc[2], cc[3]};
#pragma unroll
            for (int j = 0; j < 16; j++) s[SRC_INTT ? j : 0] = fp_to_u64(fp_canonical(fp_mulmod(v[j], ninv, m), m));
        } else {
            const uint64_t q = a.moduli[st];
            const uint64_t *itw = a.pro_itw + ((size_t)st << (a.log_n + 1));
            uint64_t v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = job.src[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))];
            if (p1 > 0) {
                inner(v, [&](uint64_t *w, uint32_t idx) { gs_block<(p1 > 0 ? p1 : 1)>(w, itw, idx, q); });
#pragma unroll
                for (int j = 0; j < 16; j++) lds[skew(e_near(j))] = v[j];
                __syncthreads();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = lds[skew(e_far(j))];
            }
            outer(v, [&](uint64_t *w, uint32_t idx) { gs_block<p0>(w, itw, idx, q); });
#pragma unroll
            for (int j = 0; j < 16; j++) s[SRC_INTT ? j : 0] = reduce_2q(v[j], q);
        }
        // (the forward pass below writes and reads the same LDS slots in the same order as the inverse pass read and
        // wrote them: a thread's own slots t + T i first, then a barrier)
    }
    const bool fp = BE == NTT_BACKEND_FP || (BE == NTT_BACKEND_MIXED && ((a.fp_mask >> job.table) & 1));
    if (BE != NTT_BACKEND_INT && fp) {
        const FpCtx c = fp_ctx(a, job.table);
        double v[16];
        if (FWD) {
            bool reduce_first = true;
            if constexpr (SRC_INTT) {
                const uint64_t q = a.moduli[job.table], r1 = a.barrett[2 * job.table + 1];
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = fp_from_u64(barrett64(s[SRC_INTT ? j : 0], q, r1));
                reduce_first = false;
            } else if (a.pro_mode == NTT_PRO_MODDOWN_RESCALE) {
                const uint64_t *tsrc = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
                const uint64_t *dsrc = a.pro_src2 + ((size_t)job.poly * a.pro2_poly_stride << a.log_n);
                const FpMod ml = fp_ctx(a, a.pro_last).m;
                const double wd = fp_from_u64(a.pro_w[2 * job.limb]), wl = fp_from_u64(a.pro_w[2 * a.pro_last]);
                const FpTw w{wd, wd * c.m.qinv}, wlast{wl, wl * ml.qinv};
                const uint64_t qj = a.moduli[job.table], rj = a.barrett[2 * job.table + 1];
                const uint64_t qlast = a.moduli[a.pro_last], rlast = a.barrett[2 * a.pro_last + 1];
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    const uint64_t ds = dsrc[glob(e_far(j))];
                    const uint64_t dl = a.pro_k1 ? barrett64(ds, qlast, rlast) : ds;
                    const uint64_t dj = a.pro_k1 ? barrett64(ds, qj, rj) : job.in[glob(e_far(j))];
                    // coefficient of the dropped limb of the ModDown result, canonical mod q_last
                    const double r = fp_canonical(fp_from_u64(tsrc[glob(e_far(j))]) - fp_mulmod(fp_from_u64(dl), wlast, ml), ml);
                    v[j] = fp_mulmod(fp_from_u64(dj), w, c.m) + fp_reduce(r, c.m);
                }
            } else if (a.pro_mode == NTT_PRO_BROADCAST_REDUCE) {
                // one source limb for every limb: it may exceed this limb's prime, so reduce first
                const uint64_t *src = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = fp_from_u64(src[glob(e_far(j))]);
            } else if (a.pro_mode == NTT_PRO_SOURCE_REDUCE) {
                const uint64_t q = a.moduli[job.table], r1 = a.barrett[2 * job.table + 1];
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = fp_from_u64(barrett64(job.src[glob(e_far(j))], q, r1));
                reduce_first = false;
            } else {
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = fp_from_u64(job.in[glob(e_far(j))]);
                reduce_first = false;
            }
            if (reduce_first)
                outer(v, [&](double *w, uint32_t idx) { fp_ct_block<p0, true>(w, c.tw, idx, c.m); });
            else
                outer(v, [&](double *w, uint32_t idx) { fp_ct_block<p0, false>(w, c.tw, idx, c.m); });
            if (p1 > 0) {
#pragma unroll
                for (int j = 0; j < 16; j++) ld[skew(e_far(j))] = v[j];
                __syncthreads();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = ld[skew(e_near(j))];
                inner(v, [&](double *w, uint32_t idx) { fp_ct_block<(p1 > 0 ? p1 : 1), true>(w, c.tw, idx, c.m); });
            }
            // lazy signed doubles go to the blocks pass
#pragma unroll
            for (int j = 0; j < 16; j++) job.out[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))] = (uint64_t)__double_as_longlong(v[j]);
        } else {
            // input: lazy signed doubles from the blocks pass; output: canonical residues
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = __longlong_as_double((long long)job.in[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))]);
            if (p1 > 0) {
                inner(v, [&](double *w, uint32_t idx) { fp_gs_block<(p1 > 0 ? p1 : 1), true>(w, c.tw, idx, c.m); });
#pragma unroll
                for (int j = 0; j < 16; j++) ld[skew(e_near(j))] = v[j];
                __syncthreads();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = ld[skew(e_far(j))];
            }
            outer(v, [&](double *w, uint32_t idx) { fp_gs_block<p0, true>(w, c.tw, idx, c.m); });
            const FpTw scale = inverse_scale(a, job, c.m);
#pragma unroll
            for (int j = 0; j < 16; j++)
                job.out[glob(e_far(j))] = fp_to_u64(fp_canonical(fp_mulmod(v[j], scale, c.m), c.m));
        }
        return;
    }

    const IntCtx c = int_ctx(a, job.table);
    const uint64_t q = c.q;
    uint64_t v[16];
    if (FWD) {
        if constexpr (SRC_INTT) {
            const uint64_t r1 = a.barrett[2 * job.table + 1];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = barrett64(s[SRC_INTT ? j : 0], q, r1);
        } else if (a.pro_mode == NTT_PRO_BROADCAST_REDUCE || a.pro_mode == NTT_PRO_SOURCE_REDUCE) {
            const uint64_t r1 = a.barrett[2 * job.table + 1];
            const uint64_t *src = a.pro_mode == NTT_PRO_SOURCE_REDUCE ? job.src : a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = barrett64(src[glob(e_far(j))], q, r1);
        } else if (a.pro_mode == NTT_PRO_MODDOWN_RESCALE) {
            const uint64_t r1 = a.barrett[2 * job.table + 1];
            const uint64_t *tsrc = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
            const uint64_t *dsrc = a.pro_src2 + ((size_t)job.poly * a.pro2_poly_stride << a.log_n);
            const uint64_t ql = a.moduli[a.pro_last];
            const Shoup w = load_shoup(a.pro_w, job.limb), wlast = load_shoup(a.pro_w, a.pro_last);
            const uint64_t rlast = a.barrett[2 * a.pro_last + 1];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const uint64_t ds = dsrc[glob(e_far(j))];
                const uint64_t dl = a.pro_k1 ? barrett64(ds, ql, rlast) : ds;
                const uint64_t dj = a.pro_k1 ? barrett64(ds, q, r1) : job.in[glob(e_far(j))];
                const uint64_t r = sub_mod(tsrc[glob(e_far(j))], mul_shoup(dl, wlast, ql), ql);
                v[j] = add_mod(mul_shoup(dj, w, q), barrett64(r, q, r1), q);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = job.in[glob(e_far(j))];
        }
        outer(v, [&](uint64_t *w, uint32_t idx) { ct_block<p0>(w, c.tw, idx, q); });
        if (p1 > 0) {
#pragma unroll
            for (int j = 0; j < 16; j++) lds[skew(e_far(j))] = v[j];
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = lds[skew(e_near(j))];
            inner(v, [&](uint64_t *w, uint32_t idx) { ct_block<(p1 > 0 ? p1 : 1)>(w, c.tw, idx, q); });
        }
        // lazy values in [0, 4q) go to the blocks pass
#pragma unroll
        for (int j = 0; j < 16; j++) job.out[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))] = v[j];
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = job.in[p1 > 0 ? glob(e_near(j)) : glob(e_far(j))];
        if (p1 > 0) {
            inner(v, [&](uint64_t *w, uint32_t idx) { gs_block<(p1 > 0 ? p1 : 1)>(w, c.tw, idx, q); });
#pragma unroll
            for (int j = 0; j < 16; j++) lds[skew(e_near(j))] = v[j];
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = lds[skew(e_far(j))];
        }
        outer(v, [&](uint64_t *w, uint32_t idx) { gs_block<p0>(w, c.tw, idx, q); });
        if (a.epi_mode == NTT_EPI_MUL) {
            const Shoup w = load_shoup(a.w, job.limb);
#pragma unroll
            for (int j = 0; j < 16; j++) job.out[glob(e_far(j))] = mul_shoup(v[j], w, q);
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) job.out[glob(e_far(j))] = reduce_2q(v[j], q);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// rows pass: stages 0 .. LD-1 (forward) over an R = 2^LD rows x 256 matrix
// ---------------------------------------------------------------------------------------------------
template <int LD, bool FWD, int BE, int TL, bool SRC_INTT = false>
__global__ __launch_bounds__((1 << TL) / 16) void ntt_rows_kernel(NttArgs a) {
    __shared__ uint64_t lds[(1 << TL) + (1 << (TL - 4))];
    constexpr uint32_t kRowThreads = (1u << TL) / 16;
    constexpr int LOGC = log_cols<LD, TL>();
    constexpr uint32_t C = 1u << LOGC;
    constexpr uint32_t tile_elems = 1u << (LD + LOGC);
    constexpr uint32_t tiles_per_limb = 256u >> LOGC;
    constexpr int p0 = Split<LD>::p0, p1 = Split<LD>::p1;

    const uint32_t lb = logical_block();
    const Job job = decode_job(a, lb / tiles_per_limb);
    const uint32_t col0 = (lb % tiles_per_limb) << LOGC;
    // (N = 2^17, 512 rows: the inner block would be five stages, 32 words a thread; that degree takes the tile
    // through LDS between its blocks, below)
    if constexpr (LD >= 4 && LD <= 8 && tile_elems == 16 * kRowThreads) {
        rows_direct<LD, FWD, BE, LOGC, SRC_INTT>(a, job, col0, lds);
        return;
    }
    static_assert(!SRC_INTT || (LD >= 4 && LD <= 8 && tile_elems == 16 * kRowThreads), "only the register rows pass");
    double *ld = reinterpret_cast<double *>(lds);

    // the back end of this workgroup's limb: fixed by the launch, or (mixed) by the limb's prime
    const bool fp = BE == NTT_BACKEND_FP || (BE == NTT_BACKEND_MIXED && ((a.fp_mask >> job.table) & 1));
    if (BE != NTT_BACKEND_INT && fp) {
        const FpCtx c = fp_ctx(a, job.table);
        if (FWD) {
            // input: canonical residues (or one broadcast source limb); output: lazy signed doubles
            const uint64_t *bsrc = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
            const uint64_t *src = a.pro_mode == NTT_PRO_BROADCAST_REDUCE ? bsrc : job.in;
            if (a.pro_mode == NTT_PRO_MODDOWN_RESCALE) {
                const uint64_t *dsrc = a.pro_src2 + ((size_t)job.poly * a.pro2_poly_stride << a.log_n);
                const FpMod ml = fp_ctx(a, a.pro_last).m;
                const double wd = fp_from_u64(a.pro_w[2 * job.limb]), wl = fp_from_u64(a.pro_w[2 * a.pro_last]);
                const FpTw w{wd, wd * c.m.qinv}, wlast{wl, wl * ml.qinv};
                const uint64_t qj = a.moduli[job.table], rj = a.barrett[2 * job.table + 1];
                const uint64_t qlast = a.moduli[a.pro_last], rlast = a.barrett[2 * a.pro_last + 1];
                for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                    uint32_t row = e >> LOGC, col = e & (C - 1);
                    const size_t g = (size_t)row * 256 + col0 + col;
                    const uint64_t ds = dsrc[g];
                    const uint64_t dl = a.pro_k1 ? barrett64(ds, qlast, rlast) : ds;
                    const uint64_t dj = a.pro_k1 ? barrett64(ds, qj, rj) : src[g];
                    // coefficient of the dropped limb of the ModDown result, canonical mod q_last
                    const double r = fp_canonical(fp_from_u64(bsrc[g]) - fp_mulmod(fp_from_u64(dl), wlast, ml), ml);
                    ld[skew(e)] = fp_mulmod(fp_from_u64(dj), w, c.m) + fp_reduce(r, c.m);
                }
            } else if (a.pro_mode == NTT_PRO_SOURCE_REDUCE) {
                const uint64_t q = a.moduli[job.table], r1 = a.barrett[2 * job.table + 1];
                for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                    uint32_t row = e >> LOGC, col = e & (C - 1);
                    ld[skew(e)] = fp_from_u64(barrett64(job.src[(size_t)row * 256 + col0 + col], q, r1));
                }
            } else {
                for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                    uint32_t row = e >> LOGC, col = e & (C - 1);
                    ld[skew(e)] = fp_from_u64(src[(size_t)row * 256 + col0 + col]);
                }
            }
            __syncthreads();
            // a broadcast source may exceed this limb's prime: reduce first in that case
            if (a.pro_mode != NTT_PLAIN)
                tile_pass_fp<p0, true, true>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
            else
                tile_pass_fp<p0, true, false>(lds, tile_elems, LD - p0 + LOGC, 1u, c);
            __syncthreads();
            if (p1 > 0) {
                tile_pass_fp<(p1 > 0 ? p1 : 1), true, true>(lds, tile_elems, LOGC, 1u << p0, c);
                __syncthreads();
            }
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = lds[skew(e)];
            }
        } else {
            // input: lazy signed doubles from the blocks pass; output: canonical residues
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
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
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = fp_to_u64(fp_canonical(fp_mulmod(ld[skew(e)], scale, c.m), c.m));
            }
        }
        return;
    }

    const IntCtx c = int_ctx(a, job.table);
    const uint64_t q = c.q;
    if (FWD && (a.pro_mode == NTT_PRO_BROADCAST_REDUCE || a.pro_mode == NTT_PRO_SOURCE_REDUCE)) {
        const uint64_t r1 = a.barrett[2 * job.table + 1];
        const uint64_t *src = a.pro_mode == NTT_PRO_SOURCE_REDUCE ? job.src : a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
            uint32_t row = e >> LOGC, col = e & (C - 1);
            lds[skew(e)] = barrett64(src[(size_t)row * 256 + col0 + col], q, r1);
        }
    } else if (FWD && a.pro_mode == NTT_PRO_MODDOWN_RESCALE) {
        const uint64_t r1 = a.barrett[2 * job.table + 1];
        const uint64_t *tsrc = a.pro_src + ((size_t)job.poly * a.pro_poly_stride << a.log_n);
        const uint64_t *dsrc = a.pro_src2 + ((size_t)job.poly * a.pro2_poly_stride << a.log_n);
        const uint64_t ql = a.moduli[a.pro_last];
        const Shoup w = load_shoup(a.pro_w, job.limb), wlast = load_shoup(a.pro_w, a.pro_last);
        const uint64_t rlast = a.barrett[2 * a.pro_last + 1];
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
            uint32_t row = e >> LOGC, col = e & (C - 1);
            const size_t g = (size_t)row * 256 + col0 + col;
            const uint64_t ds = dsrc[g];
            const uint64_t dl = a.pro_k1 ? barrett64(ds, ql, rlast) : ds;
            const uint64_t dj = a.pro_k1 ? barrett64(ds, q, r1) : job.in[g];
            const uint64_t r = sub_mod(tsrc[g], mul_shoup(dl, wlast, ql), ql);
            lds[skew(e)] = add_mod(mul_shoup(dj, w, q), barrett64(r, q, r1), q);
        }
    } else {
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
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
        for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
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
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = mul_shoup(lds[skew(e)], w, q);
            }
        } else {
            for (uint32_t e = threadIdx.x; e < tile_elems; e += kRowThreads) {
                uint32_t row = e >> LOGC, col = e & (C - 1);
                job.out[(size_t)row * 256 + col0 + col] = reduce_2q(lds[skew(e)], q);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Whole-limb transform for N <= 2^14 (FP64 back end, plain forward / inverse with the optional inverse scaling):
// one workgroup of N / 16 threads per limb keeps the limb in LDS (at most 136 KiB of the CU's 160) between its
// register blocks, so the limb crosses memory once in each direction instead of twice, in one launch instead of two.
// Forward: the first block (stages 0..3, words t + j N/16) comes straight from the coalesced load; the blocks after
// it exchange through LDS (skewed by a word per 16); the last block's results return to LDS for a coalesced store of
// canonical residues.  Inverse: the mirror image, the last block (words t + j N/16) is scaled and stored from
// registers.  LOGN = 4 NB4 + REM: NB4 blocks of four stages and one of REM stages at the fine end.
// ---------------------------------------------------------------------------------------------------
template <int LOGN, bool FWD>
__global__ __launch_bounds__((1 << LOGN) / 16) void ntt_limb_fp_kernel(NttArgs a) {
    constexpr uint32_t N = 1u << LOGN, T = N / 16;
    constexpr int NB4 = LOGN / 4, REM = LOGN % 4, PER = 16 >> REM;
    static_assert(LOGN >= 9 && LOGN <= 14, "a limb of at most 2^14 words");
    __shared__ double ld[N + N / 16];
    const Job job = decode_job(a, blockIdx.x);
    const FpCtx c = fp_ctx(a, job.table);
    const FpMod m = c.m;
    const uint32_t t = threadIdx.x;
    double v[16];
    // block k (stages 4k .. 4k+3) of thread t: words base + (j << low), twiddle index (1 << 4k) + upper
    auto geom = [&](int k, uint32_t &base, uint32_t &low, uint32_t &idx) {
        low = (uint32_t)(LOGN - 4 * (k + 1));
        const uint32_t upper = t >> low;
        base = (upper << (low + 4)) | (t & ((1u << low) - 1));
        idx = (1u << (4 * k)) + upper;
    };
    if (FWD) {
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = fp_from_u64(job.in[t + T * j]);
        fp_ct_block<4, false>(v, c.tw, 1u, m);
#pragma unroll
        for (int j = 0; j < 16; j++) ld[skew(t + T * j)] = v[j];
        lds_barrier();
#pragma unroll
        for (int k = 1; k < NB4; k++) {
            uint32_t base, low, idx;
            geom(k, base, low, idx);
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base + ((uint32_t)j << low))];
            fp_ct_block<4, true>(v, c.tw, idx, m);
#pragma unroll
            for (int j = 0; j < 16; j++) ld[skew(base + ((uint32_t)j << low))] = v[j];
            lds_barrier();
        }
        if constexpr (REM > 0) {
#pragma unroll
            for (int gi = 0; gi < PER; gi++) {
                const uint32_t g = t * PER + gi, base = g << REM;
                double w[1 << REM];
#pragma unroll
                for (int j = 0; j < (1 << REM); j++) w[j] = ld[skew(base + j)];
                fp_ct_block<(REM > 0 ? REM : 1), true>(w, c.tw, (1u << (4 * NB4)) + g, m);
#pragma unroll
                for (int j = 0; j < (1 << REM); j++) ld[skew(base + j)] = w[j];
            }
            lds_barrier();
        }
#pragma unroll
        for (int j = 0; j < 16; j++) job.out[t + T * j] = fp_to_u64(fp_canonical(ld[skew(t + T * j)], m));
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++) ld[skew(t + T * j)] = fp_from_u64(job.in[t + T * j]);
        lds_barrier();
        if constexpr (REM > 0) {
#pragma unroll
            for (int gi = 0; gi < PER; gi++) {
                const uint32_t g = t * PER + gi, base = g << REM;
                double w[1 << REM];
#pragma unroll
                for (int j = 0; j < (1 << REM); j++) w[j] = ld[skew(base + j)];
                fp_gs_block<(REM > 0 ? REM : 1), false>(w, c.tw, (1u << (4 * NB4)) + g, m);
#pragma unroll
                for (int j = 0; j < (1 << REM); j++) ld[skew(base + j)] = w[j];
            }
            lds_barrier();
        }
#pragma unroll
        for (int k = NB4 - 1; k >= 0; k--) {
            uint32_t base, low, idx;
            geom(k, base, low, idx);
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base + ((uint32_t)j << low))];
            if (REM == 0 && k == NB4 - 1)
                fp_gs_block<4, false>(v, c.tw, idx, m);   // canonical inputs
            else
                fp_gs_block<4, true>(v, c.tw, idx, m);
            if (k > 0) {
#pragma unroll
                for (int j = 0; j < 16; j++) ld[skew(base + ((uint32_t)j << low))] = v[j];
                lds_barrier();
            }
        }
        // block 0: base = t, low = log2(T): the coalesced store pattern
        const FpTw scale = inverse_scale(a, job, m);
#pragma unroll
        for (int j = 0; j < 16; j++) job.out[t + T * j] = fp_to_u64(fp_canonical(fp_mulmod(v[j], scale, m), m));
    }
}

template <bool FWD>
hipError_t launch_limb_fp(const NttArgs &a, uint32_t n_jobs, hipStream_t s) {
    switch (a.log_n) {
#define HE_CASE(LOGN) \
    case LOGN: hipLaunchKernelGGL((ntt_limb_fp_kernel<LOGN, FWD>), dim3(n_jobs), dim3((1u << LOGN) / 16), 0, s, a); break;
        HE_CASE(9) HE_CASE(10) HE_CASE(11) HE_CASE(12) HE_CASE(13) HE_CASE(14)
#undef HE_CASE
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// The launches that the whole-limb kernel covers and wins.  A limb is one workgroup on one CU: up to N = 2^12 that is
// faster than two launches whatever the number of limbs (10-12 us against 15-16 us for a forward + inverse pair);
// a limb of 2^13 or 2^14 words takes one CU 9 or 17 us, so there the kernel pays only when the launch has enough limbs
// to occupy the chip (measured break-even: 64 and 192 limbs; at 256 limbs 23 against 34 us and 50 against 60 us).
// a.one_pass = 2 forces it (tests).
inline bool one_pass_ok(const NttArgs &a, int backend, bool forward, uint32_t n_jobs) {
    if (!a.one_pass || backend != NTT_BACKEND_FP || a.log_n > 14 || a.jobs || a.pro_mode != NTT_PLAIN || a.in_galois ||
        !(a.epi_mode == NTT_PLAIN || (!forward && a.epi_mode == NTT_EPI_MUL)))
        return false;
    return a.one_pass == 2 || a.log_n <= 12 || n_jobs >= (a.log_n == 13 ? 64u : 192u);
}

// ---------------------------------------------------------------------------------------------------
// Base conversion fused with the rows pass of the forward transform that follows it (FP64 back end, N >= 2^12).
//
// Both operate on the same set of coefficients: a tile of all 2^LD rows x C columns of the limb's (N / 256) x 256
// view.  A workgroup of 256 threads owns a tile of 2048 coefficients (8 per thread) of one unit (a ModUp digit or a
// ModDown polynomial) and a group of the unit's output limbs.  Every thread keeps its 8 coefficients of the unit's
// (at most 8) input limbs in registers; for each output limb of the group it forms sum_i x_i M[r][i] for its
// coefficients, which are exactly the 8 words of its first register block of the rows pass (rows 2^(LD-3) apart),
// runs the first three stages on them, and the tile then crosses LDS between the remaining register blocks.  The
// converted limbs never exist in coefficient form in memory: 2 limb transfers and one launch less per output limb
// than conversion kernel + rows pass.  The groups of one tile re-read the same inputs (from L2: they run on one XCD).
//
// mdr (merged ModDown + rescale): the last matrix row belongs to the limb that the rescale drops; with
// r = t - sum_i x_i M[last][i] mod q_last (t: the limb right before the unit's inputs), output limb j receives
// sum_i x_i M[j][i] + (r mod q_j); the matrix carries the factor P^-1.
// ---------------------------------------------------------------------------------------------------
constexpr int kFuseLog = 11;
constexpr uint32_t kFuseWords = 1u << kFuseLog;

// LDS index of tile word e: 8 words of padding per 32 and 8 more per 256, so that the 32 lanes of a half-wave that
// read the words {32 a + 8 j + c}, {256 u + 32 j + c'} or {256 u + 32 j + 8 w + c} of one register slot j hit distinct
// 8-byte banks
__device__ __forceinline__ uint32_t skew8(uint32_t e) { return e + ((e >> 5) << 3) + ((e >> 8) << 3); }
constexpr uint32_t kFuseLds = kFuseWords + (kFuseWords >> 2) + (kFuseWords >> 5);

struct BconvRowsK {
    BconvRows b;
    uint32_t compute_groups, copy_groups, rows_per;
};

// register block of LOGR stages on the groups of a tile that lives in LDS (tile index bits: [upper][LOGR bits][low_bits]);
// P words per thread; twl: entries 0..255 of the limb's twiddle table, in LDS; LAST: the results go to global memory
// (lazy signed doubles for the blocks pass), else back to LDS
template <int LD, int P, int LOGR, bool LAST, bool SWZ = false>
__device__ __forceinline__ void fuse_block(double *ld, const double *twl, uint32_t s0, FpMod m, uint64_t *dst, uint32_t col0) {
    auto slot = [](uint32_t e) { return SWZ ? e ^ ((((e >> 5) ^ (e >> 8)) & 3u) << 3) : skew8(e); };
    constexpr int LOGC = kFuseLog - LD;
    constexpr uint32_t C = 1u << LOGC, T = kFuseWords / P;
    constexpr int R = 1 << LOGR, PER = P >> LOGR;
    const uint32_t low_bits = (uint32_t)(LD - LOGR + LOGC) - s0;
    const uint32_t low_mask = (1u << low_bits) - 1;
#pragma unroll
    for (int gi = 0; gi < PER; gi++) {
        const uint32_t g = threadIdx.x + T * gi;
        const uint32_t upper = g >> low_bits;
        const uint32_t base = (upper << (low_bits + LOGR)) | (g & low_mask);
        double v[R];
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = ld[slot(base + ((uint32_t)j << low_bits))];
        fp_ct_block<LOGR, 2>(v, twl, (1u << s0) + upper, m);
#pragma unroll
        for (int j = 0; j < R; j++) {
            const uint32_t e = base + ((uint32_t)j << low_bits);
            if (LAST)
                dst[(size_t)(e >> LOGC) * 256 + col0 + (e & (C - 1))] = (uint64_t)__double_as_longlong(v[j]);
            else
                ld[slot(e)] = v[j];
        }
    }
}

// the stages S0 .. LD-1 of the rows pass, in register blocks of at most log2(P) stages with the tile in LDS between them
template <int LD, int P, int S0>
__device__ __forceinline__ void fuse_rest(double *ld, const double *twl, FpMod m, uint64_t *dst, uint32_t col0) {
    constexpr int LOGP = P == 8 ? 3 : 2;
    constexpr int LOGR = (LD - S0) < LOGP ? (LD - S0) : LOGP;
    constexpr bool LAST = S0 + LOGR == LD;
    fuse_block<LD, P, LOGR, LAST>(ld, twl, S0, m, dst, col0);
    if constexpr (!LAST) {
        lds_barrier();
        fuse_rest<LD, P, S0 + LOGR>(ld, twl, m, dst, col0);
    }
}

// a value that every lane of the wave holds (read from LDS with one address) as a scalar
__device__ __forceinline__ double uniform_f64(double v) {
    const long long b = __double_as_longlong(v);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}

// output limbs per workgroup, at most (the LDS arrays of the rows' constants have this many entries; their loader
// strides over the workgroup, whatever its size)
constexpr uint32_t kFuseMaxRows = 24;

// P = coefficients per thread.  8: 256 threads, two waves per SIMD.  (4, with 512 threads and four waves per SIMD,
// compiles but measured 1.7 times slower at N = 2^16: the inputs' registers spill, and a tile needs twice the LDS
// exchanges and barriers.)
//
// Thread -> coefficient mapping.  The thread's P words are rows row0 + i 2^(LD-3) of one column (the first register
// block pairs exactly these).  At N = 2^16 (LD = 8: 256 rows x 8 columns) wave w takes row0 = w + 4 j, j = lane / 8:
// the second register block (stages 3..5, rows that differ in bits 2..4) then exchanges words inside the wave only, so
// the tile needs one workgroup barrier per output limb (before the last block) instead of three; the tile and the
// twiddles are double / triple buffered so that the next limb's first block never waits for this limb's last one.
// Other degrees use row0 = thread / C and a barrier after every block.
template <int LD, int P>
__global__ __launch_bounds__(kFuseWords / P) __attribute__((amdgpu_waves_per_eu(P == 8 ? 2 : 4)))
void bconv_rows_fp_kernel(NttArgs a, BconvRowsK p) {
    constexpr bool WAVE_B = LD == 8 && P == 8;
    __shared__ double ld[WAVE_B ? 2 : 1][kFuseLds];
    __shared__ double twl[3][256];
    __shared__ double mrow[kFuseMaxRows][18];
    __shared__ uint32_t mlimb[kFuseMaxRows], mtable[kFuseMaxRows];
    static_assert(LD >= 4 && LD <= 8 && (P == 8 || P == 4), "N from 2^12 to 2^16");
    constexpr int LOGC = kFuseLog - LD, LOGP = P == 8 ? 3 : 2;
    constexpr uint32_t T = kFuseWords / P;
    constexpr uint32_t C = 1u << LOGC, tiles_per_limb = 256u >> LOGC, row_step = T >> LOGC;
    const size_t n = (size_t)1 << a.log_n;

    // consecutive logical ids (one XCD, one L2): the groups of one tile, which read the same inputs
    uint32_t lb = logical_block();
    const uint32_t groups = p.compute_groups + p.copy_groups;
    const uint32_t grp = lb % groups;
    lb /= groups;
    const uint32_t tile = lb % tiles_per_limb, uidx = lb / tiles_per_limb;
    const uint32_t item = uidx / p.b.n_units;
    const BconvDesc d = p.b.descs[uidx - item * p.b.n_units];
    const uint32_t col0 = tile << LOGC;
    // word i of this thread: row row0 + i row_step, column col of the tile = tile word e0 + T i
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row0 = WAVE_B ? wave + 4 * (lane >> 3) : threadIdx.x >> LOGC;
    const uint32_t col = threadIdx.x & (C - 1);
    const uint32_t e0 = (row0 << LOGC) + col;
    const size_t g0 = (size_t)row0 * 256 + col0 + col;
    constexpr size_t gstep = (size_t)row_step * 256;
    uint64_t *out = p.b.out_base + item * p.b.out_item_stride + d.out_off;

    if (grp >= p.compute_groups) {
        // limbs that pass through unchanged (a digit's own limbs keep their NTT form)
        const uint64_t *from = p.b.copy_base + item * p.b.copy_item_stride;
        const uint32_t first = (grp - p.compute_groups) * p.rows_per;
        for (uint32_t r = first; r < first + p.rows_per && r < d.copy_count; r++) {
            const size_t limb = (size_t)(d.copy_first + r) << a.log_n;
            uint64_t w[P];
#pragma unroll
            for (int i = 0; i < P; i++) w[i] = from[limb + g0 + gstep * i];
#pragma unroll
            for (int i = 0; i < P; i++) out[limb + g0 + gstep * i] = w[i];
        }
        return;
    }
    const uint32_t n_rows = p.b.mdr ? d.n_out - 1 : d.n_out;
    const uint32_t r_begin = grp * p.rows_per;
    const uint32_t r_end = r_begin + p.rows_per < n_rows ? r_begin + p.rows_per : n_rows;
    if (r_begin >= n_rows) return;

    // The constants of this group's output limbs (matrix row, modulus, output limb, table) go to LDS once, and are
    // read back into scalar registers limb by limb: a scalar load per limb would stall the workgroup for a cache miss.
    const double *mat = p.b.mat_fp + 2 * d.mat_off;
    for (uint32_t w = threadIdx.x; w < (r_end - r_begin) * 18; w += T) {
        const uint32_t rl = w / 18, c = w - rl * 18, r = r_begin + rl;
        const uint32_t table = p.b.out_table[d.map_off + r];
        // (the matrices are padded: 8 pairs can be fetched whatever the row's length)
        mrow[rl][c] = c < 16 ? mat[2 * (size_t)r * d.n_in + c] : a.fp_consts[4 * (size_t)table + (c - 16)];
        if (c == 0) {
            mlimb[rl] = p.b.out_limb[d.map_off + r];
            mtable[rl] = table;
        }
    }
    // entries 1..255 of the first limb's table: every twiddle of the rows pass
    double tw_cur = a.tw_fp[((size_t)p.b.out_table[d.map_off + r_begin] << a.log_n) + (threadIdx.x & 255)];

    // the unit's inputs at this thread's P coefficients (limbs past n_in repeat the last one; their matrix entries
    // are replaced by zero below), all loads in flight together
    const uint64_t *x = p.b.x_base + item * p.b.x_item_stride + d.x_off;
    double xv[8][P];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const uint32_t kk = (uint32_t)k < d.n_in ? (uint32_t)k : d.n_in - 1;
#pragma unroll
        for (int i = 0; i < P; i++) xv[k][i] = fp_from_u64(x[((size_t)kk << a.log_n) + g0 + gstep * i]);
    }

    double rr[P];
#pragma unroll
    for (int i = 0; i < P; i++) rr[i] = 0.0;
    if (p.b.mdr) {
        // coefficients of the dropped limb of the ModDown result, canonical mod q_last
        const uint32_t last = d.n_out - 1;
        const FpMod ml = fp_ctx(a, p.b.out_table[d.map_off + last]).m;
        const double *row = mat + 2 * (size_t)last * d.n_in;
        const uint64_t *tsrc = x - n;
#pragma unroll
        for (int i = 0; i < P; i++) rr[i] = fp_from_u64(tsrc[g0 + gstep * i]);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const bool on = (uint32_t)k < d.n_in;
            const FpTw w{on ? row[2 * k] : 0.0, on ? row[2 * k + 1] : 0.0};
#pragma unroll
            for (int i = 0; i < P; i++) rr[i] -= fp_mulmod(xv[k][i], w, ml);
        }
#pragma unroll
        for (int i = 0; i < P; i++) rr[i] = fp_canonical(rr[i], ml);
    }
    if (threadIdx.x < 256) twl[r_begin % 3][threadIdx.x] = tw_cur;
    lds_barrier();

    for (uint32_t r = r_begin; r < r_end; r++) {
        const uint32_t rl = r - r_begin;
        // the next output limb's twiddles travel while this one is computed
        double tw_nxt = 0.0;
        const bool more = r + 1 < r_end;
        if (more) tw_nxt = a.tw_fp[((size_t)mtable[rl + 1] << a.log_n) + (threadIdx.x & 255)];
        const FpMod mod{uniform_f64(mrow[rl][16]), uniform_f64(mrow[rl][17])};
        const uint32_t limb = __builtin_amdgcn_readfirstlane(mlimb[rl]);
        const double *tws = twl[r % 3];
        double *tile_ld = ld[WAVE_B ? (r & 1) : 0];
        // sum_k x_k M_k as an exact pair (hi, lo) before any reduction, four operations per term instead of the seven of
        // a modular product and an addition.  hi runs in [2^103, 2^104), where doubles are the multiples of 2^51: the
        // fused multiply-add t = fl(x w + hi) rounds the exact sum to such a multiple (eight products below 2^100 keep
        // it under 2^104), t - hi is exact, x w - (t - hi) is the rounding error, an integer of at most 2^50 in
        // magnitude that the second fused multiply-add returns exactly, and eight of those sum exactly (<= 2^53).
        // The value is (hi - 2^103) + lo; it is reduced once per output word.
        double hi[P], lo[P];
#pragma unroll
        for (int i = 0; i < P; i++) {
            hi[i] = 0x1p103;
            lo[i] = 0.0;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const double w = (uint32_t)k < d.n_in ? uniform_f64(mrow[rl][2 * k]) : 0.0;
#pragma unroll
            for (int i = 0; i < P; i++) {
                const double t = __builtin_fma(xv[k][i], w, hi[i]);
                const double step = t - hi[i];
                lo[i] += __builtin_fma(xv[k][i], w, -step);
                hi[i] = t;
            }
        }
        // (hi - 2^103) / 2^51 is an integer below 2^52; times c = 2^51 mod m it is congruent to the high part.  The
        // modular product takes it as it is: for |x| < 2^52 the quotient estimate is off by at most 1.5 |x| 2^-52 + 1,
        // so |x c - k m| <= 2.5 m < 2^53 and every step stays exact.  With the rescale term (canonical for the dropped
        // prime, below 2^50, added as it is) |v| <= 3 m + 2^50 <= 4 x 2^50: the bound that the register blocks of
        // this pass start from (they reduce only what they do not multiply, see fp_ct_block).
        const double c51 = fp_reduce(0x1p51, mod);
        const FpTw w51{c51, c51 * mod.qinv};
        double v[P];
#pragma unroll
        for (int i = 0; i < P; i++) {
            v[i] = fp_mulmod((hi[i] - 0x1p103) * 0x1p-51, w51, mod) + fp_reduce(lo[i], mod);
            if (p.b.mdr) v[i] += rr[i];
        }
        // the first log2(P) stages pair rows that differ in their top bits: this thread's own P words
        fp_ct_block<LOGP, 2>(v, tws, 1u, mod);
#pragma unroll
        for (int i = 0; i < P; i++) tile_ld[skew8(e0 + T * i)] = v[i];
        uint64_t *dst = out + ((size_t)limb << a.log_n);
        if constexpr (WAVE_B) {
            // stages 3..5 inside the wave: lane (u, col) takes rows 32 u + 4 j + wave, which lanes of this wave wrote
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            const uint32_t u = lane >> 3;
            const uint32_t base = ((32 * u + wave) << LOGC) + col;
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = tile_ld[skew8(base + ((uint32_t)(4 * j) << LOGC))];
            fp_ct_block<3, 2>(v, tws, 8u + u, mod);
#pragma unroll
            for (int j = 0; j < 8; j++) tile_ld[skew8(base + ((uint32_t)(4 * j) << LOGC))] = v[j];
            // the twiddles of the next limb become visible with the same barrier (their buffer was last read two
            // limbs ago, and every wave has passed the barrier of the limb in between)
            if (more) twl[(r + 1) % 3][threadIdx.x] = tw_nxt;
            lds_barrier();
            fuse_block<LD, P, 2, true>(tile_ld, tws, 6, mod, dst, col0);
        } else {
            lds_barrier();
            fuse_rest<LD, P, LOGP>(tile_ld, tws, mod, dst, col0);
            if (more && threadIdx.x < 256) twl[(r + 1) % 3][threadIdx.x] = tw_nxt;
            lds_barrier();  // every read of this tile is done before the next output limb overwrites it
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// The same fusion at N = 2^16 with the matrix product of the conversion on the int8 matrix cores.
//
// sum_i x_i M[r][i] mod q_r is a 64-term integer product per 7-bit digit of the constants M_ij = M[r][i] 2^(8 j) mod q_r,
// over the bytes x_ij of the inputs as they lie in memory (BconvRows::mx_tab).  One v_mfma_i32_16x16x64_i8 forms it for 16
// coefficients, four output rows and four digits; two of them (digits 0..3, 4..7) leave the 8 digit sums S_e < 2^21 of
// (row rr, coefficient c) in lane 16 rr + c, and
//     sum_e S_e 2^(7 e) = lo + 2^28 hi,   lo = S_0 + 2^7 S_1 + 2^14 S_2 + 2^21 S_3 < 2^43,  hi likewise,
// becomes the lazy residue (hi x (2^28 mod q)) mod q + lo with one modular product: 13 FP64-rate operations and two
// matrix instructions per word against 44 operations for the eight exact multiply-adds on the vector units.
//
// Wave w of the workgroup owns the coefficients of rows w + 4 j + 32 i (j, i < 8) of the 256 x 8 tile, as in the kernel
// above; lane (kg, c) keeps the words of input limbs 2 kg, 2 kg + 1 for coefficient c of each of 32 sets of 16
// coefficients (set (g, i): (j, column) = (2 g + c / 8, c % 8), row w + 4 j + 32 i), which is at once the B operand of the
// set.  Output rows go four at a time: lane (rr, c) receives row rr's words of every set, i.e. for each g the 8 words
// i = 0..7 of one first register block, runs the block on them and stores them to row rr's tile in LDS.  The second block
// (stages 3..5) stays inside the wave tile by tile, the third follows a workgroup barrier, as above.
//
// LDS index of tile word e = (row << 3) | column: bits 4..3 are XORed with bits 6..5 and bits 9..8.  The accesses of
// a half-wave vary the column and either bit 5 (first block), bits 9..8 (second) or bits 6..5 (third) with bits 4..3
// fixed, so they fall into distinct 8-byte banks; consecutive tiles start 16 words apart modulo 32, which separates the
// two output rows that the lanes of a half-wave store in the first block.
// ---------------------------------------------------------------------------------------------------
typedef int v4i __attribute__((ext_vector_type(4)));
constexpr uint32_t kMxStride = kFuseWords + 16;
__device__ __forceinline__ uint32_t swz8(uint32_t e) { return e ^ ((((e >> 5) ^ (e >> 8)) & 3u) << 3); }

template <bool MDR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void bconv_rows_mx_kernel(NttArgs a, BconvRowsK p) {
    __shared__ double tiles[4 * kMxStride];
    __shared__ double twl[4][256];
    __shared__ double rconst[2][4][4];         // per group parity and row: q, 1/q, the constant that the digit sums lack
    __shared__ uint32_t rlimb[2][4];
    __shared__ uint32_t rtable[kFuseMaxRows + 4];
    constexpr int LOGC = 3;
    constexpr uint32_t tiles_per_limb = 32;

    uint32_t lb = logical_block();
    const uint32_t groups = p.compute_groups + p.copy_groups;
    const uint32_t grp = lb % groups;
    lb /= groups;
    const uint32_t tile = lb % tiles_per_limb, uidx = lb / tiles_per_limb;
    const uint32_t item = uidx / p.b.n_units;
    const BconvDesc d = p.b.descs[uidx - item * p.b.n_units];
    const uint32_t col0 = tile << LOGC;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, kg = lane >> 4, cn = lane & 15;
    uint64_t *out = p.b.out_base + item * p.b.out_item_stride + d.out_off;

    if (grp >= p.compute_groups) {
        // limbs that pass through unchanged (a digit's own limbs keep their NTT form)
        const uint64_t *from = p.b.copy_base + item * p.b.copy_item_stride;
        const uint32_t first = (grp - p.compute_groups) * p.rows_per;
        const size_t g0 = (size_t)(threadIdx.x >> LOGC) * 256 + col0 + (threadIdx.x & 7);
        for (uint32_t r = first; r < first + p.rows_per && r < d.copy_count; r++) {
            const size_t limb = (size_t)(d.copy_first + r) << 16;
            uint64_t w[8];
#pragma unroll
            for (int i = 0; i < 8; i++) w[i] = from[limb + g0 + (size_t)i * 32 * 256];
#pragma unroll
            for (int i = 0; i < 8; i++) out[limb + g0 + (size_t)i * 32 * 256] = w[i];
        }
        return;
    }
    const uint32_t n_rows = MDR ? d.n_out - 1 : d.n_out;
    const uint32_t r_begin = grp * p.rows_per;
    const uint32_t r_end = r_begin + p.rows_per < n_rows ? r_begin + p.rows_per : n_rows;
    if (r_begin >= n_rows) return;

    // the tables of this workgroup's rows (rows past the end repeat the last one; they are computed and not stored)
    if (threadIdx.x < kFuseMaxRows + 4) {
        const uint32_t r = r_begin + threadIdx.x < r_end ? r_begin + threadIdx.x : r_end - 1;
        rtable[threadIdx.x] = p.b.out_table[d.map_off + r];
    }
    // the inputs: bytes 0..6 as signed numbers (x - 128), byte 7 (zero: the residues are below 2^50) stays zero
    const uint64_t *x = p.b.x_base + item * p.b.x_item_stride + d.x_off;
    const uint32_t l0 = 2 * kg < d.n_in ? 2 * kg : d.n_in - 1, l1 = 2 * kg + 1 < d.n_in ? 2 * kg + 1 : d.n_in - 1;
    // (a uniform base and 32-bit byte offsets: one address register per load in flight instead of two)
    const char *xbytes = reinterpret_cast<const char *>(x);
    int xb[32][4];   // (scalars: the merged mode rewrites single bytes of them in place)
    auto operand = [&](int s) { return v4i{xb[s][0], xb[s][1], xb[s][2], xb[s][3]}; };
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const uint32_t G = cn + 16 * g;
        const uint32_t o = ((wave + 4 * (G >> 3)) * 256 + (G & 7) + col0) * 8;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t oi = o + (uint32_t)i * (32 * 256 * 8);
            const uint64_t u0 = *reinterpret_cast<const uint64_t *>(xbytes + ((l0 << 19) + oi)) ^ 0x0080808080808080ull;
            const uint64_t u1 = *reinterpret_cast<const uint64_t *>(xbytes + ((l1 << 19) + oi)) ^ 0x0080808080808080ull;
            xb[8 * g + i][0] = (int)(uint32_t)u0;
            xb[8 * g + i][1] = (int)(uint32_t)(u0 >> 32);
            xb[8 * g + i][2] = (int)(uint32_t)u1;
            xb[8 * g + i][3] = (int)(uint32_t)(u1 >> 32);
        }
    }
    if (MDR) {
        // merged ModDown + rescale: r = (t - sum_i x_i M[last][i]) mod q_last, canonical, is added to every output row;
        // its bytes 0..6 go into byte 7 of the words of limbs 0..6, where the rows' records hold the digits of 2^(8 i).
        // The record of the dropped row repeats it in all four row slots, so that every lane holds r of its coefficient.
        // t, the limb before the unit's inputs, crosses LDS (the tiles are not in use yet): fetched per lane where it is
        // needed, its 32 words would wait in registers beside the inputs.
        {
            const uint64_t *tsrc = x - ((size_t)1 << 16) + col0 + (size_t)(threadIdx.x >> LOGC) * 256 + (threadIdx.x & 7);
            uint64_t *tl = reinterpret_cast<uint64_t *>(tiles);
            uint64_t tw[8];
#pragma unroll
            for (int i = 0; i < 8; i++) tw[i] = tsrc[(size_t)i * 32 * 256];
#pragma unroll
            for (int i = 0; i < 8; i++) tl[threadIdx.x + 256 * i] = tw[i];   // tile word (row << 3) | column
        }
        lds_barrier();
        const uint32_t ltable = p.b.out_table[d.map_off + d.n_out - 1];
        const FpMod ml{a.fp_consts[4 * (size_t)ltable], a.fp_consts[4 * (size_t)ltable + 1]};
        const v4i *lrec = reinterpret_cast<const v4i *>(p.b.mx_last);
        const v4i la = lrec[lane], lh = lrec[64 + lane];
        const double *loff = reinterpret_cast<const double *>(lrec + 128);
        const double off = loff[0];
        const double c28 = fp_reduce(0x1p28, ml);
        const FpTw w28{c28, c28 * ml.qinv};
        const uint64_t *tl = reinterpret_cast<const uint64_t *>(tiles);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t G = cn + 16 * g;
            const uint32_t e = ((wave + 4 * (G >> 3)) << LOGC) | (G & 7);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const v4i zero = {0, 0, 0, 0};
                const v4i lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(la, operand(8 * g + i), zero, 0, 0, 0);
                const v4i hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(lh, operand(8 * g + i), zero, 0, 0, 0);
                const int l01 = lo.x + lo.y * 128, l23 = lo.z + lo.w * 128;
                const int h01 = hi.x + hi.y * 128, h23 = hi.z + hi.w * 128;
                const double ld = __builtin_fma((double)l23, 16384.0, (double)l01) + off;
                const double hd = __builtin_fma((double)h23, 16384.0, (double)h01);
                const double t = fp_from_u64(tl[e + ((uint32_t)(32 * i) << LOGC)]);
                const uint64_t r = fp_to_u64(fp_canonical(t - (fp_mulmod(hd, w28, ml) + ld), ml));
                const uint32_t b0 = (uint32_t)(r >> (16 * kg)) & 0xffu, b1 = (uint32_t)(r >> (16 * kg + 8)) & 0xffu;
                // (in place: as a new value in the source, the compiler keeps the old and the new operand beside each other,
                // 32 times four registers)
                asm volatile("v_or_b32 %0, %0, %1" : "+v"(xb[8 * g + i][1]) : "v"((b0 ^ 0x80u) << 24));
                asm volatile("v_or_b32 %0, %0, %1" : "+v"(xb[8 * g + i][3]) : "v"((b1 ^ 0x80u) << 24));
            }
        }
        lds_barrier();   // the tiles are free again
    }
    const v4i *rec = reinterpret_cast<const v4i *>(p.b.mx_tab) + ((size_t)d.mx_off + (r_begin >> 2)) * kMxRecord;
    lds_barrier();   // rtable

    // Twiddles: entries 1..63 of a row's table serve the first two blocks, 64..255 the third.  Thread t fetches entry
    // t % 64 of row t / 64 for the first part and entries 64 + t % 64 + 64 c (c < 3) of that row for the second.
    const uint32_t trow = threadIdx.x >> 6, tcol = threadIdx.x & 63;
    auto low_part = [&](uint32_t k) {   // group k of this workgroup: (entry tcol of row trow, that row's constants)
        return a.tw_fp[((size_t)rtable[4 * k + trow] << 16) + tcol];
    };
    auto stage_consts = [&](uint32_t k, const v4i *rc) {
        if (threadIdx.x < 16) {
            const uint32_t rr = threadIdx.x >> 2, c = threadIdx.x & 3;
            const double *off = reinterpret_cast<const double *>(rc + 128);
            rconst[k & 1][rr][c] = c < 2 ? a.fp_consts[4 * (size_t)rtable[4 * k + rr] + c] : off[2 * rr + (c - 2)];
        }
        if (threadIdx.x >= 16 && threadIdx.x < 20) {
            const uint32_t rr = threadIdx.x - 16;
            const uint32_t r = r_begin + 4 * k + rr < r_end ? r_begin + 4 * k + rr : r_end - 1;
            rlimb[k & 1][rr] = p.b.out_limb[d.map_off + r];
        }
    };
    twl[trow][tcol] = low_part(0);
    stage_consts(0, rec);
    lds_barrier();

    // a group's matrix digits (from L2: every workgroup of the unit reads the same ones); the next group's are requested
    // as soon as the first block has issued its last product
    v4i alo = rec[lane], ahi = rec[64 + lane];
    uint32_t k = 0;
    for (uint32_t r0 = r_begin; r0 < r_end; r0 += 4, rec += kMxRecord, k++) {
        const uint32_t nr = r_end - r0 < 4 ? r_end - r0 : 4;
        const bool more = r0 + 4 < r_end;
        {
            // first block, lane (rr, c) on row rr = kg
            const FpMod mod{rconst[k & 1][kg][0], rconst[k & 1][kg][1]};
            const double off = rconst[k & 1][kg][2];
            const double c28 = fp_reduce(0x1p28, mod);
            const FpTw w28{c28, c28 * mod.qinv};
            const double *tws = twl[kg];
            double *tile_ld = tiles + kg * kMxStride;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                // (opaque: computed once for the whole loop, the 32 store addresses would occupy registers through all of it)
                uint32_t cn_ = cn;
                asm volatile("" : "+v"(cn_));
                const uint32_t G = cn_ + 16 * g;
                const uint32_t z = swz8(((wave + 4 * (G >> 3)) << LOGC) | (G & 7));
                double v[8];
                // (the products of set i + 1 are issued before set i's are taken up: the matrix cores need 16 cycles each)
                const v4i zero = {0, 0, 0, 0};
                v4i lo_next = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo, operand(8 * g), zero, 0, 0, 0);
                v4i hi_next = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi, operand(8 * g), zero, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const v4i lo = lo_next, hi = hi_next;
                    if (i < 7) {
                        lo_next = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo, operand(8 * g + i + 1), zero, 0, 0, 0);
                        hi_next = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi, operand(8 * g + i + 1), zero, 0, 0, 0);
                    }
                    // signed digit sums (the bytes entered as x - 128): |S| < 2^21, the pairs below 2^29, lo and hi exact
                    const int l01 = lo.x + lo.y * 128, l23 = lo.z + lo.w * 128;
                    const int h01 = hi.x + hi.y * 128, h23 = hi.z + hi.w * 128;
                    const double ld = __builtin_fma((double)l23, 16384.0, (double)l01) + off;
                    const double hd = __builtin_fma((double)h23, 16384.0, (double)h01);
                    // |v| <= (1/2 + 2^-8) q + 2^44 + q: within the 4 x 2^50 that the register blocks of this pass start from
                    v[i] = fp_mulmod(hd, w28, mod) + ld;
                }
                fp_ct_block<3, 2>(v, tws, 1u, mod);
                // word i is 32 i rows further: bits 10..8 of the tile index, of which the slot takes bits 9..8 into bits 4..3
#pragma unroll
                for (int i = 0; i < 8; i++) tile_ld[z ^ (uint32_t)(((i & 3) << 3) | (i << 8))] = v[i];
            }
        }
        if (more) {
            alo = rec[kMxRecord + lane];
            ahi = rec[kMxRecord + 64 + lane];
        }
        // the twiddles of the third block travel during the second
        double tw_hi[3];
#pragma unroll
        for (int c = 0; c < 3; c++) tw_hi[c] = a.tw_fp[((size_t)rtable[4 * k + trow] << 16) + 64 + tcol + 64 * c];
        // stages 3..5 inside the wave, tile by tile: lane (u, col) takes rows 32 u + 4 j + wave, which lanes of this wave wrote
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        {
            // (all four tiles, also those of rows past the end: the words of the next tile are read before the block of
            // the current one runs)
            const uint32_t u = lane >> 3;
            const uint32_t base = ((32 * u + wave) << LOGC) + (lane & 7);
            double vn[8];
#pragma unroll
            for (int j = 0; j < 8; j++) vn[j] = tiles[swz8(base + ((uint32_t)(4 * j) << LOGC))];
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                const FpMod mod{uniform_f64(rconst[k & 1][rr][0]), uniform_f64(rconst[k & 1][rr][1])};
                double *tile_ld = tiles + rr * kMxStride;
                double v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = vn[j];
                if (rr < 3) {
#pragma unroll
                    for (int j = 0; j < 8; j++) vn[j] = tile_ld[kMxStride + swz8(base + ((uint32_t)(4 * j) << LOGC))];
                }
                fp_ct_block<3, 2>(v, twl[rr], 8u + u, mod);
#pragma unroll
                for (int j = 0; j < 8; j++) tile_ld[swz8(base + ((uint32_t)(4 * j) << LOGC))] = v[j];
            }
        }
        // (the third block of the previous group, the last reader of these entries, ended before that group's last barrier)
#pragma unroll
        for (int c = 0; c < 3; c++) twl[trow][64 + tcol + 64 * c] = tw_hi[c];
        lds_barrier();
        // the next group's first twiddles and constants travel during the third block
        double tw_lo = 0.0;
        if (more) tw_lo = low_part(k + 1);
        for (uint32_t rr = 0; rr < nr; rr++) {
            const FpMod mod{uniform_f64(rconst[k & 1][rr][0]), uniform_f64(rconst[k & 1][rr][1])};
            const uint32_t limb = __builtin_amdgcn_readfirstlane(rlimb[k & 1][rr]);
            fuse_block<8, 8, 2, true, true>(tiles + rr * kMxStride, twl[rr], 6, mod, out + ((size_t)limb << 16), col0);
        }
        if (more) {
            // entries 0..63 were last read by the second block, before the barrier above
            twl[trow][tcol] = tw_lo;
            stage_consts(k + 1, rec + kMxRecord);
        }
        lds_barrier();  // every read of the tiles is done before the next four rows overwrite them
    }
}

// ---------------------------------------------------------------------------------------------------
// blocks pass: the 8 stages that stay inside 256 consecutive words
//
// A workgroup of T threads owns a tile of 16 T consecutive words (T = 128 or 256) and walks through every
// limb of its unit: the limbs of one unit share a modulus, hence a twiddle table, and the table is as large
// as a limb, so reading it once per unit instead of once per limb removes up to half of the pass's HBM
// traffic.  The next limb's tile is fetched into registers while the current one is transformed.
// ---------------------------------------------------------------------------------------------------
struct Unit {
    uint32_t j0, jstride, count;
};

// map mode: unit = (limb i, group of `batch` polynomials); list mode: unit = group of consecutive jobs
__device__ __forceinline__ Unit decode_unit(const NttArgs &a, uint32_t u) {
    if (a.jobs) {
        const uint32_t item = u / a.n_groups;
        const LimbGroup g = a.groups[u - item * a.n_groups];
        return Unit{item * a.n_jobs + g.first, 1u, g.count};
    }
    const uint32_t limb = u % a.map.limbs, pg = u / a.map.limbs;
    const uint32_t p0 = pg * a.batch;
    const uint32_t cnt = a.n_polys - p0 < a.batch ? a.n_polys - p0 : a.batch;
    return Unit{p0 * a.map.limbs + limb, a.map.limbs, cnt};
}

// A workgroup of T threads owns 16 T consecutive words: T = 256 or 128 for N >= 2048, N / 16 below that, so
// that every thread moves exactly 16 words and no access needs a bounds check (straight-line code lets the
// compiler count the loads and stores in flight instead of draining them at every step).
struct BlocksGeom {
    uint32_t idx0, idx1;
    size_t off;
    Unit unit;
};

__device__ __forceinline__ BlocksGeom blocks_geom(const NttArgs &a) {
    const uint32_t lr = a.log_n - 8;                       // log2(number of 256-blocks per limb)
    const uint32_t tile_elems = blockDim.x << 4;
    const uint32_t log_b = 31 - __builtin_clz(tile_elems >> 8);  // blocks per tile = 2^log_b
    const uint32_t tiles_per_limb = 1u << (lr - log_b);
    const uint32_t lb = logical_block();
    BlocksGeom g;
    g.unit = decode_unit(a, lb / tiles_per_limb);
    const uint32_t tile = lb % tiles_per_limb;
    g.off = (size_t)tile * tile_elems;
    const uint32_t blk0 = tile << log_b;                   // first 256-block of this tile within the limb
    g.idx0 = (1u << lr) + blk0;
    g.idx1 = (1u << (lr + 4)) + (blk0 << 4);
    return g;
}

constexpr int kPer = 16;  // words per thread in the blocks pass
constexpr int kMaxGroup = 4;  // most jobs in one LimbGroup

// FP64 back end.  EPI compiles the fused forward epilogues in (they cost 64 registers).  Two waves per SIMD: with
// the epilogues the kernel needs 254 registers; left to itself the compiler spreads into the accumulation registers
// and a single wave, which costs a third more time (three waves would spill, and measure slower).
// GAL: the inverse pass gathers its input through a Galois permutation (a.in_galois); an instantiation of its own, so
// that the index arithmetic costs the other launches no registers
// TW_LDS (forward pass with an epilogue): the 30 twiddles of a thread live in LDS behind the tile instead of in 60
// registers, which leaves room for the next tile's words in registers while the current one is transformed and its
// epilogue operands travel: without it that fetch waits until the epilogue has stored, and every tile of the loop
// exposes one round trip to memory.  LDS: the tile (17 T words), 15 T / 16 words of the first block's twiddles (one set
// per 16 threads), 15 T of the second block's.
template <bool FWD, bool EPI, bool GAL, bool TW_LDS = false>
__device__ __forceinline__ void ntt_blocks_fp_body(const NttArgs &a, uint64_t *lds) {
    const uint32_t nthreads = blockDim.x;
    const BlocksGeom g = blocks_geom(a);
    const size_t off = g.off;
    const size_t n = (size_t)1 << a.log_n;
    double *ld = reinterpret_cast<double *>(lds);
    const bool fma_mode = EPI && a.epi_mode == NTT_EPI_FMA_SUB_MUL;   // ((a * pro_w + b) - v) * w
    const bool has_addend = EPI && (a.epi_mode == NTT_EPI_SUB_MUL_ADD || fma_mode);

    Job job = decode_job(a, g.unit.j0);
    if (a.unit_filter == 1 && !((a.fp_mask >> job.table) & 1)) return;   // (the whole workgroup: a unit has one prime)
    const FpCtx fc = fp_ctx(a, job.table);
    const FpMod m = fc.m;

    // this thread's group in either register pass, and its twiddles (the same for every limb of the unit)
    const uint32_t gi = threadIdx.x;
    const uint32_t base0 = ((gi >> 4) << 8) | (gi & 15);   // pass with stride 16
    const uint32_t base1 = gi << 4;                        // pass with stride 1
    double tw0[15], tw1[15];
    fp_load_block_tw<4>(tw0, fc.tw, g.idx0 + (gi >> 4));
    fp_load_block_tw<4>(tw1, fc.tw, g.idx1 + gi);
    double *ltw0 = ld + 17 * nthreads, *ltw1 = ltw0 + 15 * (nthreads >> 4);

    // list mode: the unit's jobs are read before the first store, so that they stay scalar loads
    LimbJob pre[kMaxGroup];
    const uint32_t item = a.jobs ? g.unit.j0 / a.n_jobs : 0;
    const uint32_t first = g.unit.j0 - item * (a.jobs ? a.n_jobs : 0);
#pragma unroll
    for (int i = 0; i < kMaxGroup; i++) pre[i] = (a.jobs && (uint32_t)i < g.unit.count) ? a.jobs[first + i] : LimbJob{0, 0};
    const size_t item_off = a.jobs ? item * a.item_stride : 0;
    auto entry = [&](uint32_t b) {
        if (!a.jobs) return decode_job(a, g.unit.j0 + b * g.unit.jstride);
        LimbJob lj = pre[0];
#pragma unroll
        for (int i = 1; i < kMaxGroup; i++) lj = b == (uint32_t)i ? pre[i] : lj;
        return Job{a.in + item_off + (size_t)lj.data_limb * n, a.out + item_off + (size_t)lj.data_limb * n, lj.table, 0, 0, nullptr};
    };

    uint64_t nx[kPer];
    auto stage = [&]() {  // prefetched words -> LDS
#pragma unroll
        for (int i = 0; i < kPer; i++) {
            const uint32_t e = threadIdx.x + i * nthreads;
            if (!FWD)
                ld[skew(e)] = fp_from_u64(nx[i]);
            else
                lds[skew(e)] = nx[i];
        }
        lds_barrier();
    };
    // inverse pass of a rotation: the input is sigma(in), gathered here (map mode only)
    const uint32_t in_elt = (FWD || !GAL) ? 0u : a.in_galois;
    auto fetch = [&](const Job &j) {
        const uint64_t *src = (FWD ? j.out : j.in) + off;  // the forward blocks pass continues on the rows pass's output
        if (!FWD && GAL && in_elt) {
#pragma unroll
            for (int i = 0; i < kPer; i++)
                nx[i] = j.in[galois_index((uint32_t)off + threadIdx.x + i * nthreads, in_elt, a.log_n)];
        } else {
#pragma unroll
            for (int i = 0; i < kPer; i++) nx[i] = src[threadIdx.x + i * nthreads];
        }
    };
    fetch(job);
    if (TW_LDS) {
        // (stride 15: the threads of a wave read their sets from distinct banks; 16 threads share a set of the first block)
#pragma unroll
        for (int i = 0; i < 15; i++) {
            if ((gi & 15) == 0) ltw0[(gi >> 4) * 15 + i] = tw0[i];
            ltw1[gi * 15 + i] = tw1[i];
        }
    } else {
        // the twiddles have arrived before the loop starts: inside it only the prefetch is in flight
#pragma unroll
        for (int i = 0; i < 15; i++) asm volatile("" ::"v"(tw0[i]), "v"(tw1[i]));
    }
    stage();

    for (uint32_t b = 0;; b++) {
        // the next limb's tile and this limb's epilogue operands travel while the butterflies run
        const bool more = b + 1 < g.unit.count;
        // (with a fused epilogue the registers go to its operands instead and the next tile is fetched late)
        Job next = job;
        if (more) next = entry(b + 1);
        if (more && (!EPI || TW_LDS)) fetch(next);
        const size_t epi_off = off + (size_t)job.limb * n;
        // SUB_MUL_ADD adds onto the polynomials named by epi_b_mask only (a rotation adds onto c0, not c1)
        const bool add_b = has_addend && (fma_mode || ((a.epi_b_mask >> (job.poly & 31)) & 1));
        uint64_t *dst = (FWD && EPI) ? a.epi_dst + (size_t)job.poly * a.epi_dst_poly_stride * n + epi_off : job.out + off;
        uint64_t pre_a[EPI ? kPer : 1], pre_b[EPI ? kPer : 1];
        if (FWD && EPI) {
            const uint64_t *minuend = a.epi_a + (size_t)job.poly * a.epi_a_poly_stride * n + epi_off;
            const uint64_t *addend = add_b ? a.epi_b + (size_t)job.poly * a.epi_b_poly_stride * n + epi_off : minuend;
#pragma unroll
            for (int i = 0; i < kPer; i++) pre_a[EPI ? i : 0] = minuend[threadIdx.x + i * nthreads];
#pragma unroll
            for (int i = 0; i < kPer; i++) pre_b[EPI ? i : 0] = addend[threadIdx.x + i * nthreads];
        }

        double v[16];
        if (FWD) {
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base0 + (j << 4))];
            if (TW_LDS) {
                double t[15];
#pragma unroll
                for (int i = 0; i < 15; i++) t[i] = ltw0[(gi >> 4) * 15 + i];
                fp_ct_block_tw<4, true>(v, t, m);
            } else {
                fp_ct_block_tw<4, true>(v, tw0, m);
            }
#pragma unroll
            for (int j = 0; j < 16; j++) ld[skew(base0 + (j << 4))] = v[j];
            lds_barrier();
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base1 + j)];
            if (TW_LDS) {
                double t[15];
#pragma unroll
                for (int i = 0; i < 15; i++) t[i] = ltw1[gi * 15 + i];
                fp_ct_block_tw<4, true>(v, t, m);
            } else {
                fp_ct_block_tw<4, true>(v, tw1, m);
            }
#pragma unroll
            for (int j = 0; j < 16; j++) ld[skew(base1 + j)] = v[j];
            lds_barrier();
#pragma unroll
            // (an epilogue subtracts the word as the second block left it, at most 5.3 q in magnitude: its difference from
            // a minuend below 1.9 q stays below 2^53 and goes through one modular product)
            for (int i = 0; i < kPer; i++) v[i] = EPI ? ld[skew(threadIdx.x + i * nthreads)] : fp_canonical(ld[skew(threadIdx.x + i * nthreads)], m);
            if (EPI) {
                const double wd = fp_from_u64(a.w[2 * job.limb]);
                const FpTw w{wd, wd * m.qinv};
                if (fma_mode) {
                    const double pd = fp_from_u64(a.pro_w[2 * job.limb]);
                    const FpTw pw{pd, pd * m.qinv};
#pragma unroll
                    for (int i = 0; i < kPer; i++) {
                        const double lhs = fp_mulmod(fp_from_u64(pre_a[EPI ? i : 0]), pw, m) + fp_from_u64(pre_b[EPI ? i : 0]);
                        v[i] = fp_canonical(fp_mulmod(lhs - v[i], w, m), m);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < kPer; i++) {
                        double r = fp_mulmod(fp_from_u64(pre_a[EPI ? i : 0]) - v[i], w, m);
                        if (add_b) r += fp_from_u64(pre_b[EPI ? i : 0]);
                        v[i] = fp_canonical(r, m);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < kPer; i++) dst[threadIdx.x + i * nthreads] = fp_to_u64(v[i]);
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base1 + j)];
            fp_gs_block_tw<4, false>(v, tw1, m);
#pragma unroll
            for (int j = 0; j < 16; j++) ld[skew(base1 + j)] = v[j];
            lds_barrier();
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ld[skew(base0 + (j << 4))];
            fp_gs_block_tw<4, true>(v, tw0, m);
#pragma unroll
            for (int j = 0; j < 16; j++) ld[skew(base0 + (j << 4))] = v[j];
            lds_barrier();
            // lazy signed doubles go to the rows pass
            uint64_t o[kPer];
#pragma unroll
            for (int i = 0; i < kPer; i++) o[i] = lds[skew(threadIdx.x + i * nthreads)];
#pragma unroll
            for (int i = 0; i < kPer; i++) dst[threadIdx.x + i * nthreads] = o[i];
        }
        if (!more) break;
        if (EPI && !TW_LDS) fetch(next);
        lds_barrier();  // every read of this tile is done before the next one overwrites it
        stage();
        job = next;
    }
}

template <bool FWD, bool EPI, bool GAL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void ntt_blocks_fp_kernel(NttArgs a) {
    __shared__ uint64_t lds[kLdsWords];
    ntt_blocks_fp_body<FWD, EPI, GAL>(a, lds);
}

// the forward pass with an epilogue: twiddles in LDS (blocks_epi_lds_bytes of dynamic LDS)
extern __shared__ uint64_t dyn_lds[];
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void ntt_blocks_fp_epi_kernel(NttArgs a) {
    ntt_blocks_fp_body<true, true, false, true>(a, dyn_lds);
}
inline size_t blocks_epi_lds_bytes(uint32_t threads) { return 8 * (size_t)(17 * threads + 15 * (threads >> 4) + 15 * threads); }

// Forward blocks pass of ModUp fused with the key-switch inner product.  Workgroup = (limb t of Ql u P, tile of
// 16 T words): its first T threads transform that tile of every digit in turn; all 2 T threads then multiply
// it by a key polynomial (threads below T by the first, the others by the second) and accumulate in registers.
// The key tiles are fetched before the butterflies start, so that they travel meanwhile; the digit that owns
// limb t contributes the input itself.
template <uint32_t T>
__global__ __launch_bounds__(2 * T) __attribute__((amdgpu_waves_per_eu(2))) void ntt_blocks_fp_inner_kernel(NttArgs a, KsFuseArgs x) {
    constexpr uint32_t kInnerTile = 16 * T + T;   // words of one skewed tile
    __shared__ uint64_t lds[2 * kInnerTile];
    constexpr uint32_t half = T, tile_elems = half << 4;
    const uint32_t role = threadIdx.x >= half ? 1u : 0u;       // which key polynomial this thread accumulates
    const uint32_t tid = threadIdx.x - role * half;
    const uint32_t lr = a.log_n - 8;
    const uint32_t log_b = 31 - __builtin_clz(tile_elems >> 8);
    const uint32_t tiles_per_limb = 1u << (lr - log_b);
    const uint32_t LK = x.L + x.K;
    const size_t n = (size_t)1 << a.log_n;
    uint32_t lb, item = 0;
    if (x.items > 1) {
        // hardware id -> XCD id & 7; inside an XCD the items of one (limb, tile) are consecutive
        const uint32_t pairs = LK * tiles_per_limb, id = blockIdx.x;
        if (pairs % 8 == 0) {
            const uint32_t s = id >> 3;
            item = s % x.items;
            lb = (s / x.items) * 8 + (id & 7);
        } else {
            item = id / pairs;
            lb = id - item * pairs;
        }
    } else {
        // plain order, last limb first: the special limbs have one digit more to transform than the others, so their
        // workgroups start first and are spread over all XCDs (a tile's twiddles are its own: nothing to share)
        lb = gridDim.x - 1 - blockIdx.x;
    }
    const uint32_t t = lb / tiles_per_limb, tile = lb % tiles_per_limb;
    const size_t off = (size_t)tile * tile_elems;
    const uint32_t blk0 = tile << log_b;
    const uint32_t table = t < x.L ? t : x.size_q + (t - x.L);
    const uint32_t own = t < x.L ? t / x.K : 0xffffffffu;
    // (locals: a modified copy of the argument structs would move their pointer tables to scratch memory)
    const uint64_t *own_base = x.own + item * x.own_item_stride;
    const uint64_t *lazy_base = a.out + item * a.item_stride;
    uint64_t *out_base = x.out + item * (2 * (size_t)LK * n);
    const uint64_t *fold_base = x.fold_ct ? x.fold_ct + item * x.fold_item_stride : nullptr;
    double *ld = reinterpret_cast<double *>(lds);
    const FpCtx fc = fp_ctx(a, table);
    const FpMod m = fc.m;

    const uint32_t base0 = ((tid >> 4) << 8) | (tid & 15);
    const uint32_t base1 = tid << 4;
    // the twiddles stay in the table (the digits after the first find them in cache)
    const uint32_t idx0 = (1u << lr) + blk0 + (tid >> 4), idx1 = (1u << (lr + 4)) + (blk0 << 4) + tid;

    // the 15 + 15 twiddles of the two register blocks are the same for every digit: loaded once, ahead of everything
    // else (fetched inside the blocks they would each cost a round trip to L2 that nothing covers)
    double twA[15], twB[15];
    fp_load_block_tw<4>(twA, fc.tw, idx0);
    fp_load_block_tw<4>(twB, fc.tw, idx1);

    const size_t key_off = ((size_t)role * x.size_qp + table) * n + off;
    double acc[kPer];
    if (own != 0xffffffffu) {
        const uint64_t *src = own_base + (size_t)t * n;
        const uint64_t *key = x.evk.p[own] + key_off;
        uint64_t c[kPer];
        if (x.own_galois) {
#pragma unroll
            for (int i = 0; i < kPer; i++) c[i] = src[galois_index((uint32_t)off + tid + i * half, x.own_galois, a.log_n)];
        } else {
#pragma unroll
            for (int i = 0; i < kPer; i++) c[i] = src[(uint32_t)off + tid + i * half];
        }
#pragma unroll
        for (int i = 0; i < kPer; i++) {
            const double w = fp_from_u64(key[tid + i * half]);
            acc[i] = fp_mulmod(fp_from_u64(c[i]), FpTw{w, w * m.qinv}, m);
        }
    } else {
#pragma unroll
        for (int i = 0; i < kPer; i++) acc[i] = 0.0;
    }

    // The other digits two at a time: the threads of role 0 transform the first one's tile, those of role 1 the
    // second one's (each into its own LDS tile, the same sequence of steps at the same time), then every thread
    // multiplies both tiles by its key polynomial.  With the transforms on one role only, half of the workgroup's
    // waves (and the SIMDs they sit on) would idle during the butterflies.
    auto skip_own = [&](uint32_t d) { return d == own ? d + 1 : d; };
    for (uint32_t da = skip_own(0); da < x.beta;) {
        const uint32_t db = skip_own(da + 1);
        const bool two = db < x.beta;
        const uint32_t mine = role ? db : da;
        const bool work = role ? two : true;
        // key words of the first digit are requested before the butterflies, those of the second after them (they
        // arrive while the first tile is multiplied): both sets up front would not fit the register file
        uint64_t pka[kPer], pkb[kPer];
        const uint64_t *ka = x.evk.p[da] + key_off, *kb = x.evk.p[two ? db : da] + key_off;
#pragma unroll
        for (int i = 0; i < kPer; i++) pka[i] = ka[tid + i * half];
        double *ldm = ld + role * kInnerTile;
        const uint64_t *src = lazy_base + ((size_t)mine * LK + t) * n + off;  // lazy values left by the rows pass
        if (work) {
            // the 16 words of the first register block (stride 16 inside a 256-block) straight from global memory:
            // 16 neighbouring threads read one 128-byte line per access
            double v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = __longlong_as_double((long long)src[base0 + (j << 4)]);
            fp_ct_block_tw<4, true>(v, twA, m);
#pragma unroll
            for (int j = 0; j < 16; j++) ldm[skew(base0 + (j << 4))] = v[j];
        }
        lds_barrier();
#pragma unroll
        for (int i = 0; i < kPer / 2; i++) pkb[i] = kb[tid + i * half];
        if (work) {
            double v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = ldm[skew(base1 + j)];
            fp_ct_block_tw<4, true>(v, twB, m);
#pragma unroll
            for (int j = 0; j < 16; j++) ldm[skew(base1 + j)] = v[j];
        }
#pragma unroll
        for (int i = kPer / 2; i < kPer; i++) pkb[i] = kb[tid + i * half];
        lds_barrier();
        // The transformed words go into the products as the second block leaves them (at most 5.3 q in magnitude):
        // each term is then at most (1/2 + 0.375 x 5.3) q < 2.5 q, and an accumulator that starts a pair below q ends
        // it below 6 q < 2^53; one reduction per pair instead of one per word and digit.
#pragma unroll
        for (int i = 0; i < kPer; i++) {
            const double w = fp_from_u64(pka[i]);
            acc[i] += fp_mulmod(ld[skew(tid + i * half)], FpTw{w, w * m.qinv}, m);
        }
        if (two) {
#pragma unroll
            for (int i = 0; i < kPer; i++) {
                const double w = fp_from_u64(pkb[i]);
                acc[i] += fp_mulmod(ld[kInnerTile + skew(tid + i * half)], FpTw{w, w * m.qinv}, m);
            }
        }
#pragma unroll
        for (int i = 0; i < kPer; i++) acc[i] = fp_reduce(acc[i], m);
        lds_barrier();  // every read of these tiles is done before the next pair overwrites them
        da = skip_own(db + 1);
    }
    if (x.add_c0 && !role && t < x.L) {
        // a rotation: polynomial 0 gains P sigma(c0), which ModDown's division by P turns into sigma(c0)
        const uint64_t *c0 = x.add_c0 + (size_t)t * n;
        const double pd = fp_from_u64(x.p_mod_q[2 * t]);
        const FpTw pw{pd, pd * m.qinv};
#pragma unroll
        for (int i = 0; i < kPer; i++) {
            const uint32_t e = (uint32_t)off + tid + i * half;
            acc[i] += fp_mulmod(fp_from_u64(c0[x.own_galois ? galois_index(e, x.own_galois, a.log_n) : e]), pw, m);
        }
    }
    uint64_t *o = out_base + ((size_t)role * LK + t) * n + off;
    if (fold_base && t == x.L - 1) {
        const uint64_t *cl = fold_base + ((size_t)role * x.L + t) * n + off;
        const double wd = fp_from_u64(x.fold_w[0]);
        const FpTw w{wd, wd * m.qinv};
#pragma unroll
        for (int i = 0; i < kPer; i++)
            acc[i] = fp_mulmod(fp_canonical(acc[i], m), w, m) + fp_from_u64(cl[tid + i * half]);
    }
#pragma unroll
    for (int i = 0; i < kPer; i++) o[tid + i * half] = fp_to_u64(fp_canonical(acc[i], m));
}

// Tensor product fused with the blocks pass of the inverse transform of its third polynomial (FP64 back end, one
// workgroup per (limb, tile of 16 T words)): (d0, d1, d2) = (a0 b0, a0 b1 + a1 b0, a1 b1) from the four input tiles,
// all three written as canonical residues (d2 in NTT form is what the key switch multiplies by its own digit's key),
// and d2 goes on through the 8 inverse stages inside 256 consecutive words; the lazy words are left in a.out for the
// rows pass.  One read of d2 and one launch less than tensor kernel + inverse transform.
template <bool SQUARE>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1))) void tensor_intt_blocks_fp_kernel(NttArgs a, TensorFuse x) {
    __shared__ uint64_t lds[kLdsWords];
    double *ld = reinterpret_cast<double *>(lds);
    const uint32_t nthreads = blockDim.x;
    const BlocksGeom g = blocks_geom(a);
    const Job job = decode_job(a, g.unit.j0);
    const FpCtx fc = fp_ctx(a, job.table);
    const FpMod m = fc.m;
    const size_t n = (size_t)1 << a.log_n;
    const uint32_t gi = threadIdx.x;
    const uint32_t base0 = ((gi >> 4) << 8) | (gi & 15);
    const uint32_t base1 = gi << 4;
    double tw0[15], tw1[15];
    fp_load_block_tw<4>(tw0, fc.tw, g.idx0 + (gi >> 4));
    fp_load_block_tw<4>(tw1, fc.tw, g.idx1 + gi);

    const size_t lo = (size_t)job.limb * n + g.off, poly = (size_t)x.L * n;
    // the launch has 1.5 waves per SIMD at N = 2^16, L = 24: all 64 loads of a thread are in flight at once
#pragma unroll
    for (int i = 0; i < kPer; i++) {
        const uint32_t e = threadIdx.x + i * nthreads;
        const double a0 = fp_from_u64(x.ct1[lo + e]), a1 = fp_from_u64(x.ct1[poly + lo + e]);
        double d0, d1, d2;
        if (SQUARE) {
            d0 = fp_canonical(fp_mulmod(a0, FpTw{a0, a0 * m.qinv}, m), m);
            d2 = fp_canonical(fp_mulmod(a1, FpTw{a1, a1 * m.qinv}, m), m);
            const double mm = fp_mulmod(a0, FpTw{a1, a1 * m.qinv}, m);
            d1 = fp_canonical(mm + mm, m);
        } else {
            const double b0 = fp_from_u64(x.ct2[lo + e]), b1 = fp_from_u64(x.ct2[poly + lo + e]);
            d0 = fp_canonical(fp_mulmod(a0, FpTw{b0, b0 * m.qinv}, m), m);
            d2 = fp_canonical(fp_mulmod(a1, FpTw{b1, b1 * m.qinv}, m), m);
            // Karatsuba: (a0 + a1)(b0 + b1) - d0 - d2; both factors are below 2 q, the product is reduced to
            // |r| <= 2 q and the difference stays below 4 q < 2^53
            const double sb = b0 + b1;
            const double mm = fp_mulmod(a0 + a1, FpTw{sb, sb * m.qinv}, m);
            d1 = fp_canonical(mm - d0 - d2, m);
        }
        x.d01[lo + e] = fp_to_u64(d0);
        x.d01[poly + lo + e] = fp_to_u64(d1);
        x.d2[lo + e] = fp_to_u64(d2);
        ld[skew(e)] = d2;
    }
#pragma unroll
    for (int i = 0; i < 15; i++) asm volatile("" ::"v"(tw0[i]), "v"(tw1[i]));
    lds_barrier();
    double v[16];
#pragma unroll
    for (int j = 0; j < 16; j++) v[j] = ld[skew(base1 + j)];
    fp_gs_block_tw<4, false>(v, tw1, m);
#pragma unroll
    for (int j = 0; j < 16; j++) ld[skew(base1 + j)] = v[j];
    lds_barrier();
#pragma unroll
    for (int j = 0; j < 16; j++) v[j] = ld[skew(base0 + (j << 4))];
    fp_gs_block_tw<4, true>(v, tw0, m);
#pragma unroll
    for (int j = 0; j < 16; j++) ld[skew(base0 + (j << 4))] = v[j];
    lds_barrier();
    // lazy signed doubles go to the rows pass
    uint64_t *dst = job.out + g.off;
    uint64_t o[kPer];
#pragma unroll
    for (int i = 0; i < kPer; i++) o[i] = lds[skew(threadIdx.x + i * nthreads)];
#pragma unroll
    for (int i = 0; i < kPer; i++) dst[threadIdx.x + i * nthreads] = o[i];
}

// Integer back end (twiddles stay in the table: 30 Shoup pairs per thread do not fit in registers).  Three waves
// per SIMD (168 registers, 24 bytes of spill in the forward kernel) hide the latency of the epilogue's operand loads
// better than the two waves that 196 registers allow.
// PRE: the operands of a fused epilogue are requested together with the tile, so that they travel while the
// butterflies run (32 more registers: for the mixed kernel, which is compiled for two waves per SIMD and serves the
// small launches, where nothing else covers that round trip).
template <bool FWD, bool GAL, bool PRE = false>
__device__ __forceinline__ void ntt_blocks_int_body(const NttArgs &a, uint64_t *lds) {
    const uint32_t nthreads = blockDim.x;
    const uint32_t tile_elems = nthreads << 4;
    const BlocksGeom g = blocks_geom(a);
    const size_t off = g.off;
    const size_t n = (size_t)1 << a.log_n;
    const bool fma_mode = FWD && a.epi_mode == NTT_EPI_FMA_SUB_MUL;
    const bool epi = FWD && (a.epi_mode == NTT_EPI_SUB_MUL || a.epi_mode == NTT_EPI_SUB_MUL_ADD || fma_mode);
    const bool has_addend = FWD && (a.epi_mode == NTT_EPI_SUB_MUL_ADD || fma_mode);

    if (a.unit_filter == 2 && ((a.fp_mask >> decode_job(a, g.unit.j0).table) & 1)) return;
    for (uint32_t b = 0; b < g.unit.count; b++) {
        const Job job = decode_job(a, g.unit.j0 + b * g.unit.jstride);
        const IntCtx ic = int_ctx(a, job.table);
        const uint64_t q = ic.q;
        const uint64_t *src = (FWD ? job.out : job.in) + off;
        if (!FWD && GAL && a.in_galois) {
#pragma unroll
            for (int i = 0; i < kPer; i++)
                lds[skew(threadIdx.x + i * nthreads)] = job.in[galois_index((uint32_t)off + threadIdx.x + i * nthreads, a.in_galois, a.log_n)];
        } else {
#pragma unroll
            for (int i = 0; i < kPer; i++) lds[skew(threadIdx.x + i * nthreads)] = src[threadIdx.x + i * nthreads];
        }
        const size_t epi_off = off + (size_t)job.limb * n;
        const uint64_t *minuend = epi ? a.epi_a + (size_t)job.poly * a.epi_a_poly_stride * n + epi_off : nullptr;
        const bool add_b = has_addend && (fma_mode || ((a.epi_b_mask >> (job.poly & 31)) & 1));
        const uint64_t *addend = add_b ? a.epi_b + (size_t)job.poly * a.epi_b_poly_stride * n + epi_off : minuend;
        uint64_t pre_a[PRE ? kPer : 1], pre_b[PRE ? kPer : 1];
        if (PRE && epi) {
#pragma unroll
            for (int i = 0; i < kPer; i++) pre_a[PRE ? i : 0] = minuend[threadIdx.x + i * nthreads];
#pragma unroll
            for (int i = 0; i < kPer; i++) pre_b[PRE ? i : 0] = addend[threadIdx.x + i * nthreads];
        }
        __syncthreads();
        if (FWD) {
            tile_pass<4, true>(lds, tile_elems, 4, g.idx0, ic);
            __syncthreads();
            tile_pass<4, true>(lds, tile_elems, 0, g.idx1, ic);
            __syncthreads();
            if (epi) {
                uint64_t *dst = a.epi_dst + (size_t)job.poly * a.epi_dst_poly_stride * n + epi_off;
                const Shoup w = load_shoup(a.w, job.limb);
                const Shoup pw = fma_mode ? load_shoup(a.pro_w, job.limb) : w;
#pragma unroll
                for (int i = 0; i < kPer; i++) {
                    const uint32_t e = threadIdx.x + i * nthreads;
                    const uint64_t c = reduce_4q(lds[skew(e)], q);
                    const uint64_t ma = PRE ? pre_a[PRE ? i : 0] : minuend[e];
                    uint64_t r;
                    if (fma_mode) {
                        const uint64_t mb = PRE ? pre_b[PRE ? i : 0] : addend[e];
                        r = mul_shoup(sub_mod(add_mod(mul_shoup(ma, pw, q), mb, q), c, q), w, q);
                    } else {
                        r = mul_shoup(sub_mod(ma, c, q), w, q);
                        if (add_b) r = add_mod(r, PRE ? pre_b[PRE ? i : 0] : addend[e], q);
                    }
                    dst[e] = r;
                }
            } else {
#pragma unroll
                for (int i = 0; i < kPer; i++) {
                    const uint32_t e = threadIdx.x + i * nthreads;
                    job.out[off + e] = reduce_4q(lds[skew(e)], q);
                }
            }
        } else {
            tile_pass<4, false>(lds, tile_elems, 0, g.idx1, ic);
            __syncthreads();
            tile_pass<4, false>(lds, tile_elems, 4, g.idx0, ic);
            __syncthreads();
            // lazy values in [0, 2q) go to the rows pass
#pragma unroll
            for (int i = 0; i < kPer; i++) {
                const uint32_t e = threadIdx.x + i * nthreads;
                job.out[off + e] = lds[skew(e)];
            }
        }
        __syncthreads();  // every read of this tile is done before the next one overwrites it
    }
}

template <bool FWD, bool GAL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void ntt_blocks_int_kernel(NttArgs a) {
    __shared__ uint64_t lds[kLdsWords];
    ntt_blocks_int_body<FWD, GAL>(a, lds);
}

// Mixed back end: the limbs of a unit share a modulus, so the whole workgroup takes one branch.  EPI as in
// ntt_blocks_fp_kernel: the FP64 body compiled with the fused epilogues addresses their operands unconditionally,
// so it is only launched when the launch has an epilogue.
template <bool FWD, bool EPI, bool GAL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void ntt_blocks_mixed_kernel(NttArgs a) {
    __shared__ uint64_t lds[kLdsWords];
    const Job first = decode_job(a, blocks_geom(a).unit.j0);
    if ((a.fp_mask >> first.table) & 1)
        ntt_blocks_fp_body<FWD, EPI, GAL>(a, lds);
    else
        ntt_blocks_int_body<FWD, GAL, FWD && EPI>(a, lds);
}

template <bool FWD, int FP>
hipError_t launch_rows(const NttArgs &a, uint32_t n_jobs, hipStream_t s) {
    const int ld = (int)a.log_n - 8;
    auto grid = [&](int ldv, int tl) {
        int logc = (tl - ldv) < 8 ? (tl - ldv) : 8;
        return dim3(n_jobs * (256u >> logc));
    };
    // small launches (fewer 4096-word tiles than CUs) are bound by the latency of one workgroup: quarter tiles
    const bool small = ld >= 5 && n_jobs * (256u >> (kTileLog - ld < 8 ? kTileLog - ld : 8)) < 256;
    if (a.pro_mode == NTT_PRO_SOURCE_INTT_REDUCE) {
        // one instantiation per degree, on quarter tiles, which follows fp_mask limb by limb: the mask stands for the
        // launch's back end here
        if (!FWD || !ntt_source_intt_ok(a.log_n, n_jobs, 0) || !a.pro_itw || (a.pro_src_fp_mask && !a.pro_itw_fp))
            return hipErrorInvalidValue;
        NttArgs b = a;
        b.fp_mask = FP == NTT_BACKEND_INT ? 0 : (FP == NTT_BACKEND_FP ? ~(uint64_t)0 : a.fp_mask);
        if (ld == 7)
            hipLaunchKernelGGL((ntt_rows_kernel<7, true, NTT_BACKEND_MIXED, 10, true>), grid(7, 10), dim3(64), 0, s, b);
        else
            hipLaunchKernelGGL((ntt_rows_kernel<8, true, NTT_BACKEND_MIXED, 10, true>), grid(8, 10), dim3(64), 0, s, b);
        return hipGetLastError();
    }
    switch (ld) {
#define HE_CASE(LD)                                                                               \
    case LD:                                                                                      \
        hipLaunchKernelGGL((ntt_rows_kernel<LD, FWD, FP, 12>), grid(LD, 12), dim3(256), 0, s, a); \
        break;
#define HE_CASE2(LD)                                                                                  \
    case LD:                                                                                          \
        if (small)                                                                                    \
            hipLaunchKernelGGL((ntt_rows_kernel<LD, FWD, FP, 10>), grid(LD, 10), dim3(64), 0, s, a);  \
        else                                                                                          \
            hipLaunchKernelGGL((ntt_rows_kernel<LD, FWD, FP, 12>), grid(LD, 12), dim3(256), 0, s, a); \
        break;
        HE_CASE(1) HE_CASE(2) HE_CASE(3) HE_CASE(4) HE_CASE2(5) HE_CASE2(6) HE_CASE2(7) HE_CASE2(8) HE_CASE(9)
#undef HE_CASE
#undef HE_CASE2
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Geometry of the blocks pass: polynomials per unit (map mode) and workgroup size, chosen so that the grid
// still fills 256 CUs a few times over.
struct BlocksPlan {
    uint32_t batch, threads, grid;
};

BlocksPlan plan_blocks(const NttArgs &a, uint32_t n_polys) {
    const uint32_t n = 1u << a.log_n;
    // threads of a workgroup for a wished tile of `want` words (a limb may be smaller than that)
    auto threads = [&](uint32_t want) { return (n < want ? n : want) >> 4; };
    auto tiles = [&](uint32_t want) { return n / (threads(want) << 4); };
    BlocksPlan p;
    uint32_t units;
    if (a.jobs) {
        p.batch = 1;
        units = a.n_groups * (a.items ? a.items : 1);
    } else {
        // batching pays once the launch has enough workgroups without splitting the polynomials
        p.batch = (n_polys > 1 && a.map.limbs * tiles(2048) >= 512) ? n_polys : 1;
        units = a.map.limbs * ((n_polys + p.batch - 1) / p.batch);
    }
    const uint32_t want = units * tiles(4096) >= 1024 ? 4096 : (units * tiles(2048) >= 256 ? 2048 : 1024);
    p.threads = threads(want);
    p.grid = units * tiles(want);
    return p;
}

constexpr uint32_t kSplitMixedGrid = 1024;   // workgroups from which a mixed blocks pass runs as two kernels

template <bool FWD, int FP>
hipError_t launch_blocks(NttArgs a, uint32_t n_polys, hipStream_t s) {
    const BlocksPlan p = plan_blocks(a, n_polys);
    a.batch = p.batch;
    a.n_polys = n_polys;
    const bool epi = FWD && (a.epi_mode == NTT_EPI_SUB_MUL || a.epi_mode == NTT_EPI_SUB_MUL_ADD ||
                             a.epi_mode == NTT_EPI_FMA_SUB_MUL);
    // the Galois gather of an inverse pass's input lives in instantiations of its own
    const bool gal = !FWD && a.in_galois != 0 && !a.jobs;
    const dim3 grid(p.grid), block(p.threads);
    if (FP == NTT_BACKEND_MIXED && p.grid >= kSplitMixedGrid) {
        // A large mixed launch runs as two kernels over the same grid, each leaving the other's units at once: the
        // integer body then has its own three waves per SIMD (the mixed kernel is compiled for the FP64 body's
        // registers: two), which its unpipelined load -> butterflies -> store sequence needs.
        a.unit_filter = 1;
        if (gal)
            hipLaunchKernelGGL((ntt_blocks_fp_kernel<false, false, true>), grid, block, 0, s, a);
        else if (epi)
            hipLaunchKernelGGL((ntt_blocks_fp_kernel<FWD, FWD, false>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((ntt_blocks_fp_kernel<FWD, false, false>), grid, block, 0, s, a);
        a.unit_filter = 2;
        if (gal)
            hipLaunchKernelGGL((ntt_blocks_int_kernel<false, true>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((ntt_blocks_int_kernel<FWD, false>), grid, block, 0, s, a);
        return hipGetLastError();
    }
    if (gal) {
        if (FP == NTT_BACKEND_MIXED)
            hipLaunchKernelGGL((ntt_blocks_mixed_kernel<false, false, true>), grid, block, 0, s, a);
        else if (!FP)
            hipLaunchKernelGGL((ntt_blocks_int_kernel<false, true>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((ntt_blocks_fp_kernel<false, false, true>), grid, block, 0, s, a);
    } else if (FP == NTT_BACKEND_MIXED && epi)
        hipLaunchKernelGGL((ntt_blocks_mixed_kernel<FWD, FWD, false>), grid, block, 0, s, a);
    else if (FP == NTT_BACKEND_MIXED)
        hipLaunchKernelGGL((ntt_blocks_mixed_kernel<FWD, false, false>), grid, block, 0, s, a);
    else if (!FP)
        hipLaunchKernelGGL((ntt_blocks_int_kernel<FWD, false>), grid, block, 0, s, a);
    else if (epi)
        hipLaunchKernelGGL(ntt_blocks_fp_epi_kernel, grid, block, blocks_epi_lds_bytes(p.threads), s, a);
    else
        hipLaunchKernelGGL((ntt_blocks_fp_kernel<FWD, false, false>), grid, block, 0, s, a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_bconv_rows(const NttArgs &a, const BconvRows &b, const Tuning &tune, hipStream_t s) {
    if (a.log_n < 12 || a.log_n > 16 || !b.mat_fp || b.n_units == 0) return hipErrorInvalidValue;
    const uint32_t forced = tune.fuse_rows_forced <= kFuseMaxRows ? tune.fuse_rows_forced : 0;
    const uint32_t items = b.items ? b.items : 1;
    const int ld = (int)a.log_n - 8;
    const uint32_t tiles = 256u >> (kFuseLog - ld);
    const uint32_t rows = b.mdr ? b.max_rows - 1 : b.max_rows;
    if (rows == 0) return hipErrorInvalidValue;
    // Output limbs per workgroup.  The kernel is bound by instruction issue, so a CU's time is the number of workgroups
    // it is dealt times a workgroup's work: r rows plus about 1.5 rows' worth of fetching and converting its 8 x 8 block
    // of inputs and setting up.  Few rows per workgroup pay that overhead often, many leave CUs with one workgroup more
    // than others; the count that minimises ceil(workgroups / CUs) x (r + 1.5) matches the measured order at N = 2^16
    // (one operation: 3 and 6 equal, 4 and 8 slower; 8 operations: 207, 179, 168 us at 3, 8, 12 rows).  A CU with a
    // single workgroup has one wave per SIMD and nothing to cover its waits with (ModDown of one operation: 24.2 us in
    // 256 workgroups of 6 rows against 22.5 us in 512 of 3), so fewer than two per CU count as two.
    // the matrix-core kernel (N = 2^16) takes the output rows four at a time
    // (merged ModDown + rescale: the matrix-core kernel first forms the rescale term for its whole tile, two rows' worth of
    // work that pays once a workgroup has many rows, i.e. once the launch fills the chip without splitting the rows:
    // 98 against 114 us for 8 operations, 27.8 against 25.3 us for one)
    const bool mx = ld == 8 && b.mx_tab && !tune.no_matrix_bconv &&
                    (!b.mdr || (b.mx_last && (uint64_t)b.n_units * items * tiles >= (tune.cus ? tune.cus : 256)));
    const uint32_t step = mx ? 4 : 1;
    uint32_t target = mx ? (forced + 3) / 4 * 4 : forced;
    if (!target) {
        const uint32_t cus = tune.cus ? tune.cus : 256;
        uint64_t best = ~0ull;
        for (uint32_t r = step; r <= kFuseMaxRows && r < rows + step; r += step) {
            const uint64_t wgs = (uint64_t)b.n_units * items * tiles * ((rows + r - 1) / r);
            const uint64_t per_cu = (wgs + cus - 1) / cus;
            const uint64_t cost = (per_cu < 2 ? 2 : per_cu) * (2 * r + 3);
            if (cost < best) {
                best = cost;
                target = r;
            }
        }
    }
    BconvRowsK p{b, (rows + target - 1) / target, 0, target};
    p.copy_groups = b.copy_base ? (b.max_copy + target - 1) / target : 0;
    const uint64_t wgs = (uint64_t)b.n_units * items * tiles * (p.compute_groups + p.copy_groups);
    if (wgs > 0x7fffffffu) return hipErrorInvalidValue;
    const dim3 grid((uint32_t)wgs);
    if (mx) {
        if (b.mdr)
            hipLaunchKernelGGL(bconv_rows_mx_kernel<true>, grid, dim3(256), 0, s, a, p);
        else
            hipLaunchKernelGGL(bconv_rows_mx_kernel<false>, grid, dim3(256), 0, s, a, p);
        return hipGetLastError();
    }
    switch (ld) {
#define HE_CASE(LD) \
    case LD: hipLaunchKernelGGL((bconv_rows_fp_kernel<LD, 8>), grid, dim3(kFuseWords / 8), 0, s, a, p); break;
        HE_CASE(4) HE_CASE(5) HE_CASE(6) HE_CASE(7) HE_CASE(8)
#undef HE_CASE
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_ntt_forward(const NttArgs &a, uint32_t n_polys, int backend, hipStream_t s, bool rows_done) {
    if (a.log_n < 9 || a.log_n > 17 || backend < NTT_BACKEND_INT || backend > NTT_BACKEND_MIXED) return hipErrorInvalidValue;
    const uint32_t n_jobs = a.jobs ? a.n_jobs * (a.items ? a.items : 1) : n_polys * a.map.limbs;
    if (n_jobs == 0) return hipSuccess;
    if (!rows_done && one_pass_ok(a, backend, true, n_jobs)) return launch_limb_fp<true>(a, n_jobs, s);
    hipError_t e = rows_done                    ? hipSuccess
                   : backend == NTT_BACKEND_MIXED ? launch_rows<true, NTT_BACKEND_MIXED>(a, n_jobs, s)
                   : backend                    ? launch_rows<true, NTT_BACKEND_FP>(a, n_jobs, s)
                                                : launch_rows<true, NTT_BACKEND_INT>(a, n_jobs, s);
    if (e != hipSuccess) return e;
    return backend == NTT_BACKEND_MIXED ? launch_blocks<true, NTT_BACKEND_MIXED>(a, n_polys, s)
           : backend                    ? launch_blocks<true, NTT_BACKEND_FP>(a, n_polys, s)
                                        : launch_blocks<true, NTT_BACKEND_INT>(a, n_polys, s);
}

hipError_t launch_ntt_forward_inner(const NttArgs &a, const KsFuseArgs &x, hipStream_t s, bool rows_done) {
    if (a.log_n < 9 || a.log_n > 17 || !a.jobs) return hipErrorInvalidValue;
    const uint32_t items = x.items ? x.items : 1;
    if (items > 1 && (x.own_galois || x.add_c0 || (a.items ? a.items : 1) != items)) return hipErrorInvalidValue;
    if (a.n_jobs && !rows_done) {
        hipError_t e = launch_rows<true, NTT_BACKEND_FP>(a, a.n_jobs * items, s);
        if (e != hipSuccess) return e;
    }
    const uint32_t n = 1u << a.log_n;
    // tiles of 1024 words (workgroups of two waves, four of them on a CU): 229 us against 244 us with 2048-word tiles
    // for 8 x (24 + 8) limbs of 2^16 words, 39.7 against 42.8 us for one ciphertext's; 512-word tiles measure the same
    const uint32_t tile = n < 1024 ? n : 1024;
    if ((uint64_t)(x.L + x.K) * (n / tile) * items > 0x7fffffffu) return hipErrorInvalidValue;
    const dim3 grid((x.L + x.K) * (n / tile) * items);
    if (tile == 1024)
        hipLaunchKernelGGL(ntt_blocks_fp_inner_kernel<64>, grid, dim3(128), 0, s, a, x);
    else
        hipLaunchKernelGGL(ntt_blocks_fp_inner_kernel<32>, grid, dim3(64), 0, s, a, x);
    return hipGetLastError();
}

hipError_t launch_tensor_intt_blocks(NttArgs a, const TensorFuse &x, hipStream_t s) {
    if (a.log_n < 9 || a.log_n > 17 || a.jobs || a.map.limbs != x.L || x.L == 0) return hipErrorInvalidValue;
    const BlocksPlan p = plan_blocks(a, 1);
    a.batch = 1;
    a.n_polys = 1;
    if (x.square)
        hipLaunchKernelGGL(tensor_intt_blocks_fp_kernel<true>, dim3(p.grid), dim3(p.threads), 0, s, a, x);
    else
        hipLaunchKernelGGL(tensor_intt_blocks_fp_kernel<false>, dim3(p.grid), dim3(p.threads), 0, s, a, x);
    return hipGetLastError();
}

bool ntt_source_intt_ok(uint32_t log_n, uint32_t n_jobs, uint32_t n_tables) {
    if (log_n < 15 || log_n > 16 || n_tables > 64) return false;
    const uint32_t ld = log_n - 8;
    return n_jobs * (256u >> (kTileLog - ld)) < 256;   // what launch_rows calls a small launch
}

hipError_t launch_ntt_inverse(const NttArgs &a, uint32_t n_polys, int backend, hipStream_t s, bool blocks_done,
                              bool rows_skipped) {
    if (a.log_n < 9 || a.log_n > 17 || backend < NTT_BACKEND_INT || backend > NTT_BACKEND_MIXED) return hipErrorInvalidValue;
    const uint32_t n_jobs = a.jobs ? a.n_jobs * (a.items ? a.items : 1) : n_polys * a.map.limbs;
    if (n_jobs == 0) return hipSuccess;
    if (!blocks_done && !rows_skipped && one_pass_ok(a, backend, false, n_jobs)) return launch_limb_fp<false>(a, n_jobs, s);
    hipError_t e = blocks_done                    ? hipSuccess
                   : backend == NTT_BACKEND_MIXED ? launch_blocks<false, NTT_BACKEND_MIXED>(a, n_polys, s)
                   : backend                    ? launch_blocks<false, NTT_BACKEND_FP>(a, n_polys, s)
                                                : launch_blocks<false, NTT_BACKEND_INT>(a, n_polys, s);
    if (e != hipSuccess || rows_skipped) return e;
    NttArgs rows = a;
    rows.in = a.out;  // the rows pass continues in place on the output buffer
    rows.in_poly_stride = a.out_poly_stride;
    return backend == NTT_BACKEND_MIXED ? launch_rows<false, NTT_BACKEND_MIXED>(rows, n_jobs, s)
           : backend                    ? launch_rows<false, NTT_BACKEND_FP>(rows, n_jobs, s)
                                        : launch_rows<false, NTT_BACKEND_INT>(rows, n_jobs, s);
}

}  // namespace he
