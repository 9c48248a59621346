// CKKS encoding and decoding on the device: the special FFT over the orbit 5^j mod 2N (HEAAN's fftSpecial /
// fftSpecialInv butterfly network, cahel-main/src/fft.cu:194-453), rounding to integer coefficients
// (src/rns_base.cu:121-156) and the CRT composition of a decrypted plaintext (src/rns_base.cu:325-459).
//
// All floating-point steps are plain IEEE double operations in a fixed order (this file is compiled without
// contraction): a butterfly is u = a + b, t = (a - b) * w with the four-multiplication complex product, so
// the result does not depend on how the butterflies are spread over threads.
//
// Layout: v = `slots` complex values as double2.  The stages whose span exceeds one tile of 2048 values (at most 5)
// run as one kernel over global memory, every thread holding the values that those stages combine; all the others
// run inside LDS in a single kernel.
#include "kernels.h"
#include "modarith.cuh"

namespace he {

namespace {

constexpr int kThreads = 256;
constexpr uint32_t kFftTile = 2048;  // complex values per workgroup in the LDS kernel (32 KiB)

__device__ __forceinline__ double2 cmul(double2 a, double2 w) {
    return double2{a.x * w.x - a.y * w.y, a.x * w.y + a.y * w.x};
}

// twiddle of butterfly j in a stage of span len: e^{+-2 pi i (5^j mod 4 len) / (4 len)}
template <bool INVERSE>
__device__ __forceinline__ double2 stage_twiddle(const FftTables &t, uint32_t len, uint32_t j) {
    const uint32_t lenq = len << 2, gap = (2u << t.log_n) / lenq;
    const uint32_t r = t.rot_group[j] & (lenq - 1);
    return t.ksi[(INVERSE ? lenq - r : r) * gap];
}

// INVERSE (encode): decimation in frequency,  (a, b) -> (a + b, (a - b) w)
// forward (decode): decimation in time,       (a, b) -> (a + b w, a - b w)
template <bool INVERSE>
__device__ __forceinline__ void butterfly(double2 &a, double2 &b, double2 w) {
    if (INVERSE) {
        const double2 u{a.x + b.x, a.y + b.y};
        const double2 d{a.x - b.x, a.y - b.y};
        a = u;
        b = cmul(d, w);
    } else {
        const double2 t = cmul(b, w);
        const double2 u = a;
        a = double2{u.x + t.x, u.y + t.y};
        b = double2{u.x - t.x, u.y - t.y};
    }
}

// Where an encoding starts from: the caller's real and imaginary parts (zero padded from `count` on) instead of the
// scratch vector.  re = nullptr: the scratch vector itself.
struct FftSource {
    const double *re, *im;
    uint32_t count;
    size_t value_stride;          // doubles between the items' values
    unsigned long long *max_bits; // one per item, cleared here for the rounding kernel to accumulate into
};

__device__ __forceinline__ double2 source_value(const FftSource &src, uint32_t item, uint32_t i) {
    if (i >= src.count) return double2{0.0, 0.0};
    const size_t at = item * src.value_stride + i;
    return double2{src.re[at], src.im ? src.im[at] : 0.0};
}

constexpr int kTopThreads = 64;

// The R stages of span > tile in one kernel over global memory: thread `id` of an item holds the 2^R values
// id + h * tile, which those stages combine among themselves only; every butterfly is the one that a launch per
// stage with a thread per butterfly would compute (same operands, same twiddle).  blockIdx.y = item (vectors `slots`
// apart).  INVERSE runs the spans slots, slots / 2, .., 2 tile; forward 2 tile, .., slots.
template <bool INVERSE, int R>
__global__ __launch_bounds__(kTopThreads) void cfft_top_kernel(double2 *v, uint32_t tile, FftTables t, uint32_t slots,
                                                               FftSource src) {
    constexpr int E = 1 << R;
    const uint32_t id = blockIdx.x * kTopThreads + threadIdx.x;
    v += (size_t)blockIdx.y * slots;
    double2 e[E];
    if (INVERSE && src.re) {
        if (id == 0) src.max_bits[blockIdx.y] = 0;
#pragma unroll
        for (int h = 0; h < E; h++) e[h] = source_value(src, blockIdx.y, id + h * tile);
    } else {
#pragma unroll
        for (int h = 0; h < E; h++) e[h] = v[id + h * tile];
    }
#pragma unroll
    for (int st = 0; st < R; st++) {
        const int half = INVERSE ? E >> (st + 1) : 1 << st;   // distance of a butterfly's operands, in h
        const uint32_t len = tile * 2 * half;
#pragma unroll
        for (int b = 0; b < E / 2; b++) {
            const int lo = b & (half - 1), h0 = (b / half) * 2 * half + lo;
            butterfly<INVERSE>(e[h0], e[h0 + half], stage_twiddle<INVERSE>(t, len, id + lo * tile));
        }
    }
#pragma unroll
    for (int h = 0; h < E; h++) v[id + h * tile] = e[h];
}

// every stage of span <= tile inside LDS; tile = min(slots, kFftTile) values per workgroup
template <bool INVERSE>
__global__ __launch_bounds__(kThreads) void cfft_lds_kernel(double2 *v, uint32_t tile, FftTables t, uint32_t slots,
                                                            FftSource src) {
    __shared__ double2 s[kFftTile];
    double2 *g = v + (size_t)blockIdx.y * slots + (size_t)blockIdx.x * tile;
    if (INVERSE && src.re) {
        // (only when the whole vector is this one tile: otherwise the wider stages have run before)
        if (threadIdx.x == 0) src.max_bits[blockIdx.y] = 0;
        for (uint32_t i = threadIdx.x; i < tile; i += kThreads) s[i] = source_value(src, blockIdx.y, i);
    } else {
        for (uint32_t i = threadIdx.x; i < tile; i += kThreads) s[i] = g[i];
    }
    __syncthreads();
    for (uint32_t k = 2; k <= tile; k <<= 1) {
        const uint32_t len = INVERSE ? (tile << 1) / k : k;   // tile, tile/2, ..., 2  or  2, 4, ..., tile
        const uint32_t lenh = len >> 1;
        for (uint32_t b = threadIdx.x; b < (tile >> 1); b += kThreads) {
            const uint32_t j = b & (lenh - 1), pos = ((b / lenh) * len) + j;
            double2 x = s[pos], y = s[pos + lenh];
            butterfly<INVERSE>(x, y, stage_twiddle<INVERSE>(t, len, j));
            s[pos] = x;
            s[pos + lenh] = y;
        }
        __syncthreads();
    }
    for (uint32_t i = threadIdx.x; i < tile; i += kThreads) g[i] = s[i];
}

// The same for a full tile of kFftTile = 2048 values, 8 values per thread: the 11 stages run as register blocks of
// 3 + 3 + 3 + 2 stages with the tile in LDS between them (4 exchanges instead of 11), and the 24 twiddles a thread
// needs are fetched ahead of everything (each is a table look-up behind a table look-up: inside the stages, 11 such
// round trips to L2 in a row were most of the kernel's time).  Every butterfly has the operands and the twiddle it
// has in cfft_lds_kernel, so the results are the same bit for bit.
// Block of top span Lb = 8 S (S = 256, 32, 4): thread (hi, lo) = (tid / S, tid mod S) holds hi Lb + lo + k S, k < 8;
// stage i of it (span Lb >> i) pairs k with k + (4 >> i) and takes twiddle lo + (k mod (4 >> i)) S.
template <bool INVERSE>
__global__ __launch_bounds__(kThreads) void cfft_lds8_kernel(double2 *v, FftTables t, uint32_t slots, FftSource src) {
    constexpr uint32_t T = kFftTile;
    static_assert(T == 2048 && kThreads == 256, "8 values per thread");
    __shared__ double2 s[T + T / 32];
    auto sk = [](uint32_t e) { return e + (e >> 5); };   // (a group of 4 lanes reads 32 values apart in the S = 4 block)
    double2 *g = v + (size_t)blockIdx.y * slots + (size_t)blockIdx.x * T;
    const uint32_t tid = threadIdx.x;
    double2 tw[3][7], twd[3];
#pragma unroll
    for (int b = 0; b < 3; b++) {
        const uint32_t S = 256u >> (3 * b), Lb = 8 * S, lo = tid & (S - 1);
#pragma unroll
        for (int k = 0; k < 4; k++) tw[b][k] = stage_twiddle<INVERSE>(t, Lb, lo + k * S);
#pragma unroll
        for (int k = 0; k < 2; k++) tw[b][4 + k] = stage_twiddle<INVERSE>(t, Lb / 2, lo + k * S);
        tw[b][6] = stage_twiddle<INVERSE>(t, Lb / 4, lo);
    }
    twd[0] = stage_twiddle<INVERSE>(t, 4, 0);
    twd[1] = stage_twiddle<INVERSE>(t, 4, 1);
    twd[2] = stage_twiddle<INVERSE>(t, 2, 0);
    if (INVERSE && src.re) {
        // (only when the whole vector is this one tile: otherwise the wider stages have run before)
        if (tid == 0) src.max_bits[blockIdx.y] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) s[sk(tid + i * kThreads)] = source_value(src, blockIdx.y, tid + i * kThreads);
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) s[sk(tid + i * kThreads)] = g[tid + i * kThreads];
    }
    __syncthreads();
    auto block3 = [&](int b) {
        const uint32_t S = 256u >> (3 * b), Lb = 8 * S;
        const uint32_t base = (tid / S) * Lb + (tid & (S - 1));
        double2 e[8];
#pragma unroll
        for (int k = 0; k < 8; k++) e[k] = s[sk(base + k * S)];
        if (INVERSE) {
#pragma unroll
            for (int k = 0; k < 4; k++) butterfly<true>(e[k], e[k + 4], tw[b][k]);
#pragma unroll
            for (int k = 0; k < 4; k++) butterfly<true>(e[(k & 1) + 4 * (k >> 1)], e[(k & 1) + 4 * (k >> 1) + 2], tw[b][4 + (k & 1)]);
#pragma unroll
            for (int k = 0; k < 8; k += 2) butterfly<true>(e[k], e[k + 1], tw[b][6]);
        } else {
#pragma unroll
            for (int k = 0; k < 8; k += 2) butterfly<false>(e[k], e[k + 1], tw[b][6]);
#pragma unroll
            for (int k = 0; k < 4; k++) butterfly<false>(e[(k & 1) + 4 * (k >> 1)], e[(k & 1) + 4 * (k >> 1) + 2], tw[b][4 + (k & 1)]);
#pragma unroll
            for (int k = 0; k < 4; k++) butterfly<false>(e[k], e[k + 4], tw[b][k]);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) s[sk(base + k * S)] = e[k];
        __syncthreads();
    };
    // spans 4 and 2: two groups of 4 consecutive values per thread
    auto block2 = [&]() {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const uint32_t base = 4 * (tid + r * kThreads);
            double2 e[4];
#pragma unroll
            for (int k = 0; k < 4; k++) e[k] = s[sk(base + k)];
            if (INVERSE) {
                butterfly<true>(e[0], e[2], twd[0]);
                butterfly<true>(e[1], e[3], twd[1]);
                butterfly<true>(e[0], e[1], twd[2]);
                butterfly<true>(e[2], e[3], twd[2]);
            } else {
                butterfly<false>(e[0], e[1], twd[2]);
                butterfly<false>(e[2], e[3], twd[2]);
                butterfly<false>(e[0], e[2], twd[0]);
                butterfly<false>(e[1], e[3], twd[1]);
            }
#pragma unroll
            for (int k = 0; k < 4; k++) s[sk(base + k)] = e[k];
        }
        __syncthreads();
    };
    if (INVERSE) {
        block3(0);
        block3(1);
        block3(2);
        block2();
    } else {
        block2();
        block3(2);
        block3(1);
        block3(0);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) g[tid + i * kThreads] = s[sk(tid + i * kThreads)];
}

// The largest magnitude of an item's coefficients (the bit patterns of non-negative doubles order like the values):
// reduced over the wave, then over the workgroup, one atomic per workgroup.  Atomics on one address are served one
// after the other: one per thread took most of the rounding kernel's time, one per wave still half of it.  Every
// thread of the workgroup calls this.
__device__ __forceinline__ void block_max_to(unsigned long long *dst, unsigned long long m) {
    __shared__ unsigned long long wave_max[kThreads / 64];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const unsigned long long o = __shfl_xor(m, d);
        m = o > m ? o : m;
    }
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kThreads / 64; w++) m = wave_max[w] > m ? wave_max[w] : m;
        if (m) atomicMax(dst, m);
    }
}

// Where the rounded coefficients go: as doubles to coeffs [items][N], or (out given) as residues of the first `limbs`
// primes to out [items][limbs][N], items out_item_stride words apart.
struct RoundSink {
    double *coeffs;
    uint64_t *out;
    const uint64_t *moduli, *barrett;
    uint32_t limbs;
    size_t out_item_stride;
};

// residue of a rounded real coefficient (below 2^63 in magnitude: the caller checks the maximum)
__device__ __forceinline__ uint64_t real_residue(double c, uint64_t q, uint64_t r1) {
    const uint64_t r = barrett64((uint64_t)fabs(c), q, r1);
    return c < 0 ? neg_mod(r, q) : r;
}

// coefficient c of the plaintext: real parts fill the first half, imaginary parts the second, `gap` apart;
// value i comes from position bitrev(i) of the transformed vector
__global__ __launch_bounds__(kThreads) void encode_round_kernel(const double2 *v, uint32_t log_slots, uint32_t gap,
                                                                uint32_t half, double fix, RoundSink sink,
                                                                unsigned long long *max_bits) {
    const uint32_t c = blockIdx.x * kThreads + threadIdx.x;
    v += (size_t)blockIdx.y << log_slots;
    double *coeffs = sink.coeffs + (size_t)blockIdx.y * 2 * half;
    max_bits += blockIdx.y;
    const bool imag = c >= half;
    const uint32_t k = imag ? c - half : c;
    double val = 0.0;
    if (k % gap == 0) {
        const uint32_t i = k / gap;
        const double2 z = v[__brev(i) >> (32 - log_slots)];
        val = round((imag ? z.y : z.x) * fix);
    }
    if (sink.out) {
        uint64_t *o = sink.out + blockIdx.y * sink.out_item_stride + c;
        for (uint32_t l = 0; l < sink.limbs; l++)
            o[(size_t)l * 2 * half] = real_residue(val, sink.moduli[l], sink.barrett[2 * l + 1]);
    } else {
        coeffs[c] = val;
    }
    block_max_to(max_bits, (unsigned long long)__double_as_longlong(fabs(val)));
}

// The same for full packing (gap = 1, at least 256 slots): the bit reversal as a tiled transpose through LDS, so that
// both the reads of the transformed vector and the writes of the coefficients touch whole cache lines (with one thread
// per coefficient every lane of a wave reads a line of its own).  Slot i = (top 4 bits | middle | low 4 bits); a
// workgroup takes one value of the middle bits: thread (x, y) reads the slot with low bits y and top bits brev4(x),
// which sits at position (brev4(y) | brev(middle) | x) of the vector (consecutive in x), and writes the slot with low
// bits x and top bits brev4(y) (consecutive in x), real part to coefficient i, imaginary part to coefficient N/2 + i.
__global__ __launch_bounds__(kThreads) void encode_round_tiled_kernel(const double2 *v, uint32_t log_slots, uint32_t half,
                                                                      double fix, RoundSink sink, unsigned long long *max_bits) {
    __shared__ double2 tile[16][17];
    const uint32_t x = threadIdx.x & 15, y = threadIdx.x >> 4, mid = blockIdx.x, mid_bits = log_slots - 8;
    v += (size_t)blockIdx.y << log_slots;
    double *coeffs = sink.coeffs + (size_t)blockIdx.y * 2 * half;
    max_bits += blockIdx.y;
    const uint32_t rmid = mid_bits ? __brev(mid) >> (32 - mid_bits) : 0;
    const uint32_t brev4_y = __brev(y) >> 28;
    tile[y][x] = v[(brev4_y << (log_slots - 4)) | (rmid << 4) | x];
    __syncthreads();
    const double2 z = tile[x][y];
    const uint32_t i = (brev4_y << (log_slots - 4)) | (mid << 4) | x;
    const double re = round(z.x * fix), im = round(z.y * fix);
    if (sink.out) {
        uint64_t *o = sink.out + blockIdx.y * sink.out_item_stride + i;
        for (uint32_t l = 0; l < sink.limbs; l++) {
            const uint64_t q = sink.moduli[l], r1 = sink.barrett[2 * l + 1];
            o[(size_t)l * 2 * half] = real_residue(re, q, r1);
            o[(size_t)l * 2 * half + half] = real_residue(im, q, r1);
        }
    } else {
        coeffs[i] = re;
        coeffs[half + i] = im;
    }
    const double big = fabs(re) > fabs(im) ? fabs(re) : fabs(im);
    block_max_to(max_bits, (unsigned long long)__double_as_longlong(big));
}

constexpr int kMaxComposeLimbs = 64;

// Garner's mixed-radix composition of one coefficient, centred around zero, as a double divided by the scale.
// thread s < slots: real part of value s, else imaginary part of value s - slots; stored at position bitrev.
// LIMBS > 0: the number of limbs at compile time (the digits then stay in registers; with a run-time count the array
// lives in scratch memory), 0: any number up to kMaxComposeLimbs.
template <int LIMBS>
__global__ __launch_bounds__(kThreads) void decode_compose_kernel(const uint64_t *res, uint32_t limbs_rt, uint32_t log_n,
                                                                  uint32_t log_slots, uint32_t gap, double inv_scale,
                                                                  const uint64_t *moduli, const uint64_t *barrett,
                                                                  const uint64_t *garner_inv, uint32_t garner_stride,
                                                                  double2 *v) {
    const uint32_t limbs = LIMBS ? (uint32_t)LIMBS : limbs_rt;
    const uint32_t s = blockIdx.x * kThreads + threadIdx.x;
    const uint32_t slots = 1u << log_slots, half = 1u << (log_n - 1);
    if (s >= 2 * slots) return;
    res += ((size_t)blockIdx.y * limbs) << log_n;   // blockIdx.y = item: dense plaintexts, dense slot vectors
    v += (size_t)blockIdx.y * slots;
    const bool imag = s >= slots;
    const uint32_t i0 = imag ? s - slots : s;
    const size_t coeff = (imag ? half : 0) + (size_t)i0 * gap;
    uint64_t d[LIMBS ? LIMBS : kMaxComposeLimbs];
#pragma unroll
    for (uint32_t i = 0; i < limbs; i++) {
        const uint64_t q = moduli[i], r0 = barrett[2 * i], r1 = barrett[2 * i + 1];
        uint64_t t = res[((size_t)i << log_n) + coeff];
#pragma unroll
        for (uint32_t j = 0; j < i; j++) {
            const uint64_t dj = barrett64(d[j], q, r1);
            t = mul_mod(sub_mod(t, dj, q), garner_inv[(size_t)i * garner_stride + j], q, r0, r1);
        }
        d[i] = t;
    }
    // negative iff the digits, read from the top, exceed those of (Q - 1) / 2, whose digits are (q_i - 1) / 2
    // (written without early exits so that the loops unroll: `decided` / `carry` play the part of the breaks)
    bool negative = false, decided = false;
#pragma unroll
    for (uint32_t k = 0; k < limbs; k++) {
        const uint32_t i = limbs - 1 - k;
        const uint64_t h = (moduli[i] - 1) >> 1;
        if (!decided && d[i] != h) {
            negative = d[i] > h;
            decided = true;
        }
    }
    if (negative) {
        // Q - v = (Q - 1 - v) + 1: digit-wise complement, then increment
        bool carry = true;
#pragma unroll
        for (uint32_t i = 0; i < limbs; i++) {
            uint64_t x = moduli[i] - 1 - d[i];
            if (carry) {
                x++;
                carry = x >= moduli[i];
                if (carry) x = 0;
            }
            d[i] = x;
        }
    }
    double acc = 0.0;
#pragma unroll
    for (uint32_t k = 0; k < limbs; k++) {
        const uint32_t i = limbs - 1 - k;
        acc = acc * (double)moduli[i] + (double)d[i];
    }
    const double val = (negative ? -acc : acc) * inv_scale;
    double *slot = reinterpret_cast<double *>(&v[__brev(i0) >> (32 - log_slots)]);
    slot[imag ? 1 : 0] = val;
}

template <bool INVERSE>
hipError_t run_fft(double2 *v, uint32_t slots, uint32_t items, const FftTables &t, hipStream_t s, FftSource src) {
    const uint32_t tile = slots < kFftTile ? slots : kFftTile;
    const dim3 top_grid(tile / kTopThreads, items), lds_grid(slots / tile, items);
    const uint32_t wide = 31 - __builtin_clz(slots / tile);   // stages of span > tile
    const FftSource none{nullptr, nullptr, 0, 0, nullptr};
    auto top = [&](FftSource from) {
        switch (wide) {
            case 1: hipLaunchKernelGGL((cfft_top_kernel<INVERSE, 1>), top_grid, dim3(kTopThreads), 0, s, v, tile, t, slots, from); break;
            case 2: hipLaunchKernelGGL((cfft_top_kernel<INVERSE, 2>), top_grid, dim3(kTopThreads), 0, s, v, tile, t, slots, from); break;
            case 3: hipLaunchKernelGGL((cfft_top_kernel<INVERSE, 3>), top_grid, dim3(kTopThreads), 0, s, v, tile, t, slots, from); break;
            case 4: hipLaunchKernelGGL((cfft_top_kernel<INVERSE, 4>), top_grid, dim3(kTopThreads), 0, s, v, tile, t, slots, from); break;
            case 5: hipLaunchKernelGGL((cfft_top_kernel<INVERSE, 5>), top_grid, dim3(kTopThreads), 0, s, v, tile, t, slots, from); break;
            default: return hipErrorInvalidValue;
        }
        return hipSuccess;
    };
    if (INVERSE) {
        if (wide)
            if (hipError_t e = top(src)) return e;
        if (tile == kFftTile)
            hipLaunchKernelGGL(cfft_lds8_kernel<true>, lds_grid, dim3(kThreads), 0, s, v, t, slots, wide ? none : src);
        else
            hipLaunchKernelGGL(cfft_lds_kernel<true>, lds_grid, dim3(kThreads), 0, s, v, tile, t, slots, wide ? none : src);
    } else {
        if (tile == kFftTile)
            hipLaunchKernelGGL(cfft_lds8_kernel<false>, lds_grid, dim3(kThreads), 0, s, v, t, slots, none);
        else
            hipLaunchKernelGGL(cfft_lds_kernel<false>, lds_grid, dim3(kThreads), 0, s, v, tile, t, slots, none);
        if (wide)
            if (hipError_t e = top(none)) return e;
    }
    return hipGetLastError();
}

// out[item][i] = v[item][i] for i < count: the leading slots of every item, packed
__global__ __launch_bounds__(kThreads) void take_slots_kernel(const double2 *v, uint32_t slots, uint32_t count, double2 *out) {
    const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
    if (i < count) out[(size_t)blockIdx.y * count + i] = v[(size_t)blockIdx.y * slots + i];
}

}  // namespace

hipError_t launch_ckks_encode(const FftTables &t, const double *re, const double *im, uint32_t count, uint32_t slots,
                              double scale, double2 *v, double *coeffs, uint64_t *max_bits, uint32_t items,
                              size_t value_stride, hipStream_t s, const Tables *tab, uint64_t *out, uint32_t limbs,
                              size_t out_item_stride) {
    const uint32_t n = 1u << t.log_n, log_slots = 31 - __builtin_clz(slots);
    if (items == 0 || items > 65535 || (out ? (!tab || limbs == 0) : !coeffs)) return hipErrorInvalidValue;
    unsigned long long *maxima = reinterpret_cast<unsigned long long *>(max_bits);
    hipError_t e = run_fft<true>(v, slots, items, t, s, FftSource{re, im, count, value_stride, maxima});
    if (e != hipSuccess) return e;
    const RoundSink sink{coeffs, out, out ? tab->moduli : nullptr, out ? tab->barrett : nullptr, limbs, out_item_stride};
    if (slots == n / 2 && log_slots >= 8)
        hipLaunchKernelGGL(encode_round_tiled_kernel, dim3(slots / kThreads, items), dim3(kThreads), 0, s, v, log_slots, n / 2,
                           scale / (double)slots, sink, maxima);
    else
        hipLaunchKernelGGL(encode_round_kernel, dim3((n + kThreads - 1) / kThreads, items), dim3(kThreads), 0, s, v, log_slots,
                           (n / 2) / slots, n / 2, scale / (double)slots, sink, maxima);
    return hipGetLastError();
}

hipError_t launch_ckks_decode(const FftTables &t, const Tables &tab, const uint64_t *res, uint32_t limbs,
                              uint32_t slots, double scale, const uint64_t *garner_inv, uint32_t garner_stride,
                              double2 *v, uint32_t items, hipStream_t s) {
    const uint32_t n = 1u << t.log_n, log_slots = 31 - __builtin_clz(slots);
    if (limbs == 0 || limbs > (uint32_t)kMaxComposeLimbs || items == 0 || items > 65535) return hipErrorInvalidValue;
    const dim3 grid((2 * slots + kThreads - 1) / kThreads, items);
#define HE_COMPOSE(L)                                                                                                     \
    hipLaunchKernelGGL(decode_compose_kernel<L>, grid, dim3(kThreads), 0, s, res, limbs, t.log_n, log_slots, (n / 2) / slots, \
                       1.0 / scale, tab.moduli, tab.barrett, garner_inv, garner_stride, v)
    switch (limbs) {
        case 1: HE_COMPOSE(1); break;
        case 2: HE_COMPOSE(2); break;
        case 3: HE_COMPOSE(3); break;
        case 4: HE_COMPOSE(4); break;
        default: HE_COMPOSE(0); break;
    }
#undef HE_COMPOSE
    return run_fft<false>(v, slots, items, t, s, FftSource{nullptr, nullptr, 0, 0, nullptr});
}

hipError_t launch_take_slots(const double2 *v, uint32_t slots, uint32_t items, uint32_t count, double2 *out, hipStream_t s) {
    if (count == 0 || count > slots || items == 0 || items > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(take_slots_kernel, dim3((count + kThreads - 1) / kThreads, items), dim3(kThreads), 0, s, v, slots,
                       count, out);
    return hipGetLastError();
}

}  // namespace he
