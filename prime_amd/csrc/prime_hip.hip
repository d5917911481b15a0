// libprime_hip.so - HIP kernels (gfx950 / CDNA4, wave64) and C ABI for the int8 pseudo-gradient
// compression path: fp64 statistics, uint8 quantization, 256-bin lookup build, lookup
// dequantization and the ring's accumulate + requantize step.  All kernels are HBM-bound
// streams: 16-byte loads per lane, 1024-thread workgroups that loop over tiles, histogram
// traffic kept in LDS.  Grid-level reductions are two-stage: every workgroup stores its
// partial result, a small second kernel adds the partials in a fixed order.
//
// Arithmetic follows the reference's CPU ops (paths relative to the reference checkout):
//   src/zeroband/C/csrc/compression.cpp:9-43    quantize      -> quantize_code()
//   src/zeroband/C/csrc/compression.cpp:45-104  average       -> hist_add() / lut_finalize_kernel
//   src/zeroband/C/csrc/compression.cpp:106-125 scale formula -> finalize_qparams()
//   src/zeroband/C/csrc/collectives.cpp:8-22    index add/set -> dequant_kernel
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <vector>

#include "../../include/prime_hip.h"

namespace {

// Build-time tuning (defaults: the best of a sweep on MI355X).
#ifndef PRIME_UNROLL
#define PRIME_UNROLL 4                   // 16-byte loads in flight per lane
#endif
#ifndef PRIME_THREADS
#define PRIME_THREADS 1024               // workgroup size of the streaming kernels
#endif
#ifndef PRIME_COUNT_REPLICAS
#define PRIME_COUNT_REPLICAS 16          // LDS copies of each counter in the code-population kernel
#endif
#ifndef PRIME_BLOCKS_PER_CU
#define PRIME_BLOCKS_PER_CU 2            // resident workgroups per compute unit (32 wavefronts)
#endif

constexpr int kThreads = PRIME_THREADS;   // wavefronts of 64
constexpr int kBatchThreads = 512;       // workgroup of the one-tensor-per-workgroup kernel
constexpr int kWaves = kThreads / 64;
constexpr int kBins = 256;               // compression.cpp:5
constexpr int kZeroPoint = 128;          // compression.cpp:107
constexpr int kMaxGrid = 2048;           // per-workgroup partial slots in the workspace
constexpr int kUnroll = PRIME_UNROLL;
constexpr int kDivUnroll = PRIME_UNROLL > 2 ? 2 : PRIME_UNROLL;   // vectors per step in the kernels that divide
// wavefronts per SIMD the streaming kernels are compiled for (4 SIMDs per compute unit, at
// most 8 wavefronts each): bounds their register use so that PRIME_BLOCKS_PER_CU workgroups fit
constexpr int kWavesPerSimd = (PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4 > 8 ? 8
                              : ((PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4 < 1 ? 1 : (PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4);
constexpr int kFinalThreads = 1024;      // workgroup size of the second-stage kernels
constexpr int kLutBinsPerBlock = 4;      // bins one second-stage workgroup reduces (64 bytes per partial)
constexpr int64_t kMaxElems = int64_t(1) << 40;   // per-workgroup counts are 32-bit

struct BinAcc {
    double sum;
    unsigned long long cnt;
};

// Every kernel stores its per-workgroup partial results here with plain stores; the kernel
// boundary makes them visible to the second stage.  Nothing has to be zero between calls.
struct Workspace {
    prime_qparams qp;                    // scale of the tensor in flight
    uint32_t code_map[kBins / 4];        // old code -> new code of a requantization in the code domain
    unsigned long long code_total[kBins];   // population of each code over the whole tensor
    double part_sum[kMaxGrid];
    double part_sq[kMaxGrid];
    union {
        BinAcc hist[kMaxGrid][kBins];    // 4 KiB per workgroup
        uint32_t code_cnt[kMaxGrid][kBins];   // per-workgroup populations of each code value
    };
};

typedef float f4a __attribute__((ext_vector_type(4)));   // 16-byte aligned
typedef uint32_t u4a __attribute__((ext_vector_type(4)));   // 16 codes, 16-byte aligned

// Under-aligned views for buffers that are only element aligned (a chunk or a view that
// starts at an odd element).  They are distinct struct types, so the alignment survives
// template deduction; the compiler picks accesses that are legal for that alignment.
struct __attribute__((packed, aligned(4))) F4U { float x, y, z, w; };
struct __attribute__((packed)) U32U { uint32_t v; };
struct __attribute__((packed)) U4U { uint32_t x, y, z, w; };

// Streamed accesses, 4 floats / 4 codes at vector index i.  ALIGNED means the float buffer is
// 16-byte aligned and the code buffer 4-byte aligned.  NT adds the non-temporal hint to loads:
// it pays on tensors far larger than the 256 MB last-level cache and costs on smaller ones, so
// the host picks it by size.  Write-once outputs are always stored non-temporally.
template <bool ALIGNED, bool NT> struct Mem;

template <bool NT> struct Mem<true, NT> {
    static __device__ __forceinline__ f4a ldf4(const float* p, int64_t i) {
        const f4a* q = reinterpret_cast<const f4a*>(p) + i;
        return NT ? __builtin_nontemporal_load(q) : *q;
    }
    static __device__ __forceinline__ void stf4(float* p, int64_t i, f4a v, bool streaming) {
        f4a* q = reinterpret_cast<f4a*>(p) + i;
        if (streaming) __builtin_nontemporal_store(v, q);
        else *q = v;
    }
    static __device__ __forceinline__ uint32_t ldu32(const uint8_t* p, int64_t i) {
        const uint32_t* q = reinterpret_cast<const uint32_t*>(p) + i;
        return NT ? __builtin_nontemporal_load(q) : *q;
    }
    static __device__ __forceinline__ void stu32(uint8_t* p, int64_t i, uint32_t v) {
        __builtin_nontemporal_store(v, reinterpret_cast<uint32_t*>(p) + i);
    }
};

template <bool NT> struct Mem<false, NT> {
    static __device__ __forceinline__ f4a ldf4(const float* p, int64_t i) {
        const F4U t = reinterpret_cast<const F4U*>(p)[i];
        return f4a{t.x, t.y, t.z, t.w};
    }
    static __device__ __forceinline__ void stf4(float* p, int64_t i, f4a v, bool) {
        reinterpret_cast<F4U*>(p)[i] = F4U{v.x, v.y, v.z, v.w};
    }
    static __device__ __forceinline__ uint32_t ldu32(const uint8_t* p, int64_t i) {
        return reinterpret_cast<const U32U*>(p)[i].v;
    }
    static __device__ __forceinline__ void stu32(uint8_t* p, int64_t i, uint32_t v) {
        reinterpret_cast<U32U*>(p)[i] = U32U{v};
    }
};

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// compression.cpp:23-24 for one element.  std::round is half away from zero; the
// float -> int32 conversion follows x86 (out of range and NaN give INT_MIN) and the
// zero-point add wraps, so NaN, +-inf and huge values land on code 0 as on the CPU.
__device__ __forceinline__ int quantize_code(float x, float inv_scale, int zero_point) {
    const float r = __builtin_roundf(x * inv_scale);
    const int ri = (r >= -2147483648.0f && r < 2147483648.0f) ? static_cast<int>(r) : INT_MIN;
    const int q = static_cast<int>(static_cast<unsigned>(ri) + static_cast<unsigned>(zero_point));
    return min(max(q, 0), 255);
}

// compression.cpp:113-116: std = double(norm) / sqrt(numel - 1), scale = 6 * std / 256,
// narrowed to float at the quantizer's argument (:119).  norm() returns an fp32 tensor, so
// the fp64 sum of squares is rounded to float once after the square root.
__device__ __forceinline__ void finalize_from_norm(float norm, double sum, double sumsq, int64_t n, prime_qparams* qp);

__device__ __forceinline__ void finalize_qparams(double sum, double sumsq, int64_t n, prime_qparams* qp) {
    finalize_from_norm(static_cast<float>(sqrt(sumsq)), sum, sumsq, n, qp);
}

__device__ __forceinline__ void finalize_from_norm(float norm, double sum, double sumsq, int64_t n, prime_qparams* qp) {
    const double std_unbiased = static_cast<double>(norm) / sqrt(static_cast<double>(n - 1));
    const double scale = 6.0 * std_unbiased / 256.0;
    const float sf = static_cast<float>(scale);
    qp->scale = sf;
    qp->inv_scale = 1.0f / sf;           // compression.cpp:16
    qp->sum = sum;
    qp->sumsq = sumsq;
    qp->n = n;
}

// Workgroup reduction of (sum, sumsq) in a fixed order; the workgroup's partial goes to the
// workspace for stats_finalize_kernel.
__device__ __forceinline__ void block_stats_store(double s, double q, Workspace* ws) {
    __shared__ double sh_s[kWaves];
    __shared__ double sh_q[kWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    s = wave_sum(s);
    q = wave_sum(q);
    if (lane == 0) { sh_s[wave] = s; sh_q[wave] = q; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        ws->part_sum[blockIdx.x] = S;
        ws->part_sq[blockIdx.x] = Q;
    }
}

// True when the tensor's spread is below about two bins: std < 0.05 rms, from the fp64 sums.
__device__ __forceinline__ bool narrow_distribution(double sum, double sumsq, int64_t n) {
    if (n < 2) return false;
    const double mean = sum / static_cast<double>(n);
    const double ms = sumsq / static_cast<double>(n);
    const double var = ms - mean * mean;
    return var * 400.0 <= ms;            // also true for an all-zero tensor; false when a sum is NaN
}

// Second stage of the statistics run by a whole workgroup of the consuming kernel: every
// workgroup adds the same partials in the same order, so all of them derive the same scale
// bit for bit and no separate launch is needed.  Returns 1 / scale; workgroup 0 publishes
// the record.
template <int THREADS>
__device__ __forceinline__ float block_scale_from_partials(Workspace* ws, int nparts, int64_t n, prime_qparams* out,
                                                           int* hot_base = nullptr) {
    __shared__ double sh_s[THREADS / 64];
    __shared__ double sh_q[THREADS / 64];
    __shared__ float sh_inv;
    __shared__ int sh_hot;
    constexpr int kIters = (kMaxGrid + THREADS - 1) / THREADS;
    double ps[kIters], pq[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {       // all loads in flight at once
        const int i = threadIdx.x + k * THREADS;
        ps[k] = i < nparts ? ws->part_sum[i] : 0.0;
        pq[k] = i < nparts ? ws->part_sq[i] : 0.0;
    }
    double a = 0.0, b = 0.0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) { a += ps[k]; b += pq[k]; }
    a = wave_sum(a);
    b = wave_sum(b);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sh_s[wave] = a; sh_q[wave] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < THREADS / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        prime_qparams qp;
        finalize_qparams(S, Q, n, &qp);
        sh_inv = qp.inv_scale;
        sh_hot = narrow_distribution(S, Q, n) ? quantize_code(static_cast<float>(S / static_cast<double>(n)), qp.inv_scale, kZeroPoint) - 1
                                              : INT_MIN;
        if (blockIdx.x == 0) {
            ws->qp = qp;
            if (out) *out = qp;
        }
    }
    __syncthreads();
    if (hot_base) *hot_base = sh_hot;
    return sh_inv;
}

// Second stage of the statistics: one workgroup adds the partials (tree of fixed shape) and
// derives the scale.
__global__ __launch_bounds__(kFinalThreads) void stats_finalize_kernel(Workspace* ws, int nparts, int64_t n,
                                                                        prime_qparams* out) {
    (void)block_scale_from_partials<kFinalThreads>(ws, nparts, n, out);
}

// Work distribution of the streaming kernels.  The tensor is cut into rows of kThreads
// 16-byte vectors (16 KiB of floats per row at 1024 threads).  Main part: tiles of kUnroll
// consecutive rows dealt round-robin to the G workgroups, so the whole grid sweeps the tensor
// as one sliding window of contiguous 64 KiB pieces and every access of the main part is
// unguarded.  Tail (fewer than G tiles): single rows dealt round-robin, so no workgroup
// streams more than one row beyond the average.  body(i0, stride, full) handles the kUnroll
// vectors i0 + j * stride (j < U) of the calling lane; `full` is a compile-time flag (true_type in the
// main part): unless it is set, each vector needs the check i < nvec.
// U is the number of vectors body handles per call (kUnroll unless the kernel needs the registers:
// the kernels that divide keep two operands per vector and a division sequence live).
template <int U = kUnroll, typename Body>
__device__ __forceinline__ void sweep(int64_t nvec, Body&& body) {
    const int64_t G = gridDim.x;
    const int64_t rows = (nvec + kThreads - 1) / kThreads;
    const int64_t rounds = (nvec / kThreads) / (G * U);
    for (int64_t k = 0; k < rounds; ++k)
        body(((k * G + blockIdx.x) * U) * kThreads + threadIdx.x, static_cast<int64_t>(kThreads), std::true_type{});
    const int64_t r0 = rounds * G * U + blockIdx.x;
    if (r0 < rows) body(r0 * kThreads + threadIdx.x, G * kThreads, std::false_type{});
}

__device__ __forceinline__ void stats_add4(const f4a v, double& s, double& q) {
    const double a = v.x, b = v.y, c = v.z, d = v.w;
    s += a; q = fma(a, a, q);
    s += b; q = fma(b, b, q);
    s += c; q = fma(c, c, q);
    s += d; q = fma(d, d, q);
}

// K1: sum and sum of squares in fp64.  4 bytes per element.
template <bool ALIGNED, bool NT>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void stats_kernel(const float* __restrict__ x, int64_t n, Workspace* ws) {
    using M = Mem<ALIGNED, NT>;
    const int64_t nvec = n >> 2;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            if (j & 1) stats_add4(v[j], s1, q1); else stats_add4(v[j], s0, q0);
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const double v = x[(nvec << 2) + threadIdx.x];
        s0 += v;
        q0 = fma(v, v, q0);
    }
    block_stats_store(s0 + s1, q0 + q1, ws);
}

// The norm as libtorch's CPU kernel accumulates it (the value compression.cpp:113 actually
// receives): eight fp32 lanes, lane j taking elements j, j + 8, ... by fused multiply-add, lanes
// added 0..7, then the n % 8 tail in order (a group of four as separately rounded products, the
// rest by fused multiply-add) and a float square root.  The chains are serial by definition, so
// this is one workgroup: fifteen wavefronts stage tiles in LDS, eight lanes of the first accumulate.  It exists
// to reproduce the reference's output bit for bit; the streaming kernels compute the exact sum.
constexpr int kLiteralTile = 8192;                       // floats per stage (two stages in LDS)
constexpr int kLiteralRow = kLiteralTile / 8 + 8;        // lane j's elements, padded: conflict-free stores
__global__ __launch_bounds__(kFinalThreads) void norm_literal_kernel(const float* __restrict__ x, int64_t n, Workspace* ws,
                                                                      prime_qparams* out) {
    // tile[buf][j * kLiteralRow + k] = element 8 k + j of the stage: lane j reads its chain in order,
    // four elements per LDS access.  Wavefront 0 accumulates stage s while the others load stage s + 1.
    __shared__ __attribute__((aligned(16))) float tile[2][8 * kLiteralRow];
    const int64_t m = n - (n % 8);
    const int64_t stages = (m + kLiteralTile - 1) / kLiteralTile;
    auto load_stage = [&](int64_t s, int first, int step) {
        const int64_t base = s * kLiteralTile;
        const int count = static_cast<int>(m - base < kLiteralTile ? m - base : kLiteralTile);   // a multiple of 8
        float* t = tile[s & 1];
        for (int i = first; i < count; i += step) t[(i & 7) * kLiteralRow + (i >> 3)] = x[base + i];
    };
    float acc = 0.0f;
    if (stages > 0) load_stage(0, threadIdx.x, kFinalThreads);
    __syncthreads();
    for (int64_t s = 0; s < stages; ++s) {
        if (threadIdx.x >= 64) {
            if (s + 1 < stages) load_stage(s + 1, threadIdx.x - 64, kFinalThreads - 64);
        } else if (threadIdx.x < 8) {
            const int64_t base = s * kLiteralTile;
            const int per_lane = static_cast<int>(m - base < kLiteralTile ? m - base : kLiteralTile) >> 3;
            const float* t = tile[s & 1] + threadIdx.x * kLiteralRow;
            int k = 0;
            for (; k + 16 <= per_lane; k += 16) {
                f4a v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f4a*>(t + k + 4 * u);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    acc = __builtin_fmaf(v[u].x, v[u].x, acc);
                    acc = __builtin_fmaf(v[u].y, v[u].y, acc);
                    acc = __builtin_fmaf(v[u].z, v[u].z, acc);
                    acc = __builtin_fmaf(v[u].w, v[u].w, acc);
                }
            }
            for (; k < per_lane; ++k) acc = __builtin_fmaf(t[k], t[k], acc);
        }
        __syncthreads();
    }
    if (threadIdx.x < 64) {
        float total = __shfl(acc, 0, 64);
#pragma unroll
        for (int j = 1; j < 8; ++j) total += __shfl(acc, j, 64);
        if (threadIdx.x == 0) {
            int64_t i = m;
            if (n - i >= 4) {
                for (int k = 0; k < 4; ++k) {
                    const float sq = x[i + k] * x[i + k];     // rounded on its own (contraction is off)
                    total += sq;
                }
                i += 4;
            }
            for (; i < n; ++i) total = __builtin_fmaf(x[i], x[i], total);
            const float norm = __builtin_sqrtf(total);
            prime_qparams qp;
            finalize_from_norm(norm, __builtin_nan(""), static_cast<double>(norm) * static_cast<double>(norm), n, &qp);
            ws->qp = qp;
            if (out) *out = qp;
        }
    }
}

// LDS histogram: R copies of each bin, chosen by lane, so that lanes of one wavefront that
// hit the same bin mostly hit different addresses (and banks).  Sums are fp64, counts u32
// (a workgroup never sees 2^32 elements: n is capped at 2^40 and the grid is at least one
// workgroup per compute unit once n is that large).
template <int R>
struct LdsHist {
    double sum[kBins * R];
    unsigned cnt[kBins * R];
};

template <int R>
__device__ __forceinline__ void hist_zero(LdsHist<R>& h) {
    for (int i = threadIdx.x; i < kBins * R; i += kThreads) { h.sum[i] = 0.0; h.cnt[i] = 0u; }
}

template <int R>
__device__ __forceinline__ void hist_add(LdsHist<R>& h, int code, float x) {
    const int slot = code * R + (threadIdx.x & (R - 1));
    __hip_atomic_fetch_add(&h.sum[slot], static_cast<double>(x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __hip_atomic_fetch_add(&h.cnt[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Register-side accumulators for a tensor whose values crowd into a few codes (a constant, or
// weights near 1 whose spread is a fraction of a bin): LDS atomics of a wavefront on one address
// serialize, so the three codes around the code of the mean are summed per lane and reach LDS
// once per wavefront.  Used only when the statistics say the tensor is that narrow.
struct HotCodes {
    int base;                 // hot codes are base, base + 1, base + 2
    double s0 = 0.0, s1 = 0.0, s2 = 0.0;
    unsigned c0 = 0, c1 = 0, c2 = 0;
};

template <int R>
__device__ __forceinline__ void hist_add_hot(LdsHist<R>& h, HotCodes& hot, int code, float x) {
    const unsigned d = static_cast<unsigned>(code - hot.base);
    if (d < 3u) {
        const double v = x;
        hot.s0 += d == 0 ? v : 0.0;
        hot.s1 += d == 1 ? v : 0.0;
        hot.s2 += d == 2 ? v : 0.0;
        hot.c0 += d == 0;
        hot.c1 += d == 1;
        hot.c2 += d == 2;
    } else {
        hist_add(h, code, x);
    }
}

// Every lane of the wavefront must call this (it shuffles); lane 0 adds the wavefront's totals.
template <int R>
__device__ __forceinline__ void hist_flush_hot(LdsHist<R>& h, const HotCodes& hot) {
    const double s[3] = {wave_sum(hot.s0), wave_sum(hot.s1), wave_sum(hot.s2)};
    unsigned c[3] = {hot.c0, hot.c1, hot.c2};
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) c[k] += __shfl_down(c[k], off, 64);
    if ((threadIdx.x & 63) == 0) {
        const int rep = (threadIdx.x >> 6) & (R - 1);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int code = hot.base + k;
            if (c[k] && code >= 0 && code < kBins) {
                __hip_atomic_fetch_add(&h.sum[code * R + rep], s[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(&h.cnt[code * R + rep], c[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
    }
}

// Store the workgroup's histogram (copies added in a fixed order) as its partial: one
// 16-byte store per lane, 4 KiB contiguous per workgroup.
template <int R>
__device__ __forceinline__ void hist_store(LdsHist<R>& h, Workspace* ws) {
    for (int b = threadIdx.x; b < kBins; b += kThreads) {
        BinAcc acc{0.0, 0ull};
#pragma unroll
        for (int r = 0; r < R; ++r) { acc.sum += h.sum[b * R + r]; acc.cnt += h.cnt[b * R + r]; }
        ws->hist[blockIdx.x][b] = acc;
    }
}

// K2 (+K3 when HIST): quantize to uint8, 4 codes packed per 32-bit store, and the 256-bin
// sum / count histogram of the same elements.  5 bytes per element.
template <bool ALIGNED, bool NT, bool HIST, int R>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void quantize_kernel(const float* __restrict__ x, int64_t n, float scale_val,
                                                            int stats_parts, prime_qparams* qp_out, int zero_point,
                                                            uint8_t* __restrict__ codes, Workspace* ws) {
    using M = Mem<ALIGNED, NT>;
    __shared__ LdsHist<HIST ? R : 1> hist;
    if (HIST) hist_zero(hist);
    // the scale: given by value, or derived here from the statistics partials of the pass before
    // (stats_parts < 0: the record a preceding kernel left in the workspace)
    int hot_base = INT_MIN;              // set when the statistics show a tensor crowded into a few codes
    const float inv = stats_parts > 0   ? block_scale_from_partials<kThreads>(ws, stats_parts, n, qp_out, &hot_base)
                      : stats_parts < 0 ? ws->qp.inv_scale
                                        : 1.0f / scale_val;
    if (HIST) __syncthreads();
    const int64_t nvec = n >> 2;
    auto pass = [&](auto narrow_t) {
        constexpr bool narrow = decltype(narrow_t)::value;
        HotCodes hot;
        hot.base = hot_base;
        auto add = [&](int code, float xv) {
            if (narrow) hist_add_hot(hist, hot, code, xv);
            else hist_add(hist, code, xv);
        };
        sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
            constexpr bool full = decltype(full_t)::value;
            f4a v[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                const int64_t i = i0 + j * stride;
                v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                const int64_t i = i0 + j * stride;
                if (full || i < nvec) {
                    const int a = quantize_code(v[j].x, inv, zero_point);
                    const int b = quantize_code(v[j].y, inv, zero_point);
                    const int c = quantize_code(v[j].z, inv, zero_point);
                    const int d = quantize_code(v[j].w, inv, zero_point);
                    M::stu32(codes, i, static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) |
                                           (static_cast<uint32_t>(c) << 16) | (static_cast<uint32_t>(d) << 24));
                    if (HIST) {
                        add(a, v[j].x);
                        add(b, v[j].y);
                        add(c, v[j].z);
                        add(d, v[j].w);
                    }
                }
            }
        });
        if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
            const int64_t i = (nvec << 2) + threadIdx.x;
            const float v = x[i];
            const int a = quantize_code(v, inv, zero_point);
            codes[i] = static_cast<uint8_t>(a);
            if (HIST) add(a, v);
        }
        if (HIST && narrow) hist_flush_hot(hist, hot);
    };
    if (HIST && hot_base != INT_MIN) pass(std::true_type{});
    else pass(std::false_type{});
    if (HIST) {
        __syncthreads();
        hist_store(hist, ws);
    }
}

// K3 alone: histogram of x under caller-supplied codes (average_buckets).  5 bytes per element.
template <bool ALIGNED, int R>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void hist_kernel(const float* __restrict__ x, const uint8_t* __restrict__ codes,
                                                        int64_t n, int n_bins, Workspace* ws) {
    using M = Mem<ALIGNED, false>;
    __shared__ LdsHist<R> hist;
    hist_zero(hist);
    __syncthreads();
    const int64_t nvec = n >> 2;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a v[kUnroll];
        uint32_t c[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            v[j] = ok ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
            c[j] = ok ? M::ldu32(codes, i) : 0u;
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
                const int a = c[j] & 255, b = (c[j] >> 8) & 255, cc = (c[j] >> 16) & 255, d = c[j] >> 24;
                if (a < n_bins) hist_add(hist, a, v[j].x);     // compression.cpp:70
                if (b < n_bins) hist_add(hist, b, v[j].y);
                if (cc < n_bins) hist_add(hist, cc, v[j].z);
                if (d < n_bins) hist_add(hist, d, v[j].w);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        const int a = codes[i];
        if (a < n_bins) hist_add(hist, a, x[i]);
    }
    __syncthreads();
    hist_store(hist, ws);
}

// Second stage of the lookup build.  Workgroup j owns bins 4j .. 4j+3 (64 contiguous bytes
// of every partial): lane (row, bin) adds partials row, row + 256, ... in order, the 256
// rows are then added by a tree of fixed shape.  Mean = fp64 sum / count rounded to float
// once; an empty bin gives 0.0f (compression.cpp:100).  Entries >= 256 of a longer table
// are 0.0f.
__global__ __launch_bounds__(kFinalThreads) void lut_finalize_kernel(const Workspace* __restrict__ ws, int nparts,
                                                                      float* __restrict__ lut, int64_t n_bins,
                                                                      unsigned long long* __restrict__ counts) {
    constexpr int kRows = kFinalThreads / kLutBinsPerBlock;
    __shared__ double sh_sum[kFinalThreads];
    __shared__ unsigned long long sh_cnt[kFinalThreads];
    const int bl = threadIdx.x % kLutBinsPerBlock;
    const int row = threadIdx.x / kLutBinsPerBlock;
    const int bin = blockIdx.x * kLutBinsPerBlock + bl;
    constexpr int kIters = kMaxGrid / kRows;
    BinAcc part[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {          // all loads in flight at once
        const int p = row + k * kRows;
        part[k] = p < nparts ? ws->hist[p][bin] : BinAcc{0.0, 0ull};
    }
    double s = 0.0;
    unsigned long long c = 0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) { s += part[k].sum; c += part[k].cnt; }
    sh_sum[threadIdx.x] = s;
    sh_cnt[threadIdx.x] = c;
    __syncthreads();
    for (int half = kRows / 2; half > 0; half >>= 1) {
        if (row < half) {
            sh_sum[threadIdx.x] += sh_sum[threadIdx.x + half * kLutBinsPerBlock];
            sh_cnt[threadIdx.x] += sh_cnt[threadIdx.x + half * kLutBinsPerBlock];
        }
        __syncthreads();
    }
    if (row == 0 && bin < n_bins) {
        const unsigned long long cc = sh_cnt[threadIdx.x];
        lut[bin] = cc ? static_cast<float>(sh_sum[threadIdx.x] / static_cast<double>(cc)) : 0.0f;
        if (counts) counts[bin] = cc;
    }
    if (blockIdx.x == 0)
        for (int64_t b = kBins + threadIdx.x; b < n_bins; b += kFinalThreads) lut[b] = 0.0f;
}

// ---- requantization in the code domain ----------------------------------------------------
// The all-gather forwards uniform_8bit_quantize(chunk) of a chunk that was just set to
// lut_in[codes_in] (collectives.cpp:204-215).  Such a chunk holds at most 256 distinct values, so
// its quantization is a function of the received codes alone: the statistics follow from the
// population of each code, the new code of an element from a 256-entry map, and a new lookup
// entry is the population-weighted mean of the old entries that map to it.  3 bytes per element
// (codes read twice, written once) instead of a pass over the fp32 chunk.

// 16 codes at vector index i; ALIGNED means both code buffers are 16-byte aligned.
template <bool ALIGNED>
__device__ __forceinline__ u4a ld_codes16(const uint8_t* p, int64_t i) {
    if (ALIGNED) return reinterpret_cast<const u4a*>(p)[i];
    const U4U t = reinterpret_cast<const U4U*>(p)[i];
    return u4a{t.x, t.y, t.z, t.w};
}

template <bool ALIGNED>
__device__ __forceinline__ void st_codes16(uint8_t* p, int64_t i, u4a v) {
    if (ALIGNED) __builtin_nontemporal_store(v, reinterpret_cast<u4a*>(p) + i);
    else reinterpret_cast<U4U*>(p)[i] = U4U{v.x, v.y, v.z, v.w};
}

// Pass 1: population of each code value, one partial per workgroup.  1 byte per element.
template <bool ALIGNED, int R>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void code_count_kernel(const uint8_t* __restrict__ codes, int64_t n,
                                                                              Workspace* ws) {
    __shared__ unsigned cnt[kBins * R];
    for (int i = threadIdx.x; i < kBins * R; i += kThreads) cnt[i] = 0u;
    __syncthreads();
    const int rep = threadIdx.x & (R - 1);
    auto bump = [&](uint32_t code) {
        __hip_atomic_fetch_add(&cnt[code * R + rep], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    const int64_t nvec = n >> 4;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        u4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? ld_codes16<ALIGNED>(codes, i) : u4a{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t w = v[j][k];
                    bump(w & 255);
                    bump((w >> 8) & 255);
                    bump((w >> 16) & 255);
                    bump(w >> 24);
                }
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 15)) bump(codes[(nvec << 4) + threadIdx.x]);
    __syncthreads();
    for (int b = threadIdx.x; b < kBins; b += kThreads) {
        unsigned c = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) c += cnt[b * R + r];
        ws->code_cnt[blockIdx.x][b] = c;
    }
}

// Between the passes, first kernel: total population of each code.  Workgroup j owns codes
// 4j .. 4j+3 (16 contiguous bytes of every partial); lane (row, code) adds partials row,
// row + 256, ..., then the rows are added by a tree of fixed shape.
__global__ __launch_bounds__(kFinalThreads) void code_total_kernel(Workspace* ws, int nparts) {
    constexpr int kRows = kFinalThreads / kLutBinsPerBlock;
    __shared__ unsigned long long sh_cnt[kFinalThreads];
    const int bl = threadIdx.x % kLutBinsPerBlock;
    const int row = threadIdx.x / kLutBinsPerBlock;
    const int bin = blockIdx.x * kLutBinsPerBlock + bl;
    constexpr int kIters = kMaxGrid / kRows;
    uint32_t part[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {          // all loads in flight at once
        const int p = row + k * kRows;
        part[k] = p < nparts ? ws->code_cnt[p][bin] : 0u;
    }
    unsigned long long c = 0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) c += part[k];
    sh_cnt[threadIdx.x] = c;
    __syncthreads();
    for (int half = kRows / 2; half > 0; half >>= 1) {
        if (row < half) sh_cnt[threadIdx.x] += sh_cnt[threadIdx.x + half * kLutBinsPerBlock];
        __syncthreads();
    }
    if (row == 0) ws->code_total[bin] = sh_cnt[threadIdx.x];
}

// Between the passes, second kernel, one workgroup: the statistics
// sum = sum_c count_c * lut_in[c] and sumsq = sum_c count_c * lut_in[c]^2 in fp64, the scale
// (compression.cpp:113-116), the map old code -> new code (:23-24 applied to lut_in[c]) and the
// new lookup table (:99-101).  Entries of lut_in whose code does not occur are ignored.
__global__ __launch_bounds__(kFinalThreads) void requant_plan_kernel(Workspace* ws, const float* __restrict__ lut_in, int64_t n,
                                                                      float* __restrict__ lut_out, prime_qparams* qp_out) {
    struct Rec {
        double term;                 // count * value
        unsigned long long count;
        int target;                  // new code, -1 when the old code does not occur
        int pad;
    };
    constexpr int kGroups = kFinalThreads / kBins;
    constexpr int kSpan = kBins / kGroups;
    __shared__ Rec rec[kBins];
    __shared__ double sh_s[kBins / 64], sh_q[kBins / 64];
    __shared__ float sh_inv;
    __shared__ double g_sum[kGroups][kBins];
    __shared__ unsigned long long g_cnt[kGroups][kBins];
    const int bin = threadIdx.x & (kBins - 1);
    float v = 0.0f;
    unsigned long long t = 0;
    if (threadIdx.x < kBins) {
        t = ws->code_total[bin];
        v = lut_in[bin];
        double s = 0.0, q = 0.0;
        if (t) {
            const double dv = v, dc = static_cast<double>(t);
            s = dc * dv;
            q = dc * (dv * dv);
        }
        rec[bin].term = s;
        rec[bin].count = t;
        s = wave_sum(s);
        q = wave_sum(q);
        if ((threadIdx.x & 63) == 0) { sh_s[threadIdx.x >> 6] = s; sh_q[threadIdx.x >> 6] = q; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kBins / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        prime_qparams qp;
        finalize_qparams(S, Q, n, &qp);
        sh_inv = qp.inv_scale;
        ws->qp = qp;
        if (qp_out) *qp_out = qp;
    }
    __syncthreads();
    int target = 0;
    if (threadIdx.x < kBins) {
        target = quantize_code(v, sh_inv, kZeroPoint);
        rec[bin].target = t ? target : -1;
    }
    __syncthreads();
    {
        // new entry `bin`: population-weighted mean of the old entries that map to it; the 256 old
        // codes are split over kGroups groups of lanes, joined in a fixed order
        const int group = threadIdx.x / kBins;
        double sum = 0.0;
        unsigned long long k = 0;
#pragma unroll 16
        for (int j = 0; j < kSpan; ++j) {
            const Rec r = rec[group * kSpan + j];
            const bool hit = r.target == bin;
            sum += hit ? r.term : 0.0;
            k += hit ? r.count : 0ull;
        }
        g_sum[group][bin] = sum;
        g_cnt[group][bin] = k;
    }
    __syncthreads();
    if (threadIdx.x < kBins) {
        double sum = g_sum[0][bin];
        unsigned long long k = g_cnt[0][bin];
#pragma unroll
        for (int g = 1; g < kGroups; ++g) { sum += g_sum[g][bin]; k += g_cnt[g][bin]; }
        lut_out[bin] = k ? static_cast<float>(sum / static_cast<double>(k)) : 0.0f;
        // four adjacent lanes pack their new codes into one word of the map
        uint32_t word = static_cast<uint32_t>(target) << (8 * (bin & 3));
        word |= __shfl_xor(word, 1, 64);
        word |= __shfl_xor(word, 2, 64);
        if ((bin & 3) == 0) ws->code_map[bin >> 2] = word;
    }
}

// Pass 2: codes_out[i] = map[codes_in[i]].  2 bytes per element.
template <bool ALIGNED>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void code_remap_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out,
                                                                              int64_t n, const Workspace* __restrict__ ws) {
    __shared__ uint32_t map_words[kBins / 4];
    if (threadIdx.x < kBins / 4) map_words[threadIdx.x] = ws->code_map[threadIdx.x];
    __syncthreads();
    const uint8_t* map = reinterpret_cast<const uint8_t*>(map_words);
    auto remap = [&](uint32_t w) {
        return static_cast<uint32_t>(map[w & 255]) | (static_cast<uint32_t>(map[(w >> 8) & 255]) << 8) |
               (static_cast<uint32_t>(map[(w >> 16) & 255]) << 16) | (static_cast<uint32_t>(map[w >> 24]) << 24);
    };
    const int64_t nvec = n >> 4;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        u4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? ld_codes16<ALIGNED>(in, i) : u4a{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) st_codes16<ALIGNED>(out, i, u4a{remap(v[j].x), remap(v[j].y), remap(v[j].z), remap(v[j].w)});
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 15)) {
        const int64_t i = (nvec << 4) + threadIdx.x;
        out[i] = map[in[i]];
    }
}

__global__ void lut_zero_kernel(float* __restrict__ lut, int64_t n_bins, unsigned long long* __restrict__ counts) {
    for (int64_t b = threadIdx.x; b < n_bins; b += blockDim.x) {
        lut[b] = 0.0f;
        if (counts && b < kBins) counts[b] = 0ull;
    }
}

// K5 / K4 pass A: out = lut[codes] (collectives.cpp:16-22) or out += lut[codes] (:8-14),
// the lookup table held in LDS; with STATS the fp64 sum and sum of squares of the updated
// values are taken in the same pass (the next quantization's scale).  With DIV the updated value
// is divided by `divisor` before it is stored and counted: chunk.div_(world_size) of
// ReduceOp::AVG (collectives.cpp:155-159) folded into the last accumulation of a chunk.
template <bool ADD, bool STATS, bool ALIGNED, bool NT, bool DIV = false>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void dequant_kernel(float* __restrict__ out, const float* __restrict__ lut,
                                                           const uint8_t* __restrict__ codes, int64_t n, Workspace* ws,
                                                           float divisor) {
    using M = Mem<ALIGNED, NT>;
    __shared__ float s_lut[kBins];
    for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut[b];
    __syncthreads();
    const int64_t nvec = n >> 2;
    constexpr int U = DIV ? kDivUnroll : kUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    sweep<U>(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        uint32_t c[U];
        f4a a[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            c[j] = ok ? M::ldu32(codes, i) : 0u;
            if (ADD) a[j] = ok ? M::ldf4(out, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            f4a v;
            v.x = s_lut[c[j] & 255];
            v.y = s_lut[(c[j] >> 8) & 255];
            v.z = s_lut[(c[j] >> 16) & 255];
            v.w = s_lut[c[j] >> 24];
            if (ADD) v += a[j];
            if (DIV) v = v / divisor;
            if (full || i < nvec) {
                M::stf4(out, i, v, !STATS);   // with STATS the quantize pass reads it again: no streaming hint
                if (STATS) {
                    if (j & 1) stats_add4(v, s1, q1); else stats_add4(v, s0, q0);
                }
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float v = s_lut[codes[i]];
        if (ADD) v += out[i];
        if (DIV) v = v / divisor;
        out[i] = v;
        if (STATS) {
            const double d = v;
            s0 += d;
            q0 = fma(d, d, q0);
        }
    }
    if (STATS) block_stats_store(s0 + s1, q0 + q1, ws);
}

// Small tensors: one workgroup per tensor of a flat buffer does the whole of
// uniform_8bit_quantize (statistics, scale, codes, lookup) without touching the workspace.
// With VEC (flat buffer 16-byte aligned, code buffer 4-byte aligned) the part of the tensor
// between its first and last multiple-of-4 global index is read as 16-byte vectors and its
// codes stored 4 at a time; the ragged ends, which share vectors with the neighbouring
// tensors, go element by element.  The second read of a tensor comes from L2.
template <bool VEC>
__global__ __launch_bounds__(kBatchThreads) void batched_kernel(const float* __restrict__ x, const int64_t* __restrict__ offsets,
                                                                uint8_t* __restrict__ codes, float* __restrict__ luts,
                                                                prime_qparams* __restrict__ qps) {
    constexpr int R = 4;
    __shared__ LdsHist<R> hist;
    __shared__ double sh_s[kBatchThreads / 64];
    __shared__ double sh_q[kBatchThreads / 64];
    __shared__ prime_qparams sh_qp;
    __shared__ int sh_hot_base;          // >= -1: the tensor is narrow, hot codes start here; INT_MIN: it is not
    const int64_t t = blockIdx.x;
    const int64_t lo = offsets[t];
    const int64_t hi = offsets[t + 1];
    const int64_t n = hi - lo;
    // [lo, a) and [b, hi) element by element, [a, b) as vectors
    int64_t a = VEC ? (lo + 3) & ~int64_t(3) : hi;
    int64_t b = VEC ? hi & ~int64_t(3) : hi;
    if (a > b) { a = hi; b = hi; }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < kBins * R; i += kBatchThreads) { hist.sum[i] = 0.0; hist.cnt[i] = 0u; }
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    const f4a* __restrict__ x4 = reinterpret_cast<const f4a*>(x);
    constexpr int U = 4;
    for (int64_t v0 = (a >> 2) + threadIdx.x; v0 < (b >> 2); v0 += kBatchThreads * U) {
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            v[j] = i < (b >> 2) ? x4[i] : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (j & 1) stats_add4(v[j], s1, q1); else stats_add4(v[j], s0, q0);
        }
    }
    for (int64_t i = lo + threadIdx.x; i < a; i += kBatchThreads) {        // ragged head (everything without VEC)
        const double v = x[i];
        s0 += v;
        q0 = fma(v, v, q0);
    }
    for (int64_t i = b + threadIdx.x; i < hi; i += kBatchThreads) {        // ragged tail
        const double v = x[i];
        s1 += v;
        q1 = fma(v, v, q1);
    }
    double s = wave_sum(s0 + s1);
    double q = wave_sum(q0 + q1);
    if (lane == 0) { sh_s[wave] = s; sh_q[wave] = q; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kBatchThreads / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        finalize_qparams(S, Q, n, &sh_qp);
        if (qps) qps[t] = sh_qp;
        sh_hot_base = narrow_distribution(S, Q, n)
                          ? quantize_code(static_cast<float>(S / static_cast<double>(n)), sh_qp.inv_scale, kZeroPoint) - 1
                          : INT_MIN;
    }
    __syncthreads();
    const float inv = sh_qp.inv_scale;
    uint32_t* __restrict__ c4 = reinterpret_cast<uint32_t*>(codes);
    auto second_pass = [&](auto narrow_t) {
    constexpr bool narrow = decltype(narrow_t)::value;
    HotCodes hot;
    hot.base = sh_hot_base;
    auto add = [&](int code, float xv) {
        if (narrow) hist_add_hot(hist, hot, code, xv);
        else hist_add(hist, code, xv);
    };
    for (int64_t v0 = (a >> 2) + threadIdx.x; v0 < (b >> 2); v0 += kBatchThreads * U) {
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            v[j] = i < (b >> 2) ? x4[i] : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = v0 + j * kBatchThreads;
            if (i < (b >> 2)) {
                const int ca = quantize_code(v[j].x, inv, kZeroPoint);
                const int cb = quantize_code(v[j].y, inv, kZeroPoint);
                const int cc = quantize_code(v[j].z, inv, kZeroPoint);
                const int cd = quantize_code(v[j].w, inv, kZeroPoint);
                c4[i] = static_cast<uint32_t>(ca) | (static_cast<uint32_t>(cb) << 8) | (static_cast<uint32_t>(cc) << 16) |
                        (static_cast<uint32_t>(cd) << 24);
                add(ca, v[j].x);
                add(cb, v[j].y);
                add(cc, v[j].z);
                add(cd, v[j].w);
            }
        }
    }
    for (int part = 0; part < 2; ++part) {
        const int64_t from = part ? b : lo, to = part ? hi : a;
        for (int64_t i = from + threadIdx.x; i < to; i += kBatchThreads) {
            const float v = x[i];
            const int c = quantize_code(v, inv, kZeroPoint);
            codes[i] = static_cast<uint8_t>(c);
            add(c, v);
        }
    }
    if (narrow) hist_flush_hot(hist, hot);
    };
    if (sh_hot_base != INT_MIN) second_pass(std::true_type{});
    else second_pass(std::false_type{});
    __syncthreads();
    for (int bin = threadIdx.x; bin < kBins; bin += kBatchThreads) {
        double sum = 0.0;
        unsigned long long cnt = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) { sum += hist.sum[bin * R + r]; cnt += hist.cnt[bin * R + r]; }
        luts[t * kBins + bin] = cnt ? static_cast<float>(sum / static_cast<double>(cnt)) : 0.0f;
    }
}

__global__ void fill_zero_kernel(uint32_t* p, int64_t nwords) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < nwords;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = 0u;
}

// chunk /= world_size for ReduceOp::AVG (collectives.cpp:155-159): an fp32 division in place.
template <bool ALIGNED>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void div_kernel(float* __restrict__ x, int64_t n, float d) {
    using M = Mem<ALIGNED, false>;
    const int64_t nvec = n >> 2;
    constexpr int U = kDivUnroll;
    sweep<U>(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) M::stf4(x, i, v[j] / d, false);
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        x[i] = x[i] / d;
    }
}

// The pseudo-gradient of one bucket as Diloco.sync_pseudo_gradient forms it
// (src/zeroband/diloco.py:93-101): grad = outer_param - inner_param, then the whole flat buffer
// divided by the world size; an fp32 subtraction and an fp32 division per element.
// 12 bytes per element.
template <bool ALIGNED>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void pseudo_gradient_kernel(const float* __restrict__ outer,
                                                                                   const float* __restrict__ inner, int64_t n,
                                                                                   float world_size, float* __restrict__ out) {
    using M = Mem<ALIGNED, false>;
    const int64_t nvec = n >> 2;
    constexpr int U = kDivUnroll;
    sweep<U>(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a a[U], b[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            a[j] = ok ? M::ldf4(outer, i) : f4a{0.f, 0.f, 0.f, 0.f};
            b[j] = ok ? M::ldf4(inner, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) M::stf4(out, i, (a[j] - b[j]) / world_size, false);
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        out[i] = (outer[i] - inner[i]) / world_size;
    }
}

// A chunk's first touch in the ring when the pseudo-gradient has not been written yet: every
// chunk of a rank is visited exactly once in the reduce-scatter (collectives.cpp:115-116), so
// grad = (outer - inner) / world_size (diloco.py:93-101) can be formed in the pass that would
// otherwise read it back.  With CODES the received message is accumulated,
// acc = grad + lut[codes] (collectives.cpp:128-133), and with a divisor other than 1 the sum is
// divided (ReduceOp::AVG, :155-159).  The fp64 sum and sum of squares of what is stored are the
// statistics of the quantization that follows.  12 bytes per element, 13 with codes.
template <bool CODES, bool ALIGNED>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void first_touch_kernel(const float* __restrict__ outer,
                                                                               const float* __restrict__ inner, int64_t n,
                                                                               float world_size, const uint8_t* __restrict__ codes,
                                                                               const float* __restrict__ lut, float divisor,
                                                                               float* __restrict__ out, Workspace* ws) {
    using M = Mem<ALIGNED, false>;
    __shared__ float s_lut[kBins];
    if (CODES) {
        for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut[b];
        __syncthreads();
    }
    const bool div = divisor != 1.0f;
    const int64_t nvec = n >> 2;
    constexpr int U = kDivUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    sweep<U>(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a a[U], b[U];
        uint32_t c[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            a[j] = ok ? M::ldf4(outer, i) : f4a{0.f, 0.f, 0.f, 0.f};
            b[j] = ok ? M::ldf4(inner, i) : f4a{0.f, 0.f, 0.f, 0.f};
            if (CODES) c[j] = ok ? M::ldu32(codes, i) : 0u;
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t i = i0 + j * stride;
            f4a v = (a[j] - b[j]) / world_size;
            if (CODES) {
                f4a l;
                l.x = s_lut[c[j] & 255];
                l.y = s_lut[(c[j] >> 8) & 255];
                l.z = s_lut[(c[j] >> 16) & 255];
                l.w = s_lut[c[j] >> 24];
                v += l;
                if (div) v = v / divisor;
            }
            if (full || i < nvec) {
                M::stf4(out, i, v, false);       // the quantize pass reads it again: no streaming hint
                if (j & 1) stats_add4(v, s1, q1); else stats_add4(v, s0, q0);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float v = (outer[i] - inner[i]) / world_size;
        if (CODES) {
            v += s_lut[codes[i]];
            if (div) v = v / divisor;
        }
        out[i] = v;
        const double d = v;
        s0 += d;
        q0 = fma(d, d, q0);
    }
    block_stats_store(s0 + s1, q0 + q1, ws);
}

// One element of the outer optimizer, torch.optim.SGD(lr, momentum, nesterov=True) as the
// reference builds it (src/zeroband/diloco.py:72-74) and libtorch's CPU kernels round it:
//   buf = buf * mu + g     (a product and a sum, each rounded; buf = g on the first step)
//   d   = fma(buf, mu, g)  (add with alpha: one rounding)
//   p   = fma(d, -lr, p)
__device__ __forceinline__ void outer_sgd_one(float& p, float& buf, float g, float neg_lr, float mu, bool first) {
    buf = first ? g : buf * mu + g;
    const float d = fmaf(buf, mu, g);
    p = fmaf(d, neg_lr, p);
}

// Outer step of DiLoCo on one bucket (diloco.py:212-215): SGD with Nesterov momentum on the
// outer parameters with the reduced pseudo-gradient, and the copy of the new parameters to
// the inner model (sync_inner_model, :137-144) in the same pass.  The gradient is fp32
// (24 bytes per element) or, with CODES, uint8 codes and their lookup table (21 bytes per
// element, and the dequantize pass is saved).
template <bool CODES, bool ALIGNED>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void outer_step_kernel(float* __restrict__ param, float* __restrict__ mom,
                                                                              const float* __restrict__ grad,
                                                                              const uint8_t* __restrict__ codes,
                                                                              const float* __restrict__ lut,
                                                                              float* __restrict__ inner, int64_t n, float neg_lr,
                                                                              float mu, int first) {
    using M = Mem<ALIGNED, false>;
    __shared__ float s_lut[kBins];
    if (CODES) {
        for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut[b];
        __syncthreads();
    }
    const int64_t nvec = n >> 2;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a p[kUnroll], m[kUnroll], g[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            const bool ok = full || i < nvec;
            p[j] = ok ? M::ldf4(param, i) : f4a{0.f, 0.f, 0.f, 0.f};
            m[j] = (ok && !first) ? M::ldf4(mom, i) : f4a{0.f, 0.f, 0.f, 0.f};
            if (CODES) {
                const uint32_t c = ok ? M::ldu32(codes, i) : 0u;
                g[j] = f4a{s_lut[c & 255], s_lut[(c >> 8) & 255], s_lut[(c >> 16) & 255], s_lut[c >> 24]};
            } else {
                g[j] = ok ? M::ldf4(grad, i) : f4a{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float pc = p[j][c], mc = m[j][c];
                    outer_sgd_one(pc, mc, g[j][c], neg_lr, mu, first);
                    p[j][c] = pc;
                    m[j][c] = mc;
                }
                M::stf4(param, i, p[j], false);
                M::stf4(mom, i, m[j], false);
                if (inner) M::stf4(inner, i, p[j], true);
            }
        }
    });
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float p = param[i];
        float m = first ? 0.f : mom[i];
        const float g = CODES ? s_lut[codes[i]] : grad[i];
        outer_sgd_one(p, m, g, neg_lr, mu, first);
        param[i] = p;
        mom[i] = m;
        if (inner) inner[i] = p;
    }
}

__global__ __launch_bounds__(kThreads, kWavesPerSimd) void copy_kernel(f4a* __restrict__ dst, const f4a* __restrict__ src, int64_t nvec) {
    using M = Mem<true, false>;
    sweep(nvec, [&](int64_t i0, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        f4a v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) v[j] = M::ldf4(reinterpret_cast<const float*>(src), i);
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * stride;
            if (full || i < nvec) M::stf4(reinterpret_cast<float*>(dst), i, v[j], true);
        }
    });
}

// ---------------------------------------------------------------------------------------------
// host side

thread_local char g_err[256] = "";

int fail(int code, const char* what) {
    snprintf(g_err, sizeof(g_err), "%s", what);
    return code;
}

int hip_fail(hipError_t e, const char* where) {
    snprintf(g_err, sizeof(g_err), "%s: %s", where, hipGetErrorString(e));
    return static_cast<int>(e);
}

struct Options {
    int blocks_per_cu = PRIME_BLOCKS_PER_CU;
    int nt_load_min_mib = 512;      // tensors of at least this many MiB are loaded with the non-temporal hint
    int nt_second_min_mib = 0;      // the same for the quantize pass that re-reads a tensor: its last use, always hinted
    int hist_replicas = 8;          // 1, 2, 4, 8 or 16 copies of each LDS bin
};
Options g_opt;

int cu_count() {
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cus[dev] = v;
    }
    return cus[dev];
}

constexpr int64_t kRowElems = static_cast<int64_t>(kThreads) * 4;

// Workgroups for a streaming kernel: one per row of kThreads 16-byte vectors until the
// device is full (blocks_per_cu per compute unit), then each takes a longer span.
int grid_for(int64_t n) {
    int64_t tiles = (n + kRowElems - 1) / kRowElems;
    if (tiles < 1) tiles = 1;
    int64_t cap = static_cast<int64_t>(cu_count()) * g_opt.blocks_per_cu;
    if (cap > kMaxGrid) cap = kMaxGrid;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

inline bool use_nt(int64_t n) { return (n >> 18) >= g_opt.nt_load_min_mib; }   // n floats = n / 2^18 MiB

inline bool aligned_to(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int launch_check(const char* where) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, where);
}

// Optional per-launch timing with HIP events on the launch stream (prime_hip_profile_begin /
// _end): what a benchmark reads to price each kernel against the memory roofline.  Off by
// default; when off a launch site pays one branch.
enum KernelId {
    kIdStats, kIdStatsFinalize, kIdQuantize, kIdQuantizeHist, kIdHist, kIdLutFinalize, kIdDequantSet, kIdDequantAdd,
    kIdDequantAddStats, kIdDequantSetStats, kIdBatched, kIdCopy, kIdFill, kIdPseudoGrad, kIdOuterStep, kIdOuterStepCodes, kIdDiv, kIdFirstTouch, kIdFirstTouchCodes, kIdCodeCount, kIdCodeTotal, kIdRequantPlan, kIdCodeRemap, kIdNormLiteral, kIdCount
};
const char* const kKernelNames[kIdCount] = {
    "stats_kernel", "stats_finalize_kernel", "quantize_kernel", "quantize_kernel+hist", "hist_kernel", "lut_finalize_kernel",
    "dequant_kernel<set>", "dequant_kernel<add>", "dequant_kernel<add,stats>", "dequant_kernel<set,stats>",
    "batched_kernel", "copy_kernel", "fill_zero_kernel", "pseudo_gradient_kernel", "outer_step_kernel", "outer_step_kernel<codes>", "div_kernel",
    "first_touch_kernel", "first_touch_kernel<codes>", "code_count_kernel", "code_total_kernel", "requant_plan_kernel", "code_remap_kernel", "norm_literal_kernel"};

struct TimedLaunch {
    int id;
    double bytes;
    hipEvent_t a, b;
};
struct Profiler {
    std::atomic<bool> on{false};
    std::mutex m;
    std::vector<TimedLaunch> launches;
};
Profiler g_prof;

// Every kernel launch of the library goes through here.  With timing on, the launch carries a
// start and a stop event that take the dispatch's own begin and end timestamps (the same
// interval a kernel trace reports); otherwise it is a plain launch.
template <typename... KArgs, typename... Args>
void launch(int id, double algo_bytes, void (*kernel)(KArgs...), int grid, int threads, hipStream_t st, Args... args) {
    if (!g_prof.on) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, st, static_cast<KArgs>(args)...);
        return;
    }
    TimedLaunch t{};
    t.id = id;
    t.bytes = algo_bytes;
    if (hipEventCreate(&t.a) != hipSuccess || hipEventCreate(&t.b) != hipSuccess) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, st, static_cast<KArgs>(args)...);
        return;
    }
    hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(threads), 0, st, t.a, t.b, 0, static_cast<KArgs>(args)...);
    std::lock_guard<std::mutex> lock(g_prof.m);
    g_prof.launches.push_back(t);
}

int run_stats_finalize(Workspace* ws, int nparts, int64_t n, prime_qparams* out, hipStream_t st) {
    launch(kIdStatsFinalize, 16.0 * nparts, stats_finalize_kernel, 1, kFinalThreads, st, ws, nparts, n, out);
    return launch_check("stats_finalize_kernel");
}

// First stage only: returns the number of partials through *parts.
int run_stats_partials(const float* x, int64_t n, Workspace* ws, hipStream_t st, int* parts) {
    const int grid = grid_for(n);
    if (!aligned_to(x, 16))
        launch(kIdStats, 4.0 * n, stats_kernel<false, false>, grid, kThreads, st, x, n, ws);
    else if (use_nt(n))
        launch(kIdStats, 4.0 * n, stats_kernel<true, true>, grid, kThreads, st, x, n, ws);
    else
        launch(kIdStats, 4.0 * n, stats_kernel<true, false>, grid, kThreads, st, x, n, ws);
    *parts = grid;
    return launch_check("stats_kernel");
}

int run_stats(const float* x, int64_t n, prime_qparams* out, Workspace* ws, hipStream_t st) {
    int parts = 0;
    if (int rc = run_stats_partials(x, n, ws, st, &parts)) return rc;
    return run_stats_finalize(ws, parts, n, out, st);
}

template <bool HIST, int R>
void launch_quantize_r(bool al, int grid, hipStream_t st, const float* x, int64_t n, float scale, int stats_parts,
                       prime_qparams* qp_out, int zp, uint8_t* codes, Workspace* ws) {
    const int id = HIST ? kIdQuantizeHist : kIdQuantize;
    if (!al)
        launch(id, 5.0 * n, quantize_kernel<false, false, HIST, R>, grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws);
    else if (stats_parts > 0 ? (n >> 18) >= g_opt.nt_second_min_mib : use_nt(n))
        launch(id, 5.0 * n, quantize_kernel<true, true, HIST, R>, grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws);
    else
        launch(id, 5.0 * n, quantize_kernel<true, false, HIST, R>, grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws);
}

// stats_parts > 0: take the scale from that many statistics partials in the workspace (and
// publish it to qp_out); otherwise use `scale`.  Returns the grid size through *grid_out: the
// number of histogram partials written.
int run_quantize(const float* x, int64_t n, float scale, int stats_parts, prime_qparams* qp_out, int zp, uint8_t* codes,
                 Workspace* ws, bool hist, hipStream_t st, int* grid_out) {
    const int grid = grid_for(n);
    const bool al = aligned_to(x, 16) && aligned_to(codes, 4);
    if (!hist) {
        launch_quantize_r<false, 1>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws);
    } else {
        switch (g_opt.hist_replicas) {
            case 1: launch_quantize_r<true, 1>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws); break;
            case 2: launch_quantize_r<true, 2>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws); break;
            default: launch_quantize_r<true, 8>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws); break;
            case 16: launch_quantize_r<true, 16>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws); break;
            case 4: launch_quantize_r<true, 4>(al, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws); break;
        }
    }
    if (grid_out) *grid_out = grid;
    return launch_check("quantize_kernel");
}

int run_lut_finalize(const Workspace* ws, int nparts, float* lut, int64_t n_bins, uint64_t* counts, hipStream_t st) {
    if (nparts == 0) {
        launch(kIdLutFinalize, 0.0, lut_zero_kernel, 1, 256, st, lut, n_bins, reinterpret_cast<unsigned long long*>(counts));
        return launch_check("lut_zero_kernel");
    }
    launch(kIdLutFinalize, 16.0 * kBins * nparts, lut_finalize_kernel, kBins / kLutBinsPerBlock, kFinalThreads, st, ws, nparts, lut,
           n_bins, reinterpret_cast<unsigned long long*>(counts));
    return launch_check("lut_finalize_kernel");
}

template <bool ADD, bool STATS, bool DIV = false>
int run_dequant(float* out, const float* lut, const uint8_t* codes, int64_t n, Workspace* ws, hipStream_t st, int* grid_out,
                float divisor = 1.0f) {
    const int grid = grid_for(n);
    const int id = STATS ? (ADD ? kIdDequantAddStats : kIdDequantSetStats) : (ADD ? kIdDequantAdd : kIdDequantSet);
    const double bytes = (ADD ? 9.0 : 5.0) * n;
    if (!(aligned_to(out, 16) && aligned_to(codes, 4)))
        launch(id, bytes, dequant_kernel<ADD, STATS, false, false, DIV>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
    else if (use_nt(n))
        launch(id, bytes, dequant_kernel<ADD, STATS, true, true, DIV>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
    else
        launch(id, bytes, dequant_kernel<ADD, STATS, true, false, DIV>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
    if (grid_out) *grid_out = grid;
    return launch_check("dequant_kernel");
}

// Workgroups for a kernel that streams 16 codes per lane and step.
int grid_for_codes(int64_t n) { return grid_for((n + 3) / 4); }

// (codes_out, lut_out) = uniform_8bit_quantize(lut_in[codes_in]) without the fp32 tensor.
int run_requantize_codes(const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out, float* lut_out,
                         prime_qparams* qp_out, Workspace* ws, hipStream_t st) {
    const int grid = grid_for_codes(n);
    const bool al = aligned_to(codes_in, 16) && aligned_to(codes_out, 16);
    if (al)
        launch(kIdCodeCount, 1.0 * n, code_count_kernel<true, PRIME_COUNT_REPLICAS>, grid, kThreads, st, codes_in, n, ws);
    else
        launch(kIdCodeCount, 1.0 * n, code_count_kernel<false, PRIME_COUNT_REPLICAS>, grid, kThreads, st, codes_in, n, ws);
    if (int rc = launch_check("code_count_kernel")) return rc;
    launch(kIdCodeTotal, 4.0 * kBins * grid, code_total_kernel, kBins / kLutBinsPerBlock, kFinalThreads, st, ws, grid);
    if (int rc = launch_check("code_total_kernel")) return rc;
    launch(kIdRequantPlan, 0.0, requant_plan_kernel, 1, kFinalThreads, st, ws, lut_in, n, lut_out, qp_out);
    if (int rc = launch_check("requant_plan_kernel")) return rc;
    if (al)
        launch(kIdCodeRemap, 2.0 * n, code_remap_kernel<true>, grid, kThreads, st, codes_in, codes_out, n, ws);
    else
        launch(kIdCodeRemap, 2.0 * n, code_remap_kernel<false>, grid, kThreads, st, codes_in, codes_out, n, ws);
    return launch_check("code_remap_kernel");
}

bool bad_n(int64_t n) { return n < 0 || n > kMaxElems; }

}  // namespace

extern "C" {

int prime_hip_abi_version(void) { return PRIME_HIP_ABI_VERSION; }

const char* prime_hip_last_error(void) { return g_err; }

int prime_hip_set_option(const char* name, int value) {
    if (!name) return fail(PRIME_EINVAL, "option name is null");
    if (!strcmp(name, "blocks_per_cu")) {
        if (value < 1 || value > 16) return fail(PRIME_EINVAL, "blocks_per_cu must be 1..16");
        g_opt.blocks_per_cu = value;
    } else if (!strcmp(name, "hist_replicas")) {
        if (value != 1 && value != 2 && value != 4 && value != 8 && value != 16)
            return fail(PRIME_EINVAL, "hist_replicas must be 1, 2, 4, 8 or 16");
        g_opt.hist_replicas = value;
    } else if (!strcmp(name, "nt_load_min_mib")) {
        if (value < 0) return fail(PRIME_EINVAL, "nt_load_min_mib must be >= 0");
        g_opt.nt_load_min_mib = value;
    } else if (!strcmp(name, "nt_second_min_mib")) {
        if (value < 0) return fail(PRIME_EINVAL, "nt_second_min_mib must be >= 0");
        g_opt.nt_second_min_mib = value;
    } else {
        return fail(PRIME_EINVAL, "unknown option");
    }
    return 0;
}

int prime_hip_get_option(const char* name, int* value) {
    if (!name || !value) return fail(PRIME_EINVAL, "null argument");
    if (!strcmp(name, "blocks_per_cu")) *value = g_opt.blocks_per_cu;
    else if (!strcmp(name, "hist_replicas")) *value = g_opt.hist_replicas;
    else if (!strcmp(name, "nt_load_min_mib")) *value = g_opt.nt_load_min_mib;
    else if (!strcmp(name, "nt_second_min_mib")) *value = g_opt.nt_second_min_mib;
    else if (!strcmp(name, "unroll")) *value = kUnroll;
    else if (!strcmp(name, "threads")) *value = kThreads;
    else return fail(PRIME_EINVAL, "unknown option");
    return 0;
}

int prime_hip_profile_begin(void) {
    std::lock_guard<std::mutex> lock(g_prof.m);
    for (auto& t : g_prof.launches) { (void)hipEventDestroy(t.a); (void)hipEventDestroy(t.b); }
    g_prof.launches.clear();
    g_prof.on = true;
    return 0;
}

int prime_hip_profile_end(prime_kernel_time* out, int capacity, int* count) {
    if (!out || !count || capacity < 0) return fail(PRIME_EINVAL, "prime_hip_profile_end: bad argument");
    std::lock_guard<std::mutex> lock(g_prof.m);
    g_prof.on = false;
    prime_kernel_time acc[kIdCount];
    memset(acc, 0, sizeof(acc));
    int rc = 0;
    for (auto& t : g_prof.launches) {
        float ms = 0.f;
        hipError_t e = hipEventSynchronize(t.b);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, t.a, t.b);
        if (e != hipSuccess && rc == 0) rc = hip_fail(e, "prime_hip_profile_end");
        acc[t.id].launches += 1;
        acc[t.id].total_ms += ms;
        acc[t.id].algo_bytes += t.bytes;
        (void)hipEventDestroy(t.a);
        (void)hipEventDestroy(t.b);
    }
    g_prof.launches.clear();
    int k = 0;
    for (int id = 0; id < kIdCount; ++id) {
        if (!acc[id].launches) continue;
        if (k < capacity) {
            snprintf(acc[id].name, sizeof(acc[id].name), "%s", kKernelNames[id]);
            out[k] = acc[id];
        }
        ++k;
    }
    *count = k;
    return rc;
}

int64_t prime_workspace_bytes(void) { return static_cast<int64_t>(sizeof(Workspace)); }

int prime_workspace_init(void* ws, int64_t ws_bytes, prime_stream_t stream) {
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    if (ws_bytes < static_cast<int64_t>(sizeof(Workspace))) return fail(PRIME_EWORKSPACE, "workspace too small");
    if (!aligned_to(ws, 16)) return fail(PRIME_EWORKSPACE, "workspace must be 16-byte aligned");
    // Only the scale record is ever read before it is written by the same call sequence;
    // clear it so that a stray read is defined.
    launch(kIdFill, 0.0, fill_zero_kernel, 1, 64, static_cast<hipStream_t>(stream), static_cast<uint32_t*>(ws),
           static_cast<int64_t>(sizeof(prime_qparams) / 4));
    return launch_check("fill_zero_kernel");
}

int prime_stats_f32(const float* x, int64_t n, prime_qparams* out, void* ws, prime_stream_t stream) {
    if (bad_n(n) || (!x && n > 0) || !out) return fail(PRIME_EINVAL, "prime_stats_f32: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    return run_stats(x, n, out, static_cast<Workspace*>(ws), static_cast<hipStream_t>(stream));
}

int prime_quantize_u8(const float* x, int64_t n, float scale, int32_t zero_point, uint8_t* codes, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!x || !codes))) return fail(PRIME_EINVAL, "prime_quantize_u8: bad argument");
    if (n == 0) return 0;
    return run_quantize(x, n, scale, 0, nullptr, zero_point, codes, nullptr, false, static_cast<hipStream_t>(stream), nullptr);
}

int prime_average_buckets(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins, float* lut, uint64_t* counts,
                          void* ws, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_average_buckets: bad argument");
    if (n_bins < 1 || n_bins > (1 << 24)) return fail(PRIME_EINVAL, "prime_average_buckets: n_bins out of range");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    int grid = 0;
    if (n > 0) {
        grid = grid_for(n);
        const int nb = static_cast<int>(n_bins < kBins ? n_bins : kBins);
        if (aligned_to(x, 16) && aligned_to(codes, 4))
            launch(kIdHist, 5.0 * n, hist_kernel<true, 8>, grid, kThreads, st, x, codes, n, nb, w);
        else
            launch(kIdHist, 5.0 * n, hist_kernel<false, 8>, grid, kThreads, st, x, codes, n, nb, w);
        if (int rc = launch_check("hist_kernel")) return rc;
    }
    return run_lut_finalize(w, grid, lut, n_bins, counts, st);
}

int prime_quantize_lookup_u8(const float* x, int64_t n, float scale, uint8_t* codes, float* lut, void* ws,
                             prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_quantize_lookup_u8: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    int grid = 0;
    if (n > 0)
        if (int rc = run_quantize(x, n, scale, 0, nullptr, kZeroPoint, codes, w, true, st, &grid)) return rc;
    return run_lut_finalize(w, grid, lut, kBins, nullptr, st);
}

int prime_uniform_8bit_quantize(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out, void* ws,
                                prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n == 0) {
        if (int rc = run_stats(x, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, 0, lut, kBins, nullptr, st);
    }
    int parts = 0, grid = 0;
    if (int rc = run_stats_partials(x, n, w, st, &parts)) return rc;
    if (int rc = run_quantize(x, n, 0.0f, parts, qparams_out, kZeroPoint, codes, w, true, st, &grid)) return rc;
    return run_lut_finalize(w, grid, lut, kBins, nullptr, st);
}

int prime_norm_literal_f32(const float* x, int64_t n, prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && !x)) return fail(PRIME_EINVAL, "prime_norm_literal_f32: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    launch(kIdNormLiteral, 4.0 * n, norm_literal_kernel, 1, kFinalThreads, static_cast<hipStream_t>(stream), x, n,
           static_cast<Workspace*>(ws), qparams_out);
    return launch_check("norm_literal_kernel");
}

int prime_uniform_8bit_quantize_literal(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out,
                                        void* ws, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_literal: bad argument");
    if (int rc = prime_norm_literal_f32(x, n, qparams_out, ws, stream)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    int grid = 0;
    if (n > 0)
        if (int rc = run_quantize(x, n, 0.0f, -1, nullptr, kZeroPoint, codes, w, true, st, &grid)) return rc;
    return run_lut_finalize(w, grid, lut, kBins, nullptr, st);
}

int prime_uniform_8bit_quantize_buckets(const float* const* xs, const int64_t* ns, int64_t count, uint8_t* const* codes,
                                        float* luts, prime_qparams* qparams_out, void* const* workspaces,
                                        const prime_stream_t* streams, int n_streams) {
    if (count < 0 || n_streams < 1 || (count > 0 && (!xs || !ns || !codes || !luts)) || !workspaces || !streams)
        return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_buckets: bad argument");
    for (int k = 0; k < n_streams; ++k)
        if (!workspaces[k]) return fail(PRIME_EWORKSPACE, "prime_uniform_8bit_quantize_buckets: a workspace is null");
    for (int64_t i = 0; i < count; ++i) {
        const int k = static_cast<int>(i % n_streams);
        if (int rc = prime_uniform_8bit_quantize(xs[i], ns[i], codes[i], luts + i * kBins, qparams_out ? qparams_out + i : nullptr,
                                                 workspaces[k], streams[k]))
            return rc;
    }
    return 0;
}

int prime_uniform_8bit_quantize_batched(const float* x, const int64_t* offsets, int64_t count, uint8_t* codes, float* luts,
                                        prime_qparams* qparams_out, prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!offsets || !luts))) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_batched: bad argument");
    if (count > 0x7fffffff) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_batched: too many tensors");
    if (count == 0) return 0;
    if (aligned_to(x, 16) && aligned_to(codes, 4))
        launch(kIdBatched, 0.0, batched_kernel<true>, static_cast<int>(count), kBatchThreads, static_cast<hipStream_t>(stream), x,
               offsets, codes, luts, qparams_out);
    else
        launch(kIdBatched, 0.0, batched_kernel<false>, static_cast<int>(count), kBatchThreads, static_cast<hipStream_t>(stream), x,
               offsets, codes, luts, qparams_out);
    return launch_check("batched_kernel");
}

int prime_dequant_set(float* out, const float* lut, const uint8_t* codes, int64_t n, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!out || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_dequant_set: bad argument");
    if (n == 0) return 0;
    return run_dequant<false, false>(out, lut, codes, n, nullptr, static_cast<hipStream_t>(stream), nullptr);
}

int prime_dequant_add(float* out, const float* lut, const uint8_t* codes, int64_t n, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!out || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_dequant_add: bad argument");
    if (n == 0) return 0;
    return run_dequant<true, false>(out, lut, codes, n, nullptr, static_cast<hipStream_t>(stream), nullptr);
}

int prime_requantize_codes(const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out, float* lut_out,
                           prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!codes_in || !codes_out)) || !lut_in || !lut_out)
        return fail(PRIME_EINVAL, "prime_requantize_codes: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n == 0) {
        if (int rc = run_stats(lut_in, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, 0, lut_out, kBins, nullptr, st);
    }
    return run_requantize_codes(codes_in, lut_in, n, codes_out, lut_out, qparams_out, w, st);
}

}  // extern "C"

namespace {

// One received message of the ring: chunk (+)= lut_in[codes_in] with the statistics of the
// result taken in the same pass, then the requantization of the chunk.
template <bool ADD>
int ring_step(float* chunk, const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out, float* lut_out,
              prime_qparams* qparams_out, void* ws, prime_stream_t stream, const char* who, float divisor = 1.0f) {
    if (bad_n(n) || (n > 0 && (!chunk || !codes_in || !codes_out)) || !lut_in || !lut_out) return fail(PRIME_EINVAL, who);
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n == 0) {
        if (int rc = run_stats(chunk, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, 0, lut_out, kBins, nullptr, st);
    }
    int grid = 0;
    if (ADD && divisor != 1.0f) {
        if (int rc = run_dequant<ADD, true, ADD>(chunk, lut_in, codes_in, n, w, st, &grid, divisor)) return rc;
    } else {
        if (int rc = run_dequant<ADD, true>(chunk, lut_in, codes_in, n, w, st, &grid)) return rc;
    }
    if (int rc = run_quantize(chunk, n, 0.0f, grid, qparams_out, kZeroPoint, codes_out, w, true, st, &grid)) return rc;
    return run_lut_finalize(w, grid, lut_out, kBins, nullptr, st);
}

}  // namespace

extern "C" {

int prime_ring_reduce_step(float* acc, const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out,
                           float* lut_out, prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    return ring_step<true>(acc, codes_in, lut_in, n, codes_out, lut_out, qparams_out, ws, stream,
                           "prime_ring_reduce_step: bad argument");
}

int prime_ring_reduce_div_step(float* acc, const uint8_t* codes_in, const float* lut_in, int64_t n, float divisor,
                               uint8_t* codes_out, float* lut_out, prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    if (!(divisor == divisor) || divisor == 0.0f) return fail(PRIME_EINVAL, "prime_ring_reduce_div_step: divisor must be a non-zero number");
    return ring_step<true>(acc, codes_in, lut_in, n, codes_out, lut_out, qparams_out, ws, stream,
                           "prime_ring_reduce_div_step: bad argument", divisor);
}

int prime_ring_gather_step(float* chunk, const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out,
                           float* lut_out, prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    return ring_step<false>(chunk, codes_in, lut_in, n, codes_out, lut_out, qparams_out, ws, stream,
                            "prime_ring_gather_step: bad argument");
}

int prime_div_f32(float* x, int64_t n, float divisor, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && !x)) return fail(PRIME_EINVAL, "prime_div_f32: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (aligned_to(x, 16))
        launch(kIdDiv, 8.0 * n, div_kernel<true>, grid_for(n), kThreads, st, x, n, divisor);
    else
        launch(kIdDiv, 8.0 * n, div_kernel<false>, grid_for(n), kThreads, st, x, n, divisor);
    return launch_check("div_kernel");
}

int prime_pseudo_gradient_f32(const float* outer, const float* inner, int64_t n, float world_size, float* out,
                              prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!outer || !inner || !out))) return fail(PRIME_EINVAL, "prime_pseudo_gradient_f32: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = grid_for(n);
    if (aligned_to(outer, 16) && aligned_to(inner, 16) && aligned_to(out, 16))
        launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<true>, grid, kThreads, st, outer, inner, n, world_size, out);
    else
        launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<false>, grid, kThreads, st, outer, inner, n, world_size, out);
    return launch_check("pseudo_gradient_kernel");
}

int prime_ring_first_touch(const float* outer, const float* inner, int64_t n, float world_size, const uint8_t* codes_in,
                           const float* lut_in, float divisor, float* grad_out, uint8_t* codes_out, float* lut_out,
                           prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!outer || !inner || !grad_out || !codes_out)) || !lut_out || (codes_in && !lut_in))
        return fail(PRIME_EINVAL, "prime_ring_first_touch: bad argument");
    if (!(divisor == divisor) || divisor == 0.0f) return fail(PRIME_EINVAL, "prime_ring_first_touch: divisor must be a non-zero number");
    if (!codes_in && divisor != 1.0f)
        return fail(PRIME_EINVAL, "prime_ring_first_touch: a divisor goes with a received message only (fold it into world_size)");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n == 0) {
        if (int rc = run_stats(outer, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, 0, lut_out, kBins, nullptr, st);
    }
    int grid = grid_for(n);
    const bool al = aligned_to(outer, 16) && aligned_to(inner, 16) && aligned_to(grad_out, 16) && (!codes_in || aligned_to(codes_in, 4));
    if (codes_in) {
        if (al)
            launch(kIdFirstTouchCodes, 13.0 * n, first_touch_kernel<true, true>, grid, kThreads, st, outer, inner, n, world_size,
                   codes_in, lut_in, divisor, grad_out, w);
        else
            launch(kIdFirstTouchCodes, 13.0 * n, first_touch_kernel<true, false>, grid, kThreads, st, outer, inner, n, world_size,
                   codes_in, lut_in, divisor, grad_out, w);
    } else {
        if (al)
            launch(kIdFirstTouch, 12.0 * n, first_touch_kernel<false, true>, grid, kThreads, st, outer, inner, n, world_size,
                   nullptr, nullptr, 1.0f, grad_out, w);
        else
            launch(kIdFirstTouch, 12.0 * n, first_touch_kernel<false, false>, grid, kThreads, st, outer, inner, n, world_size,
                   nullptr, nullptr, 1.0f, grad_out, w);
    }
    if (int rc = launch_check("first_touch_kernel")) return rc;
    if (int rc = run_quantize(grad_out, n, 0.0f, grid, qparams_out, kZeroPoint, codes_out, w, true, st, &grid)) return rc;
    return run_lut_finalize(w, grid, lut_out, kBins, nullptr, st);
}

int prime_outer_sgd_nesterov_f32(float* param, float* momentum_buf, const float* grad, float* inner_out, int64_t n, float lr,
                                 float momentum, int first_step, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!param || !momentum_buf || !grad)))
        return fail(PRIME_EINVAL, "prime_outer_sgd_nesterov_f32: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = grid_for(n);
    const bool al = aligned_to(param, 16) && aligned_to(momentum_buf, 16) && aligned_to(grad, 16) && aligned_to(inner_out, 16);
    const double bytes = (inner_out ? 24.0 : 20.0) * n;
    if (al)
        launch(kIdOuterStep, bytes, outer_step_kernel<false, true>, grid, kThreads, st, param, momentum_buf, grad, nullptr, nullptr,
               inner_out, n, -lr, momentum, first_step);
    else
        launch(kIdOuterStep, bytes, outer_step_kernel<false, false>, grid, kThreads, st, param, momentum_buf, grad, nullptr, nullptr,
               inner_out, n, -lr, momentum, first_step);
    return launch_check("outer_step_kernel");
}

int prime_outer_sgd_nesterov_u8(float* param, float* momentum_buf, const uint8_t* codes, const float* lut, float* inner_out,
                                int64_t n, float lr, float momentum, int first_step, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!param || !momentum_buf || !codes)) || !lut)
        return fail(PRIME_EINVAL, "prime_outer_sgd_nesterov_u8: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = grid_for(n);
    const bool al = aligned_to(param, 16) && aligned_to(momentum_buf, 16) && aligned_to(codes, 4) && aligned_to(inner_out, 16);
    const double bytes = (inner_out ? 21.0 : 17.0) * n;
    if (al)
        launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, true>, grid, kThreads, st, param, momentum_buf, nullptr, codes, lut,
               inner_out, n, -lr, momentum, first_step);
    else
        launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, false>, grid, kThreads, st, param, momentum_buf, nullptr, codes, lut,
               inner_out, n, -lr, momentum, first_step);
    return launch_check("outer_step_kernel");
}

int prime_copy_bytes(void* dst, const void* src, int64_t n_bytes, prime_stream_t stream) {
    if (n_bytes < 0 || (n_bytes > 0 && (!dst || !src))) return fail(PRIME_EINVAL, "prime_copy_bytes: bad argument");
    if ((n_bytes & 15) || !aligned_to(dst, 16) || !aligned_to(src, 16))
        return fail(PRIME_EINVAL, "prime_copy_bytes: size and pointers must be multiples of 16");
    if (n_bytes == 0) return 0;
    const int64_t nvec = n_bytes >> 4;
    const int grid = grid_for(nvec * 4);
    launch(kIdCopy, 2.0 * n_bytes, copy_kernel, grid, kThreads, static_cast<hipStream_t>(stream), static_cast<f4a*>(dst),
           static_cast<const f4a*>(src), nvec);
    return launch_check("copy_kernel");
}

}  // extern "C"
