// libprime_hip.so - HIP kernels (gfx950 / CDNA4, wave64) and C ABI for the int8 pseudo-gradient
// compression path: fp64 statistics, uint8 quantization, 256-bin lookup build, lookup
// dequantization and the ring's accumulate + requantize step.  All kernels are HBM-bound
// streams: 16-byte loads per lane, 256-thread workgroups that loop over tiles, histogram
// traffic kept in LDS and merged once per workgroup.
//
// Arithmetic follows the reference's CPU ops (paths relative to the reference checkout):
//   src/zeroband/C/csrc/compression.cpp:9-43    quantize      -> quantize_code()
//   src/zeroband/C/csrc/compression.cpp:45-104  average       -> hist_add() / lut_finalize_kernel
//   src/zeroband/C/csrc/compression.cpp:106-125 scale formula -> finalize_qparams()
//   src/zeroband/C/csrc/collectives.cpp:8-22    index add/set -> dequant_kernel
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/prime_hip.h"

namespace {

constexpr int kThreads = 256;            // 4 wavefronts of 64
constexpr int kWaves = kThreads / 64;
constexpr int kBins = 256;               // compression.cpp:5
constexpr int kZeroPoint = 128;          // compression.cpp:107
constexpr int kMaxGrid = 4096;           // partial-sum slots in the workspace
constexpr int kUnroll = 4;               // 16-byte loads in flight per lane

struct Workspace {
    uint32_t ticket;                     // grid-level "last workgroup" counter, 0 between calls
    uint32_t pad[3];
    prime_qparams qp;                    // scale of the tensor in flight
    double hist_sum[kBins];              // 0 between calls
    unsigned long long hist_cnt[kBins];  // 0 between calls
    double part_sum[kMaxGrid];
    double part_sq[kMaxGrid];
};

typedef float f4a __attribute__((ext_vector_type(4)));                 // 16-byte aligned
typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));     // element aligned only
typedef uint32_t u32a;
typedef uint32_t u32u __attribute__((aligned(1)));

template <bool ALIGNED> struct Vec;
template <> struct Vec<true> { using f4 = f4a; using u32 = u32a; };
template <> struct Vec<false> { using f4 = f4u; using u32 = u32u; };

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
__device__ __forceinline__ void finalize_qparams(double sum, double sumsq, int64_t n, prime_qparams* qp) {
    const float norm = static_cast<float>(sqrt(sumsq));
    const double std_unbiased = static_cast<double>(norm) / sqrt(static_cast<double>(n - 1));
    const double scale = 6.0 * std_unbiased / 256.0;
    const float sf = static_cast<float>(scale);
    qp->scale = sf;
    qp->inv_scale = 1.0f / sf;           // compression.cpp:16
    qp->sum = sum;
    qp->sumsq = sumsq;
    qp->n = n;
}

// Workgroup reduction of (sum, sumsq), one partial per workgroup, and a second stage run by
// whichever workgroup takes the last ticket.  The second stage adds the partials in a fixed
// order, so the scale does not depend on scheduling.
__device__ __forceinline__ void block_stats_finish(double s, double q, int64_t n, Workspace* ws,
                                                   prime_qparams* out) {
    __shared__ double sh_s[kWaves];
    __shared__ double sh_q[kWaves];
    __shared__ int sh_last;
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
        __threadfence();
        const unsigned t = __hip_atomic_fetch_add(&ws->ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        sh_last = (t == gridDim.x - 1);
    }
    __syncthreads();
    if (!sh_last) return;
    __threadfence();
    double a = 0.0, b = 0.0;
    for (int i = threadIdx.x; i < static_cast<int>(gridDim.x); i += kThreads) {
        a += ws->part_sum[i];
        b += ws->part_sq[i];
    }
    a = wave_sum(a);
    b = wave_sum(b);
    __syncthreads();
    if (lane == 0) { sh_s[wave] = a; sh_q[wave] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        finalize_qparams(S, Q, n, &ws->qp);
        if (out) *out = ws->qp;
        ws->ticket = 0;
    }
}

__device__ __forceinline__ void stats_add4(const f4a v, double& s, double& q) {
    const double a = v.x, b = v.y, c = v.z, d = v.w;
    s += a; q = fma(a, a, q);
    s += b; q = fma(b, b, q);
    s += c; q = fma(c, c, q);
    s += d; q = fma(d, d, q);
}

// K1: sum and sum of squares in fp64.  4 bytes per element.
template <bool ALIGNED>
__global__ __launch_bounds__(kThreads) void stats_kernel(const float* __restrict__ x, int64_t n, Workspace* ws,
                                                         prime_qparams* out) {
    using f4 = typename Vec<ALIGNED>::f4;
    const f4* __restrict__ x4 = reinterpret_cast<const f4*>(x);
    const int64_t nvec = n >> 2;
    const int64_t tile = static_cast<int64_t>(kThreads) * kUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    for (int64_t base = blockIdx.x * tile; base < nvec; base += static_cast<int64_t>(gridDim.x) * tile) {
        f4a v[kUnroll];
        const int64_t i0 = base + threadIdx.x;
        if (base + tile <= nvec) {
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) v[j] = x4[i0 + j * kThreads];
        } else {
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                const int64_t i = i0 + j * kThreads;
                v[j] = i < nvec ? static_cast<f4a>(x4[i]) : f4a{0.f, 0.f, 0.f, 0.f};
            }
        }
        stats_add4(v[0], s0, q0);
        stats_add4(v[1], s1, q1);
        stats_add4(v[2], s0, q0);
        stats_add4(v[3], s1, q1);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const double v = x[(nvec << 2) + threadIdx.x];
        s0 += v;
        q0 = fma(v, v, q0);
    }
    block_stats_finish(s0 + s1, q0 + q1, n, ws, out);
}

// LDS histogram: R copies of each bin, chosen by lane, so that lanes of one wavefront that
// hit the same bin mostly hit different addresses (and banks).  Sums are fp64, counts u32
// (a workgroup never sees 2^32 elements: the grid is sized so that it cannot).
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

// Merge a workgroup's histogram into the workspace accumulators (one fp64 and one u64
// hardware atomic per non-empty bin).
template <int R>
__device__ __forceinline__ void hist_flush(LdsHist<R>& h, Workspace* ws) {
    const int b = threadIdx.x;   // kThreads == kBins
    double s = 0.0;
    unsigned long long c = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) { s += h.sum[b * R + r]; c += h.cnt[b * R + r]; }
    if (c) {
        unsafeAtomicAdd(&ws->hist_sum[b], s);
        __hip_atomic_fetch_add(&ws->hist_cnt[b], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// K2 (+K3 when HIST): quantize to uint8, 4 codes packed per 32-bit store, and the 256-bin
// sum / count histogram of the same elements.  5 bytes per element.
template <bool ALIGNED, bool HIST, int R>
__global__ __launch_bounds__(kThreads) void quantize_kernel(const float* __restrict__ x, int64_t n, float scale_val,
                                                            const prime_qparams* __restrict__ qp, int zero_point,
                                                            uint8_t* __restrict__ codes, Workspace* ws, int reverse) {
    using f4 = typename Vec<ALIGNED>::f4;
    using u32 = typename Vec<ALIGNED>::u32;
    __shared__ LdsHist<HIST ? R : 1> hist;
    if (HIST) {
        hist_zero(hist);
        __syncthreads();
    }
    const float inv = qp ? qp->inv_scale : 1.0f / scale_val;
    const f4* __restrict__ x4 = reinterpret_cast<const f4*>(x);
    u32* __restrict__ c4 = reinterpret_cast<u32*>(codes);
    const int64_t nvec = n >> 2;
    const int64_t tile = static_cast<int64_t>(kThreads) * kUnroll;
    const int64_t ntiles = (nvec + tile - 1) / tile;
    for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const int64_t base = (reverse ? ntiles - 1 - t : t) * tile;
        const int64_t i0 = base + threadIdx.x;
        f4a v[kUnroll];
        const bool full = base + tile <= nvec;
        if (full) {
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) v[j] = x4[i0 + j * kThreads];
        } else {
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                const int64_t i = i0 + j * kThreads;
                v[j] = i < nvec ? static_cast<f4a>(x4[i]) : f4a{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * kThreads;
            if (full || i < nvec) {
                const int a = quantize_code(v[j].x, inv, zero_point);
                const int b = quantize_code(v[j].y, inv, zero_point);
                const int c = quantize_code(v[j].z, inv, zero_point);
                const int d = quantize_code(v[j].w, inv, zero_point);
                c4[i] = static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) |
                        (static_cast<uint32_t>(c) << 16) | (static_cast<uint32_t>(d) << 24);
                if (HIST) {
                    hist_add(hist, a, v[j].x);
                    hist_add(hist, b, v[j].y);
                    hist_add(hist, c, v[j].z);
                    hist_add(hist, d, v[j].w);
                }
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        const float v = x[i];
        const int a = quantize_code(v, inv, zero_point);
        codes[i] = static_cast<uint8_t>(a);
        if (HIST) hist_add(hist, a, v);
    }
    if (HIST) {
        __syncthreads();
        hist_flush(hist, ws);
    }
}

// K3 alone: histogram of x under caller-supplied codes (average_buckets).  5 bytes per element.
template <bool ALIGNED, int R>
__global__ __launch_bounds__(kThreads) void hist_kernel(const float* __restrict__ x, const uint8_t* __restrict__ codes,
                                                        int64_t n, int n_bins, Workspace* ws) {
    using f4 = typename Vec<ALIGNED>::f4;
    using u32 = typename Vec<ALIGNED>::u32;
    __shared__ LdsHist<R> hist;
    hist_zero(hist);
    __syncthreads();
    const f4* __restrict__ x4 = reinterpret_cast<const f4*>(x);
    const u32* __restrict__ c4 = reinterpret_cast<const u32*>(codes);
    const int64_t nvec = n >> 2;
    for (int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; i < nvec;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        const f4a v = x4[i];
        const uint32_t c = c4[i];
        const int a = c & 255, b = (c >> 8) & 255, cc = (c >> 16) & 255, d = c >> 24;
        if (a < n_bins) hist_add(hist, a, v.x);     // compression.cpp:70
        if (b < n_bins) hist_add(hist, b, v.y);
        if (cc < n_bins) hist_add(hist, cc, v.z);
        if (d < n_bins) hist_add(hist, d, v.w);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        const int a = codes[i];
        if (a < n_bins) hist_add(hist, a, x[i]);
    }
    __syncthreads();
    hist_flush(hist, ws);
}

// Turn the workspace accumulators into the lookup table and clear them for the next call.
// Mean = fp64 sum / count, rounded to float once; an empty bin gives 0.0f (compression.cpp:100).
__global__ __launch_bounds__(kThreads) void lut_finalize_kernel(Workspace* ws, float* __restrict__ lut, int64_t n_bins,
                                                                unsigned long long* __restrict__ counts) {
    for (int64_t b = threadIdx.x; b < n_bins; b += kThreads) {
        float m = 0.0f;
        if (b < kBins) {
            const double s = ws->hist_sum[b];
            const unsigned long long c = ws->hist_cnt[b];
            if (c) m = static_cast<float>(s / static_cast<double>(c));
            if (counts) counts[b] = c;
        }
        lut[b] = m;
    }
    ws->hist_sum[threadIdx.x] = 0.0;
    ws->hist_cnt[threadIdx.x] = 0ull;
}

// K5 / K4 pass A: out = lut[codes] (collectives.cpp:16-22) or out += lut[codes] (:8-14),
// the lookup table held in LDS; with STATS the fp64 sum and sum of squares of the updated
// values are taken in the same pass (the next quantization's scale).
template <bool ADD, bool STATS, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void dequant_kernel(float* __restrict__ out, const float* __restrict__ lut,
                                                           const uint8_t* __restrict__ codes, int64_t n, Workspace* ws,
                                                           prime_qparams* qp_out) {
    using f4 = typename Vec<ALIGNED>::f4;
    using u32 = typename Vec<ALIGNED>::u32;
    __shared__ float s_lut[kBins];
    s_lut[threadIdx.x] = lut[threadIdx.x];
    __syncthreads();
    f4* __restrict__ o4 = reinterpret_cast<f4*>(out);
    const u32* __restrict__ c4 = reinterpret_cast<const u32*>(codes);
    const int64_t nvec = n >> 2;
    const int64_t tile = static_cast<int64_t>(kThreads) * kUnroll;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    for (int64_t base = blockIdx.x * tile; base < nvec; base += static_cast<int64_t>(gridDim.x) * tile) {
        const int64_t i0 = base + threadIdx.x;
        const bool full = base + tile <= nvec;
        uint32_t c[kUnroll];
        f4a a[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * kThreads;
            const bool ok = full || i < nvec;
            c[j] = ok ? static_cast<uint32_t>(c4[i]) : 0u;
            if (ADD) a[j] = ok ? static_cast<f4a>(o4[i]) : f4a{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const int64_t i = i0 + j * kThreads;
            f4a v;
            v.x = s_lut[c[j] & 255];
            v.y = s_lut[(c[j] >> 8) & 255];
            v.z = s_lut[(c[j] >> 16) & 255];
            v.w = s_lut[c[j] >> 24];
            if (ADD) v += a[j];
            if (full || i < nvec) {
                o4[i] = v;
                if (STATS) {
                    if (j & 1) stats_add4(v, s1, q1); else stats_add4(v, s0, q0);
                }
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        float v = s_lut[codes[i]];
        if (ADD) v += out[i];
        out[i] = v;
        if (STATS) {
            const double d = v;
            s0 += d;
            q0 = fma(d, d, q0);
        }
    }
    if (STATS) block_stats_finish(s0 + s1, q0 + q1, n, ws, qp_out);
}

// Small tensors: one workgroup per tensor of a flat buffer does the whole of
// uniform_8bit_quantize (statistics, scale, codes, lookup) without touching the workspace.
__global__ __launch_bounds__(kThreads) void batched_kernel(const float* __restrict__ x, const int64_t* __restrict__ offsets,
                                                           uint8_t* __restrict__ codes, float* __restrict__ luts,
                                                           prime_qparams* __restrict__ qps) {
    __shared__ LdsHist<1> hist;
    __shared__ double sh_s[kWaves];
    __shared__ double sh_q[kWaves];
    __shared__ prime_qparams sh_qp;
    const int64_t t = blockIdx.x;
    const int64_t lo = offsets[t];
    const int64_t n = offsets[t + 1] - lo;
    const float* __restrict__ xp = x + lo;
    uint8_t* __restrict__ cp = codes + lo;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    hist_zero(hist);
    double s = 0.0, q = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += kThreads) {
        const double v = xp[i];
        s += v;
        q = fma(v, v, q);
    }
    s = wave_sum(s);
    q = wave_sum(q);
    if (lane == 0) { sh_s[wave] = s; sh_q[wave] = q; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        finalize_qparams(S, Q, n, &sh_qp);
        if (qps) qps[t] = sh_qp;
    }
    __syncthreads();
    const float inv = sh_qp.inv_scale;
    for (int64_t i = threadIdx.x; i < n; i += kThreads) {
        const float v = xp[i];
        const int c = quantize_code(v, inv, kZeroPoint);
        cp[i] = static_cast<uint8_t>(c);
        hist_add(hist, c, v);
    }
    __syncthreads();
    const unsigned c = hist.cnt[threadIdx.x];
    luts[t * kBins + threadIdx.x] = c ? static_cast<float>(hist.sum[threadIdx.x] / static_cast<double>(c)) : 0.0f;
}

__global__ void fill_zero_kernel(uint32_t* p, int64_t nwords) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < nwords;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = 0u;
}

__global__ __launch_bounds__(kThreads) void copy_kernel(f4a* __restrict__ dst, const f4a* __restrict__ src, int64_t nvec) {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; i < nvec;
         i += static_cast<int64_t>(gridDim.x) * kThreads)
        dst[i] = src[i];
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
    int blocks_per_cu = 8;
    int hist_replicas = 4;          // 1, 2, 4 or 8 copies of each LDS bin
    int reverse_second_pass = 0;    // walk the quantize pass from the end of the tensor
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

// Workgroups for a kernel whose workgroups each loop over tiles of `tile_elems` elements.
int grid_for(int64_t n, int64_t tile_elems) {
    int64_t tiles = (n + tile_elems - 1) / tile_elems;
    if (tiles < 1) tiles = 1;
    int64_t cap = static_cast<int64_t>(cu_count()) * g_opt.blocks_per_cu;
    if (cap > kMaxGrid) cap = kMaxGrid;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

inline bool aligned_to(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

constexpr int64_t kTileElems = static_cast<int64_t>(kThreads) * kUnroll * 4;

int launch_check(const char* where) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, where);
}

int run_stats(const float* x, int64_t n, prime_qparams* out, Workspace* ws, hipStream_t st) {
    const int grid = grid_for(n, kTileElems);
    if (aligned_to(x, 16))
        hipLaunchKernelGGL(stats_kernel<true>, dim3(grid), dim3(kThreads), 0, st, x, n, ws, out);
    else
        hipLaunchKernelGGL(stats_kernel<false>, dim3(grid), dim3(kThreads), 0, st, x, n, ws, out);
    return launch_check("stats_kernel");
}

template <bool HIST, int R>
void launch_quantize_r(bool al, int grid, hipStream_t st, const float* x, int64_t n, float scale, const prime_qparams* qp,
                       int zp, uint8_t* codes, Workspace* ws, int reverse) {
    if (al)
        hipLaunchKernelGGL((quantize_kernel<true, HIST, R>), dim3(grid), dim3(kThreads), 0, st, x, n, scale, qp, zp, codes, ws, reverse);
    else
        hipLaunchKernelGGL((quantize_kernel<false, HIST, R>), dim3(grid), dim3(kThreads), 0, st, x, n, scale, qp, zp, codes, ws, reverse);
}

int run_quantize(const float* x, int64_t n, float scale, const prime_qparams* qp, int zp, uint8_t* codes, Workspace* ws,
                 bool hist, int reverse, hipStream_t st) {
    const int grid = grid_for(n, kTileElems);
    const bool al = aligned_to(x, 16) && aligned_to(codes, 4);
    if (!hist) {
        launch_quantize_r<false, 1>(al, grid, st, x, n, scale, qp, zp, codes, ws, reverse);
    } else {
        switch (g_opt.hist_replicas) {
            case 1: launch_quantize_r<true, 1>(al, grid, st, x, n, scale, qp, zp, codes, ws, reverse); break;
            case 2: launch_quantize_r<true, 2>(al, grid, st, x, n, scale, qp, zp, codes, ws, reverse); break;
            case 8: launch_quantize_r<true, 8>(al, grid, st, x, n, scale, qp, zp, codes, ws, reverse); break;
            default: launch_quantize_r<true, 4>(al, grid, st, x, n, scale, qp, zp, codes, ws, reverse); break;
        }
    }
    return launch_check("quantize_kernel");
}

int run_lut_finalize(Workspace* ws, float* lut, int64_t n_bins, uint64_t* counts, hipStream_t st) {
    hipLaunchKernelGGL(lut_finalize_kernel, dim3(1), dim3(kThreads), 0, st, ws, lut, n_bins,
                       reinterpret_cast<unsigned long long*>(counts));
    return launch_check("lut_finalize_kernel");
}

template <bool ADD, bool STATS>
int run_dequant(float* out, const float* lut, const uint8_t* codes, int64_t n, Workspace* ws, prime_qparams* qp_out,
                hipStream_t st) {
    const int grid = grid_for(n, kTileElems);
    if (aligned_to(out, 16) && aligned_to(codes, 4))
        hipLaunchKernelGGL((dequant_kernel<ADD, STATS, true>), dim3(grid), dim3(kThreads), 0, st, out, lut, codes, n, ws, qp_out);
    else
        hipLaunchKernelGGL((dequant_kernel<ADD, STATS, false>), dim3(grid), dim3(kThreads), 0, st, out, lut, codes, n, ws, qp_out);
    return launch_check("dequant_kernel");
}

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
        if (value != 1 && value != 2 && value != 4 && value != 8) return fail(PRIME_EINVAL, "hist_replicas must be 1, 2, 4 or 8");
        g_opt.hist_replicas = value;
    } else if (!strcmp(name, "reverse_second_pass")) {
        g_opt.reverse_second_pass = value ? 1 : 0;
    } else {
        return fail(PRIME_EINVAL, "unknown option");
    }
    return 0;
}

int prime_hip_get_option(const char* name, int* value) {
    if (!name || !value) return fail(PRIME_EINVAL, "null argument");
    if (!strcmp(name, "blocks_per_cu")) *value = g_opt.blocks_per_cu;
    else if (!strcmp(name, "hist_replicas")) *value = g_opt.hist_replicas;
    else if (!strcmp(name, "reverse_second_pass")) *value = g_opt.reverse_second_pass;
    else return fail(PRIME_EINVAL, "unknown option");
    return 0;
}

int64_t prime_workspace_bytes(void) { return static_cast<int64_t>(sizeof(Workspace)); }

int prime_workspace_init(void* ws, int64_t ws_bytes, prime_stream_t stream) {
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    if (ws_bytes < static_cast<int64_t>(sizeof(Workspace))) return fail(PRIME_EWORKSPACE, "workspace too small");
    if (!aligned_to(ws, 16)) return fail(PRIME_EWORKSPACE, "workspace must be 16-byte aligned");
    const int64_t words = static_cast<int64_t>(sizeof(Workspace) / 4);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(32), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint32_t*>(ws), words);
    return launch_check("fill_zero_kernel");
}

int prime_stats_f32(const float* x, int64_t n, prime_qparams* out, void* ws, prime_stream_t stream) {
    if (n < 0 || (!x && n > 0) || !out) return fail(PRIME_EINVAL, "prime_stats_f32: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    return run_stats(x, n, out, static_cast<Workspace*>(ws), static_cast<hipStream_t>(stream));
}

int prime_quantize_u8(const float* x, int64_t n, float scale, int32_t zero_point, uint8_t* codes, prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!x || !codes))) return fail(PRIME_EINVAL, "prime_quantize_u8: bad argument");
    if (n == 0) return 0;
    return run_quantize(x, n, scale, nullptr, zero_point, codes, nullptr, false, 0, static_cast<hipStream_t>(stream));
}

int prime_average_buckets(const float* x, const uint8_t* codes, int64_t n, int64_t n_bins, float* lut, uint64_t* counts,
                          void* ws, prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_average_buckets: bad argument");
    if (n_bins < 1 || n_bins > (1 << 24)) return fail(PRIME_EINVAL, "prime_average_buckets: n_bins out of range");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n > 0) {
        const int grid = grid_for(n, static_cast<int64_t>(kThreads) * 4 * 4);
        const int nb = static_cast<int>(n_bins < kBins ? n_bins : kBins);
        if (aligned_to(x, 16) && aligned_to(codes, 4))
            hipLaunchKernelGGL((hist_kernel<true, 4>), dim3(grid), dim3(kThreads), 0, st, x, codes, n, nb, w);
        else
            hipLaunchKernelGGL((hist_kernel<false, 4>), dim3(grid), dim3(kThreads), 0, st, x, codes, n, nb, w);
        if (int rc = launch_check("hist_kernel")) return rc;
    }
    return run_lut_finalize(w, lut, n_bins, counts, st);
}

int prime_quantize_lookup_u8(const float* x, int64_t n, float scale, uint8_t* codes, float* lut, void* ws,
                             prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_quantize_lookup_u8: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n > 0)
        if (int rc = run_quantize(x, n, scale, nullptr, kZeroPoint, codes, w, true, 0, st)) return rc;
    return run_lut_finalize(w, lut, kBins, nullptr, st);
}

int prime_uniform_8bit_quantize(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out, void* ws,
                                prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (int rc = run_stats(x, n, qparams_out, w, st)) return rc;
    if (n > 0)
        if (int rc = run_quantize(x, n, 0.0f, &w->qp, kZeroPoint, codes, w, true, g_opt.reverse_second_pass, st)) return rc;
    return run_lut_finalize(w, lut, kBins, nullptr, st);
}

int prime_uniform_8bit_quantize_batched(const float* x, const int64_t* offsets, int64_t count, uint8_t* codes, float* luts,
                                        prime_qparams* qparams_out, prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!offsets || !luts))) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_batched: bad argument");
    if (count > 0x7fffffff) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_batched: too many tensors");
    if (count == 0) return 0;
    hipLaunchKernelGGL(batched_kernel, dim3(static_cast<unsigned>(count)), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       x, offsets, codes, luts, qparams_out);
    return launch_check("batched_kernel");
}

int prime_dequant_set(float* out, const float* lut, const uint8_t* codes, int64_t n, prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!out || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_dequant_set: bad argument");
    if (n == 0) return 0;
    return run_dequant<false, false>(out, lut, codes, n, nullptr, nullptr, static_cast<hipStream_t>(stream));
}

int prime_dequant_add(float* out, const float* lut, const uint8_t* codes, int64_t n, prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!out || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_dequant_add: bad argument");
    if (n == 0) return 0;
    return run_dequant<true, false>(out, lut, codes, n, nullptr, nullptr, static_cast<hipStream_t>(stream));
}

int prime_ring_reduce_step(float* acc, const uint8_t* codes_in, const float* lut_in, int64_t n, uint8_t* codes_out,
                           float* lut_out, prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    if (n < 0 || (n > 0 && (!acc || !codes_in || !codes_out)) || !lut_in || !lut_out)
        return fail(PRIME_EINVAL, "prime_ring_reduce_step: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (n == 0) {
        if (int rc = run_stats(acc, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, lut_out, kBins, nullptr, st);
    }
    if (int rc = run_dequant<true, true>(acc, lut_in, codes_in, n, w, qparams_out, st)) return rc;
    if (int rc = run_quantize(acc, n, 0.0f, &w->qp, kZeroPoint, codes_out, w, true, g_opt.reverse_second_pass, st)) return rc;
    return run_lut_finalize(w, lut_out, kBins, nullptr, st);
}

int prime_copy_bytes(void* dst, const void* src, int64_t n_bytes, prime_stream_t stream) {
    if (n_bytes < 0 || (n_bytes > 0 && (!dst || !src))) return fail(PRIME_EINVAL, "prime_copy_bytes: bad argument");
    if ((n_bytes & 15) || !aligned_to(dst, 16) || !aligned_to(src, 16))
        return fail(PRIME_EINVAL, "prime_copy_bytes: size and pointers must be multiples of 16");
    if (n_bytes == 0) return 0;
    const int64_t nvec = n_bytes >> 4;
    const int grid = grid_for(nvec, kThreads);
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<f4a*>(dst), static_cast<const f4a*>(src), nvec);
    return launch_check("copy_kernel");
}

}  // extern "C"
