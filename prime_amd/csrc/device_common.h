// Shared device-side pieces of the streaming kernels: tuning constants, the workspace layout,
// aligned / element-aligned memory access, the quantizer of one element, the scale formula,
// workgroup reductions, the work distribution (sweep) and the LDS histogram.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.


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
