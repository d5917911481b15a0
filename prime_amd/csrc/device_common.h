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
#ifndef PRIME_BATCH_THREADS
#define PRIME_BATCH_THREADS 512
#endif
constexpr int kBatchThreads = PRIME_BATCH_THREADS;   // workgroup of the one-tensor-per-workgroup kernel
constexpr int kWaves = kThreads / 64;
constexpr int kBins = 256;               // compression.cpp:5
constexpr int kZeroPoint = 128;          // compression.cpp:107
constexpr int kMaxGrid = 2048;           // per-workgroup partial slots in the workspace
constexpr int kUnroll = PRIME_UNROLL;
constexpr int kDivUnroll = PRIME_UNROLL > 2 ? 2 : PRIME_UNROLL;   // vectors per step in the kernels that divide
#ifndef PRIME_SHOT_THREADS
#define PRIME_SHOT_THREADS 256
#endif
constexpr int kShotThreads = PRIME_SHOT_THREADS;   // workgroup of a one-tile-per-workgroup launch
#ifndef PRIME_SHOT_UNROLL
#define PRIME_SHOT_UNROLL 2
#endif
constexpr int kShotUnroll = PRIME_SHOT_UNROLL;   // rows of its tile
// The tile of a one-workgroup-per-tile launch, by kind of kernel (lanes, rows of that many 16-byte vectors).  Kernels that
// only stream (copy, divide, pseudo-gradient, outer step) do best with the smallest tile there is, one wavefront and one
// vector per lane: at 2^28 elements the pseudo-gradient takes 482 us instead of 552 (256 lanes, two rows), the outer step
// 1060 instead of 1160, a copy 321 instead of 347.  Kernels that first bring the lookup table into LDS want that cost spread
// over more lanes: accumulate 128 lanes x 2 rows (373 against 380 us), outer step from codes 128 x 1 (915 against 1005),
// set 256 x 2 (211; 64 x 1: 389); the plain quantizer (16 bytes in, 4 out) 256 x 2 (208; 64 x 1: 257).
#ifndef PRIME_STREAM_SHOT_THREADS
#define PRIME_STREAM_SHOT_THREADS 64
#endif
#ifndef PRIME_STREAM_SHOT_ROWS
#define PRIME_STREAM_SHOT_ROWS 1
#endif
constexpr int kStreamShotThreads = PRIME_STREAM_SHOT_THREADS, kStreamShotRows = PRIME_STREAM_SHOT_ROWS;
constexpr int kCodesStepShotThreads = 128, kCodesStepShotRows = 1;
constexpr int kAddShotThreads = 128, kAddShotRows = 2;
// wavefronts per SIMD the streaming kernels are compiled for (4 SIMDs per compute unit, at
// most 8 wavefronts each): bounds their register use so that PRIME_BLOCKS_PER_CU workgroups fit
constexpr int kWavesPerSimd = (PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4 > 8 ? 8
                              : ((PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4 < 1 ? 1 : (PRIME_THREADS / 64) * PRIME_BLOCKS_PER_CU / 4);
constexpr int kFinalThreads = 1024;      // workgroup size of the second-stage kernels
constexpr int kLutBinsPerBlock = 4;      // bins one second-stage workgroup reduces (64 bytes per partial)
constexpr int64_t kMaxElems = int64_t(1) << 40;   // per-workgroup counts are 32-bit

constexpr int kSegMax = 64;              // tensors of one segmented launch (their descriptors travel as kernel arguments)

// One bin of a workgroup's histogram partial, 16 bytes, in one of two forms.  BinAcc: the fp64 sum
// of the bin's elements and their number.  BinPart (the fixed-point histogram of the fused quantize
// pass): the integer sum of the elements' residuals from the centre of the bin, in units of 2^-22 of
// a bin width, and their number.  Integer partials add up to the same totals whichever workgroup saw
// which element, so the table built from them does not depend on how the tensor was dealt out.
struct BinAcc {
    double sum;
    unsigned long long cnt;
};
struct BinPart {
    long long units;
    unsigned long long cnt;
};
// Where a workgroup leaves its elements beyond the range of the fixed-point residual (they all have
// code 0 or 255): their number and the fp64 sum of their values, per side (0: code 0, 1: code 255).
// The workspace keeps them as one array per side and quantity, indexed by workgroup, so that the
// second stage reads them with coalesced loads; side 1 lies kMaxGrid entries after side 0.
struct FarSlot {
    double* sum;
    unsigned long long* cnt;
};
// Which of the two forms the partials of the launch before have, and the 1 / scale their residuals refer to.
enum { kHistFp = 0, kHistFixed = 1 };
struct HistInfo {
    float inv;
    int mode;
};

// What one tensor of a segmented launch leaves between the kernels.
struct SegRecord {
    prime_qparams qp;
    HistInfo info;
    int pad[2];
};

// Every kernel stores its per-workgroup partial results here with plain stores; the kernel
// boundary makes them visible to the second stage.  Nothing has to be zero between calls.
struct Workspace {
    prime_qparams qp;                    // scale of the tensor in flight
    uint32_t code_map[kBins / 4];        // old code -> new code of a requantization in the code domain
    unsigned long long code_total[kBins];   // population of each code over the whole tensor
    HistInfo hist_info;                  // form of the histogram partials below
    unsigned tile_counter;               // next tile of the part of a pass that is dealt out on demand
    unsigned pad;
    double part_sum[kMaxGrid];
    double part_sq[kMaxGrid];
    double far_sum[2][kMaxGrid];
    unsigned long long far_cnt[2][kMaxGrid];
    union alignas(16) {
        BinAcc hist[kMaxGrid][kBins];    // 4 KiB per workgroup
        BinPart hist_fixed[kMaxGrid][kBins];
        uint32_t code_cnt[kMaxGrid][kBins];   // per-workgroup populations of each code value
    };
    // segmented launches: per tensor the record and the statistics partials of as many workgroups as
    // the one-tensor entry point would launch for it; the histogram partials share the rows above
    SegRecord seg[kSegMax];
    double seg_part_sum[kSegMax][kMaxGrid];
    double seg_part_sq[kSegMax][kMaxGrid];
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

// Cache policy of a streamed store (the cache-policy bits of gfx950 memory instructions).
// Write-through (agent scope: the line leaves the XCD's L2 at once instead of waiting there,
// dirty, for an eviction that then competes with the read stream) is the fastest for the code
// and fp32 outputs that sit beside a larger read stream; non-temporal is the fastest for a plain
// copy far larger than the last-level cache; plain write-back is best when the next kernel reads
// the data back at once.
constexpr int kStorePlain = 0;
constexpr int kStoreNt = 2;              // nt
constexpr int kStoreWriteThrough = 16;   // sc1

// A window of a buffer for buffer instructions: a wave-uniform base plus a 32-bit byte offset
// per lane.  The hardware drops stores and returns zero for loads at or beyond `bytes`.
struct Window {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ Window(const void* base, int64_t bytes) {
        const int64_t lim = bytes < 0 ? 0 : (bytes > 0x7fffffff ? 0x7fffffff : bytes);
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(lim), 0x00020000);
    }
    template <int POLICY>
    __device__ __forceinline__ void st32(uint32_t byte_off, uint32_t v) const {
        __builtin_amdgcn_raw_buffer_store_b32(v, rsrc, static_cast<int>(byte_off), 0, POLICY);
    }
    template <int POLICY>
    __device__ __forceinline__ void st128(uint32_t byte_off, f4a v) const {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4a, v), rsrc, static_cast<int>(byte_off), 0, POLICY);
    }
};

// The value of lane i + N of the same row of 16 lanes (N < 16), by data-parallel primitives: no LDS
// traffic, unlike a shuffle.  Lanes whose source lies outside their row get an unspecified value.
template <int N>
__device__ __forceinline__ double row_down(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = static_cast<int>(b), hi = static_cast<int>(b >> 32);
    const int lo2 = __builtin_amdgcn_update_dpp(lo, lo, 0x100 + N, 0xf, 0xf, false);     // row_shl:N
    const int hi2 = __builtin_amdgcn_update_dpp(hi, hi, 0x100 + N, 0xf, 0xf, false);
    return __longlong_as_double((static_cast<long long>(hi2) << 32) | static_cast<unsigned>(lo2));
}

// Sum over the wavefront, valid in lane 0: lane i adds lane i + 32, then i + 16, 8, 4, 2, 1 (a fixed
// tree, so the result depends on the values alone).  Lane 0 only ever takes from lanes below 16 in
// the last four steps, which therefore stay inside a row.
__device__ __forceinline__ double wave_sum(double v) {
    v += __shfl_down(v, 32, 64);
    v += __shfl_down(v, 16, 64);
    v += row_down<8>(v);
    v += row_down<4>(v);
    v += row_down<2>(v);
    v += row_down<1>(v);
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

// sqrt(n - 1) of the scale formula, for a caller that computes it ahead of the sums (the root of an
// integer-valued double is the same correctly rounded value wherever it is taken).
__device__ __forceinline__ double root_of_n_minus_1(int64_t n) { return sqrt(static_cast<double>(n - 1)); }

__device__ __forceinline__ void finalize_from_norm_root(float norm, double root_nm1, double sum, double sumsq, int64_t n, prime_qparams* qp) {
    const double std_unbiased = static_cast<double>(norm) / root_nm1;
    const double scale = 6.0 * std_unbiased / 256.0;
    const float sf = static_cast<float>(scale);
    qp->scale = sf;
    qp->inv_scale = 1.0f / sf;           // compression.cpp:16
    qp->sum = sum;
    qp->sumsq = sumsq;
    qp->n = n;
}

__device__ __forceinline__ void finalize_from_norm(float norm, double sum, double sumsq, int64_t n, prime_qparams* qp) {
    finalize_from_norm_root(norm, root_of_n_minus_1(n), sum, sumsq, n, qp);
}

// Workgroup reduction of (sum, sumsq) in a fixed order; the workgroup's partial goes to the
// workspace for stats_finalize_kernel.
__device__ __forceinline__ void block_stats_store(double s, double q, double* part_sum, double* part_sq, int slot) {
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
        part_sum[slot] = S;
        part_sq[slot] = Q;
    }
}
__device__ __forceinline__ void block_stats_store(double s, double q, Workspace* ws, int slot) {
    block_stats_store(s, q, ws->part_sum, ws->part_sq, slot);
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
// bit for bit and no separate launch is needed.  Returns 1 / scale; the workgroup with `publish`
// set stores the record to `rec` and, if given, `out`.
// The reduction itself: lane i brings the partial sums of workgroup i (and of i + THREADS, ...)
// already added up as a (sum) and b (sum of squares).
template <int THREADS>
__device__ __forceinline__ float block_scale_reduce(double a, double b, int64_t n, bool publish, prime_qparams* rec, prime_qparams* out,
                                                    int* hot_base) {
    __shared__ double sh_s[THREADS / 64];
    __shared__ double sh_q[THREADS / 64];
    __shared__ float sh_inv;
    __shared__ float sh_mean;
    __shared__ int sh_narrow;
    // sqrt(n - 1) does not wait for the sums: taken here, ahead of the barrier (the empty statement keeps it here)
    double root_nm1 = root_of_n_minus_1(n);
    asm volatile("" : "+v"(root_nm1));
    a = wave_sum(a);
    b = wave_sum(b);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sh_s[wave] = a; sh_q[wave] = b; }
    __syncthreads();
    // two chains of fp64 divisions and roots hang on the sums: the scale, and whether the tensor crowds into a few
    // codes (and which).  The first lanes of two wavefronts take one each, side by side; both add the wavefronts'
    // sums in the same order.
    constexpr int kSecond = THREADS > 64 ? 64 : 0;
    if (threadIdx.x == 0 || threadIdx.x == kSecond) {
        double S = sh_s[0], Q = sh_q[0];
#pragma unroll
        for (int w = 1; w < THREADS / 64; ++w) { S += sh_s[w]; Q += sh_q[w]; }
        if (threadIdx.x == 0) {
            prime_qparams qp;
            finalize_from_norm_root(static_cast<float>(sqrt(Q)), root_nm1, S, Q, n, &qp);
            sh_inv = qp.inv_scale;
            if (publish) {
                *rec = qp;
                if (out) *out = qp;
            }
        }
        if (threadIdx.x == kSecond) {
            sh_narrow = narrow_distribution(S, Q, n);
            sh_mean = static_cast<float>(S / static_cast<double>(n));
        }
    }
    __syncthreads();
    const float inv = sh_inv;
    if (hot_base) *hot_base = sh_narrow ? quantize_code(sh_mean, inv, kZeroPoint) - 1 : INT_MIN;
    return inv;
}

// `meanwhile()` runs between the issue of the partials' loads and their first use: work of the calling kernel
// that does not depend on the scale (zeroing its LDS tables) goes there, under the loads' trip to memory.
struct NothingMeanwhile { __device__ __forceinline__ void operator()() const {} };

template <int THREADS, typename Meanwhile = NothingMeanwhile>
__device__ __forceinline__ float block_scale_from_partials(const double* part_sum, const double* part_sq, int nparts, int64_t n,
                                                           bool publish, prime_qparams* rec, prime_qparams* out, int* hot_base = nullptr,
                                                           Meanwhile&& meanwhile = Meanwhile{}) {
    constexpr int kIters = (kMaxGrid + THREADS - 1) / THREADS;
    double ps[kIters], pq[kIters];
#pragma unroll
    for (int k = 0; k < kIters; ++k) {       // all loads in flight at once
        const int i = threadIdx.x + k * THREADS;
        ps[k] = i < nparts ? part_sum[i] : 0.0;
        pq[k] = i < nparts ? part_sq[i] : 0.0;
    }
    meanwhile();
    double a = 0.0, b = 0.0;
#pragma unroll
    for (int k = 0; k < kIters; ++k) { a += ps[k]; b += pq[k]; }
    return block_scale_reduce<THREADS>(a, b, n, publish, rec, out, hot_base);
}

template <int THREADS, typename Meanwhile = NothingMeanwhile>
__device__ __forceinline__ float block_scale_from_partials(Workspace* ws, int nparts, int64_t n, prime_qparams* out,
                                                           int* hot_base = nullptr, Meanwhile&& meanwhile = Meanwhile{}) {
    return block_scale_from_partials<THREADS>(ws->part_sum, ws->part_sq, nparts, n, blockIdx.x == 0, &ws->qp, out, hot_base,
                                              static_cast<Meanwhile&&>(meanwhile));
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
// sweep_tiles hands body the workgroup-uniform first vector of the piece (the lane adds threadIdx.x),
// which a buffer window needs as its base, and with REVERSE walks the tensor from its end: a pass that
// re-reads what the pass before it has just streamed then starts with the part the last-level
// cache still holds instead of the part that has already been displaced.
// sweep_tiles_of walks the share of workgroup `slot` of `G`; sweep_tiles and sweep walk the calling workgroup's own.
template <int U = kUnroll, bool REVERSE = false, typename Body>
__device__ __forceinline__ void sweep_tiles_of(int64_t nvec, int64_t slot, int64_t G, Body&& body) {
    const int64_t rows = (nvec + kThreads - 1) / kThreads;
    const int64_t rounds = (nvec / kThreads) / (G * U);
    const int64_t r0 = rounds * G * U + slot;
    if (REVERSE && r0 < rows) body(r0 * kThreads, G * kThreads, std::false_type{});
    for (int64_t kk = 0; kk < rounds; ++kk) {
        const int64_t k = REVERSE ? rounds - 1 - kk : kk;
        body(((k * G + slot) * U) * kThreads, static_cast<int64_t>(kThreads), std::true_type{});
    }
    if (!REVERSE && r0 < rows) body(r0 * kThreads, G * kThreads, std::false_type{});
}

// The same walk with the last part of the whole tiles dealt on demand.  The workgroups of a long
// launch do not finish together (on a 2^28-element pass the first ends 10 % ahead of the last), and
// tiles that are handed out one by one near the end fill that gap.  `dyn_percent` of the rounds are
// taken out of the round-robin deal and handed out through `counter` (device memory that holds 0
// when the launch starts; null: everything stays round-robin): a workgroup asks for its next tile
// while it streams the one before, so the trip to the counter is not waited for.  Which workgroup
// gets which of these tiles differs from run to run: only for passes whose per-workgroup results add
// up to the same totals in any order (integer histogram partials; codes depend on nothing but the
// element).  Every workgroup of the launch must call this (it uses barriers while tiles are left).
//
// mix_rounds (REVERSE only): the last that many rounds of the tensor are in the last-level cache (the pass before
// left them there).  Instead of first, they are visited spread evenly among the rounds of the part that comes
// from memory, so that cache and memory deliver side by side for the whole pass instead of one after the other.
template <int U, bool REVERSE, typename Body>
__device__ __forceinline__ void sweep_tiles_dynamic(int64_t nvec, int64_t slot, int64_t G, unsigned* counter, int dyn_percent, Body&& body,
                                                    int64_t mix_rounds = 0) {
    __shared__ unsigned sh_next[2];
    const int64_t rows = (nvec + kThreads - 1) / kThreads;
    const int64_t rounds = (nvec / kThreads) / (G * U);
    const int64_t dyn_rounds = counter ? rounds * dyn_percent / 100 : 0;
    const int64_t static_rounds = rounds - dyn_rounds;
    const int64_t dyn_tiles = dyn_rounds * G;
    const int64_t r0 = rounds * G * U + slot;
    // forward: static tiles [0, static_rounds * G), then the dynamic ones, then the ragged rows;
    // reverse: the ragged rows, static tiles from the end down to dyn_tiles, then the dynamic ones [0, dyn_tiles) downwards
    if (REVERSE && r0 < rows) body(r0 * kThreads, G * kThreads, std::false_type{});
    const bool mixed = REVERSE && mix_rounds > 0 && mix_rounds < static_rounds;
    for (int64_t kk = 0; kk < static_rounds; ++kk) {
        int64_t k = REVERSE ? rounds - 1 - kk : kk;
        if (mixed) {
            // the cached rounds spread evenly over the walk: position kk takes one when the running share crosses an integer
            const int64_t before = kk * mix_rounds / static_rounds, after = (kk + 1) * mix_rounds / static_rounds;
            k = after > before ? rounds - 1 - before : rounds - 1 - mix_rounds - (kk - before);
        }
        body(((k * G + slot) * U) * kThreads, static_cast<int64_t>(kThreads), std::true_type{});
    }
    if (dyn_tiles > 0) {
        if (threadIdx.x == 0) sh_next[0] = atomicAdd(counter, 1u);
        __syncthreads();
        unsigned cur = sh_next[0];
        int ph = 0;
        while (cur < dyn_tiles) {
            unsigned ahead = 0;
            if (threadIdx.x == 0) ahead = atomicAdd(counter, 1u);          // the tile after this one, asked for while this one streams
            const int64_t tile = REVERSE ? dyn_tiles - 1 - cur : static_rounds * G + cur;
            body((tile * U) * kThreads, static_cast<int64_t>(kThreads), std::true_type{});
            if (threadIdx.x == 0) sh_next[ph ^ 1] = ahead;
            __syncthreads();
            cur = sh_next[ph ^ 1];
            ph ^= 1;
        }
    }
    if (!REVERSE && r0 < rows) body(r0 * kThreads, G * kThreads, std::false_type{});
}

template <int U = kUnroll, bool REVERSE = false, typename Body>
__device__ __forceinline__ void sweep_tiles(int64_t nvec, Body&& body) {
    sweep_tiles_of<U, REVERSE>(nvec, blockIdx.x, gridDim.x, body);
}

// The walk of a kernel that keeps nothing from one tile to the next.  ONESHOT: the launch has one
// workgroup of T lanes per tile of U rows of T vectors, and the workgroup ends after its tile.  On
// this device a kernel that writes as much as these do runs faster that way than as a loop: at 2^28
// elements a plain copy takes 322 us instead of 358 us, 4 bytes in / 16 bytes out 204 us instead of
// 240 us (256 lanes, two rows).  Otherwise the looping sweep above (T must be kThreads).
template <int T, int U, bool ONESHOT, typename Body>
__device__ __forceinline__ void walk_tiles_of(int64_t nvec, int64_t slot, int64_t G, Body&& body) {
    if constexpr (ONESHOT) {
        const int64_t base = slot * (T * U);
        if (base + T * U <= nvec) body(base, static_cast<int64_t>(T), std::true_type{});
        else if (base < nvec) body(base, static_cast<int64_t>(T), std::false_type{});
    } else {
        static_assert(ONESHOT || T == kThreads, "the looping sweep is laid out for kThreads lanes");
        sweep_tiles_of<U, false>(nvec, slot, G, body);
    }
}

template <int T, int U, bool ONESHOT, typename Body>
__device__ __forceinline__ void walk_tiles(int64_t nvec, Body&& body) {
    walk_tiles_of<T, U, ONESHOT>(nvec, blockIdx.x, gridDim.x, body);
}

template <int U = kUnroll, typename Body>
__device__ __forceinline__ void sweep(int64_t nvec, Body&& body) {
    sweep_tiles<U, false>(nvec, [&](int64_t base, int64_t stride, auto full_t) { body(base + threadIdx.x, stride, full_t); });
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

// Histogram of the quantize pass in fixed point: one 64-bit LDS atomic per element.  An element with
// code c lies d = x * inv - (c - 128) bins from the centre of its bin (|d| <= 1/2 unless c is 0 or
// 255, where the clipped elements collect); the bin's sum of x is ((c - 128) * count + sum of d) / inv.
// d comes from one fused multiply-add (a single rounding of the exact x * inv - k) and is added as the
// integer floor(d * 2^22 + 1/2) + 2^31 in bits [47:0] of the slot, with 1 in bits [63:48]: count and sum
// in one atomic, integer sums that do not depend on the order of the additions.  Per element the
// table carries an error below 2^-23 of a bin width.  Elements with |x * inv| > 628 (or not a number)
// are beyond the range of the 32-bit residual: they count with residual 0 and their x goes to a pair of
// fp64 accumulators (they all have code 0 or 255).  A slot holds 2^16 - 1 additions; the workgroup
// moves the slots into 64-bit accumulators before any slot can have seen that many.
constexpr float kResidualOne = 4194304.0f;      // 2^22
constexpr float kFarBins = 628.0f;              // the residual of a nearer element is below 512 bins
constexpr int kFarCopies = 16;
constexpr int kMaxCopies = 8;                   // LDS copies of a bin, chosen per launch: 1, 2, 4 or 8

// `shift` = log2 of the number of copies of each bin in use: lanes pick a copy by lane id, so that
// lanes of a wavefront that meet in one bin spread over several addresses.  Few copies are fastest on
// data that spreads over many bins; a tensor crowded into a few bins (a constant, weights near 1)
// wants all eight.
struct ResidualHist {
    unsigned long long slot[kBins * kMaxCopies];
    long long wide_sum[kBins];
    unsigned long long wide_cnt[kBins];
    double far_sum[2][kFarCopies];
    unsigned far_cnt[2][kFarCopies];
    // main rounds between two flushes: kThreads >> shift lanes share a slot and add 4 * kUnroll elements each per round
    static __device__ __forceinline__ int flush_rounds(int shift) { return 65535 / ((kThreads >> shift) * 4 * kUnroll) - 2; }
};
static_assert(65535 / (kThreads * 4 * kUnroll) - 2 >= 1, "a slot must hold more than three rounds of a whole workgroup");

template <int T = kThreads>          // T = lanes of the calling workgroup
__device__ __forceinline__ void rhist_zero(ResidualHist& h, int shift) {
    for (int i = threadIdx.x; i < (kBins << shift); i += T) h.slot[i] = 0ull;
    for (int i = threadIdx.x; i < kBins; i += T) { h.wide_sum[i] = 0; h.wide_cnt[i] = 0ull; }
    if (threadIdx.x < 2 * kFarCopies) {
        h.far_sum[threadIdx.x / kFarCopies][threadIdx.x % kFarCopies] = 0.0;
        h.far_cnt[threadIdx.x / kFarCopies][threadIdx.x % kFarCopies] = 0u;
    }
}

// floor(v + 1/2) as an integer, in one instruction (computed exactly: no sum that could round).
__device__ __forceinline__ int round_half_up(float v) {
    int r;
    asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// The residual d of x from the centre `centre` (= code - 128, as a float) of its bin, in units of
// 2^-22 bin: floor(d * 2^22 + 1/2), d from one fused multiply-add.  Meaningless (and replaced) for
// far elements.
__device__ __forceinline__ int residual_units(float x, float inv, float centre) {
    return round_half_up(__builtin_fmaf(x, inv, -centre) * kResidualOne);
}
__device__ __forceinline__ int residual_fixed(float x, float inv, int code) {
    return residual_units(x, inv, static_cast<float>(code - kZeroPoint));
}

// `copy` = the lane's copy index, threadIdx.x & ((1 << shift) - 1).  H is ResidualHist or any struct
// with its `slot`, `far_sum` and `far_cnt` members.
template <typename H>
__device__ __forceinline__ void rhist_add(H& h, int shift, int copy, int code, int fixed) {
    const unsigned long long v = (1ull << 48) | static_cast<unsigned long long>(static_cast<unsigned>(fixed) ^ 0x80000000u);
    __hip_atomic_fetch_add(&h.slot[(code << shift) + copy], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

__device__ __forceinline__ bool is_far(float x, float inv) { return !(__builtin_fabsf(x * inv) <= kFarBins); }

template <typename H>
__device__ __forceinline__ void rhist_add_far(H& h, int code, float x) {
    const int side = code == kBins - 1, c = threadIdx.x & (kFarCopies - 1);
    __hip_atomic_fetch_add(&h.far_sum[side][c], static_cast<double>(x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __hip_atomic_fetch_add(&h.far_cnt[side][c], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// round_half_away(clamp(q, -128, 127)) as a float, for |q| <= kFarBins: the centre of the bin of a
// product q = x * inv when the zero point is 128, i.e. code - 128.  trunc(c + copysign(0.49999997, c))
// equals roundf(c) for every float in that range (0.49999997 is the float below 1/2: adding 1/2 itself
// would round 0.49999997 up to 1; checked exhaustively on the host, tests/test_host.py).
__device__ __forceinline__ float round_centre(float q) {
    const float c = __builtin_amdgcn_fmed3f(q, -128.0f, 127.0f);
    return __builtin_truncf(c + __builtin_copysignf(0.49999997f, c));
}

// The four elements of one vector in the fused pass: their packed codes (returned) and their
// histogram entries (no barrier inside: lanes may skip it).  Products within kFarBins take the short
// instruction sequence; a vector with a product beyond it, or not a number, takes the general one.
// Short sequence, per element: the centre k of the bin as a float (round_centre), then k + 1.5 * 2^23
// + 128 as a float, whose bit pattern is a constant plus the code: the low byte is the code for the
// packed word, and the whole pattern shifted left addresses the slot (the constant is taken out of
// the lane's base offset, modulo 2^32), so that the code never exists as an integer of its own.
template <typename H>
__device__ __forceinline__ uint32_t rhist_quantize4(H& h, int shift, int copy, const f4a v, float inv) {
    const float qa = v.x * inv, qb = v.y * inv, qc = v.z * inv, qd = v.w * inv;
    const bool ra = !(__builtin_fabsf(qa) <= kFarBins), rb = !(__builtin_fabsf(qb) <= kFarBins),
               rc = !(__builtin_fabsf(qc) <= kFarBins), rd = !(__builtin_fabsf(qd) <= kFarBins);
    if (!(ra | rb | rc | rd)) {
        constexpr float kMagic = 12582912.0f + kZeroPoint;            // 1.5 * 2^23 + 128: bits 0x4B400080 + (code - 128)
        constexpr uint32_t kMagicBits = 0x4B400000u;
        const float ka = round_centre(qa), kb = round_centre(qb), kc = round_centre(qc), kd = round_centre(qd);
        const uint32_t ua = __float_as_uint(ka + kMagic), ub = __float_as_uint(kb + kMagic),
                       uc = __float_as_uint(kc + kMagic), ud = __float_as_uint(kd + kMagic);      // kMagicBits + code
        const int s3 = shift + 3;                                     // a slot is 8 bytes
        uint32_t base = (static_cast<uint32_t>(copy) << 3) - (kMagicBits << s3);
        asm("" : "+v"(base));             // opaque: keeps the constant out of every element's address arithmetic
        char* slots = reinterpret_cast<char*>(h.slot);
        auto add = [&](uint32_t u, int units) {
            const unsigned long long val = (1ull << 48) | static_cast<unsigned long long>(static_cast<unsigned>(units) ^ 0x80000000u);
            __hip_atomic_fetch_add(reinterpret_cast<unsigned long long*>(slots + ((u << s3) + base)), val, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
        };
        add(ua, residual_units(v.x, inv, ka));
        add(ub, residual_units(v.y, inv, kb));
        add(uc, residual_units(v.z, inv, kc));
        add(ud, residual_units(v.w, inv, kd));
        const uint32_t lo = __builtin_amdgcn_perm(ub, ua, 0x0c0c0400u);   // code a | code b << 8
        const uint32_t hi = __builtin_amdgcn_perm(ud, uc, 0x0c0c0400u);
        return lo | (hi << 16);
    }
    const int a = quantize_code(v.x, inv, kZeroPoint), b = quantize_code(v.y, inv, kZeroPoint),
              c = quantize_code(v.z, inv, kZeroPoint), d = quantize_code(v.w, inv, kZeroPoint);
    int fa = 0, fb = 0, fc = 0, fd = 0;
    if (ra) rhist_add_far(h, a, v.x); else fa = residual_fixed(v.x, inv, a);
    if (rb) rhist_add_far(h, b, v.y); else fb = residual_fixed(v.y, inv, b);
    if (rc) rhist_add_far(h, c, v.z); else fc = residual_fixed(v.z, inv, c);
    if (rd) rhist_add_far(h, d, v.w); else fd = residual_fixed(v.w, inv, d);
    rhist_add(h, shift, copy, a, fa);
    rhist_add(h, shift, copy, b, fb);
    rhist_add(h, shift, copy, c, fc);
    rhist_add(h, shift, copy, d, fd);
    return static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) | (static_cast<uint32_t>(c) << 16) | (static_cast<uint32_t>(d) << 24);
}

// Move the slots into the 64-bit accumulators.  Called by all lanes of the workgroup (two barriers).
template <int T = kThreads>
__device__ __forceinline__ void rhist_flush(ResidualHist& h, int shift) {
    __syncthreads();
    for (int b = threadIdx.x; b < kBins; b += T) {
        unsigned long long cnt = 0, sum = 0;
        for (int r = 0; r < (1 << shift); ++r) {
            const unsigned long long v = h.slot[(b << shift) + r];
            h.slot[(b << shift) + r] = 0ull;
            cnt += v >> 48;
            sum += v & 0xffffffffffffull;
        }
        h.wide_sum[b] += static_cast<long long>(sum) - static_cast<long long>(cnt << 31);
        h.wide_cnt[b] += cnt;
    }
    __syncthreads();
}

// The fp64 sum of a bin's elements from the integer totals over the whole tensor: the count, the sum
// of the residuals in units of 2^-22 bin (as hi * 2^32 + lo: the sum of the partials' upper and of their
// lower halves, so that no 64-bit total can overflow) and, for the two clip bins, the far elements'
// count and fp64 sum.  One conversion from exact integers: the same value however the tensor was dealt out.
__device__ __forceinline__ double fixed_bin_sum(unsigned long long cnt, long long units_hi, unsigned long long units_lo,
                                                unsigned long long far_n, double far_s, float inv, int b) {
    const double centre = static_cast<double>(static_cast<long long>(cnt - far_n) * (b - kZeroPoint));
    const double units = static_cast<double>(units_hi) * 4294967296.0 + static_cast<double>(units_lo);
    return (centre + units * (1.0 / kResidualOne)) / static_cast<double>(inv) + far_s;
}
__device__ __forceinline__ long long units_hi(long long units) { return units >> 32; }
__device__ __forceinline__ unsigned long long units_lo(long long units) { return static_cast<unsigned long long>(units) & 0xffffffffull; }

__device__ __forceinline__ float mean_entry(double sum, unsigned long long cnt) {      // compression.cpp:99-101
    return cnt ? static_cast<float>(sum / static_cast<double>(cnt)) : 0.0f;
}

// The far elements of side `side` (0: bin 0, 1: bin 255), their copies added in order.
template <typename H>
__device__ __forceinline__ void rhist_far_side(const H& h, int side, unsigned long long& far_n, double& far_s) {
    far_n = 0;
    far_s = 0.0;
#pragma unroll
    for (int c = 0; c < kFarCopies; ++c) far_n += h.far_cnt[side][c];
    if (far_n == 0) return;              // the usual case; the sums are all 0.0 then, and so is their total
#pragma unroll
    for (int c = 0; c < kFarCopies; ++c) far_s += h.far_sum[side][c];
}

// The sum of v over the four lanes of the lane's row of sixteen that share its index modulo 4, in every lane:
// two rotations within the row (data-parallel moves).
__device__ __forceinline__ unsigned long long sum_row_mod4(unsigned long long v) {
    auto rotated = [](unsigned long long x, auto ctrl_t) {
        constexpr int kCtrl = decltype(ctrl_t)::value;
        const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(x), kCtrl, 0xf, 0xf, false);
        const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(x >> 32), kCtrl, 0xf, 0xf, false);
        return (static_cast<unsigned long long>(static_cast<unsigned>(hi)) << 32) | static_cast<unsigned>(lo);
    };
    v += rotated(v, std::integral_constant<int, 0x128>{});      // row_ror:8
    v += rotated(v, std::integral_constant<int, 0x124>{});      // row_ror:4
    return v;
}

// The same over the sixteen such lanes of the whole wavefront: then two exchanges between the rows.
__device__ __forceinline__ unsigned long long sum_lanes_mod4(unsigned long long v) {
    v = sum_row_mod4(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// The value of the lane D (1 or 2) away within the lane's group of four, by a data-parallel move (no trip
// through the LDS crossbar).
template <int D>
__device__ __forceinline__ unsigned long long quad_xor(unsigned long long v) {
    static_assert(D == 1 || D == 2, "a neighbour within the quad");
    constexpr int kCtrl = D == 1 ? 0xB1 : 0x4E;          // quad_perm [1, 0, 3, 2] / [2, 3, 0, 1]
    const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), kCtrl, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(v >> 32), kCtrl, 0xf, 0xf, false);
    return (static_cast<unsigned long long>(static_cast<unsigned>(hi)) << 32) | static_cast<unsigned>(lo);
}

// The workgroup's partial: 4 KiB of integer bin totals to `row`, the far elements to `far`.
// T / kBins neighbouring lanes share a bin: each adds its part of the bin's copies, the lanes are joined by
// exchanges and the first of them adds what earlier flushes left in the 64-bit accumulators (integers: any
// order gives the same totals).  One barrier; the slots are left as they are.
template <int T = kThreads>
__device__ __forceinline__ void rhist_store(ResidualHist& h, int shift, BinPart* __restrict__ row, const FarSlot far) {
    constexpr int kPer = T / kBins;
    static_assert(kPer == 1 || kPer == 2 || kPer == 4, "one, two or four lanes per bin");
    __syncthreads();
    const int b = threadIdx.x / kPer, q = threadIdx.x % kPer;
    unsigned long long cnt = 0, sum = 0;
    for (int r = q; r < (1 << shift); r += kPer) {
        const unsigned long long v = h.slot[(b << shift) + r];
        cnt += v >> 48;
        sum += v & 0xffffffffffffull;
    }
    if constexpr (kPer >= 4) {
        cnt += quad_xor<2>(cnt);
        sum += quad_xor<2>(sum);
    }
    if constexpr (kPer >= 2) {
        cnt += quad_xor<1>(cnt);
        sum += quad_xor<1>(sum);
    }
    if (q == 0) row[b] = BinPart{h.wide_sum[b] + static_cast<long long>(sum) - static_cast<long long>(cnt << 31), h.wide_cnt[b] + cnt};
    if (threadIdx.x < 2) {
        unsigned long long far_n;
        double far_s;
        rhist_far_side(h, threadIdx.x, far_n, far_s);
        far.cnt[threadIdx.x * kMaxGrid] = far_n;
        far.sum[threadIdx.x * kMaxGrid] = far_s;
    }
}

// The far elements of side `side` over the partials [p0, p1), by the calling wavefront (all 64 lanes call;
// the totals are valid in lane 0): lane l adds partials p0 + l, p0 + l + 64, ... (four loads in flight), the
// lanes are then added by the fixed tree of wave_sum.
__device__ __forceinline__ void far_totals(const Workspace* __restrict__ ws, int p0, int p1, int side, double& far_s, unsigned long long& far_n) {
    const int lane = threadIdx.x & 63;
    double fs = 0.0;
    unsigned long long fn = 0;
    for (int q = p0 + lane; q < p1; q += 4 * 64) {
        double s[4];
        unsigned long long c[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int p = q + 64 * k;
            s[k] = p < p1 ? ws->far_sum[side][p] : 0.0;
            c[k] = p < p1 ? ws->far_cnt[side][p] : 0ull;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) { fs += s[k]; fn += c[k]; }
    }
    if (__ballot(fn != 0) == 0) {        // the usual case: no far element anywhere; the sums are all 0.0 then
        far_s = 0.0;
        far_n = 0;
        return;
    }
    far_s = wave_sum(fs);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) fn += __shfl_down(fn, off, 64);
    far_n = fn;
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

// Bin b of the workgroup's histogram: its copies added in a fixed order.
template <int R>
__device__ __forceinline__ BinAcc hist_bin(const LdsHist<R>& h, int b) {
    BinAcc acc{0.0, 0ull};
#pragma unroll
    for (int r = 0; r < R; ++r) { acc.sum += h.sum[b * R + r]; acc.cnt += h.cnt[b * R + r]; }
    return acc;
}

// Store the workgroup's histogram as the partial of workgroup `slot`: one 16-byte store per lane,
// 4 KiB contiguous per workgroup.
template <int R>
__device__ __forceinline__ void hist_store(LdsHist<R>& h, BinAcc* __restrict__ row) {
    for (int b = threadIdx.x; b < kBins; b += kThreads) row[b] = hist_bin(h, b);
}
