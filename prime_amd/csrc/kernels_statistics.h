// Statistics: fp64 sum and sum of squares (first stage per workgroup, second stage in one
// workgroup), and the norm accumulated in libtorch's order for bit-for-bit reproduction.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

// Second stage of the statistics: one workgroup adds the partials (tree of fixed shape) and
// derives the scale.
__global__ __launch_bounds__(kFinalThreads) void stats_finalize_kernel(Workspace* ws, int nparts, int64_t n,
                                                                        prime_qparams* out) {
    (void)block_scale_from_partials<kFinalThreads>(ws, nparts, n, out);
}

// The statistics partial of workgroup `slot` of a grid of G, computed by the calling workgroup and
// stored in the workspace: fp64 sum and sum of squares of the rows that workgroup owns.
//
// With NT the loads carry the non-temporal hint, except from vector `keep_from` on: what a hinted load
// brings in does not stay in the last-level cache, and the pass that re-reads the tensor from its end
// finds there what this pass read last without the hint.
constexpr int64_t kKeepNothing = INT64_MAX;
template <bool ALIGNED, bool NT, int U = kUnroll>
__device__ __forceinline__ void stats_partial(const float* __restrict__ x, int64_t n, int slot, int G, double* part_sum, double* part_sq,
                                              int64_t keep_from = kKeepNothing) {
    using M = Mem<ALIGNED, NT>;
    using Kept = Mem<ALIGNED, false>;
    const int64_t nvec = n >> 2;
    double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
    sweep_tiles_of<U, false>(nvec, slot, G, [&](int64_t base, int64_t stride, auto full_t) {
        constexpr bool full = decltype(full_t)::value;
        const int64_t i0 = base + threadIdx.x;
        f4a v[U];
        if (NT && base >= keep_from) {
            asm volatile("" ::: "memory");        // keeps the two sets of loads apart: merged, they would lose the hint
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int64_t i = i0 + j * stride;
                v[j] = (full || i < nvec) ? Kept::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
            }
            asm volatile("" ::: "memory");
        } else {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int64_t i = i0 + j * stride;
                v[j] = (full || i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (j & 1) stats_add4(v[j], s1, q1); else stats_add4(v[j], s0, q0);
        }
    });
    if (slot == 0 && threadIdx.x < (n & 3)) {
        const double v = x[(nvec << 2) + threadIdx.x];
        s0 += v;
        q0 = fma(v, v, q0);
    }
    block_stats_store(s0 + s1, q0 + q1, part_sum, part_sq, slot);
}

// The statistics partials of K consecutive slots, first, first + 1, ..., of a grid of G by ONE workgroup,
// for a tensor so short that no slot has a whole tile (fewer than G * U rows: every slot owns the rows
// slot, slot + G, ... only).  Each slot's sums are formed exactly as stats_partial forms them - the same
// additions in the same order - but the K slots' loads are in flight together and their reductions
// run side by side: a workgroup that plays one such slot has a single 16 KiB row in flight.
template <int U, int K>
__device__ __forceinline__ void stats_partial_short(const float* __restrict__ x, int64_t n, int first, int G, double* part_sum,
                                                    double* part_sq) {
    using M = Mem<true, false>;
    __shared__ double sh_s[K][kWaves];
    __shared__ double sh_q[K][kWaves];
    const int64_t nvec = n >> 2;
    const int64_t rows = (nvec + kThreads - 1) / kThreads;
    f4a v[K][U];
#pragma unroll
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t row = first + k + static_cast<int64_t>(j) * G;
            const int64_t i = row * kThreads + threadIdx.x;
            v[k][j] = (first + k < G && first + k < rows && i < nvec) ? M::ldf4(x, i) : f4a{0.f, 0.f, 0.f, 0.f};
        }
    }
    double s[K], q[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        double s0 = 0.0, q0 = 0.0, s1 = 0.0, q1 = 0.0;
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (j & 1) stats_add4(v[k][j], s1, q1); else stats_add4(v[k][j], s0, q0);
        }
        if (first + k == 0 && threadIdx.x < (n & 3)) {
            const double t = x[(nvec << 2) + threadIdx.x];
            s0 += t;
            q0 = fma(t, t, q0);
        }
        s[k] = s0 + s1;
        q[k] = q0 + q1;
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {                 // independent chains: the compiler overlaps them
        s[k] = wave_sum(s[k]);
        q[k] = wave_sum(q[k]);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) { sh_s[k][wave] = s[k]; sh_q[k][wave] = q[k]; }
    }
    __syncthreads();
    if (threadIdx.x < K && first + static_cast<int>(threadIdx.x) < G) {
        double S = sh_s[threadIdx.x][0], Q = sh_q[threadIdx.x][0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[threadIdx.x][w]; Q += sh_q[threadIdx.x][w]; }
        part_sum[first + threadIdx.x] = S;
        part_sq[first + threadIdx.x] = Q;
    }
}

// K1: sum and sum of squares in fp64.  4 bytes per element.
// U = rows per tile: 4 from 2^27 elements up, 2 below (a 51 M-element bucket: 33.3 against 34.4 us).
template <bool ALIGNED, bool NT, int U = kUnroll>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void stats_kernel(const float* __restrict__ x, int64_t n, Workspace* ws,
                                                                                int64_t keep_from) {
    if (blockIdx.x == 0 && threadIdx.x == 0) ws->tile_counter = 0u;      // for the quantize pass that follows (sweep_tiles_dynamic)
    stats_partial<ALIGNED, NT, U>(x, n, blockIdx.x, gridDim.x, ws->part_sum, ws->part_sq, keep_from);
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
