// Segmented launches: up to kSegMax tensors (or ring chunks) go through a pass in ONE launch, each
// with as many workgroups as its size wants, so that a set of mid-size tensors pays three kernel
// boundaries in all instead of three per tensor (the ring all-reduce of one layer bucket cuts it
// into 2 W chunks, collectives.cpp:89-90, and the per-layer loop of diloco.py:108-110 visits one
// bucket after the other).  Results equal the one-tensor entry points' bit for bit:
//  * statistics: tensor t has `parts[t]` partial slots, the grid the one-tensor entry point would
//    launch for it, and the workgroup that plays slot v adds exactly what workgroup v of that grid
//    adds, in the same order (stats_partial / dequant_block are written for "workgroup `slot` of G");
//    the consuming pass adds the slots as the one-tensor quantize kernel does;
//  * codes depend on the element and the scale alone;
//  * the histogram partials are integers (BinPart), so their totals do not depend on how many
//    workgroups shared a tensor or which of them saw which tile.
// What may differ in its last bit: the lookup entries of a tensor whose 1 / scale is zero or not
// finite (fp64 partials, rare), and bins 0 / 255 of a tensor with elements beyond the fixed-point
// range in more than one workgroup (fp64 sums of those elements, already dependent on arrival order).
//
// The tensors' descriptors travel by value in the kernel arguments (no device-side table to fill
// before the launch); a workgroup finds its tensor by a binary search over the block ranges.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

struct SegJob {
    int count;
    int first[kSegMax + 1];              // workgroups [first[t], first[t + 1]) of this launch belong to tensor t
    int parts[kSegMax];                  // statistics partials of tensor t: the grid of the one-tensor entry point
    unsigned long long two_row;          // bit t: the pass of this launch takes tiles of two rows on tensor t
    int64_t n[kSegMax];
    float* x[kSegMax];                   // the tensor / the ring chunk (updated in place by a ring step)
    uint8_t* codes[kSegMax];             // codes out
    const uint8_t* codes_in[kSegMax];    // the received message of a ring step
    const float* lut_in[kSegMax];
};
static_assert(sizeof(SegJob) <= 4000, "the descriptors must fit the kernel argument segment");

// The tensor whose block range holds `block`: the last t with first[t] <= block.
__device__ __forceinline__ int seg_tensor_of(const int* first, int count, int block) {
    int lo = 0, hi = count;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (first[mid] <= block) lo = mid; else hi = mid;
    }
    return lo;
}

// A tensor with fewer rows than one tile per statistics slot: its slots own single rows, and one
// workgroup plays several of them at once (stats_partial_short): eight vectors per lane in flight.
__host__ __device__ constexpr int seg_short_slots(bool two_row) { return two_row ? 4 : 2; }
__host__ __device__ inline bool seg_short(int64_t n, int parts, bool two_row) {
    return ((n >> 2) / kThreads) / (static_cast<int64_t>(parts) * (two_row ? 2 : kUnroll)) == 0;
}

// K1 for every tensor of the job: one workgroup per statistics slot (per group of slots of a short tensor).
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void seg_stats_kernel(const SegJob job, Workspace* ws) {
    const int t = seg_tensor_of(job.first, job.count, blockIdx.x);
    const int v = blockIdx.x - job.first[t];
    const int64_t n = job.n[t];
    const int G = job.parts[t];
    const bool two = (job.two_row >> t) & 1;
    double* ps = ws->seg_part_sum[t];
    double* pq = ws->seg_part_sq[t];
    if (seg_short(n, G, two)) {
        if (two) stats_partial_short<2, seg_short_slots(true)>(job.x[t], n, v * seg_short_slots(true), G, ps, pq);
        else stats_partial_short<kUnroll, seg_short_slots(false)>(job.x[t], n, v * seg_short_slots(false), G, ps, pq);
    } else if (two) {
        stats_partial<true, false, 2>(job.x[t], n, v, G, ps, pq);
    } else {
        stats_partial<true, false, kUnroll>(job.x[t], n, v, G, ps, pq);
    }
}

// First pass of a ring step for every chunk of the job: chunk (+)= lut_in[codes_in] [/ divisor] with
// the statistics of the result, one workgroup per statistics slot.
template <bool ADD, bool DIV, int POLICY>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void seg_dequant_kernel(const SegJob job, float divisor, Workspace* ws) {
    __shared__ float s_lut[kBins];
    const int t = seg_tensor_of(job.first, job.count, blockIdx.x);
    const int v = blockIdx.x - job.first[t];
    dequant_block<ADD, true, true, false, DIV, POLICY, false, kShotUnroll>(job.x[t], job.lut_in[t], job.codes_in[t], job.n[t], ws->seg_part_sum[t],
                                                                          ws->seg_part_sq[t], divisor, v, job.parts[t], s_lut);
}

// K2 + K3 for every tensor of the job: tensor t is shared by the workgroups of its block range, each
// of which derives the tensor's scale from the statistics slots and leaves one histogram partial in
// the row of its block index.
template <int POLICY>
__global__ __launch_bounds__(kThreads, kWavesPerSimd) void seg_quantize_kernel(const SegJob job, prime_qparams* qp_out, Workspace* ws,
                                                                                int copies_shift) {
    __shared__ QuantHist hist_mem;
    const int t = seg_tensor_of(job.first, job.count, blockIdx.x);
    const int p = blockIdx.x - job.first[t];
    const int P = job.first[t + 1] - job.first[t];
    const int64_t n = job.n[t];
    int narrow = INT_MIN;
    const float inv = block_scale_from_partials<kThreads>(ws->seg_part_sum[t], ws->seg_part_sq[t], job.parts[t], n, p == 0, &ws->seg[t].qp,
                                                          qp_out ? qp_out + t : nullptr, &narrow, [&]() { rhist_zero(hist_mem.fixed, 3); });
    const HistOut out{ws->hist[blockIdx.x], FarSlot{&ws->far_sum[0][blockIdx.x], &ws->far_cnt[0][blockIdx.x]}, &ws->seg[t].info, p == 0, nullptr, 0, true};
    if ((job.two_row >> t) & 1)
        quantize_block<true, true, true, true, POLICY, 2>(job.x[t], n, inv, narrow, kZeroPoint, job.codes[t], out, copies_shift, p, P, hist_mem);
    else
        quantize_block<true, true, true, true, POLICY, kUnroll>(job.x[t], n, inv, narrow, kZeroPoint, job.codes[t], out, copies_shift, p, P, hist_mem);
}

// The lookup tables of the job: 64 workgroups of 256 lanes per tensor, each owning four bins, as in
// lut_finalize_kernel; the tensor's partials are rows first[t] .. first[t + 1] of the quantize launch.
// Lane (row, bin) adds partials row, row + 64, ... (four loads in flight); fp64 partials in that order,
// then over the rows by a fixed tree.
constexpr int kSegFinalThreads = 256;
constexpr int kSegFinalBlocks = kBins / kLutBinsPerBlock;          // workgroups per tensor
__global__ __launch_bounds__(kSegFinalThreads) void seg_lut_finalize_kernel(const SegJob job, const Workspace* __restrict__ ws, float* __restrict__ luts) {
    constexpr int kRows = kSegFinalThreads / kLutBinsPerBlock;      // 64
    constexpr int kWavesHere = kSegFinalThreads / 64;
    constexpr int kInFlight = 4;
    __shared__ double sh_sum[kSegFinalThreads];
    __shared__ unsigned long long sh_lo[kSegFinalThreads];
    __shared__ unsigned long long sh_cnt[kSegFinalThreads];
    __shared__ double sh_far_s;
    __shared__ unsigned long long sh_far_n;
    const int t = blockIdx.x / kSegFinalBlocks, j = blockIdx.x % kSegFinalBlocks;
    const int bl = threadIdx.x % kLutBinsPerBlock, row = threadIdx.x / kLutBinsPerBlock;
    const int bin = j * kLutBinsPerBlock + bl;
    const int p0 = job.first[t], p1 = job.first[t + 1];
    const HistInfo info = ws->seg[t].info;
    unsigned long long cnt = 0, lo = 0;
    long long hi = 0;
    double sum = 0.0;
    // both readings of a partial are added up (the integer one and the fp64 one): which one holds is known
    // when the record has arrived, with the first partials
    for (int q0 = p0 + row; q0 < p1; q0 += kRows * kInFlight) {
        BinAcc e[kInFlight];
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const int p = q0 + k * kRows;
            e[k] = p < p1 ? ws->hist[p][bin] : BinAcc{0.0, 0ull};
        }
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            cnt += e[k].cnt;
            const long long u = __double_as_longlong(e[k].sum);      // BinPart::units
            hi += units_hi(u);
            lo += units_lo(u);
            sum += e[k].sum;
        }
    }
    // the far elements of bins 0 and 255: the last wavefront of the workgroup that owns the bin
    const bool clip_block = j == 0 || j == kSegFinalBlocks - 1;
    if (clip_block && threadIdx.x >= kSegFinalThreads - 64) {
        double fs;
        unsigned long long fn;
        far_totals(ws, p0, p1, j != 0, fs, fn);
        if (threadIdx.x == kSegFinalThreads - 64) { sh_far_s = fs; sh_far_n = fn; }
    }
    const bool fixed = info.mode == kHistFixed;
    float* lut = luts + static_cast<int64_t>(t) * kBins;
    if (fixed) {
        cnt = sum_row_mod4(cnt);
        lo = sum_row_mod4(lo);
        hi = static_cast<long long>(sum_row_mod4(static_cast<unsigned long long>(hi)));
        if ((threadIdx.x & 15) < kLutBinsPerBlock) {
            const int slot = (threadIdx.x >> 4) * kLutBinsPerBlock + bl;
            sh_cnt[slot] = cnt;
            sh_lo[slot] = lo;
            sh_sum[slot] = __longlong_as_double(hi);
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            static_assert(kWavesHere * 16 == 64, "one slot per lane of the first wavefront");
            const unsigned long long cc = sum_lanes_mod4(sh_cnt[threadIdx.x]);
            const unsigned long long ll = sum_lanes_mod4(sh_lo[threadIdx.x]);
            const long long hh = static_cast<long long>(sum_lanes_mod4(static_cast<unsigned long long>(__double_as_longlong(sh_sum[threadIdx.x]))));
            if (row == 0) {
                const bool far_bin = bin == 0 || bin == kBins - 1;
                lut[bin] = mean_entry(fixed_bin_sum(cc, hh, ll, far_bin ? sh_far_n : 0ull, far_bin ? sh_far_s : 0.0, info.inv, bin), cc);
            }
        }
    } else {
        sh_cnt[threadIdx.x] = cnt;
        sh_sum[threadIdx.x] = sum;
        __syncthreads();
        if (threadIdx.x < 64) {
            unsigned long long cw[kWavesHere];
            double sw[kWavesHere];
#pragma unroll
            for (int w = 0; w < kWavesHere; ++w) {
                cw[w] = sh_cnt[threadIdx.x + 64 * w];
                sw[w] = sh_sum[threadIdx.x + 64 * w];
            }
#pragma unroll
            for (int h = kWavesHere / 2; h > 0; h >>= 1) {
#pragma unroll
                for (int i = 0; i < h; ++i) {
                    cw[i] += cw[i + h];
                    sw[i] += sw[i + h];
                }
            }
            unsigned long long cc = cw[0];
            double s = sw[0];
#pragma unroll
            for (int d = 32; d >= kLutBinsPerBlock; d >>= 1) {
                cc += __shfl_xor(cc, d, 64);
                s += __shfl_xor(s, d, 64);
            }
            if (row == 0) lut[bin] = mean_entry(s, cc);
        }
    }
}

// ---- elementwise passes over many tensors ---------------------------------------------------------
// The per-parameter loops either side of the all-reduce (src/zeroband/diloco.py:93-99 and the outer
// optimizer's step over its parameter list, :72-74, :212-215) as one launch: one 256-lane workgroup
// per tile of each tensor.  Elementwise arithmetic: the results are the one-tensor kernels'.
struct SegPointwiseJob {
    int count;
    int first[kSegMax + 1];              // workgroups [first[t], first[t + 1]) belong to tensor t
    int64_t n[kSegMax];
    float* a[kSegMax];                   // pseudo-gradient: outer      outer step: param
    float* b[kSegMax];                   //                  inner                  momentum buffer
    float* c[kSegMax];                   //                  out                    gradient
    float* d[kSegMax];                   //                                         inner model (may be null)
};
static_assert(sizeof(SegPointwiseJob) <= 4000, "the descriptors must fit the kernel argument segment");

template <int POLICY>
__global__ __launch_bounds__(kStreamShotThreads, 8) void seg_pseudo_gradient_kernel(const SegPointwiseJob job, float world_size) {
    const int t = seg_tensor_of(job.first, job.count, blockIdx.x);
    pseudo_gradient_block<true, true, POLICY, true>(job.a[t], job.b[t], job.n[t], world_size, job.c[t], blockIdx.x - job.first[t],
                                                   job.first[t + 1] - job.first[t]);
}

template <int POLICY>
__global__ __launch_bounds__(kStreamShotThreads, 8) void seg_outer_step_kernel(const SegPointwiseJob job, float neg_lr, float mu, int first) {
    const int t = seg_tensor_of(job.first, job.count, blockIdx.x);
    outer_step_block<false, true, true, POLICY, true>(job.a[t], job.b[t], job.c[t], nullptr, nullptr, job.d[t], job.n[t], neg_lr, mu, first,
                                                     blockIdx.x - job.first[t], job.first[t + 1] - job.first[t], nullptr);
}
