// uniform_8bit_quantize of a small tensor in one launch of one workgroup: statistics, scale,
// codes, histogram and lookup table (compression.cpp:106-125) with the results of the three-launch
// sequence bit for bit.  The three launches give a tensor of up to kSmallSlots rows (of kThreads
// 16-byte vectors) one workgroup per row; here one workgroup takes their places one after the
// other - the same additions in the same order, the same partials - so nothing is handed from one
// workgroup to another and no launch waits for the one before it.  Each lane loads its vector of
// every row once and keeps it in registers for both passes; the per-row partials stay in
// registers and LDS.
//
// Included by prime_hip.hip inside its anonymous namespace; not a translation unit of its own.

constexpr int kSmallSlots = 4;
constexpr int kSmallShift = 2;          // four LDS copies of each bin per row (any number gives the same integer sums)
static_assert(kThreads == 1024 && kBins == 256 && kSmallSlots == 4, "lane -> (row, bin) covers four rows of 256 bins; the tree is written for four rows");

// One row's fixed-point histogram: a row adds at most 4 * kThreads + 3 elements, so no slot can
// overflow its 16-bit count and the slots are read out directly, without the 64-bit accumulators.
struct SmallRowHist {
    unsigned long long slot[kBins << kSmallShift];
    double far_sum[2][kFarCopies];
    unsigned far_cnt[2][kFarCopies];
};

__device__ __forceinline__ BinAcc binacc_add(BinAcc a, BinAcc b) { return BinAcc{a.sum + b.sum, a.cnt + b.cnt}; }

// What lut_finalize_kernel makes of the partials of rows 0..3 for one bin: each first added to 0.0,
// then row r with r + 2, then r with r + 1.  (Its tree first adds rows r + 128, r + 64, ... r + 4,
// which do not exist here and count as zero: adding them changes nothing.)
__device__ __forceinline__ float lut_entry_of_rows(const BinAcc (&part)[kSmallSlots], int rows) {
    BinAcc leaf[kSmallSlots];
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) leaf[r] = r < rows ? BinAcc{0.0 + part[r].sum, part[r].cnt} : BinAcc{0.0, 0ull};
    const BinAcc t = binacc_add(binacc_add(leaf[0], leaf[2]), binacc_add(leaf[1], leaf[3]));
    return t.cnt ? static_cast<float>(t.sum / static_cast<double>(t.cnt)) : 0.0f;
}

// `rows` <= kSmallSlots is the grid the three-launch sequence uses for this tensor: one workgroup per
// row of whole vectors (the last of them may be left with the ragged end only, or with nothing).
// SRC says where the values come from: the tensor as it stands (uniform_8bit_quantize), or a ring
// step's first pass folded in - x = lut_in[codes_in] (gather step), x += lut_in[codes_in] (reduce
// step), the same divided by `divisor` (the last accumulation of an averaged chunk) - with the
// updated values written back, as dequant_kernel<.., STATS, ..> does ahead of the quantize pass.
enum SmallSource { kSmallTensor = 0, kSmallSet = 1, kSmallAdd = 2, kSmallAddDiv = 3 };

template <bool ALIGNED, int SRC>
__global__ __launch_bounds__(kThreads) void uniform_small_kernel(float* __restrict__ x, int64_t n, int rows,
                                                                 prime_qparams* qp_out, uint8_t* __restrict__ codes,
                                                                 float* __restrict__ lut, Workspace* ws, int copies_shift,
                                                                 const uint8_t* codes_in, const float* lut_in,
                                                                 float divisor) {
    using M = Mem<ALIGNED, false>;
    union Hists {
        QuantHist one;                    // row by row, when the histogram is not the fixed-point one
        SmallRowHist row[kSmallSlots];    // all rows side by side
    };
    __shared__ Hists hists;
    QuantHist& hist = hists.one;
    __shared__ double sh_s[kSmallSlots][kWaves];
    __shared__ double sh_q[kSmallSlots][kWaves];
    __shared__ double sh_part_s[kSmallSlots];
    __shared__ double sh_part_q[kSmallSlots];
    __shared__ float s_lut[SRC == kSmallTensor ? 1 : kBins];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t nvec = n >> 2;
    const int tail = static_cast<int>(n & 3);
    if (SRC != kSmallTensor) {
        for (int b = threadIdx.x; b < kBins; b += kThreads) s_lut[b] = lut_in[b];
        __syncthreads();
    }

    // the lane's vector of every row, and its element of the ragged end
    f4a v[kSmallSlots];
    bool has[kSmallSlots];
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) {
        const int64_t i = static_cast<int64_t>(r) * kThreads + threadIdx.x;
        has[r] = r < rows && i < nvec;
        v[r] = f4a{0.f, 0.f, 0.f, 0.f};
        if (SRC == kSmallTensor || SRC == kSmallAdd || SRC == kSmallAddDiv) {
            if (has[r]) v[r] = M::ldf4(x, i);
        }
        if (SRC != kSmallTensor && has[r]) {
            const uint32_t c = M::ldu32(codes_in, i);
            f4a l;
            l.x = s_lut[c & 255];
            l.y = s_lut[(c >> 8) & 255];
            l.z = s_lut[(c >> 16) & 255];
            l.w = s_lut[c >> 24];
            if (SRC == kSmallSet) v[r] = l;
            else v[r] = l + v[r];
            if (SRC == kSmallAddDiv) v[r] = v[r] / divisor;
            M::stf4(x, i, v[r], false);
        }
    }
    const bool has_tail = static_cast<int>(threadIdx.x) < tail;
    float tail_v = 0.0f;
    if (has_tail) {
        const int64_t i = (nvec << 2) + threadIdx.x;
        if (SRC == kSmallTensor) {
            tail_v = x[i];
        } else {
            tail_v = s_lut[codes_in[i]];
            if (SRC != kSmallSet) tail_v += x[i];
            if (SRC == kSmallAddDiv) tail_v = tail_v / divisor;
            x[i] = tail_v;
        }
    }

    // statistics: per row what stats_partial computes for the workgroup of that row; the rows that
    // exist are reduced side by side (their shuffle chains overlap), the others not at all
    auto stats_of = [&](auto count) {
        constexpr int N = decltype(count)::value;
        double s[N], q[N];
#pragma unroll
        for (int r = 0; r < N; ++r) {
            s[r] = 0.0;
            q[r] = 0.0;
            stats_add4(v[r], s[r], q[r]);
            if (r == 0 && has_tail) {
                const double t = tail_v;
                s[r] += t;
                q[r] = fma(t, t, q[r]);
            }
            s[r] += 0.0;                  // the second accumulator pair of the streaming kernel stays at zero
            q[r] += 0.0;
        }
#pragma unroll
        for (int r = 0; r < N; ++r) {                 // independent chains: the compiler overlaps them
            s[r] = wave_sum(s[r]);
            q[r] = wave_sum(q[r]);
        }
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < N; ++r) { sh_s[r][wave] = s[r]; sh_q[r][wave] = q[r]; }
        }
    };
    if (rows <= 1) stats_of(std::integral_constant<int, 1>{});
    else if (rows == 2) stats_of(std::integral_constant<int, 2>{});
    else stats_of(std::integral_constant<int, kSmallSlots>{});
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < rows) {
        double S = sh_s[threadIdx.x][0], Q = sh_q[threadIdx.x][0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { S += sh_s[threadIdx.x][w]; Q += sh_q[threadIdx.x][w]; }
        sh_part_s[threadIdx.x] = S;
        sh_part_q[threadIdx.x] = Q;
    }
    __syncthreads();
    // scale: lane i of the reduction brings the partial of workgroup i
    int narrow = INT_MIN;
    const bool mine = static_cast<int>(threadIdx.x) < rows;
    const double pa = (0.0 + (mine ? sh_part_s[threadIdx.x & (kSmallSlots - 1)] : 0.0)) + 0.0;
    const double pb = (0.0 + (mine ? sh_part_q[threadIdx.x & (kSmallSlots - 1)] : 0.0)) + 0.0;
    const float inv = block_scale_reduce<kThreads>(pa, pb, n, true, &ws->qp, qp_out, &narrow);

    // codes and histogram; the modes are those of quantize_block
    enum { kFixed, kFp, kBin0 };
    const int mode = !(__builtin_fabsf(inv) < __builtin_inff()) ? kBin0 : inv != 0.0f ? kFixed : kFp;
    BinAcc part[kSmallSlots];
#pragma unroll
    for (int r = 0; r < kSmallSlots; ++r) part[r] = BinAcc{0.0, 0ull};
    const int64_t ti = (nvec << 2) + threadIdx.x;
    if (mode == kFixed) {
        // all rows at once, each into its own histogram
        unsigned long long* all = &hists.row[0].slot[0];
        for (int i = threadIdx.x; i < rows * static_cast<int>(sizeof(SmallRowHist) / 8); i += kThreads) all[i] = 0ull;   // zero bits are 0.0 and 0u too
        __syncthreads();
        const int copy = threadIdx.x & ((1 << kSmallShift) - 1);
#pragma unroll
        for (int r = 0; r < kSmallSlots; ++r) {
            const int64_t i = static_cast<int64_t>(r) * kThreads + threadIdx.x;
            if (has[r]) M::stu32(codes, i, rhist_quantize4(hists.row[r], kSmallShift, copy, v[r], inv));
        }
        if (has_tail) {
            const int a = quantize_code(tail_v, inv, kZeroPoint);
            codes[ti] = static_cast<uint8_t>(a);
            const bool far = is_far(tail_v, inv);
            if (far) rhist_add_far(hists.row[0], a, tail_v);
            rhist_add(hists.row[0], kSmallShift, copy, a, far ? 0 : residual_fixed(tail_v, inv, a));
        }
        __syncthreads();
        // lane -> (row, bin): the bin's integer totals of that row's partial, left where the bin's slots were
        const int bin = threadIdx.x & (kBins - 1);
#pragma unroll
        for (int pass = 0; pass < kSmallSlots * kBins / kThreads; ++pass) {
            const int r = pass * (kThreads / kBins) + (threadIdx.x >> 8);
            if (r >= rows) continue;      // uniform over the wavefront
            SmallRowHist& h = hists.row[r];
            unsigned long long cnt = 0, sum = 0;
#pragma unroll
            for (int c = 0; c < (1 << kSmallShift); ++c) {
                const unsigned long long s = h.slot[(bin << kSmallShift) + c];
                cnt += s >> 48;
                sum += s & 0xffffffffffffull;
            }
            static_assert(kSmallShift >= 1, "the totals take the place of two slots");
            h.slot[(bin << kSmallShift)] = static_cast<unsigned long long>(static_cast<long long>(sum) - static_cast<long long>(cnt << 31));
            h.slot[(bin << kSmallShift) + 1] = cnt;
        }
        __syncthreads();
        if (threadIdx.x < kBins) {
            // what lut_finalize_kernel makes of these partials: integer totals over the rows, the far
            // elements' sums added in the order of its tree, one conversion
            unsigned long long cnt = 0, lo = 0, far_n = 0;
            long long hi = 0;
            double leaf[kSmallSlots];
            const bool far_bin = bin == 0 || bin == kBins - 1;
#pragma unroll
            for (int r = 0; r < kSmallSlots; ++r) {
                leaf[r] = 0.0;
                if (r < rows) {
                    const long long u = static_cast<long long>(hists.row[r].slot[(bin << kSmallShift)]);
                    hi += units_hi(u);
                    lo += units_lo(u);
                    cnt += hists.row[r].slot[(bin << kSmallShift) + 1];
                    if (far_bin) {
                        unsigned long long fn;
                        double fs;
                        rhist_far_side(hists.row[r], bin != 0, fn, fs);
                        far_n += fn;
                        leaf[r] = 0.0 + fs;
                    }
                }
            }
            const double far_s = (leaf[0] + leaf[2]) + (leaf[1] + leaf[3]);
            lut[threadIdx.x] = mean_entry(fixed_bin_sum(cnt, hi, lo, far_n, far_s, inv, bin), cnt);
        }
        if (threadIdx.x == 0) ws->hist_info = HistInfo{inv, kHistFixed};
        return;
    } else {
        // row by row through one histogram (rare: a zero or non-finite 1 / scale)
        auto set_part = [&](int r, BinAcc e) {
#pragma unroll
            for (int k = 0; k < kSmallSlots; ++k)
                if (r == k) part[k] = e;
        };
        for (int r = 0; r < rows; ++r) {
            const int64_t i = static_cast<int64_t>(r) * kThreads + threadIdx.x;
            f4a vr = v[0];
            bool hr = has[0];
#pragma unroll
            for (int k = 1; k < kSmallSlots; ++k)
                if (r == k) { vr = v[k]; hr = has[k]; }
            int a = 0, b = 0, c = 0, d = 0;
            if (hr) {
                a = quantize_code(vr.x, inv, kZeroPoint);
                b = quantize_code(vr.y, inv, kZeroPoint);
                c = quantize_code(vr.z, inv, kZeroPoint);
                d = quantize_code(vr.w, inv, kZeroPoint);
                M::stu32(codes, i, static_cast<uint32_t>(a) | (static_cast<uint32_t>(b) << 8) | (static_cast<uint32_t>(c) << 16) |
                                       (static_cast<uint32_t>(d) << 24));
            }
            const bool tail_here = r == 0 && has_tail;
            const int ta = tail_here ? quantize_code(tail_v, inv, kZeroPoint) : 0;
            if (tail_here) codes[ti] = static_cast<uint8_t>(ta);
            if (mode == kFp) {
                hist_zero(hist.fp);
                __syncthreads();
                if (hr) {
                    hist_add(hist.fp, a, vr.x);
                    hist_add(hist.fp, b, vr.y);
                    hist_add(hist.fp, c, vr.z);
                    hist_add(hist.fp, d, vr.w);
                }
                if (tail_here) hist_add(hist.fp, ta, tail_v);
                __syncthreads();
                if (threadIdx.x < kBins) set_part(r, hist_bin(hist.fp, threadIdx.x));
                __syncthreads();
            } else {                      // every code is 0: one sum, lanes then wavefronts in the order of hist_store_bin0
                double ls = 0.0;
                unsigned long long lc = 0;
                if (hr) {
                    ls += static_cast<double>(vr.x);
                    ls += static_cast<double>(vr.y);
                    ls += static_cast<double>(vr.z);
                    ls += static_cast<double>(vr.w);
                    lc += 4;
                }
                if (tail_here) { ls += static_cast<double>(tail_v); lc += 1; }
                const BinAcc total = block_sum_bin0(ls, lc);
                if (threadIdx.x == 0) set_part(r, total);
            }
        }
    }
    if (threadIdx.x < kBins) lut[threadIdx.x] = lut_entry_of_rows(part, rows);
}
