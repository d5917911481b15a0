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

// device code, by topic (each header is written to live inside this namespace)
#include "device_common.h"
#include "kernels_statistics.h"
#include "kernels_quantize.h"
#include "kernels_small.h"
#include "kernels_codes.h"
#include "kernels_outer.h"
#include "kernels_segmented.h"

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
    int blocks_per_cu = 1;          // workgroups per compute unit a streaming kernel is launched with
    int large_read_grid_eighths = 7;   // read-heavy kernels on large tensors: workgroups = this many eighths of the compute units
    int64_t large_read_min_elems = int64_t(1) << 27;
    int stats_grid_eighths = 6;        // the statistics pass on such tensors: at most this many eighths (0: as the line above)
    int nt_load_min_mib = 512;      // tensors of at least this many MiB are loaded with the non-temporal hint
    int stats_keep_mib = 256;       // the statistics pass of uniform_8bit_quantize: all but the last this many MiB hinted (0: as the line above)
    int mix_cached = 1;             // the quantize pass visits what the statistics pass kept spread among the rest of the tensor
    int mixed_grid_eighths = 8;     // and then runs on this many eighths of the compute units (0: as the other read-heavy passes)
    int nt_second_min_mib = 0;      // the same for the quantize pass that re-reads a tensor: its last use, always hinted
    int average_replicas = 8;       // 1, 2, 4, 8 or 16 copies of each LDS bin of average_buckets' fp64 histogram
    int hist_replicas = 4;          // 1, 2, 4 or 8 copies of each LDS bin of the fused quantize pass
    int code_store_policy = kStoreNt;   // cache policy of the code stores (0 plain, 2 nt, 16 write-through)
    int reverse_second_pass = 1;    // the pass that re-reads a tensor walks it from its end
    int grid_cap = 0;               // experiment: upper bound on the workgroups of a streaming kernel (0: none)
    int f32_store_policy = kStoreWriteThrough;          // fp32 outputs nobody reads back soon (dequantize, outer step)
    int f32_reread_store_policy = kStoreWriteThrough;   // fp32 outputs the next kernel reads back (ring step, first touch)
    int copy_store_policy = kStoreWriteThrough;         // the plain copy (the byte counters' yardstick)
    int one_shot = 1;                                   // kernels that keep nothing between tiles: one workgroup per tile instead of a loop
    int64_t one_shot_min_elems = int64_t(1) << 16;      // ... from this many elements up
    // cache policy of their fp32 stores.  Write-through: as fast as non-temporal from 2^27 elements up (the outer
    // step alone loses 2-3 %) and well ahead below (pseudo-gradient at 2^26: 109 against 128 us)
    int one_shot_store_policy = kStoreWriteThrough;
    int64_t small_max_elems = int64_t(1) << 14;         // uniform_8bit_quantize takes one launch of one workgroup up to this many elements (0: never)
    // the statistics and quantize kernels take tiles of two rows instead of four below this many elements (0: never):
    // a 51 M-element bucket 74.5 against 78.4 us for the three launches, 2^26 elements 93.5 against 97.4;
    // from 2^27 up four rows win (2^27: 196 against 207 us, 2^28: 378 against 404)
    int64_t two_row_below_elems = int64_t(1) << 27;
    // the fused quantize + histogram pass hands out the last rounds of its tiles on demand instead of round-robin
    // (percent of the rounds; 0: never), on tensors of at least dynamic_tail_min_elems elements.  At 2^28 elements
    // (a tile streams for 3 us, longer than the trip to the counter) 5 % takes the pass from 226 to 221 us, 10 % to 222,
    // 25 % to 224; on a 51 M-element bucket (two-row tiles, 1 us each) any share costs: 37.5 us against 39.8 at 5 %
    int dynamic_tail_percent = 5;
    int64_t dynamic_tail_min_elems = int64_t(1) << 27;
    int segment_blocks_per_cu = 2;
    // a tensor of more elements than this fills the device on its own and takes the one-tensor path inside a segmented call:
    // eight tensors of 2^24 elements 201 us segmented against 283 us one by one (ring step 333 against 385), of 2^25
    // 396 against 453 (ring step 683 against 643), of 2^26 812 against 804 (ring step 1407 against 1207)
    int64_t segment_max_elems = int64_t(1) << 25;
    int64_t segment_ring_max_elems = int64_t(1) << 24;  // workgroups per compute unit the quantize pass of a segmented launch shares out among its tensors
    int64_t set_four_rows_max_elems = int64_t(1) << 25;  // the one-workgroup-per-tile dequantize set takes tiles of four rows up to this many elements (0: never)
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

// Workgroups for a streaming kernel: one per row of kThreads 16-byte vectors until the device is
// full (blocks_per_cu per compute unit), then each takes a longer span.  One 1024-thread workgroup
// per compute unit is at least as fast as two from 4 Mi elements up (fewer concurrent streams into
// HBM), and with `reads` (a kernel that reads at least as much as it writes) tensors of 2^27 elements
// or more do best on seven eighths of the compute units: at 2^28 elements the statistics pass goes
// from 158 to 152 us and the quantize pass from 241 to 218 us; the statistics pass, which only reads, does
// better still on six eighths (2^27: 79.9 -> 77.2 us, 2^28: 156 -> 151 us, 2^29: 307 -> 299 us; below 2^27
// elements every compute unit stays ahead for both).  A kernel that mostly writes
// (dequantize set) wants every compute unit.
int grid_for(int64_t n, bool reads = false) {
    int64_t tiles = (n + kRowElems - 1) / kRowElems;
    if (tiles < 1) tiles = 1;
    int64_t cap = static_cast<int64_t>(cu_count()) * g_opt.blocks_per_cu;
    if (reads && n >= g_opt.large_read_min_elems && g_opt.large_read_grid_eighths > 0) {
        const int64_t c = static_cast<int64_t>(cu_count()) / 8 * g_opt.large_read_grid_eighths;
        if (c >= 8 && c < cap) cap = c;
    }
    if (cap > kMaxGrid) cap = kMaxGrid;
    if (g_opt.grid_cap > 0 && cap > g_opt.grid_cap) cap = g_opt.grid_cap;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

// Workgroups (= partials) of the statistics pass over a tensor: every path that stands in for that pass takes its
// slots from here, so that the fp64 sums are added in one order whichever entry point runs.
int stats_grid_for(int64_t n) {
    int grid = grid_for(n, true);
    if (n >= g_opt.large_read_min_elems && g_opt.stats_grid_eighths > 0)
        grid = std::min(grid, std::max(8, cu_count() / 8 * g_opt.stats_grid_eighths));
    return grid;
}

// One workgroup per tile for a kernel launched ONESHOT.
int shot_grid(int64_t nvec, int rows = kShotUnroll, int threads = kShotThreads) {
    const int64_t tile = static_cast<int64_t>(threads) * rows;
    return static_cast<int>((nvec + tile - 1) / tile);
}
int stream_shot_grid(int64_t nvec) { return shot_grid(nvec, kStreamShotRows, kStreamShotThreads); }
// (a dispatch counts its work-items in 32 bits, and a launch of one vector per lane has one work-item per vector: beyond
// 2^33 elements the looping kernels take over)
inline bool one_shot(int64_t n) { return g_opt.one_shot && n >= g_opt.one_shot_min_elems && n <= (int64_t(1) << 33); }

// after_writer: the kernel before wrote the tensor (ring step, pseudo-gradient) instead of reading it: half the limit
// (ring step of 2^26 elements: the quantize pass 51 us with four rows, 62 with two; of 2^25: 27.4 and 26.4)
inline bool two_row_tiles(int64_t n, bool after_writer = false) { return (after_writer ? 2 * n : n) < g_opt.two_row_below_elems; }
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
    kIdDequantAddStats, kIdDequantSetStats, kIdBatched, kIdCopy, kIdFill, kIdPseudoGrad, kIdOuterStep, kIdOuterStepCodes, kIdDiv, kIdFirstTouchCodes, kIdCodeCount, kIdCodeTotal, kIdRequantPlan, kIdCodeRemap, kIdNormLiteral, kIdUniformSmall,
    kIdSegStats, kIdSegDequantAdd, kIdSegDequantSet, kIdSegQuantize, kIdSegLutFinalize, kIdSegPseudoGrad, kIdSegOuterStep, kIdCount
};
const char* const kKernelNames[kIdCount] = {
    "stats_kernel", "stats_finalize_kernel", "quantize_kernel", "quantize_kernel+hist", "hist_kernel", "lut_finalize_kernel",
    "dequant_kernel<set>", "dequant_kernel<add>", "dequant_kernel<add,stats>", "dequant_kernel<set,stats>",
    "batched_kernel", "copy_kernel", "fill_zero_kernel", "pseudo_gradient_kernel", "outer_step_kernel", "outer_step_kernel<codes>", "div_kernel",
    "first_touch_kernel<codes>", "code_count_kernel", "code_total_kernel", "requant_plan_kernel", "code_remap_kernel", "norm_literal_kernel", "uniform_small_kernel",
    "seg_stats_kernel", "seg_dequant_kernel<add,stats>", "seg_dequant_kernel<set,stats>", "seg_quantize_kernel+hist", "seg_lut_finalize_kernel",
    "seg_pseudo_gradient_kernel", "seg_outer_step_kernel"};

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

// Calls f with the store policy as a compile-time constant.
template <typename F>
void with_policy(int policy, F&& f) {
    if (policy == kStoreNt) f(std::integral_constant<int, kStoreNt>{});
    else if (policy == kStoreWriteThrough) f(std::integral_constant<int, kStoreWriteThrough>{});
    else f(std::integral_constant<int, kStorePlain>{});
}

int run_stats_finalize(Workspace* ws, int nparts, int64_t n, prime_qparams* out, hipStream_t st) {
    launch(kIdStatsFinalize, 16.0 * nparts, stats_finalize_kernel, 1, kFinalThreads, st, ws, nparts, n, out);
    return launch_check("stats_finalize_kernel");
}

// First stage only: returns the number of partials through *parts.
// Whether the statistics pass of uniform_8bit_quantize on n elements leaves the tensor's end in the last-level cache
// (and how much of it, in MiB) for the quantize pass: 0 when the tensor fits there anyway.
int kept_end_mib(int64_t n) {
    return g_opt.reverse_second_pass && g_opt.stats_keep_mib > 0 && (n >> 18) > g_opt.stats_keep_mib ? g_opt.stats_keep_mib : 0;
}

// reread: the quantize pass follows and walks the tensor from its end.  What a hinted load brings in does not stay
// in the last-level cache, so the statistics pass then reads the last stats_keep_mib MiB without the hint and the
// rest with it: 2^28 elements 364 instead of 377 us for the whole call (the quantize pass 202 instead of 217 us),
// 2^27 185 instead of 196 us; up to 256 MiB nothing is hinted, as before.
int run_stats_partials(const float* x, int64_t n, Workspace* ws, hipStream_t st, int* parts, bool reread = false) {
    const int grid = stats_grid_for(n);
    const bool two = two_row_tiles(n);
    const bool keep_end = reread && g_opt.reverse_second_pass && g_opt.stats_keep_mib > 0;
    const bool nt = keep_end ? kept_end_mib(n) > 0 : use_nt(n);
    const int64_t keep_from = keep_end ? (n >> 2) - (static_cast<int64_t>(g_opt.stats_keep_mib) << 16) : kKeepNothing;
    if (!aligned_to(x, 16))
        launch(kIdStats, 4.0 * n, stats_kernel<false, false>, grid, kThreads, st, x, n, ws, kKeepNothing);
    else if (nt)
        launch(kIdStats, 4.0 * n, two ? stats_kernel<true, true, 2> : stats_kernel<true, true>, grid, kThreads, st, x, n, ws, keep_from);
    else
        launch(kIdStats, 4.0 * n, two ? stats_kernel<true, false, 2> : stats_kernel<true, false>, grid, kThreads, st, x, n, ws, kKeepNothing);
    *parts = grid;
    return launch_check("stats_kernel");
}

int run_stats(const float* x, int64_t n, prime_qparams* out, Workspace* ws, hipStream_t st) {
    int parts = 0;
    if (int rc = run_stats_partials(x, n, ws, st, &parts)) return rc;
    return run_stats_finalize(ws, parts, n, out, st);
}

template <bool HIST, bool REVERSE, int POLICY>
void launch_quantize_p(bool al, bool two, int grid, hipStream_t st, const float* x, int64_t n, float scale, int stats_parts,
                       prime_qparams* qp_out, int zp, uint8_t* codes, Workspace* ws, int mix_mib) {
    const int id = HIST ? kIdQuantizeHist : kIdQuantize;
    int shift = 0;
    while ((1 << (shift + 1)) <= g_opt.hist_replicas) ++shift;
    // tiles on demand need the workspace's tile counter at zero: the lookup finalize that ends every call with a
    // fused pass leaves it so (as do the passes that write statistics partials, and prime_workspace_init)
    const int dyn = HIST && n >= g_opt.dynamic_tail_min_elems ? g_opt.dynamic_tail_percent : 0;
    // rounds of tiles at the tensor's end that the statistics pass left in the last-level cache
    const int mix = !(REVERSE && HIST) ? 0
                    : static_cast<int>((static_cast<int64_t>(mix_mib) << 20) / (static_cast<int64_t>(grid) * (two ? 2 : kUnroll) * kRowElems * 4));
    if (!al)
        launch(id, 5.0 * n, quantize_kernel<false, false, HIST, REVERSE, kStorePlain>, grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, shift, dyn, 0);
    else if ((n >> 18) >= g_opt.nt_second_min_mib)      // the quantize pass is always the last reader of the tensor
        launch(id, 5.0 * n, two ? quantize_kernel<true, true, HIST, REVERSE, POLICY, 2> : quantize_kernel<true, true, HIST, REVERSE, POLICY>,
               grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, shift, dyn, mix);
    else
        launch(id, 5.0 * n, two ? quantize_kernel<true, false, HIST, REVERSE, POLICY, 2> : quantize_kernel<true, false, HIST, REVERSE, POLICY>,
               grid, kThreads, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, shift, dyn, mix);
}

template <bool HIST>
void launch_quantize_r(bool al, bool two, bool reverse, int grid, hipStream_t st, const float* x, int64_t n, float scale, int stats_parts,
                       prime_qparams* qp_out, int zp, uint8_t* codes, Workspace* ws, int mix_mib) {
#define PRIME_Q(REV, POL) launch_quantize_p<HIST, REV, POL>(al, two, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, mix_mib)
    const int pol = g_opt.code_store_policy;
    if (reverse) {
        if (pol == kStoreNt) PRIME_Q(true, kStoreNt);
        else if (pol == kStorePlain) PRIME_Q(true, kStorePlain);
        else PRIME_Q(true, kStoreWriteThrough);
    } else {
        if (pol == kStoreNt) PRIME_Q(false, kStoreNt);
        else if (pol == kStorePlain) PRIME_Q(false, kStorePlain);
        else PRIME_Q(false, kStoreWriteThrough);
    }
#undef PRIME_Q
}

// stats_parts > 0: take the scale from that many statistics partials in the workspace (and
// publish it to qp_out); otherwise use `scale`.  Returns the grid size through *grid_out: the
// number of histogram partials written.  second_pass: the tensor has just been streamed by the
// kernel before this one, so walk it from its end (what the last-level cache still holds comes first).
int run_quantize(const float* x, int64_t n, float scale, int stats_parts, prime_qparams* qp_out, int zp, uint8_t* codes,
                 Workspace* ws, bool hist, hipStream_t st, int* grid_out, bool second_pass = false, bool after_writer = false) {
    if (hist && zp != kZeroPoint) return fail(PRIME_EINVAL, "the fused quantize + lookup pass has zero point 128");
    // After the statistics pass of the same call the tensor's end is in the last-level cache: the pass visits those
    // tiles spread among the others, so that cache and memory deliver side by side (2^28 elements: 203 -> 190 us), and
    // then does best on every compute unit (187 us) instead of seven eighths of them.
    // Only for tensors of at least twice what is kept: with most of the tensor in the cache, visiting the cached tiles
    // later means finding fewer of them still there (100 M elements, 381 MiB: 74 us walked from the end, 87 us mixed).
    const int kept = second_pass && !after_writer && hist && g_opt.mix_cached ? kept_end_mib(n) : 0;
    const int mix_mib = (n >> 18) >= 2 * static_cast<int64_t>(kept) ? kept : 0;
    const int grid = mix_mib > 0 && g_opt.mixed_grid_eighths > 0
                         ? std::min(grid_for(n), std::max(8, cu_count() / 8 * g_opt.mixed_grid_eighths)) : grid_for(n, true);
    const bool al = aligned_to(x, 16) && aligned_to(codes, 4);
    if (!hist && stats_parts == 0 && al && one_shot(n)) {
        with_policy(g_opt.code_store_policy, [&](auto P) {
            launch(kIdQuantize, 5.0 * n, quantize_shot_kernel<decltype(P)::value>, shot_grid(n >> 2), kShotThreads, st, x, n, scale, zp, codes);
        });
        if (grid_out) *grid_out = 0;
        return launch_check("quantize_shot_kernel");
    }
    const bool rev = second_pass && g_opt.reverse_second_pass;
    const bool two = two_row_tiles(n, after_writer);
    if (!hist) launch_quantize_r<false>(al, two, rev, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, 0);
    else launch_quantize_r<true>(al, two, rev, grid, st, x, n, scale, stats_parts, qp_out, zp, codes, ws, mix_mib);
    if (grid_out) *grid_out = grid;
    return launch_check("quantize_kernel");
}

int run_lut_finalize(Workspace* ws, int nparts, float* lut, int64_t n_bins, uint64_t* counts, hipStream_t st) {
    if (nparts == 0) {
        launch(kIdLutFinalize, 0.0, lut_zero_kernel, 1, 256, st, lut, n_bins, reinterpret_cast<unsigned long long*>(counts));
        return launch_check("lut_zero_kernel");
    }
    if (nparts <= 256)
        launch(kIdLutFinalize, 16.0 * kBins * nparts, lut_finalize_kernel<256, 256>, kBins / kLutBinsPerBlock, 256, st, ws, nparts, lut, n_bins,
               reinterpret_cast<unsigned long long*>(counts));
    else
        launch(kIdLutFinalize, 16.0 * kBins * nparts, lut_finalize_kernel<kFinalThreads, kMaxGrid>, kBins / kLutBinsPerBlock, kFinalThreads, st, ws,
               nparts, lut, n_bins, reinterpret_cast<unsigned long long*>(counts));
    return launch_check("lut_finalize_kernel");
}

template <bool ADD, bool STATS, bool DIV, int POLICY>
void launch_dequant(int id, double bytes, int grid, hipStream_t st, float* out, const float* lut, const uint8_t* codes, int64_t n,
                    Workspace* ws, float divisor) {
    if (!(aligned_to(out, 16) && aligned_to(codes, 4))) {
        launch(id, bytes, dequant_kernel<ADD, STATS, false, false, DIV, kStorePlain>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
        return;
    }
    if constexpr (!STATS) {
        if (one_shot(n)) {
            with_policy(g_opt.one_shot_store_policy, [&](auto P) {
                if (!ADD && n <= g_opt.set_four_rows_max_elems)
                    launch(id, bytes, dequant_kernel<ADD, false, true, true, DIV, decltype(P)::value, true, 4>, shot_grid(n >> 2, 4), kShotThreads, st,
                           out, lut, codes, n, ws, divisor);
                else if (ADD)
                    launch(id, bytes, dequant_kernel<ADD, false, true, true, DIV, decltype(P)::value, true, kAddShotRows, kAddShotThreads>,
                           shot_grid(n >> 2, kAddShotRows, kAddShotThreads), kAddShotThreads, st, out, lut, codes, n, ws, divisor);
                else
                    launch(id, bytes, dequant_kernel<ADD, false, true, true, DIV, decltype(P)::value, true>, shot_grid(n >> 2), kShotThreads, st, out, lut,
                           codes, n, ws, divisor);
            });
            return;
        }
    }
    if (use_nt(n))
        launch(id, bytes, dequant_kernel<ADD, STATS, true, true, DIV, POLICY>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
    else
        launch(id, bytes, dequant_kernel<ADD, STATS, true, false, DIV, POLICY>, grid, kThreads, st, out, lut, codes, n, ws, divisor);
}

// The fp32 stores of a pass whose output the next kernel reads back at once (STATS: the quantize
// pass follows) take f32_reread_store_policy, the others f32_store_policy.
template <bool ADD, bool STATS, bool DIV = false>
int run_dequant(float* out, const float* lut, const uint8_t* codes, int64_t n, Workspace* ws, hipStream_t st, int* grid_out,
                float divisor = 1.0f) {
    const int grid = grid_for(n, ADD);        // accumulate reads 5 bytes per element and writes 4; set reads 1 and writes 4
    const int id = STATS ? (ADD ? kIdDequantAddStats : kIdDequantSetStats) : (ADD ? kIdDequantAdd : kIdDequantSet);
    const double bytes = (ADD ? 9.0 : 5.0) * n;
    const int pol = STATS ? g_opt.f32_reread_store_policy : g_opt.f32_store_policy;
    with_policy(pol, [&](auto policy) {
        launch_dequant<ADD, STATS, DIV, decltype(policy)::value>(id, bytes, grid, st, out, lut, codes, n, ws, divisor);
    });
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
    if (al && g_opt.reverse_second_pass)
        launch(kIdCodeRemap, 2.0 * n, code_remap_kernel<true, true>, grid, kThreads, st, codes_in, codes_out, n, ws);
    else if (al)
        launch(kIdCodeRemap, 2.0 * n, code_remap_kernel<true>, grid, kThreads, st, codes_in, codes_out, n, ws);
    else
        launch(kIdCodeRemap, 2.0 * n, code_remap_kernel<false>, grid, kThreads, st, codes_in, codes_out, n, ws);
    return launch_check("code_remap_kernel");
}

bool bad_n(int64_t n) { return n < 0 || n > kMaxElems; }

}  // namespace

// Scratch of the entry point that allocates nothing: one Workspace per GPU in the code object's
// own device memory (10.1 MiB, held by every device the library runs on until the process
// ends).  In host code the array's name is only a stand-in for the symbol, not a device address:
// the address is looked up once per device with hipGetSymbolAddress, kept, and every launch and
// every other use of the memory gets that pointer.
static __device__ __align__(256) unsigned char scratch[sizeof(Workspace)];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// *out = the current device's copy of `scratch`.  Returns 0, or the error code (text set).
int scratch_workspace(Workspace** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(PRIME_EINVAL, "device index out of range for the built-in scratch");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!ptr) return fail(PRIME_EWORKSPACE, "hipGetSymbolAddress(scratch) returned a null address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = static_cast<Workspace*>(g_scratch_ptr[dev]);
    return 0;
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
        if (value != 1 && value != 2 && value != 4 && value != 8)
            return fail(PRIME_EINVAL, "hist_replicas must be 1, 2, 4 or 8");
        g_opt.hist_replicas = value;
    } else if (!strcmp(name, "average_replicas")) {
        if (value != 1 && value != 2 && value != 4 && value != 8 && value != 16)
            return fail(PRIME_EINVAL, "average_replicas must be 1, 2, 4, 8 or 16");
        g_opt.average_replicas = value;
    } else if (!strcmp(name, "code_store_policy")) {
        if (value != kStorePlain && value != kStoreNt && value != kStoreWriteThrough)
            return fail(PRIME_EINVAL, "code_store_policy must be 0 (plain), 2 (non-temporal) or 16 (write-through)");
        g_opt.code_store_policy = value;
    } else if (!strcmp(name, "f32_store_policy") || !strcmp(name, "f32_reread_store_policy") || !strcmp(name, "copy_store_policy")) {
        if (value != kStorePlain && value != kStoreNt && value != kStoreWriteThrough)
            return fail(PRIME_EINVAL, "a store policy must be 0 (plain), 2 (non-temporal) or 16 (write-through)");
        (name[0] == 'c' ? g_opt.copy_store_policy : name[4] == 's' ? g_opt.f32_store_policy : g_opt.f32_reread_store_policy) = value;
    } else if (!strcmp(name, "large_read_grid_eighths")) {
        if (value < 0 || value > 16) return fail(PRIME_EINVAL, "large_read_grid_eighths must be 0 (off) .. 16");
        g_opt.large_read_grid_eighths = value;
    } else if (!strcmp(name, "stats_grid_eighths")) {
        if (value < 0 || value > 16) return fail(PRIME_EINVAL, "stats_grid_eighths must be 0 (off) .. 16");
        g_opt.stats_grid_eighths = value;
    } else if (!strcmp(name, "large_read_min_mi_elems")) {
        if (value < 0) return fail(PRIME_EINVAL, "large_read_min_mi_elems must be >= 0");
        g_opt.large_read_min_elems = static_cast<int64_t>(value) << 20;
    } else if (!strcmp(name, "grid_cap")) {
        if (value < 0) return fail(PRIME_EINVAL, "grid_cap must be >= 0 (0: none)");
        g_opt.grid_cap = value;
    } else if (!strcmp(name, "one_shot")) {
        g_opt.one_shot = value != 0;
    } else if (!strcmp(name, "one_shot_store_policy")) {
        if (value != kStorePlain && value != kStoreNt && value != kStoreWriteThrough)
            return fail(PRIME_EINVAL, "a store policy must be 0 (plain), 2 (non-temporal) or 16 (write-through)");
        g_opt.one_shot_store_policy = value;
    } else if (!strcmp(name, "small_max_elems")) {
        if (value < 0) return fail(PRIME_EINVAL, "small_max_elems must be >= 0 (0: off)");
        g_opt.small_max_elems = value;
    } else if (!strcmp(name, "two_row_below_mi_elems")) {
        if (value < 0 || value > 8192) return fail(PRIME_EINVAL, "two_row_below_mi_elems must be in [0, 8192] (0: off)");
        g_opt.two_row_below_elems = static_cast<int64_t>(value) << 20;
    } else if (!strcmp(name, "set_four_rows_max_mi_elems")) {
        if (value < 0 || value > 8192) return fail(PRIME_EINVAL, "set_four_rows_max_mi_elems must be in [0, 8192] (0: off)");
        g_opt.set_four_rows_max_elems = static_cast<int64_t>(value) << 20;
    } else if (!strcmp(name, "dynamic_tail_percent")) {
        if (value < 0 || value > 100) return fail(PRIME_EINVAL, "dynamic_tail_percent must be 0 (off) .. 100");
        g_opt.dynamic_tail_percent = value;
    } else if (!strcmp(name, "dynamic_tail_min_mi_elems")) {
        if (value < 0 || value > 8192) return fail(PRIME_EINVAL, "dynamic_tail_min_mi_elems must be in [0, 8192]");
        g_opt.dynamic_tail_min_elems = static_cast<int64_t>(value) << 20;
    } else if (!strcmp(name, "segment_blocks_per_cu")) {
        if (value < 1 || value > 8) return fail(PRIME_EINVAL, "segment_blocks_per_cu must be 1..8");
        g_opt.segment_blocks_per_cu = value;
    } else if (!strcmp(name, "segment_max_mi_elems") || !strcmp(name, "segment_ring_max_mi_elems")) {
        if (value < 0 || value > 8192) return fail(PRIME_EINVAL, "segment_max_mi_elems / segment_ring_max_mi_elems must be in [0, 8192]");
        (name[8] == 'r' ? g_opt.segment_ring_max_elems : g_opt.segment_max_elems) = static_cast<int64_t>(value) << 20;
    } else if (!strcmp(name, "reverse_second_pass")) {
        g_opt.reverse_second_pass = value != 0;
    } else if (!strcmp(name, "nt_load_min_mib")) {
        if (value < 0) return fail(PRIME_EINVAL, "nt_load_min_mib must be >= 0");
        g_opt.nt_load_min_mib = value;
    } else if (!strcmp(name, "mix_cached")) {
        g_opt.mix_cached = value != 0;
    } else if (!strcmp(name, "mixed_grid_eighths")) {
        if (value < 0 || value > 16) return fail(PRIME_EINVAL, "mixed_grid_eighths must be 0 (off) .. 16");
        g_opt.mixed_grid_eighths = value;
    } else if (!strcmp(name, "stats_keep_mib")) {
        if (value < 0) return fail(PRIME_EINVAL, "stats_keep_mib must be >= 0");
        g_opt.stats_keep_mib = value;
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
    else if (!strcmp(name, "code_store_policy")) *value = g_opt.code_store_policy;
    else if (!strcmp(name, "reverse_second_pass")) *value = g_opt.reverse_second_pass;
    else if (!strcmp(name, "segment_blocks_per_cu")) *value = g_opt.segment_blocks_per_cu;
    else if (!strcmp(name, "segment_max_mi_elems")) *value = static_cast<int>(g_opt.segment_max_elems >> 20);
    else if (!strcmp(name, "segment_ring_max_mi_elems")) *value = static_cast<int>(g_opt.segment_ring_max_elems >> 20);
    else if (!strcmp(name, "dynamic_tail_percent")) *value = g_opt.dynamic_tail_percent;
    else if (!strcmp(name, "dynamic_tail_min_mi_elems")) *value = static_cast<int>(g_opt.dynamic_tail_min_elems >> 20);
    else if (!strcmp(name, "large_read_grid_eighths")) *value = g_opt.large_read_grid_eighths;
    else if (!strcmp(name, "large_read_min_mi_elems")) *value = static_cast<int>(g_opt.large_read_min_elems >> 20);
    else if (!strcmp(name, "average_replicas")) *value = g_opt.average_replicas;
    else if (!strcmp(name, "grid_cap")) *value = g_opt.grid_cap;
    else if (!strcmp(name, "one_shot")) *value = g_opt.one_shot;
    else if (!strcmp(name, "one_shot_store_policy")) *value = g_opt.one_shot_store_policy;
    else if (!strcmp(name, "small_max_elems")) *value = static_cast<int>(g_opt.small_max_elems);
    else if (!strcmp(name, "two_row_below_mi_elems")) *value = static_cast<int>(g_opt.two_row_below_elems >> 20);
    else if (!strcmp(name, "set_four_rows_max_mi_elems")) *value = static_cast<int>(g_opt.set_four_rows_max_elems >> 20);
    else if (!strcmp(name, "f32_store_policy")) *value = g_opt.f32_store_policy;
    else if (!strcmp(name, "f32_reread_store_policy")) *value = g_opt.f32_reread_store_policy;
    else if (!strcmp(name, "copy_store_policy")) *value = g_opt.copy_store_policy;
    else if (!strcmp(name, "nt_load_min_mib")) *value = g_opt.nt_load_min_mib;
    else if (!strcmp(name, "nt_second_min_mib")) *value = g_opt.nt_second_min_mib;
    else if (!strcmp(name, "stats_keep_mib")) *value = g_opt.stats_keep_mib;
    else if (!strcmp(name, "stats_grid_eighths")) *value = g_opt.stats_grid_eighths;
    else if (!strcmp(name, "mix_cached")) *value = g_opt.mix_cached;
    else if (!strcmp(name, "mixed_grid_eighths")) *value = g_opt.mixed_grid_eighths;
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
    // Read before the same call sequence writes them: the scale record (cleared so that a stray read is
    // defined) and the tile counter of the fused pass, which must start at zero.  The head of the workspace
    // up to the counter is cleared.
    static_assert(offsetof(Workspace, tile_counter) % 4 == 0 && offsetof(Workspace, tile_counter) < 16384, "the counter sits in the head");
    launch(kIdFill, 0.0, fill_zero_kernel, 1, 64, static_cast<hipStream_t>(stream), static_cast<uint32_t*>(ws),
           static_cast<int64_t>(offsetof(Workspace, tile_counter) / 4 + 1));
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
        grid = grid_for(n, true);
        const int nb = static_cast<int>(n_bins < kBins ? n_bins : kBins);
        const bool al = aligned_to(x, 16) && aligned_to(codes, 4);
        auto go = [&](auto copies) {
            constexpr int R = decltype(copies)::value;
            if (al && nb == kBins && use_nt(n)) launch(kIdHist, 5.0 * n, hist_kernel<true, R, true, true>, grid, kThreads, st, x, codes, n, nb, w);
            else if (al && nb == kBins) launch(kIdHist, 5.0 * n, hist_kernel<true, R, false, true>, grid, kThreads, st, x, codes, n, nb, w);
            else if (al) launch(kIdHist, 5.0 * n, hist_kernel<true, R, false, false>, grid, kThreads, st, x, codes, n, nb, w);
            else launch(kIdHist, 5.0 * n, hist_kernel<false, R, false, false>, grid, kThreads, st, x, codes, n, nb, w);
        };
        switch (g_opt.average_replicas) {
            case 1: go(std::integral_constant<int, 1>{}); break;
            case 2: go(std::integral_constant<int, 2>{}); break;
            case 4: go(std::integral_constant<int, 4>{}); break;
            case 16: go(std::integral_constant<int, 16>{}); break;
            default: go(std::integral_constant<int, 8>{}); break;
        }
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

}  // extern "C"

namespace {

// The single launch of one workgroup, when the tensor is small enough: at most small_max_elems
// elements and a three-launch grid of one workgroup per row, at most kSmallSlots of them.
bool small_applies(int64_t n) {
    if (n <= 0 || n > g_opt.small_max_elems) return false;
    const int64_t grid = grid_for(n, true);
    const int64_t rows = (n / 4 + kThreads - 1) / kThreads;        // rows of whole vectors; the grid counts the ragged end too
    return grid <= kSmallSlots && rows <= grid;
}

template <int SRC>
int run_small(float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qp_out, Workspace* ws, hipStream_t st,
              const uint8_t* codes_in, const float* lut_in, float divisor) {
    const int rows = grid_for(n, true);
    int shift = 0;
    while ((1 << (shift + 1)) <= g_opt.hist_replicas) ++shift;
    if (aligned_to(x, 16) && aligned_to(codes, 4) && aligned_to(codes_in, 4))
        launch(kIdUniformSmall, (SRC == kSmallTensor ? 9.0 : SRC == kSmallSet ? 10.0 : 14.0) * n, uniform_small_kernel<true, SRC>, 1, kThreads, st, x, n,
               rows, qp_out, codes, lut, ws, shift, codes_in, lut_in, divisor);
    else
        launch(kIdUniformSmall, (SRC == kSmallTensor ? 9.0 : SRC == kSmallSet ? 10.0 : 14.0) * n, uniform_small_kernel<false, SRC>, 1, kThreads, st, x, n,
               rows, qp_out, codes, lut, ws, shift, codes_in, lut_in, divisor);
    return launch_check("uniform_small_kernel");
}

int run_uniform_small(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qp_out, Workspace* ws, hipStream_t st) {
    // (the kernel only reads the tensor when it is the source)
    return run_small<kSmallTensor>(const_cast<float*>(x), n, codes, lut, qp_out, ws, st, nullptr, nullptr, 1.0f);
}

int uniform_three_launches(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out, Workspace* w, hipStream_t st) {
    if (n == 0) {
        if (int rc = run_stats(x, 0, qparams_out, w, st)) return rc;
        return run_lut_finalize(w, 0, lut, kBins, nullptr, st);
    }
    int parts = 0, grid = 0;
    if (int rc = run_stats_partials(x, n, w, st, &parts, true)) return rc;
    if (int rc = run_quantize(x, n, 0.0f, parts, qparams_out, kZeroPoint, codes, w, true, st, &grid, true)) return rc;
    return run_lut_finalize(w, grid, lut, kBins, nullptr, st);
}

int uniform_checked(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out, void* ws, prime_stream_t stream,
                    bool may_take_one_launch = true) {
    if (bad_n(n) || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize: bad argument");
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    if (may_take_one_launch && small_applies(n)) return run_uniform_small(x, n, codes, lut, qparams_out, w, st);
    return uniform_three_launches(x, n, codes, lut, qparams_out, w, st);
}

}  // namespace

extern "C" {

int prime_uniform_8bit_quantize(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out, void* ws,
                                prime_stream_t stream) {
    return uniform_checked(x, n, codes, lut, qparams_out, ws, stream);
}

int prime_uniform_8bit_quantize_noalloc(const float* x, int64_t n, uint8_t* codes, float* lut, prime_qparams* qparams_out,
                                        prime_stream_t stream) {
    if (n > kMaxElems) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_noalloc: n exceeds the 2^40 elements the built-in scratch is laid out for");
    if (n < 0 || (n > 0 && (!x || !codes)) || !lut) return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_noalloc: bad argument");
    Workspace* w = nullptr;
    if (int rc = scratch_workspace(&w)) return rc;
    // Nothing in the workspace has to start at zero: every partial a kernel reads was stored by the
    // kernel before it in this same call.
    return prime_uniform_8bit_quantize(x, n, codes, lut, qparams_out, w, stream);
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
    // Several streams pay off while a bucket leaves part of the device idle at its ramps.  A bucket of 2^27 elements or
    // more fills the device on its own and keeps its end in the last-level cache between its two passes, which a
    // neighbour on another stream would displace (8 x 2^27 elements: 1.47 ms on one stream, 1.54 ms on two; 6 x 2^28:
    // 2.12 against 2.40 ms): with such a bucket in the set everything goes to the first stream.
    for (int64_t i = 0; i < count; ++i)
        if (ns[i] >= g_opt.large_read_min_elems) n_streams = 1;
    for (int64_t i = 0; i < count; ++i) {
        const int k = static_cast<int>(i % n_streams);
        if (int rc = uniform_checked(xs[i], ns[i], codes[i], luts + i * kBins, qparams_out ? qparams_out + i : nullptr,
                                     workspaces[k], streams[k]))
            return rc;
    }
    return 0;
}

int prime_uniform_8bit_quantize_batched(const float* x, const int64_t* offsets, int64_t count, uint8_t* codes, float* luts,
                                        prime_qparams* qparams_out, prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!offsets || !luts || !x || !codes)))
        return fail(PRIME_EINVAL, "prime_uniform_8bit_quantize_batched: bad argument");
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
    if (small_applies(n)) {               // one launch of one workgroup, the same results bit for bit
        if (!ADD) return run_small<kSmallSet>(chunk, n, codes_out, lut_out, qparams_out, w, st, codes_in, lut_in, 1.0f);
        if (divisor != 1.0f) return run_small<kSmallAddDiv>(chunk, n, codes_out, lut_out, qparams_out, w, st, codes_in, lut_in, divisor);
        return run_small<kSmallAdd>(chunk, n, codes_out, lut_out, qparams_out, w, st, codes_in, lut_in, 1.0f);
    }
    int grid = 0;
    if (ADD && divisor != 1.0f) {
        if (int rc = run_dequant<ADD, true, ADD>(chunk, lut_in, codes_in, n, w, st, &grid, divisor)) return rc;
    } else {
        if (int rc = run_dequant<ADD, true>(chunk, lut_in, codes_in, n, w, st, &grid)) return rc;
    }
    if (int rc = run_quantize(chunk, n, 0.0f, grid, qparams_out, kZeroPoint, codes_out, w, true, st, &grid, true, true)) return rc;
    return run_lut_finalize(w, grid, lut_out, kBins, nullptr, st);
}

}  // namespace

namespace {

// ---- segmented launches -------------------------------------------------------------------------
enum SegKind { kSegUniform = 0, kSegReduce = 1, kSegGather = 2, kSegReduceDiv = 3 };

// One group of at most kSegMax tensors, all 16-byte (codes: 4-byte) aligned and non-empty: three
// launches.  luts / qps point at the group's first entry.
int run_segment_group(SegKind kind, int count, float* const* xs, const int64_t* ns, uint8_t* const* codes, const uint8_t* const* codes_in,
                      const float* const* luts_in, float divisor, float* luts, prime_qparams* qps, Workspace* w, hipStream_t st) {
    SegJob job;
    memset(&job, 0, sizeof(job));
    job.count = count;
    const bool add = kind == kSegReduce || kind == kSegReduceDiv;
    int64_t total = 0;
    double bytes_a = 0.0, bytes_q = 0.0;
    for (int t = 0; t < count; ++t) {
        job.n[t] = ns[t];
        job.x[t] = xs[t];
        job.codes[t] = codes[t];
        job.codes_in[t] = codes_in ? codes_in[t] : nullptr;
        job.lut_in[t] = luts_in ? luts_in[t] : nullptr;
        // the statistics slots: the grid the one-tensor entry point launches for its first pass
        job.parts[t] = kind == kSegUniform ? stats_grid_for(ns[t]) : grid_for(ns[t], add);
        if (kind == kSegUniform && two_row_tiles(ns[t])) job.two_row |= 1ull << t;
        total += ns[t];
        bytes_a += (kind == kSegUniform ? 4.0 : add ? 9.0 : 5.0) * ns[t];
        bytes_q += 5.0 * ns[t];
    }
    job.first[0] = 0;
    for (int t = 0; t < count; ++t) {
        int blocks = job.parts[t];
        const bool two = (job.two_row >> t) & 1;
        if (kind == kSegUniform && seg_short(ns[t], job.parts[t], two)) blocks = (blocks + seg_short_slots(two) - 1) / seg_short_slots(two);
        job.first[t + 1] = job.first[t] + blocks;
    }
    const int grid_a = job.first[count];
    if (kind == kSegUniform) {
        launch(kIdSegStats, bytes_a, seg_stats_kernel, grid_a, kThreads, st, job, w);
    } else {
        with_policy(g_opt.f32_reread_store_policy, [&](auto P) {
            constexpr int POL = decltype(P)::value;
            if (kind == kSegGather) launch(kIdSegDequantSet, bytes_a, seg_dequant_kernel<false, false, POL>, grid_a, kThreads, st, job, divisor, w);
            else if (kind == kSegReduceDiv && divisor != 1.0f)
                launch(kIdSegDequantAdd, bytes_a, seg_dequant_kernel<true, true, POL>, grid_a, kThreads, st, job, divisor, w);
            else launch(kIdSegDequantAdd, bytes_a, seg_dequant_kernel<true, false, POL>, grid_a, kThreads, st, job, divisor, w);
        });
    }
    if (int rc = launch_check("segmented first pass")) return rc;
    // the quantize pass: segment_blocks_per_cu workgroups per compute unit, shared out by size; a tensor
    // gets at least one and at most one per tile
    const int64_t budget = static_cast<int64_t>(cu_count()) * g_opt.segment_blocks_per_cu;
    job.two_row = 0;
    int first = 0;
    for (int t = 0; t < count; ++t) {
        const bool two = two_row_tiles(ns[t], kind != kSegUniform);
        if (two) job.two_row |= 1ull << t;
        const int64_t rows = (ns[t] + kRowElems - 1) / kRowElems;
        const int64_t tiles = (rows + (two ? 2 : kUnroll) - 1) / (two ? 2 : kUnroll);
        int64_t share = (budget * ns[t] + total / 2) / total;
        if (share > tiles) share = tiles;
        if (share < 1) share = 1;
        job.first[t] = first;
        first += static_cast<int>(share);
    }
    job.first[count] = first;
    if (first > kMaxGrid) return fail(PRIME_EINVAL, "segmented launch: more workgroups than histogram rows in the workspace");
    int shift = 0;
    while ((1 << (shift + 1)) <= g_opt.hist_replicas) ++shift;
    launch(kIdSegQuantize, bytes_q, seg_quantize_kernel<kStoreNt>, first, kThreads, st, job, qps, w, shift);
    if (int rc = launch_check("seg_quantize_kernel")) return rc;
    launch(kIdSegLutFinalize, 16.0 * kBins * first, seg_lut_finalize_kernel, count * kSegFinalBlocks, kSegFinalThreads, st, job, w, luts);
    return launch_check("seg_lut_finalize_kernel");
}

int ring_step_one(SegKind kind, float* chunk, const uint8_t* codes_in, const float* lut_in, int64_t n, float divisor, uint8_t* codes_out,
                  float* lut_out, prime_qparams* qp, void* ws, prime_stream_t stream);

// Every tensor of the call: those a segmented launch can take go in groups of kSegMax, the others
// (empty, or not aligned for vector access) through the one-tensor entry point, which gives the same results.
int run_segmented(SegKind kind, const char* who, float* const* xs, const int64_t* ns, int64_t count, uint8_t* const* codes,
                  const uint8_t* const* codes_in, const float* const* luts_in, float divisor, float* luts, prime_qparams* qps, void* ws,
                  prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!xs || !ns || !codes || !luts)) || (count > 0 && kind != kSegUniform && (!codes_in || !luts_in)))
        return fail(PRIME_EINVAL, who);
    if (!ws) return fail(PRIME_EWORKSPACE, "workspace is null");
    if (kind == kSegReduceDiv && (!(divisor == divisor) || divisor == 0.0f)) return fail(PRIME_EINVAL, "segmented ring step: divisor must be a non-zero number");
    for (int64_t i = 0; i < count; ++i) {
        if (bad_n(ns[i]) || (ns[i] > 0 && (!xs[i] || !codes[i])) || (kind != kSegUniform && ((ns[i] > 0 && !codes_in[i]) || !luts_in[i])))
            return fail(PRIME_EINVAL, who);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    Workspace* w = static_cast<Workspace*>(ws);
    float* gx[kSegMax];
    int64_t gn[kSegMax];
    uint8_t* gc[kSegMax];
    const uint8_t* gci[kSegMax];
    const float* gli[kSegMax];
    int64_t i = 0;
    while (i < count) {
        // a group: consecutive tensors that qualify (outputs of a group are contiguous in luts / qps)
        int g = 0;
        const int64_t start = i;
        while (i < count && g < kSegMax) {
            const bool ok = ns[i] > 0 && ns[i] <= (kind == kSegUniform ? g_opt.segment_max_elems : g_opt.segment_ring_max_elems) &&
                            aligned_to(xs[i], 16) && aligned_to(codes[i], 4) && (kind == kSegUniform || aligned_to(codes_in[i], 4));
            if (!ok) break;
            gx[g] = xs[i];
            gn[g] = ns[i];
            gc[g] = codes[i];
            gci[g] = codes_in ? codes_in[i] : nullptr;
            gli[g] = luts_in ? luts_in[i] : nullptr;
            ++g;
            ++i;
        }
        if (g == 1) {                     // a group of one gains nothing over the one-tensor entry point
            i = start;
            g = 0;
        }
        if (g > 0) {
            if (int rc = run_segment_group(kind, g, gx, gn, gc, codes_in ? gci : nullptr, luts_in ? gli : nullptr, divisor, luts + start * kBins,
                                           qps ? qps + start : nullptr, w, st))
                return rc;
            continue;
        }
        prime_qparams* qp = qps ? qps + i : nullptr;
        int rc;
        if (kind == kSegUniform) rc = uniform_checked(xs[i], ns[i], codes[i], luts + i * kBins, qp, ws, stream);
        else rc = ring_step_one(kind, xs[i], codes_in[i], luts_in[i], ns[i], divisor, codes[i], luts + i * kBins, qp, ws, stream);
        if (rc) return rc;
        ++i;
    }
    return 0;
}

int ring_step_one(SegKind kind, float* chunk, const uint8_t* codes_in, const float* lut_in, int64_t n, float divisor, uint8_t* codes_out,
                  float* lut_out, prime_qparams* qp, void* ws, prime_stream_t stream) {
    if (kind == kSegGather) return ring_step<false>(chunk, codes_in, lut_in, n, codes_out, lut_out, qp, ws, stream, "segmented ring step: bad argument");
    return ring_step<true>(chunk, codes_in, lut_in, n, codes_out, lut_out, qp, ws, stream, "segmented ring step: bad argument",
                           kind == kSegReduceDiv ? divisor : 1.0f);
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

int prime_uniform_8bit_quantize_segmented(const float* const* xs, const int64_t* ns, int64_t count, uint8_t* const* codes, float* luts,
                                          prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    return run_segmented(kSegUniform, "prime_uniform_8bit_quantize_segmented: bad argument", const_cast<float* const*>(xs), ns, count, codes, nullptr,
                         nullptr, 1.0f, luts, qparams_out, ws, stream);
}

int prime_ring_reduce_step_segmented(float* const* accs, const uint8_t* const* codes_in, const float* const* luts_in, const int64_t* ns,
                                     int64_t count, uint8_t* const* codes_out, float* luts_out, prime_qparams* qparams_out, void* ws,
                                     prime_stream_t stream) {
    return run_segmented(kSegReduce, "prime_ring_reduce_step_segmented: bad argument", accs, ns, count, codes_out, codes_in, luts_in, 1.0f, luts_out,
                         qparams_out, ws, stream);
}

int prime_ring_reduce_div_step_segmented(float* const* accs, const uint8_t* const* codes_in, const float* const* luts_in, const int64_t* ns,
                                         int64_t count, float divisor, uint8_t* const* codes_out, float* luts_out,
                                         prime_qparams* qparams_out, void* ws, prime_stream_t stream) {
    return run_segmented(kSegReduceDiv, "prime_ring_reduce_div_step_segmented: bad argument", accs, ns, count, codes_out, codes_in, luts_in, divisor,
                         luts_out, qparams_out, ws, stream);
}

int prime_ring_gather_step_segmented(float* const* chunks, const uint8_t* const* codes_in, const float* const* luts_in, const int64_t* ns,
                                     int64_t count, uint8_t* const* codes_out, float* luts_out, prime_qparams* qparams_out, void* ws,
                                     prime_stream_t stream) {
    return run_segmented(kSegGather, "prime_ring_gather_step_segmented: bad argument", chunks, ns, count, codes_out, codes_in, luts_in, 1.0f, luts_out,
                         qparams_out, ws, stream);
}

int prime_div_f32(float* x, int64_t n, float divisor, prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && !x)) return fail(PRIME_EINVAL, "prime_div_f32: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (aligned_to(x, 16) && one_shot(n))
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdDiv, 8.0 * n, div_kernel<true, decltype(P)::value, true>, stream_shot_grid(n >> 2), kStreamShotThreads, st, x, n, divisor);
        });
    else if (aligned_to(x, 16))
        with_policy(g_opt.f32_store_policy, [&](auto P) {
            launch(kIdDiv, 8.0 * n, div_kernel<true, decltype(P)::value>, grid_for(n), kThreads, st, x, n, divisor);
        });
    else
        launch(kIdDiv, 8.0 * n, div_kernel<false, kStorePlain>, grid_for(n), kThreads, st, x, n, divisor);
    return launch_check("div_kernel");
}

int prime_pseudo_gradient_f32(const float* outer, const float* inner, int64_t n, float world_size, float* out,
                              prime_stream_t stream) {
    if (bad_n(n) || (n > 0 && (!outer || !inner || !out))) return fail(PRIME_EINVAL, "prime_pseudo_gradient_f32: bad argument");
    if (n == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int grid = grid_for(n);
    const bool pg_aligned = aligned_to(outer, 16) && aligned_to(inner, 16) && aligned_to(out, 16);
    if (pg_aligned && one_shot(n))
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<true, true, decltype(P)::value, true>, stream_shot_grid(n >> 2), kStreamShotThreads, st, outer,
                   inner, n, world_size, out);
        });
    else if (pg_aligned)
        with_policy(g_opt.f32_store_policy, [&](auto P) {
            if (use_nt(n))
                launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<true, true, decltype(P)::value>, grid, kThreads, st, outer, inner, n, world_size, out);
            else
                launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<true, false, decltype(P)::value>, grid, kThreads, st, outer, inner, n, world_size, out);
        });
    else
        launch(kIdPseudoGrad, 12.0 * n, pseudo_gradient_kernel<false, false, kStorePlain>, grid, kThreads, st, outer, inner, n, world_size, out);
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
    if (!codes_in) {
        // Nothing received yet: the pseudo-gradient as one workgroup per tile, then the three launches of
        // uniform_8bit_quantize (21 bytes per element) are faster than the looping pass that takes the
        // statistics along, plus the quantize pass (17 bytes per element): 197 against 211 us at 2^26 elements.
        if (int rc = prime_pseudo_gradient_f32(outer, inner, n, world_size, grad_out, stream)) return rc;
        return uniform_checked(grad_out, n, codes_out, lut_out, qparams_out, ws, stream);
    }
    int grid = grid_for(n, true);
    const bool al = aligned_to(outer, 16) && aligned_to(inner, 16) && aligned_to(grad_out, 16) && aligned_to(codes_in, 4);
    // a power of two divides exactly as its reciprocal multiplies: x / 2^k == x * 2^-k bit for bit
    auto pow2 = [](float f) {
        uint32_t b;
        memcpy(&b, &f, 4);
        const uint32_t e = b >> 23;                  // sign 0, exponent field
        return (b & 0x7fffffu) == 0 && e >= 2 && e <= 252;
    };
    // outer, inner and the message are read once: always with the non-temporal hint, so that what the last-level cache
    // keeps is the gradient this pass writes and the quantize pass reads back (2^26 elements: that pass 52 instead of 66 us)
    if (al && pow2(world_size) && pow2(divisor))
        with_policy(g_opt.f32_reread_store_policy, [&](auto P) {
            launch(kIdFirstTouchCodes, 13.0 * n, first_touch_kernel<true, true, true, decltype(P)::value, true>, grid, kThreads, st, outer,
                   inner, n, 1.0f / world_size, codes_in, lut_in, 1.0f / divisor, grad_out, w);
        });
    else if (al)
        with_policy(g_opt.f32_reread_store_policy, [&](auto P) {
            launch(kIdFirstTouchCodes, 13.0 * n, first_touch_kernel<true, true, true, decltype(P)::value>, grid, kThreads, st, outer,
                   inner, n, world_size, codes_in, lut_in, divisor, grad_out, w);
        });
    else
        launch(kIdFirstTouchCodes, 13.0 * n, first_touch_kernel<true, false, false, kStorePlain>, grid, kThreads, st, outer, inner, n, world_size,
               codes_in, lut_in, divisor, grad_out, w);
    if (int rc = launch_check("first_touch_kernel")) return rc;
    if (int rc = run_quantize(grad_out, n, 0.0f, grid, qparams_out, kZeroPoint, codes_out, w, true, st, &grid, true, true)) return rc;
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
    const uint8_t* no_codes = nullptr;
    const float* no_lut = nullptr;
    if (al && one_shot(n))
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdOuterStep, bytes, outer_step_kernel<false, true, true, decltype(P)::value, true>, stream_shot_grid(n >> 2), kStreamShotThreads, st, param,
                   momentum_buf, grad, no_codes, no_lut, inner_out, n, -lr, momentum, first_step);
        });
    else if (al)
        with_policy(g_opt.f32_store_policy, [&](auto P) {
            if (use_nt(n))
                launch(kIdOuterStep, bytes, outer_step_kernel<false, true, true, decltype(P)::value>, grid, kThreads, st, param, momentum_buf,
                       grad, no_codes, no_lut, inner_out, n, -lr, momentum, first_step);
            else
                launch(kIdOuterStep, bytes, outer_step_kernel<false, true, false, decltype(P)::value>, grid, kThreads, st, param, momentum_buf,
                       grad, no_codes, no_lut, inner_out, n, -lr, momentum, first_step);
        });
    else
        launch(kIdOuterStep, bytes, outer_step_kernel<false, false, false, kStorePlain>, grid, kThreads, st, param, momentum_buf, grad, no_codes,
               no_lut, inner_out, n, -lr, momentum, first_step);
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
    const float* no_grad = nullptr;
    if (al && one_shot(n))
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, true, true, decltype(P)::value, true>, shot_grid(n >> 2, kCodesStepShotRows, kCodesStepShotThreads), kCodesStepShotThreads, st, param,
                   momentum_buf, no_grad, codes, lut, inner_out, n, -lr, momentum, first_step);
        });
    else if (al)
        with_policy(g_opt.f32_store_policy, [&](auto P) {
            if (use_nt(n))
                launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, true, true, decltype(P)::value>, grid, kThreads, st, param,
                       momentum_buf, no_grad, codes, lut, inner_out, n, -lr, momentum, first_step);
            else
                launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, true, false, decltype(P)::value>, grid, kThreads, st, param,
                       momentum_buf, no_grad, codes, lut, inner_out, n, -lr, momentum, first_step);
        });
    else
        launch(kIdOuterStepCodes, bytes, outer_step_kernel<true, false, false, kStorePlain>, grid, kThreads, st, param, momentum_buf, no_grad, codes,
               lut, inner_out, n, -lr, momentum, first_step);
    return launch_check("outer_step_kernel");
}

int prime_pseudo_gradient_f32_segmented(const float* const* outers, const float* const* inners, const int64_t* ns, int64_t count,
                                        float world_size, float* const* outs, prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!outers || !inners || !ns || !outs))) return fail(PRIME_EINVAL, "prime_pseudo_gradient_f32_segmented: bad argument");
    for (int64_t i = 0; i < count; ++i)
        if (bad_n(ns[i]) || (ns[i] > 0 && (!outers[i] || !inners[i] || !outs[i])))
            return fail(PRIME_EINVAL, "prime_pseudo_gradient_f32_segmented: bad argument");
    hipStream_t st = static_cast<hipStream_t>(stream);
    SegPointwiseJob job;
    auto flush = [&]() -> int {
        if (job.count == 0) return 0;
        double bytes = 0.0;
        for (int t = 0; t < job.count; ++t) bytes += 12.0 * job.n[t];
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdSegPseudoGrad, bytes, seg_pseudo_gradient_kernel<decltype(P)::value>, job.first[job.count], kStreamShotThreads, st, job, world_size);
        });
        job.count = 0;
        return launch_check("seg_pseudo_gradient_kernel");
    };
    memset(&job, 0, sizeof(job));
    for (int64_t i = 0; i < count; ++i) {
        if (ns[i] == 0) continue;
        const bool al = aligned_to(outers[i], 16) && aligned_to(inners[i], 16) && aligned_to(outs[i], 16);
        if (!al || ns[i] > (int64_t(1) << 33)) {         // the one-tensor entry point takes what a one-workgroup-per-tile launch cannot
            if (int rc = prime_pseudo_gradient_f32(outers[i], inners[i], ns[i], world_size, outs[i], stream)) return rc;
            continue;
        }
        const int blocks = stream_shot_grid(ns[i] >> 2) > 0 ? stream_shot_grid(ns[i] >> 2) : 1;
        if (job.count == kSegMax || job.first[job.count] + static_cast<int64_t>(blocks) > 0x7fffffff)
            if (int rc = flush()) return rc;
        const int t = job.count++;
        job.n[t] = ns[i];
        job.a[t] = const_cast<float*>(outers[i]);
        job.b[t] = const_cast<float*>(inners[i]);
        job.c[t] = outs[i];
        job.first[t + 1] = job.first[t] + blocks;
    }
    return flush();
}

int prime_outer_sgd_nesterov_f32_segmented(float* const* params, float* const* momentum_bufs, const float* const* grads,
                                           float* const* inner_outs, const int64_t* ns, int64_t count, float lr, float momentum,
                                           int first_step, prime_stream_t stream) {
    if (count < 0 || (count > 0 && (!params || !momentum_bufs || !grads || !ns)))
        return fail(PRIME_EINVAL, "prime_outer_sgd_nesterov_f32_segmented: bad argument");
    for (int64_t i = 0; i < count; ++i)
        if (bad_n(ns[i]) || (ns[i] > 0 && (!params[i] || !momentum_bufs[i] || !grads[i])))
            return fail(PRIME_EINVAL, "prime_outer_sgd_nesterov_f32_segmented: bad argument");
    hipStream_t st = static_cast<hipStream_t>(stream);
    SegPointwiseJob job;
    auto flush = [&]() -> int {
        if (job.count == 0) return 0;
        double bytes = 0.0;
        for (int t = 0; t < job.count; ++t) bytes += (job.d[t] ? 24.0 : 20.0) * job.n[t];
        with_policy(g_opt.one_shot_store_policy, [&](auto P) {
            launch(kIdSegOuterStep, bytes, seg_outer_step_kernel<decltype(P)::value>, job.first[job.count], kStreamShotThreads, st, job, -lr, momentum,
                   first_step);
        });
        job.count = 0;
        return launch_check("seg_outer_step_kernel");
    };
    memset(&job, 0, sizeof(job));
    for (int64_t i = 0; i < count; ++i) {
        if (ns[i] == 0) continue;
        float* inner = inner_outs ? inner_outs[i] : nullptr;
        const bool al = aligned_to(params[i], 16) && aligned_to(momentum_bufs[i], 16) && aligned_to(grads[i], 16) && aligned_to(inner, 16);
        if (!al || ns[i] > (int64_t(1) << 33)) {
            if (int rc = prime_outer_sgd_nesterov_f32(params[i], momentum_bufs[i], grads[i], inner, ns[i], lr, momentum, first_step, stream)) return rc;
            continue;
        }
        const int blocks = stream_shot_grid(ns[i] >> 2) > 0 ? stream_shot_grid(ns[i] >> 2) : 1;
        if (job.count == kSegMax || job.first[job.count] + static_cast<int64_t>(blocks) > 0x7fffffff)
            if (int rc = flush()) return rc;
        const int t = job.count++;
        job.n[t] = ns[i];
        job.a[t] = params[i];
        job.b[t] = momentum_bufs[i];
        job.c[t] = const_cast<float*>(grads[i]);
        job.d[t] = inner;
        job.first[t + 1] = job.first[t] + blocks;
    }
    return flush();
}

int prime_copy_bytes(void* dst, const void* src, int64_t n_bytes, prime_stream_t stream) {
    if (n_bytes < 0 || (n_bytes > 0 && (!dst || !src))) return fail(PRIME_EINVAL, "prime_copy_bytes: bad argument");
    if ((n_bytes & 15) || !aligned_to(dst, 16) || !aligned_to(src, 16))
        return fail(PRIME_EINVAL, "prime_copy_bytes: size and pointers must be multiples of 16");
    if (n_bytes == 0) return 0;
    const int64_t nvec = n_bytes >> 4;
    const int grid = grid_for(nvec * 4);
    with_policy(g_opt.copy_store_policy, [&](auto P) {
        if (one_shot(nvec * 4))
            launch(kIdCopy, 2.0 * n_bytes, copy_kernel<decltype(P)::value, true>, stream_shot_grid(nvec), kStreamShotThreads, static_cast<hipStream_t>(stream),
                   static_cast<f4a*>(dst), static_cast<const f4a*>(src), nvec);
        else
            launch(kIdCopy, 2.0 * n_bytes, copy_kernel<decltype(P)::value>, grid, kThreads, static_cast<hipStream_t>(stream),
                   static_cast<f4a*>(dst), static_cast<const f4a*>(src), nvec);
    });
    return launch_check("copy_kernel");
}

}  // extern "C"
