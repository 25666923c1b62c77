// Kernels and C-ABI entry points of the GPT-NeoX decode step for MI355X (gfx950).
// The device building blocks and the design overview live in cfpp_device.hpp.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "cfpp.h"
#include "cfpp_device.hpp"

using namespace cfpp;

// =================================================================================================
// kernels
// =================================================================================================
namespace {

// EX (hidden == NCH*512) is a template parameter of every kernel, chosen by the host: a run-time branch
// between the two variants makes the compiler keep two copies of the in-flight tiles.

// The rows a streaming wave takes from a row range [lo, hi) shared by `nw` waves, as tiles of RPI rows:
// tile t covers rows first + t*step + j*sit, j < RPI, below `end`.  Wave w owns the contiguous rows
// lo + [w n / nw, (w+1) n / nw) in units of RPI rows; it walks through memory sequentially, so it meets every
// memory channel and page in turn and channel conflicts average out within the wave.  (Interleaved ownership,
// wave w taking tiles w, w + nw, ..., was measured slower.)
struct RowWalk { int first, step, sit, end, ntiles; };
template <int RPI>
__device__ __forceinline__ RowWalk row_walk(int w, int nw, int lo, int hi) {
    const int units = (hi - lo + RPI - 1) / RPI;
    RowWalk rw;
    const int u0 = mul_div(w, units, nw), u1 = mul_div(w + 1, units, nw);
    rw.first = lo + u0 * RPI; rw.step = RPI; rw.sit = 1; rw.ntiles = u1 - u0;
    rw.end = lo + u1 * RPI < hi ? lo + u1 * RPI : hi;
    return rw;
}
template <int RPI>
__device__ __forceinline__ int walk_row(const RowWalk& rw, int k) { return rw.first + (k / RPI) * rw.step + (k % RPI) * rw.sit; }

// QKV rows of one streaming wave; result = dot + bias as raw fp32.
template <int NCH, bool EX>
__device__ __forceinline__ void qkv_rows(const LayerParams& p, const half2_t (&x1)[NCH][4], const RowWalk& rw, int lane,
                                         RowTile<NCH, StageARpi<NCH>::value>& pre, RowPark& park) {
    constexpr int RPI = StageARpi<NCH>::value;
    const int first = rw.first, step = rw.step;
    const half_t bias0 = pre.bias;
    gemv_tiles<NCH, RPI, EX, RollTiles<NCH>::value>(
        p.w_qkv, p.H, rw.end, rw.sit, rw.ntiles, [=](int t) { return first + t * step; }, x1, lane, pre, park,
        [&](const RowPark& pk, int k0) {
            if (lane < pk.n) {
                const int row = walk_row<RPI>(rw, k0 + lane);
                float bias = (float)bias0;                       // the first segment's was requested with the first tile
                if (k0 != 0 && p.b_qkv != nullptr) bias = (float)p.b_qkv[row];
                st_agent(p.qkv_raw + row, pk.slot[lane] + (p.b_qkv != nullptr ? bias : 0.f));
            }
        });
}
template <int NCH, bool EX>
__device__ __forceinline__ void qkv_prefetch(const LayerParams& p, const RowWalk& rw, int lane,
                                             RowTile<NCH, StageARpi<NCH>::value>& pre) {
    prefetch_row_tile<NCH, StageARpi<NCH>::value, EX>(pre, p.w_qkv, p.H, rw.first, rw.sit, rw.end, rw.ntiles, lane);
    pre.bias = row_bias_request(p.b_qkv, p.w_qkv, walk_row<StageARpi<NCH>::value>(rw, lane), rw.end);
}

// MLP-up rows of one streaming wave (tiles of kUpRpi adjacent rows); result = gelu(dot + bias) as fp16.
// up_prefetch requests the first tile (before something slow: a LayerNorm, an event), up_rows consumes it.
template <int NCH, bool EX>
__device__ __forceinline__ void up_prefetch(const LayerParams& p, const RowWalk& rw, int lane, RowTile<NCH, kUpRpi>& pre) {
    // (a layer without MLP has no W_up at all: its waves, which have no tiles, request row 0 of W_qkv instead)
    prefetch_row_tile<NCH, kUpRpi, EX>(pre, p.w_up != nullptr ? p.w_up : p.w_qkv, p.H, rw.first, rw.sit, rw.end,
                                       p.w_up != nullptr ? rw.ntiles : 0, lane);
    pre.bias = row_bias_request(p.b_up, p.w_qkv, walk_row<kUpRpi>(rw, lane), rw.end);
}
template <int NCH, bool EX>
__device__ __forceinline__ void up_rows(const LayerParams& p, const half2_t (&x2)[NCH][4], const RowWalk& rw, int lane,
                                        RowTile<NCH, kUpRpi>& pre, RowPark& park) {
    const int first = rw.first, step = rw.step;
    const half_t bias0 = pre.bias;
    gemv_tiles<NCH, kUpRpi, EX, RollTiles<NCH>::value>(
        p.w_up, p.H, rw.end, rw.sit, rw.ntiles, [=](int t) { return first + t * step; }, x2, lane, pre, park,
        [&](const RowPark& pk, int k0) {
            if (lane < pk.n) {
                const int row = walk_row<kUpRpi>(rw, k0 + lane);
                float bias = (float)bias0;                       // the first segment's was requested with the first tile
                if (k0 != 0) bias = (float)p.b_up[row];
                st_agent(p.inter + row, (half_t)gelu_tanh(pk.slot[lane] + bias));
            }
        });
}

// The rows [lo, hi) of one pass (0: QKV, 1 + g: MLP-up phase g), as tiles of RPI rows shared dynamically
// by the streaming waves of this workgroup's team.
template <int RPI>
__device__ __forceinline__ TileTeam make_team(const LayerParams& p, int pass, int lo, int hi, int b, int G, int wave) {
    const int nteams = (G + kTeamWgs - 1) / kTeamWgs, k = b / kTeamWgs;
    const int wgs = (G - k * kTeamWgs) < kTeamWgs ? (G - k * kTeamWgs) : kTeamWgs;
    const int T = (hi - lo + RPI - 1) / RPI;
    const int t0 = mul_div(T, k, nteams), t1 = mul_div(T, k + 1, nteams);
    TileTeam tm;
    tm.counter = p.team + ((size_t)pass * (kMaxGrid / kTeamWgs) + k) * kMailboxInts;
    tm.j = (b - k * kTeamWgs) * kStreamers + wave;
    tm.nw = wgs * kStreamers;
    tm.row0 = lo + t0 * RPI;
    tm.ntiles = t1 - t0;
    tm.end = hi;
    return tm;
}
// MLP-up rows: result = gelu(dot + bias) as fp16
template <int NCH, bool EX>
__device__ __forceinline__ void up_team_rows(const LayerParams& p, const half2_t (&x2)[NCH][4], const TileTeam& tm, int lane,
                                             TeamTiles<NCH, kUpRpi>& tt, RowParkIds& park) {
    gemv_team<NCH, kUpRpi, EX, RollTiles<NCH>::value>(p.w_up, p.H, tm, x2, lane, tt, park, [&](const RowParkIds& pk) {
        const int row = lane < pk.n ? pk.row[lane] : -1;
        const float bias = team_bias<NCH, kUpRpi>(tm, tt, p.b_up, row, row >= 0);     // by all lanes: values cross lanes
        if (row >= 0) st_agent(p.inter + row, (half_t)gelu_tanh(pk.slot[lane] + bias));
    });
}

// ---- split mode: one launch per stage ----------------------------------------------------------
// Three launches; no workgroup waits for another inside any of them (the kernel boundary is the barrier), so this mode
// runs wherever the one-launch kernel cannot be guaranteed its co-residency (reference
// include/5090/pythia_2b8/pythia_kernel_dispatch_split.cu:158-214 splits at the same places, QKV | attention | MLP, but
// runs its stages strictly one after the other):
//   k_stage_qkv   LayerNorm + QKV rows, NW waves per workgroup (eight when that leaves every wave three tiles);
//   k_stage_mid   eight waves per workgroup: four stream the MLP-up rows (they depend on the layer input only), four
//                 run the (head, split) attention items - a chain of dependent round trips that would otherwise be a
//                 launch of its own with nothing to hide behind;
//   k_stage_c     O projection on four waves beside the MLP-down rows on the other four, residual.
template <int NCH, int NW, bool EX>
__global__ __launch_bounds__(NW * 64) void k_stage_qkv(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ float park_mem[NW][kParkRows];
    __shared__ LnShared<NCH> lns;
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);   // wave index in a scalar register
    const int gw = blockIdx.x * NW + wave, nw = gridDim.x * NW;
    RowPark park{park_mem[wave], 0};
    const RowWalk qw = row_walk<StageARpi<NCH>::value>(gw, nw, 0, 3 * p.H);
    LnOwn<NCH, NW> own;
    ln_coop_load<NCH, NW, false>(own, norm_spec(p), wave, lane);
    __builtin_amdgcn_sched_barrier(0);   // the LayerNorm inputs go out first
    RowTile<NCH, StageARpi<NCH>::value> t0;
    qkv_prefetch<NCH, EX>(p, qw, lane, t0);
    ln_coop_finish<NCH, NW, false>(own, norm_spec(p), lns, wave, lane);
    half2_t xr[NCH][4];
    ln_fetch<NCH>(lns, 0, lane, xr);
    qkv_rows<NCH, EX>(p, xr, qw, lane, t0, park);
}

// MLP-up rows on the streaming waves of the first p.up_wgs workgroups (one per compute unit), attention items on the
// other four waves: wave hw of workgroup b takes item b + hw G.  The host sizes the grid so that every item has a wave
// (workgroups beyond p.up_wgs have no rows and only run items; nothing here waits for another workgroup, so they may
// start whenever a compute unit has room).  The two halves share nothing but the workgroup barriers of the norm, which
// the attention waves only pass through with their item's loads in flight.  (One item per wave and no loop: a loop
// around the item makes the compiler keep more than 256 registers alive.)
template <int NCH, bool EX>
__global__ __launch_bounds__(2 * kStreamers * 64) void k_stage_mid(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ float park_mem[kStreamers][kParkRows];
    __shared__ LnShared<NCH> lns;
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int G = gridDim.x, b = blockIdx.x;
    const SeqLen sl = load_seq_len(p);      // by every wave: thread 0 of workgroup 0 reports a length that is out of range
    // the post-attention LayerNorm of the input row (slot 0 holds it: only one row is needed here)
    NormSpec ns = norm_spec(p);
    ns.w1 = p.ln2_w; ns.b1 = p.ln2_b;
    if (wave < kStreamers) {
        LnOwn<NCH, kStreamers> own;
        ln_coop_load<NCH, kStreamers, false>(own, ns, wave, lane);
        __builtin_amdgcn_sched_barrier(0);
        RowTile<NCH, kUpRpi> u0;
        const bool rows = b < p.up_wgs;
        const RowWalk uw = row_walk<kUpRpi>((rows ? b : 0) * kStreamers + wave, p.up_wgs * kStreamers, 0, rows ? p.F : 0);
        up_prefetch<NCH, EX>(p, uw, lane, u0);
        ln_coop_finish<NCH, kStreamers, false>(own, ns, lns, wave, lane);
        RowPark park{park_mem[wave], 0};
        half2_t xr[NCH][4];
        ln_fetch<NCH>(lns, 0, lane, xr);
        up_rows<NCH, EX>(p, xr, uw, lane, u0, park);
    } else {
        const int hw = wave - kStreamers;
        const int nsplit = effective_split(p, sl.S), per_head = items_per_head(nsplit);
        const int nitems = p.heads * per_head;
        AttnItem it;
        int item = b + hw * G;
        if (item < nitems) attn_prefetch(p, it, item / per_head, item % per_head, nsplit, sl, lane);
        ln_coop_bystander(ns);
        __builtin_amdgcn_s_setprio(3);   // few instructions, long dependent latencies: let them issue at once
        if (item < nitems) attention_item(p, it, lane, 0, 0);
    }
}

// Norm + gated MLP-up (SwiGLU): inter[r] = silu(Wg[r] . n) * (Wu[r] . n), n = norm(x), with p.w_up = [Wg; Wu] ([2F, H]).
// A tile is the pair (gate row r, up row r + F); a wave owns a contiguous range of pairs.
template <int NCH, bool EX>
__global__ __launch_bounds__(kStreamers * 64) void k_gated_up(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ float park_mem[kStreamers][kParkRows];
    __shared__ LnShared<NCH> lns;
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int gw = blockIdx.x * kStreamers + wave, nw = gridDim.x * kStreamers;
    RowPark park{park_mem[wave], 0};
    const int F = p.F;
    const int first = mul_div(gw, F, nw), count = mul_div(gw + 1, F, nw) - first;
    LnOwn<NCH, kStreamers> own;
    ln_coop_load<NCH, kStreamers, false>(own, norm_spec(p), wave, lane);
    __builtin_amdgcn_sched_barrier(0);   // the norm inputs go out first
    RowTile<NCH, 2> t0;
    prefetch_row_tile<NCH, 2, EX>(t0, p.w_up, p.H, first, F, 2 * F, count, lane);
    ln_coop_finish<NCH, kStreamers, false>(own, norm_spec(p), lns, wave, lane);
    half2_t xr[NCH][4];
    ln_fetch<NCH>(lns, 0, lane, xr);
    gemv_tiles<NCH, 2, EX>(
        p.w_up, p.H, 2 * F, F, count, [=](int t) { return first + t; }, xr, lane, t0, park,
        [&](const RowPark& pk, int k0) {
            if (2 * lane + 1 < pk.n) {
                const int row = first + k0 / 2 + lane;
                p.inter[row] = (half_t)(silu(pk.slot[2 * lane]) * pk.slot[2 * lane + 1]);
            }
        });
}

// The whole gated MLP block in one launch: norm -> gate/up pairs in kUpPhases phases (a wave owns a contiguous range
// of pairs of every phase; event kBarUp + g after phase g) -> down rows of stage C, which start on phase g of the
// intermediate as soon as its event is complete, with their first weight tiles requested before the wait.  One
// workgroup per compute unit, all co-resident; launch tag from the workspace's launch generation.
template <int NCH, int CPD, bool EX>
__global__ __launch_bounds__(kStreamers * 64) void k_gated_mlp(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ float park_mem[kStreamers][kParkRows];
    __shared__ LnShared<NCH> lns;
    __shared__ StageCShared shc;
    __shared__ int arrived[kUpPhases];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int gen = launch_generation_request(p.grp, lane);
    const int G = gridDim.x, b = blockIdx.x;
    const int gw = b * kStreamers + wave, nw = G * kStreamers;
    const StatusSink status = status_sink(p);
    if (threadIdx.x < kUpPhases) arrived[threadIdx.x] = 0;
    RowPark park{park_mem[wave], 0};
    const int F = p.F;
    auto share = [&](int g, int& first, int& count) {      // this wave's pairs of phase g
        const int lo = g == 0 ? 0 : up_phase_rows(CPD, g - 1, F), hi = up_phase_rows(CPD, g, F);
        const int f0 = lo + mul_div(gw, hi - lo, nw), f1 = lo + mul_div(gw + 1, hi - lo, nw);
        first = f0; count = f1 - f0;
    };
    int first, count;
    share(0, first, count);
    LnOwn<NCH, kStreamers> own;
    ln_coop_load<NCH, kStreamers, false>(own, norm_spec(p), wave, lane);
    __builtin_amdgcn_sched_barrier(0);   // the norm inputs go out first
    RowTile<NCH, 2> t0;
    prefetch_row_tile<NCH, 2, EX>(t0, p.w_up, p.H, first, F, 2 * F, count, lane);
    ln_coop_finish<NCH, kStreamers, false>(own, norm_spec(p), lns, wave, lane);
    const int tag = launch_generation_tag(gen, lane);
    half2_t xr[NCH][4];
    ln_fetch<NCH>(lns, 0, lane, xr);
#pragma unroll
    for (int g = 0; g < kUpPhases; ++g) {
        const int f = first;
        gemv_tiles<NCH, 2, EX>(
            p.w_up, p.H, 2 * F, F, count, [=](int t) { return f + t; }, xr, lane, t0, park,
            [&](const RowPark& pk, int k0) {
                if (2 * lane + 1 < pk.n) st_agent(p.inter + f + k0 / 2 + lane, (half_t)(silu(pk.slot[2 * lane]) * pk.slot[2 * lane + 1]));
            });
        // counted in before the next pass's first tile is requested: the count waits for this wave's stores, and would
        // wait for that tile as well
        event_arrive(p.bar, p.grp, p.mbox, kBarUp + g, G, &arrived[g], kStreamers, tag);
        if (g + 1 < kUpPhases) {
            share(g + 1, first, count);
            prefetch_row_tile<NCH, 2, EX>(t0, p.w_up, p.H, first, F, 2 * F, count, lane);
        }
    }
    const StageC c = make_stage_c(p);
    stage_c_rows<NCH, CPD>(c, b, G, shc, true, wave, wave, kStreamers, lane,
                           [&](int g) { event_wait(p.mbox, kBarUp + g, tag, status); }, [] {});
    if (wave == 0) launch_generation_leave(p.grp, b, lane);
}

// one (head, split) item per wave
__global__ __launch_bounds__(kStreamers * 64) void k_stage_b(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);   // wave index in a scalar register
    const SeqLen sl = load_seq_len(p);
    const int nsplit = effective_split(p, sl.S), per_head = items_per_head(nsplit);
    const int item = blockIdx.x * kStreamers + wave;
    if (item < p.heads * per_head) {
        AttnItem it;
        attn_prefetch(p, it, item / per_head, item % per_head, nsplit, sl, lane);
        attention_item(p, it, lane, 0, 0);
    }
}

template <int NCH, int CPD>
__global__ __launch_bounds__(kStreamers * 64) void k_stage_c(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ StageCShared sh;
    const int wave = first_lane(threadIdx.x >> 6);
    const StageC c = make_stage_c(p);
    stage_c_rows<NCH, CPD>(c, blockIdx.x, gridDim.x, sh, true, wave, wave, kStreamers, threadIdx.x & 63, [](int) {}, [] {});
}
// The same with eight waves, shared out as in the one-launch kernel: MLP-down rows on four waves, the O projection on the
// other four (all eight when there is no MLP-down pass).  Which wave computes a row does not change its value.
template <int NCH, int CPD>
__global__ __launch_bounds__(2 * kStreamers * 64) void k_stage_c8(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ StageCShared sh;
    const int wave = first_lane(threadIdx.x >> 6);
    const StageC c = make_stage_c(p);
    const bool streamer = wave < kStreamers, all_o = c.K2 == 0;
    stage_c_rows<NCH, CPD>(c, blockIdx.x, gridDim.x, sh, streamer, wave, all_o ? wave : (streamer ? -1 : wave - kStreamers),
                           all_o ? 2 * kStreamers : kStreamers, threadIdx.x & 63, [](int) {}, [] {});
}

// ---- fused mode: one persistent launch ---------------------------------------------------------
// One workgroup per compute unit, eight waves: four streaming waves (one per SIMD) and four attention waves.
//   all waves:      LayerNorm shared through LDS (each wave loads one 512-half chunk of the row).
//   streaming wave: first QKV tile requested before the LayerNorm -> its QKV rows -> bump kBarQkv -> its MLP-up
//                   tiles, phase by phase (by ticket within a team of workgroups when the phases are long
//                   enough), bumping kBarUp + g after phase g -> MLP-down rows of stage C, phase by phase
//                   (first weight tile in flight, then wait for kBarUp + g): the first down phase only needs
//                   the first up phase of every workgroup, so a workgroup that is late with its MLP-up rows
//                   holds up nobody until the second half of the down pass.
//   attention wave: shares the QKV rows with the streaming waves when every wave still gets three tiles; owns at
//                   most one (head, split) item (the host caps the KV splits so that one attention wave per
//                   workgroup stays without: that one carries the MLP-up arrivals of its workgroup to the
//                   device-wide counters): requests its first K/V tiles and RoPE coefficients, waits for
//                   kBarQkv, runs the item at raised wave priority (the last wave of a head merges its
//                   splits and bumps kBarHeads), then does the O-projection rows of stage C (all rows
//                   requested, then wait for kBarHeads).  Attention is a chain of dependent memory round
//                   trips; it and the O projection run beside the MLP-up / MLP-down streaming instead of in
//                   front of it.
//   all waves:      row reduction in LDS, bias, residual.
// Nothing is reset at the end: counters zero themselves and flags carry a launch tag (from the launch generation of the
// workspace, or from the caller's step counter in the whole-model decoder).  All workgroups must be
// co-resident (the host launches one per compute unit); every wait is bounded.
constexpr int kXcds = 8;      // chiplets (accelerator complex dies) of the device, each with its own L2
constexpr long long kXcdGroupBytes = 3 << 19;     // 1.5 MB of the 4 MB
struct FusedShared { int arrived[1 + kUpPhases]; int give_up; };


template <int NCH>
struct FusedLds {
    FusedShared q;
    StageCShared shc;
    LnShared<NCH> lns;
    float park_mem[kStreamers][kParkRows];
    int park_rows[kStreamers][kParkRows];
    float park_attn[kStreamers][kParkRows];   // QKV rows of the attention waves
};

// One layer; `gen_word` is the word the launch tag derives from (the generation of the workspace, or the caller's step
// counter), requested at the start of the launch.
// CHAIN: the launch runs the layers of a whole model one after the other (k_fused_stack), and this is one of them.  Its
// input row is the previous layer's output row, written by all workgroups: `wait_prev` makes the workgroup wait until all
// of them have said so (layer_done_wait for the previous layer's tag, tag - 1), with the first weight tiles already
// requested; `announce` makes it say so itself once its output rows are stored.  Rows that cross layers go past the caches.
template <int NCH, int CPD, bool EX, bool BYX, bool CHAIN = false>
__device__ __forceinline__ bool fused_layer(const LayerParams& p, int gen_word, FusedLds<NCH>& lds, bool wait_prev = false,
                                            bool announce = false) {
    FusedShared& q = lds.q;
    StageCShared& shc = lds.shc;
    LnShared<NCH>& lns = lds.lns;
    float (&park_mem)[kStreamers][kParkRows] = lds.park_mem;
    int (&park_rows)[kStreamers][kParkRows] = lds.park_rows;
    int thread = threadIdx.x, lane_id = threadIdx.x & 63;
    // In a loop over layers the compiler would work out everything that depends on the lane alone once, in front of the
    // loop, and keep it in registers across all layers (two dozen of them, in a function that has none to spare):
    // the lane index is made opaque per layer, so that those values are worked out where they are used.
    if constexpr (CHAIN) asm volatile("" : "+v"(lane_id), "+v"(thread));
    const int lane = lane_id, wave = first_lane(thread >> 6);   // wave index in a scalar register
    const int G = gridDim.x, b = blockIdx.x;
    const int nsw = G * kStreamers;                 // streaming waves in the grid
    const StatusSink status = status_sink(p);
    const int seq_requested = seq_len_request(p);     // on its way before anything else
    if (thread <= kUpPhases) q.arrived[thread] = 0;
    if (CHAIN && thread == kUpPhases + 1) q.give_up = 0;
    __syncthreads();
    trace_mark(p, 0);
    trace_value(p, 8, __builtin_amdgcn_s_getreg((3 << 11) | 20));   // XCC_ID: which XCD this workgroup runs on
    trace_value(p, 11, __builtin_amdgcn_s_getreg((31 << 11) | 4));  // HW_ID: wave slot, SIMD, CU, SE

    // LayerNorm by all eight waves.  Its (few) loads go out first; behind them the first QKV tile of a streaming
    // wave, so that it is on its way while the statistics are computed
    constexpr int kFusedWaves = 2 * kStreamers;
    constexpr int RPIA = StageARpi<NCH>::value;
    // QKV rows: shared by all eight waves of every workgroup (the attention waves have nothing else to do until the
    // QKV rows exist, and twice as many loads in flight stream faster), or by the streaming waves only
    // (only when that leaves every wave three tiles or more: with fewer, the attention waves start their items later
    // than the shorter QKV pass gains)
    const int qkv_units = (3 * p.H + RPIA - 1) / RPIA;
    const bool qkv8 = qkv_units >= 3 * G * kFusedWaves;
    const RowWalk qw = qkv8 ? row_walk<RPIA>(b * kFusedWaves + wave, G * kFusedWaves, 0, 3 * p.H)
                            : row_walk<RPIA>(b * kStreamers + (wave < kStreamers ? wave : 0), nsw, 0,
                                             wave < kStreamers ? 3 * p.H : 0);
    const int qkv_arrivals = qkv8 ? kFusedWaves : kStreamers;
    const int hw = wave - kStreamers;
    RowTile<NCH, StageARpi<NCH>::value> t0;
    // The norm, with or without a first weight tile requested behind its inputs.  The two cases are two copies of the code,
    // not one copy with a branch around the tile's loads: behind such a branch the compiler's wait for the norm's inputs
    // waits for the tile as well (it counts the loads in flight by the shorter path), and the norm of the whole workgroup
    // then starts when the slowest wave's tile has arrived instead of when the input row has.
    auto norm_phase = [&](auto with_tile) {
        LnOwn<NCH, kFusedWaves> own;
        if constexpr (CHAIN) {
            // the weight tile does not depend on the previous layer: requested first, it is on its way while the last
            // workgroups finish that layer.  One wave polls, the others wait for it at the barrier.
            if constexpr (decltype(with_tile)::value) qkv_prefetch<NCH, EX>(p, qw, lane, t0);
            if (wait_prev) {
                if (wave == kFusedWaves - 1 &&
                    !layer_done_wait(p.grp, G, first_lane(gen_word) * p.tag_mul + p.tag_add, status, lane) && lane == 0)
                    q.give_up = 1;
                __syncthreads();
            }
            ln_coop_load<NCH, kFusedWaves, true, true>(own, norm_spec(p), wave, lane);
        } else {
            ln_coop_load<NCH, kFusedWaves, true>(own, norm_spec(p), wave, lane);
            __builtin_amdgcn_sched_barrier(0);   // the LayerNorm inputs go out first
            if constexpr (decltype(with_tile)::value) qkv_prefetch<NCH, EX>(p, qw, lane, t0);
        }
        trace_mark(p, 14);
#ifdef CFPP_TRACE
        trace_value(p, 15, wall_clock64() + (long long)(own.rx[0].x & 0u));     // the wave's chunk of the input row has arrived
#endif
        ln_coop_finish<NCH, kFusedWaves, true>(own, norm_spec(p), lns, wave, lane);
    };
    if (qkv8 || wave < kStreamers) norm_phase(std::true_type{});
    else norm_phase(std::false_type{});
    // A wait for the previous layer that expired (the status flag is raised: some workgroup is not running, which the
    // host's co-residency check is there to exclude) ends the launch for this workgroup: every later wait would expire as
    // well, a second at a time.  The workgroups that wait for this one give up at their own next layer.
    if (CHAIN && wait_prev && q.give_up) return false;
    trace_mark(p, 1);
    // The launch tag and the sequence length were requested at the top of the kernel.  They are looked at (`resolve`)
    // only once a wave has used up its first weight tile: every load of a wave returns in order, so by then they are
    // there for free, whereas waiting for them right here would also wait for the tile in flight, with the request for
    // the next tile still to come - a memory round trip with nothing in flight at the start of every wave's rows.
    int tag = 0, nsplit = 1, per_head = 2, item_lo = 0, item_step = 1, nitems = 0, head_lo = 0, attn_count = 0;
    SeqLen sl{0, true};
    bool by_xcd = false, agent_up = false;
    // Which (head, split) items the attention waves of this workgroup take.  Normally item b + hw G.  When a head's slice
    // of a cache row is not a whole number of 128-byte memory lines (80-dim heads: 160 bytes), neighbouring heads share
    // lines, and each of the eight chiplets, with its own L2, would fetch a shared line again: the heads are then dealt
    // out in eight groups of adjacent heads, one per chiplet (workgroup b runs on chiplet b mod 8; if a machine places
    // them differently, only this saving is lost), so that a line is fetched once.  Only while the K and V rows of a
    // group of heads stay in that L2 beside the weight stream (measured on Pythia-2.8B: TPOT -2.5 % at context 1024, -1.2 %
    // at 512, but +0.7 % at 1536 and +1.5 % at 4096).
    // BYX is the host's part of the condition (head size, head count and grid; a template flag, so that layers whose
    // heads are whole lines carry none of this).
    // Counting an arrival device-wide is two dependent atomic round trips for the wave that does it, and a
    // streaming wave that stops for them falls behind its workgroup (and then is the last one again at the next
    // event).  When the workgroup has an attention wave without an item (fewer than four items), the streaming
    // waves only drain their stores and count themselves in LDS at the MLP-up events, and that idle wave carries
    // the count to the device-wide counters.  (Not at the QKV event: the attention waves wait for that one, and
    // an arrival that goes through another wave reaches them later.)
    auto resolve = [&]() {
        tag = p.tag_src != nullptr ? first_lane(gen_word) * p.tag_mul + p.tag_add + 1 : launch_generation_tag(gen_word, lane);
        sl = seq_len_check(p, first_lane(seq_requested));
        nsplit = effective_split(p, sl.S);
        per_head = items_per_head(nsplit);
        by_xcd = BYX && (long long)sl.S * (p.heads / kXcds) * p.D * 4 <= kXcdGroupBytes;
        item_lo = by_xcd ? b / kXcds : b;
        item_step = by_xcd ? G / kXcds : G;
        nitems = (by_xcd ? p.heads / kXcds : p.heads) * per_head;        // of this workgroup's chiplet / of the layer
        head_lo = by_xcd ? (b % kXcds) * (p.heads / kXcds) : 0;
        attn_count = nitems > item_lo ? (nitems - item_lo + item_step - 1) / item_step : 0;
        agent_up = p.arrival_agents && attn_count < kStreamers;
    };
    auto stream_arrive = [&](int event, int* lds_ctr, bool agent) {
        if (agent) {
            drain_memory_ops();
            if (lane == 0) __hip_atomic_fetch_add(lds_ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            event_arrive(p.bar, p.grp, p.mbox, event, G, lds_ctr, kStreamers, tag, lane);
        }
    };
    auto agent_serve = [&](int event, int* lds_ctr) {
        if (lane == 0) {
            int spins = 0;
            while (__hip_atomic_load(lds_ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < kStreamers) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > kSpinLimit * 8) { raise_status(status, kStatusSpin); break; }
            }
        }
        __builtin_amdgcn_wave_barrier();
        event_arrive(p.bar, p.grp, p.mbox, event, G, nullptr, 1, tag, lane);
    };

    if (wave < kStreamers) {
        RowPark spark{park_mem[wave], 0};
        RowParkIds park{park_mem[wave], park_rows[wave], 0};
        half2_t xr[NCH][4];   // ln1(x) for the QKV rows, then ln2(x) for the MLP-up rows
        ln_fetch<NCH>(lns, 0, lane, xr);
        qkv_rows<NCH, EX>(p, xr, qw, lane, t0, spark);
        resolve();
        // the MLP-up tiles of a phase are handed out dynamically within the team (only when a wave can expect four
        // tiles or more per phase: with fewer, the static shares are already as fine as the tickets, and the ticket
        // round trips cost more than they balance)
        TileTeam utm = make_team<kUpRpi>(p, 1, 0, up_phase_rows(CPD, 0, p.F), b, G, wave);
        const bool dynamic = utm.ntiles >= 4 * utm.nw;
        // A wave counts itself in for an event before it requests the first tile of its next pass: the count has to wait
        // for the wave's stores, and that wait would be for the requested tile as well (one counter covers both).  The
        // exception are the MLP-up phases with shared tiles, where the request goes first: there the tile in flight
        // at the hand-over is worth more than the earlier event (both orders measured, on both models).
        if (dynamic) {
            TeamTiles<NCH, kUpRpi> ut;
            event_arrive(p.bar, p.grp, p.mbox, kBarQkv, G, &q.arrived[0], qkv_arrivals, tag, lane);
            team_prefetch<NCH, kUpRpi, EX>(p.w_up, p.H, utm, lane, ut, p.b_up);
            trace_mark(p, 2);
            ln_fetch<NCH>(lns, 1, lane, xr);
#pragma unroll
            for (int g = 0; g < kUpPhases; ++g) {
                up_team_rows<NCH, EX>(p, xr, utm, lane, ut, park);
                if (g + 1 < kUpPhases) {
                    utm = make_team<kUpRpi>(p, 2 + g, up_phase_rows(CPD, g, p.F), up_phase_rows(CPD, g + 1, p.F), b, G, wave);
                    team_prefetch<NCH, kUpRpi, EX>(p.w_up, p.H, utm, lane, ut, p.b_up);
                }
                stream_arrive(kBarUp + g, &q.arrived[1 + g], agent_up);
                trace_mark(p, g == kUpPhases - 1 ? 5 : 12);
            }
        } else {
            RowTile<NCH, kUpRpi> u0;
            RowWalk uw = row_walk<kUpRpi>(b * kStreamers + wave, nsw, 0, up_phase_rows(CPD, 0, p.F));
            event_arrive(p.bar, p.grp, p.mbox, kBarQkv, G, &q.arrived[0], qkv_arrivals, tag, lane);
            up_prefetch<NCH, EX>(p, uw, lane, u0);
            trace_mark(p, 2);
            ln_fetch<NCH>(lns, 1, lane, xr);
#pragma unroll
            for (int g = 0; g < kUpPhases; ++g) {
                up_rows<NCH, EX>(p, xr, uw, lane, u0, spark);
                stream_arrive(kBarUp + g, &q.arrived[1 + g], agent_up);
                if (g + 1 < kUpPhases) {
                    uw = row_walk<kUpRpi>(b * kStreamers + wave, nsw, up_phase_rows(CPD, g, p.F), up_phase_rows(CPD, g + 1, p.F));
                    up_prefetch<NCH, EX>(p, uw, lane, u0);
                }
                trace_mark(p, g == kUpPhases - 1 ? 5 : 12);
            }
        }
    } else {
        // an attention wave takes the (head, split) item b + hw G (the host caps the KV splits so that no wave has
        // more than one item: attn_count <= kStreamers); what does not depend on the QKV rows (first K/V tiles,
        // RoPE coefficients) is requested before waiting for them
        if (qkv8) {
            RowPark hpark{lds.park_attn[hw], 0};
            half2_t xq[NCH][4];
            ln_fetch<NCH>(lns, 0, lane, xq);
            // ahead of the streaming wave on the same SIMD: that one goes on to its MLP-up tiles as soon as its own
            // QKV rows are done, and would keep pushing this wave's last QKV tile, which every attention item waits for,
            // further back
            __builtin_amdgcn_s_setprio(2);
            qkv_rows<NCH, EX>(p, xq, qw, lane, t0, hpark);
            resolve();
            event_arrive(p.bar, p.grp, p.mbox, kBarQkv, G, &q.arrived[0], qkv_arrivals, tag, lane);
            __builtin_amdgcn_s_setprio(0);
            trace_mark(p, 2);
        } else {
            resolve();
        }
        if (hw < attn_count) {
            AttnItem it;
            const int item = item_lo + hw * item_step;
            attn_prefetch(p, it, head_lo + item / per_head, item % per_head, nsplit, sl, lane);
            event_wait(p.mbox, kBarQkv, tag, status, lane);
            __builtin_amdgcn_s_setprio(3);   // few instructions, long dependent latencies: let them issue at once
            trace_mark(p, 3);
            attention_item(p, it, lane, G, tag);
            trace_mark(p, 4);
            __builtin_amdgcn_s_setprio(0);
        } else if (hw == kStreamers - 1 && agent_up) {
#pragma unroll
            for (int g = 0; g < kUpPhases; ++g) agent_serve(kBarUp + g, &q.arrived[1 + g]);
        }
    }
    trace_mark(p, 9);
    {
        const StageC c = make_stage_c(p);
        const bool streamer = wave < kStreamers;
        // without an MLP-down pass (attention-only layers) all eight waves share the O-projection rows
        const bool all_o = c.K2 == 0;
        stage_c_rows<NCH, CPD, CHAIN>(
            c, b, G, shc, streamer, wave, all_o ? wave : (streamer ? -1 : wave - kStreamers), all_o ? 2 * kStreamers : kStreamers, lane,
            [&](int g) { event_wait(p.mbox, kBarUp + g, tag, status, lane); trace_mark(p, g == 0 ? 6 : 13); },
            [&] { event_wait(p.mbox, kBarHeads, tag, status, lane); trace_mark(p, 7); }, thread);
    }
    trace_mark(p, 10);
    if constexpr (CHAIN) {
        // the wave that stored this workgroup's output rows raises the workgroup's flag for the next layer
        if (wave == 0 && announce) layer_done_post(p.grp, b, tag, lane);
    } else if (wave == 0 && p.tag_src == nullptr) {
        launch_generation_leave(p.grp, b, lane);      // the flags of this launch turn stale for the next one
    }
    return true;
}

// one layer, parameters in the kernel arguments
template <int NCH, int CPD, bool EX, bool BYX>
__global__ __launch_bounds__(2 * kStreamers * 64) void k_fused(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ FusedLds<NCH> lds;
    // what the flag value (tag) of this launch derives from: requested first, needed at the first event.  The workspace's
    // launch generation (launch_generation_request: a counter per lane), or a counter that the caller advances between
    // launches (a whole-model step: step counter x layers + layer).
    // (a vector load; nothing looks at the value until the wave has used up its first weight tile)
    const int gen_lane = threadIdx.x & 63;
    const int gen_word = counter_peek(p.tag_src != nullptr ? p.tag_src : group_counter(p.grp, kBarExit, gen_lane % kEventGroups));
    fused_layer<NCH, CPD, EX, BYX>(p, gen_word, lds);
}

// All layers of a model in one launch: `table[l]` holds layer l's parameters (tags from the caller's step counter: tag_src
// set, tag_add = l, so that consecutive layers have consecutive tags).  A workgroup that has finished a layer goes on to
// the next one's first weight tiles while others are still busy, and the layers hand their rows over through an event
// instead of a launch boundary.  All workgroups must be co-resident, as for k_fused.
typedef __attribute__((address_space(4))) const LayerParams ConstLayerParams;
template <int NCH, int CPD, bool EX, bool BYX>
__global__ __launch_bounds__(2 * kStreamers * 64) void k_fused_stack(const LayerParams* table, int n_layers) {
    __shared__ FusedLds<NCH> lds;
    const int gen_word = first_lane(counter_peek(((ConstLayerParams*)table)->tag_src));     // the same word for every layer
    for (int l = 0; l < n_layers; ++l) {
        const LayerParams& p = *(const LayerParams*)((ConstLayerParams*)table + l);
        if (!fused_layer<NCH, CPD, EX, BYX, true>(p, gen_word, lds, l > 0, l + 1 < n_layers)) break;
    }
}

// ---- whole-model helpers -----------------------------------------------------------------------
// hidden <- embed[token]   (after the host has set the token; between steps the LM head's last workgroup does this)
__global__ void k_embed(const half_t* __restrict__ embed, const int* __restrict__ state, int H, int vocab,
                        half_t* __restrict__ hidden) {
    int tok = state[0];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i < H) *reinterpret_cast<u32x4*>(hidden + i) = ld16(embed + (size_t)tok * H + i);
}

// What the last workgroup of the LM head to finish does for a whole-model step: the greedy pick over the workgroups'
// best (value, index) pairs, the step's bookkeeping, and the next token's embedding row.
struct LmTail {
    float* best_val;      // one pair per workgroup; nullptr: logits only
    int* best_idx;
    int* state;           // {token, seq_len, step, steps since creation}
    int* done;            // workgroups that have recorded their pair; the last one sets it back to 0
    int* history;
    int hist_cap;
    const half_t* embed;  // [vocab, H]
    half_t* next_x;       // <- embed[token picked]
};

// logits = W LN(x); with a tail, token <- argmax, seq_len <- seq_len + 1, history[step] <- token, next_x <- embed[token]
template <int NCH, bool EX>
__global__ __launch_bounds__(kStreamers * 64) void k_lm_head(const half_t* __restrict__ x, int H, float eps,
                                                      const half_t* __restrict__ ln_w, const half_t* __restrict__ ln_b,
                                                      const half_t* __restrict__ W, int vocab, float* __restrict__ logits,
                                                      LmTail tail) {
    touch_kernel_arguments<128>();
    constexpr int NWV = kStreamers;
    __shared__ float sv[NWV];
    __shared__ int si[NWV];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);   // wave index in a scalar register
    const int gw = blockIdx.x * NWV + wave, nw = gridDim.x * NWV;
    constexpr int RPIA = StageARpi<NCH>::value;
    __shared__ float park_mem[NWV][kParkRows];
    RowPark park{park_mem[wave], 0};
    const RowWalk rw = row_walk<RPIA>(gw, nw, 0, vocab);   // contiguous rows per wave
    __shared__ LnShared<NCH> lns;
    LnOwn<NCH, NWV> own;
    const NormSpec ns{x, nullptr, ln_w, ln_b, nullptr, nullptr, H, 0, eps};
    ln_coop_load<NCH, NWV, false>(own, ns, wave, lane);
    __builtin_amdgcn_sched_barrier(0);   // the LayerNorm inputs go out first
    RowTile<NCH, RPIA> t0;
    prefetch_row_tile<NCH, RPIA, EX>(t0, W, H, rw.first, rw.sit, rw.end, rw.ntiles, lane);
    ln_coop_finish<NCH, NWV, false>(own, ns, lns, wave, lane);
    half2_t x1[NCH][4];
    ln_fetch<NCH>(lns, 0, lane, x1);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    const int first = rw.first, step = rw.step;
    gemv_tiles<NCH, RPIA, EX>(
        W, H, rw.end, rw.sit, rw.ntiles, [=](int t) { return first + t * step; }, x1, lane, t0, park,
        [&](const RowPark& pk, int k0) {
            if (lane < pk.n) {
                const int row = walk_row<RPIA>(rw, k0 + lane);
                const float v = pk.slot[lane];
                logits[row] = v;
                if (v > bv || (v == bv && row < bi)) { bv = v; bi = row; }
            }
        });
    // lanes hold the best of the rows they wrote: reduce over the wave (ties to the lower index)
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ov = xor_shfl(bv, m);
        const int oi = __shfl_xor(bi, m, kWave);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (tail.best_val == nullptr) return;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    __shared__ int last;
    if (threadIdx.x == 0) {
        for (int w = 1; w < NWV; ++w)
            if (sv[w] > bv || (sv[w] == bv && si[w] < bi)) { bv = sv[w]; bi = si[w]; }
        st_agent(tail.best_val + blockIdx.x, bv);
        st_agent(reinterpret_cast<uint32_t*>(tail.best_idx) + blockIdx.x, (uint32_t)bi);
        drain_memory_ops();     // the pair is in memory before this workgroup counts as done
        last = __hip_atomic_fetch_add(tail.done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (int)gridDim.x - 1;
    }
    __syncthreads();
    if (!last) return;
    // every workgroup has recorded its pair: pick over them (ties go to the lower index, whatever the reduction order)
    bv = -INFINITY;
    bi = 0x7fffffff;
    for (int i = threadIdx.x; i < (int)gridDim.x; i += NWV * 64) {
        const float v = ld_agent(tail.best_val + i);
        const int r = counter_peek(tail.best_idx + i);
        if (v > bv || (v == bv && r < bi)) { bv = v; bi = r; }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float ov = xor_shfl(bv, m);
        const int oi = __shfl_xor(bi, m, kWave);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    for (int w = 0; w < NWV; ++w)
        if (sv[w] > bv || (sv[w] == bv && si[w] < bi)) { bv = sv[w]; bi = si[w]; }
    bi = bi < 0 ? 0 : (bi >= vocab ? vocab - 1 : bi);
    for (int i = threadIdx.x * 8; i < H; i += NWV * 64 * 8)
        *reinterpret_cast<u32x4*>(tail.next_x + i) = ld16(tail.embed + (size_t)bi * H + i);
    if (threadIdx.x == 0) {
        const int step = tail.state[2];
        tail.state[0] = bi;
        tail.state[1] = tail.state[1] + 1;
        tail.state[2] = step + 1;
        tail.state[3] = tail.state[3] + 1;      // steps since the stack was created: never reset, launch tags derive from it
        if (step < tail.hist_cap) tail.history[step] = bi;
        __hip_atomic_store(tail.done, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

constexpr int kStateDone = 8;   // word of the stack's state block that counts the LM head's finished workgroups

__global__ void k_set_state(int* state, int token, int seq_len) {
    if (threadIdx.x == 0 && blockIdx.x == 0) { state[0] = token; state[1] = seq_len; state[2] = 0; }
}

__global__ void k_fill_zero(uint32_t* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace

// =================================================================================================
// host side
// =================================================================================================
namespace {

// ---- batched decode over paged caches ---------------------------------------------------------------------
// Several sequences take one decode step together (reference include/5090/llama/kernel_batch_sglang.cuh:43-60: one
// cluster per (sequence, head)).  Here the weight rows are streamed once for a group of up to kBatchTile
// sequences: the normalised input rows of the group sit in LDS as fp16, and every weight tile in registers is
// multiplied with each of them before the next tile arrives.  Three launches: norm + QKV rows (k_batch_gemv),
// attention items over (sequence, head, split) with cache rows looked up through the page table
// (k_batch_attn), O-projection rows (k_batch_gemv again).
constexpr int kBatchTile = 8;        // sequences sharing one pass over the weights
constexpr int kBatchParkRows = 32;   // rows a wave may own in one launch
struct BatchGemv {
    const half_t* W; int R, K;                    // weight rows [R, K]
    const half_t *x, *x_add; half_t* sum_out;     // [batch][K]; x_add: optional second row, sum_out: fp16(x + x_add)
    const half_t* norm_w; float eps;              // RMSNorm weight (null: the rows are used as they are)
    float* out_f32; half_t* out_f16;              // [batch][R], one of the two
    int batch;
};
template <int NCH, bool EX>
__global__ __launch_bounds__(kStreamers * 64) void k_batch_gemv(BatchGemv a) {
    __shared__ __attribute__((aligned(16))) half_t xs[kBatchTile][NCH * kChunk];
    __shared__ float park[kStreamers][kBatchParkRows * kBatchTile];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int gw = blockIdx.x * kStreamers + wave, nw = gridDim.x * kStreamers;
    constexpr int RPI = 2;
    const RowWalk rw = row_walk<RPI>(gw, nw, 0, a.R);
    const int nrows = rw.end > rw.first ? rw.end - rw.first : 0;
    for (int t0 = 0; t0 < a.batch; t0 += kBatchTile) {
        const int nb = a.batch - t0 < kBatchTile ? a.batch - t0 : kBatchTile;
        __syncthreads();     // the previous group's rows in LDS are no longer needed
        RowTile<NCH, RPI> ta, tb;
        if (rw.ntiles > 0) load_row_tile<NCH, RPI, EX>(ta, a.W, a.K, rw.first, 1, rw.end, lane);
        // a wave prepares whole rows: sum with the residual (rounded to fp16), RMS statistics in fp32, fp16 result
        for (int tk = wave; tk < nb; tk += kStreamers) {
            const size_t base = (size_t)(t0 + tk) * a.K;
            float v[NCH][8];
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int col = i * kChunk + lane * 8;
                const bool in = col < a.K;
                u32x4 r = {0u, 0u, 0u, 0u};
                if (in) r = ld16(a.x + base + col);
                unpack8(r, v[i]);
                if (a.x_add != nullptr) {
                    u32x4 ra = {0u, 0u, 0u, 0u};
                    if (in) ra = ld16(a.x_add + base + col);
                    float w[8];
                    unpack8(ra, w);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[i][j] += w[j];
                    r = pack8(v[i]);
                    unpack8(r, v[i]);
                    if (in && a.sum_out != nullptr && blockIdx.x == 0) *reinterpret_cast<u32x4*>(a.sum_out + base + col) = r;
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) ss = fmadd(v[i][j], v[i][j], ss);
            }
            float rstd = 1.f;
            if (a.norm_w != nullptr) rstd = 1.0f / sqrtf(wave_sum(ss) / (float)a.K + a.eps);
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int col = i * kChunk + lane * 8;
                if (a.norm_w != nullptr) {
                    float g[8];
                    u32x4 rg = {0u, 0u, 0u, 0u};
                    if (col < a.K) rg = ld16(a.norm_w + col);
                    unpack8(rg, g);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[i][j] = v[i][j] * rstd * g[j];
                }
                *reinterpret_cast<u32x4*>(&xs[tk][col]) = pack8(v[i]);
            }
        }
        __syncthreads();
        int prow = 0;
        // Sequences are taken two at a time and every dot product is split over two accumulators, so that eight
        // independent chains of dot instructions (and four independent reductions) are in flight: with one wave
        // per SIMD nothing else hides their latencies.
        auto fetch_x = [&](int tk, half2_t (&xv)[NCH][4]) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const u32x4 q = *reinterpret_cast<const u32x4*>(&xs[tk][i * kChunk + lane * 8]);
                xv[i][0] = as_h2(q.x); xv[i][1] = as_h2(q.y); xv[i][2] = as_h2(q.z); xv[i][3] = as_h2(q.w);
            }
        };
        auto consume = [&](const RowTile<NCH, RPI>& t, int valid) {
            int tk = 0;
            for (; tk + 2 <= nb; tk += 2) {
                half2_t xa[NCH][4], xb[NCH][4];
                fetch_x(tk, xa);
                fetch_x(tk + 1, xb);
                float acc[RPI][2][2];
#pragma unroll
                for (int j = 0; j < RPI; ++j) {
                    acc[j][0][0] = acc[j][0][1] = acc[j][1][0] = acc[j][1][1] = 0.f;
#pragma unroll
                    for (int i = 0; i < NCH; ++i) {
                        acc[j][0][i & 1] = dot8(t.w[j][i], xa[i], acc[j][0][i & 1]);
                        acc[j][1][i & 1] = dot8(t.w[j][i], xb[i], acc[j][1][i & 1]);
                    }
                }
#pragma unroll
                for (int j = 0; j < RPI; ++j) {
                    const float ra = wave_sum(acc[j][0][0] + acc[j][0][1]);
                    const float rb = wave_sum(acc[j][1][0] + acc[j][1][1]);
                    if (j < valid && lane == 0) {
                        park[wave][tk * kBatchParkRows + prow + j] = ra;
                        park[wave][(tk + 1) * kBatchParkRows + prow + j] = rb;
                    }
                }
            }
            if (tk < nb) {
                half2_t xa[NCH][4];
                fetch_x(tk, xa);
#pragma unroll
                for (int j = 0; j < RPI; ++j) {
                    float a0 = 0.f, a1 = 0.f;
#pragma unroll
                    for (int i = 0; i < NCH; ++i) {
                        if (i & 1) a1 = dot8(t.w[j][i], xa[i], a1);
                        else a0 = dot8(t.w[j][i], xa[i], a0);
                    }
                    const float ra = wave_sum(a0 + a1);
                    if (j < valid && lane == 0) park[wave][tk * kBatchParkRows + prow + j] = ra;
                }
            }
            prow += valid;
        };
        auto valid_rows = [&](int t) { const int left = nrows - t * RPI; return left < RPI ? left : RPI; };
        auto load = [&](RowTile<NCH, RPI>& t, int i) { load_row_tile<NCH, RPI, EX>(t, a.W, a.K, rw.first + i * RPI, 1, rw.end, lane); };
        int t = 0;
        for (; t + 2 < rw.ntiles; t += 2) {
            load(tb, t + 1);
            consume(ta, RPI);
            __builtin_amdgcn_sched_barrier(0);
            load(ta, t + 2);
            consume(tb, RPI);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (t + 1 < rw.ntiles) {
            load(tb, t + 1);
            consume(ta, RPI);
            __builtin_amdgcn_sched_barrier(0);
            consume(tb, valid_rows(t + 1));
        } else if (t < rw.ntiles) {
            consume(ta, valid_rows(t));
        }
        __builtin_amdgcn_sched_barrier(0);
        // one (sequence, row) result per lane
        for (int idx = lane; idx < nrows * nb; idx += kWave) {
            const int tk = idx / nrows, r = idx - tk * nrows;
            const float val = park[wave][tk * kBatchParkRows + r];
            const size_t o = (size_t)(t0 + tk) * a.R + rw.first + r;
            if (a.out_f32 != nullptr) a.out_f32[o] = val;
            else a.out_f16[o] = (half_t)val;
        }
    }
}

// The same products on the matrix cores: from about eight sequences on, the dot-instruction kernel above is bound
// by its arithmetic, not by the weight stream.  A workgroup owns 16 weight rows; its eight waves split the row
// length, and each wave requests its whole share (16 rows x K/8) at once.  v_mfma_f32_16x16x32_f16 then multiplies
// that 16 x 32 weight block with the matching 32 x 16 block of the (normalised) input rows of 16 sequences; lane l
// supplies row l % 16 and the eight k values of group l / 16 for both operands, so both are loaded with the same
// address pattern.  The input rows come from global memory (every workgroup reads the same few rows: cache hits).
// The weights stay in registers while further groups of 16 sequences are processed.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
struct BatchMfma {
    const half_t* W; int R, K;         // weight rows [R, K]; R % 16 == 0, K % 256 == 0
    const half_t* x;                   // [batch][K]
    float* out_f32; half_t* out_f16;   // [batch][R], one of the two
    int batch;
    // k_batch_mfma_pipe with up to 16 sequences, norm_w not null: the rows of x are raw; the product is taken with
    // fp16(r * norm_w), r = fp16(x + x_add), and scaled by rstd(r) afterwards (the RMSNorm of r, with its one factor per
    // sequence applied to the sums instead of to every element); r goes to sum_out.  x_add and sum_out are not null then.
    const half_t *x_add, *norm_w;
    half_t* sum_out;
    float eps;
};
template <int KSTEPS>
__global__ __launch_bounds__(512) void k_batch_mfma(BatchMfma a) {
    __shared__ f32x4_t red[8][64];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int r0 = blockIdx.x * 16;
    const size_t koff = (size_t)wave * (a.K / 8) + 8 * (lane >> 4);
    const half_t* wp = a.W + (size_t)(r0 + (lane & 15)) * a.K + koff;
    u32x4 w[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) w[s] = ld_stream16(wp + 32 * s);
    for (int t0 = 0; t0 < a.batch; t0 += 16) {
        const int tok = t0 + (lane & 15) < a.batch ? t0 + (lane & 15) : a.batch - 1;
        const half_t* xp = a.x + (size_t)tok * a.K + koff;
        u32x4 x[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) x[s] = ld16(xp + 32 * s);
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, w[s]), __builtin_bit_cast(half8_t, x[s]), acc, 0, 0, 0);
        __syncthreads();      // the previous group's partial sums have been read
        red[wave][lane] = acc;
        __syncthreads();
        // acc[i] of lane l belongs to weight row r0 + 4 (l / 16) + i and sequence t0 + l % 16; wave i adds up element i
        if (wave < 4) {
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += red[u][lane][wave];
            const int seq = t0 + (lane & 15), row = r0 + 4 * (lane >> 4) + wave;
            if (seq < a.batch) {
                const size_t o = (size_t)seq * a.R + row;
                if (a.out_f32 != nullptr) a.out_f32[o] = sum;
                else a.out_f16[o] = (half_t)sum;
            }
        }
    }
}

// Variant for row lengths of 2048 or 4096: the weights are requested row by row (a load instruction fetches 1 KB of
// one row, as the row-streaming kernels do; the operand layout above makes an instruction fetch 64 bytes from each
// of 16 rows) and take the operand layout on their way through LDS: a wave writes 16 rows x 256 halfs at a time
// (rows padded by 16 bytes, so that the sixteen rows a read touches fall into different banks) and reads the
// 16 x 32 blocks back.
constexpr int kMfmaRowBytes = kChunk + 16;
constexpr int kMfmaFullRowBytes = 2 * kChunk + 16;     // a wave's whole 512-half share of a row, same padding
// One workgroup per compute unit walks over its share of the 16-row blocks; wave w owns the
// 512 halfs [512 w, 512 w + 512) of every row (NW = K / 512 waves).  The weights of the next block are requested
// before the current one is multiplied, so the weight stream does not stop for the multiply / reduce phase of a
// block.
template <int NW, bool ONE>
__global__ __launch_bounds__(NW * 64) void k_batch_mfma_pipe(BatchMfma a) {
    __shared__ __attribute__((aligned(16))) unsigned char stage[NW][16 * (ONE ? kMfmaFullRowBytes : kMfmaRowBytes)];
    __shared__ f32x4_t red[NW][64];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int nblocks = a.R / 16;
    const int b0 = mul_div(blockIdx.x, nblocks, gridDim.x), b1 = mul_div(blockIdx.x + 1, nblocks, gridDim.x);
    if (b0 >= b1) return;
    const size_t k0 = (size_t)wave * kChunk;
    unsigned char* mine = stage[wave];
    auto request = [&](u32x4 (&w)[16], int blk) {
#pragma unroll
        for (int j = 0; j < 16; ++j) w[j] = ld_stream16(a.W + (size_t)(blk * 16 + j) * a.K + k0 + lane * 8);
    };
    auto load_x = [&](u32x4 (&x)[16], int t0) {
        const int tok = t0 + (lane & 15) < a.batch ? t0 + (lane & 15) : a.batch - 1;
        const half_t* xp = a.x + (size_t)tok * a.K + k0 + 8 * (lane >> 4);
#pragma unroll
        for (int s = 0; s < 16; ++s) x[s] = ld16(xp + 32 * s);
    };
    // rows -> operand layout through LDS (two halves of 256 halfs)
    auto rearrange = [&](const u32x4 (&w)[16], u32x4 (&op)[16]) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            if ((lane >> 5) == hf) {
#pragma unroll
                for (int j = 0; j < 16; ++j) *reinterpret_cast<u32x4*>(mine + j * kMfmaRowBytes + (lane & 31) * 16) = w[j];
            }
#pragma unroll
            for (int s = 0; s < 8; ++s)
                op[hf * 8 + s] = *reinterpret_cast<const u32x4*>(mine + (lane & 15) * kMfmaRowBytes + s * 64 + (lane >> 4) * 16);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
    };
    // multiply with one group of 16 sequences, add the NW partial sums up, store
    float rs = 1.f;        // factor on the sums of sequence lane % 16 (the RMSNorm's, when this launch takes the norm)
    auto multiply = [&](const u32x4 (&op)[16], const u32x4 (&x)[16], int blk, int t0) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 16; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, op[s]), __builtin_bit_cast(half8_t, x[s]), acc, 0, 0, 0);
        __syncthreads();
        red[wave][lane] = acc;
        __syncthreads();
        if (wave < 4) {
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < NW; ++u) sum += red[u][lane][wave];
            sum *= rs;
            const int seq = t0 + (lane & 15), row = blk * 16 + 4 * (lane >> 4) + wave;
            if (seq < a.batch) {
                const size_t o = (size_t)seq * a.R + row;
                if (a.out_f32 != nullptr) a.out_f32[o] = sum;
                else a.out_f16[o] = (half_t)sum;
            }
        }
    };
    if constexpr (ONE) {
        // up to 16 sequences: their input rows are the same for every block and stay in registers, so the only loads
        // inside the loop are the weights.  A wave stages its whole 512-half share of the 16 rows at once, and a row's
        // registers take the next block's row as soon as the row is in LDS: the number of requests in flight stays at
        // fifteen or sixteen instead of draining to none once per block
        u32x4 w[16], x0[16];
        request(w, b0);
        if (a.norm_w == nullptr) {
            load_x(x0, 0);
        } else {
            // Every workgroup takes the add + RMSNorm of the rows upon itself while its first weights travel (no launch for
            // the norm).  A wave loads its 512-column share of all sixteen rows row by row (1 KB per load instruction, as
            // it loads the weights), leaves r * norm_w in its staging buffer and reads the operand layout back, the way
            // the weight blocks go.  No wave waits for another before the products start: the factor rstd, one per
            // sequence, which needs the whole row, is applied to the sums.  Workgroup 0 stores the rows r.
            __shared__ float ssq[NW][16];
            const size_t col = k0 + lane * 8;
            const u32x4 gw = ld16(a.norm_w + col);
            u32x4 xa[16], xb[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) xa[r] = ld16(a.x + (size_t)(r < a.batch ? r : a.batch - 1) * a.K + col);
#pragma unroll
            for (int r = 0; r < 16; ++r) xb[r] = ld16(a.x_add + (size_t)(r < a.batch ? r : a.batch - 1) * a.K + col);
            // fp16 pair arithmetic: the sum of two fp16 values and the product of two fp16 values are exact in fp32, so
            // rounding them once to fp16 is what the pair instructions do as well; the squares are summed in fp32
            float mine_ss = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t ax[4] = {xa[r].x, xa[r].y, xa[r].z, xa[r].w}, bx[4] = {xb[r].x, xb[r].y, xb[r].z, xb[r].w};
                const uint32_t gx[4] = {gw.x, gw.y, gw.z, gw.w};
                uint32_t rr[4], yy[4];
                float ss = 0.f;
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const half2_t t = as_h2(ax[q4]) + as_h2(bx[q4]);
                    rr[q4] = as_u32(t);
                    ss = __builtin_amdgcn_fdot2(t, t, ss, false);
                    yy[q4] = as_u32(t * as_h2(gx[q4]));
                }
                const u32x4 rv = {rr[0], rr[1], rr[2], rr[3]}, yv = {yy[0], yy[1], yy[2], yy[3]};
                if (blockIdx.x == 0 && r < a.batch) *reinterpret_cast<u32x4*>(a.sum_out + (size_t)r * a.K + col) = rv;
                ss = wave_sum(ss);
                if (lane == r) mine_ss = ss;
                *reinterpret_cast<u32x4*>(mine + r * kMfmaFullRowBytes + lane * 16) = yv;
            }
            if (lane < 16) ssq[wave][lane] = mine_ss;
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
            for (int s = 0; s < 16; ++s)
                x0[s] = *reinterpret_cast<const u32x4*>(mine + (lane & 15) * kMfmaFullRowBytes + s * 64 + (lane >> 4) * 16);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int u = 0; u < NW; ++u) tot += ssq[u][lane & 15];
            rs = 1.0f / sqrtf(tot / (float)a.K + a.eps);
        }
        // The input rows are waited for here, once (with the first block's weights, requested before them and needed next
        // anyway).  Left to the compiler, the wait sits in front of every multiply of every block - it cannot tell the
        // first trip of the loop from the others - and, the rows being the newest loads it knows of, that wait covers the
        // next block's weights as well: no block's loads would overlap the multiply of the block before.
#pragma unroll
        for (int s = 0; s < 16; ++s) asm volatile("" : "+v"(x0[s]));
        // WITH_NEXT: the registers of a row take the next block's row as soon as the row is in LDS.  The last block is a
        // copy of the code without those requests, not a condition around them (a load under a condition makes every
        // wait of the loop assume the path without it and wait for more than it needs).
        auto block = [&](int blk, auto with_next) {
            u32x4 op[16];
            const half_t* next = a.W + (size_t)((blk + 1) * 16) * a.K + k0 + lane * 8;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                *reinterpret_cast<u32x4*>(mine + j * kMfmaFullRowBytes + lane * 16) = w[j];
                if constexpr (decltype(with_next)::value) w[j] = ld_stream16(next + (size_t)j * a.K);
                asm volatile("" ::: "memory");        // keep the store / request pairs in this order
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
            for (int s = 0; s < 16; ++s)
                op[s] = *reinterpret_cast<const u32x4*>(mine + (lane & 15) * kMfmaFullRowBytes + s * 64 + (lane >> 4) * 16);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            multiply(op, x0, blk, 0);
        };
        for (int blk = b0; blk + 1 < b1; ++blk) block(blk, std::true_type{});
        block(b1 - 1, std::false_type{});
    } else {
        u32x4 wa[16], wb[16];
        request(wa, b0);
        auto block = [&](u32x4 (&w)[16], int blk) {
            u32x4 op[16];
            rearrange(w, op);
            for (int t0 = 0; t0 < a.batch; t0 += 16) {
                u32x4 x[16];
                load_x(x, t0);         // cache hits
                multiply(op, x, blk, t0);
            }
        };
        int blk = b0;
        for (; blk + 1 < b1; blk += 2) {
            request(wb, blk + 1);
            block(wa, blk);
            if (blk + 2 < b1) request(wa, blk + 2);
            block(wb, blk + 1);
        }
        if (blk < b1) block(wa, blk);
    }
}

// (Fused add +) RMSNorm of the input rows, one wave per sequence: y = fp16(r * rstd * w), r = fp16(x + x_add) -> sum_out
// (r = x without x_add).
struct BatchNorm {
    const half_t *x, *x_add, *norm_w;
    half_t *sum_out, *y;
    float eps;
    int K, batch;
};
template <int NCH>
__global__ __launch_bounds__(kStreamers * 64) void k_batch_norm(BatchNorm a) {
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int seq = blockIdx.x * kStreamers + wave;
    if (seq >= a.batch) return;
    const size_t base = (size_t)seq * a.K;
    float v[NCH][8];
    float ss = 0.f;
    u32x4 gw[NCH];       // the norm weights travel together with the rows
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col = i * kChunk + lane * 8;
        gw[i] = ld16(a.norm_w + (col < a.K ? col : 0));
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col = i * kChunk + lane * 8;
        const bool in = col < a.K;
        u32x4 r = {0u, 0u, 0u, 0u}, ra = {0u, 0u, 0u, 0u};
        if (in) r = ld16(a.x + base + col);
        unpack8(r, v[i]);
        if (a.x_add != nullptr) {
            if (in) ra = ld16(a.x_add + base + col);
            float w[8];
            unpack8(ra, w);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] += w[j];
            r = pack8(v[i]);
            unpack8(r, v[i]);
            if (in) *reinterpret_cast<u32x4*>(a.sum_out + base + col) = r;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = fmadd(v[i][j], v[i][j], ss);
    }
    const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)a.K + a.eps);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col = i * kChunk + lane * 8;
        if (col < a.K) {
            float g[8];
            unpack8(gw[i], g);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] = v[i][j] * rstd * g[j];
            *reinterpret_cast<u32x4*>(a.y + base + col) = pack8(v[i]);
        }
    }
}

// ---- products with weights stored [in, out] ---------------------------------------------------------------
// y[o] = sum_k x[k] W[k][o] for `nsec` matrices stacked along k (W row s K + k belongs to matrix s; the outputs of
// matrix s go to y[s O ..]): the layout of the reference's plain llama_decoder_layer op (reference
// include/5090/llama/llama_kernel_dispatch.cu:44-58: tensor map with the output features innermost).  A workgroup
// owns a panel of 512 output columns and a slice of the k range: every load instruction of a wave fetches 1 KB of
// one weight row, lane l accumulates its eight columns with the row's x[k] (broadcast from the lane that holds it).
// The slices of a panel meet in a scratch buffer; the workgroup that delivers the last one adds them up in slice
// order (fixed order: the result does not depend on timing).
struct GemvT {
    const half_t* W; int K, O, nsec;
    const half_t* x;                 // [K] fp16
    const half_t* norm_w; float eps; // not null: x stands for fp16(x * rstd(x) * norm_w), the RMSNorm of the row
    float* part;                     // [panels][slices][512]
    int* cnt;                        // [panels], zero between launches
    float* out_f32; half_t* out_f16; // [nsec O], one of the two
    int slices;                      // k slices per panel
};
__global__ __launch_bounds__(kStreamers * 64) void k_gemv_t(GemvT a) {
    __shared__ float red[kStreamers][kChunk];
    __shared__ int last_flag;
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int ppm = (a.O + kChunk - 1) / kChunk;            // panels per matrix
    const int panels = a.nsec * ppm;
    const int panel = blockIdx.x % panels, slice = blockIdx.x / panels;
    if (slice >= a.slices) return;
    const int sec = panel / ppm, col = (panel - sec * ppm) * kChunk + lane * 8;
    const bool in = col < a.O;
    // this wave's rows: slice `slice` of K, quarter `wave` of the slice
    const int part_id = slice * kStreamers + wave, nparts = a.slices * kStreamers;
    const int k0 = mul_div(part_id, a.K, nparts), k1 = mul_div(part_id + 1, a.K, nparts);
    const half_t* wp = a.W + ((size_t)sec * a.K) * a.O + (in ? col : 0);
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    float rstd = 1.f;
    if (a.norm_w != nullptr) {         // every wave takes the statistics of the whole row itself: 2 bytes per k
        float ss = 0.f;
        for (int c0 = lane * 8; c0 < a.K; c0 += kChunk) {
            float f[8];
            unpack8(ld16(a.x + c0), f);
#pragma unroll
            for (int j = 0; j < 8; ++j) ss = fmadd(f[j], f[j], ss);
        }
        rstd = 1.0f / sqrtf(wave_sum(ss) / (float)a.K + a.eps);
    }
    constexpr int kRows = 8;           // rows requested together
    for (int kb = k0; kb < k1; kb += 64) {
        const int n = k1 - kb < 64 ? k1 - kb : 64;
        float xv = lane < n ? (float)a.x[kb + lane] : 0.f;           // x[kb + lane]; rows past the range get 0
        if (a.norm_w != nullptr && lane < n) xv = (float)(half_t)(xv * rstd * (float)a.norm_w[kb + lane]);
        for (int r = 0; r < n; r += kRows) {
            u32x4 w[kRows];
#pragma unroll
            for (int u = 0; u < kRows; ++u) {
                const int k = kb + r + u < k1 ? kb + r + u : k1 - 1;
                w[u] = ld_stream16(wp + (size_t)k * a.O);
            }
#pragma unroll
            for (int u = 0; u < kRows; ++u) {
                const float xk = rl(xv, r + u < 64 ? r + u : 63);    // 0 for rows past the range
                float f[8];
                unpack8(w[u], f);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmadd(xk, f[j], acc[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) red[wave][lane * 8 + j] = acc[j];
    __syncthreads();
    // thread t owns columns 2t and 2t + 1 of the panel from here on (kChunk == 2 * workgroup size)
    static_assert(kChunk == 2 * kStreamers * 64, "two columns per thread");
    const int c = 2 * threadIdx.x;
    float* mine = a.part + ((size_t)panel * a.slices + slice) * kChunk;
    st_agent2(mine + c, red[0][c] + red[1][c] + red[2][c] + red[3][c], red[0][c + 1] + red[1][c + 1] + red[2][c + 1] + red[3][c + 1]);
    drain_memory_ops();
    __syncthreads();
    if (threadIdx.x == 0) {
        const int done = __hip_atomic_fetch_add(a.cnt + panel, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = done == a.slices - 1;
        if (last_flag) __hip_atomic_store(a.cnt + panel, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_flag) return;
    const int pc0 = (panel - sec * ppm) * kChunk;
    if (pc0 + c >= a.O) return;                       // O is a multiple of 8: both columns or none
    // the slices in order, eight requests in flight at a time (requests past the last slice repeat it: a batch
    // without branches, so that none of its loads waits for another)
    const float* col0 = a.part + (size_t)panel * a.slices * kChunk + c;
    float s0 = 0.f, s1 = 0.f;
    for (int sl = 0; sl < a.slices; sl += 8) {
        float u[8], v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int q = sl + i < a.slices ? sl + i : a.slices - 1;
            ld_agent2(col0 + (size_t)q * kChunk, u[i], v[i]);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (sl + i < a.slices) { s0 += u[i]; s1 += v[i]; }
    }
    const size_t o = (size_t)sec * a.O + pc0 + c;
    if (a.out_f32 != nullptr) { a.out_f32[o] = s0; a.out_f32[o + 1] = s1; }
    else { a.out_f16[o] = (half_t)s0; a.out_f16[o + 1] = (half_t)s1; }
}

// stage B with GPT-J pairing of the rotary dims
__global__ __launch_bounds__(kStreamers * 64) void k_stage_b_pairs(LayerParams p) {
    touch_kernel_arguments<kLayerKernargBytes>();
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const SeqLen sl = load_seq_len(p);
    const int nsplit = effective_split(p, sl.S), per_head = items_per_head(nsplit);
    const int item = blockIdx.x * kStreamers + wave;
    if (item < p.heads * per_head) {
        AttnItem it;
        attn_prefetch<false, true>(p, it, item / per_head, item % per_head, nsplit, sl, lane);
        attention_item<false, true>(p, it, lane, 0, 0);
    }
}

struct BatchAttn {
    int batch, layer_id;
    const int *indptr, *indices;                           // page table: rows indices[indptr[b] .. indptr[b+1]-1) hold
                                                           // the sequence, the last entry is the row of the new token
    const unsigned long long *k_ptrs, *v_ptrs;             // per-layer cache base addresses
    const long long* positions;                            // [batch]
    const float* cos_sin;                                  // [positions][D]: cos of the D/2 pair angles, then sin
};
// One wave per (sequence, head, split); the parameter block of the single-sequence kernels, re-pointed at the
// sequence's rows.  With one, two or four split slots per head the four waves of a workgroup hold whole heads, and a
// head's partial results meet in LDS behind a workgroup barrier instead of in scratch memory behind a counter (three
// dependent memory round trips less at the end of every item).
__global__ __launch_bounds__(kStreamers * 64) void k_batch_attn(LayerParams p, BatchAttn b) {
    touch_kernel_arguments<kLayerKernargBytes>();
    __shared__ AttnLdsPart parts[kStreamers];
    const int lane = threadIdx.x & 63, wave = first_lane(threadIdx.x >> 6);
    const int item = blockIdx.x * kStreamers + wave;
    const int slots = p.max_split;                          // item slots per head (split 0 carries the new token)
    const bool in_wg = slots == 1 || slots == 2 || slots == 4;
    const int per_seq = p.heads * slots;
    const int seq = item / per_seq;
    bool active = seq < b.batch;
    const int rem = item - seq * per_seq;
    const int head = rem / slots, sp = rem - head * slots;
    int S = 0, nsplit = 1, start = 0;
    if (active) {
        start = b.indptr[seq];
        S = b.indptr[seq + 1] - 1 - start;
        if (S < 0) {
            if (lane == 0) raise_status(status_sink(p), kStatusSeq);
            active = false;
        } else {
            nsplit = effective_split(p, S);
            active = sp < nsplit;
        }
    }
    if (!in_wg && !active) return;
    LayerParams q = p;
    if (active) {
        q.kv_rows = b.indices + start;
        // The cache addresses come out of a table, so the compiler cannot see what kind of memory they point to and would
        // use generic-address loads, whose completion it cannot count: every wait would then be for all loads in flight.
        // Naming the address space (device memory) keeps them ordinary global loads.
        typedef __attribute__((address_space(1))) half_t* GlobalHalf;
        q.k_cache = (half_t*)(GlobalHalf)b.k_ptrs[b.layer_id];
        q.v_cache = (half_t*)(GlobalHalf)b.v_ptrs[b.layer_id];
        q.cos = b.cos_sin + (size_t)b.positions[seq] * p.D;
        q.sin = q.cos + p.D / 2;
        q.rope_stride = 0;
        q.qkv_raw += (size_t)seq * 3 * p.H;
        q.attn_vec += (size_t)seq * p.H;
        q.k_new += (size_t)seq * p.H;
        q.v_new += (size_t)seq * p.H;
        q.part_ml += (size_t)seq * p.heads * kMaxSplit * 2;
        q.part_acc += (size_t)seq * p.heads * kMaxSplit * p.D;
        q.head_cnt += (size_t)seq * p.heads * kHeadCntStride;
        AttnItem it;
        attn_prefetch<true>(q, it, head, sp, nsplit, SeqLen{S, true}, lane);
        attention_item<true>(q, it, lane, 0, 0, in_wg ? &parts[wave] : nullptr);
    }
    if (!in_wg) return;
    __syncthreads();
    if (active && sp == 0) {
        // the head's splits are waves wave .. wave + nsplit - 1; lane l merges dims 2 l and 2 l + 1, in split order
        float M = kNegBig;
        for (int i = 0; i < nsplit; ++i) M = fmaxf(M, parts[wave + i].m);
        const int t2 = lane * 2;
        const bool dact = t2 < p.D;
        float L = 0.f, A0 = 0.f, A1 = 0.f;
        for (int i = 0; i < nsplit; ++i) {
            const float sc = fast_exp2(parts[wave + i].m - M);
            L += parts[wave + i].l * sc;
            A0 = fmadd(parts[wave + i].acc[dact ? t2 : 0], sc, A0);
            A1 = fmadd(parts[wave + i].acc[dact ? t2 + 1 : 0], sc, A1);
        }
        if (dact) {
            const half2_t o = {(half_t)(A0 / L), (half_t)(A1 / L)};
            *reinterpret_cast<half2_t*>(q.attn_vec + (size_t)head * p.D + t2) = o;
        }
    }
}


// What the library keeps per device, set up at the first call on that device.
struct DeviceInfo {
    int cus = 0;
    bool ok = false;
    int* host_status = nullptr;        // a line of pinned host memory: device-side failure flags land here as well, one word per flag
    int* host_status_dev = nullptr;    // the device's address of that line
    std::map<const void*, int> blocks_per_cu;   // occupancy of the one-launch kernels, by kernel
    void* static_scratch = nullptr;    // address of this device's copy of the file-scope scratch array
};
std::mutex g_device_mu;

// Scratch memory of cfpp_neox_layer_decode_static, the entry point that allocates nothing: one array per device,
// part of the library's code object, held by every device the library runs on until the process ends.  Host code
// must not use the array's name as an address (on the host it is a stand-in, not device memory): the address of
// a device's copy comes from hipGetSymbolAddress, once per device (static_scratch_address).
constexpr size_t kStaticScratchBytes = 1280u << 10;      // 1.25 MiB: a Pythia-6.9B layer needs 1.19 MiB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// set while an entry point that must not allocate runs on this thread: the per-device set-up then does not create the
// pinned status line (that entry point refuses to run without it, see cfpp_neox_layer_decode_static)
thread_local bool tl_no_alloc = false;

// The per-device record, set up under the lock on first use (compute units; the pinned status line unless the calling
// entry point must not allocate).  Every field is written under g_device_mu and never changes once set.
DeviceInfo& device_info() {
    static DeviceInfo info[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    DeviceInfo& d = info[dev];
    std::lock_guard<std::mutex> lock(g_device_mu);
    if (!d.ok) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            d.cus = prop.multiProcessorCount;
            d.ok = true;
        }
        (void)hipGetLastError();
    }
    if (d.ok && d.host_status == nullptr && !tl_no_alloc) {
        void* h = nullptr;
        if (hipHostMalloc(&h, 64, hipHostMallocMapped) == hipSuccess && h != nullptr) {
            std::memset(h, 0, 64);
            void* dp = nullptr;
            if (hipHostGetDevicePointer(&dp, h, 0) == hipSuccess && dp != nullptr) {
                d.host_status_dev = reinterpret_cast<int*>(dp);
                d.host_status = reinterpret_cast<int*>(h);
            } else {
                (void)hipHostFree(h);
            }
        }
        (void)hipGetLastError();
    }
    return d;
}

// The failure flags the kernels have stored in the pinned status line of a device (one word per flag), as a bit mask.
int host_status_flags(const DeviceInfo& di, bool clear) {
    if (!di.host_status) return 0;
    volatile int* w = reinterpret_cast<volatile int*>(di.host_status);
    const int flags = (w[0] ? kStatusSpin : 0) | (w[1] ? kStatusSeq : 0);
    if (clear) { w[0] = 0; w[1] = 0; }
    return flags;
}

// The address of the current device's copy of `scratch`, looked up on first use per device.
int static_scratch_address(void** out) {
    DeviceInfo& di = device_info();
    if (!di.ok) return (int)hipErrorNoDevice;
    std::lock_guard<std::mutex> lock(g_device_mu);
    if (di.static_scratch == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) & 255u)) return (int)hipErrorInvalidSymbol;
        di.static_scratch = ptr;
    }
    *out = di.static_scratch;
    return CFPP_OK;
}

// non-zero: some launch on this device has raised a failure flag since the word was last cleared
int pending_device_failure() { return host_status_flags(device_info(), false); }
#define CFPP_REFUSE_AFTER_FAILURE()                          \
    do {                                                     \
        if (pending_device_failure()) return CFPP_ERR_DEVICE; \
    } while (0)

constexpr size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#ifdef CFPP_TRACE
long long* g_trace = nullptr;   // see cfpp_debug_set_trace
#endif

struct WorkspaceLayout {
    size_t qkv_raw, attn_vec, inter, part_ml, part_acc, head_cnt, bar, grp, mbox, team, total;
};

WorkspaceLayout workspace_layout(const cfpp_neox_dims& d) {
    WorkspaceLayout w{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
    w.qkv_raw = take((size_t)3 * d.hidden * 4);
    w.attn_vec = take((size_t)d.hidden * 2);
    w.inter = take((size_t)d.ffn * 2);
    w.part_ml = take((size_t)d.heads * kMaxSplit * 2 * 4);
    w.part_acc = take((size_t)d.heads * kMaxSplit * d.head_dim * 4);
    w.head_cnt = take((size_t)d.heads * kHeadCntStride * 4);
    w.bar = take(64);
    w.grp = take((size_t)(kBarExit + 1) * kEventGroups * kMailboxInts * 4);
    w.mbox = take((size_t)kMaxGrid * kMailboxInts * 4);
    w.team = take((size_t)(1 + kUpPhases) * (kMaxGrid / kTeamWgs) * kMailboxInts * 4);
    w.total = off;
    return w;
}

int check_dims(const cfpp_neox_dims* d) {
    if (!d) return CFPP_ERR_NULL;
    if (d->hidden <= 0 || d->heads <= 0 || d->head_dim <= 0 || d->ffn <= 0) return CFPP_ERR_DIMS;
    if (d->hidden != d->heads * d->head_dim) return CFPP_ERR_DIMS;
    if (d->hidden % 8 || d->ffn % 8 || d->head_dim % 8) return CFPP_ERR_DIMS;
    if (d->head_dim > 128 || d->hidden > 8 * kChunk) return CFPP_ERR_DIMS;
    if (d->rotary_dim < 0 || d->rotary_dim > d->head_dim || (d->rotary_dim & 1)) return CFPP_ERR_DIMS;
    if (!(d->eps > 0.f)) return CFPP_ERR_DIMS;
    return CFPP_OK;
}

// launch geometry for one set of dims
struct Plan {
    int nch;        // 512-half chunks of the hidden row (stage-A and O-projection registers)
    int cpd;        // MLP-down chunks per streaming wave
};

int make_plan(const cfpp_neox_dims& d, Plan* out) {
    Plan p{};
    p.nch = (d.hidden + kChunk - 1) / kChunk;
    p.cpd = ((d.ffn + kChunk - 1) / kChunk + kStreamers - 1) / kStreamers;
    if (p.nch < 1 || p.nch > 8 || p.cpd < 1 || p.cpd > 8) return CFPP_ERR_DIMS;
    *out = p;
    return CFPP_OK;
}

#define CFPP_HIP(expr)                                   \
    do {                                                 \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess) return (int)e_;            \
    } while (0)

int launch_check() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? CFPP_OK : (int)e;
}

// Set by cfpp_stack_profile_step around a layer launch: the fused kernel is then launched with these events
// attached to its dispatch (kernel start / kernel end), which is the duration a profiler reports.
struct KernelEvents { hipEvent_t start, stop; };
thread_local KernelEvents* tl_kernel_events = nullptr;

// ---- template dispatch ---------------------------------------------------------------------------
template <int NCH>
int launch_stage_qkv_t(const LayerParams& p, int grid, hipStream_t st) {
    // eight waves per workgroup when every wave still gets three tiles (twice the loads in flight), else four
    constexpr int RPIA = StageARpi<NCH>::value;
    const bool wide = (3 * p.H + RPIA - 1) / RPIA >= 3 * grid * 2 * kStreamers;
    const bool ex = p.H == NCH * kChunk;
    if (wide) {
        if (ex) hipLaunchKernelGGL((k_stage_qkv<NCH, 2 * kStreamers, true>), dim3(grid), dim3(2 * kStreamers * 64), 0, st, p);
        else hipLaunchKernelGGL((k_stage_qkv<NCH, 2 * kStreamers, false>), dim3(grid), dim3(2 * kStreamers * 64), 0, st, p);
    } else {
        if (ex) hipLaunchKernelGGL((k_stage_qkv<NCH, kStreamers, true>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
        else hipLaunchKernelGGL((k_stage_qkv<NCH, kStreamers, false>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    }
    return launch_check();
}
template <int NCH>
int launch_stage_mid_t(const LayerParams& p, int grid, hipStream_t st) {
    if (p.H == NCH * kChunk) hipLaunchKernelGGL((k_stage_mid<NCH, true>), dim3(grid), dim3(2 * kStreamers * 64), 0, st, p);
    else hipLaunchKernelGGL((k_stage_mid<NCH, false>), dim3(grid), dim3(2 * kStreamers * 64), 0, st, p);
    return launch_check();
}
// stage C: eight waves when the O projection is part of it, four for the MLP-down rows alone
template <int NCH, int CPD>
int launch_stage_c_t(const LayerParams& p, int grid, hipStream_t st) {
    if (p.c_use_o) hipLaunchKernelGGL((k_stage_c8<NCH, CPD>), dim3(grid), dim3(2 * kStreamers * 64), 0, st, p);
    else hipLaunchKernelGGL((k_stage_c<NCH, CPD>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    return launch_check();
}
// The one-launch kernels wait for each other's workgroups inside the launch, so every workgroup of the grid has to
// be resident at the same time.  What the library can establish itself is that the device has room for the grid
// when nothing else runs on it: the kernel's occupancy (workgroups per compute unit for its registers and LDS) times
// the compute units.  A grid that does not fit is not launched in one piece; the caller takes the per-stage launches
// instead.  What it cannot see is other work: kernels of other streams or processes that hold compute units while a
// one-launch kernel starts can keep some of its workgroups waiting; the bounded waits then expire, the failure flag
// is raised and the next call on the device reports CFPP_ERR_DEVICE.
bool one_launch_fits(const void* fn, int block_threads, int grid) {
    DeviceInfo& di = device_info();     // (takes and releases the lock itself)
    int per_cu = 0;
    {
        std::lock_guard<std::mutex> lock(g_device_mu);
        auto it = di.blocks_per_cu.find(fn);
        if (it != di.blocks_per_cu.end()) per_cu = it->second;
        else {
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, block_threads, 0) != hipSuccess) {
                (void)hipGetLastError();
                per_cu = 0;
            }
            di.blocks_per_cu[fn] = per_cu;
        }
    }
    return cfpp_one_launch_fits(grid, di.cus, per_cu) != 0;
}

// BYX (attention items dealt out per chiplet): heads that are not whole 128-byte lines, in a number and on a grid that
// divide by the chiplets
template <int NCH, int CPD>
const void* fused_fn(const LayerParams& p, int grid) {
    const bool byx = (p.D * 2) % 128 != 0 && p.heads % kXcds == 0 && grid % kXcds == 0;
    if (p.H == NCH * kChunk) return byx ? (const void*)(k_fused<NCH, CPD, true, true>) : (const void*)(k_fused<NCH, CPD, true, false>);
    return byx ? (const void*)(k_fused<NCH, CPD, false, true>) : (const void*)(k_fused<NCH, CPD, false, false>);
}
template <int NCH, int CPD>
int launch_fused_t(const LayerParams& p, int grid, hipStream_t st) {
    const void* fn = fused_fn<NCH, CPD>(p, grid);
    LayerParams pp = p;
    void* args[] = {&pp};
    if (tl_kernel_events) {
        // profiling: the events are attached to the dispatch itself and stamp the start and the end of the kernel
        CFPP_HIP(hipExtLaunchKernel(fn, dim3(grid), dim3(2 * kStreamers * 64), args, 0, st, tl_kernel_events->start,
                                    tl_kernel_events->stop, 0));
        return CFPP_OK;
    }
    CFPP_HIP(hipLaunchKernel(fn, dim3(grid), dim3(2 * kStreamers * 64), args, 0, st));
    return CFPP_OK;
}
template <int NCH, int CPD>
bool fused_fits_t(const LayerParams& p, int grid) { return one_launch_fits(fused_fn<NCH, CPD>(p, grid), 2 * kStreamers * 64, grid); }
// the same choice for the launch that runs all layers of a model
template <int NCH, int CPD>
const void* fused_stack_fn(const LayerParams& p, int grid) {
    const bool byx = (p.D * 2) % 128 != 0 && p.heads % kXcds == 0 && grid % kXcds == 0;
    // only for hidden sizes that fill their last 512-column chunk (the other instantiations do not fit the register file
    // without spilling; such models take one launch per layer)
    if (p.H != NCH * kChunk) return nullptr;
    return byx ? (const void*)(k_fused_stack<NCH, CPD, true, true>) : (const void*)(k_fused_stack<NCH, CPD, true, false>);
}
template <int NCH, int CPD>
int launch_fused_stack_t(const LayerParams& p0, const LayerParams* table, int n_layers, int grid, hipStream_t st) {
    const void* fn = fused_stack_fn<NCH, CPD>(p0, grid);
    if (fn == nullptr) return CFPP_ERR_DIMS;
    void* args[] = {&table, &n_layers};
    if (tl_kernel_events) {
        CFPP_HIP(hipExtLaunchKernel(fn, dim3(grid), dim3(2 * kStreamers * 64), args, 0, st, tl_kernel_events->start,
                                    tl_kernel_events->stop, 0));
        return CFPP_OK;
    }
    CFPP_HIP(hipLaunchKernel(fn, dim3(grid), dim3(2 * kStreamers * 64), args, 0, st));
    return CFPP_OK;
}
template <int NCH, int CPD>
bool fused_stack_fits_t(const LayerParams& p, int grid) {
    const void* fn = fused_stack_fn<NCH, CPD>(p, grid);
    return fn != nullptr && one_launch_fits(fn, 2 * kStreamers * 64, grid);
}

// hidden chunks that occur in CFPP_SHAPE_CASES below (both lists can be narrowed on the compiler's command line for a
// quick experimental build; the shapes left out are then refused with CFPP_ERR_DIMS)
#ifndef CFPP_NCH_CASES
#define CFPP_NCH_CASES(X) X(1) X(2) X(4) X(5) X(8)
#endif
// (hidden chunks, MLP-down chunks per streaming wave).  The Pythia family has ffn = 4 hidden, so both
// numbers coincide: 512 -> (1,1), 768/1024 -> (2,2), 2048 -> (4,4), 2560 -> (5,5), 4096 -> (8,8);
// (8,6) is hidden 4096 with ffn 11008
#ifndef CFPP_SHAPE_CASES
#define CFPP_SHAPE_CASES(X) X(1, 1) X(2, 2) X(4, 4) X(5, 5) X(8, 8) X(8, 6)
#endif

int launch_stage_qkv(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
    switch (pl.nch) {
#define X(n) case n: return launch_stage_qkv_t<n>(p, grid, st);
        CFPP_NCH_CASES(X)
#undef X
    }
    return CFPP_ERR_DIMS;
}
int launch_stage_mid(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
    switch (pl.nch) {
#define X(n) case n: return launch_stage_mid_t<n>(p, grid, st);
        CFPP_NCH_CASES(X)
#undef X
    }
    return CFPP_ERR_DIMS;
}
int launch_stage_c(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return launch_stage_c_t<a, b>(p, grid, st);
    CFPP_SHAPE_CASES(X)
#undef X
    return CFPP_ERR_DIMS;
}
int launch_fused(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return launch_fused_t<a, b>(p, grid, st);
    CFPP_SHAPE_CASES(X)
#undef X
    return CFPP_ERR_DIMS;
}
bool fused_fits(const Plan& pl, const LayerParams& p, int grid) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return fused_fits_t<a, b>(p, grid);
    CFPP_SHAPE_CASES(X)
#undef X
    return false;
}
// `p0` is the first entry of `table` (device memory), on the host
int launch_fused_stack(const Plan& pl, const LayerParams& p0, const LayerParams* table, int n_layers, int grid, hipStream_t st) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return launch_fused_stack_t<a, b>(p0, table, n_layers, grid, st);
    CFPP_SHAPE_CASES(X)
#undef X
    return CFPP_ERR_DIMS;
}
bool fused_stack_fits(const Plan& pl, const LayerParams& p, int grid) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return fused_stack_fits_t<a, b>(p, grid);
    CFPP_SHAPE_CASES(X)
#undef X
    return false;
}
template <int NCH>
int launch_gated_up_t(const LayerParams& p, int grid, hipStream_t st) {
    if (p.H == NCH * kChunk) hipLaunchKernelGGL((k_gated_up<NCH, true>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    else hipLaunchKernelGGL((k_gated_up<NCH, false>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    return launch_check();
}
int launch_gated_up(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
#define X(a) if (pl.nch == a) return launch_gated_up_t<a>(p, grid, st);
    CFPP_NCH_CASES(X)
#undef X
    return CFPP_ERR_DIMS;
}

template <int NCH, int CPD>
int launch_gated_mlp_t(const LayerParams& p, int grid, hipStream_t st) {
    if (p.H == NCH * kChunk) hipLaunchKernelGGL((k_gated_mlp<NCH, CPD, true>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    else hipLaunchKernelGGL((k_gated_mlp<NCH, CPD, false>), dim3(grid), dim3(kStreamers * 64), 0, st, p);
    return launch_check();
}
int launch_gated_mlp(const Plan& pl, const LayerParams& p, int grid, hipStream_t st) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return launch_gated_mlp_t<a, b>(p, grid, st);
    CFPP_SHAPE_CASES(X)
#undef X
    return CFPP_ERR_DIMS;
}
bool gated_mlp_fits(const Plan& pl, const LayerParams& p, int grid) {
#define X(a, b)                                                                                                        \
    if (pl.nch == a && pl.cpd == b)                                                                                    \
        return one_launch_fits(p.H == a * kChunk ? (const void*)(k_gated_mlp<a, b, true>) : (const void*)(k_gated_mlp<a, b, false>), \
                               kStreamers * 64, grid);
    CFPP_SHAPE_CASES(X)
#undef X
    return false;
}

bool shape_supported(const Plan& pl) {
#define X(a, b) if (pl.nch == a && pl.cpd == b) return true;
    CFPP_SHAPE_CASES(X)
#undef X
    return false;
}

// upper bound of the KV splits per head the kernels will use for a sequence length (device code
// computes the same value from the actual length: effective_split)
// workgroups of a streaming launch: one per compute unit
int streaming_grid() {
    DeviceInfo& di = device_info();
    return di.cus > 0 ? di.cus : 256;
}

// workgroups of the fused launch: one per compute unit, all co-resident
int fused_grid() {
    DeviceInfo& di = device_info();
    const int grid = di.cus > 0 ? di.cus : 256;
    return grid > kMaxGrid ? kMaxGrid : grid;
}

int split_bound(int seq_hint, int max_split) {
    int n = (seq_hint + kSplitRows - 1) / kSplitRows;
    n = n < 1 ? 1 : n;
    return n < max_split ? n : max_split;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// KV splits per head at most: `item_waves` attention waves per workgroup of the fused launch get an item
int split_cap(int heads, int item_waves) {
    int ms = kMaxSplit - 1;               // + the new token's item
    const int per_head = fused_grid() * item_waves / (heads > 0 ? heads : 1);
    if (ms > per_head - 1) ms = per_head < 2 ? 1 : per_head - 1;     // one of a head's item slots is the new token's
    return ms;
}
int fill_params(const cfpp_neox_dims* d, const cfpp_neox_weights* w, const cfpp_neox_io* io, void* workspace,
                size_t ws_bytes, bool need_down, bool need_out, LayerParams* out, Plan* plan) {
    int rc = check_dims(d);
    if (rc) return rc;
    if (!w || !io || !workspace) return CFPP_ERR_NULL;
    const void* req[] = {w->ln_w, w->ln_b, w->w_qkv, w->b_qkv, w->w_o, w->b_o, w->post_ln_w, w->post_ln_b,
                         w->w_up, w->b_up, io->input, io->k_new, io->v_new, io->k_cache, io->v_cache, io->cos, io->sin};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    if (need_down && (!w->w_down || !w->b_down)) return CFPP_ERR_NULL;
    if (need_out && !io->output) return CFPP_ERR_NULL;
    if (!need_out && (!io->attn_output || !io->mlp_intermediate)) return CFPP_ERR_NULL;
    if (io->cache_rows < 0 || io->rope_stride < 0) return CFPP_ERR_SEQ;
    // a length the host knows is checked here; one in device memory is checked by the kernels (load_seq_len)
    if (!io->d_seq_len && (io->seq_len < 0 || io->seq_len > io->cache_rows)) return CFPP_ERR_SEQ;
    if (!io->d_seq_len && io->rope_stride > 0 && io->seq_len >= io->cache_rows) return CFPP_ERR_SEQ;
    if (io->d_seq_len && io->cache_rows < 1) return CFPP_ERR_SEQ;
    const WorkspaceLayout L = workspace_layout(*d);
    if (ws_bytes < L.total || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CFPP_ERR_WORKSPACE;
    rc = make_plan(*d, plan);
    if (rc) return rc;
    if (!shape_supported(*plan)) return CFPP_ERR_DIMS;

    LayerParams p{};
    p.H = d->hidden; p.heads = d->heads; p.D = d->head_dim; p.rot = d->rotary_dim; p.F = d->ffn;
    p.eps = d->eps;
    p.qscale = (float)(1.4426950408889634 / std::sqrt((double)d->head_dim));
    auto h = [](const void* q) { return reinterpret_cast<const half_t*>(q); };
    auto hm = [](void* q) { return reinterpret_cast<half_t*>(q); };
    p.ln_w = h(w->ln_w); p.ln_b = h(w->ln_b); p.w_qkv = h(w->w_qkv); p.b_qkv = h(w->b_qkv);
    p.w_o = h(w->w_o); p.b_o = h(w->b_o); p.ln2_w = h(w->post_ln_w); p.ln2_b = h(w->post_ln_b);
    p.w_up = h(w->w_up); p.b_up = h(w->b_up); p.w_down = h(w->w_down); p.b_down = h(w->b_down);
    p.x = h(io->input); p.out = hm(io->output);
    p.k_new = hm(io->k_new); p.v_new = hm(io->v_new); p.k_cache = hm(io->k_cache); p.v_cache = hm(io->v_cache);
    p.cache_rows = io->cache_rows;
    p.cos = io->cos; p.sin = io->sin; p.rope_stride = io->rope_stride;
    p.seq_len = io->seq_len; p.d_seq_len = io->d_seq_len;
    p.seq_cap = (io->d_seq_len && io->max_seq_len > 0) ? io->max_seq_len : io->cache_rows;
    // one (head, split) item per attention wave of the fused launch at most: an item more than that would
    // start only after some wave has finished its first one, and end the attention phase late
    // ... and one attention wave per workgroup is better left without an item when the layer has MLP rows: it then
    // carries the MLP-up arrivals of its workgroup (arrival_agents), which gains more than the finer KV split
    // (6.9B at context 2048: TPOT 2.42 instead of 2.49 ms)
    p.arrival_agents = 1;
    p.max_split = split_cap(d->heads, kStreamers - 1);
    p.norm_rms = 0; p.qkv_head_stride = 3 * d->head_dim; p.qkv_k_off = d->head_dim; p.qkv_v_off = 2 * d->head_dim;
    p.append_kv = 1; p.x_add = nullptr; p.x_sum_out = nullptr; p.c_add_sum = 0;
    char* ws = reinterpret_cast<char*>(workspace);
    p.qkv_raw = reinterpret_cast<float*>(ws + L.qkv_raw);
    p.attn_vec = reinterpret_cast<half_t*>(ws + L.attn_vec);
    p.inter = reinterpret_cast<half_t*>(ws + L.inter);
    p.part_ml = reinterpret_cast<float*>(ws + L.part_ml);
    p.part_acc = reinterpret_cast<float*>(ws + L.part_acc);
    p.head_cnt = reinterpret_cast<int*>(ws + L.head_cnt);
    p.bar = reinterpret_cast<int*>(ws + L.bar);
    p.grp = reinterpret_cast<int*>(ws + L.grp);
    p.mbox = reinterpret_cast<int*>(ws + L.mbox);
    p.team = reinterpret_cast<int*>(ws + L.team);
    p.c_base0 = p.x; p.c_base1 = nullptr; p.c_use_o = 1; p.c_use_down = 1;
    p.host_status = device_info().host_status_dev;
#ifdef CFPP_TRACE
    p.trace = g_trace;
#endif
    *out = p;
    return CFPP_OK;
}

int seq_hint_of(const cfpp_neox_io* io) {
    return io->d_seq_len ? (io->max_seq_len > 0 ? io->max_seq_len : io->cache_rows) : io->seq_len;
}

int grid_for_streaming(const Plan&) { return streaming_grid(); }

int run_split(const Plan& pl, LayerParams& p, int seq_hint, hipStream_t st);
// One layer in the requested mode.  The one-launch kernel is used only when the device can hold its whole grid and
// every attention wave gets at most one (head, split) item; otherwise the per-stage launches compute the same result.
int run_layer(const Plan& pl, LayerParams& p, int mode, int seq_hint, hipStream_t st) {
    if (mode == CFPP_MODE_SPLIT) return run_split(pl, p, seq_hint, st);
    const int grid = fused_grid();
    // every attention wave of the one-launch kernel takes at most one item
    if ((long long)p.heads * (p.max_split + 1) > (long long)grid * kStreamers || !fused_fits(pl, p, grid))
        return run_split(pl, p, seq_hint, st);
    return launch_fused(pl, p, grid, st);
}

int run_split(const Plan& pl, LayerParams& p, int seq_hint, hipStream_t st) {
    const int grid = grid_for_streaming(pl);
    int rc = launch_stage_qkv(pl, p, grid, st);
    if (rc) return rc;
    // one attention wave per (head, split) item
    const int bgrid = (p.heads * (split_bound(seq_hint, p.max_split) + 1) + kStreamers - 1) / kStreamers;
    if (p.F > 0) {
        // attention items beside the MLP-up rows: the rows on one workgroup per compute unit, more workgroups (items
        // only) when there are more items than that gives attention waves
        p.up_wgs = grid;
        if ((rc = launch_stage_mid(pl, p, bgrid > grid ? bgrid : grid, st))) return rc;
    } else {
        // no MLP in this layer: the attention items alone
        hipLaunchKernelGGL(k_stage_b, dim3(bgrid), dim3(kStreamers * 64), 0, st, p);
        if ((rc = launch_check())) return rc;
    }
    return launch_stage_c(pl, p, grid, st);
}

}  // namespace

// =================================================================================================
// C ABI
// =================================================================================================
// ---- launchers of the batched LLaMA attention block ---------------------------------------------------
namespace {
struct BatchLayout { size_t qkv_raw, x_norm, attn_vec, k_new, v_new, part_ml, part_acc, head_cnt, bar, total; };
BatchLayout batch_layout(const cfpp_neox_dims& d, int batch) {
    BatchLayout w{};
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t at = off; off += align_up(bytes, 256); return at; };
    const size_t B = (size_t)batch, H = (size_t)d.hidden;
    w.qkv_raw = take(B * 3 * H * 4);
    w.x_norm = take(B * H * 2);
    w.attn_vec = take(B * H * 2);
    w.k_new = take(B * H * 2);
    w.v_new = take(B * H * 2);
    w.part_ml = take(B * d.heads * kMaxSplit * 2 * 4);
    w.part_acc = take(B * d.heads * kMaxSplit * (size_t)d.head_dim * 4);
    w.head_cnt = take(B * d.heads * kHeadCntStride * 4);
    w.bar = take(64 * 4);
    w.total = off;
    return w;
}
template <int NCH>
int launch_batch_gemv_t(const BatchGemv& a, int grid, hipStream_t st) {
    if (a.K == NCH * kChunk) hipLaunchKernelGGL((k_batch_gemv<NCH, true>), dim3(grid), dim3(kStreamers * 64), 0, st, a);
    else hipLaunchKernelGGL((k_batch_gemv<NCH, false>), dim3(grid), dim3(kStreamers * 64), 0, st, a);
    return (int)hipGetLastError();
}
int launch_batch_mfma(const BatchMfma& a, hipStream_t st) {
    const int grid = a.R / 16;
    if (a.K == 4096 || a.K == 2048) {
        const int wgs = streaming_grid() < grid ? streaming_grid() : grid;
        const bool one = a.batch <= 16;
        if (a.K == 4096) {
            if (one) hipLaunchKernelGGL((k_batch_mfma_pipe<8, true>), dim3(wgs), dim3(512), 0, st, a);
            else hipLaunchKernelGGL((k_batch_mfma_pipe<8, false>), dim3(wgs), dim3(512), 0, st, a);
        } else {
            if (one) hipLaunchKernelGGL((k_batch_mfma_pipe<4, true>), dim3(wgs), dim3(256), 0, st, a);
            else hipLaunchKernelGGL((k_batch_mfma_pipe<4, false>), dim3(wgs), dim3(256), 0, st, a);
        }
        return (int)hipGetLastError();
    }
    if (a.K != 1024) return CFPP_ERR_DIMS;
    hipLaunchKernelGGL((k_batch_mfma<4>), dim3(grid), dim3(512), 0, st, a);
    return (int)hipGetLastError();
}
// the kernel that takes the norm of the rows upon itself: the pipelined one, with its input rows kept in registers
bool batch_mfma_norm_inside(int k, int batch) { return (k == 4096 || k == 2048) && batch <= 16; }
bool batch_mfma_supported(int rows, int k) { return rows % 16 == 0 && k % 256 == 0 && (k == 1024 || k == 2048 || k == 4096); }
int launch_batch_norm(int nch, const BatchNorm& a, hipStream_t st) {
    const dim3 grid((a.batch + kStreamers - 1) / kStreamers), block(kStreamers * 64);
    switch (nch) {
        case 1: hipLaunchKernelGGL((k_batch_norm<1>), grid, block, 0, st, a); break;
        case 2: hipLaunchKernelGGL((k_batch_norm<2>), grid, block, 0, st, a); break;
        case 4: hipLaunchKernelGGL((k_batch_norm<4>), grid, block, 0, st, a); break;
        case 5: hipLaunchKernelGGL((k_batch_norm<5>), grid, block, 0, st, a); break;
        case 8: hipLaunchKernelGGL((k_batch_norm<8>), grid, block, 0, st, a); break;
        default: return CFPP_ERR_DIMS;
    }
    return (int)hipGetLastError();
}
int launch_batch_gemv(int nch, const BatchGemv& a, int grid, hipStream_t st) {
    switch (nch) {
        case 1: return launch_batch_gemv_t<1>(a, grid, st);
        case 2: return launch_batch_gemv_t<2>(a, grid, st);
        case 4: return launch_batch_gemv_t<4>(a, grid, st);
        case 5: return launch_batch_gemv_t<5>(a, grid, st);
        case 8: return launch_batch_gemv_t<8>(a, grid, st);
        default: return CFPP_ERR_DIMS;
    }
}
}  // namespace


extern "C" {

const char* cfpp_version(void) { return "cfpp 0.1 (gfx950)"; }

const char* cfpp_status_str(int s) {
    switch (s) {
        case CFPP_OK: return "ok";
        case CFPP_ERR_NULL: return "a required pointer is NULL";
        case CFPP_ERR_DIMS: return "unsupported layer dimensions";
        case CFPP_ERR_SEQ: return "seq_len out of range for the KV cache";
        case CFPP_ERR_WORKSPACE: return "workspace too small or not 256-byte aligned";
        case CFPP_ERR_CONTEXT: return "unknown context id or pointers differ from context creation";
        case CFPP_ERR_MODE: return "unknown mode";
        case CFPP_ERR_DEVICE: return "device-side failure flag raised";
        case CFPP_ERR_ALIGN: return "tensor pointer is not 16-byte aligned";
        case CFPP_ERR_ALIAS: return "an output overlaps an input";
        case CFPP_ERR_STATIC_SCRATCH: return "the layer needs more scratch than the static array of the allocation-free entry point holds";
        case CFPP_ERR_NOT_INITIALISED: return "cfpp_init() has not run on this device (the allocation-free entry point cannot create the failure-flag word itself)";
        default: break;
    }
    if (s > 0) return hipGetErrorString((hipError_t)s);
    return "unknown status";
}

size_t cfpp_neox_workspace_bytes(const cfpp_neox_dims* dims) {
    if (check_dims(dims)) return 0;
    return workspace_layout(*dims).total;
}

int cfpp_neox_layer_decode(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io, int mode,
                           void* workspace, size_t workspace_bytes, void* stream) {
    if (mode != CFPP_MODE_FUSED && mode != CFPP_MODE_SPLIT) return CFPP_ERR_MODE;
    LayerParams p;
    Plan pl;
    int rc = fill_params(dims, w, io, workspace, workspace_bytes, true, true, &p, &pl);
    if (rc) return rc;
    CFPP_REFUSE_AFTER_FAILURE();
    return run_layer(pl, p, mode, seq_hint_of(io), reinterpret_cast<hipStream_t>(stream));
}

int cfpp_init(void) {
    DeviceInfo& di = device_info();          // compute units, pinned status word
    if (!di.ok) return (int)hipErrorNoDevice;
    void* ptr = nullptr;
    return static_scratch_address(&ptr);     // this device's copy of the static scratch array
}

size_t cfpp_static_scratch_bytes(void) { return kStaticScratchBytes; }

int cfpp_neox_layer_decode_static(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io, int mode,
                                  void* stream) {
    if (mode != CFPP_MODE_FUSED && mode != CFPP_MODE_SPLIT) return CFPP_ERR_MODE;
    int rc = check_dims(dims);
    if (rc) return rc;
    const WorkspaceLayout L = workspace_layout(*dims);
    if (L.total > kStaticScratchBytes) return CFPP_ERR_STATIC_SCRATCH;
    struct NoAlloc { NoAlloc() { tl_no_alloc = true; } ~NoAlloc() { tl_no_alloc = false; } } guard;
    {
        // A failure inside the kernels (an expired wait, a device-side length out of range) is reported through the
        // pinned status line of the device.  This call may not create it (it allocates nothing), and the status word
        // inside the scratch array is cleared by the next call: without the line a failure would be lost, so the
        // call insists on cfpp_init() (or any other launching entry point) having run on this device before.
        const DeviceInfo& di = device_info();
        if (!di.ok) return (int)hipErrorNoDevice;
        if (di.host_status == nullptr) return CFPP_ERR_NOT_INITIALISED;
    }
    void* ws = nullptr;
    if ((rc = static_scratch_address(&ws))) return rc;
    LayerParams p;
    Plan pl;
    if ((rc = fill_params(dims, w, io, ws, kStaticScratchBytes, true, true, &p, &pl))) return rc;
    CFPP_REFUSE_AFTER_FAILURE();
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // The array keeps what the last call left there, possibly under another geometry's layout: the words that must
    // start at zero (arrival counters, event counters, mailboxes, ticket counters, launch generation) are cleared by
    // a small kernel in front of the layer (not a memset node: the call may be recorded into a graph).
    const size_t words = (L.total - L.head_cnt) / 4;
    hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(ws) + L.head_cnt), words);
    if ((rc = launch_check())) return rc;
    return run_layer(pl, p, mode, seq_hint_of(io), st);
}

int cfpp_neox_attention_mlp_up(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io,
                               void* workspace, size_t workspace_bytes, void* stream) {
    LayerParams p;
    Plan pl;
    int rc = fill_params(dims, w, io, workspace, workspace_bytes, false, false, &p, &pl);
    if (rc) return rc;
    if (!aligned16(io->attn_output) || !aligned16(io->mlp_intermediate)) return CFPP_ERR_ALIGN;
    CFPP_REFUSE_AFTER_FAILURE();
    p.inter = reinterpret_cast<half_t*>(io->mlp_intermediate);   // MLP-up writes the caller's tensor directly
    p.out = reinterpret_cast<half_t*>(io->attn_output);          // stage C: W_o attn + b_o only
    p.c_base0 = nullptr; p.c_base1 = nullptr; p.c_use_o = 1; p.c_use_down = 0;
    return run_split(pl, p, seq_hint_of(io), reinterpret_cast<hipStream_t>(stream));
}

// LLaMA attention block: the NeoX kernels with RMSNorm, stacked [q;k;v] rows, whole-head RoPE, no biases, no cache
// write, no MLP.
static cfpp_neox_dims llama_dims(int32_t hidden, int32_t heads, int32_t head_dim, float eps) {
    // ffn only sizes the (unused) MLP scratch and picks an existing kernel instantiation
    return cfpp_neox_dims{hidden, heads, head_dim, head_dim, 4 * hidden, eps};
}
size_t cfpp_llama_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim) {
    const cfpp_neox_dims d = llama_dims(hidden, heads, head_dim, 1e-6f);
    return cfpp_neox_workspace_bytes(&d);
}
int cfpp_llama_attention_decode(const cfpp_llama_attn* a, void* workspace, size_t workspace_bytes, void* stream) {
    if (!a || !workspace) return CFPP_ERR_NULL;
    const cfpp_neox_dims d = llama_dims(a->hidden, a->heads, a->head_dim, a->eps);
    int rc = check_dims(&d);
    if (rc) return rc;
    const void* req[] = {a->rms_w, a->w_qkv, a->w_o, a->input, a->output, a->k_new, a->v_new, a->k_cache, a->v_cache, a->cos, a->sin};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    if (a->residual && !aligned16(a->residual)) return CFPP_ERR_ALIGN;
    if (a->seq_len < 0) return CFPP_ERR_SEQ;
    if (a->mode != CFPP_MODE_FUSED && a->mode != CFPP_MODE_SPLIT) return CFPP_ERR_MODE;
    const WorkspaceLayout L = workspace_layout(d);
    if (workspace_bytes < L.total || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CFPP_ERR_WORKSPACE;
    Plan pl;
    if ((rc = make_plan(d, &pl))) return rc;
    if (!shape_supported(pl)) return CFPP_ERR_DIMS;
    CFPP_REFUSE_AFTER_FAILURE();

    // start from the NeoX parameter block of the same geometry, then switch the family-specific parts
    cfpp_neox_weights w{};
    w.ln_w = a->rms_w; w.ln_b = a->rms_w; w.w_qkv = a->w_qkv; w.b_qkv = a->rms_w; w.w_o = a->w_o; w.b_o = a->rms_w;
    w.post_ln_w = a->rms_w; w.post_ln_b = a->rms_w; w.w_up = a->w_qkv; w.b_up = a->rms_w; w.w_down = a->w_qkv; w.b_down = a->rms_w;
    cfpp_neox_io io{};
    io.input = a->input; io.output = a->output; io.k_new = a->k_new; io.v_new = a->v_new;
    io.k_cache = const_cast<void*>(a->k_cache); io.v_cache = const_cast<void*>(a->v_cache);
    io.cache_rows = a->seq_len; io.cos = a->cos; io.sin = a->sin; io.rope_stride = 0; io.seq_len = a->seq_len;
    LayerParams p;
    if ((rc = fill_params(&d, &w, &io, workspace, workspace_bytes, true, true, &p, &pl))) return rc;
    p.F = 0;                                     // no MLP rows in stage A
    p.arrival_agents = 0;
    p.max_split = split_cap(d.heads, kStreamers);    // ... so no attention wave is kept free for MLP-up arrivals
    p.ln_b = nullptr; p.ln2_w = nullptr; p.ln2_b = nullptr; p.b_qkv = nullptr; p.b_o = nullptr;
    p.w_up = nullptr; p.b_up = nullptr; p.w_down = nullptr; p.b_down = nullptr;
    p.norm_rms = 1;
    p.qkv_head_stride = d.head_dim; p.qkv_k_off = d.hidden; p.qkv_v_off = 2 * d.hidden;
    p.append_kv = 0;
    p.rope_half_table = 1;                       // cos / sin hold the D/2 pair angles
    p.x_add = reinterpret_cast<const half_t*>(a->residual);
    p.x_sum_out = reinterpret_cast<half_t*>(a->residual);
    p.c_base0 = nullptr; p.c_base1 = nullptr; p.c_use_o = 1; p.c_use_down = 0;
    p.c_add_sum = a->add_residual ? 1 : 0;
    // one launch (the attention waves fetch their K/V tiles while the streaming waves do the QKV rows) or one per stage
    return run_layer(pl, p, a->mode, a->seq_len, reinterpret_cast<hipStream_t>(stream));
}

// The reference's plain llama_decoder_layer op: as cfpp_llama_attention_decode without a residual, with weights stored
// [in, out] and GPT-J pairing of the rotary dims.  Three launches: QKV products (with the norm of the input row), attention items, O products.
size_t cfpp_llama_plain_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim) {
    const size_t base = cfpp_llama_workspace_bytes(hidden, heads, head_dim);
    if (base == 0) return 0;
    const int grid = streaming_grid();
    const int ppm = (hidden + kChunk - 1) / kChunk;
    const size_t units = (size_t)(3 * ppm > grid ? 3 * ppm : grid) + 3 * ppm;     // (panels x slices) never exceeds this
    return base + align_up(units * kChunk * 4, 256) + align_up((size_t)3 * ppm * 4, 256);
}
int cfpp_llama_attention_plain(const cfpp_llama_attn* a, void* workspace, size_t workspace_bytes, void* stream) {
    if (!a || !workspace) return CFPP_ERR_NULL;
    const cfpp_neox_dims d = llama_dims(a->hidden, a->heads, a->head_dim, a->eps);
    int rc = check_dims(&d);
    if (rc) return rc;
    const void* req[] = {a->rms_w, a->w_qkv, a->w_o, a->input, a->output, a->k_new, a->v_new, a->k_cache, a->v_cache, a->cos, a->sin};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    if (a->residual != nullptr || a->add_residual || a->mode != CFPP_MODE_FUSED) return CFPP_ERR_MODE;      // no residual stream, one variant
    if (a->seq_len < 0) return CFPP_ERR_SEQ;
    const size_t need = cfpp_llama_plain_workspace_bytes(a->hidden, a->heads, a->head_dim);
    if (need == 0) return CFPP_ERR_DIMS;
    if (workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CFPP_ERR_WORKSPACE;
    const WorkspaceLayout L = workspace_layout(d);
    Plan pl;
    if ((rc = make_plan(d, &pl))) return rc;
    if (!shape_supported(pl)) return CFPP_ERR_DIMS;
    char* ws = reinterpret_cast<char*>(workspace);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int grid = streaming_grid();
    const int H = d.hidden, ppm = (H + kChunk - 1) / kChunk;
    const size_t units = (size_t)(3 * ppm > grid ? 3 * ppm : grid) + 3 * ppm;
    float* part = reinterpret_cast<float*>(ws + L.total);
    int* cnt = reinterpret_cast<int*>(ws + L.total + align_up(units * kChunk * 4, 256));
    auto h = [](const void* q) { return reinterpret_cast<const half_t*>(q); };
    CFPP_REFUSE_AFTER_FAILURE();

    cfpp_neox_weights w{};
    w.ln_w = a->rms_w; w.ln_b = a->rms_w; w.w_qkv = a->w_qkv; w.b_qkv = a->rms_w; w.w_o = a->w_o; w.b_o = a->rms_w;
    w.post_ln_w = a->rms_w; w.post_ln_b = a->rms_w; w.w_up = a->w_qkv; w.b_up = a->rms_w; w.w_down = a->w_qkv; w.b_down = a->rms_w;
    cfpp_neox_io io{};
    io.input = a->input; io.output = a->output; io.k_new = a->k_new; io.v_new = a->v_new;
    io.k_cache = const_cast<void*>(a->k_cache); io.v_cache = const_cast<void*>(a->v_cache);
    io.cache_rows = a->seq_len; io.cos = a->cos; io.sin = a->sin; io.rope_stride = 0; io.seq_len = a->seq_len;
    LayerParams p;
    if ((rc = fill_params(&d, &w, &io, workspace, workspace_bytes, true, true, &p, &pl))) return rc;
    p.F = 0;
    p.arrival_agents = 0;
    p.max_split = split_cap(d.heads, kStreamers);
    p.qkv_head_stride = d.head_dim; p.qkv_k_off = H; p.qkv_v_off = 2 * H;
    p.append_kv = 0;

    auto gemv = [&](const half_t* W, int nsec, const half_t* x, const half_t* norm_w, float* out_f32, half_t* out_f16) {
        GemvT g{};
        g.W = W; g.K = H; g.O = H; g.nsec = nsec; g.x = x; g.norm_w = norm_w; g.eps = a->eps; g.part = part; g.cnt = cnt;
        g.out_f32 = out_f32; g.out_f16 = out_f16;
        const int panels = nsec * ppm;
        g.slices = grid / panels < 1 ? 1 : (grid / panels > 64 ? 64 : grid / panels);
        hipLaunchKernelGGL(k_gemv_t, dim3(panels * g.slices), dim3(kStreamers * 64), 0, st, g);
        return (int)hipGetLastError();
    };
    // the QKV launch normalises the input row on its way in (a separate norm launch was measured slower)
    if ((rc = gemv(h(a->w_qkv), 3, h(a->input), h(a->rms_w), p.qkv_raw, nullptr))) return rc;
    const int bgrid = (p.heads * (split_bound(a->seq_len, p.max_split) + 1) + kStreamers - 1) / kStreamers;
    hipLaunchKernelGGL(k_stage_b_pairs, dim3(bgrid), dim3(kStreamers * 64), 0, st, p);
    if ((rc = (int)hipGetLastError())) return rc;
    return gemv(h(a->w_o), 1, p.attn_vec, nullptr, nullptr, reinterpret_cast<half_t*>(a->output));
}

size_t cfpp_llama_mlp_workspace_bytes(int32_t hidden, int32_t ffn) {
    if (hidden <= 0 || ffn <= 0 || hidden % 8 || ffn % 8 || hidden > 8 * kChunk) return 0;
    // intermediate row, then the words of the one-launch variant: flags / counters, group counters, mailboxes
    return align_up((size_t)ffn * 2, 256) + 256 + align_up((size_t)(kBarExit + 1) * kEventGroups * kMailboxInts * 4, 256) +
           (size_t)kMaxGrid * kMailboxInts * 4;
}
int cfpp_llama_mlp(const cfpp_llama_mlp_args* m, void* workspace, size_t workspace_bytes, void* stream) {
    if (!m || !workspace) return CFPP_ERR_NULL;
    const size_t need = cfpp_llama_mlp_workspace_bytes(m->hidden, m->ffn);
    if (need == 0 || !(m->eps > 0.f)) return CFPP_ERR_DIMS;
    if (m->mode != CFPP_MODE_FUSED && m->mode != CFPP_MODE_SPLIT) return CFPP_ERR_MODE;
    if (workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CFPP_ERR_WORKSPACE;
    const void* req[] = {m->rms_w, m->w_gate_up, m->w_down, m->input, m->output};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    Plan pl{};
    pl.nch = (m->hidden + kChunk - 1) / kChunk;
    pl.cpd = ((m->ffn + kChunk - 1) / kChunk + kStreamers - 1) / kStreamers;
    if (pl.nch < 1 || pl.nch > 8 || pl.cpd < 1 || pl.cpd > 8 || !shape_supported(pl)) return CFPP_ERR_DIMS;
    auto h = [](const void* q) { return reinterpret_cast<const half_t*>(q); };
    LayerParams p{};
    p.H = m->hidden; p.F = m->ffn; p.eps = m->eps; p.norm_rms = 1;
    p.x = h(m->input); p.ln_w = h(m->rms_w);
    p.w_up = h(m->w_gate_up); p.w_down = h(m->w_down);
    p.inter = reinterpret_cast<half_t*>(workspace);
    p.out = reinterpret_cast<half_t*>(m->output);
    p.c_base0 = p.x; p.c_use_o = 0; p.c_use_down = 1;
    p.host_status = device_info().host_status_dev;
    CFPP_REFUSE_AFTER_FAILURE();
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    char* ws = reinterpret_cast<char*>(workspace) + align_up((size_t)m->ffn * 2, 256);
    p.bar = reinterpret_cast<int*>(ws);
    p.grp = reinterpret_cast<int*>(ws + 256);
    p.mbox = reinterpret_cast<int*>(ws + 256 + align_up((size_t)(kBarExit + 1) * kEventGroups * kMailboxInts * 4, 256));
    // one launch (the down rows wait for the phases of the intermediate inside the kernel) when the device holds the
    // whole grid; two launches (gate/up rows, down rows) otherwise or on request
    if (m->mode == CFPP_MODE_FUSED && gated_mlp_fits(pl, p, fused_grid())) return launch_gated_mlp(pl, p, fused_grid(), st);
    const int grid = streaming_grid();
    int rc = launch_gated_up(pl, p, grid, st);
    if (rc) return rc;
    return launch_stage_c(pl, p, grid, st);
}

// ---- LLaMA attention block, batched over paged caches ---------------------------------------------------
size_t cfpp_llama_batch_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim, int32_t batch) {
    const cfpp_neox_dims d = llama_dims(hidden, heads, head_dim, 1e-6f);
    if (check_dims(&d) || batch < 1) return 0;
    return batch_layout(d, batch).total;
}

int cfpp_llama_batch_decode(const cfpp_llama_batch* a, void* workspace, size_t workspace_bytes, void* stream) {
    if (!a || !workspace) return CFPP_ERR_NULL;
    const cfpp_neox_dims d = llama_dims(a->hidden, a->heads, a->head_dim, a->eps);
    int rc = check_dims(&d);
    if (rc) return rc;
    if (a->batch < 1 || a->layer_id < 0) return CFPP_ERR_DIMS;
    const void* req[] = {a->rms_w, a->w_qkv, a->w_o, a->input, a->residual, a->residual_out, a->output, a->cos_sin};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    if (!a->paged_kv_indptr || !a->paged_kv_indices || !a->k_cache_ptrs || !a->v_cache_ptrs || !a->positions) return CFPP_ERR_NULL;
    // the sum input + residual is written while other workgroups still read both rows
    if (a->residual_out == a->input || a->residual_out == a->residual) return CFPP_ERR_ALIAS;
    const BatchLayout L = batch_layout(d, a->batch);
    if (workspace_bytes < L.total || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CFPP_ERR_WORKSPACE;
    const int nch = (d.hidden + kChunk - 1) / kChunk;
    // two workgroups per compute unit for the row streams: a second wave per SIMD covers the latencies of the
    // per-sequence reductions
    const int grid = streaming_grid() * 2;
    const int waves = grid * kStreamers;
    if (grid < 1 || (3 * d.hidden + waves - 1) / waves + 2 > kBatchParkRows) return CFPP_ERR_DIMS;
    char* ws = reinterpret_cast<char*>(workspace);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    auto h = [](const void* q) { return reinterpret_cast<const half_t*>(q); };

    // matrix-core kernels where the geometry allows (and from two sequences on: a single sequence is served as
    // well by the dot-instruction kernel, without the separate norm launch)
    const bool mfma = batch_mfma_supported(d.hidden, d.hidden) && a->batch >= 2;
    CFPP_REFUSE_AFTER_FAILURE();
    if (mfma) {
        BatchMfma m{};
        m.W = h(a->w_qkv); m.R = 3 * d.hidden; m.K = d.hidden;
        m.out_f32 = reinterpret_cast<float*>(ws + L.qkv_raw); m.out_f16 = nullptr; m.batch = a->batch;
        if (batch_mfma_norm_inside(d.hidden, a->batch)) {
            // up to 16 sequences: every workgroup of the QKV launch takes the norm upon itself (no launch for it)
            m.x = h(a->input); m.x_add = h(a->residual); m.norm_w = h(a->rms_w);
            m.sum_out = reinterpret_cast<half_t*>(a->residual_out); m.eps = a->eps;
        } else {
            BatchNorm n{};
            n.x = h(a->input); n.x_add = h(a->residual); n.norm_w = h(a->rms_w);
            n.sum_out = reinterpret_cast<half_t*>(a->residual_out); n.y = reinterpret_cast<half_t*>(ws + L.x_norm);
            n.eps = a->eps; n.K = d.hidden; n.batch = a->batch;
            if ((rc = launch_batch_norm(nch, n, st))) return rc;
            m.x = reinterpret_cast<const half_t*>(ws + L.x_norm);
        }
        if ((rc = launch_batch_mfma(m, st))) return rc;
    }
    BatchGemv g{};
    g.W = h(a->w_qkv); g.R = 3 * d.hidden; g.K = d.hidden;
    g.x = h(a->input); g.x_add = h(a->residual); g.sum_out = reinterpret_cast<half_t*>(a->residual_out);
    g.norm_w = h(a->rms_w); g.eps = a->eps;
    g.out_f32 = reinterpret_cast<float*>(ws + L.qkv_raw); g.out_f16 = nullptr;
    g.batch = a->batch;
    if (!mfma && (rc = launch_batch_gemv(nch, g, grid, st))) return rc;

    LayerParams p{};
    p.H = d.hidden; p.heads = d.heads; p.D = d.head_dim; p.rot = d.head_dim; p.F = 0;
    p.eps = a->eps;
    p.qscale = (float)(1.4426950408889634 / std::sqrt((double)d.head_dim));
    p.qkv_raw = reinterpret_cast<float*>(ws + L.qkv_raw);
    p.attn_vec = reinterpret_cast<half_t*>(ws + L.attn_vec);
    p.k_new = reinterpret_cast<half_t*>(ws + L.k_new);
    p.v_new = reinterpret_cast<half_t*>(ws + L.v_new);
    p.part_ml = reinterpret_cast<float*>(ws + L.part_ml);
    p.part_acc = reinterpret_cast<float*>(ws + L.part_acc);
    p.head_cnt = reinterpret_cast<int*>(ws + L.head_cnt);
    p.bar = reinterpret_cast<int*>(ws + L.bar);
    p.host_status = device_info().host_status_dev;
    p.qkv_head_stride = d.head_dim; p.qkv_k_off = d.hidden; p.qkv_v_off = 2 * d.hidden;
    p.append_kv = 1;
    p.rope_half_table = 1;                       // a cos_sin row holds the D/2 pair angles' cosines, then their sines
    // enough (sequence, head, split) items for one wave per SIMD, and no more: an item costs the same few memory round
    // trips at its start and at its end however long it is, and two tiles in flight per wave keep the memory busy
    // (measured: 2 % to 4 % faster than two waves per SIMD with items half as long, 7 % faster than four)
    int ms = (streaming_grid() * kStreamers) / (a->batch * d.heads);
    ms = ms < 1 ? 1 : (ms > 32 ? 32 : ms);
    p.max_split = ms;
    BatchAttn b{};
    b.batch = a->batch; b.layer_id = a->layer_id;
    b.indptr = a->paged_kv_indptr; b.indices = a->paged_kv_indices;
    b.k_ptrs = reinterpret_cast<const unsigned long long*>(a->k_cache_ptrs);
    b.v_ptrs = reinterpret_cast<const unsigned long long*>(a->v_cache_ptrs);
    b.positions = reinterpret_cast<const long long*>(a->positions);
    b.cos_sin = a->cos_sin;
    const long long items = (long long)a->batch * d.heads * p.max_split;
    const int agrid = (int)((items + kStreamers - 1) / kStreamers);
    hipLaunchKernelGGL(k_batch_attn, dim3(agrid), dim3(kStreamers * 64), 0, st, p, b);
    if ((rc = (int)hipGetLastError())) return rc;

    BatchGemv o{};
    o.W = h(a->w_o); o.R = d.hidden; o.K = d.hidden;
    o.x = reinterpret_cast<const half_t*>(ws + L.attn_vec);
    o.out_f16 = reinterpret_cast<half_t*>(a->output);
    o.batch = a->batch;
    if (mfma) {
        BatchMfma m{};
        m.W = o.W; m.R = o.R; m.K = o.K; m.x = o.x; m.out_f32 = nullptr; m.out_f16 = o.out_f16; m.batch = o.batch;
        return launch_batch_mfma(m, st);
    }
    return launch_batch_gemv(nch, o, grid, st);
}

int cfpp_neox_mlp_down(const cfpp_neox_dims* dims, const void* input, const void* attn_output,
                       const void* mlp_intermediate, const void* w_down, const void* b_down, void* output,
                       void* /* workspace: not needed */, size_t /* workspace_bytes */, void* stream) {
    int rc = check_dims(dims);
    if (rc) return rc;
    const void* req[] = {input, attn_output, mlp_intermediate, w_down, b_down, output};
    for (const void* q : req) {
        if (!q) return CFPP_ERR_NULL;
        if (!aligned16(q)) return CFPP_ERR_ALIGN;
    }
    Plan pl;
    if ((rc = make_plan(*dims, &pl))) return rc;
    if (!shape_supported(pl)) return CFPP_ERR_DIMS;
    LayerParams p{};
    p.H = dims->hidden; p.heads = dims->heads; p.D = dims->head_dim; p.rot = dims->rotary_dim; p.F = dims->ffn;
    p.w_down = reinterpret_cast<const half_t*>(w_down); p.b_down = reinterpret_cast<const half_t*>(b_down);
    p.inter = const_cast<half_t*>(reinterpret_cast<const half_t*>(mlp_intermediate));
    p.out = reinterpret_cast<half_t*>(output);
    p.c_base0 = reinterpret_cast<const half_t*>(input);
    p.c_base1 = reinterpret_cast<const half_t*>(attn_output);
    p.c_use_o = 0; p.c_use_down = 1;
    return launch_stage_c(pl, p, grid_for_streaming(pl), reinterpret_cast<hipStream_t>(stream));
}

int cfpp_workspace_check(const cfpp_neox_dims* dims, void* workspace, void* stream) {
    if (check_dims(dims)) return CFPP_ERR_DIMS;
    if (!workspace) return CFPP_ERR_NULL;
    const WorkspaceLayout L = workspace_layout(*dims);
    int* bar = reinterpret_cast<int*>(reinterpret_cast<char*>(workspace) + L.bar);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    int host[kBarStatus + 1] = {0};
    CFPP_HIP(hipMemcpyAsync(host, bar, sizeof(host), hipMemcpyDeviceToHost, st));
    CFPP_HIP(hipStreamSynchronize(st));
    bool bad = false;
    for (int i = 0; i <= kBarStatus; ++i) bad = bad || host[i] != 0;
    if (bad) {
        // a raised flag (or counters left mid-flight by an expired wait): clear so the workspace is reusable
        CFPP_HIP(hipMemsetAsync(workspace, 0, L.total, st));
        CFPP_HIP(hipStreamSynchronize(st));
        return CFPP_ERR_DEVICE;
    }
    return CFPP_OK;
}

int cfpp_device_status(int clear) {
    return host_status_flags(device_info(), clear != 0);
}

int cfpp_one_launch_fits(int grid, int compute_units, int blocks_per_cu) {
    if (grid < 1 || compute_units < 1 || blocks_per_cu < 1) return 0;
    return (long long)grid <= (long long)compute_units * blocks_per_cu ? 1 : 0;
}

#ifdef CFPP_TRACE
// Profiling builds only (not declared in cfpp.h): when set to a device buffer of [workgroups][16 waves][16 slots]
// int64, every fused launch stores 100 MHz timestamps of its phase boundaries there; NULL switches it off.
int cfpp_debug_set_trace(void* device_buffer) {
    g_trace = reinterpret_cast<long long*>(device_buffer);
    return CFPP_OK;
}
#endif

// ---- per-layer contexts --------------------------------------------------------------------------
namespace {
struct Ctx {
    cfpp_neox_dims dims{};
    const void *w_qkv = nullptr, *w_o = nullptr, *w_up = nullptr, *w_down = nullptr;
    void *k_cache = nullptr, *v_cache = nullptr;
    int cache_rows = 0, max_seq_len = 0, device = 0;
    void* slab = nullptr;          // output | k_new | v_new | workspace
    cfpp_ctx_buffers bufs{};
    void* ws = nullptr;
    size_t ws_bytes = 0;
};
std::map<std::pair<int, int64_t>, Ctx> g_ctx;
std::mutex g_ctx_mu;

void ctx_release(Ctx& c) {
    if (c.slab) {
        int cur = 0;
        (void)hipGetDevice(&cur);
        if (cur != c.device) (void)hipSetDevice(c.device);
        (void)hipFree(c.slab);
        if (cur != c.device) (void)hipSetDevice(cur);
        c.slab = nullptr;
    }
}
}  // namespace

int cfpp_ctx_create(int family, int64_t id, const cfpp_neox_dims* dims, const void* w_qkv, const void* w_o,
                    const void* w_up, const void* w_down, void* k_cache, void* v_cache, int32_t cache_rows,
                    int32_t max_seq_len, cfpp_ctx_buffers* out_buffers) {
    int rc = check_dims(dims);
    if (rc) return rc;
    Plan pl;
    if ((rc = make_plan(*dims, &pl))) return rc;
    if (!w_qkv || !w_o || !w_up || !w_down || !k_cache || !v_cache) return CFPP_ERR_NULL;
    if (cache_rows <= 0 || max_seq_len < 0 || max_seq_len > cache_rows) return CFPP_ERR_SEQ;
    Ctx c;
    c.dims = *dims;
    c.w_qkv = w_qkv; c.w_o = w_o; c.w_up = w_up; c.w_down = w_down;
    c.k_cache = k_cache; c.v_cache = v_cache; c.cache_rows = cache_rows;
    c.max_seq_len = max_seq_len > 0 ? max_seq_len : cache_rows;
    CFPP_HIP(hipGetDevice(&c.device));
    const size_t hb = align_up((size_t)dims->hidden * 2, 256);
    c.ws_bytes = workspace_layout(*dims).total;
    CFPP_HIP(hipMalloc(&c.slab, 3 * hb + c.ws_bytes));
    hipError_t e = hipMemset(c.slab, 0, 3 * hb + c.ws_bytes);
    if (e != hipSuccess) { (void)hipFree(c.slab); return (int)e; }
    char* base = reinterpret_cast<char*>(c.slab);
    c.bufs.output = base; c.bufs.k_new = base + hb; c.bufs.v_new = base + 2 * hb;
    c.ws = base + 3 * hb;
    std::lock_guard<std::mutex> lock(g_ctx_mu);
    auto key = std::make_pair(family, id);
    auto it = g_ctx.find(key);
    if (it != g_ctx.end()) { ctx_release(it->second); g_ctx.erase(it); }
    g_ctx[key] = c;
    if (out_buffers) *out_buffers = c.bufs;
    return CFPP_OK;
}

int cfpp_ctx_step(int family, int64_t id, const cfpp_neox_weights* w, const cfpp_neox_io* io, int mode, void* stream,
                  cfpp_ctx_buffers* out_buffers) {
    if (!w || !io) return CFPP_ERR_NULL;
    Ctx c;
    {
        std::lock_guard<std::mutex> lock(g_ctx_mu);
        auto it = g_ctx.find(std::make_pair(family, id));
        if (it == g_ctx.end()) return CFPP_ERR_CONTEXT;
        c = it->second;
    }
    if (io->k_cache != c.k_cache || io->v_cache != c.v_cache) return CFPP_ERR_CONTEXT;
    if ((w->w_qkv && w->w_qkv != c.w_qkv) || (w->w_o && w->w_o != c.w_o) || (w->w_up && w->w_up != c.w_up) ||
        (w->w_down && w->w_down != c.w_down))
        return CFPP_ERR_CONTEXT;
    cfpp_neox_weights ww = *w;
    ww.w_qkv = c.w_qkv; ww.w_o = c.w_o; ww.w_up = c.w_up; ww.w_down = c.w_down;
    cfpp_neox_io ii = *io;
    ii.output = c.bufs.output; ii.k_new = c.bufs.k_new; ii.v_new = c.bufs.v_new;
    ii.cache_rows = c.cache_rows;
    if (ii.max_seq_len <= 0) ii.max_seq_len = c.max_seq_len;
    if (out_buffers) *out_buffers = c.bufs;
    return cfpp_neox_layer_decode(&c.dims, &ww, &ii, mode, c.ws, c.ws_bytes, stream);
}

int cfpp_ctx_check(int family, int64_t id, void* stream) {
    Ctx c;
    {
        std::lock_guard<std::mutex> lock(g_ctx_mu);
        auto it = g_ctx.find(std::make_pair(family, id));
        if (it == g_ctx.end()) return CFPP_ERR_CONTEXT;
        c = it->second;
    }
    return cfpp_workspace_check(&c.dims, c.ws, stream);
}

int cfpp_ctx_destroy(int family, int64_t id) {
    std::lock_guard<std::mutex> lock(g_ctx_mu);
    auto it = g_ctx.find(std::make_pair(family, id));
    if (it == g_ctx.end()) return CFPP_OK;
    ctx_release(it->second);
    g_ctx.erase(it);
    return CFPP_OK;
}

// ---- LM head -------------------------------------------------------------------------------------
namespace {
int launch_lm_head(int H, int vocab, float eps, const void* x, const void* ln_w, const void* ln_b, const void* W,
                   float* logits, const LmTail& tail, int grid, hipStream_t st) {
    const int nch = (H + kChunk - 1) / kChunk;
    auto h = [](const void* q) { return reinterpret_cast<const half_t*>(q); };
    switch (nch) {
#define X(n)                                                                                                    \
    case n:                                                                                                     \
        if (H == n * kChunk)                                                                                    \
            hipLaunchKernelGGL((k_lm_head<n, true>), dim3(grid), dim3(kStreamers * 64), 0, st, h(x), H, eps, h(ln_w),  \
                               h(ln_b), h(W), vocab, logits, tail);                                             \
        else                                                                                                    \
            hipLaunchKernelGGL((k_lm_head<n, false>), dim3(grid), dim3(kStreamers * 64), 0, st, h(x), H, eps, h(ln_w), \
                               h(ln_b), h(W), vocab, logits, tail);                                             \
        return launch_check();
        CFPP_NCH_CASES(X)
#undef X
    }
    return CFPP_ERR_DIMS;
}
}  // namespace

// Row shares are worked out in 32 bits on the device (mul_div): wave index x rows must stay below 2^32.  The layer shapes
// are bounded by check_dims (at most 8192 waves x 16384 rows); the LM head's rows are the vocabulary.
constexpr int kMaxVocab = 1 << 19;
int cfpp_neox_lm_head(int32_t hidden, int32_t vocab, float eps, const void* x, const void* ln_w, const void* ln_b,
                      const void* w, float* logits, void* stream) {
    if (!x || !ln_w || !ln_b || !w || !logits) return CFPP_ERR_NULL;
    if (hidden <= 0 || hidden % 8 || hidden > 8 * kChunk || vocab <= 0 || vocab > kMaxVocab) return CFPP_ERR_DIMS;
    if (!aligned16(x) || !aligned16(ln_w) || !aligned16(ln_b) || !aligned16(w)) return CFPP_ERR_ALIGN;
    Plan pl{};
    return launch_lm_head(hidden, vocab, eps, x, ln_w, ln_b, w, logits, LmTail{}, grid_for_streaming(pl),
                          reinterpret_cast<hipStream_t>(stream));
}

// ---- whole-model decode --------------------------------------------------------------------------
struct cfpp_neox_stack {
    cfpp_neox_stack_desc desc{};
    std::vector<cfpp_neox_weights> layers;
    std::vector<void*> kc, vc;
    Plan plan{};
    int device = 0, grid = 0;
    char* slab = nullptr;
    int* state = nullptr;         // {token, seq_len, step, steps since creation, ..., [kStateDone] LM-head workgroups done}
    half_t* hidden[2] = {nullptr, nullptr};
    half_t* x0 = nullptr;         // embedding row of the current token: written by set_state, then by each step's LM head
    half_t *k_new = nullptr, *v_new = nullptr;
    float* logits = nullptr;
    float* best_val = nullptr;
    int* best_idx = nullptr;
    int* history = nullptr;
    int hist_cap = 0;
    // fused mode, when the device holds the whole grid: the layers' parameters in device memory, for the one launch that
    // runs all of them (null: one launch per layer)
    LayerParams* table = nullptr;
    LayerParams first{};          // table[0], on the host
#ifdef CFPP_TRACE
    std::vector<LayerParams> host_table;     // profiling builds: the table is rewritten when the trace buffer changes
    long long* table_trace = nullptr;
#endif
    void* ws = nullptr;
    size_t ws_bytes = 0;
    // the device-resident position changes only through set_state and the steps, all of which pass through the host:
    // this mirror lets the host refuse steps that would run past the caches (-1: not set yet)
    long long host_seq_len = -1;
    hipStream_t own_stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipStream_t exec_stream = nullptr;
};

namespace {
cfpp_neox_io stack_layer_io(const cfpp_neox_stack* s, int l) {
    const cfpp_neox_dims& d = s->desc.dims;
    cfpp_neox_io io{};
    io.input = l == 0 ? s->x0 : s->hidden[l & 1];
    io.output = s->hidden[(l + 1) & 1];
    io.k_new = s->k_new; io.v_new = s->v_new;
    io.k_cache = s->kc[l]; io.v_cache = s->vc[l];
    io.cache_rows = s->desc.cache_rows;
    io.cos = s->desc.rope_cos; io.sin = s->desc.rope_sin;
    io.rope_stride = d.rotary_dim;
    io.seq_len = 0;
    io.d_seq_len = s->state + 1;
    io.max_seq_len = s->desc.cache_rows;
    return io;
}
int stack_layer_params(const cfpp_neox_stack* s, int l, LayerParams* p, Plan* pl) {
    const cfpp_neox_io io = stack_layer_io(s, l);
    const int rc = fill_params(&s->desc.dims, &s->layers[l], &io, s->ws, s->ws_bytes, true, true, p, pl);
    if (rc) return rc;
    // launch tags from the stack's step counter: no launch has to publish a generation for the next one
    p->tag_src = s->state + 3; p->tag_mul = s->desc.n_layers; p->tag_add = l;
    return CFPP_OK;
}
int stack_enqueue_layer(cfpp_neox_stack* s, int l, hipStream_t st) {
    LayerParams p;
    Plan pl;
    const int rc = stack_layer_params(s, l, &p, &pl);
    if (rc) return rc;
    const cfpp_neox_io io = stack_layer_io(s, l);
    return run_layer(pl, p, s->desc.mode, seq_hint_of(&io), st);
}
// all layers: one launch when the stack has its table, one per layer otherwise
int stack_enqueue_layers(cfpp_neox_stack* s, hipStream_t st) {
#ifdef CFPP_TRACE
    // layer l stamps into its own [workgroups][waves][slots] block of the trace buffer
    if (s->table != nullptr && s->table_trace != g_trace) {
        for (size_t l = 0; l < s->host_table.size(); ++l)
            s->host_table[l].trace = g_trace ? g_trace + l * ((size_t)kMaxGrid * kMaxWaves * kTraceSlots) : nullptr;
        CFPP_HIP(hipStreamSynchronize(st));
        CFPP_HIP(hipMemcpy(s->table, s->host_table.data(), s->host_table.size() * sizeof(LayerParams), hipMemcpyHostToDevice));
        s->table_trace = g_trace;
    }
#endif
    if (s->table != nullptr) return launch_fused_stack(s->plan, s->first, s->table, s->desc.n_layers, fused_grid(), st);
    for (int l = 0; l < s->desc.n_layers; ++l) {
        const int rc = stack_enqueue_layer(s, l, st);
        if (rc) return rc;
    }
    return CFPP_OK;
}
// Fills the table if the one launch for all layers can be used: fused mode, every attention wave with one item at
// most, the whole grid co-resident.
int stack_make_table(cfpp_neox_stack* s, LayerParams* dev_table) {
    if (s->desc.mode != CFPP_MODE_FUSED) return CFPP_OK;
    std::vector<LayerParams> host(s->desc.n_layers);
    Plan pl;
    for (int l = 0; l < s->desc.n_layers; ++l)
        if (stack_layer_params(s, l, &host[l], &pl) != CFPP_OK) return CFPP_OK;     // the steps report what is wrong
    const int grid = fused_grid();
    if (grid > kLayerFlagWgs || (long long)host[0].heads * (host[0].max_split + 1) > (long long)grid * kStreamers ||
        !fused_stack_fits(pl, host[0], grid))
        return CFPP_OK;
    const hipError_t e = hipMemcpy(dev_table, host.data(), host.size() * sizeof(LayerParams), hipMemcpyHostToDevice);
    if (e != hipSuccess) return (int)e;
    s->first = host[0];
    s->table = dev_table;
#ifdef CFPP_TRACE
    s->host_table = host;
    s->table_trace = host[0].trace;
#endif
    return CFPP_OK;
}

LmTail stack_tail(const cfpp_neox_stack* s) {
    return LmTail{s->best_val, s->best_idx, s->state, s->state + kStateDone, s->history, s->hist_cap,
                  reinterpret_cast<const half_t*>(s->desc.embed), s->x0};
}
// the layers (one launch for all of them, or one each), then the LM head, whose last workgroup picks the token, advances
// the state and fetches the picked token's embedding row for the next step
int stack_enqueue_step(cfpp_neox_stack* s, hipStream_t st) {
    const cfpp_neox_dims& d = s->desc.dims;
    const int rc = stack_enqueue_layers(s, st);
    if (rc) return rc;
    return launch_lm_head(d.hidden, s->desc.vocab, d.eps, s->hidden[s->desc.n_layers & 1], s->desc.final_ln_w,
                          s->desc.final_ln_b, s->desc.lm_head, s->logits, stack_tail(s), s->grid, st);
}
}  // namespace

int cfpp_stack_create(const cfpp_neox_stack_desc* desc, cfpp_neox_stack** out) {
    if (!desc || !out) return CFPP_ERR_NULL;
    int rc = check_dims(&desc->dims);
    if (rc) return rc;
    if (desc->n_layers <= 0 || desc->vocab <= 0 || desc->vocab > kMaxVocab || desc->cache_rows <= 0) return CFPP_ERR_DIMS;
    if (!desc->layers || !desc->embed || !desc->final_ln_w || !desc->final_ln_b || !desc->lm_head || !desc->k_caches ||
        !desc->v_caches || !desc->rope_cos || !desc->rope_sin)
        return CFPP_ERR_NULL;
    if (desc->mode != CFPP_MODE_FUSED && desc->mode != CFPP_MODE_SPLIT && desc->mode != CFPP_MODE_FUSED_LAYERS) return CFPP_ERR_MODE;
    cfpp_neox_stack* s = new cfpp_neox_stack();
    s->desc = *desc;
    s->layers.assign(desc->layers, desc->layers + desc->n_layers);
    s->kc.assign(desc->k_caches, desc->k_caches + desc->n_layers);
    s->vc.assign(desc->v_caches, desc->v_caches + desc->n_layers);
    s->desc.layers = nullptr; s->desc.k_caches = nullptr; s->desc.v_caches = nullptr;
    if ((rc = make_plan(desc->dims, &s->plan))) { delete s; return rc; }
    hipError_t e = hipGetDevice(&s->device);
    if (e != hipSuccess) { delete s; return (int)e; }
    s->grid = grid_for_streaming(s->plan);
    s->hist_cap = 1 << 16;
    const cfpp_neox_dims& d = desc->dims;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
    const size_t o_state = take(64), o_h0 = take((size_t)d.hidden * 2), o_h1 = take((size_t)d.hidden * 2);
    const size_t o_x0 = take((size_t)d.hidden * 2);
    const size_t o_table = take((size_t)desc->n_layers * sizeof(LayerParams));
    const size_t o_k = take((size_t)d.hidden * 2), o_v = take((size_t)d.hidden * 2);
    const size_t o_logits = take((size_t)desc->vocab * 4);
    const size_t o_bv = take((size_t)s->grid * 4), o_bi = take((size_t)s->grid * 4);
    const size_t o_hist = take((size_t)s->hist_cap * 4);
    s->ws_bytes = workspace_layout(d).total;
    const size_t o_ws = take(s->ws_bytes);
    e = hipMalloc(reinterpret_cast<void**>(&s->slab), off);
    if (e != hipSuccess) { delete s; return (int)e; }
    e = hipMemset(s->slab, 0, off);
    if (e != hipSuccess) { (void)hipFree(s->slab); delete s; return (int)e; }
    s->state = reinterpret_cast<int*>(s->slab + o_state);
    s->hidden[0] = reinterpret_cast<half_t*>(s->slab + o_h0);
    s->hidden[1] = reinterpret_cast<half_t*>(s->slab + o_h1);
    s->x0 = reinterpret_cast<half_t*>(s->slab + o_x0);
    s->k_new = reinterpret_cast<half_t*>(s->slab + o_k);
    s->v_new = reinterpret_cast<half_t*>(s->slab + o_v);
    s->logits = reinterpret_cast<float*>(s->slab + o_logits);
    s->best_val = reinterpret_cast<float*>(s->slab + o_bv);
    s->best_idx = reinterpret_cast<int*>(s->slab + o_bi);
    s->history = reinterpret_cast<int*>(s->slab + o_hist);
    s->ws = s->slab + o_ws;
    // the state block starts as token 0 at position 0: its embedding row, so that steps without set_state are defined
    hipLaunchKernelGGL(k_embed, dim3((d.hidden / 8 + 255) / 256), dim3(256), 0, nullptr,
                       reinterpret_cast<const half_t*>(desc->embed), s->state, d.hidden, desc->vocab, s->x0);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) { (void)hipFree(s->slab); delete s; return (int)e; }
    if ((rc = stack_make_table(s, reinterpret_cast<LayerParams*>(s->slab + o_table)))) { (void)hipFree(s->slab); delete s; return rc; }
    *out = s;
    return CFPP_OK;
}

int cfpp_stack_set_state(cfpp_neox_stack* s, int32_t token, int32_t seq_len, void* stream) {
    if (!s) return CFPP_ERR_NULL;
    if (seq_len < 0 || seq_len >= s->desc.cache_rows) return CFPP_ERR_SEQ;     // the next step appends row seq_len
    if (token < 0 || token >= s->desc.vocab) return CFPP_ERR_DIMS;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(k_set_state, dim3(1), dim3(64), 0, st, s->state, token, seq_len);
    int rc = launch_check();
    if (rc) return rc;
    const int H = s->desc.dims.hidden;
    hipLaunchKernelGGL(k_embed, dim3((H / 8 + 255) / 256), dim3(256), 0, st,
                       reinterpret_cast<const half_t*>(s->desc.embed), s->state, H, s->desc.vocab, s->x0);
    rc = launch_check();
    if (!rc) s->host_seq_len = seq_len;
    return rc;
}

namespace {
// `n` more steps need cache rows host_seq_len .. host_seq_len + n - 1
int stack_room(const cfpp_neox_stack* s, long long n) {
    const long long at = s->host_seq_len < 0 ? 0 : s->host_seq_len;
    return at + n <= (long long)s->desc.cache_rows ? CFPP_OK : CFPP_ERR_SEQ;
}
void stack_advance(cfpp_neox_stack* s, long long n) { s->host_seq_len = (s->host_seq_len < 0 ? 0 : s->host_seq_len) + n; }
}  // namespace

int cfpp_stack_step(cfpp_neox_stack* s, void* stream) {
    if (!s) return CFPP_ERR_NULL;
    int rc = stack_room(s, 1);
    if (rc) return rc;
    CFPP_REFUSE_AFTER_FAILURE();
    rc = stack_enqueue_step(s, reinterpret_cast<hipStream_t>(stream));
    if (!rc) stack_advance(s, 1);
    return rc;
}

int cfpp_stack_layers_per_launch(const cfpp_neox_stack* s) {
    if (!s) return CFPP_ERR_NULL;
    return s->table != nullptr ? s->desc.n_layers : 1;
}

int cfpp_stack_check(cfpp_neox_stack* s, void* stream) {
    if (!s) return CFPP_ERR_NULL;
    return cfpp_workspace_check(&s->desc.dims, s->ws, stream);
}

int cfpp_stack_graph_steps(cfpp_neox_stack* s, int32_t n_steps, void* stream) {
    if (!s) return CFPP_ERR_NULL;
    if (n_steps < 0) return CFPP_ERR_DIMS;
    int room = stack_room(s, n_steps);
    if (room) return room;
    CFPP_REFUSE_AFTER_FAILURE();
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (!st) {
        if (!s->own_stream) CFPP_HIP(hipStreamCreateWithFlags(&s->own_stream, hipStreamDefault));   // ordered with the null stream
        st = s->own_stream;
    }
    if (!s->exec) {
        CFPP_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeRelaxed));
        int rc = stack_enqueue_step(s, st);
        hipGraph_t g = nullptr;
        hipError_t e = hipStreamEndCapture(st, &g);
        if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
        if (e != hipSuccess) return (int)e;
        s->graph = g;
        CFPP_HIP(hipGraphInstantiate(&s->exec, s->graph, nullptr, nullptr, 0));
    }
    for (int i = 0; i < n_steps; ++i) {
        CFPP_HIP(hipGraphLaunch(s->exec, st));
        stack_advance(s, 1);
    }
    if (!stream) CFPP_HIP(hipStreamSynchronize(st));
    return CFPP_OK;
}

int cfpp_stack_profile_step(cfpp_neox_stack* s, void* stream, float* layer_ms, float* lm_head_ms, float* total_ms) {
    if (!s) return CFPP_ERR_NULL;
    {
        const int room = stack_room(s, 1);
        if (room) return room;
    }
    CFPP_REFUSE_AFTER_FAILURE();
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int L = s->desc.n_layers;
    std::vector<hipEvent_t> ev(L + 3);
    for (auto& e : ev) CFPP_HIP(hipEventCreate(&e));
    // fused mode: one kernel per layer, timed from its own start to its own end (with all layers in one launch: that
    // launch, and every layer is reported as its share of it); split mode (three kernels per layer): stream events
    // between the layers, which include the launch gaps
    const bool chain = s->table != nullptr;
    bool fused = chain;
    if (!chain && s->desc.mode != CFPP_MODE_SPLIT && s->desc.dims.heads <= fused_grid() * kStreamers) {
        const cfpp_neox_io io0 = stack_layer_io(s, 0);
        LayerParams p0;
        Plan pl0;
        if (fill_params(&s->desc.dims, &s->layers[0], &io0, s->ws, s->ws_bytes, true, true, &p0, &pl0) == CFPP_OK)
            fused = fused_fits(pl0, p0, fused_grid());
    }
    std::vector<KernelEvents> kev(chain ? 1 : (fused ? L : 0));
    for (auto& k : kev) {
        CFPP_HIP(hipEventCreate(&k.start));
        CFPP_HIP(hipEventCreate(&k.stop));
    }
    int rc = CFPP_OK;
    {
        const cfpp_neox_dims& d = s->desc.dims;
        CFPP_HIP(hipEventRecord(ev[L + 2], st));     // start of the step
        if (chain) {
            tl_kernel_events = &kev[0];
            rc = stack_enqueue_layers(s, st);
            tl_kernel_events = nullptr;
        }
        for (int l = 0; l < L && !rc && !chain; ++l) {
            CFPP_HIP(hipEventRecord(ev[l], st));
            if (fused) tl_kernel_events = &kev[l];
            rc = stack_enqueue_layer(s, l, st);
            tl_kernel_events = nullptr;
        }
        if (!rc) {
            CFPP_HIP(hipEventRecord(ev[L], st));
            rc = launch_lm_head(d.hidden, s->desc.vocab, d.eps, s->hidden[L & 1], s->desc.final_ln_w, s->desc.final_ln_b,
                                s->desc.lm_head, s->logits, stack_tail(s), s->grid, st);
            CFPP_HIP(hipEventRecord(ev[L + 1], st));
        }
    }
    hipEvent_t end;
    CFPP_HIP(hipEventCreate(&end));
    CFPP_HIP(hipEventRecord(end, st));
    CFPP_HIP(hipEventSynchronize(end));
    if (!rc) {
        float all = 0.f;
        if (chain) CFPP_HIP(hipEventElapsedTime(&all, kev[0].start, kev[0].stop));
        for (int l = 0; l < L; ++l) {
            float ms = all / (float)L;
            if (chain) {}
            else if (fused) CFPP_HIP(hipEventElapsedTime(&ms, kev[l].start, kev[l].stop));
            else CFPP_HIP(hipEventElapsedTime(&ms, ev[l], ev[l + 1]));
            if (layer_ms) layer_ms[l] = ms;
        }
        float ms = 0.f;
        CFPP_HIP(hipEventElapsedTime(&ms, ev[L], ev[L + 1]));
        if (lm_head_ms) *lm_head_ms = ms;
        CFPP_HIP(hipEventElapsedTime(&ms, ev[L + 2], end));
        if (total_ms) *total_ms = ms;
    }
    for (auto& e : ev) (void)hipEventDestroy(e);
    for (auto& k : kev) { (void)hipEventDestroy(k.start); (void)hipEventDestroy(k.stop); }
    (void)hipEventDestroy(end);
    if (!rc) stack_advance(s, 1);
    return rc;
}

int cfpp_stack_buffers(cfpp_neox_stack* s, float** logits, void** hidden, int32_t** state, int32_t** history,
                       int32_t* history_capacity) {
    if (!s) return CFPP_ERR_NULL;
    if (logits) *logits = s->logits;
    if (hidden) *hidden = s->hidden[s->desc.n_layers & 1];
    if (state) *state = s->state;
    if (history) *history = s->history;
    if (history_capacity) *history_capacity = s->hist_cap;
    return CFPP_OK;
}

int cfpp_stack_destroy(cfpp_neox_stack* s) {
    if (!s) return CFPP_OK;
    if (s->exec) (void)hipGraphExecDestroy(s->exec);
    if (s->graph) (void)hipGraphDestroy(s->graph);
    if (s->own_stream) (void)hipStreamDestroy(s->own_stream);
    if (s->slab) (void)hipFree(s->slab);
    delete s;
    return CFPP_OK;
}

}  // extern "C"
