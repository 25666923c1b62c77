// Device-side building blocks of the GPT-NeoX decode step for gfx950 (wave64, CDNA4).
//
// The layer is five matrix-vector products plus one single-query attention, all bound by HBM
// bandwidth.  The decomposition used here (it replaces the reference's one-cluster-per-head
// scheme, include/5090/pythia_2b8/kernel.cuh:51-949):
//
//   stage A  LayerNorm statistics in registers of every wave; one wave streams whole weight rows of
//            W_qkv (then W_up) with 16-byte non-temporal lane loads, 512 contiguous halfs per
//            wave-load, fp32 accumulation through v_dot2_f32_f16 and a DPP row reduction; the dot
//            products are parked in LDS and finished after the loop, one row per lane
//            (bias -> raw q/k/v in fp32, or bias -> tanh-GELU -> fp16 intermediate).
//   stage B  split-KV single-query attention: one wave per (head, KV split); 16 lanes per cache
//            row, exp2-domain online softmax in fp32, fp32 partials in scratch, and the last wave
//            to finish a head merges that head's partials in split order.  RoPE is applied when
//            q / k are read from the raw fp32 scratch; the (head, split 0) wave appends the rotated
//            K and V to the cache and returns them.
//   stage C  out = x + b_o + b_down + W_o attn + W_down h; rows are split over workgroups.  MLP-down
//            is K-split over the streaming waves of a workgroup (activation slices in registers),
//            the O projection is row-per-wave; a fixed-order LDS reduction finishes each row:
//            deterministic, no atomics on data.
//
// The same device functions are used by the per-stage kernels (split mode: the kernel boundary is
// the barrier) and by the persistent fused kernel (device-wide barriers with bounded waits).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cfpp {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kChunk = 512;            // halfs covered by one wave-wide 16-byte load
constexpr int kMaxSplit = 64;          // partial results per head: KV splits (the effective count follows seq_len) + the new token's item
constexpr int kSplitRows = 64;         // target cache rows per (head, split) item
constexpr int kMaxWaves = 16;          // waves per workgroup
constexpr int kRowBatch = 32;          // stage-C rows per workgroup pass
constexpr int kUpRpi = 2;              // adjacent MLP-up rows per tile
// How a streaming wave keeps its loads in flight: two tiles, the loads of the next one issued in one burst before the
// current one is reduced (false), or one tile whose registers are refilled one by one as they are used (true: half the
// bytes in flight, no bursts).  Measured on whole-model decode steps: rows of five 1 KB chunks (Pythia-2.8B) gain
// 1.4 % with the second, rows of eight (Pythia-6.9B) lose 0.7 % with it; the LM head is the same either way.
template <int NCH> struct RollTiles { static constexpr bool value = NCH <= 5; };
constexpr int kStreamers = 4;          // streaming waves per workgroup: one per SIMD of the compute unit
constexpr int kUpPhases = 2;           // the MLP intermediate is produced and consumed in this many phases
constexpr float kNegBig = -1.0e30f;
constexpr int kSpinLimit = 1 << 20;    // bounded device-side waits (order of a second)
constexpr int kHeadCntStride = 16;     // ints between the arrival counters of two heads: returning atomics of different
                                       // heads must not meet in one cache line (they serialise at the memory side; with
                                       // all 32 counters in one line the items of a Pythia-2.8B layer ended 1 us later)

enum : int { kStatusSpin = 1, kStatusSeq = 2 };
// Slots of LayerParams::bar.  The event counters reset themselves (the arrival that completes a count
// stores zero); flags are not reset at all: a launch raises a flag by writing its tag, which no earlier
// launch on the workspace has used (launch_generation below, or a counter of the caller's).
enum BarSlot : int {
    kBarQkv = 0,                      // streaming waves that have written their QKV rows
    kBarUp = 1,                       // kBarUp + g: streaming waves that have written their MLP-up rows of phase g (kUpPhases slots)
    kBarHeads = kBarUp + kUpPhases,   // heads whose attention output is merged
    kBarExit = kBarHeads + 1,         // workgroups that have finished (only its group counters are used, see launch_generation)
    kBarStatus = kBarExit + 1,        // failure flags (kStatusSpin, kStatusSeq); never reset by the kernels
    kBarGen = kBarStatus + 1          // (unused)
};
static_assert(kBarGen < 16, "the slots are the ints of one 64-byte line");

struct LayerParams {
    int H, heads, D, rot, F;
    float eps, qscale;
    const half_t *ln_w, *ln_b, *w_qkv, *b_qkv, *w_o, *b_o, *ln2_w, *ln2_b, *w_up, *b_up, *w_down, *b_down;
    const half_t* x;
    half_t *out, *k_new, *v_new, *k_cache, *v_cache;
    int cache_rows;
    const float *cos, *sin;
    int rope_stride;
    int rope_half_table;    // rotate-half RoPE: 0 = cos/sin hold one entry per rotary dim and dim d uses entry d (GPT-NeoX ops);
                            // 1 = they hold rot/2 entries, the angles of the pairs, and dims d and d + rot/2 share entry d
    int seq_len;
    const int* d_seq_len;
    int seq_cap;        // largest sequence length the launch geometry was sized for (a device-side length beyond it is refused)
    int max_split;      // cap on the KV splits per head (<= kMaxSplit)
    const int* kv_rows;     // paged caches: cache row r of this sequence lives in row kv_rows[r] of k_cache / v_cache (null: r itself)
    const int* tag_src;     // launch tags from a counter the caller advances between launches (null: from kBarGen)
    int tag_mul, tag_add;   // tag = tag_src[0] * tag_mul + tag_add + 1
    int arrival_agents;     // an idle attention wave carries the streaming waves' MLP-up arrivals to the device-wide counters
    int up_wgs;             // split mode: workgroups that share the MLP-up rows of the middle launch (it may have more, for attention items)
    // layer family switches (defaults = GPT-NeoX): RMSNorm instead of LayerNorm; where head h's raw q, k, v sit in
    // qkv_raw (NeoX interleaves [h][q|k|v][D]: stride 3D, offsets D and 2D; LLaMA stacks [q;k;v]: stride D,
    // offsets H and 2H); whether split 0 appends the new K/V row to the caches
    int norm_rms, qkv_head_stride, qkv_k_off, qkv_v_off, append_kv;
    const half_t* x_add;    // nullable: a second input row added to x (fp16-rounded) before the norm ...
    half_t* x_sum_out;      // ... and where the sum is stored (the caller's residual stream)
    int c_add_sum;          // stage C adds that sum (or x itself when there is no x_add) to the output
    // scratch
    float* qkv_raw;     // [3H] fp32: W_qkv ln1(x) + b_qkv, before RoPE
    half_t* attn_vec;   // [H] fp16: merged attention output (input of the O projection)
    half_t* inter;      // [F] fp16: gelu(W_up ln2(x) + b_up)
    float* part_ml;     // [heads][kMaxSplit][2] running max (log2 domain) and denominator
    float* part_acc;    // [heads][kMaxSplit][D]
    int* head_cnt;      // [heads][kHeadCntStride] arrival counters (one 64-byte line per head), self-resetting
    int* bar;           // device-wide counters, see BarSlot
    int* grp;           // [events][kEventGroups] group counters, one 64-byte line each
    int* mbox;          // [kMaxGrid][kMailboxInts] event flags, one line per workgroup
    int* team;          // [1 + kUpPhases][kMaxGrid / kTeamWgs][kMailboxInts] ticket counters of the tile teams (QKV, MLP-up phases)
    // stage-C selection (split API halves)
    const half_t* c_base0;   // residual terms added to the output (nullable)
    const half_t* c_base1;
    int c_use_o, c_use_down;
    int* host_status;   // nullable: a word in pinned host memory that receives every failure flag as well, so that the
                        // host sees a failed launch without reading device memory
#ifdef CFPP_TRACE
    long long* trace;   // per-workgroup phase timestamps of the fused kernel (null = off); profiling builds only
#endif
};

// Phase timestamps of the fused kernel exist in profiling builds (-DCFPP_TRACE) only.
constexpr int kTraceSlots = 16;
#ifdef CFPP_TRACE
__device__ __forceinline__ void trace_value(const LayerParams& p, int slot, long long v) {
    if (p.trace != nullptr && (threadIdx.x & 63) == 0)
        p.trace[((size_t)blockIdx.x * kMaxWaves + (threadIdx.x >> 6)) * kTraceSlots + slot] = v;
}
__device__ __forceinline__ void trace_mark(const LayerParams& p, int slot) {
    if (p.trace != nullptr && (threadIdx.x & 63) == 0)
        p.trace[((size_t)blockIdx.x * kMaxWaves + (threadIdx.x >> 6)) * kTraceSlots + slot] = wall_clock64();
}
#else
__device__ __forceinline__ void trace_value(const LayerParams&, int, long long) {}
__device__ __forceinline__ void trace_mark(const LayerParams&, int) {}
#endif

// ------------------------------------------------------------------------------------------------
// loads / conversions
// ------------------------------------------------------------------------------------------------
// The parameter block of a kernel (several hundred bytes) does not fit the scalar registers, so the compiler loads it
// piecemeal, where each piece is first needed, and waits for each piece: at the start of a launch every one of those
// loads misses the (just invalidated) scalar cache, and half a dozen dependent misses in a row stood in front of the
// first weight request.  Reading one word of every 64-byte line of the kernel-argument segment up front, all in
// flight together, turns them into one miss; everything after that hits.
template <int BYTES>
__device__ __forceinline__ void touch_kernel_arguments() {
    typedef __attribute__((address_space(4))) const int ConstInt;
    ConstInt* ka = (ConstInt*)__builtin_amdgcn_kernarg_segment_ptr();
    int acc = 0;
#pragma unroll
    for (int off = 0; off < BYTES; off += 64) acc ^= ka[off / 4];
    asm volatile("; kernel arguments resident (%0)" ::"s"(acc));
}
// bytes of the kernel-argument segment of a kernel whose only explicit argument is a LayerParams (+ the hidden ones
// the runtime appends: grid and block sizes)
constexpr int kLayerKernargBytes = 448;
__device__ __forceinline__ u32x4 ld_stream16(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ u32x4 ld16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }

// Device-coherent accessors for values that cross workgroups inside one launch.  Every XCD has its
// own L2, so plain stores may sit dirty in one L2 while another XCD reads a stale line.  Relaxed
// agent-scope atomics compile to sc1 stores (write through) and sc1 loads (miss in the caches), which
// makes the hand-off coherent without agent-scope fences; those fences write back / invalidate the
// whole L2 and cost far more than the data they protect.  The producer drains its stores
// (s_waitcnt 0) before it bumps the counter the consumer polls.
__device__ __forceinline__ void st_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(half_t* p, half_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent2(float* p, float a, float b) {   // p 8-byte aligned
    const uint64_t v = (uint64_t)__float_as_uint(a) | ((uint64_t)__float_as_uint(b) << 32);
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void ld_agent2(const float* p, float& a, float& b) {   // p 8-byte aligned
    const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    a = __uint_as_float((uint32_t)v);
    b = __uint_as_float((uint32_t)(v >> 32));
}
__device__ __forceinline__ u32x4 ld_agent16(const void* p) {
    const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
    const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
    return r;
}
__device__ __forceinline__ half_t ld_agent(const half_t* p) {
    const unsigned short u = __hip_atomic_load(reinterpret_cast<const unsigned short*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(half_t, u);
}
// all memory operations this wave has issued are complete
__device__ __forceinline__ void drain_memory_ops() { __builtin_amdgcn_s_waitcnt(0); }

__device__ __forceinline__ half2_t as_h2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
    half2_t a = as_h2(v.x), b = as_h2(v.y), c = as_h2(v.z), d = as_h2(v.w);
    f[0] = (float)a.x; f[1] = (float)a.y; f[2] = (float)b.x; f[3] = (float)b.y;
    f[4] = (float)c.x; f[5] = (float)c.y; f[6] = (float)d.x; f[7] = (float)d.y;
}
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    half2_t a = {(half_t)f[0], (half_t)f[1]}, b = {(half_t)f[2], (half_t)f[3]};
    half2_t c = {(half_t)f[4], (half_t)f[5]}, d = {(half_t)f[6], (half_t)f[7]};
    u32x4 r = {as_u32(a), as_u32(b), as_u32(c), as_u32(d)};
    return r;
}
__device__ __forceinline__ float dot8(u32x4 w, const half2_t (&x)[4], float acc) {
    acc = __builtin_amdgcn_fdot2(as_h2(w.x), x[0], acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(w.y), x[1], acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(w.z), x[2], acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(w.w), x[3], acc, false);
    return acc;
}

// ------------------------------------------------------------------------------------------------
// wave64 reductions: DPP rotations inside a 16-lane row, then v_readlane across the four rows
// ------------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row16_sum(float v) {    // every lane of a 16-lane row gets the row sum
    v += dpp_mov<0x128>(v);   // row_ror:8
    v += dpp_mov<0x124>(v);   // row_ror:4
    v += dpp_mov<0x122>(v);   // row_ror:2
    v += dpp_mov<0x121>(v);   // row_ror:1
    return v;
}
__device__ __forceinline__ float rl(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {     // wave-uniform result
    v = row16_sum(v);
    return (rl(v, 0) + rl(v, 16)) + (rl(v, 32) + rl(v, 48));
}
__device__ __forceinline__ float xor_shfl(float v, int mask) { return __shfl_xor(v, mask, kWave); }
__device__ __forceinline__ int first_lane(int v) { return __builtin_amdgcn_readfirstlane(v); }

// ------------------------------------------------------------------------------------------------
// math
// ------------------------------------------------------------------------------------------------
// The library is compiled with -ffp-contract=off and every fused multiply-add is written out (fmadd below): the
// per-stage kernels and the one-launch kernel inline the same functions into different surroundings, and a compiler
// that is free to contract a*b + c*d either way (or not at all) can round the same expression differently in two
// kernels - enough to flip an fp16 rounding of a rotated K value once in a few thousand, which the bit-exact
// split == fused checks at full model depth catch.
__device__ __forceinline__ float fmadd(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
// tanh-GELU, 0.5 x (1 + tanh(sqrt(2/pi)(x + 0.044715 x^3))) with tanh(u) = 1 - 2/(1 + e^{2u}) on the
// native exp2 (reference include/5090/pythia_2b8/kernel.cuh:26-49 builds the same from ex2.approx).
__device__ __forceinline__ float gelu_tanh(float x) {
    const float u = 0.7978845608028654f * fmadd(0.044715f * x * x, x, x);
    const float e = __builtin_amdgcn_exp2f(u * 2.8853900817779268f);   // e^{2u}
    const float t = 1.0f - 2.0f / (1.0f + e);
    return 0.5f * x * (1.0f + t);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// SiLU, x / (1 + e^{-x}), on the native exp2
__device__ __forceinline__ float silu(float x) { return x / (1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x)); }

// ------------------------------------------------------------------------------------------------
// device-wide synchronisation (bounded spins; a timeout raises a status flag and falls through)
// ------------------------------------------------------------------------------------------------
// Device-wide events.  The wave whose arrival completes an event writes a flag into one mailbox line
// per workgroup, and waiters poll only their own workgroup's line.  (Letting every waiting wave poll a
// shared counter floods a single memory channel with coherent loads and slows the streaming loads of the
// whole chip.)
constexpr int kMailboxInts = 16;       // one 64-byte line per workgroup
constexpr int kMaxGrid = 1024;         // workgroups a fused launch may have

// floor(a * b / c) for the shares of rows, tiles and workgroups (0 <= a, b; 0 < c; a * b < 2^32, which the host checks
// for the shapes it accepts).  32-bit on purpose: a 64-bit division is a few hundred instructions on this hardware, and
// the first one sits in front of every wave's first load.
__device__ __forceinline__ int mul_div(int a, int b, int c) { return (int)(((unsigned)a * (unsigned)b) / (unsigned)c); }
__device__ __forceinline__ void counter_add(int* ctr, int v) {
    __hip_atomic_fetch_add(ctr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int counter_peek(const int* ctr) {
    return __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Failure flags go to the workspace's status word and, when the launch has one, to pinned host memory: one word
// per flag (host[0] for kStatusSpin, host[1] for kStatusSeq), written with a plain system-scope store, so that two
// different flags never overwrite each other and no read-modify-write has to cross the bus.
struct StatusSink { int* dev; int* host; };
__device__ __forceinline__ void raise_status(const StatusSink& s, int flag) {
    __hip_atomic_fetch_or(s.dev, flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (s.host != nullptr) __hip_atomic_store(s.host + (flag == kStatusSpin ? 0 : 1), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// Arrivals are counted hierarchically, because a thousand waves adding to one address serialise at the
// memory side (tens of nanoseconds each) and every one of them waits for its return value: first in LDS
// among the waves of a workgroup (when `lds_ctr` is given), then in one of kEventGroups group counters
// (workgroup index modulo kEventGroups, each on its own 64-byte line), then in the event's top counter.
// Only the last arrival of each level goes on to the next one.
constexpr int kEventGroups = 16;
__device__ __forceinline__ int* group_counter(int* grp, int event, int g) {
    return grp + (event * kEventGroups + g) * kMailboxInts;
}
// Called by a whole wave after its stores: drains them and counts the arrival; `per_wg` waves of every
// workgroup arrive (1 if lds_ctr is null).  The wave that completes a count zeroes it for the next launch;
// the one that completes the event writes `tag` into mailbox slot `event` of all `nwg` workgroups and
// returns true.
// (`lane_in`: the caller's lane index, for callers that keep it opaque to the optimiser.)
__device__ __forceinline__ bool event_arrive(int* bar, int* grp, int* mbox, int event, int nwg, int* lds_ctr, int per_wg, int tag,
                                             int lane_in = -1) {
    const int lane = lane_in >= 0 ? lane_in : (int)(threadIdx.x & 63);
    drain_memory_ops();
    int go = 1;
    if (lds_ctr != nullptr) {
        if (lane == 0) go = (__hip_atomic_fetch_add(lds_ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == per_wg - 1);
        go = __builtin_amdgcn_readfirstlane(go);
    }
    if (!go) return false;
    const int g = blockIdx.x % kEventGroups;
    const int gsize = (nwg - g + kEventGroups - 1) / kEventGroups;
    int* gc = group_counter(grp, event, g);
    if (lane == 0) {
        go = (__hip_atomic_fetch_add(gc, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gsize - 1);
        if (go) __hip_atomic_store(gc, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    go = __builtin_amdgcn_readfirstlane(go);
    if (!go) return false;
    const int ngroups = nwg < kEventGroups ? nwg : kEventGroups;
    if (lane == 0) {
        go = (__hip_atomic_fetch_add(bar + event, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngroups - 1);
        if (go) __hip_atomic_store(bar + event, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    go = __builtin_amdgcn_readfirstlane(go);
    if (!go) return false;
    if (mbox != nullptr) {
        for (int w = lane; w < nwg; w += kWave)
            __hip_atomic_store(mbox + w * kMailboxInts + event, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}
// One lane polls this workgroup's mailbox line, the wave leaves together.  Data published before the
// arrivals must be read with ld_agent / ld_agent16.  A wait that expires raises a status flag and
// falls through.
__device__ __forceinline__ void event_wait(const int* mbox, int slot, int tag, const StatusSink& status, int lane_in = -1) {
    if ((lane_in >= 0 ? lane_in : (int)(threadIdx.x & 63)) == 0) {
        const int* f = mbox + blockIdx.x * kMailboxInts + slot;
        int spins = 0;
        while (counter_peek(f) != tag) {
            __builtin_amdgcn_s_sleep(2);
            if (++spins > kSpinLimit) { raise_status(status, kStatusSpin); break; }
        }
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// The launch generation of a workspace: the number of workgroups that have ever finished a one-launch kernel on it,
// kept in the kEventGroups group counters of kBarExit (never reset).  A workgroup that leaves adds one to the counter
// of its group without waiting for the result (launch_generation_leave); the next launch starts after this one has
// completed, reads the counters (one per lane, launch_generation_request) and takes their sum + 1 as its tag
// (launch_generation_tag): larger than any tag before it.  Within a launch every workgroup sees the same sum: none can
// leave before all of them have passed the device-wide events, and they read the counters first thing.  (Publishing a
// generation word from the last workgroup to leave instead took that workgroup two dependent atomics, with their
// return values, at the very end of every launch.)
__device__ __forceinline__ int launch_generation_request(int* grp, int lane) {
    return counter_peek(group_counter(grp, kBarExit, lane % kEventGroups));
}
__device__ __forceinline__ int launch_generation_tag(int requested, int lane) {
    int v = lane < kEventGroups ? requested : 0;
    static_assert(kEventGroups == 16, "the sum below runs over sixteen lanes");
    v += __shfl_xor(v, 8, kWave);
    v += __shfl_xor(v, 4, kWave);
    v += __shfl_xor(v, 2, kWave);
    v += __shfl_xor(v, 1, kWave);
    return __builtin_amdgcn_readfirstlane(v) + 1;
}
__device__ __forceinline__ void launch_generation_leave(int* grp, int wg, int lane) {
    if (lane == 0) __hip_atomic_fetch_add(group_counter(grp, kBarExit, wg % kEventGroups), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

constexpr int kLayerFlagWgs = kEventGroups * kMailboxInts;
// (One 16-byte load per lane that goes past the caches like an agent-scope atomic load, as a single instruction: a buffer
// load with the sc1 bit, cache policy 16.  The descriptor is a raw buffer over the kLayerFlagWgs words; 0x00020000 is the
// data-format field of word 3 that gfx9 buffer descriptors of 32-bit elements carry.)
__device__ __forceinline__ bool flags_all_set(const int* flags, int nwg, int tag, int lane) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(flags), 0, kLayerFlagWgs * 4, 0x00020000);
    const u32x4 f = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16, 0, 16);
    const int i = lane * 4;
    const bool ok = (i >= nwg || (int)(f.x - (uint32_t)tag) >= 0) && (i + 1 >= nwg || (int)(f.y - (uint32_t)tag) >= 0) &&
                    (i + 2 >= nwg || (int)(f.z - (uint32_t)tag) >= 0) && (i + 3 >= nwg || (int)(f.w - (uint32_t)tag) >= 0);
    return __builtin_amdgcn_ballot_w64(!ok) == 0;
}
// The hand-over between two layers of one launch: every workgroup has its own flag word (the words are the group
// counters of kBarExit, which such a launch does not count in: kLayerFlagWgs workgroups at most) and stores its
// layer's tag there once its output rows are in memory; a waiting wave reads all the words with one load per lane
// until none is behind.  No counter has to be carried through the memory side's atomic units on the way from the last
// row stored to the first row read: two round trips less than an event.
__device__ __forceinline__ void layer_done_post(int* grp, int wg, int tag, int lane) {
    drain_memory_ops();
    if (lane == 0) st_agent(reinterpret_cast<uint32_t*>(group_counter(grp, kBarExit, 0)) + wg, (uint32_t)tag);
}
// (false: the wait expired; the status flag is raised)
__device__ __forceinline__ bool layer_done_wait(int* grp, int nwg, int tag, const StatusSink& status, int lane) {
    const int* flags = group_counter(grp, kBarExit, 0);
    int spins = 0;
    bool ok = true;
    while (!flags_all_set(flags, nwg, tag, lane)) {
        __builtin_amdgcn_s_sleep(2);
        if (++spins > kSpinLimit) {
            if (lane == 0) raise_status(status, kStatusSpin);
            ok = false;
            break;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return ok;
}

__device__ __forceinline__ StatusSink status_sink(const LayerParams& p) { return StatusSink{p.bar + kBarStatus, p.host_status}; }

// The number of valid cache rows S of this step.  A host-side length may equal the cache rows (the append is then
// skipped, k_new / v_new are still returned).  A device-side length, or RoPE tables indexed by the position
// (rope_stride > 0, one table row per cache row), need S < cache_rows: the step reads table row S and appends cache
// row S.  A device-side length must also stay within seq_cap, the bound the host sized the launches for (the grid of the
// attention items in split mode).  Anything else raises kStatusSeq; the step then runs on a clamped length without
// appending, so that no access leaves the caches or the tables, and its results mean nothing.
struct SeqLen { int S; bool ok; };
// The length in device memory is requested first thing in a kernel (seq_len_request; the word of the workspace that is
// read instead when there is none keeps the load unconditional: a conditional load is waited for where the branches join)
// and looked at where it is needed (seq_len_check).  Requested where it is needed, after the norm, it made every wave wait
// for one more memory round trip with its first weight tile already used up and nothing else in flight.
__device__ __forceinline__ int seq_len_request(const LayerParams& p) {
    const int* src = p.d_seq_len ? p.d_seq_len : p.bar;
    return *src;
}
__device__ __forceinline__ SeqLen seq_len_check(const LayerParams& p, int requested) {
    int S = p.d_seq_len ? requested : p.seq_len;
    int limit = (p.d_seq_len != nullptr || p.rope_stride > 0) ? p.cache_rows - 1 : p.cache_rows;
    if (p.d_seq_len != nullptr && p.seq_cap < limit) limit = p.seq_cap;
    const bool ok = S >= 0 && S <= limit;
    if (!ok) {
        if (threadIdx.x == 0 && blockIdx.x == 0) raise_status(status_sink(p), kStatusSeq);
        S = (S < 0 || limit < 0) ? 0 : limit;
    }
    return SeqLen{S, ok};
}
__device__ __forceinline__ SeqLen load_seq_len(const LayerParams& p) { return seq_len_check(p, seq_len_request(p)); }
// KV splits per head for a sequence length: about kSplitRows cache rows per item
__device__ __forceinline__ int effective_split(const LayerParams& p, int S) {
    int n = (S + kSplitRows - 1) / kSplitRows;
    n = n < 1 ? 1 : n;
    return n < p.max_split ? n : p.max_split;
}
// items of one head: the KV splits and the new token
__device__ __forceinline__ int items_per_head(int nsplit) { return nsplit + 1; }

// ------------------------------------------------------------------------------------------------
// stage A: LayerNorm shared by the workgroup, then row-per-wave streaming GEMV
// ------------------------------------------------------------------------------------------------
// The NW waves of a workgroup split the input row into 512-half chunks (chunk i belongs to wave i % NW):
// a wave loads its chunks of x and of the affine vectors, the chunk sums meet in LDS (mean, then
// variance, two-pass, fp32; chunk partials are added in chunk order, so the result does not depend on
// NW), and the normalised rows are left in LDS as packed fp16: slot 0 with the input LayerNorm's affine
// transform, slot 1 (if TWO) with the post-attention LayerNorm's, which shares the statistics because
// the residual is parallel (reference include/5090/pythia_2b8/kernel.cuh:811-818).  Every streaming wave
// then copies the row it needs into registers (lane l holds columns i*512 + 8l .. +8 of every chunk i;
// columns >= H are zero).  Letting every wave load the whole row itself makes a thousand waves ask for
// the same few cache lines at the same moment, which costs several microseconds at the start of a launch.
template <int NCH>
struct LnShared {
    float part[2][NCH];
    __attribute__((aligned(16))) half_t y[2][NCH * kChunk];
};
template <int NCH, int NW>
struct LnOwn {
    static constexpr int OWN = (NCH + NW - 1) / NW;
    u32x4 rx[OWN], ra[OWN], rw1[OWN], rb1[OWN], rw2[OWN], rb2[OWN];      // ra: the second input row (x_add), if there is one
};

// What the cooperative norm needs to know about its inputs.
struct NormSpec {
    const half_t *x, *x_add;        // input row; optional second row added to it (sum rounded to fp16)
    const half_t *w1, *b1, *w2, *b2;   // affine vectors of slot 0 and (TWO) slot 1; a null bias is zero, a null w2 skips slot 1
    int H, rms;                     // rms: RMSNorm (no mean subtraction) instead of LayerNorm
    float eps;
};
__device__ __forceinline__ NormSpec norm_spec(const LayerParams& p) {
    return NormSpec{p.x, p.x_add, p.ln_w, p.ln_b, p.ln2_w, p.ln2_b, p.H, p.norm_rms, p.eps};
}

// COH: the input rows were written earlier in this same launch by other workgroups (a launch that runs several layers):
// they are read past the caches, like everything else that crosses workgroups inside a launch.
template <int NCH, int NW, bool TWO, bool COH = false>
__device__ __forceinline__ void ln_coop_load(LnOwn<NCH, NW>& o, const NormSpec& ns, int wave, int lane) {
    const u32x4 z = {0u, 0u, 0u, 0u};
    auto row16 = [](const half_t* q) { if constexpr (COH) return ld_agent16(q); else return ld16(q); };
#pragma unroll
    for (int k = 0; k < LnOwn<NCH, NW>::OWN; ++k) {
        const int col = (wave + k * NW) * kChunk + lane * 8;
        const bool in = wave + k * NW < NCH && col < ns.H;
        o.rx[k] = in ? row16(ns.x + col) : z;
        o.rw1[k] = in ? ld16(ns.w1 + col) : z;
        o.rb1[k] = (in && ns.b1) ? ld16(ns.b1 + col) : z;
        if (TWO) {
            o.rw2[k] = (in && ns.w2) ? ld16(ns.w2 + col) : z;
            o.rb2[k] = (in && ns.b2) ? ld16(ns.b2 + col) : z;
        }
        // the second input row, if there is one, is only requested here (without one, the first is requested again and
        // dropped): adding it up right away would make the wave wait for both rows before anything else can be requested
        o.ra[k] = in ? row16((ns.x_add != nullptr ? ns.x_add : ns.x) + col) : z;
    }
}
// x <- fp16(x + x_add), as the reference's fused add + RMSNorm does (reference include/5090/llama/kernel_sglang.cuh:98-105).
// The sum is stored by stage C, once every workgroup has read both rows: x_sum_out may be x_add itself.
template <int NCH, int NW>
__device__ __forceinline__ void ln_coop_add(LnOwn<NCH, NW>& o, const NormSpec& ns) {
    if (ns.x_add == nullptr) return;
#pragma unroll
    for (int k = 0; k < LnOwn<NCH, NW>::OWN; ++k) {
        float a[8], b[8];
        unpack8(o.rx[k], a); unpack8(o.ra[k], b);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] += b[j];
        o.rx[k] = pack8(a);
    }
}

// Every wave of the workgroup must call this (workgroup barriers inside).
template <int NCH, int NW, bool TWO>
__device__ __forceinline__ void ln_coop_finish(LnOwn<NCH, NW>& o, const NormSpec& ns, LnShared<NCH>& sh, int wave, int lane) {
    constexpr int OWN = LnOwn<NCH, NW>::OWN;
    ln_coop_add<NCH, NW>(o, ns);
    const int H = ns.H;
    float mean = 0.f;
    if (!ns.rms) {
#pragma unroll
        for (int k = 0; k < OWN; ++k) {
            const int i = wave + k * NW;
            if (i < NCH) {
                float xv[8], s = 0.f;
                unpack8(o.rx[k], xv);     // lanes past H hold zeros
#pragma unroll
                for (int j = 0; j < 8; ++j) s += xv[j];
                s = wave_sum(s);
                if (lane == 0) sh.part[0][i] = s;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NCH; ++i) mean += sh.part[0][i];
        mean /= (float)H;
    }
#pragma unroll
    for (int k = 0; k < OWN; ++k) {
        const int i = wave + k * NW;
        if (i < NCH) {
            float xv[8], q = 0.f;
            unpack8(o.rx[k], xv);
            if (i * kChunk + lane * 8 < H) {
#pragma unroll
                for (int j = 0; j < 8; ++j) { const float d = xv[j] - mean; q = fmadd(d, d, q); }
            }
            q = wave_sum(q);
            if (lane == 0) sh.part[1][i] = q;
        }
    }
    __syncthreads();
    float var = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) var += sh.part[1][i];
    const float rstd = 1.0f / sqrtf(var / (float)H + ns.eps);
#pragma unroll
    for (int k = 0; k < OWN; ++k) {
        const int i = wave + k * NW;
        if (i < NCH) {
            const bool in = i * kChunk + lane * 8 < H;
            float xv[8], g[8], b[8], y[8];
            unpack8(o.rx[k], xv); unpack8(o.rw1[k], g); unpack8(o.rb1[k], b);
#pragma unroll
            for (int j = 0; j < 8; ++j) y[j] = in ? fmadd((xv[j] - mean) * rstd, g[j], b[j]) : 0.f;
            *reinterpret_cast<u32x4*>(&sh.y[0][i * kChunk + lane * 8]) = pack8(y);
            if (TWO) {
                unpack8(o.rw2[k], g); unpack8(o.rb2[k], b);
#pragma unroll
                for (int j = 0; j < 8; ++j) y[j] = in ? fmadd((xv[j] - mean) * rstd, g[j], b[j]) : 0.f;
                *reinterpret_cast<u32x4*>(&sh.y[1][i * kChunk + lane * 8]) = pack8(y);
            }
        }
    }
    __syncthreads();
}

// For waves of the workgroup that take no part in the norm (they hold other work in flight): the workgroup barriers
// of ln_coop_finish, nothing else.
__device__ __forceinline__ void ln_coop_bystander(const NormSpec& ns) {
    if (!ns.rms) __syncthreads();
    __syncthreads();
    __syncthreads();
}

// The normalised row of slot `which`, into the registers of this wave.
template <int NCH>
__device__ __forceinline__ void ln_fetch(const LnShared<NCH>& sh, int which, int lane, half2_t (&dst)[NCH][4]) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(&sh.y[which][i * kChunk + lane * 8]);
        dst[i][0] = as_h2(v.x); dst[i][1] = as_h2(v.y); dst[i][2] = as_h2(v.z); dst[i][3] = as_h2(v.w);
    }
    __builtin_amdgcn_sched_barrier(0);   // keep later weight loads from being scheduled above this point
}

// RPI weight rows of K = up to NCH*512 halfs held in registers.
template <int NCH, int RPI>
struct RowTile {
    u32x4 w[RPI][NCH];
    half_t bias;     // of the row that this lane stores after the wave's first segment of rows, requested with the first tile
                     // (row_bias_request; the functions that have no use for it leave it alone)
};

// The value that lane `lane` adds to the row it stores when a wave's parked rows are written out: requested together with
// the wave's first tile, because at the end of the rows it would be one more memory round trip, behind the tile already
// requested for the next pass, between the wave's last product and the event that other waves wait for.  `row` is clamped
// into [0, end); a null `b` reads `readable` instead (any readable device memory; the caller ignores the value).
__device__ __forceinline__ half_t row_bias_request(const half_t* __restrict__ b, const void* readable, int row, int end) {
    const half_t* __restrict__ src = b != nullptr ? b : reinterpret_cast<const half_t*>(readable);
    int r = row < end ? row : end - 1;
    r = r > 0 ? r : 0;
    return src[r];
}

// Issue the loads of rows r, r+stride, ... (RPI of them; rows >= nrows repeat row r).  EXACT: K ==
// NCH*512, every lane load is in range; otherwise out-of-range lane loads are redirected to column 0
// (their activation registers are zero, so they add nothing).
template <int NCH, int RPI, bool EXACT>
__device__ __forceinline__ void load_row_tile(RowTile<NCH, RPI>& t, const half_t* __restrict__ W, int K, int r, int stride,
                                              int nrows, int lane) {
    const int colb = lane * 8;
#pragma unroll
    for (int j = 0; j < RPI; ++j) {
        int rr = r + j * stride;
        rr = rr < nrows ? rr : r;
        const half_t* rp = W + (size_t)rr * (size_t)K;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (EXACT) {
                // scalar base per group of four chunks + one lane offset + immediate: the 13-bit immediate
                // of a global load reaches 4 KB, and per-chunk lane offsets would cost registers
                const half_t* gp = rp + (i / 4) * (4 * kChunk);
                t.w[j][i] = ld_stream16(gp + colb + (i % 4) * kChunk);
            } else {
                const int c = i * kChunk + colb;
                t.w[j][i] = ld_stream16(rp + (c < K ? c : 0));
            }
        }
    }
}

// The first tile of a wave's row range, requested ahead of something slow (a norm, an event) WITHOUT a branch around the
// loads: a wave that has no tile requests row 0 (and drops it).  With `if (ntiles > 0)` around them, the compiler's
// wait-count bookkeeping takes the shorter path at the join behind the branch: the next wait for anything older
// (the norm's inputs) then waits for the whole tile as well.
template <int NCH, int RPI, bool EXACT>
__device__ __forceinline__ void prefetch_row_tile(RowTile<NCH, RPI>& t, const half_t* __restrict__ W, int K, int first, int stride,
                                                  int end, int ntiles, int lane) {
    const bool any = ntiles > 0;
    load_row_tile<NCH, RPI, EXACT>(t, W, K, any ? first : 0, stride, any ? end : 1, lane);
}

// chunk i of the weight row at rp (same addressing as load_row_tile)
template <int NCH, bool EXACT>
__device__ __forceinline__ u32x4 load_row_chunk(const half_t* __restrict__ rp, int K, int i, int colb) {
    if (EXACT) return ld_stream16(rp + (i / 4) * (4 * kChunk) + colb + (i % 4) * kChunk);
    const int c = i * kChunk + colb;
    return ld_stream16(rp + (c < K ? c : 0));
}

// Dot products of a wave's rows are parked in LDS (one float per row, written by lane 0) and written to
// global memory after the streaming loop, one row per lane: a global store inside the loop would share
// the vmcnt counter with the weight loads, and with loads and stores both pending the compiler has to
// wait for everything, which empties the load pipeline once per tile.
constexpr int kParkRows = 64;
struct RowPark {
    float* slot;    // this wave's kParkRows floats in LDS
    int n;          // rows parked so far
};

template <int NCH, int RPI>
__device__ __forceinline__ void finish_row_tile(const RowTile<NCH, RPI>& t, const half2_t (&x)[NCH][4], int valid, int lane,
                                                RowPark& park) {
#pragma unroll
    for (int j = 0; j < RPI; ++j) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) acc = dot8(t.w[j][i], x[i], acc);
        acc = wave_sum(acc);
        if (j < valid) {
            if (lane == 0) park.slot[park.n] = acc;
            park.n += 1;
        }
    }
}

// The same for a full tile that is not the wave's last: every register of the tile is refilled with the same chunk of
// tile `nr` (rows nr + j*stride; rows >= nrows repeat row nr) right after it has been used, so the wave has one tile
// in flight at all times and never a burst of two.
template <int NCH, int RPI, bool EXACT>
__device__ __forceinline__ void finish_refill_row_tile(RowTile<NCH, RPI>& t, const half2_t (&x)[NCH][4], int lane, RowPark& park,
                                                       const half_t* __restrict__ W, int K, int nr, int stride, int nrows) {
    const int colb = lane * 8;
#pragma unroll
    for (int j = 0; j < RPI; ++j) {
        int rr = nr + j * stride;
        rr = rr < nrows ? rr : nr;
        const half_t* rp = W + (size_t)rr * (size_t)K;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            acc = dot8(t.w[j][i], x[i], acc);
            t.w[j][i] = load_row_chunk<NCH, EXACT>(rp, K, i, colb);
        }
        acc = wave_sum(acc);
        if (lane == 0) park.slot[park.n] = acc;
        park.n += 1;
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Tiles t = 0 .. ntiles-1 of one wave: tile t covers rows row_of(t) + j*stride_in_tile, j < RPI (rows >=
// nrows do not exist).  Two tiles are in flight: the loads of the next tile are issued before the current
// one is reduced.  `pre` already holds the loads of tile 0 (issued by the caller before something slow:
// the LayerNorm prologue or a barrier).  The loop body is free of branches, because a conditional load
// makes the compiler's wait-count bookkeeping assume the shorter path and drain the pipeline at every
// tile; the last one or two tiles of a segment are peeled off behind the loop instead, so that no tile is
// ever loaded twice.
// The tiles are processed in segments of kParkRows rows; `flush(park, first_index)` runs after each
// segment, outside the streaming loop (no global store may sit inside it, see RowPark), with the first
// tile of the next segment already in flight; parked value k (counting from first_index) belongs to the
// k-th row this wave finished.
// tiles per flush segment: even, so a segment is a whole number of loop trips
template <int RPI> constexpr int park_seg_tiles() { return (kParkRows / RPI) & ~1; }
template <int NCH, int RPI, bool EXACT, bool ROLL = false, class RowOf, class Flush>
__device__ __forceinline__ void gemv_tiles(const half_t* __restrict__ W, int K, int nrows, int stride_in_tile, int ntiles,
                                           RowOf&& row_of, const half2_t (&x)[NCH][4], int lane, RowTile<NCH, RPI>& pre,
                                           RowPark& park, Flush&& flush) {
    constexpr int kSegTiles = park_seg_tiles<RPI>();
    static_assert(kSegTiles >= 2, "tile larger than the park");
    auto valid_rows = [&](int t) {   // only the last tile of a wave can be short
        int v = 0;
        const int r = row_of(t);
#pragma unroll
        for (int j = 0; j < RPI; ++j) v += (r + j * stride_in_tile < nrows) ? 1 : 0;
        return v;
    };
    auto load = [&](RowTile<NCH, RPI>& t, int i) { load_row_tile<NCH, RPI, EXACT>(t, W, K, row_of(i), stride_in_tile, nrows, lane); };
    int done = 0;
    if (ROLL) {
        for (int seg = 0; seg < ntiles; seg += kSegTiles) {
            const int seg_end = seg + kSegTiles < ntiles ? seg + kSegTiles : ntiles;
            for (int t = seg; t + 1 < seg_end; ++t)
                finish_refill_row_tile<NCH, RPI, EXACT>(pre, x, lane, park, W, K, row_of(t + 1), stride_in_tile, nrows);
            if (seg_end < ntiles) finish_refill_row_tile<NCH, RPI, EXACT>(pre, x, lane, park, W, K, row_of(seg_end), stride_in_tile, nrows);
            else finish_row_tile<NCH, RPI>(pre, x, valid_rows(seg_end - 1), lane, park);
            __builtin_amdgcn_sched_barrier(0);
            flush(park, done);
            done += park.n;
            park.n = 0;
        }
        return;
    }
    for (int seg = 0; seg < ntiles; seg += kSegTiles) {
        const int seg_end = seg + kSegTiles < ntiles ? seg + kSegTiles : ntiles;
        RowTile<NCH, RPI> other;
        int t = seg;
        for (; t + 2 < seg_end; t += 2) {     // tiles t+1 and t+2 exist and are full
            load(other, t + 1);
            finish_row_tile<NCH, RPI>(pre, x, RPI, lane, park);
            __builtin_amdgcn_sched_barrier(0);   // a third tile's loads must not be scheduled above this point
            load(pre, t + 2);
            finish_row_tile<NCH, RPI>(other, x, RPI, lane, park);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (t + 1 < seg_end) {
            load(other, t + 1);
            finish_row_tile<NCH, RPI>(pre, x, RPI, lane, park);
            __builtin_amdgcn_sched_barrier(0);
            if (seg_end < ntiles) load(pre, seg_end);
            finish_row_tile<NCH, RPI>(other, x, valid_rows(t + 1), lane, park);
        } else {
            finish_row_tile<NCH, RPI>(pre, x, valid_rows(t), lane, park);
            if (seg_end < ntiles) load(pre, seg_end);
        }
        __builtin_amdgcn_sched_barrier(0);
        flush(park, done);
        done += park.n;
        park.n = 0;
    }
}

// ---- dynamically shared tiles ---------------------------------------------------------------------
// Compute units do not stream at the same speed (whole chiplets differ by tens of percent, differently
// from machine to machine), so equal static shares leave the fast ones waiting for the slowest.  A team
// of `nw` waves (the streaming waves of kTeamWgs consecutive workgroups, which the dispatcher places on
// different chiplets) therefore shares the `ntiles` tiles of a row range: wave j starts with tiles j and
// j + nw, and every further tile is a ticket from the team's counter, requested two tiles ahead of its use
// (the atomic is issued before the loads of the tile in between, so its result is back before theirs).
// Every wave ends with exactly one ticket past the end, so a team issues max(ntiles - 2 nw, 0) + nw
// requests per pass; the wave that gets the last of them zeroes the counter for the next launch.
constexpr int kTeamWgs = 8;
struct TileTeam {
    int* counter;      // the team's ticket counter (own 64-byte line), zero between launches
    int j, nw;         // this wave's index in the team, waves in the team
    int row0;          // first row of the team's range
    int ntiles;        // tiles (of RPI adjacent rows) in the range
    int end;           // rows >= end do not exist
};
struct RowParkIds {
    float* slot;       // this wave's kParkRows floats in LDS
    int* row;          // and the rows they belong to (-1: none)
    int n;
};
__device__ __forceinline__ int ticket_request(int* counter, int lane) {
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return old;     // meaningful in lane 0; read with first_lane() when needed
}
template <int NCH, int RPI>
__device__ __forceinline__ void finish_team_tile(const RowTile<NCH, RPI>& t, const half2_t (&x)[NCH][4], int row, int end, int lane,
                                                 RowParkIds& park) {
#pragma unroll
    for (int j = 0; j < RPI; ++j) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) acc = dot8(t.w[j][i], x[i], acc);
        acc = wave_sum(acc);
        if (lane == 0) {
            park.slot[park.n + j] = acc;
            park.row[park.n + j] = row + j < end ? row + j : -1;
        }
    }
    park.n += RPI;
}
template <int NCH, int RPI, bool EXACT>
__device__ __forceinline__ void finish_refill_team_tile(RowTile<NCH, RPI>& t, const half2_t (&x)[NCH][4], int row, int end, int lane,
                                                        RowParkIds& park, const half_t* __restrict__ W, int K, int nr) {
    const int colb = lane * 8;
#pragma unroll
    for (int j = 0; j < RPI; ++j) {
        const int rr = nr + j < end ? nr + j : nr;
        const half_t* rp = W + (size_t)rr * (size_t)K;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            acc = dot8(t.w[j][i], x[i], acc);
            t.w[j][i] = load_row_chunk<NCH, EXACT>(rp, K, i, colb);
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            park.slot[park.n + j] = acc;
            park.row[park.n + j] = row + j < end ? row + j : -1;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    park.n += RPI;
}
// team_prefetch requests the wave's first ticket and its two static tiles (before something slow: the
// LayerNorm, an event); gemv_team consumes them.  flush(park) runs outside the streaming loop, when the
// park is full and at the end; parked value k belongs to row park.row[k].
constexpr int kTeamBiasRegs = 4;       // a team's rows of a pass whose biases its waves hold: 64 per register
template <int NCH, int RPI>
struct TeamTiles {
    RowTile<NCH, RPI> a, b;
    int req;
    half_t bias[kTeamBiasRegs];        // lane l, register k: the bias of row tm.row0 + 64 k + l (team_bias_held)
};
// A wave cannot know which rows of the team's range it will get, so it requests the biases of all of them (when the
// range is short enough), one row per lane and register, and picks its rows' values from the lanes that hold them when
// it stores them (team_bias).  For the reason see row_bias_request.
template <int RPI>
__device__ __forceinline__ bool team_bias_held(const TileTeam& tm) { return tm.ntiles * RPI <= 64 * kTeamBiasRegs; }
template <int NCH, int RPI>
__device__ __forceinline__ float team_bias(const TileTeam& tm, const TeamTiles<NCH, RPI>& tt, const half_t* __restrict__ b, int row,
                                           bool valid) {
    if (team_bias_held<RPI>(tm)) {          // the same for the whole wave
        const int rel = valid ? row - tm.row0 : 0;
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < kTeamBiasRegs; ++k) {
            const int got = __builtin_amdgcn_ds_bpermute((rel & 63) << 2, (int)__builtin_bit_cast(unsigned short, tt.bias[k]));
            if ((rel >> 6) == k) v = (float)__builtin_bit_cast(half_t, (unsigned short)got);
        }
        return v;
    }
    return valid ? (float)b[row] : 0.f;
}
template <int NCH, int RPI, bool EXACT>
__device__ __forceinline__ void team_prefetch(const half_t* __restrict__ W, int K, const TileTeam& tm, int lane,
                                              TeamTiles<NCH, RPI>& tt, const half_t* __restrict__ bias) {
    tt.req = ticket_request(tm.counter, lane);
    if (tm.j < tm.ntiles) load_row_tile<NCH, RPI, EXACT>(tt.a, W, K, tm.row0 + tm.j * RPI, 1, tm.end, lane);
#pragma unroll
    for (int k = 0; k < kTeamBiasRegs; ++k) tt.bias[k] = row_bias_request(bias, W, tm.row0 + 64 * k + lane, tm.end);
}
template <int NCH, int RPI, bool EXACT, bool ROLL = false, class Flush>
__device__ __forceinline__ void gemv_team(const half_t* __restrict__ W, int K, const TileTeam& tm, const half2_t (&x)[NCH][4],
                                          int lane, TeamTiles<NCH, RPI>& tt, RowParkIds& park, Flush&& flush) {
    static_assert(kParkRows >= 3 * RPI, "tile larger than the park");
    const int total = (tm.ntiles > 2 * tm.nw ? tm.ntiles - 2 * tm.nw : 0) + tm.nw;    // requests per pass
    auto row_of = [&](int t) { return tm.row0 + t * RPI; };
    auto load = [&](RowTile<NCH, RPI>& t, int i) { load_row_tile<NCH, RPI, EXACT>(t, W, K, row_of(i), 1, tm.end, lane); };
    auto retire = [&](int old) {      // the team's last request re-arms the counter
        if (lane == 0 && old == total - 1) __hip_atomic_store(tm.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    int req = tt.req;
    int tA = tm.j, tB = tm.j + tm.nw;
    if (tA >= tm.ntiles) {            // nothing for this wave: its one request is past the end
        retire(req);
        return;
    }
    if (tB >= tm.ntiles) {            // one tile only
        finish_team_tile<NCH, RPI>(tt.a, x, row_of(tA), tm.end, lane, park);
        retire(req);
        flush(park);
        park.n = 0;
        return;
    }
    if (ROLL) {
        // one tile in flight: tt.a holds tile tA and is refilled with tile tN while it is used; the ticket for the tile
        // after tN was requested before tN's loads, so it is back before they are
        int tN = tB;
        bool more = true;
        while (more) {
            while (park.n + 2 * RPI <= kParkRows) {
                if (tN < 0) {
                    finish_team_tile<NCH, RPI>(tt.a, x, row_of(tA), tm.end, lane, park);
                    more = false;
                    break;
                }
                finish_refill_team_tile<NCH, RPI, EXACT>(tt.a, x, row_of(tA), tm.end, lane, park, W, K, row_of(tN));
                tA = tN;
                const int old = first_lane(req);
                const int tn = 2 * tm.nw + old;
                if (tn >= tm.ntiles) {
                    retire(old);
                    tN = -1;
                } else {
                    tN = tn;
                    req = ticket_request(tm.counter, lane);
                }
            }
            flush(park);
            park.n = 0;
        }
        return;
    }
    load(tt.b, tB);
    bool more = true;
    while (more) {
        // the streaming loop: no stores, no conditional loads; it is left when the tickets run out or the
        // park is full
        while (park.n + 3 * RPI <= kParkRows) {     // a trip parks up to three tiles
            finish_team_tile<NCH, RPI>(tt.a, x, row_of(tA), tm.end, lane, park);
            int old = first_lane(req);
            int tn = 2 * tm.nw + old;
            if (tn >= tm.ntiles) {
                retire(old);
                finish_team_tile<NCH, RPI>(tt.b, x, row_of(tB), tm.end, lane, park);
                more = false;
                break;
            }
            req = ticket_request(tm.counter, lane);
            load(tt.a, tn);
            tA = tn;
            __builtin_amdgcn_sched_barrier(0);
            finish_team_tile<NCH, RPI>(tt.b, x, row_of(tB), tm.end, lane, park);
            old = first_lane(req);
            tn = 2 * tm.nw + old;
            if (tn >= tm.ntiles) {
                retire(old);
                finish_team_tile<NCH, RPI>(tt.a, x, row_of(tA), tm.end, lane, park);
                more = false;
                break;
            }
            req = ticket_request(tm.counter, lane);
            load(tt.b, tn);
            tB = tn;
            __builtin_amdgcn_sched_barrier(0);
        }
        flush(park);
        park.n = 0;
    }
}

template <int NCH>
struct StageARpi { static constexpr int value = (16 / NCH) > 0 ? (16 / NCH) : 1; };

// ------------------------------------------------------------------------------------------------
// stage B: split-KV single-query attention, one wave per (head, split) item
// ------------------------------------------------------------------------------------------------
// NeoX rotate-half RoPE on the first `rot` dims of a head vector held in raw fp32 scratch
// (reference include/5090/pythia_2b8/kernel.cuh:395-421): d < rot/2 -> v[d] cos[d] - v[d+rot/2] sin[d];
// rot/2 <= d < rot -> v[d] cos[d] + v[d-rot/2] sin[d]; d >= rot passes through.
// A lane produces dims d0 .. d0+7.  rope_coeffs fetches cos and the signed sin of those dims (1 and 0 for
// dims >= rot): they do not depend on the layer's own results, so they can be requested early.
// rope_load8 requests the lane's own values and their rotation partners together (one memory round trip).
// PAIRS: dim d rotates with d +- rot/2 (false, NeoX) or with its neighbour d ^ 1 (true, GPT-J: even dims take
// -sin, odd dims +sin, and the tables are indexed by the dim itself; reference include/5090/llama/kernel.cuh:280-313).
// Rotate-half tables come in two shapes.  The Pythia ops read cos[d] / sin[d] for every d < rot (reference
// include/5090/pythia_2b8/kernel.cuh:395-399): the two halves of the table need not repeat, and the reference's
// own unit test draws an independent angle per entry (tests/test_pythia.py:24-42).  The sglang LLaMA ops hold only
// the rot/2 angles of the pairs and read entry d mod rot/2 (reference include/5090/llama/kernel_sglang.cuh:292-293):
// `half_table`.
struct RopeCoeffs { float c[8], sg[8]; };
template <bool PAIRS = false>
__device__ __forceinline__ void rope_coeffs(int d0, int rot, const float* __restrict__ cs, const float* __restrict__ sn,
                                            bool act, bool half_table, const float* __restrict__ readable, RopeCoeffs& rc) {
    // Every lane loads all sixteen values, whether it needs them or not (a lane or dim without rotation reads entry 0,
    // a geometry without rotation reads `readable`, any readable device memory): loads under a condition would each
    // be waited for where their branch ends, one memory round trip after the other.
    const int hr = rot >> 1;
    const float* __restrict__ c0 = rot > 0 ? cs : readable;
    const float* __restrict__ s0 = rot > 0 ? sn : readable;
    float cv[8], sv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int d = d0 + j;
        const bool rotd = act && d < rot;
        const int t = PAIRS ? d : ((half_table && d >= hr) ? d - hr : d);
        const int ti = rotd ? t : 0;
        cv[j] = c0[ti];
        sv[j] = s0[ti];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int d = d0 + j;
        const bool rotd = act && d < rot;
        rc.c[j] = rotd ? cv[j] : 1.f;
        if (PAIRS) rc.sg[j] = rotd ? ((d & 1) ? sv[j] : -sv[j]) : 0.f;
        else rc.sg[j] = rotd ? (d < hr ? -sv[j] : sv[j]) : 0.f;
    }
}
// The raw values of a lane's eight dims and of their rotation partners: rope_request issues the loads, rope_finish
// rotates.  Requests for several vectors (q and k of the new token) issued back to back share one memory round trip.
struct RopeRaw { float a[8], pr[8]; };
template <bool PAIRS = false>
__device__ __forceinline__ void rope_request(const float* __restrict__ v, int d0, int rot, bool act, RopeRaw& r) {
    const int hr = rot >> 1;
    if (act) {
        ld_agent2(v + d0, r.a[0], r.a[1]); ld_agent2(v + d0 + 2, r.a[2], r.a[3]);
        ld_agent2(v + d0 + 4, r.a[4], r.a[5]); ld_agent2(v + d0 + 6, r.a[6], r.a[7]);
        if (!PAIRS) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int d = d0 + j;
                const int pd = d < rot ? (d < hr ? d + hr : d - hr) : d;
                r.pr[j] = ld_agent(v + pd);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) { r.a[j] = 0.f; r.pr[j] = 0.f; }
    }
}
template <bool PAIRS = false>
__device__ __forceinline__ void rope_finish(const RopeRaw& r, int d0, int rot, const RopeCoeffs& rc, bool act, float (&out)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float pr = PAIRS ? r.a[j ^ 1] : r.pr[j];          // GPT-J: the neighbour is one of the lane's own eight dims
        out[j] = act ? (d0 + j < rot ? fmadd(r.a[j], rc.c[j], pr * rc.sg[j]) : r.a[j]) : 0.f;
    }
}
__device__ __forceinline__ void raw_load8(const float* __restrict__ v, int d0, bool act, float (&out)[8]) {
    if (act) {
        ld_agent2(v + d0, out[0], out[1]); ld_agent2(v + d0 + 2, out[2], out[3]);
        ld_agent2(v + d0 + 4, out[4], out[5]); ld_agent2(v + d0 + 6, out[6], out[7]);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) out[j] = 0.f;
    }
}

// A head's attention is split into nsplit items over its cache rows plus one item for the new token (item index
// nsplit: it rotates and returns the new K / V row, appends it, and contributes the new token's score and value);
// attn_items_per_head = nsplit + 1 partial results meet in the merge.  Keeping the new token out of the cache items
// makes them all alike: the one that used to carry it needed a second dependent memory round trip and ended last.
// (The batched kernel, PAGED, keeps the new token in split 0, with its k and v requested together with q: it has a few
// splits per head only, sized to fill the device exactly once, and an extra item per head would start a second round.)
// One cache item: the wave's four 16-lane groups take cache rows begin+g, begin+g+4, ...; lane
// `sub` of a group holds dims 8 sub .. 8 sub + 7 of its row (lanes with 8 sub >= D contribute nothing).
// A tile is kAttnT rows per group (32 rows per wave).  An item is a chain of dependent memory round
// trips, so everything that does not depend on this layer's QKV rows is requested ahead of them by
// attn_prefetch: the first two K/V tiles and the RoPE coefficients.  In the fused kernel that happens while
// the attention waves would otherwise sit waiting for the QKV rows.
constexpr int kAttnT = 8;
constexpr int kAttnTileRows = 4 * kAttnT;
struct KvTile { u32x4 k[kAttnT], v[kAttnT]; };
struct KvRows { int r[kAttnT]; };     // paged caches: the cache rows of a tile's kAttnT rows of this lane's group
struct AttnItem {
    int head, sp, nsplit, S, begin, end, ntiles;
    bool append_ok;     // the sequence length was valid: split 0 may append the new row
    KvTile t0, t1;
    KvRows r0, r1;      // PAGED: page-table entries of the tiles that t0 / t1 take next
    RopeCoeffs rc;
};
// PAGED: the page-table entries of tile i (rows past the end repeat the last row, tiles past the end as well).  They
// are requested two tiles before the K/V rows they address, so that a tile costs one memory round trip, not two.
__device__ __forceinline__ void attn_request_rows(const LayerParams& p, const AttnItem& it, KvRows& rows, int i, int lane) {
    const int r = it.begin + i * kAttnTileRows + (lane >> 4);
#pragma unroll
    for (int t = 0; t < kAttnT; ++t) rows.r[t] = p.kv_rows[min(r + t * 4, it.end - 1)];
}
__device__ __forceinline__ void attn_load_tile_rows(const LayerParams& p, const AttnItem& it, KvTile& kv, const KvRows& rows, int lane) {
    const int sub = lane & 15;
    const int d0 = sub * 8 < p.D ? sub * 8 : 0;
    const half_t* __restrict__ kc = p.k_cache + (size_t)it.head * p.D + d0;
    const half_t* __restrict__ vc = p.v_cache + (size_t)it.head * p.D + d0;
#pragma unroll
    for (int t = 0; t < kAttnT; ++t) {
        kv.k[t] = ld16(kc + (size_t)rows.r[t] * p.H);
        kv.v[t] = ld16(vc + (size_t)rows.r[t] * p.H);
    }
}
// tile i of the item; rows past the end re-read the last row (masked when used): no conditional loads
// PAGED: rows go through p.kv_rows
template <bool PAGED = false>
__device__ __forceinline__ void attn_load_tile(const LayerParams& p, const AttnItem& it, KvTile& kv, int i, int lane) {
    const int grp = lane >> 4, sub = lane & 15;
    const int d0 = sub * 8 < p.D ? sub * 8 : 0;      // idle lanes read (and ignore) the first dims
    const half_t* __restrict__ kc = p.k_cache + (size_t)it.head * p.D + d0;
    const half_t* __restrict__ vc = p.v_cache + (size_t)it.head * p.D + d0;
    const int r = it.begin + i * kAttnTileRows + grp;
#pragma unroll
    for (int t = 0; t < kAttnT; ++t) {
        int row = (r + t * 4 < it.end) ? r + t * 4 : it.end - 1;
        if (PAGED) row = p.kv_rows[row];
        kv.k[t] = ld16(kc + (size_t)row * p.H);
        kv.v[t] = ld16(vc + (size_t)row * p.H);
    }
}
template <bool PAGED = false, bool PAIRS = false>
__device__ __forceinline__ void attn_prefetch(const LayerParams& p, AttnItem& it, int head, int sp, int nsplit, SeqLen sl, int lane) {
    const int S = sl.S;
    it.head = head; it.sp = sp; it.nsplit = nsplit; it.S = S; it.append_ok = sl.ok;
    const int chunk = (S + nsplit - 1) / nsplit;
    it.begin = sp < nsplit ? sp * chunk : S;          // item nsplit (if it exists) is the new token: no cache rows
    it.end = (it.begin + chunk < S) ? it.begin + chunk : S;
    it.ntiles = it.begin < it.end ? (it.end - it.begin + kAttnTileRows - 1) / kAttnTileRows : 0;
    // the coefficients first: what waits for them then does not wait for the tiles as well
    const int sub = lane & 15;
    const bool act = sub * 8 < p.D;
    const float* __restrict__ cs = p.cos + (size_t)S * p.rope_stride;   // stride 0: the row is the position
    const float* __restrict__ sn = p.sin + (size_t)S * p.rope_stride;
    rope_coeffs<PAIRS>(act ? sub * 8 : 0, p.rot, cs, sn, act, p.rope_half_table != 0, p.qkv_raw, it.rc);
    if (PAGED) {
        if (it.ntiles > 0) {
            attn_request_rows(p, it, it.r0, 0, lane);
            attn_request_rows(p, it, it.r1, 1, lane);
            attn_load_tile_rows(p, it, it.t0, it.r0, lane);
            attn_load_tile_rows(p, it, it.t1, it.r1, lane);
            attn_request_rows(p, it, it.r0, 2, lane);
            attn_request_rows(p, it, it.r1, 3, lane);
        }
    } else {
        if (it.ntiles > 0) attn_load_tile<PAGED>(p, it, it.t0, 0, lane);
        if (it.ntiles > 1) attn_load_tile<PAGED>(p, it, it.t1, 1, lane);
    }
}

// nwg_to_signal > 0 (fused kernel): a completed head counts towards the kBarHeads event of that many workgroups.
// The partial result of an item whose head is merged inside the workgroup (AttnLdsPart, one per wave): the dims of lane
// group 0 after the merge of the wave's four groups, and the softmax state.
struct AttnLdsPart { float acc[128]; float m, l; };
template <bool PAGED = false, bool PAIRS = false>
__device__ __forceinline__ void attention_item(const LayerParams& p, AttnItem& it, int lane, int nwg_to_signal, int tag,
                                               AttnLdsPart* lds_part = nullptr) {
    const int grp = lane >> 4, sub = lane & 15;
    const int D = p.D, H = p.H;
    const int head = it.head, sp = it.sp, nsplit = it.nsplit, S = it.S, end = it.end;
    const bool act = sub * 8 < D;
    const int d0 = act ? sub * 8 : 0;
    const float* __restrict__ raw = p.qkv_raw + (size_t)head * p.qkv_head_stride;

    const RopeCoeffs& rc = it.rc;
    float m = kNegBig, l = 0.f, acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    float q[8];
    constexpr bool OWN_ITEM = !PAGED;       // the new token is item nsplit of its head; otherwise split 0 carries it
    // q, k and v of this step for the wave that handles the new token, requested together (one round trip); group 0
    // does the work: rotates, returns and appends the new row, and seeds its softmax state with the new token
    // (every group gets its unscaled q from the same request)
    auto new_token = [&]() {
        RopeRaw rq, rk;
        float vf[8], kf[8];
        const bool on = act && grp == 0;
        rope_request<PAIRS>(raw, d0, p.rot, act, rq);
        rope_request<PAIRS>(raw + p.qkv_k_off, d0, p.rot, on, rk);
        raw_load8(raw + p.qkv_v_off, d0, on, vf);
        rope_finish<PAIRS>(rq, d0, p.rot, rc, act, q);
        rope_finish<PAIRS>(rk, d0, p.rot, rc, on, kf);
        const u32x4 kp = pack8(kf), vp = pack8(vf);
        unpack8(kp, kf); unpack8(vp, vf);      // attend over the fp16 values the cache will hold
        if (on) {
            const size_t o = (size_t)head * D + d0;
            *reinterpret_cast<u32x4*>(p.k_new + o) = kp;
            *reinterpret_cast<u32x4*>(p.v_new + o) = vp;
            if (PAGED) {
                if (p.append_kv && it.append_ok) {
                    const size_t slot = (size_t)p.kv_rows[S];
                    *reinterpret_cast<u32x4*>(p.k_cache + slot * H + o) = kp;
                    *reinterpret_cast<u32x4*>(p.v_cache + slot * H + o) = vp;
                }
            } else if (p.append_kv && it.append_ok && S < p.cache_rows) {
                *reinterpret_cast<u32x4*>(p.k_cache + (size_t)S * H + o) = kp;
                *reinterpret_cast<u32x4*>(p.v_cache + (size_t)S * H + o) = vp;
            }
        }
        if (grp == 0) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) s = fmadd(q[j] * p.qscale, kf[j], s);
            s = row16_sum(s);
            m = s; l = 1.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = vf[j];
        }
    };
    if (OWN_ITEM && sp == nsplit) {
        new_token();
    } else {
        if (!OWN_ITEM && sp == 0) {
            new_token();          // split 0 of the batched kernel carries the new token
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] *= p.qscale;
        } else {
            RopeRaw rq;
            rope_request<PAIRS>(raw, d0, p.rot, act, rq);
            rope_finish<PAIRS>(rq, d0, p.rot, rc, act, q);
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] *= p.qscale;
        }

        trace_value(p, 8, wall_clock64() + (long long)(__builtin_bit_cast(unsigned, q[0]) & 0u));      // q is back and rotated
        auto process = [&](const KvTile& kv, int i) {
            const int r = it.begin + i * kAttnTileRows + grp;
            float s[kAttnT], mt = m;
#pragma unroll
            for (int t = 0; t < kAttnT; ++t) {
                float kf[8];
                unpack8(kv.k[t], kf);
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) d = fmadd(q[j], kf[j], d);
                d = row16_sum(d);
                s[t] = (r + t * 4 < end) ? d : kNegBig;
                mt = fmaxf(mt, s[t]);
            }
            const float alpha = fast_exp2(m - mt);
            l *= alpha;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] *= alpha;
#pragma unroll
            for (int t = 0; t < kAttnT; ++t) {
                const float pt = (r + t * 4 < end) ? fast_exp2(s[t] - mt) : 0.f;
                float vf[8];
                unpack8(kv.v[t], vf);
                l += pt;
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmadd(pt, vf[j], acc[j]);
            }
            m = mt;
        };
        if (PAGED) {
            // Items of a batched launch can be long: two tiles in flight all the way, and the page-table entries of the
            // two after them.  No branch in the loop (a tile past the end repeats the item's last row and is masked
            // where it is used), so that no wait covers more than the tile it is for.
            for (int i = 0; i < it.ntiles; i += 2) {
                process(it.t0, i);
                __builtin_amdgcn_sched_barrier(0);
                attn_load_tile_rows(p, it, it.t0, it.r0, lane);
                attn_request_rows(p, it, it.r0, i + 4, lane);
                __builtin_amdgcn_sched_barrier(0);
                process(it.t1, i + 1);
                __builtin_amdgcn_sched_barrier(0);
                attn_load_tile_rows(p, it, it.t1, it.r1, lane);
                attn_request_rows(p, it, it.r1, i + 5, lane);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            if (it.ntiles > 0) process(it.t0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (it.ntiles > 2) attn_load_tile<PAGED>(p, it, it.t0, 2, lane);     // the third tile travels while the second is reduced
            __builtin_amdgcn_sched_barrier(0);
            if (it.ntiles > 1) process(it.t1, 1);
            __builtin_amdgcn_sched_barrier(0);
            for (int i = 2; i < it.ntiles; ++i) {
                if (i != 2) attn_load_tile<PAGED>(p, it, it.t0, i, lane);
                process(it.t0, i);
            }
        }
    }

    // merge the four groups (lanes sub, sub+16, sub+32, sub+48 hold the same dims)
    {
        float mw = fmaxf(m, xor_shfl(m, 16));
        mw = fmaxf(mw, xor_shfl(mw, 32));
        const float sc = fast_exp2(m - mw);
        l *= sc;
        l += xor_shfl(l, 16);
        l += xor_shfl(l, 32);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float a = acc[j] * sc;
            a += xor_shfl(a, 16);
            a += xor_shfl(a, 32);
            acc[j] = a;
        }
        m = mw;
    }
    if (lds_part != nullptr) {
        // the splits of this head run in this workgroup: the partial goes to LDS, the caller merges behind a barrier
        if (grp == 0 && act) {
#pragma unroll
            for (int j = 0; j < 8; ++j) lds_part->acc[d0 + j] = acc[j];
            if (sub == 0) { lds_part->m = m; lds_part->l = l; }
        }
        return;
    }
    // publish the partial of this (head, split)
    const size_t item = (size_t)head * kMaxSplit + sp;
    if (grp == 0 && act) {
        float* dst = p.part_acc + item * D + d0;
        st_agent2(dst, acc[0], acc[1]); st_agent2(dst + 2, acc[2], acc[3]);
        st_agent2(dst + 4, acc[4], acc[5]); st_agent2(dst + 6, acc[6], acc[7]);
        if (sub == 0) st_agent2(p.part_ml + item * 2, m, l);
    }
    drain_memory_ops();
    int last = 0;
    const int nparts = OWN_ITEM ? nsplit + 1 : nsplit;      // the cache items and the new token's item
    if (lane == 0) last = (__hip_atomic_fetch_add(p.head_cnt + head * kHeadCntStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nparts - 1);
    last = first_lane(last);
    trace_mark(p, 11);       // partial published, head counter answered
    if (last) {
        // The last wave of this head merges the partial results.  Lane i fetches (m_i, l_i) of item i, so the
        // scales come from one round trip; the accumulators (two dims per lane) are fetched kMergeBatch
        // splits at a time, together with the scales, and added in split order.
        const size_t hb = (size_t)head * kMaxSplit;
        float mi = kNegBig, li = 0.f;
        if (lane < nparts) ld_agent2(p.part_ml + (hb + lane) * 2, mi, li);
        const int t2 = lane * 2;
        const bool dact = t2 < D;
        constexpr int kMergeBatch = 32;            // splits per memory round trip
        float a0[kMergeBatch], a1[kMergeBatch];
        auto load_acc = [&](int i0) {
#pragma unroll
            for (int u = 0; u < kMergeBatch; ++u) {
                const int i = i0 + u < nparts ? i0 + u : nparts - 1;
                ld_agent2(p.part_acc + (hb + i) * D + (dact ? t2 : 0), a0[u], a1[u]);
            }
        };
        load_acc(0);     // requested together with the scales: one round trip for up to kMergeBatch splits
        float M = fmaxf(mi, xor_shfl(mi, 32));
        M = fmaxf(M, xor_shfl(M, 16));
        M = fmaxf(M, xor_shfl(M, 8));
        M = fmaxf(M, xor_shfl(M, 4));
        M = fmaxf(M, xor_shfl(M, 2));
        M = fmaxf(M, xor_shfl(M, 1));
        const float sci = fast_exp2(mi - M);      // scale of split `lane`
        const float lsi = li * sci;
        float L = 0.f, A0 = 0.f, A1 = 0.f;
        for (int i0 = 0; i0 < nparts; i0 += kMergeBatch) {
            if (i0 != 0) load_acc(i0);
#pragma unroll
            for (int u = 0; u < kMergeBatch; ++u) {
                const bool in = i0 + u < nparts;
                const int i = in ? i0 + u : 0;
                const float sc = in ? rl(sci, i) : 0.f;
                L += in ? rl(lsi, i) : 0.f;
                A0 = fmadd(a0[u], sc, A0);
                A1 = fmadd(a1[u], sc, A1);
            }
        }
        if (dact) {
            const half2_t o = {(half_t)(A0 / L), (half_t)(A1 / L)};
            st_agent(reinterpret_cast<uint32_t*>(p.attn_vec + (size_t)head * D + t2), as_u32(o));
        }
        if (lane == 0) __hip_atomic_store(p.head_cnt + head * kHeadCntStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (nwg_to_signal > 0) {
            // count the head; the wave that completes the count tells every workgroup
            drain_memory_ops();
            int all = 0;
            if (lane == 0) {
                all = (__hip_atomic_fetch_add(p.bar + kBarHeads, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.heads - 1);
                if (all) __hip_atomic_store(p.bar + kBarHeads, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (first_lane(all)) {
                for (int w = lane; w < nwg_to_signal; w += kWave)
                    __hip_atomic_store(p.mbox + w * kMailboxInts + kBarHeads, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// stage C: out[r] = base0[r] + base1[r] + bias1[r] + bias2[r] + W1[r,:] x1 + W2[r,:] x2
// ------------------------------------------------------------------------------------------------
struct StageC {
    const half_t *W1, *x1, *bias1; int K1;    // O projection:  x1 = merged attention output
    const half_t *W2, *x2, *bias2; int K2;    // MLP down:      x2 = MLP intermediate
    const half_t *base0, *base1;
    half_t* out;
    int nrows;
    const half_t *sum_a, *sum_b;   // optional: sum_out[r] = fp16(sum_a[r] + sum_b[r]) (the residual stream of a fused add + norm)
    half_t* sum_out;
    int add_sum;                   // ... and the output row gets that sum added (sum_a alone if there is no sum_b)
};

__device__ __forceinline__ StageC make_stage_c(const LayerParams& p) {
    StageC c;
    c.W1 = p.c_use_o ? p.w_o : nullptr;       c.x1 = p.attn_vec; c.bias1 = p.c_use_o ? p.b_o : nullptr;       c.K1 = p.c_use_o ? p.H : 0;
    c.W2 = p.c_use_down ? p.w_down : nullptr; c.x2 = p.inter;    c.bias2 = p.c_use_down ? p.b_down : nullptr; c.K2 = p.c_use_down ? p.F : 0;
    c.base0 = p.c_base0; c.base1 = p.c_base1; c.out = p.out; c.nrows = p.H;
    c.sum_a = p.x; c.sum_b = p.x_add; c.sum_out = p.x_add ? p.x_sum_out : nullptr; c.add_sum = p.c_add_sum;
    return c;
}

// The MLP-down pass splits K over the kStreamers streaming waves of a workgroup: wave ks owns the 512-half
// chunks ks, ks + kStreamers, ... ("chunk slots" 0 .. CPD-1 of that wave).  The slots are grouped into
// kUpPhases phases; phase g needs the MLP intermediate only up to up_phase_rows(CPD, g, F), so it can
// start as soon as every MLP-up row below that bound is written, while slower workgroups are still
// busy with the rows above it.
__host__ __device__ constexpr int down_slot_end(int cpd, int g) { return ((g + 1) * cpd + kUpPhases - 1) / kUpPhases; }
__host__ __device__ constexpr int down_slot_begin(int cpd, int g) { return g == 0 ? 0 : down_slot_end(cpd, g - 1); }
__device__ __forceinline__ int up_phase_rows(int cpd, int g, int F) {
    const int r = down_slot_end(cpd, g) * kStreamers * kChunk;
    return (g == kUpPhases - 1 || r > F) ? F : r;
}

struct StageCShared {
    float red_down[kUpPhases][kRowBatch][kStreamers];   // MLP-down partials per phase and K slice
    float red_o[kRowBatch];                             // O-projection dot products
};

// One phase (chunk slots LO .. HI-1) of the MLP-down rows [b0, b1) of a streaming wave.
template <int LO, int HI>
struct DownPhase {
    static constexpr int N = HI - LO;
    static constexpr int RPI = N > 0 ? ((16 / N) > 0 ? (16 / N) : 1) : 1;
    static constexpr int NA = N > 0 ? N : 1;
    typedef u32x4 Tile[RPI][NA];

    // a chunk that does not exist for this lane reads column 0 with a zero activation slice
    static __device__ __forceinline__ int col_of(const StageC& c, int ks, int lane, int i, bool& have) {
        const int nch = (c.K2 + kChunk - 1) / kChunk;
        const int chunk = ks + (LO + i) * kStreamers;
        const int col = chunk * kChunk + lane * 8;
        have = chunk < nch && col < c.K2;
        return have ? col : 0;
    }
    // rows past the batch re-read its last row (no conditional loads, see gemv_tiles)
    static __device__ __forceinline__ void load(const StageC& c, int ks, int lane, Tile& w, int r, int b1) {
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            const int rr = (r + j < b1) ? r + j : b1 - 1;
            const half_t* rp = c.W2 + (size_t)rr * (size_t)c.K2;
#pragma unroll
            for (int i = 0; i < N; ++i) {
                bool have;
                w[j][i] = ld_stream16(rp + col_of(c, ks, lane, i, have));
            }
        }
    }
    // `wa` holds the loads of the first tile; ready() runs before the activations are read; next() runs
    // once the last tile of this phase has been requested (the caller requests the next phase's first tile).
    template <class Ready, class Next>
    static __device__ __forceinline__ void run(const StageC& c, int ks, int lane, int b0, int b1, float (*red)[kStreamers],
                                               Tile& wa, Ready&& ready, Next&& next) {
        ready();
        half2_t xs[NA][4];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            bool have;
            const int col = col_of(c, ks, lane, i, have);
            u32x4 xv = {0u, 0u, 0u, 0u};
            if (have) xv = ld_agent16(c.x2 + col);
            xs[i][0] = as_h2(xv.x); xs[i][1] = as_h2(xv.y); xs[i][2] = as_h2(xv.z); xs[i][3] = as_h2(xv.w);
        }
        auto finish = [&](const Tile& w, int r) {
#pragma unroll
            for (int j = 0; j < RPI; ++j) {
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < N; ++i) acc = dot8(w[j][i], xs[i], acc);
                acc = wave_sum(acc);
                if (r + j < b1 && lane == 0) red[r + j - b0][ks] = acc;
            }
        };
        Tile wb;
        int r = b0;
        for (; r + 2 * RPI < b1; r += 2 * RPI) {   // two tiles in flight, branch-free body, tail peeled
            load(c, ks, lane, wb, r + RPI, b1);
            finish(wa, r);
            __builtin_amdgcn_sched_barrier(0);   // a third tile's loads must not be scheduled above this point
            load(c, ks, lane, wa, r + 2 * RPI, b1);
            finish(wb, r + RPI);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (r + RPI < b1) {
            load(c, ks, lane, wb, r + RPI, b1);
            finish(wa, r);
            __builtin_amdgcn_sched_barrier(0);
            next();
            finish(wb, r + RPI);
        } else {
            next();
            finish(wa, r);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
};

// The MLP-down phases g = G .. kUpPhases-1 of the rows [b0, b1) of one streaming wave, one after the other; phase g
// waits for down_ready(g) (on the first row batch only) after its first weight tile has been requested.  A phase without
// chunk slots (small geometries have fewer slots than phases) only passes its wait.
template <int CPD, int G, class DownReady>
__device__ __forceinline__ void down_phases(const StageC& c, int ks, int lane, int b0, int b1, StageCShared& sh, bool first,
                                            DownReady&& down_ready) {
    typedef DownPhase<down_slot_begin(CPD, G), down_slot_end(CPD, G)> P;
    if constexpr (P::N > 0) {
        typename P::Tile t;
        P::load(c, ks, lane, t, b0, b1);
        P::run(c, ks, lane, b0, b1, sh.red_down[G], t, [&] { if (first) down_ready(G); }, [] {});
    } else {
        if (first) down_ready(G);
    }
    if constexpr (G + 1 < kUpPhases) down_phases<CPD, G + 1>(c, ks, lane, b0, b1, sh, first, down_ready);
}

// Stage C for the rows of workgroup `wg`, as two independent GEMVs whose results meet in LDS:
//   MLP down   K-split over the kStreamers streaming waves (wave ks owns the 512-half chunks ks, ks+4, ...
//              of W2 and x2, at most CPD of them, activation slices in registers), RPI rows per tile, two
//              tiles in flight; each wave leaves its partial dot product of every row in red_down.
//   O proj     row-per-wave over the `n_o` waves that have o_index >= 0 (row b0 + o_index, + n_o, ...),
//              the whole attention vector in registers (K1 <= NCH*512), two rows in flight; red_o.
// In the fused kernel the streaming waves do the MLP-down part and the helper waves the O projection,
// so the attention output is not needed until the (longer) MLP-down pass is over; in split mode the same
// four waves do one after the other.  `down_ready(g)` / `o_ready()` run after the first loads of a pass (of phase g) are
// in flight and before its activations are read (the fused kernel waits for the producing event there).
// The partials are added in a fixed order with the biases and residual terms: deterministic, and
// identical in both modes.  Every wave of the workgroup must call this (workgroup barriers inside).
// COH: the layer's input rows (the residual terms) were written earlier in this same launch, and its output rows are
// read later in it, by other workgroups: both go past the caches.
template <int NCH, int CPD, bool COH = false, class DownReady, class OReady>
__device__ __forceinline__ void stage_c_rows(const StageC& c, int wg, int nwg, StageCShared& sh, bool streamer, int ks,
                                             int o_index, int n_o, int lane, DownReady&& down_ready, OReady&& o_ready,
                                             int thread_in = -1) {
    const int r0 = mul_div(wg, c.nrows, nwg), r1 = mul_div(wg + 1, c.nrows, nwg);
    bool first = true;
    for (int b0 = r0; b0 < r1; b0 += kRowBatch) {
        const int b1 = (b0 + kRowBatch < r1) ? b0 + kRowBatch : r1;
        // what the epilogue of this batch adds to the dot products are inputs of the layer: requested now, so that the
        // threads that finish the rows do not start a memory round trip after the last barrier.  All six requests go out
        // back to back, whatever terms the call has (a term that does not exist reads the output row instead and is
        // dropped later), and nothing is done with the values until the epilogue: with one conditional load per term the
        // compiler waited for each of them in turn, three or four dependent memory round trips in front of the first
        // weight tile of the wave that finishes the rows - it saw every event of the pass several microseconds after the
        // other waves, and the whole workgroup ended that much later.
        const int et = thread_in >= 0 ? thread_in : (int)threadIdx.x;
        const bool finisher = et < b1 - b0;
        half_t h_b1, h_b2, h_x0, h_x1, h_sa, h_sb;      // (only read by the lanes that loaded them)
        if (first_lane(et >> 6) == 0) {     // the wave that holds the finishing lanes (a scalar branch)
            const int r = finisher ? b0 + et : b0;
            const half_t* any = c.out + r;
            auto term = [](const half_t* q) { if constexpr (COH) return ld_agent(q); else return *q; };
            h_b1 = *(c.bias1 ? c.bias1 + r : any);
            h_b2 = *(c.bias2 ? c.bias2 + r : any);
            h_x0 = term(c.base0 ? c.base0 + r : any);
            h_x1 = term(c.base1 ? c.base1 + r : any);
            h_sa = term((c.sum_b != nullptr || c.add_sum) ? c.sum_a + r : any);
            h_sb = term(c.sum_b ? c.sum_b + r : any);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (streamer && c.K2 > 0) down_phases<CPD, 0>(c, ks, lane, b0, b1, sh, first, down_ready);
        if (o_index >= 0 && c.K1 > 0) {
            // up to kORows rows of this wave are requested before the attention vector is waited for, so that
            // only one more round trip (the vector itself) follows the wait
            constexpr int kORows = 4;
            auto load_row = [&](u32x4 (&w)[NCH], int r) {
                const int rr = r < b1 ? r : b1 - 1;
                const half_t* rp = c.W1 + (size_t)rr * (size_t)c.K1;
#pragma unroll
                for (int i = 0; i < NCH; ++i) {
                    const int col = i * kChunk + lane * 8;
                    w[i] = ld_stream16(rp + (col < c.K1 ? col : 0));
                }
            };
            u32x4 w[kORows][NCH];
#pragma unroll
            for (int j = 0; j < kORows; ++j) load_row(w[j], b0 + o_index + j * n_o);
            if (first) o_ready();
            half2_t xs[NCH][4];
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int col = i * kChunk + lane * 8;
                u32x4 xv = {0u, 0u, 0u, 0u};
                if (col < c.K1) xv = ld_agent16(c.x1 + col);
                xs[i][0] = as_h2(xv.x); xs[i][1] = as_h2(xv.y); xs[i][2] = as_h2(xv.z); xs[i][3] = as_h2(xv.w);
            }
            for (int r = b0 + o_index; r < b1; r += kORows * n_o) {
#pragma unroll
                for (int j = 0; j < kORows; ++j) {
                    float acc = 0.f;
#pragma unroll
                    for (int i = 0; i < NCH; ++i) acc = dot8(w[j][i], xs[i], acc);
                    acc = wave_sum(acc);
                    const int rj = r + j * n_o;
                    if (rj < b1 && lane == 0) sh.red_o[rj - b0] = acc;
                }
                if (r + kORows * n_o < b1) {
#pragma unroll
                    for (int j = 0; j < kORows; ++j) load_row(w[j], r + (kORows + j) * n_o);
                }
            }
        }
        first = false;
        __syncthreads();
        if (finisher) {
            const int t = et, r = b0 + et;
            const float e_b1 = (float)h_b1, e_b2 = (float)h_b2, e_x0 = (float)h_x0, e_x1 = (float)h_x1, e_sa = (float)h_sa, e_sb = (float)h_sb;
            float v = 0.f;
            if (c.K2 > 0) {
#pragma unroll
                for (int g = 0; g < kUpPhases; ++g) {
                    if (down_slot_end(CPD, g) > down_slot_begin(CPD, g))
                        for (int k = 0; k < kStreamers; ++k) v += sh.red_down[g][t][k];
                }
            }
            if (c.K1 > 0) v += sh.red_o[t];
            if (c.bias1) v += e_b1;
            if (c.bias2) v += e_b2;
            if (c.base0) v += e_x0;
            if (c.base1) v += e_x1;
            if (c.sum_b != nullptr || c.add_sum) {
                // the fp16 sum the norm saw; every workgroup is past its norm by now (stage C follows the attention,
                // which follows all QKV rows), so the sum may overwrite one of its operands
                float rs = e_sa;
                if (c.sum_b != nullptr) rs = (float)(half_t)(rs + e_sb);
                if (c.sum_out) c.sum_out[r] = (half_t)rs;
                if (c.add_sum) v += rs;
            }
            if constexpr (COH) st_agent(c.out + r, (half_t)v);
            else c.out[r] = (half_t)v;
        }
        __syncthreads();
    }
}

}  // namespace cfpp
