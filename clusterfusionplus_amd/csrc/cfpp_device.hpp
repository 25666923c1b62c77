// Device-side building blocks of the GPT-NeoX decode step for gfx950 (wave64, CDNA4).
//
// The layer is five matrix-vector products plus one single-query attention, all bound by HBM
// bandwidth.  The decomposition used here (it replaces the reference's one-cluster-per-head
// scheme, include/5090/pythia_2b8/kernel.cuh:51-949):
//
//   stage A  LayerNorm statistics in registers of every wave; one wave streams whole weight rows of
//            W_qkv (then W_up) with 16-byte lane loads, 512 contiguous halfs per wave-load, fp32
//            accumulation through v_dot2_f32_f16, a DPP row reduction, and a scalar epilogue
//            (bias -> raw q/k/v in fp32, or bias -> tanh-GELU -> fp16 intermediate).
//   stage B  split-KV single-query attention: one workgroup per (head, KV split); 16 lanes per cache
//            row, exp2-domain online softmax in fp32, fp32 partials in scratch, and the last
//            workgroup to finish a head merges that head's partials in a fixed order.
//            RoPE is applied when q / k are read from the raw fp32 scratch; the (head, split 0)
//            workgroup appends the rotated K and V to the cache and returns them.
//   stage C  out = x + b_o + b_down + W_o attn + W_down h as one GEMV over the concatenated input;
//            the K dimension is split over the waves of a workgroup (the activation slice lives in
//            registers), rows are split over workgroups, and a fixed-order LDS reduction finishes
//            each row: deterministic, no atomics on data.
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
constexpr int kMaxSplit = 32;          // KV splits per head
constexpr int kMaxWaves = 16;          // waves per workgroup
constexpr int kRowBatch = 16;          // stage-C rows reduced per LDS round
constexpr float kNegBig = -1.0e30f;
constexpr long long kSpinLimit = 1LL << 20;   // bounded device-side waits (order of a second)

enum : int { kStatusSpin = 1, kStatusSeq = 2 };

struct LayerParams {
    int H, heads, D, rot, F;
    float eps, qscale;
    const half_t *ln_w, *ln_b, *w_qkv, *b_qkv, *w_o, *b_o, *ln2_w, *ln2_b, *w_up, *b_up, *w_down, *b_down;
    const half_t* x;
    half_t *out, *k_new, *v_new, *k_cache, *v_cache;
    int cache_rows;
    const float *cos, *sin;
    int rope_stride;
    int seq_len;
    const int* d_seq_len;
    int nsplit;
    // scratch
    float* qkv_raw;     // [3H] fp32: W_qkv ln1(x) + b_qkv, before RoPE
    half_t* attn_vec;   // [H] fp16: merged attention output (input of the O projection)
    half_t* inter;      // [F] fp16: gelu(W_up ln2(x) + b_up)
    float* part_ml;     // [heads][nsplit][2] running max (log2 domain) and denominator
    float* part_acc;    // [heads][nsplit][D]
    int* head_cnt;      // [heads] arrival counters, self-resetting
    int* bar;           // [0] epoch counter, [1] exit counter, [2] status flags
    // stage-C selection (split API halves)
    const half_t* c_base0;   // residual terms added to the output (nullable)
    const half_t* c_base1;
    int c_use_o, c_use_down;
};

// ------------------------------------------------------------------------------------------------
// loads / conversions
// ------------------------------------------------------------------------------------------------
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
__device__ __forceinline__ float ld_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u32x4 ld_agent16(const void* p) {
    const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
    const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
    return r;
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

// ------------------------------------------------------------------------------------------------
// math
// ------------------------------------------------------------------------------------------------
// tanh-GELU, 0.5 x (1 + tanh(sqrt(2/pi)(x + 0.044715 x^3))) with tanh(u) = 1 - 2/(1 + e^{2u}) on the
// native exp2 (reference include/5090/pythia_2b8/kernel.cuh:26-49 builds the same from ex2.approx).
__device__ __forceinline__ float gelu_tanh(float x) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float e = __builtin_amdgcn_exp2f(u * 2.8853900817779268f);   // e^{2u}
    const float t = 1.0f - 2.0f / (1.0f + e);
    return 0.5f * x * (1.0f + t);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ------------------------------------------------------------------------------------------------
// device-wide synchronisation (bounded spins; a timeout raises a status flag and falls through)
// ------------------------------------------------------------------------------------------------
// arrive: the caller has drained its stores (and, for a workgroup-wide arrival, synchronised the workgroup)
__device__ __forceinline__ void counter_add(int* ctr, int v) {
    __hip_atomic_fetch_add(ctr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// one thread polls; the whole workgroup leaves together.  Data published before the arrivals must be
// read with ld_agent / ld_agent16.
__device__ __forceinline__ void grid_wait(int* ctr, int target, int* status) {
    if (threadIdx.x == 0) {
        long long spins = 0;
        while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > kSpinLimit) {
                __hip_atomic_fetch_or(status, kStatusSpin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
        }
    }
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

__device__ __forceinline__ int load_seq_len(const LayerParams& p) {
    int S = p.d_seq_len ? *p.d_seq_len : p.seq_len;
    if (S < 0 || S > p.cache_rows) {
        if (threadIdx.x == 0 && blockIdx.x == 0)
            __hip_atomic_fetch_or(p.bar + 2, kStatusSeq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        S = S < 0 ? 0 : p.cache_rows;
    }
    return S;
}

// ------------------------------------------------------------------------------------------------
// stage A: LayerNorm into registers, then row-per-wave streaming GEMV
// ------------------------------------------------------------------------------------------------
// Every wave loads the whole input row (lane l holds columns i*512 + 8l .. +8 of every chunk i),
// computes mean and variance two-pass in fp32, and keeps both affine variants (input LN for QKV,
// post-attention LN for the MLP; they share the statistics because the residual is parallel,
// reference include/5090/pythia_2b8/kernel.cuh:811-818) as packed fp16.
template <int NCH>
__device__ __forceinline__ void load_ln_pair(const half_t* __restrict__ x, int H, float eps,
                                             const half_t* __restrict__ w1, const half_t* __restrict__ b1,
                                             const half_t* __restrict__ w2, const half_t* __restrict__ b2,
                                             int lane, half2_t (&x1)[NCH][4], half2_t (&x2)[NCH][4]) {
    float xv[NCH][8];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col = i * kChunk + lane * 8;
        if (col < H) {
            unpack8(ld16(x + col), xv[i]);
#pragma unroll
            for (int j = 0; j < 8; ++j) s += xv[i][j];
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) xv[i][j] = 0.f;
        }
    }
    const float mean = wave_sum(s) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        if (i * kChunk + lane * 8 < H) {
#pragma unroll
            for (int j = 0; j < 8; ++j) { const float d = xv[i][j] - mean; q += d * d; }
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)H + eps);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col = i * kChunk + lane * 8;
        float y1[8], y2[8];
        if (col < H) {
            float g[8], b[8];
            unpack8(ld16(w1 + col), g); unpack8(ld16(b1 + col), b);
#pragma unroll
            for (int j = 0; j < 8; ++j) y1[j] = (xv[i][j] - mean) * rstd * g[j] + b[j];
            if (w2 != nullptr) {
                unpack8(ld16(w2 + col), g); unpack8(ld16(b2 + col), b);
#pragma unroll
                for (int j = 0; j < 8; ++j) y2[j] = (xv[i][j] - mean) * rstd * g[j] + b[j];
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) y2[j] = 0.f;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) { y1[j] = 0.f; y2[j] = 0.f; }
        }
        const u32x4 p1 = pack8(y1), p2 = pack8(y2);
        x1[i][0] = as_h2(p1.x); x1[i][1] = as_h2(p1.y); x1[i][2] = as_h2(p1.z); x1[i][3] = as_h2(p1.w);
        x2[i][0] = as_h2(p2.x); x2[i][1] = as_h2(p2.y); x2[i][2] = as_h2(p2.z); x2[i][3] = as_h2(p2.w);
    }
}

// Rows first, first+stride, ... < nrows of W[nrows, K]; RPI rows in flight per wave.
// pre(row) is evaluated together with the weight loads (bias fetch); epi(row, dot, pre) is called by
// every lane with the wave-uniform dot product.  EXACT: K == NCH*512, every lane load is in range and
// addresses use immediate offsets; otherwise out-of-range lane loads are redirected to column 0 (their
// activation registers are zero, so they contribute nothing).
template <int NCH, int RPI, bool EXACT, class Pre, class Epi>
__device__ __forceinline__ void gemv_rows(const half_t* __restrict__ W, int K, int first, int stride, int nrows,
                                          const half2_t (&x)[NCH][4], int lane, Pre&& pre, Epi&& epi) {
    const int colb = lane * 8;
    int coff[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = i * kChunk + colb;
        coff[i] = (EXACT || c < K) ? c : 0;
    }
    for (int r = first; r < nrows; r += stride * RPI) {
        u32x4 w[RPI][NCH];
        float pv[RPI];
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            int rr = r + j * stride;
            rr = rr < nrows ? rr : r;
            pv[j] = pre(rr);
            const half_t* rp = W + (size_t)rr * (size_t)K;
#pragma unroll
            for (int i = 0; i < NCH; ++i) w[j][i] = ld_stream16(EXACT ? rp + colb + i * kChunk : rp + coff[i]);
        }
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) acc = dot8(w[j][i], x[i], acc);
            acc = wave_sum(acc);
            const int rr = r + j * stride;
            if (rr < nrows) epi(rr, acc, pv[j]);
        }
    }
}

template <int NCH, class Pre, class Epi>
__device__ __forceinline__ void gemv_rows_auto(const half_t* __restrict__ W, int K, int first, int stride, int nrows,
                                               const half2_t (&x)[NCH][4], int lane, Pre&& pre, Epi&& epi) {
    constexpr int RPI = (16 / NCH) > 0 ? (16 / NCH) : 1;
    if (K == NCH * kChunk) gemv_rows<NCH, RPI, true>(W, K, first, stride, nrows, x, lane, pre, epi);
    else gemv_rows<NCH, RPI, false>(W, K, first, stride, nrows, x, lane, pre, epi);
}

template <int NCH>
__device__ __forceinline__ void stage_a_qkv(const LayerParams& p, const half2_t (&x1)[NCH][4], int gw, int nw, int lane) {
    const half_t* __restrict__ bias = p.b_qkv;
    float* __restrict__ dst = p.qkv_raw;
    gemv_rows_auto<NCH>(p.w_qkv, p.H, gw, nw, 3 * p.H, x1, lane,
                        [&](int r) { return (float)bias[r]; },
                        [&](int r, float v, float b) { if (lane == 0) st_agent(dst + r, v + b); });
}
template <int NCH>
__device__ __forceinline__ void stage_a_up(const LayerParams& p, const half2_t (&x2)[NCH][4], int gw, int nw, int lane) {
    const half_t* __restrict__ bias = p.b_up;
    half_t* __restrict__ dst = p.inter;
    gemv_rows_auto<NCH>(p.w_up, p.H, gw, nw, p.F, x2, lane,
                        [&](int r) { return (float)bias[r]; },
                        [&](int r, float v, float b) { if (lane == 0) st_agent(dst + r, (half_t)gelu_tanh(v + b)); });
}

// ------------------------------------------------------------------------------------------------
// stage B: split-KV single-query attention for one (head, split) item, whole workgroup
// ------------------------------------------------------------------------------------------------
// NeoX rotate-half RoPE on the first `rot` dims of a head vector held in raw fp32 scratch
// (reference include/5090/pythia_2b8/kernel.cuh:395-421): d < rot/2 -> v[d] cos[d] - v[d+rot/2] sin[d];
// rot/2 <= d < rot -> v[d] cos[d] + v[d-rot/2] sin[d]; d >= rot passes through.
__device__ __forceinline__ float rope_elem(const float* __restrict__ v, int d, int rot,
                                           const float* __restrict__ cs, const float* __restrict__ sn) {
    const float a = ld_agent(v + d);
    if (d >= rot) return a;
    const int hr = rot >> 1;
    return d < hr ? a * cs[d] - ld_agent(v + d + hr) * sn[d] : a * cs[d] + ld_agent(v + d - hr) * sn[d];
}

struct AttnShared {
    float m[kMaxWaves];
    float l[kMaxWaves];
    float acc[kMaxWaves][128];
    int last;
};

__device__ __forceinline__ void attention_item(const LayerParams& p, int head, int sp, int S, AttnShared& sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int grp = lane >> 4, sub = lane & 15;
    const int D = p.D, H = p.H, d0 = sub * 8;
    const bool act = d0 < D;
    const float* __restrict__ raw = p.qkv_raw + (size_t)head * 3 * D;
    const float* __restrict__ cs = p.cos + (size_t)S * p.rope_stride;   // stride 0: the row is the position
    const float* __restrict__ sn = p.sin + (size_t)S * p.rope_stride;

    float q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = act ? rope_elem(raw, d0 + j, p.rot, cs, sn) * p.qscale : 0.f;

    float m = kNegBig, l = 0.f, acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;

    // the new token: split 0 owns it (appends it, returns it, and seeds its softmax state with it)
    if (sp == 0 && wave == 0 && grp == 0) {
        float kf[8], vf[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            kf[j] = act ? rope_elem(raw + D, d0 + j, p.rot, cs, sn) : 0.f;
            vf[j] = act ? ld_agent(raw + 2 * D + d0 + j) : 0.f;
        }
        const u32x4 kp = pack8(kf), vp = pack8(vf);
        unpack8(kp, kf); unpack8(vp, vf);      // attend over the fp16 values the cache will hold
        if (act) {
            const size_t o = (size_t)head * D + d0;
            *reinterpret_cast<u32x4*>(p.k_new + o) = kp;
            *reinterpret_cast<u32x4*>(p.v_new + o) = vp;
            if (S < p.cache_rows) {
                *reinterpret_cast<u32x4*>(p.k_cache + (size_t)S * H + o) = kp;
                *reinterpret_cast<u32x4*>(p.v_cache + (size_t)S * H + o) = vp;
            }
        }
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) s += q[j] * kf[j];
        s = row16_sum(s);
        m = s; l = 1.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = vf[j];
    }

    // cached rows of this split, interleaved over the (wave, 16-lane group) slots, 4 rows per step
    const int chunk = (S + p.nsplit - 1) / p.nsplit;
    const int begin = sp * chunk;
    const int end = (begin + chunk < S) ? begin + chunk : S;
    const int slots = nwaves * 4, slot = wave * 4 + grp;
    const half_t* __restrict__ kc = p.k_cache + (size_t)head * D + d0;
    const half_t* __restrict__ vc = p.v_cache + (size_t)head * D + d0;
    constexpr int T = 4;
    for (int r = begin + slot; r < end; r += slots * T) {
        u32x4 kk[T], vv[T];
        bool ok[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int row = r + t * slots;
            ok[t] = row < end;
            const u32x4 z = {0u, 0u, 0u, 0u};
            kk[t] = z; vv[t] = z;
            if (ok[t] && act) {
                kk[t] = ld16(kc + (size_t)row * H);
                vv[t] = ld16(vc + (size_t)row * H);
            }
        }
        float s[T], mt = m;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            float kf[8];
            unpack8(kk[t], kf);
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) d += q[j] * kf[j];
            d = row16_sum(d);
            s[t] = ok[t] ? d : kNegBig;
            mt = fmaxf(mt, s[t]);
        }
        const float alpha = fast_exp2(m - mt);
        l *= alpha;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] *= alpha;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float pt = ok[t] ? fast_exp2(s[t] - mt) : 0.f;
            float vf[8];
            unpack8(vv[t], vf);
            l += pt;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += pt * vf[j];
        }
        m = mt;
    }

    // merge the four groups of the wave (lanes sub, sub+16, sub+32, sub+48 hold the same dims)
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
    if (grp == 0) {
        if (sub == 0) { sh.m[wave] = m; sh.l[wave] = l; }
#pragma unroll
        for (int j = 0; j < 8; ++j) sh.acc[wave][d0 + j] = acc[j];
    }
    __syncthreads();
    // merge the waves in wave order and publish the partial of this (head, split)
    const size_t item = (size_t)head * p.nsplit + sp;
    if ((int)threadIdx.x < D) {
        float M = sh.m[0];
        for (int w = 1; w < nwaves; ++w) M = fmaxf(M, sh.m[w]);
        float L = 0.f, A = 0.f;
        for (int w = 0; w < nwaves; ++w) {
            const float sc = fast_exp2(sh.m[w] - M);
            L += sh.l[w] * sc;
            A += sh.acc[w][threadIdx.x] * sc;
        }
        st_agent(p.part_acc + item * D + threadIdx.x, A);
        if (threadIdx.x == 0) { st_agent(p.part_ml + item * 2, M); st_agent(p.part_ml + item * 2 + 1, L); }
    }
    drain_memory_ops();
    __syncthreads();
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(p.head_cnt + head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sh.last = (old == p.nsplit - 1);
    }
    __syncthreads();
    if (sh.last) {
        // the last workgroup of this head merges the splits in split order; two dims per thread
        const int t2 = threadIdx.x * 2;
        if (t2 < D) {
            const size_t hb = (size_t)head * p.nsplit;
            float M = kNegBig;
            for (int i = 0; i < p.nsplit; ++i) M = fmaxf(M, ld_agent(p.part_ml + (hb + i) * 2));
            float L = 0.f, A0 = 0.f, A1 = 0.f;
            for (int i = 0; i < p.nsplit; ++i) {
                const float sc = fast_exp2(ld_agent(p.part_ml + (hb + i) * 2) - M);
                L += ld_agent(p.part_ml + (hb + i) * 2 + 1) * sc;
                A0 += ld_agent(p.part_acc + (hb + i) * D + t2) * sc;
                A1 += ld_agent(p.part_acc + (hb + i) * D + t2 + 1) * sc;
            }
            const half2_t o = {(half_t)(A0 / L), (half_t)(A1 / L)};
            st_agent(reinterpret_cast<uint32_t*>(p.attn_vec + (size_t)head * D + t2), as_u32(o));
        }
        if (threadIdx.x == 0) __hip_atomic_store(p.head_cnt + head, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();   // sh is reused by the next item
}

// ------------------------------------------------------------------------------------------------
// stage C: out[r] = base0[r] + base1[r] + bias1[r] + bias2[r] + W1[r,:] x1 + W2[r,:] x2
// ------------------------------------------------------------------------------------------------
struct StageC {
    const half_t *W1, *x1, *bias1; int K1;
    const half_t *W2, *x2, *bias2; int K2;
    const half_t *base0, *base1;
    half_t* out;
    int nrows;
};

__device__ __forceinline__ StageC make_stage_c(const LayerParams& p) {
    StageC c;
    c.W1 = p.c_use_o ? p.w_o : nullptr;       c.x1 = p.attn_vec; c.bias1 = p.c_use_o ? p.b_o : nullptr;       c.K1 = p.c_use_o ? p.H : 0;
    c.W2 = p.c_use_down ? p.w_down : nullptr; c.x2 = p.inter;    c.bias2 = p.c_use_down ? p.b_down : nullptr; c.K2 = p.c_use_down ? p.F : 0;
    c.base0 = p.c_base0; c.base1 = p.c_base1; c.out = p.out; c.nrows = p.H;
    return c;
}

struct StageCShared { float red[kRowBatch][kMaxWaves]; };

// The workgroup's waves form RG row groups x KS K-slices (wave = rg*KS + ks).  K is cut into
// 512-half chunks over the concatenation [x1 | x2]; slice ks owns chunks ks, ks+KS, ... (at most CPW).
template <int CPW>
__device__ __forceinline__ void stage_c_rows(const StageC& c, int wg, int nwg, int KS, int RG, StageCShared& sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ks = wave % KS, rg = wave / KS;
    const int nch1 = (c.K1 + kChunk - 1) / kChunk, nch2 = (c.K2 + kChunk - 1) / kChunk;
    constexpr int RPI = (12 / CPW) > 0 ? (12 / CPW) : 1;

    // per-chunk weight pointer at row 0; a chunk that does not exist for this lane reads a valid dummy
    // location with row stride 0 and a zero activation slice
    const half_t* wp[CPW];
    int wstride[CPW];
    half2_t xs[CPW][4];
    const half_t* dummy = c.W1 ? c.W1 : c.W2;
#pragma unroll
    for (int i = 0; i < CPW; ++i) {
        const int ch = ks + i * KS;
        wp[i] = dummy; wstride[i] = 0;
        const half_t* xp = nullptr;
        if (ch < nch1) {
            const int col = ch * kChunk + lane * 8;
            if (col < c.K1) { wp[i] = c.W1 + col; wstride[i] = c.K1; xp = c.x1 + col; }
        } else if (ch < nch1 + nch2) {
            const int col = (ch - nch1) * kChunk + lane * 8;
            if (col < c.K2) { wp[i] = c.W2 + col; wstride[i] = c.K2; xp = c.x2 + col; }
        }
        u32x4 xv = {0u, 0u, 0u, 0u};
        if (xp) xv = ld_agent16(xp);
        xs[i][0] = as_h2(xv.x); xs[i][1] = as_h2(xv.y); xs[i][2] = as_h2(xv.z); xs[i][3] = as_h2(xv.w);
    }

    const int r0 = (int)(((long long)wg * c.nrows) / nwg), r1 = (int)(((long long)(wg + 1) * c.nrows) / nwg);
    for (int b0 = r0; b0 < r1; b0 += kRowBatch) {
        const int b1 = (b0 + kRowBatch < r1) ? b0 + kRowBatch : r1;
        for (int r = b0 + rg; r < b1; r += RG * RPI) {
            u32x4 w[RPI][CPW];
#pragma unroll
            for (int j = 0; j < RPI; ++j) {
                int rr = r + j * RG;
                rr = rr < b1 ? rr : r;
#pragma unroll
                for (int i = 0; i < CPW; ++i) w[j][i] = ld_stream16(wp[i] + (size_t)rr * wstride[i]);
            }
#pragma unroll
            for (int j = 0; j < RPI; ++j) {
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < CPW; ++i) acc = dot8(w[j][i], xs[i], acc);
                acc = wave_sum(acc);
                const int rr = r + j * RG;
                if (rr < b1 && lane == 0) sh.red[rr - b0][ks] = acc;
            }
        }
        __syncthreads();
        const int t = threadIdx.x;
        if (t < b1 - b0) {
            const int r = b0 + t;
            float v = 0.f;
            for (int k = 0; k < KS; ++k) v += sh.red[t][k];
            if (c.bias1) v += (float)c.bias1[r];
            if (c.bias2) v += (float)c.bias2[r];
            if (c.base0) v += (float)c.base0[r];
            if (c.base1) v += (float)c.base1[r];
            c.out[r] = (half_t)v;
        }
        __syncthreads();
    }
}

}  // namespace cfpp
