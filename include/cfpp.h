/*
 * cfpp.h - C ABI of the MI355X (gfx950) GPT-NeoX / Pythia fused decode-step library.
 *
 * Plain C: raw device pointers, sizes and a hipStream_t passed as void*.  No torch types.
 * The PyTorch extension (`clusterfusion._clusterfusion`) and any other host (a C++ serving
 * loop, ctypes) bind exactly these entry points.
 *
 * Conventions for every call that returns `int`:
 *   0  success; <0 a `cfpp_status` argument error (nothing was launched); >0 a hipError_t.
 * No entry point throws or synchronises the device (the *_check calls excepted); only the ones whose
 * comment says so allocate device memory (context / stack creation).  All launches go to the given stream.
 *
 * One-launch kernels and what they need.  CFPP_MODE_FUSED runs a whole layer as ONE launch whose workgroups wait
 * for each other's results, so all of them must be on the device at the same time.  The library launches it only
 * when the device can hold the whole grid (kernel occupancy x compute units, queried once per device and kernel)
 * and takes the per-stage launches of CFPP_MODE_SPLIT otherwise: same results, bit for bit.  What it cannot see is
 * other work on the device: while a fused launch runs, no other stream or process may keep compute units busy
 * with long kernels.  Every wait inside the kernels is bounded (about a second); one that expires raises a failure
 * flag instead of hanging, the results of that launch are invalid, and every later launching call on the device
 * returns CFPP_ERR_DEVICE until cfpp_device_status(1) has been called (re-zero the workspaces that were in use).
 *
 * Tensor contract (same as the reference's dispatch code,
 * include/5090/pythia_2b8/pythia_kernel_dispatch.cu:4-75): fp16 row-major contiguous;
 * weights in nn.Linear layout [out, in]; W_qkv / b_qkv head-interleaved [head][q|k|v][D]
 * (reference include/5090/pythia_2b8/config.h:14-18); K/V caches [rows, H] with head-major
 * columns; cos/sin fp32 with at least rotary_dim entries per position.
 */
#ifndef CFPP_H
#define CFPP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum cfpp_status {
    CFPP_OK = 0,
    CFPP_ERR_NULL = -1,        /* a required pointer is NULL */
    CFPP_ERR_DIMS = -2,        /* unsupported dimensions */
    CFPP_ERR_SEQ = -3,         /* seq_len < 0, beyond the cache rows, or (position-indexed RoPE tables) == cache rows */
    CFPP_ERR_WORKSPACE = -4,   /* workspace too small or misaligned */
    CFPP_ERR_CONTEXT = -5,     /* unknown / duplicate context id */
    CFPP_ERR_MODE = -6,        /* unknown mode */
    CFPP_ERR_DEVICE = -7,      /* a device-side failure flag is raised (bounded wait expired, bad device seq_len):
                                  by an earlier launch on this device (see cfpp_device_status) or in the workspace
                                  that was checked */
    CFPP_ERR_ALIGN = -8,       /* a tensor pointer is not 16-byte aligned */
    CFPP_ERR_ALIAS = -9,       /* an output overlaps an input it must not overlap */
    CFPP_ERR_STATIC_SCRATCH = -10, /* cfpp_neox_layer_decode_static: the geometry needs more than cfpp_static_scratch_bytes() */
    CFPP_ERR_NOT_INITIALISED = -11 /* cfpp_neox_layer_decode_static: cfpp_init() (or another launching entry point) has not
                                      run on this device yet, so the word that reports device-side failures does not exist */
} cfpp_status;

/* Layer geometry.  Pythia-2.8B = {2560,32,80,20,10240,1e-5}, Pythia-6.9B = {4096,32,128,32,16384,1e-5}
 * (reference include/5090/pythia_2b8/config.h:6-12, include/5090/pythia_6b9/config.h:6-12).
 * Supported: hidden == heads*head_dim, hidden % 8 == 0, hidden <= 4096, head_dim % 8 == 0,
 * head_dim <= 128, rotary_dim even and <= head_dim, ffn % 8 == 0, and (ceil(hidden / 512), ceil(ceil(ffn / 512) / 4))
 * one of (1,1) (2,2) (4,4) (5,5) (8,8) (8,6): the shapes the kernels are instantiated for (hidden 512, 1024, 2048,
 * 2560, 4096 with ffn = 4 hidden; hidden 4096 with ffn 11008); anything else returns CFPP_ERR_DIMS. */
typedef struct cfpp_neox_dims {
    int32_t hidden, heads, head_dim, rotary_dim, ffn;
    float eps;
} cfpp_neox_dims;

/* The 12 per-layer tensors (reference tests/benchmark_decode.py:83-96 extracts the same set). */
typedef struct cfpp_neox_weights {
    const void *ln_w, *ln_b;            /* input LayerNorm [H] */
    const void *w_qkv, *b_qkv;          /* [3H,H], [3H] head-interleaved */
    const void *w_o, *b_o;              /* [H,H], [H] */
    const void *post_ln_w, *post_ln_b;  /* post-attention LayerNorm [H] (feeds the MLP; parallel residual) */
    const void *w_up, *b_up;            /* [F,H], [F] */
    const void *w_down, *b_down;        /* [H,F], [H] */
} cfpp_neox_weights;

/* Per-call tensors.  `seq_len` counts valid cache rows BEFORE the append (reference
 * pythia_kernel_dispatch.cu:68-75).  If `d_seq_len` is non-NULL the kernels read the length
 * from that device int32 instead (needed for hipGraph replay) and cos/sin are indexed by it:
 * row = cos + seq_len * rope_stride (rope_stride 0 = the given row is the current position). */
typedef struct cfpp_neox_io {
    const void* input;       /* [H] fp16, read only */
    void* output;            /* [H] fp16 */
    void* k_new;             /* [heads*D] fp16: rotated K of the new token */
    void* v_new;             /* [heads*D] fp16 */
    void* k_cache;           /* [cache_rows, H] fp16; row seq_len is written if cache_rows > seq_len */
    void* v_cache;
    int32_t cache_rows;
    const float* cos;
    const float* sin;
    int32_t rope_stride;
    int32_t seq_len;
    const int32_t* d_seq_len;
    int32_t max_seq_len;     /* with d_seq_len: the largest length the launches are sized for (0 = cache_rows); a device-side
                                length beyond it raises the failure flag instead of being attended */
    void* attn_output;       /* split API only: [H] fp16 = W_o attn + b_o */
    void* mlp_intermediate;  /* split API only: [F] fp16 = gelu(W_up ln2(x) + b_up) */
} cfpp_neox_io;

typedef enum cfpp_mode {
    CFPP_MODE_FUSED = 0,     /* one persistent launch with device-wide barriers between the stages */
    CFPP_MODE_SPLIT = 1,     /* one plain launch per stage; the kernel boundary is the barrier */
    CFPP_MODE_FUSED_LAYERS = 2   /* cfpp_stack_* only: CFPP_MODE_FUSED with every layer a launch of its own, also where one
                                  * launch could run all layers (cfpp_stack_layers_per_launch); for comparison and profiling */
} cfpp_mode;

const char* cfpp_status_str(int status);
const char* cfpp_version(void);

/* Bytes of device scratch one layer call needs (256-byte aligned; zero it once before first use). */
size_t cfpp_neox_workspace_bytes(const cfpp_neox_dims* dims);

/* Full decoder-layer decode step.
 * Replaces pythia_2b8_decoder_layer_sm120 / pythia_6b9_decoder_layer_sm120 (reference
 * include/pybind.cpp:109-129,183-203; include/5090/pythia_2b8/pythia_kernel_dispatch.cu:4-251) in
 * CFPP_MODE_FUSED and pythia_2b8_decoder_layer_split_sm120 (include/pybind.cpp:132-151;
 * pythia_kernel_dispatch_split.cu:18-218) in CFPP_MODE_SPLIT. */
int cfpp_neox_layer_decode(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io,
                           int mode, void* workspace, size_t workspace_bytes, void* stream);

/* The same layer step for callers that cannot allocate device memory or pass a workspace around: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * The scratch memory that cfpp_neox_layer_decode takes as `workspace` is here an array inside the library
 * (cfpp_static_scratch_bytes() = 1.25 MiB per device, held until the process ends); the call allocates nothing and
 * frees nothing.  Geometries whose cfpp_neox_workspace_bytes exceeds that size return CFPP_ERR_STATIC_SCRATCH (both
 * Pythia models fit).  All calls on one device share the one array: calls on the same stream are ordered and fine,
 * calls that overlap in time on one device (two streams, two threads) race and give wrong results.  Every call
 * first clears the array's counters and flags with a small kernel (it keeps the previous call's contents), then
 * runs the same kernels as cfpp_neox_layer_decode: identical results, bit for bit.  cfpp_init() (device current) must
 * have run on the device before the first call: it creates the pinned word through which a device-side failure of
 * these launches is reported (cfpp_device_status; the status word inside the array is cleared by the next call and
 * cannot serve), which this entry point may not allocate itself.  Without it the call launches nothing and returns
 * CFPP_ERR_NOT_INITIALISED.  (Any other launching entry point of the library creates the word as well.) */
int cfpp_neox_layer_decode_static(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io,
                                  int mode, void* stream);
size_t cfpp_static_scratch_bytes(void);
/* Per-device set-up for the current device, done lazily by the other calls otherwise: compute-unit count, the
 * pinned failure-flag word (the one allocation, host memory), the address of the static scratch array. */
int cfpp_init(void);

/* First half of the split API: LN, QKV, RoPE, append, attention, O-proj (+b_o) -> io->attn_output,
 * and MLP-up + GELU -> io->mlp_intermediate; k_new / v_new / cache row as in the full layer.
 * `w->w_down`, `w->b_down` and `io->output` are ignored.
 * Replaces pythia_2b8_attention_only_sm120 (reference include/pybind.cpp:154-171;
 * pythia_kernel_dispatch_split.cu:225-359). */
int cfpp_neox_attention_mlp_up(const cfpp_neox_dims* dims, const cfpp_neox_weights* w, const cfpp_neox_io* io,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---- LLaMA attention block (sglang flavour) -------------------------------------------------------
 * r = fp16(input + residual) (stored back into `residual` when it is given; r = input otherwise);
 * n = RMSNorm(r; eps) * rms_w;  [q;k;v] = W_qkv n with W_qkv [3H, H] = [Wq; Wk; Wv] (not interleaved);
 * NeoX (rotate-half) RoPE over the whole head on q and k, cos/sin fp32 with >= head_dim/2 entries (the
 * angles of the pairs);  attention over cache rows [0, seq_len) plus the new token (the caches are NOT
 * written: k_new / v_new are returned and the caller appends);  output = W_o attn  (no bias, no residual).
 * Workspace: cfpp_llama_workspace_bytes, 256-byte aligned, zeroed once, one per stream.
 * Replaces llama_decoder_layer_sglang_sm120 (reference include/pybind.cpp:77-88;
 * include/5090/llama/llama_kernel_sglang_dispatch.cu:4-160; include/5090/llama/kernel_sglang.cuh). */
typedef struct cfpp_llama_attn {
    int32_t hidden, heads, head_dim;
    float eps;
    const void* rms_w;       /* [H] fp16 */
    const void* w_qkv;       /* [3H, H] fp16 */
    const void* w_o;         /* [H, H] fp16 */
    const void* input;       /* [H] fp16 */
    void* residual;          /* [H] fp16, in/out, may be NULL */
    void* output;            /* [H] fp16 */
    void* k_new;             /* [heads*D] fp16: rotated K of the new token */
    void* v_new;             /* [heads*D] fp16 */
    const void* k_cache;     /* [seq_len, H] fp16, read only */
    const void* v_cache;
    int32_t seq_len;         /* cache rows attended */
    const float* cos;        /* [>= D/2] fp32 */
    const float* sin;
    int32_t add_residual;    /* 0: output = W_o attn (the reference's op); 1: output = r + W_o attn (the layer's hidden state) */
    int32_t mode;            /* cfpp_mode: one launch, or one launch per stage (same results) */
} cfpp_llama_attn;

size_t cfpp_llama_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim);
int cfpp_llama_attention_decode(const cfpp_llama_attn* a, void* workspace, size_t workspace_bytes, void* stream);

/* The reference's plain op (llama_decoder_layer_sm120, reference include/pybind.cpp:66-75,280;
 * include/5090/llama/llama_kernel_dispatch.cu:4-145): output = W_o^T attn, no residual stream (residual must be NULL,
 * add_residual 0), weights stored [in, out]: w_qkv is [3H, H] = three [H_in, H_out] matrices for q, k, v stacked,
 * w_o is [H_in, H_out]; GPT-J pairing of the rotary dims (dim 2i with 2i+1; include/5090/llama/kernel.cuh:298-314)
 * with cos / sin tables of head_dim entries indexed by the dim (:280-281).  Caches are not written.  `mode` must be
 * CFPP_MODE_FUSED (0): the op has one variant, three launches.
 * Workspace: cfpp_llama_plain_workspace_bytes, 256-byte aligned, zero-initialised once, one per stream. */
size_t cfpp_llama_plain_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim);
int cfpp_llama_attention_plain(const cfpp_llama_attn* a, void* workspace, size_t workspace_bytes, void* stream);

/* ---- LLaMA MLP block ---------------------------------------------------------------------------------
 * output = input + W_down (silu(Wg n) * (Wu n)),  n = RMSNorm(input; eps) * rms_w,  w_gate_up = [Wg; Wu] ([2F, H]),
 * w_down [H, F].  One launch (norm, gated up rows in two phases, down rows + residual behind device-wide events) or
 * two (mode).  The reference fuses only the
 * attention block of a LLaMA layer (its test leaves the MLP commented out, reference tests/test_llama.py:108-110);
 * this completes the layer its benchmark configuration describes.
 * Workspace: cfpp_llama_mlp_workspace_bytes, 256-byte aligned, zero-initialised once, one per stream. */
typedef struct cfpp_llama_mlp_args {
    int32_t hidden, ffn;
    float eps;
    const void* rms_w;       /* [H] fp16 */
    const void* w_gate_up;   /* [2F, H] fp16 */
    const void* w_down;      /* [H, F] fp16 */
    const void* input;       /* [H] fp16 */
    void* output;            /* [H] fp16 */
    int32_t mode;            /* cfpp_mode: one launch, or two (gate/up rows, then down rows; same results) */
} cfpp_llama_mlp_args;

size_t cfpp_llama_mlp_workspace_bytes(int32_t hidden, int32_t ffn);
int cfpp_llama_mlp(const cfpp_llama_mlp_args* m, void* workspace, size_t workspace_bytes, void* stream);

/* ---- LLaMA attention block for a batch of sequences over paged caches ------------------------------------
 * Replaces llama_decoder_layer_batch_sglang_sm120 (reference include/pybind.cpp:90-106;
 * include/5090/llama/llama_kernel_batch_sglang_dispatch.cu:6-110; kernel_batch_sglang.cuh:43-60 arguments, :120-123
 * page table, :343-367 RoPE from cos_sin[position] and the write of the new K/V row).  For every sequence b:
 *   r = fp16(input[b] + residual[b]) -> residual_out[b];  n = RMSNorm(r) * rms_w;  [q;k;v] = W_qkv n;  NeoX RoPE over
 *   the whole head with cos_sin[positions[b]] (D/2 cosines, then D/2 sines);  the new k, v rows are stored in cache
 *   row paged_kv_indices[paged_kv_indptr[b+1] - 1];  attention over the rows paged_kv_indices[paged_kv_indptr[b] ..
 *   paged_kv_indptr[b+1] - 1) and the new token;  output[b] = W_o attn (no residual).
 * Caches are [rows, H] fp16 with head-major columns (page size 1); k_cache_ptrs / v_cache_ptrs are device arrays of
 * their base addresses per layer, read on the device.  All index arrays live in device memory and are not read by
 * the host.  residual_out must not alias input or residual (CFPP_ERR_ALIAS).
 * Workspace: cfpp_llama_batch_workspace_bytes, 256-byte aligned, zero-initialised once, one per stream. */
typedef struct cfpp_llama_batch {
    int32_t hidden, heads, head_dim;
    float eps;
    int32_t batch, layer_id;
    const void* rms_w;                /* [H] fp16 */
    const void* w_qkv;                /* [3H, H] fp16 = [Wq; Wk; Wv] */
    const void* w_o;                  /* [H, H] fp16 */
    const void* input;                /* [batch, H] fp16 */
    const void* residual;             /* [batch, H] fp16 */
    void* residual_out;               /* [batch, H] fp16 */
    void* output;                     /* [batch, H] fp16 */
    const int32_t* paged_kv_indptr;   /* [batch + 1] */
    const int32_t* paged_kv_indices;  /* [paged_kv_indptr[batch]] cache rows */
    const uint64_t* k_cache_ptrs;     /* [layers] */
    const uint64_t* v_cache_ptrs;     /* [layers] */
    const int64_t* positions;         /* [batch] */
    const float* cos_sin;             /* [max_position, D] fp32 */
} cfpp_llama_batch;

size_t cfpp_llama_batch_workspace_bytes(int32_t hidden, int32_t heads, int32_t head_dim, int32_t batch);
int cfpp_llama_batch_decode(const cfpp_llama_batch* a, void* workspace, size_t workspace_bytes, void* stream);

/* Second half: output = input + attn_output + W_down mlp_intermediate + b_down.
 * Replaces pythia_2b8_mlp_only_sm120 (reference include/pybind.cpp:174-180;
 * pythia_kernel_dispatch_split.cu:364-426).  `workspace` / `workspace_bytes` are not used (the call needs no scratch
 * memory; NULL / 0 are fine): they keep the argument list of the two halves alike. */
int cfpp_neox_mlp_down(const cfpp_neox_dims* dims, const void* input, const void* attn_output,
                       const void* mlp_intermediate, const void* w_down, const void* b_down, void* output,
                       void* workspace, size_t workspace_bytes, void* stream);

/* ---- per-layer decode contexts (persistent buffers keyed by an integer id) --------------------
 * Replaces PythiaGraphContext + create / graph_decode_step / destroy (reference
 * include/5090/pythia_2b8/pythia_kernel_dispatch_graph.cu:50-294 and the 6.9B twin;
 * include/pybind.cpp:206-267).  `family` separates the id spaces the reference keeps in two maps
 * (g_contexts / g_contexts_6b9): 0 = 2.8B ops, 1 = 6.9B ops, any other int = caller-defined. */
typedef struct cfpp_ctx_buffers {
    void* output;   /* [H] fp16, context-owned, overwritten by the next step */
    void* k_new;    /* [heads*D] fp16 */
    void* v_new;    /* [heads*D] fp16 */
} cfpp_ctx_buffers;

/* Allocates the context's output buffers and workspace on the current device (hipMalloc).
 * Duplicate id: the old context is destroyed and replaced (the reference silently overwrites). */
int cfpp_ctx_create(int family, int64_t id, const cfpp_neox_dims* dims, const void* w_qkv, const void* w_o,
                    const void* w_up, const void* w_down, void* k_cache, void* v_cache, int32_t cache_rows,
                    int32_t max_seq_len, cfpp_ctx_buffers* out_buffers);

/* One decode step on the context's buffers; `w` carries the small vectors (the four matrices in it
 * must be NULL or equal to those given at create), `io->output/k_new/v_new` are ignored, and
 * io->k_cache / v_cache must equal the create-time pointers (CFPP_ERR_CONTEXT otherwise).
 * Unknown id -> CFPP_ERR_CONTEXT.  Allocates nothing, never synchronises: capturable in a hipGraph
 * when io->d_seq_len is used. */
int cfpp_ctx_step(int family, int64_t id, const cfpp_neox_weights* w, const cfpp_neox_io* io, int mode,
                  void* stream, cfpp_ctx_buffers* out_buffers);

/* Frees the context's buffers; unknown id is a no-op returning CFPP_OK. */
int cfpp_ctx_destroy(int family, int64_t id);

/* Reads and clears the device-side failure flag of a workspace (synchronises `stream`); a workspace with a raised
 * flag is zeroed again.  Returns CFPP_OK or CFPP_ERR_DEVICE.  Not on the hot path.  cfpp_ctx_check / cfpp_stack_check
 * (below) do the same for the workspace a context or a stack owns. */
int cfpp_workspace_check(const cfpp_neox_dims* dims, void* workspace, void* stream);
int cfpp_ctx_check(int family, int64_t id, void* stream);

/* Failure flags raised by any launch on the current device since they were last cleared (bit 0: a bounded
 * device-side wait expired; bit 1: a device-side seq_len was out of range), read from pinned host memory (one word per flag)
 * that the kernels write on failure: no device synchronisation, callable at any time; flags of launches still
 * running are seen once they got there.  `clear` != 0 resets the word.  While it is non-zero every launching entry
 * point returns CFPP_ERR_DEVICE.  No counterpart in the reference (which checks no error at all). */
int cfpp_device_status(int clear);

/* The rule by which CFPP_MODE_FUSED decides whether a one-launch kernel may be launched: 1 when `grid` workgroups
 * fit `compute_units` x `blocks_per_cu` resident workgroups, else 0 (the per-stage launches are taken).  The
 * reference gets the same guarantee from cudaLaunchCooperativeKernel, which refuses a grid that cannot be
 * co-resident (include/5090/pythia_2b8/pythia_kernel_dispatch.cu:242). */
int cfpp_one_launch_fits(int grid, int compute_units, int blocks_per_cu);

/* ---- whole-model greedy decode (our counterpart of the reference's Python decode loop,
 * tests/benchmark_decode.py:147-189: embedding row -> layers -> final LayerNorm -> LM head ->
 * argmax), captured once into a hipGraph and replayed per token ------------------------------- */
typedef struct cfpp_neox_stack_desc {
    cfpp_neox_dims dims;
    int32_t n_layers;
    int32_t vocab;                     /* 1 .. 524288 */
    const cfpp_neox_weights* layers;   /* host array [n_layers] of device pointers */
    const void* embed;                 /* [vocab, H] fp16 */
    const void* final_ln_w;            /* [H] fp16 */
    const void* final_ln_b;
    const void* lm_head;               /* [vocab, H] fp16 */
    void* const* k_caches;             /* host array [n_layers] of device pointers [cache_rows, H] */
    void* const* v_caches;
    int32_t cache_rows;
    const float* rope_cos;             /* [cache_rows, rotary_dim] fp32 table indexed by position */
    const float* rope_sin;
    int32_t mode;                      /* cfpp_mode used for every layer (CFPP_MODE_FUSED_LAYERS allowed) */
} cfpp_neox_stack_desc;

typedef struct cfpp_neox_stack cfpp_neox_stack;   /* opaque */

/* Allocates state (device int32 seq_len + token, hidden ping-pong, logits, workspace). */
int cfpp_stack_create(const cfpp_neox_stack_desc* desc, cfpp_neox_stack** out);
/* Sets the device-resident (token, seq_len) the next step starts from and fetches that token's embedding row
 * (async on `stream`); seq_len < cache_rows.  The step calls below return CFPP_ERR_SEQ instead of running past
 * the last cache row. */
int cfpp_stack_set_state(cfpp_neox_stack* s, int32_t token, int32_t seq_len, void* stream);
/* One decode step launched eagerly: consumes (token, seq_len), appends K/V rows, writes logits,
 * then stores argmax as the new token and seq_len+1 and fetches the new token's embedding row (the LM head
 * launch does all of that: a step is n_layers + 1 launches in fused mode, or 2 when one launch runs all layers,
 * see cfpp_stack_layers_per_launch). */
int cfpp_stack_step(cfpp_neox_stack* s, void* stream);
/* Captures one step into a hipGraph (first call) and replays it `n_steps` times on `stream`. */
int cfpp_stack_graph_steps(cfpp_neox_stack* s, int32_t n_steps, void* stream);
/* Decoder layers that one launch of a step runs: n_layers when the stack runs all of them in a single launch (fused
 * mode, the whole grid co-resident, a hidden size of whole 512-column chunks: the layers then hand their rows over inside
 * the launch), 1 when every layer is a launch (or three, in split mode) of its own.  Fixed at creation.  CFPP_ERR_NULL
 * (negative) for a null stack. */
int cfpp_stack_layers_per_launch(const cfpp_neox_stack* s);
/* One eager decode step with a HIP event before and after every layer launch and the LM head, on
 * `stream`; synchronises.  layer_ms[n_layers], *lm_head_ms and *total_ms (whole step) receive elapsed
 * milliseconds (when one launch runs all layers, every layer_ms is that launch's duration / n_layers).  For
 * measurement; advances the state like cfpp_stack_step. */
int cfpp_stack_profile_step(cfpp_neox_stack* s, void* stream, float* layer_ms, float* lm_head_ms, float* total_ms);
/* Device pointers for inspection (read only: the token is changed through cfpp_stack_set_state, which also
 * fetches its embedding row): logits fp32 [vocab], hidden fp16 [H] after the last layer,
 * state int32[3] = {token, seq_len, steps done}, token history int32 [history_capacity]. */
int cfpp_stack_buffers(cfpp_neox_stack* s, float** logits, void** hidden, int32_t** state,
                       int32_t** history, int32_t* history_capacity);
/* cfpp_workspace_check for the stack's own workspace (synchronises `stream`). */
int cfpp_stack_check(cfpp_neox_stack* s, void* stream);
int cfpp_stack_destroy(cfpp_neox_stack* s);

/* Final LayerNorm + LM-head GEMV: logits[v] = W[v,:] . LN(x) (no bias), fp32 logits; vocab <= 524288.
 * Counterpart of F.layer_norm + embed_out in the reference loop (tests/benchmark_decode.py:180-187). */
int cfpp_neox_lm_head(int32_t hidden, int32_t vocab, float eps, const void* x, const void* ln_w,
                      const void* ln_b, const void* w, float* logits, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CFPP_H */
