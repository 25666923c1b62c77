// PyTorch-ROCm binding: the `clusterfusion` Python operator surface on top of the C ABI (cfpp.h).
//
// Same Python names, positional argument order and return tuples as the reference's binding table
// (reference include/pybind.cpp:280-297); the reference's C++ forward declarations that fix the
// argument meaning are include/pybind.cpp:109-267.  Differences, all on the safe side:
//   * every tensor is validated (device, dtype, contiguity, element count, cache capacity) and a bad
//     argument raises RuntimeError instead of reading out of bounds (the reference checks nothing);
//   * launches go to torch's current HIP stream without device-wide synchronisation;
//   * a cache with exactly `current_seq_len` rows is accepted: the append is skipped, k/v are returned;
//   * `graph_decode_step` also accepts a device int32 tensor as `current_seq_len` (with cos/sin given
//     as `[positions, rotary_dim]` tables), which makes the step replayable from a captured HIP graph.
// This file contains no device code; torch is used for tensors, streams and exceptions only.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <dlfcn.h>

#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "cfpp.h"

namespace {

using torch::Tensor;

struct Model {
    const char* name;
    int family;
    cfpp_neox_dims dims;
};
const Model kPythia2b8{"pythia_2b8", 0, {2560, 32, 80, 20, 10240, 1e-5f}};
const Model kPythia6b9{"pythia_6b9", 1, {4096, 32, 128, 32, 16384, 1e-5f}};

// Scratch buffers handed to the C ABI, one per (device, stream, geometry): calls on one stream are ordered, so they
// can share one.  Zero-initialised; the kernels leave their counters at zero after every call.
struct ScratchKey {
    int device; void* stream; int kind; int a, b, c, d;
    bool operator<(const ScratchKey& o) const {
        return std::tie(device, stream, kind, a, b, c, d) < std::tie(o.device, o.stream, o.kind, o.a, o.b, o.c, o.d);
    }
};
std::mutex g_scratch_mu;
std::map<ScratchKey, torch::Tensor> g_scratch;

void check_rc(int rc, const char* what) {
    if (rc == CFPP_ERR_DEVICE) {
        // a launch on this device has raised a failure flag: report it once, clear it, and drop the scratch buffers
        // (an expired wait leaves counters mid-flight; new buffers start from zero)
        const int flags = cfpp_device_status(1);
        {
            std::lock_guard<std::mutex> lock(g_scratch_mu);
            g_scratch.clear();
        }
        TORCH_CHECK(false, what, ": ", cfpp_status_str(rc), " (flags ", flags,
                    ": 1 = a bounded device-side wait expired, is other work running on the GPU?; 2 = a device-side "
                    "current_seq_len was out of range); results since the last successful check are invalid");
    }
    TORCH_CHECK(rc == 0, what, ": ", cfpp_status_str(rc), " (status ", rc, ")");
}

void check_half(const Tensor& t, const char* name, int64_t numel, const Tensor& like) {
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(t.device() == like.device(), name, " is on ", t.device(), " but input is on ", like.device());
    TORCH_CHECK(t.scalar_type() == torch::kFloat16, name, " must be float16, got ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.numel() == numel, name, " must have ", numel, " elements, got ", t.numel());
}

void check_rope(const Tensor& t, const char* name, int64_t min_numel, const Tensor& like) {
    TORCH_CHECK(t.defined() && t.is_cuda() && t.device() == like.device(), name, " must be a GPU tensor on the input's device");
    TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be float32, got ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.numel() >= min_numel, name, " must have at least ", min_numel, " elements, got ", t.numel());
}

int64_t check_cache(const Tensor& t, const char* name, int64_t H, const Tensor& like) {
    TORCH_CHECK(t.defined() && t.is_cuda() && t.device() == like.device(), name, " must be a GPU tensor on the input's device");
    TORCH_CHECK(t.scalar_type() == torch::kFloat16, name, " must be float16");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.dim() == 2 && t.size(1) == H, name, " must have shape [rows, ", H, "]");
    return t.size(0);
}

Tensor scratch_for(const ScratchKey& key, int64_t bytes, const torch::Device& dev) {
    TORCH_CHECK(bytes > 0, "unsupported layer dimensions");
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    auto it = g_scratch.find(key);
    if (it != g_scratch.end() && it->second.numel() >= bytes + 256) return it->second;
    Tensor ws = torch::zeros({bytes + 256}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
    g_scratch[key] = ws;
    return ws;
}
// The layout of a layer workspace depends on every dimension but the rotary one, so all of them are in the key: a
// buffer is never reused under another layout (its counters would sit on stale data).
Tensor workspace_for(const cfpp_neox_dims& d, const torch::Device& dev, hipStream_t st) {
    return scratch_for(ScratchKey{(int)dev.index(), (void*)st, 0, d.hidden, d.heads, d.head_dim, d.ffn},
                       (int64_t)cfpp_neox_workspace_bytes(&d), dev);
}
void* ws_ptr(const Tensor& ws) {
    auto p = reinterpret_cast<uintptr_t>(ws.data_ptr());
    return reinterpret_cast<void*>((p + 255) / 256 * 256);
}
// bytes of the tensor that remain behind the aligned pointer: what the C ABI checks its needs against
size_t ws_capacity(const Tensor& ws) {
    return (size_t)ws.numel() - (size_t)(reinterpret_cast<uintptr_t>(ws_ptr(ws)) - reinterpret_cast<uintptr_t>(ws.data_ptr()));
}

struct LayerArgs {
    Tensor input, weight_qkv, bias_qkv, weight_o, bias_o, k_cache, v_cache, ln_w, ln_b, cos, sin, post_ln_w,
        post_ln_b, up_w, up_b, down_w, down_b;
};

void fill_weights(const cfpp_neox_dims& d, const LayerArgs& a, bool need_down, cfpp_neox_weights* w) {
    const int64_t H = d.hidden, F = d.ffn;
    check_half(a.input, "input", H, a.input);
    check_half(a.weight_qkv, "weight_qkv", 3 * H * H, a.input);
    check_half(a.bias_qkv, "bias_qkv", 3 * H, a.input);
    check_half(a.weight_o, "weight_o", H * H, a.input);
    check_half(a.bias_o, "bias_o", H, a.input);
    check_half(a.ln_w, "layernorm_weight", H, a.input);
    check_half(a.ln_b, "layernorm_bias", H, a.input);
    check_half(a.post_ln_w, "post_ln_weight", H, a.input);
    check_half(a.post_ln_b, "post_ln_bias", H, a.input);
    check_half(a.up_w, "mlp_up_weight", F * H, a.input);
    check_half(a.up_b, "mlp_up_bias", F, a.input);
    if (need_down) {
        check_half(a.down_w, "mlp_down_weight", H * F, a.input);
        check_half(a.down_b, "mlp_down_bias", H, a.input);
    }
    w->ln_w = a.ln_w.data_ptr(); w->ln_b = a.ln_b.data_ptr();
    w->w_qkv = a.weight_qkv.data_ptr(); w->b_qkv = a.bias_qkv.data_ptr();
    w->w_o = a.weight_o.data_ptr(); w->b_o = a.bias_o.data_ptr();
    w->post_ln_w = a.post_ln_w.data_ptr(); w->post_ln_b = a.post_ln_b.data_ptr();
    w->w_up = a.up_w.data_ptr(); w->b_up = a.up_b.data_ptr();
    w->w_down = need_down ? a.down_w.data_ptr() : nullptr;
    w->b_down = need_down ? a.down_b.data_ptr() : nullptr;
}

void fill_io(const cfpp_neox_dims& d, const LayerArgs& a, int64_t seq_len, cfpp_neox_io* io) {
    const int64_t H = d.hidden;
    const int64_t rows_k = check_cache(a.k_cache, "k_cache", H, a.input);
    const int64_t rows_v = check_cache(a.v_cache, "v_cache", H, a.input);
    TORCH_CHECK(seq_len >= 0, "current_seq_len must be >= 0, got ", seq_len);
    TORCH_CHECK(rows_k >= seq_len && rows_v >= seq_len, "current_seq_len ", seq_len, " exceeds the cache rows (k ",
                rows_k, ", v ", rows_v, ")");
    check_rope(a.cos, "cos", d.rotary_dim, a.input);
    check_rope(a.sin, "sin", d.rotary_dim, a.input);
    *io = cfpp_neox_io{};
    io->input = a.input.data_ptr();
    io->k_cache = a.k_cache.data_ptr(); io->v_cache = a.v_cache.data_ptr();
    io->cache_rows = (int32_t)std::min(rows_k, rows_v);
    io->cos = a.cos.data_ptr<float>(); io->sin = a.sin.data_ptr<float>();
    io->rope_stride = 0;
    io->seq_len = (int32_t)seq_len;
}

std::tuple<Tensor, Tensor, Tensor> decoder_layer(const Model& m, int mode, const LayerArgs& a, int64_t seq_len) {
    const cfpp_neox_dims& d = m.dims;
    cfpp_neox_weights w;
    cfpp_neox_io io;
    fill_weights(d, a, true, &w);
    fill_io(d, a, seq_len, &io);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(a.input.device());
    auto opts = a.input.options();
    Tensor out = torch::empty({1, d.hidden}, opts);
    Tensor k = torch::empty({1, d.heads, d.head_dim}, opts);
    Tensor v = torch::empty({1, d.heads, d.head_dim}, opts);
    io.output = out.data_ptr(); io.k_new = k.data_ptr(); io.v_new = v.data_ptr();
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    Tensor ws = workspace_for(d, a.input.device(), st);
    check_rc(cfpp_neox_layer_decode(&d, &w, &io, mode, ws_ptr(ws), ws_capacity(ws), st), m.name);
    return std::make_tuple(out, k, v);
}

std::tuple<Tensor, Tensor, Tensor, Tensor> attention_only(const Model& m, const LayerArgs& a, int64_t seq_len) {
    const cfpp_neox_dims& d = m.dims;
    cfpp_neox_weights w;
    cfpp_neox_io io;
    fill_weights(d, a, false, &w);
    fill_io(d, a, seq_len, &io);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(a.input.device());
    auto opts = a.input.options();
    Tensor attn = torch::empty({1, d.hidden}, opts);
    Tensor inter = torch::empty({d.ffn}, opts);
    Tensor k = torch::empty({1, d.heads, d.head_dim}, opts);
    Tensor v = torch::empty({1, d.heads, d.head_dim}, opts);
    io.attn_output = attn.data_ptr(); io.mlp_intermediate = inter.data_ptr();
    io.k_new = k.data_ptr(); io.v_new = v.data_ptr();
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    Tensor ws = workspace_for(d, a.input.device(), st);
    check_rc(cfpp_neox_attention_mlp_up(&d, &w, &io, ws_ptr(ws), ws_capacity(ws), st), m.name);
    return std::make_tuple(attn, inter, k, v);
}

Tensor mlp_only(const Model& m, Tensor input, Tensor attn_output, Tensor inter, Tensor down_w, Tensor down_b) {
    const cfpp_neox_dims& d = m.dims;
    check_half(input, "input", d.hidden, input);
    check_half(attn_output, "attn_output", d.hidden, input);
    check_half(inter, "mlp_intermediate", d.ffn, input);
    check_half(down_w, "mlp_down_weight", (int64_t)d.hidden * d.ffn, input);
    check_half(down_b, "mlp_down_bias", d.hidden, input);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    Tensor out = torch::empty({1, d.hidden}, input.options());
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(cfpp_neox_mlp_down(&d, input.data_ptr(), attn_output.data_ptr(), inter.data_ptr(), down_w.data_ptr(),
                                down_b.data_ptr(), out.data_ptr(), nullptr, 0, st), m.name);
    return out;
}

// ---- decode contexts -----------------------------------------------------------------------------
struct PyCtx {
    Tensor k_cache, v_cache, w_qkv, w_o, w_up, w_down;   // keep the storage alive (the reference keeps raw pointers)
    Tensor output, k_new, v_new;                          // views of the context-owned device buffers
};
std::mutex g_mu;
std::map<std::pair<int, int64_t>, PyCtx> g_ctx;

void create_graph_context(const Model& m, int64_t id, Tensor k_cache, Tensor v_cache, Tensor w_qkv, Tensor w_o,
                          Tensor w_up, Tensor w_down, int64_t max_seq_len) {
    const cfpp_neox_dims& d = m.dims;
    const int64_t H = d.hidden, F = d.ffn;
    const int64_t rows_k = check_cache(k_cache, "k_cache", H, k_cache);
    const int64_t rows_v = check_cache(v_cache, "v_cache", H, k_cache);
    check_half(w_qkv, "weight_qkv", 3 * H * H, k_cache);
    check_half(w_o, "weight_o", H * H, k_cache);
    check_half(w_up, "mlp_up_weight", F * H, k_cache);
    check_half(w_down, "mlp_down_weight", H * F, k_cache);
    const int64_t rows = std::min(rows_k, rows_v);
    TORCH_CHECK(max_seq_len > 0 && max_seq_len <= rows, "max_seq_len ", max_seq_len, " must be in [1, cache rows = ", rows, "]");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(k_cache.device());
    cfpp_ctx_buffers b{};
    check_rc(cfpp_ctx_create(m.family, id, &d, w_qkv.data_ptr(), w_o.data_ptr(), w_up.data_ptr(), w_down.data_ptr(),
                             k_cache.data_ptr(), v_cache.data_ptr(), (int32_t)rows, (int32_t)max_seq_len, &b),
             "create_graph_context");
    auto opts = k_cache.options();
    PyCtx c{k_cache, v_cache, w_qkv, w_o, w_up, w_down,
            torch::from_blob(b.output, {1, H}, opts),
            torch::from_blob(b.k_new, {1, (int64_t)d.heads, (int64_t)d.head_dim}, opts),
            torch::from_blob(b.v_new, {1, (int64_t)d.heads, (int64_t)d.head_dim}, opts)};
    std::lock_guard<std::mutex> lock(g_mu);
    g_ctx[std::make_pair(m.family, id)] = c;
}

std::tuple<Tensor, Tensor, Tensor> graph_decode_step(const Model& m, int64_t id, Tensor input, Tensor ln_w, Tensor ln_b,
                                                     Tensor qkv_bias, Tensor o_bias, Tensor cos, Tensor sin, Tensor k_cache,
                                                     Tensor v_cache, Tensor post_ln_w, Tensor post_ln_b, Tensor up_b,
                                                     Tensor down_b, py::object current_seq_len) {
    const cfpp_neox_dims& d = m.dims;
    PyCtx c;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = g_ctx.find(std::make_pair(m.family, id));
        // the reference raises std::runtime_error("Graph context not initialized...") here
        // (include/5090/pythia_2b8/pythia_kernel_dispatch_graph.cu:231-233)
        TORCH_CHECK(it != g_ctx.end(), "Graph context ", id, " not initialized: call ", m.name, "_create_graph_context first");
        c = it->second;
    }
    const int64_t H = d.hidden, F = d.ffn;
    check_half(input, "input", H, input);
    check_half(ln_w, "layernorm_weight", H, input);
    check_half(ln_b, "layernorm_bias", H, input);
    check_half(qkv_bias, "qkv_bias", 3 * H, input);
    check_half(o_bias, "o_bias", H, input);
    check_half(post_ln_w, "post_ln_weight", H, input);
    check_half(post_ln_b, "post_ln_bias", H, input);
    check_half(up_b, "mlp_up_bias", F, input);
    check_half(down_b, "mlp_down_bias", H, input);
    TORCH_CHECK(k_cache.data_ptr() == c.k_cache.data_ptr() && v_cache.data_ptr() == c.v_cache.data_ptr(),
                "k_cache / v_cache differ from the tensors the context was created with");
    check_rope(cos, "cos", d.rotary_dim, input);
    check_rope(sin, "sin", d.rotary_dim, input);

    cfpp_neox_weights w{};
    w.ln_w = ln_w.data_ptr(); w.ln_b = ln_b.data_ptr(); w.b_qkv = qkv_bias.data_ptr(); w.b_o = o_bias.data_ptr();
    w.post_ln_w = post_ln_w.data_ptr(); w.post_ln_b = post_ln_b.data_ptr(); w.b_up = up_b.data_ptr(); w.b_down = down_b.data_ptr();
    cfpp_neox_io io{};
    io.input = input.data_ptr();
    io.k_cache = k_cache.data_ptr(); io.v_cache = v_cache.data_ptr();
    io.cos = cos.data_ptr<float>(); io.sin = sin.data_ptr<float>();
    const int64_t rows = std::min(c.k_cache.size(0), c.v_cache.size(0));
    Tensor seq_t;
    if (THPVariable_Check(current_seq_len.ptr())) {
        seq_t = THPVariable_Unpack(current_seq_len.ptr());
        TORCH_CHECK(seq_t.is_cuda() && seq_t.device() == input.device() && seq_t.scalar_type() == torch::kInt32 && seq_t.numel() == 1,
                    "a tensor current_seq_len must be one int32 on the input's device");
        TORCH_CHECK(cos.dim() == 2 && sin.dim() == 2 && cos.size(1) >= d.rotary_dim && cos.sizes() == sin.sizes() &&
                        cos.size(0) >= rows,
                    "with a tensor current_seq_len, cos/sin must be [positions >= cache rows, >= rotary_dim] tables");
        io.d_seq_len = seq_t.data_ptr<int32_t>();
        io.rope_stride = (int32_t)cos.size(1);
    } else {
        const int64_t s = current_seq_len.cast<int64_t>();
        TORCH_CHECK(s >= 0 && s <= rows, "current_seq_len ", s, " out of range for ", rows, " cache rows");
        io.seq_len = (int32_t)s;
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_rc(cfpp_ctx_step(m.family, id, &w, &io, CFPP_MODE_FUSED, st, nullptr), "graph_decode_step");
    return std::make_tuple(c.output, c.k_new, c.v_new);
}

void destroy_graph_context(const Model& m, int64_t id) {
    bool known = false;
    torch::Device dev{torch::kCPU};
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = g_ctx.find(std::make_pair(m.family, id));
        if (it != g_ctx.end()) { known = true; dev = it->second.k_cache.device(); g_ctx.erase(it); }
    }
    // the last chance to learn that a step of this context failed on the device (an expired wait, a device-side
    // current_seq_len out of range): read its status word before the buffers go
    int status = CFPP_OK;
    if (known) {
        c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
        status = cfpp_ctx_check(m.family, id, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    }
    check_rc(cfpp_ctx_destroy(m.family, id), "destroy_graph_context");
    check_rc(status, "destroy_graph_context (steps of this context)");
}

// ---- whole-model decode (our counterpart of the reference's Python decode loop) --------------------
struct PyStack {
    cfpp_neox_stack* s = nullptr;
    std::vector<Tensor> keep;
    cfpp_neox_dims dims{};
    int64_t vocab = 0;
    int64_t n_layers = 0;
    torch::Device device{torch::kCPU};
    ~PyStack() { if (s) cfpp_stack_destroy(s); }
};

std::shared_ptr<PyStack> stack_create(int64_t hidden, int64_t heads, int64_t head_dim, int64_t rotary_dim, int64_t ffn,
                                      double eps, std::vector<std::vector<Tensor>> layers, Tensor embed, Tensor final_ln_w,
                                      Tensor final_ln_b, Tensor lm_head, std::vector<Tensor> k_caches,
                                      std::vector<Tensor> v_caches, Tensor rope_cos, Tensor rope_sin, int64_t mode) {
    auto ps = std::make_shared<PyStack>();
    cfpp_neox_dims d{(int32_t)hidden, (int32_t)heads, (int32_t)head_dim, (int32_t)rotary_dim, (int32_t)ffn, (float)eps};
    ps->dims = d;
    const int64_t H = hidden, F = ffn, L = (int64_t)layers.size();
    TORCH_CHECK(L > 0 && (int64_t)k_caches.size() == L && (int64_t)v_caches.size() == L, "need one K and V cache per layer");
    TORCH_CHECK(embed.dim() == 2 && embed.size(1) == H, "embed must be [vocab, H]");
    const int64_t V = embed.size(0);
    check_half(embed, "embed", V * H, embed);
    check_half(lm_head, "lm_head", V * H, embed);
    check_half(final_ln_w, "final_ln_weight", H, embed);
    check_half(final_ln_b, "final_ln_bias", H, embed);
    std::vector<cfpp_neox_weights> lw(L);
    std::vector<void*> kc(L), vc(L);
    int64_t rows = -1;
    for (int64_t l = 0; l < L; ++l) {
        TORCH_CHECK(layers[l].size() == 12, "each layer is 12 tensors: ln_w ln_b w_qkv b_qkv w_o b_o post_ln_w post_ln_b w_up b_up w_down b_down");
        const int64_t numel[12] = {H, H, 3 * H * H, 3 * H, H * H, H, H, H, F * H, F, H * F, H};
        for (int i = 0; i < 12; ++i) { check_half(layers[l][i], "layer tensor", numel[i], embed); ps->keep.push_back(layers[l][i]); }
        const void* q[12];
        for (int i = 0; i < 12; ++i) q[i] = layers[l][i].data_ptr();
        lw[l] = cfpp_neox_weights{q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], q[8], q[9], q[10], q[11]};
        const int64_t rk = check_cache(k_caches[l], "k_cache", H, embed), rv = check_cache(v_caches[l], "v_cache", H, embed);
        TORCH_CHECK(rk == rv && (rows < 0 || rows == rk), "all caches must have the same number of rows");
        rows = rk;
        kc[l] = k_caches[l].data_ptr(); vc[l] = v_caches[l].data_ptr();
        ps->keep.push_back(k_caches[l]); ps->keep.push_back(v_caches[l]);
    }
    check_rope(rope_cos, "rope_cos", rows * rotary_dim, embed);
    check_rope(rope_sin, "rope_sin", rows * rotary_dim, embed);
    TORCH_CHECK(rope_cos.dim() == 2 && rope_cos.size(1) == rotary_dim && rope_sin.sizes() == rope_cos.sizes(),
                "rope tables must be [positions, rotary_dim]");
    for (const Tensor& t : {embed, final_ln_w, final_ln_b, lm_head, rope_cos, rope_sin}) ps->keep.push_back(t);
    cfpp_neox_stack_desc desc{};
    desc.dims = d; desc.n_layers = (int32_t)L; desc.vocab = (int32_t)V;
    desc.layers = lw.data(); desc.embed = embed.data_ptr(); desc.final_ln_w = final_ln_w.data_ptr();
    desc.final_ln_b = final_ln_b.data_ptr(); desc.lm_head = lm_head.data_ptr();
    desc.k_caches = kc.data(); desc.v_caches = vc.data(); desc.cache_rows = (int32_t)rows;
    desc.rope_cos = rope_cos.data_ptr<float>(); desc.rope_sin = rope_sin.data_ptr<float>();
    desc.mode = (int32_t)mode;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(embed.device());
    check_rc(cfpp_stack_create(&desc, &ps->s), "stack_create");
    ps->vocab = V;
    ps->n_layers = L;
    ps->device = embed.device();
    return ps;
}

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

}  // namespace

#define LAYER_ARGS                                                                                                     \
    Tensor input, Tensor weight_qkv, Tensor bias_qkv, Tensor weight_o, Tensor bias_o, Tensor k_cache, Tensor v_cache, \
        Tensor layernorm_weight, Tensor layernorm_bias, Tensor cos, Tensor sin, Tensor post_ln_weight,                \
        Tensor post_ln_bias, Tensor mlp_up_weight, Tensor mlp_up_bias
#define LAYER_PACK(dw, db)                                                                                              \
    LayerArgs { input, weight_qkv, bias_qkv, weight_o, bias_o, k_cache, v_cache, layernorm_weight, layernorm_bias, cos, \
                sin, post_ln_weight, post_ln_bias, mlp_up_weight, mlp_up_bias, dw, db }

#define DEFINE_MODEL_OPS(m, MODEL)                                                                                     \
    m.def(#MODEL "_decoder_layer", [](LAYER_ARGS, Tensor mlp_down_weight, Tensor mlp_down_bias, int64_t current_seq_len) { \
        return decoder_layer(k##MODEL, CFPP_MODE_FUSED, LAYER_PACK(mlp_down_weight, mlp_down_bias), current_seq_len);  \
    });                                                                                                                \
    m.def(#MODEL "_decoder_layer_split", [](LAYER_ARGS, Tensor mlp_down_weight, Tensor mlp_down_bias, int64_t current_seq_len) { \
        return decoder_layer(k##MODEL, CFPP_MODE_SPLIT, LAYER_PACK(mlp_down_weight, mlp_down_bias), current_seq_len);  \
    });                                                                                                                \
    m.def(#MODEL "_attention_only", [](LAYER_ARGS, int64_t current_seq_len) {                                          \
        return attention_only(k##MODEL, LAYER_PACK(Tensor(), Tensor()), current_seq_len);                              \
    });                                                                                                                \
    m.def(#MODEL "_mlp_only", [](Tensor input, Tensor attn_output, Tensor mlp_intermediate, Tensor mlp_down_weight,    \
                                 Tensor mlp_down_bias) {                                                               \
        return mlp_only(k##MODEL, input, attn_output, mlp_intermediate, mlp_down_weight, mlp_down_bias);               \
    });                                                                                                                \
    m.def(#MODEL "_create_graph_context", [](int64_t context_id, Tensor k_cache, Tensor v_cache, Tensor weight_qkv,    \
                                             Tensor weight_o, Tensor mlp_up_weight, Tensor mlp_down_weight,            \
                                             int64_t max_seq_len) {                                                    \
        create_graph_context(k##MODEL, context_id, k_cache, v_cache, weight_qkv, weight_o, mlp_up_weight,              \
                             mlp_down_weight, max_seq_len);                                                            \
    });                                                                                                                \
    m.def(#MODEL "_graph_decode_step", [](int64_t context_id, Tensor input, Tensor layernorm_weight,                   \
                                          Tensor layernorm_bias, Tensor qkv_bias, Tensor o_bias, Tensor cos, Tensor sin, \
                                          Tensor k_cache, Tensor v_cache, Tensor post_ln_weight, Tensor post_ln_bias,  \
                                          Tensor mlp_up_bias, Tensor mlp_down_bias, py::object current_seq_len) {      \
        return graph_decode_step(k##MODEL, context_id, input, layernorm_weight, layernorm_bias, qkv_bias, o_bias, cos, \
                                 sin, k_cache, v_cache, post_ln_weight, post_ln_bias, mlp_up_bias, mlp_down_bias,      \
                                 current_seq_len);                                                                     \
    });                                                                                                                \
    m.def(#MODEL "_destroy_graph_context", [](int64_t context_id) { destroy_graph_context(k##MODEL, context_id); });

namespace {
const Model& kpythia_2b8 = kPythia2b8;
const Model& kpythia_6b9 = kPythia6b9;
}  // namespace

// llama_decoder_layer_sglang of the reference (include/pybind.cpp:77-88): returns (output, residual, k, v);
// `residual` is updated in place (residual += input) as the reference does.
std::tuple<Tensor, Tensor, Tensor> llama_attention_impl(const char* op, Tensor input, c10::optional<Tensor> residual_opt,
                                                        Tensor weight_qkv, Tensor weight_o, Tensor k_cache, Tensor v_cache,
                                                        Tensor rms_input_weight, double eps, Tensor cos, Tensor sin,
                                                        int64_t num_heads, bool add_residual, bool split) {
    TORCH_CHECK(input.defined() && input.dim() >= 1, "input is undefined");
    const int64_t H = input.numel();
    TORCH_CHECK(num_heads > 0 && H % num_heads == 0, "hidden size ", H, " is not a multiple of num_heads ", num_heads);
    const int64_t D = H / num_heads;
    check_half(input, "input", H, input);
    if (residual_opt.has_value()) check_half(*residual_opt, "residual", H, input);
    check_half(weight_qkv, "weight_qkv", 3 * H * H, input);
    check_half(weight_o, "weight_o", H * H, input);
    check_half(rms_input_weight, "rms_input_weight", H, input);
    const int64_t rows_k = check_cache(k_cache, "k_cache", H, input);
    const int64_t rows_v = check_cache(v_cache, "v_cache", H, input);
    TORCH_CHECK(rows_k == rows_v, "k_cache has ", rows_k, " rows but v_cache has ", rows_v);
    check_rope(cos, "cos", D / 2, input);
    check_rope(sin, "sin", D / 2, input);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto opts = input.options();
    Tensor out = torch::empty({1, H}, opts);
    Tensor k = torch::empty({1, num_heads, D}, opts);
    Tensor v = torch::empty({1, num_heads, D}, opts);
    cfpp_llama_attn a{};
    a.hidden = (int32_t)H; a.heads = (int32_t)num_heads; a.head_dim = (int32_t)D; a.eps = (float)eps;
    a.rms_w = rms_input_weight.data_ptr(); a.w_qkv = weight_qkv.data_ptr(); a.w_o = weight_o.data_ptr();
    a.input = input.data_ptr(); a.residual = residual_opt.has_value() ? residual_opt->data_ptr() : nullptr; a.output = out.data_ptr();
    a.add_residual = add_residual ? 1 : 0;
    a.mode = split ? CFPP_MODE_SPLIT : CFPP_MODE_FUSED;
    a.k_new = k.data_ptr(); a.v_new = v.data_ptr();
    // an empty cache has no storage: any valid pointer will do, no row of it is read
    a.k_cache = rows_k > 0 ? k_cache.data_ptr() : input.data_ptr();
    a.v_cache = rows_k > 0 ? v_cache.data_ptr() : input.data_ptr();
    a.seq_len = (int32_t)rows_k;
    a.cos = cos.data_ptr<float>(); a.sin = sin.data_ptr<float>();
    const size_t bytes = cfpp_llama_workspace_bytes(a.hidden, a.heads, a.head_dim);
    TORCH_CHECK(bytes > 0, "unsupported layer dimensions (hidden ", H, ", heads ", num_heads, ")");
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const cfpp_neox_dims d{a.hidden, a.heads, a.head_dim, a.head_dim, 4 * a.hidden, a.eps};
    Tensor ws = workspace_for(d, input.device(), st);
    check_rc(cfpp_llama_attention_decode(&a, ws_ptr(ws), ws_capacity(ws), st), op);
    return std::make_tuple(out, k, v);
}

std::tuple<Tensor, Tensor, Tensor, Tensor> llama_decoder_layer_sglang(Tensor input, Tensor residual, Tensor weight_qkv,
                                                                      Tensor weight_o, Tensor k_cache, Tensor v_cache,
                                                                      Tensor rms_input_weight, double eps, Tensor cos, Tensor sin,
                                                                      int64_t num_heads, bool split) {
    auto r = llama_attention_impl("llama_decoder_layer_sglang", input, residual, weight_qkv, weight_o, k_cache, v_cache,
                                  rms_input_weight, eps, cos, sin, num_heads, false, split);
    return std::make_tuple(std::get<0>(r), residual, std::get<1>(r), std::get<2>(r));
}

// llama_decoder_layer of the reference (include/pybind.cpp:66-75,280): (input, weight_qkv, weight_o, k_cache, v_cache,
// rms_input_weight, cos, sin) -> (output, k, v).  Weights are stored [in, out] (weight_qkv = three such matrices
// stacked), the rotary dims pair up GPT-J style, cos / sin hold head_dim entries, eps is 1e-6
// (include/5090/llama/kernel.cuh:58), the caches are read only.
std::tuple<Tensor, Tensor, Tensor> llama_decoder_layer(Tensor input, Tensor weight_qkv, Tensor weight_o, Tensor k_cache,
                                                       Tensor v_cache, Tensor rms_input_weight, Tensor cos, Tensor sin,
                                                       int64_t num_heads) {
    const char* op = "llama_decoder_layer";
    TORCH_CHECK(input.defined() && input.dim() >= 1, "input is undefined");
    const int64_t H = input.numel();
    TORCH_CHECK(num_heads > 0 && H % num_heads == 0, "hidden size ", H, " is not a multiple of num_heads ", num_heads);
    const int64_t D = H / num_heads;
    check_half(input, "input", H, input);
    check_half(weight_qkv, "weight_qkv", 3 * H * H, input);
    check_half(weight_o, "weight_o", H * H, input);
    check_half(rms_input_weight, "rms_input_weight", H, input);
    const int64_t rows_k = check_cache(k_cache, "k_cache", H, input);
    const int64_t rows_v = check_cache(v_cache, "v_cache", H, input);
    TORCH_CHECK(rows_k == rows_v, "k_cache has ", rows_k, " rows but v_cache has ", rows_v);
    check_rope(cos, "cos", D, input);
    check_rope(sin, "sin", D, input);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto opts = input.options();
    Tensor out = torch::empty({1, H}, opts);
    Tensor k = torch::empty({1, num_heads, D}, opts);
    Tensor v = torch::empty({1, num_heads, D}, opts);
    cfpp_llama_attn a{};
    a.hidden = (int32_t)H; a.heads = (int32_t)num_heads; a.head_dim = (int32_t)D; a.eps = 1e-6f;
    a.rms_w = rms_input_weight.data_ptr(); a.w_qkv = weight_qkv.data_ptr(); a.w_o = weight_o.data_ptr();
    a.input = input.data_ptr(); a.residual = nullptr; a.output = out.data_ptr(); a.add_residual = 0;
    a.mode = CFPP_MODE_FUSED;
    a.k_new = k.data_ptr(); a.v_new = v.data_ptr();
    a.k_cache = rows_k > 0 ? k_cache.data_ptr() : input.data_ptr();
    a.v_cache = rows_k > 0 ? v_cache.data_ptr() : input.data_ptr();
    a.seq_len = (int32_t)rows_k;
    a.cos = cos.data_ptr<float>(); a.sin = sin.data_ptr<float>();
    const size_t bytes = cfpp_llama_plain_workspace_bytes(a.hidden, a.heads, a.head_dim);
    TORCH_CHECK(bytes > 0, "unsupported layer dimensions (hidden ", H, ", heads ", num_heads, ")");
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    Tensor ws = scratch_for(ScratchKey{(int)input.device().index(), (void*)st, 1, (int)H, (int)num_heads, (int)D, 0}, (int64_t)bytes,
                            input.device());
    check_rc(cfpp_llama_attention_plain(&a, ws_ptr(ws), ws_capacity(ws), st), op);
    return std::make_tuple(out, k, v);
}

// llama_decoder_layer_batch_decode_sglang of the reference (include/pybind.cpp:90-106,282;
// include/5090/llama/llama_kernel_batch_sglang_dispatch.cu:6-110): same positional arguments, results written into the
// caller's `output` and `residual_output`, the new K/V rows into the paged caches; returns None.  The reference reads
// head count and head size from compile-time constants; here they follow from `cos_sin` (its last dimension is the
// head size).
void llama_decoder_layer_batch_decode_sglang(Tensor output, Tensor residual_output, Tensor input, Tensor residual,
                                             Tensor weight_qkv, Tensor weight_o, Tensor paged_kv_indptr, Tensor paged_kv_indices,
                                             Tensor k_cache_ptrs, Tensor v_cache_ptrs, int64_t layer_id, Tensor rms_input_weight,
                                             double eps, Tensor positions, Tensor cos_sin) {
    const char* op = "llama_decoder_layer_batch_decode_sglang";
    TORCH_CHECK(input.defined() && input.dim() == 2, "input must have shape [batch, hidden]");
    const int64_t B = input.size(0), H = input.size(1);
    TORCH_CHECK(B >= 1, "empty batch");
    check_half(input, "input", B * H, input);
    check_half(residual, "residual", B * H, input);
    check_half(output, "output", B * H, input);
    check_half(residual_output, "residual_output", B * H, input);
    check_half(weight_qkv, "weight_qkv", 3 * H * H, input);
    check_half(weight_o, "weight_o", H * H, input);
    check_half(rms_input_weight, "rms_input_weight", H, input);
    TORCH_CHECK(cos_sin.defined() && cos_sin.is_cuda() && cos_sin.device() == input.device() && cos_sin.scalar_type() == torch::kFloat32 &&
                    cos_sin.is_contiguous() && cos_sin.dim() == 2,
                "cos_sin must be a contiguous float32 tensor [positions, head_dim] on the device of input");
    const int64_t D = cos_sin.size(1);
    TORCH_CHECK(D > 0 && H % D == 0, "hidden size ", H, " is not a multiple of the head size ", D, " (cos_sin.size(1))");
    auto check_index = [&](const Tensor& t, const char* name, torch::ScalarType ty, int64_t min_numel) {
        TORCH_CHECK(t.defined() && t.is_cuda() && t.device() == input.device() && t.is_contiguous() && t.scalar_type() == ty &&
                        t.numel() >= min_numel,
                    name, " must be a contiguous ", c10::toString(ty), " tensor with at least ", min_numel,
                    " elements on the device of input");
    };
    check_index(paged_kv_indptr, "paged_kv_indptr", torch::kInt32, B + 1);
    check_index(paged_kv_indices, "paged_kv_indices", torch::kInt32, B);
    TORCH_CHECK(layer_id >= 0, "layer_id is negative");
    check_index(k_cache_ptrs, "k_cache_ptrs", k_cache_ptrs.defined() ? k_cache_ptrs.scalar_type() : torch::kUInt64, layer_id + 1);
    check_index(v_cache_ptrs, "v_cache_ptrs", v_cache_ptrs.defined() ? v_cache_ptrs.scalar_type() : torch::kUInt64, layer_id + 1);
    TORCH_CHECK(k_cache_ptrs.element_size() == 8 && v_cache_ptrs.element_size() == 8, "cache pointer tables must hold 64-bit values");
    check_index(positions, "positions", torch::kInt64, B);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    cfpp_llama_batch a{};
    a.hidden = (int32_t)H; a.heads = (int32_t)(H / D); a.head_dim = (int32_t)D; a.eps = (float)eps;
    a.batch = (int32_t)B; a.layer_id = (int32_t)layer_id;
    a.rms_w = rms_input_weight.data_ptr(); a.w_qkv = weight_qkv.data_ptr(); a.w_o = weight_o.data_ptr();
    a.input = input.data_ptr(); a.residual = residual.data_ptr();
    a.residual_out = residual_output.data_ptr(); a.output = output.data_ptr();
    a.paged_kv_indptr = paged_kv_indptr.data_ptr<int32_t>(); a.paged_kv_indices = paged_kv_indices.data_ptr<int32_t>();
    a.k_cache_ptrs = reinterpret_cast<const uint64_t*>(k_cache_ptrs.data_ptr());
    a.v_cache_ptrs = reinterpret_cast<const uint64_t*>(v_cache_ptrs.data_ptr());
    a.positions = positions.data_ptr<int64_t>(); a.cos_sin = cos_sin.data_ptr<float>();
    const size_t bytes = cfpp_llama_batch_workspace_bytes(a.hidden, a.heads, a.head_dim, a.batch);
    TORCH_CHECK(bytes > 0, "unsupported layer dimensions (hidden ", H, ", head size ", D, ")");
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    Tensor ws = scratch_for(ScratchKey{(int)input.device().index(), (void*)st, 2, (int)H, (int)(H / D), (int)D, (int)B}, (int64_t)bytes,
                            input.device());
    check_rc(cfpp_llama_batch_decode(&a, ws_ptr(ws), ws_capacity(ws), st), op);
}

// output = input + W_down (silu(Wg n) * (Wu n)), n = RMSNorm(input) * rms_weight; gate_up_weight = [Wg; Wu] ([2F, H])
Tensor llama_mlp(Tensor input, Tensor rms_weight, Tensor gate_up_weight, Tensor down_weight, double eps, bool split) {
    TORCH_CHECK(input.defined() && input.dim() >= 1, "input is undefined");
    const int64_t H = input.numel();
    check_half(input, "input", H, input);
    check_half(rms_weight, "rms_weight", H, input);
    TORCH_CHECK(gate_up_weight.defined() && gate_up_weight.numel() % (2 * H) == 0 && gate_up_weight.numel() > 0,
                "gate_up_weight must have 2*F*", H, " elements");
    const int64_t F = gate_up_weight.numel() / (2 * H);
    check_half(gate_up_weight, "gate_up_weight", 2 * F * H, input);
    check_half(down_weight, "down_weight", H * F, input);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    Tensor out = torch::empty({1, H}, input.options());
    cfpp_llama_mlp_args m{};
    m.hidden = (int32_t)H; m.ffn = (int32_t)F; m.eps = (float)eps;
    m.rms_w = rms_weight.data_ptr(); m.w_gate_up = gate_up_weight.data_ptr(); m.w_down = down_weight.data_ptr();
    m.input = input.data_ptr(); m.output = out.data_ptr();
    m.mode = split ? CFPP_MODE_SPLIT : CFPP_MODE_FUSED;
    const size_t bytes = cfpp_llama_mlp_workspace_bytes(m.hidden, m.ffn);
    TORCH_CHECK(bytes > 0, "unsupported MLP dimensions (hidden ", H, ", ffn ", F, ")");
    hipStream_t st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    Tensor ws = scratch_for(ScratchKey{(int)input.device().index(), (void*)st, 3, (int)H, (int)F, 0, 0}, (int64_t)bytes, input.device());
    check_rc(cfpp_llama_mlp(&m, ws_ptr(ws), ws_capacity(ws), st), "llama_mlp");
    return out;
}

// A whole LLaMA layer, batch-1 decode: h = input + attention(RMSNorm(input)); out = h + MLP(RMSNorm(h)).
// Returns (out, k_new, v_new); the caches are not written.
std::tuple<Tensor, Tensor, Tensor> llama_decoder_layer_full(Tensor input, Tensor weight_qkv, Tensor weight_o, Tensor k_cache,
                                                            Tensor v_cache, Tensor rms_input_weight, Tensor rms_post_weight,
                                                            Tensor gate_up_weight, Tensor down_weight, double eps, Tensor cos,
                                                            Tensor sin, int64_t num_heads, bool split) {
    auto r = llama_attention_impl("llama_decoder_layer_full", input, c10::nullopt, weight_qkv, weight_o, k_cache, v_cache,
                                  rms_input_weight, eps, cos, sin, num_heads, true, split);
    Tensor out = llama_mlp(std::get<0>(r), rms_post_weight, gate_up_weight, down_weight, eps, split);
    return std::make_tuple(out, std::get<1>(r), std::get<2>(r));
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "MI355X (gfx950) fused GPT-NeoX / Pythia decode step";
    DEFINE_MODEL_OPS(m, pythia_2b8)
    DEFINE_MODEL_OPS(m, pythia_6b9)

    // any supported GPT-NeoX geometry (other Pythia sizes): same tensor arguments as the per-model ops
    m.def("neox_decoder_layer", [](int64_t hidden, int64_t heads, int64_t head_dim, int64_t rotary_dim, int64_t ffn, double eps,
                                   bool split, LAYER_ARGS, Tensor mlp_down_weight, Tensor mlp_down_bias, int64_t current_seq_len) {
        const Model m{"neox_decoder_layer", 2,
                      {(int32_t)hidden, (int32_t)heads, (int32_t)head_dim, (int32_t)rotary_dim, (int32_t)ffn, (float)eps}};
        TORCH_CHECK(cfpp_neox_workspace_bytes(&m.dims) > 0, "unsupported layer dimensions");
        return decoder_layer(m, split ? CFPP_MODE_SPLIT : CFPP_MODE_FUSED, LAYER_PACK(mlp_down_weight, mlp_down_bias), current_seq_len);
    });
    m.def("llama_decoder_layer_sglang", &llama_decoder_layer_sglang, py::arg("input"), py::arg("residual"), py::arg("weight_qkv"),
          py::arg("weight_o"), py::arg("k_cache"), py::arg("v_cache"), py::arg("rms_input_weight"), py::arg("eps"), py::arg("cos"),
          py::arg("sin"), py::arg("num_heads") = 32, py::arg("split") = false);
    m.def("llama_decoder_layer", &llama_decoder_layer, py::arg("input"), py::arg("weight_qkv"), py::arg("weight_o"), py::arg("k_cache"),
          py::arg("v_cache"), py::arg("rms_input_weight"), py::arg("cos"), py::arg("sin"), py::arg("num_heads") = 32);
    m.def("llama_decoder_layer_batch_decode_sglang", &llama_decoder_layer_batch_decode_sglang, py::arg("output"),
          py::arg("residual_output"), py::arg("input"), py::arg("residual"), py::arg("weight_qkv"), py::arg("weight_o"),
          py::arg("paged_kv_indptr"), py::arg("paged_kv_indices"), py::arg("k_cache_ptrs"), py::arg("v_cache_ptrs"),
          py::arg("layer_id"), py::arg("rms_input_weight"), py::arg("eps"), py::arg("positions"), py::arg("cos_sin"));
    m.def("llama_mlp", &llama_mlp, py::arg("input"), py::arg("rms_weight"), py::arg("gate_up_weight"), py::arg("down_weight"),
          py::arg("eps"), py::arg("split") = false);
    m.def("llama_decoder_layer_full", &llama_decoder_layer_full, py::arg("input"), py::arg("weight_qkv"), py::arg("weight_o"),
          py::arg("k_cache"), py::arg("v_cache"), py::arg("rms_input_weight"), py::arg("rms_post_weight"),
          py::arg("gate_up_weight"), py::arg("down_weight"), py::arg("eps"), py::arg("cos"), py::arg("sin"),
          py::arg("num_heads") = 32, py::arg("split") = false);
    m.def("cfpp_version", []() { return std::string(cfpp_version()); });
    m.def("debug_set_trace", [](c10::optional<Tensor> buf) {
        // profiling builds of the HIP library only (built with -DCFPP_TRACE): int64 device tensor of at least
        // 1024*16*16 elements, or None to switch tracing off
        typedef int (*set_trace_fn)(void*);
        set_trace_fn fn = reinterpret_cast<set_trace_fn>(dlsym(RTLD_DEFAULT, "cfpp_debug_set_trace"));
        TORCH_CHECK(fn != nullptr, "the loaded HIP library has no phase tracing: clusterfusionplus_amd/phase_trace.py loads a profiling build before the package");
        if (buf.has_value()) {
            TORCH_CHECK(buf->is_cuda() && buf->scalar_type() == torch::kInt64 && buf->is_contiguous() && buf->numel() >= 1024 * 16 * 16,
                        "trace buffer must be a contiguous int64 GPU tensor with >= 262144 elements");
            fn(buf->data_ptr());
        } else {
            fn(nullptr);
        }
    });
    m.def("device_status", [](bool clear) { return cfpp_device_status(clear ? 1 : 0); }, py::arg("clear") = false);
    m.def("one_launch_fits", [](int64_t grid, int64_t cus, int64_t per_cu) {
        return cfpp_one_launch_fits((int)grid, (int)cus, (int)per_cu) != 0;
    });
    m.def("workspace_bytes", [](int64_t hidden, int64_t heads, int64_t head_dim, int64_t rotary_dim, int64_t ffn) {
        cfpp_neox_dims d{(int32_t)hidden, (int32_t)heads, (int32_t)head_dim, (int32_t)rotary_dim, (int32_t)ffn, 1e-5f};
        return (int64_t)cfpp_neox_workspace_bytes(&d);
    });
    m.def("check_workspace", [](Tensor like, int64_t hidden, int64_t heads, int64_t head_dim, int64_t rotary_dim, int64_t ffn) {
        // reads (and clears) the device-side failure flag of the calling stream's scratch buffer
        cfpp_neox_dims d{(int32_t)hidden, (int32_t)heads, (int32_t)head_dim, (int32_t)rotary_dim, (int32_t)ffn, 1e-5f};
        c10::hip::HIPGuardMasqueradingAsCUDA guard(like.device());
        hipStream_t st = cur_stream();
        Tensor ws = workspace_for(d, like.device(), st);
        return cfpp_workspace_check(&d, ws_ptr(ws), st);
    });
    m.def("lm_head", [](Tensor x, Tensor ln_w, Tensor ln_b, Tensor w, double eps) {
        TORCH_CHECK(w.dim() == 2, "lm head weight must be [vocab, H]");
        const int64_t V = w.size(0), H = w.size(1);
        check_half(x, "x", H, x);
        check_half(ln_w, "ln_weight", H, x);
        check_half(ln_b, "ln_bias", H, x);
        check_half(w, "weight", V * H, x);
        c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
        Tensor logits = torch::empty({V}, x.options().dtype(torch::kFloat32));
        check_rc(cfpp_neox_lm_head((int32_t)H, (int32_t)V, (float)eps, x.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(),
                                   w.data_ptr(), logits.data_ptr<float>(), cur_stream()), "lm_head");
        return logits;
    });

    py::class_<PyStack, std::shared_ptr<PyStack>>(m, "NeoxStack")
        .def(py::init(&stack_create), py::arg("hidden"), py::arg("heads"), py::arg("head_dim"), py::arg("rotary_dim"),
             py::arg("ffn"), py::arg("eps"), py::arg("layers"), py::arg("embed"), py::arg("final_ln_weight"),
             py::arg("final_ln_bias"), py::arg("lm_head"), py::arg("k_caches"), py::arg("v_caches"), py::arg("rope_cos"),
             py::arg("rope_sin"), py::arg("mode") = 0)
        .def("set_state", [](PyStack& s, int64_t token, int64_t seq_len) {
            c10::hip::HIPGuardMasqueradingAsCUDA guard(s.device);
            check_rc(cfpp_stack_set_state(s.s, (int32_t)token, (int32_t)seq_len, cur_stream()), "set_state");
        })
        .def("step", [](PyStack& s) {
            c10::hip::HIPGuardMasqueradingAsCUDA guard(s.device);
            check_rc(cfpp_stack_step(s.s, cur_stream()), "step");
        })
        .def("graph_steps", [](PyStack& s, int64_t n) {
            c10::hip::HIPGuardMasqueradingAsCUDA guard(s.device);
            check_rc(cfpp_stack_graph_steps(s.s, (int32_t)n, cur_stream()), "graph_steps");
        })
        .def("layers_per_launch", [](PyStack& s) { return (int64_t)cfpp_stack_layers_per_launch(s.s); })
        .def("profile_step", [](PyStack& s) {
            // (per-layer ms list, lm head ms, whole-step ms) of one eager step timed with HIP events
            c10::hip::HIPGuardMasqueradingAsCUDA guard(s.device);
            std::vector<float> layer_ms(s.n_layers, 0.f);
            float lm = 0.f, total = 0.f;
            check_rc(cfpp_stack_profile_step(s.s, cur_stream(), layer_ms.data(), &lm, &total), "profile_step");
            return std::make_tuple(layer_ms, lm, total);
        })
        .def("logits", [](PyStack& s) {
            float* p = nullptr;
            check_rc(cfpp_stack_buffers(s.s, &p, nullptr, nullptr, nullptr, nullptr), "buffers");
            return torch::from_blob(p, {s.vocab}, torch::TensorOptions().dtype(torch::kFloat32).device(s.device));
        })
        .def("hidden", [](PyStack& s) {
            void* p = nullptr;
            check_rc(cfpp_stack_buffers(s.s, nullptr, &p, nullptr, nullptr, nullptr), "buffers");
            return torch::from_blob(p, {1, (int64_t)s.dims.hidden}, torch::TensorOptions().dtype(torch::kFloat16).device(s.device));
        })
        .def("check", [](PyStack& s) {
            // synchronises; raises if a step of this stack raised a device-side failure flag
            c10::hip::HIPGuardMasqueradingAsCUDA guard(s.device);
            check_rc(cfpp_stack_check(s.s, cur_stream()), "NeoxStack.check");
        })
        .def("state", [](PyStack& s) {
            int32_t* p = nullptr;
            check_rc(cfpp_stack_buffers(s.s, nullptr, nullptr, &p, nullptr, nullptr), "buffers");
            return torch::from_blob(p, {3}, torch::TensorOptions().dtype(torch::kInt32).device(s.device));
        })
        .def("history", [](PyStack& s) {
            int32_t* p = nullptr;
            int32_t cap = 0;
            check_rc(cfpp_stack_buffers(s.s, nullptr, nullptr, nullptr, &p, &cap), "buffers");
            return torch::from_blob(p, {(int64_t)cap}, torch::TensorOptions().dtype(torch::kInt32).device(s.device));
        });
}
