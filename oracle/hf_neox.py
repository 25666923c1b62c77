"""HuggingFace GPT-NeoX layer built locally from a config (no download) - the CPU reference the
reference project's end-to-end scripts compare against (reference tests/benchmark_decode.py:83-108
reads the same module names).

TEST INFRASTRUCTURE ONLY: used to pin `neox_oracle` and as the timed CPU baseline; never imported
by the product package.  `transformers` is a third-party library, not part of the reference.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .neox_oracle import NeoxDims


def _config(dims: NeoxDims, n_layers: int = 1, vocab: int = 128, act: str = "gelu_pytorch_tanh"):
    from transformers import GPTNeoXConfig
    cfg = GPTNeoXConfig(
        vocab_size=vocab, hidden_size=dims.hidden, num_attention_heads=dims.heads,
        intermediate_size=dims.ffn, num_hidden_layers=n_layers, hidden_act=act,
        layer_norm_eps=dims.eps, use_parallel_residual=True, attention_bias=True,
        max_position_embeddings=1 << 16, tie_word_embeddings=False,
        rope_parameters={"rope_type": "default", "rope_theta": 10000.0,
                         "partial_rotary_factor": dims.rotary_dim / dims.head_dim},
    )
    cfg._attn_implementation = "eager"
    return cfg


def _load_layer(layer, w: Dict[str, torch.Tensor], dtype):
    names = {
        "input_layernorm.weight": "ln_w", "input_layernorm.bias": "ln_b",
        "post_attention_layernorm.weight": "post_ln_w", "post_attention_layernorm.bias": "post_ln_b",
        "attention.query_key_value.weight": "w_qkv", "attention.query_key_value.bias": "b_qkv",
        "attention.dense.weight": "w_o", "attention.dense.bias": "b_o",
        "mlp.dense_h_to_4h.weight": "w_up", "mlp.dense_h_to_4h.bias": "b_up",
        "mlp.dense_4h_to_h.weight": "w_down", "mlp.dense_4h_to_h.bias": "b_down",
    }
    sd = {k: w[v].detach().cpu().to(dtype).reshape(layer.state_dict()[k].shape) for k, v in names.items()}
    layer.load_state_dict(sd, strict=True)


def build_hf_layer(dims: NeoxDims, w: Dict[str, torch.Tensor], dtype=torch.float32, act="gelu_pytorch_tanh"):
    from transformers.models.gpt_neox.modeling_gpt_neox import GPTNeoXLayer
    layer = GPTNeoXLayer(_config(dims, act=act), layer_idx=0).to(dtype).eval()
    _load_layer(layer, w, dtype)
    return layer


@torch.no_grad()
def hf_layer_decode(layer, x, k_cache, v_cache, cos, sin, seq_len: int, dims: NeoxDims, dtype=torch.float32):
    """Run one decode step through the HF layer with a pre-filled DynamicCache.
    Returns (output [1,H], k_new [1,heads,D], v_new [1,heads,D])."""
    from transformers import DynamicCache
    nh, D, H = dims.heads, dims.head_dim, dims.hidden
    K = k_cache[:seq_len].detach().cpu().to(dtype).reshape(seq_len, nh, D).permute(1, 0, 2)[None].contiguous()
    V = v_cache[:seq_len].detach().cpu().to(dtype).reshape(seq_len, nh, D).permute(1, 0, 2)[None].contiguous()
    cache = DynamicCache(ddp_cache_data=[(K, V)])
    c = cos.detach().cpu().to(dtype).reshape(-1)[: dims.rotary_dim][None, None]
    s = sin.detach().cpu().to(dtype).reshape(-1)[: dims.rotary_dim][None, None]
    out = layer(x.detach().cpu().to(dtype).reshape(1, 1, H), attention_mask=None, layer_past=cache,
                position_embeddings=(c, s))
    if isinstance(out, tuple):
        out = out[0]
    k_new = cache.layers[0].keys[0, :, -1, :][None]
    v_new = cache.layers[0].values[0, :, -1, :][None]
    return out.reshape(1, H), k_new, v_new


def build_hf_model(dims: NeoxDims, layers: List[Dict[str, torch.Tensor]], embed, final_ln_w, final_ln_b,
                   lm_head, dtype=torch.float32):
    from transformers import GPTNeoXForCausalLM
    cfg = _config(dims, n_layers=len(layers), vocab=embed.shape[0])
    model = GPTNeoXForCausalLM(cfg).to(dtype).eval()
    for i, w in enumerate(layers):
        _load_layer(model.gpt_neox.layers[i], w, dtype)
    with torch.no_grad():
        model.gpt_neox.embed_in.weight.copy_(embed.to(dtype))
        model.gpt_neox.final_layer_norm.weight.copy_(final_ln_w.to(dtype).reshape(-1))
        model.gpt_neox.final_layer_norm.bias.copy_(final_ln_b.to(dtype).reshape(-1))
        model.get_output_embeddings().weight.copy_(lm_head.to(dtype))
    return model


# ---- LLaMA (pins llama_layer_decode and llama_attention_sglang) ------------------------------------

def build_hf_llama_layer(dims, w: Dict[str, torch.Tensor], dtype=torch.float32):
    """HF LlamaDecoderLayer from a local config; `w` as in neox_oracle.llama_layer_decode (missing MLP / rms2
    entries are left at their random initialisation: the attention-only checks do not use them)."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    H = dims.hidden
    cfg = LlamaConfig(hidden_size=H, intermediate_size=max(dims.ffn, 8), num_hidden_layers=1, num_attention_heads=dims.heads,
                      num_key_value_heads=dims.heads, head_dim=dims.head_dim, rms_norm_eps=dims.eps, vocab_size=32,
                      attention_bias=False, mlp_bias=False, hidden_act="silu", max_position_embeddings=64)
    cfg._attn_implementation = "eager"
    layer = LlamaDecoderLayer(cfg, layer_idx=0).to(dtype).eval()
    f = lambda t: t.detach().cpu().to(dtype)
    with torch.no_grad():
        layer.input_layernorm.weight.copy_(f(w["rms1"]).reshape(H))
        wq, wk, wv = f(w["w_qkv"]).reshape(3, H, H)
        layer.self_attn.q_proj.weight.copy_(wq); layer.self_attn.k_proj.weight.copy_(wk); layer.self_attn.v_proj.weight.copy_(wv)
        layer.self_attn.o_proj.weight.copy_(f(w["w_o"]))
        if "rms2" in w:
            layer.post_attention_layernorm.weight.copy_(f(w["rms2"]).reshape(H))
            wg, wu = f(w["w_gate_up"]).reshape(2, dims.ffn, H)
            layer.mlp.gate_proj.weight.copy_(wg); layer.mlp.up_proj.weight.copy_(wu)
            layer.mlp.down_proj.weight.copy_(f(w["w_down"]))
    return layer


def _llama_cache(k_cache, v_cache, seq_len, dims, dtype):
    from transformers import DynamicCache
    nh, D = dims.heads, dims.head_dim
    K = k_cache[:seq_len].detach().cpu().to(dtype).reshape(seq_len, nh, D).permute(1, 0, 2)[None].contiguous()
    V = v_cache[:seq_len].detach().cpu().to(dtype).reshape(seq_len, nh, D).permute(1, 0, 2)[None].contiguous()
    return DynamicCache(ddp_cache_data=[(K, V)])


@torch.no_grad()
def hf_llama_layer_decode(layer, x, k_cache, v_cache, cos, sin, seq_len: int, dims, dtype=torch.float32):
    """One decode step through the whole HF LlamaDecoderLayer; returns (output [1,H], k_new, v_new)."""
    H, D = dims.hidden, dims.head_dim
    cache = _llama_cache(k_cache, v_cache, seq_len, dims, dtype)
    c = cos.detach().cpu().to(dtype).reshape(-1)[:D][None, None]
    s = sin.detach().cpu().to(dtype).reshape(-1)[:D][None, None]
    out = layer(x.detach().cpu().to(dtype).reshape(1, 1, H), attention_mask=None, past_key_values=cache,
                position_embeddings=(c, s))
    if isinstance(out, tuple):
        out = out[0]
    return out.reshape(1, H), cache.layers[0].keys[0, :, -1, :][None], cache.layers[0].values[0, :, -1, :][None]


@torch.no_grad()
def hf_llama_attention(layer, r, k_cache, v_cache, cos, sin, dims, dtype=torch.float32):
    """input_layernorm + self_attn of the HF layer on the (already summed) row r; returns (attn_out [1,H], k_new, v_new)."""
    H, D = dims.hidden, dims.head_dim
    S = k_cache.shape[0]
    cache = _llama_cache(k_cache, v_cache, S, dims, dtype)
    c = cos.detach().cpu().to(dtype).reshape(-1)[:D][None, None]
    s = sin.detach().cpu().to(dtype).reshape(-1)[:D][None, None]
    n = layer.input_layernorm(r.detach().cpu().to(dtype).reshape(1, 1, H))
    out = layer.self_attn(n, position_embeddings=(c, s), attention_mask=None, past_key_values=cache)
    if isinstance(out, tuple):
        out = out[0]
    return out.reshape(1, H), cache.layers[0].keys[0, :, -1, :][None], cache.layers[0].values[0, :, -1, :][None]
