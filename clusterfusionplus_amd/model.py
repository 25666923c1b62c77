"""Host-side model runner: the counterpart of the reference's full-model decode loop
(reference tests/benchmark_decode.py:60-119 `prepare_setup`, :147-189 the per-token loop), with the
loop body moved into one hipGraph replay per token (embedding row -> layers -> final LayerNorm ->
LM head -> argmax all on the device)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence

import torch


@dataclass(frozen=True)
class NeoxConfig:
    hidden: int
    heads: int
    head_dim: int
    rotary_dim: int
    ffn: int
    n_layers: int
    vocab: int
    eps: float = 1e-5
    rope_base: float = 10000.0


PYTHIA_2B8 = NeoxConfig(hidden=2560, heads=32, head_dim=80, rotary_dim=20, ffn=10240, n_layers=32, vocab=50304)
PYTHIA_6B9 = NeoxConfig(hidden=4096, heads=32, head_dim=128, rotary_dim=32, ffn=16384, n_layers=32, vocab=50432)

# order of the 12 per-layer tensors (same set the reference pulls out of the HF module,
# tests/benchmark_decode.py:83-96)
layer_tensor_order = ("ln_w", "ln_b", "w_qkv", "b_qkv", "w_o", "b_o",
                      "post_ln_w", "post_ln_b", "w_up", "b_up", "w_down", "b_down")


def rope_tables(positions: int, rotary_dim: int, base: float = 10000.0, device="cuda"):
    """fp32 cos/sin tables `[positions, rotary_dim]`, emb = cat(freqs, freqs)
    (reference tests/benchmark_decode.py:39-57)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim))
    freqs = torch.arange(positions, dtype=torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().float().to(device).contiguous(), emb.sin().float().to(device).contiguous()


# ---- prefill -> decode hand-off: HuggingFace GPT-NeoX modules and caches to this library's layout -------------

def layer_tensors_from_hf(hf_layer, dtype=torch.float16, device=None) -> Dict[str, torch.Tensor]:
    """The 12 per-layer tensors of a HuggingFace `GPTNeoXLayer`, keyed by `layer_tensor_order`
    (the set reference tests/benchmark_decode.py:83-96 pulls out of the module).  HF keeps `query_key_value`
    head-interleaved `[head][q|k|v][D]`, which is the layout the kernels read, so nothing is re-ordered."""
    a, m = hf_layer.attention, hf_layer.mlp
    src = {
        "ln_w": hf_layer.input_layernorm.weight, "ln_b": hf_layer.input_layernorm.bias,
        "w_qkv": a.query_key_value.weight, "b_qkv": a.query_key_value.bias,
        "w_o": a.dense.weight, "b_o": a.dense.bias,
        "post_ln_w": hf_layer.post_attention_layernorm.weight, "post_ln_b": hf_layer.post_attention_layernorm.bias,
        "w_up": m.dense_h_to_4h.weight, "b_up": m.dense_h_to_4h.bias,
        "w_down": m.dense_4h_to_h.weight, "b_down": m.dense_4h_to_h.bias,
    }
    out = {}
    for k in layer_tensor_order:
        t = src[k].detach().to(dtype)
        out[k] = (t.to(device) if device is not None else t).contiguous()
    return out


def kv_cache_from_hf(key: torch.Tensor, value: torch.Tensor, rows: int, dtype=torch.float16, device=None):
    """HF `past_key_values` of one layer, `[1, heads, S, D]` each, to the `[rows, heads*D]` caches the decode step
    reads and appends to (`permute(0,2,1,3).reshape(S, H)`, reference tests/benchmark_decode.py:99-108).
    Returns (k_cache, v_cache, S); rows >= S + the tokens to be generated."""
    if key.dim() != 4 or key.shape[0] != 1 or key.shape != value.shape:
        raise ValueError(f"expected key/value of shape [1, heads, S, D], got {tuple(key.shape)} / {tuple(value.shape)}")
    _, nh, S, D = key.shape
    if rows < S:
        raise ValueError(f"rows ({rows}) < cached positions ({S})")
    dev = device if device is not None else key.device
    kc = torch.zeros((rows, nh * D), dtype=dtype, device=dev)
    vc = torch.zeros((rows, nh * D), dtype=dtype, device=dev)
    kc[:S] = key.detach().permute(0, 2, 1, 3).reshape(S, nh * D).to(device=dev, dtype=dtype)
    vc[:S] = value.detach().permute(0, 2, 1, 3).reshape(S, nh * D).to(device=dev, dtype=dtype)
    return kc, vc, S


def config_from_hf(hf_config) -> NeoxConfig:
    """The geometry of a HuggingFace `GPTNeoXConfig` (the fields reference tests/benchmark_decode.py:60-81 reads from the
    loaded model).  The rotary fraction and base are under `rope_parameters` in current transformers and were
    `rotary_pct` / `rotary_emb_base` before."""
    H, nh = int(hf_config.hidden_size), int(hf_config.num_attention_heads)
    D = H // nh
    rp = getattr(hf_config, "rope_parameters", None) or {}
    pct = rp.get("partial_rotary_factor", getattr(hf_config, "rotary_pct", 0.25))
    base = rp.get("rope_theta", getattr(hf_config, "rotary_emb_base", 10000.0))
    if not getattr(hf_config, "use_parallel_residual", True):
        raise ValueError("the decode kernels implement GPT-NeoX's parallel residual only (use_parallel_residual=True)")
    return NeoxConfig(hidden=H, heads=nh, head_dim=D, rotary_dim=int(D * pct), ffn=int(hf_config.intermediate_size),
                      n_layers=int(hf_config.num_hidden_layers), vocab=int(hf_config.vocab_size),
                      eps=float(hf_config.layer_norm_eps), rope_base=float(base))


def _hf_layer_kv(past_key_values, l):
    """Layer l's (key, value) `[1, heads, S, D]` of a transformers cache object or of the legacy tuple of pairs."""
    if hasattr(past_key_values, "layers"):
        layer = past_key_values.layers[l]
        return layer.keys, layer.values
    if hasattr(past_key_values, "key_cache"):
        return past_key_values.key_cache[l], past_key_values.value_cache[l]
    return past_key_values[l][0], past_key_values[l][1]


def stack_tensors_from_hf(hf_model, past_key_values, max_rows: int, dtype=torch.float16, device=None):
    """Everything a whole-model decoder needs, taken from a HuggingFace `GPTNeoXForCausalLM` and the `past_key_values`
    of its prefill: the hand-off reference tests/benchmark_decode.py:60-119 does by hand (12 tensors per layer,
    `embed_in`, `final_layer_norm`, `embed_out`, one `[max_rows, H]` K and V cache per layer holding the prefilled
    positions).  Returns a dict with `cfg`, `layers`, `embed`, `final_ln_w`, `final_ln_b`, `lm_head`, `k_caches`,
    `v_caches` and `seq_len` (positions already in the caches)."""
    cfg = config_from_hf(hf_model.config)
    act = getattr(hf_model.config, "hidden_act", "gelu")
    if act not in ("gelu_pytorch_tanh", "gelu_new", "gelu_fast", "gelu"):
        raise ValueError(f"hidden_act {act!r}: the decode kernels compute tanh-GELU")
    if act == "gelu":
        import warnings
        warnings.warn("hidden_act 'gelu' (erf): the decode kernels compute the tanh form, as the reference's kernels do "
                      "(reference include/5090/pythia_2b8/kernel.cuh:26-49); expect differences of the order of 1e-3")
    body = hf_model.gpt_neox
    if len(body.layers) != cfg.n_layers:
        raise ValueError("config and module disagree on the number of layers")

    def conv(t):
        t = t.detach().to(dtype)
        return (t.to(device) if device is not None else t).contiguous()
    layers = [layer_tensors_from_hf(l, dtype=dtype, device=device) for l in body.layers]
    k_caches, v_caches, seq = [], [], None
    for l in range(cfg.n_layers):
        key, value = _hf_layer_kv(past_key_values, l)
        kc, vc, n = kv_cache_from_hf(key, value, rows=max_rows, dtype=dtype, device=device)
        if seq is not None and n != seq:
            raise ValueError(f"layer {l} holds {n} cached positions, layer 0 holds {seq}")
        seq = n
        k_caches.append(kc)
        v_caches.append(vc)
    if seq >= max_rows:
        raise ValueError(f"max_rows ({max_rows}) leaves no cache row for the first generated token ({seq} cached positions)")
    return {"cfg": cfg, "layers": layers, "embed": conv(body.embed_in.weight),
            "final_ln_w": conv(body.final_layer_norm.weight), "final_ln_b": conv(body.final_layer_norm.bias),
            "lm_head": conv(hf_model.get_output_embeddings().weight), "k_caches": k_caches, "v_caches": v_caches, "seq_len": seq}


class NeoxDecoder:
    """Greedy batch-1 decoder over device-resident weights and KV caches.

    `layers` is a list of dicts keyed by `layer_tensor_order`; caches are `[cache_rows, H]` fp16
    (HF `past_key_values` `[1, heads, S, D]` maps to this layout by `permute(0,2,1,3).reshape(S, H)`,
    reference tests/benchmark_decode.py:99-108)."""

    def __init__(self, cfg: NeoxConfig, layers: Sequence[Dict[str, torch.Tensor]], embed: torch.Tensor,
                 final_ln_w: torch.Tensor, final_ln_b: torch.Tensor, lm_head: torch.Tensor,
                 k_caches: List[torch.Tensor], v_caches: List[torch.Tensor], mode: str = "fused"):
        from . import _clusterfusion as native
        self.cfg = cfg
        self._layers, self._k_caches, self._v_caches = list(layers), list(k_caches), list(v_caches)   # keep the storage alive
        rows = k_caches[0].shape[0]
        self.cos, self.sin = rope_tables(rows, cfg.rotary_dim, cfg.rope_base, device=embed.device)
        packed = [[w[k].reshape(-1) if w[k].dim() == 1 else w[k] for k in layer_tensor_order] for w in layers]
        self._stack = native.NeoxStack(cfg.hidden, cfg.heads, cfg.head_dim, cfg.rotary_dim, cfg.ffn, cfg.eps,
                                       packed, embed, final_ln_w, final_ln_b, lm_head, list(k_caches), list(v_caches),
                                       self.cos, self.sin, {"fused": 0, "split": 1, "fused_layers": 2}[mode])

    @classmethod
    def from_hf(cls, hf_model, past_key_values, max_rows: int, device="cuda", mode: str = "fused"):
        """The prefill -> decode hand-off for a whole model (reference tests/benchmark_decode.py:60-119,147-189): a
        HuggingFace `GPTNeoXForCausalLM` and the `past_key_values` of its prefill become a decoder whose caches hold the
        prefilled positions and have room for `max_rows` positions in all.  Returns `(decoder, seq_len)`; continue with
        `decoder.set_state(first_generated_token, seq_len)` and `graph_steps`."""
        t = stack_tensors_from_hf(hf_model, past_key_values, max_rows, dtype=torch.float16, device=device)
        dec = cls(t["cfg"], t["layers"], t["embed"], t["final_ln_w"], t["final_ln_b"], t["lm_head"], t["k_caches"], t["v_caches"],
                  mode=mode)
        return dec, t["seq_len"]

    def set_state(self, token: int, seq_len: int):
        self._stack.set_state(int(token), int(seq_len))

    def step(self):
        """One eager decode step (one launch per kernel)."""
        self._stack.step()

    def graph_steps(self, n: int):
        """`n` decode steps, each one replay of the captured hipGraph.  Raises instead of stepping past the last
        cache row."""
        self._stack.graph_steps(int(n))

    def profile_step(self):
        """One eager step with HIP events around every layer launch: (layer_ms list, lm_head_ms, step_ms).  When one
        launch runs all layers (`layers_per_launch`), every entry of the list is that launch's duration / n_layers."""
        return self._stack.profile_step()

    @property
    def layers_per_launch(self) -> int:
        """Decoder layers per launch of a step: all of them when the stack runs the model's layers in one launch (fused
        mode on a device that holds the whole grid), else 1."""
        return int(self._stack.layers_per_launch())

    @property
    def logits(self) -> torch.Tensor:
        return self._stack.logits()

    @property
    def hidden(self) -> torch.Tensor:
        return self._stack.hidden()

    @property
    def state(self) -> torch.Tensor:
        """int32 `[token, seq_len, steps_done]` on the device; to read, not to write (`set_state` also fetches the
        token's embedding row, which every step after it hands to the next one)."""
        return self._stack.state()

    def check(self):
        """Synchronises and raises RuntimeError if a step since the last check raised a device-side failure flag
        (an expired bounded wait inside a fused launch, a position beyond the caches)."""
        self._stack.check()

    def generated(self) -> List[int]:
        """The tokens picked since `set_state`; raises if one of the steps failed on the device."""
        self.check()
        n = int(self.state[2].item())
        return self._stack.history()[:n].tolist()
