"""CPU oracle for the GPT-NeoX / Pythia decoder-block decode step.

TEST INFRASTRUCTURE ONLY.  This module is the checker for the HIP kernels: only the
test-suite, the smoke check and the CPU-baseline leg of the benchmark may import it.
The product package never does, and fails loudly when its HIP library is missing.

It restates, in plain torch on the CPU, the layer maths that the reference checks its
CUDA kernels against and that the kernels implement:

  * layer semantics            reference tests/test_pythia.py:71-160,
                               tests/test_pythia_6b9.py:89-180
  * tanh-GELU MLP              reference tests/test_pythia.py:166-180
  * partial NeoX rotary        reference tests/test_pythia.py:44-69
  * bias -> RoPE -> append     reference include/5090/pythia_2b8/kernel.cuh:383-432
  * S cached rows + new token  reference include/5090/pythia_2b8/kernel.cuh:489-506,597-638
  * shared LN statistics       reference include/5090/pythia_2b8/kernel.cuh:811-818
  * residual order             reference include/5090/pythia_2b8/kernel.cuh:939-949
  * RoPE table, cache layout,  reference tests/benchmark_decode.py:39-57,83-108,147-189
    full-model decode loop

Unlike the reference's fp16 restatement, every intermediate is kept in the working
dtype (float32 or float64); only the values the API makes visible in fp16 are rounded
(k_new, v_new, the cache row, mlp_intermediate, output) and only when `round_io=True`.

Parity pinning (what checks this file; see tests/test_oracle_*.py):
  neox_layer_decode   pinned  - HuggingFace GPTNeoXLayer built locally from a config,
                                a pure-Python float64 brute force on a tiny layer,
                                closed forms (zero weights, S=0, identical keys, ...)
  layer_norm          pinned  - torch.nn.functional.layer_norm, constant-vector closed form
  rope_partial_neox   pinned  - identity at cos=1/sin=0, norm preservation, HF apply_rotary_pos_emb
  rope_table          pinned  - HF GPTNeoXRotaryEmbedding
  gelu_tanh           pinned  - torch.nn.functional.gelu(approximate="tanh")
  neox_stack_decode   pinned  - HuggingFace GPTNeoXForCausalLM built locally (tiny config)
  llama_layer_decode  pinned  - HuggingFace LlamaDecoderLayer built locally (tiny config)
  llama_attention_sglang pinned - HuggingFace LlamaRMSNorm + LlamaAttention built locally, S=0 and
                                zero-angle closed forms
  llama_mlp           pinned  - through llama_layer_decode (HF LlamaDecoderLayer) and torch silu
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class NeoxDims:
    hidden: int
    heads: int
    head_dim: int
    rotary_dim: int
    ffn: int
    eps: float = 1e-5

    @property
    def qkv_rows(self) -> int:
        return 3 * self.heads * self.head_dim


PYTHIA_2B8 = NeoxDims(hidden=2560, heads=32, head_dim=80, rotary_dim=20, ffn=10240)
PYTHIA_6B9 = NeoxDims(hidden=4096, heads=32, head_dim=128, rotary_dim=32, ffn=16384)

LAYER_KEYS = (
    "ln_w", "ln_b", "w_qkv", "b_qkv", "w_o", "b_o",
    "post_ln_w", "post_ln_b", "w_up", "b_up", "w_down", "b_down",
)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """Biased-variance LayerNorm over the last dim (reference tests/test_pythia.py:86-88)."""
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) (reference tests/test_pythia.py:166-170)."""
    c = math.sqrt(2.0 / math.pi)
    return 0.5 * x * (1.0 + torch.tanh(c * (x + 0.044715 * x ** 3)))


def rope_table(positions: torch.Tensor, rotary_dim: int, base: float = 10000.0,
               dtype: torch.dtype = torch.float32) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin rows `[len(positions), rotary_dim]`, emb = cat(freqs, freqs)
    (reference tests/benchmark_decode.py:39-57)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim))
    freqs = positions.to(torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rope_partial_neox(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    """NeoX rotate-half RoPE on the first `rotary_dim` dims of `[..., D]`; the rest pass through
    (reference tests/test_pythia.py:44-69; kernel.cuh:395-421)."""
    cos = cos.reshape(-1)[:rotary_dim].to(t.dtype)
    sin = sin.reshape(-1)[:rotary_dim].to(t.dtype)
    half = rotary_dim // 2
    rot, rest = t[..., :rotary_dim], t[..., rotary_dim:]
    rotated = torch.cat([-rot[..., half:], rot[..., :half]], dim=-1)
    return torch.cat([rot * cos + rotated * sin, rest], dim=-1)


def _r16(t: torch.Tensor, on: bool) -> torch.Tensor:
    return t.to(torch.float16).to(t.dtype) if on else t


def neox_layer_decode(
    x: torch.Tensor,
    w: Dict[str, torch.Tensor],
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    seq_len: int,
    dims: NeoxDims,
    dtype: torch.dtype = torch.float32,
    round_io: bool = True,
    write_cache: bool = False,
) -> Dict[str, torch.Tensor]:
    """One decode step of one GPT-NeoX layer, batch 1.

    x `[1,H]`; w = dict over LAYER_KEYS with nn.Linear `[out,in]` weights and head-interleaved
    QKV `[h][q|k|v][D]`; caches `[rows,H]` with rows `[0,seq_len)` valid; cos/sin >= rotary_dim
    entries for the current position.  Returns a dict with `output [1,H]`, `k_new`/`v_new`
    `[1,heads,D]`, plus intermediates `attn_output [1,H]` (O-proj incl. bias),
    `mlp_intermediate [F]`, `attn_heads [heads,D]`, `q [heads,D]`.
    `current_seq_len` counts the valid rows before the append
    (reference pythia_kernel_dispatch.cu:68-75).
    """
    H, nh, D = dims.hidden, dims.heads, dims.head_dim
    f = lambda t: t.detach().to("cpu").to(dtype)
    xx = f(x).reshape(1, H)
    ln1 = layer_norm(xx, f(w["ln_w"]).reshape(H), f(w["ln_b"]).reshape(H), dims.eps)
    ln2 = layer_norm(xx, f(w["post_ln_w"]).reshape(H), f(w["post_ln_b"]).reshape(H), dims.eps)

    qkv = (ln1 @ f(w["w_qkv"]).t() + f(w["b_qkv"]).reshape(-1)).reshape(nh, 3, D)
    q = rope_partial_neox(qkv[:, 0, :], f(cos), f(sin), dims.rotary_dim)
    k_new = _r16(rope_partial_neox(qkv[:, 1, :], f(cos), f(sin), dims.rotary_dim), round_io)
    v_new = _r16(qkv[:, 2, :], round_io)

    kc = f(k_cache[:seq_len]).reshape(seq_len, nh, D)
    vc = f(v_cache[:seq_len]).reshape(seq_len, nh, D)
    keys = torch.cat([kc, k_new[None]], dim=0).permute(1, 0, 2)       # [nh, S+1, D]
    vals = torch.cat([vc, v_new[None]], dim=0).permute(1, 0, 2)
    scores = torch.einsum("hd,hsd->hs", q, keys) / math.sqrt(D)
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("hs,hsd->hd", p, vals)                           # [nh, D]

    attn = o.reshape(1, H) @ f(w["w_o"]).t() + f(w["b_o"]).reshape(-1)
    up = ln2 @ f(w["w_up"]).t() + f(w["b_up"]).reshape(-1)
    inter = _r16(gelu_tanh(up), round_io)
    mlp = inter @ f(w["w_down"]).t() + f(w["b_down"]).reshape(-1)
    out = _r16(xx + attn + mlp, round_io)

    if write_cache and k_cache.shape[0] > seq_len:
        k_cache[seq_len] = k_new.reshape(H).to(k_cache.dtype)
        v_cache[seq_len] = v_new.reshape(H).to(v_cache.dtype)
    return {
        "output": out, "k_new": k_new[None], "v_new": v_new[None],
        "attn_output": attn, "mlp_intermediate": inter.reshape(-1),
        "attn_heads": o, "q": q,
    }


def neox_stack_decode(
    token: int,
    embed: torch.Tensor,
    layers: List[Dict[str, torch.Tensor]],
    final_ln_w: torch.Tensor,
    final_ln_b: torch.Tensor,
    lm_head: torch.Tensor,
    k_caches: List[torch.Tensor],
    v_caches: List[torch.Tensor],
    seq_len: int,
    dims: NeoxDims,
    dtype: torch.dtype = torch.float32,
    base: float = 10000.0,
) -> Dict[str, torch.Tensor]:
    """One greedy decode step of the whole model: embedding row (fp16) -> layers (appending to
    the caches in place) -> final LayerNorm -> LM head -> argmax
    (reference tests/benchmark_decode.py:147-189)."""
    cos, sin = rope_table(torch.tensor([seq_len]), dims.rotary_dim, base)
    h = embed[token].to(torch.float16).reshape(1, dims.hidden)
    hiddens = []
    for w, kc, vc in zip(layers, k_caches, v_caches):
        r = neox_layer_decode(h, w, kc, vc, cos, sin, seq_len, dims, dtype=dtype, write_cache=True)
        h = r["output"].to(torch.float16)
        hiddens.append(h)
    hn = layer_norm(h.to(dtype), final_ln_w.to(dtype).reshape(-1), final_ln_b.to(dtype).reshape(-1), dims.eps)
    logits = hn @ lm_head.to(dtype).t()
    return {"logits": logits.reshape(-1), "next_token": int(torch.argmax(logits)), "hiddens": hiddens}


# --------------------------------------------------------------------------------------
# LLaMA-style layer (RMSNorm, full RoPE, SwiGLU, no biases)
# --------------------------------------------------------------------------------------

@dataclass(frozen=True)
class LlamaDims:
    hidden: int
    heads: int
    head_dim: int
    ffn: int
    eps: float = 1e-6


LLAMA2_7B = LlamaDims(hidden=4096, heads=32, head_dim=128, ffn=11008)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w (reference tests/test_llama.py:57-75)."""
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def llama_layer_decode(
    x: torch.Tensor,
    w: Dict[str, torch.Tensor],
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    seq_len: int,
    dims: LlamaDims,
    dtype: torch.dtype = torch.float32,
    round_io: bool = True,
) -> Dict[str, torch.Tensor]:
    """One decode step of a LLaMA-2 layer, batch 1, NeoX (rotate-half) RoPE pairing as in HF:
    h = x + Wo attn(rope(Wq n1), rope(Wk n1), Wv n1);  out = h + Wd (silu(Wg n2) * (Wu n2)),
    n1 = rmsnorm(x), n2 = rmsnorm(h).  Weights: `w_qkv [3H,H]` = [Wq;Wk;Wv] (not interleaved),
    `w_o [H,H]`, `w_gate_up [2F,H]` = [Wg;Wu], `w_down [H,F]`, `rms1 [H]`, `rms2 [H]`
    (reference tests/test_llama.py:57-113; include/5090/llama/kernel_sglang.cuh)."""
    H, nh, D = dims.hidden, dims.heads, dims.head_dim
    f = lambda t: t.detach().to("cpu").to(dtype)
    xx = f(x).reshape(1, H)
    n1 = rms_norm(xx, f(w["rms1"]).reshape(H), dims.eps)
    qkv = (n1 @ f(w["w_qkv"]).t()).reshape(3, nh, D)
    q = rope_partial_neox(qkv[0], f(cos), f(sin), D)
    k_new = _r16(rope_partial_neox(qkv[1], f(cos), f(sin), D), round_io)
    v_new = _r16(qkv[2], round_io)
    kc = f(k_cache[:seq_len]).reshape(seq_len, nh, D)
    vc = f(v_cache[:seq_len]).reshape(seq_len, nh, D)
    keys = torch.cat([kc, k_new[None]], dim=0).permute(1, 0, 2)
    vals = torch.cat([vc, v_new[None]], dim=0).permute(1, 0, 2)
    p = torch.softmax(torch.einsum("hd,hsd->hs", q, keys) / math.sqrt(D), dim=-1)
    o = torch.einsum("hs,hsd->hd", p, vals)
    attn = o.reshape(1, H) @ f(w["w_o"]).t()
    h = _r16(xx + attn, round_io)                      # the hidden state between the two blocks is an fp16 tensor
    mlp = llama_mlp(h, w, dims, dtype=dtype, round_io=round_io)
    return {"output": mlp["output"], "k_new": k_new[None], "v_new": v_new[None], "attn_output": attn, "hidden_mid": h,
            "mlp_intermediate": mlp["mlp_intermediate"], "attn_heads": o}


def llama_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], dims: LlamaDims, dtype: torch.dtype = torch.float32,
              round_io: bool = True) -> Dict[str, torch.Tensor]:
    """out = h + Wd (silu(Wg n) * (Wu n)), n = rmsnorm(h) * rms2; `w_gate_up [2F,H]` = [Wg;Wu], `w_down [H,F]`
    (HF LlamaMLP / LlamaDecoderLayer; the reference's own test leaves this block commented out,
    reference tests/test_llama.py:108-110)."""
    H = dims.hidden
    f = lambda t: t.detach().to("cpu").to(dtype)
    hh = f(h).reshape(1, H)
    n2 = rms_norm(hh, f(w["rms2"]).reshape(H), dims.eps)
    gu = (n2 @ f(w["w_gate_up"]).t()).reshape(2, dims.ffn)
    inter = _r16(torch.nn.functional.silu(gu[0]) * gu[1], round_io)
    out = _r16(hh + inter.reshape(1, -1) @ f(w["w_down"]).t(), round_io)
    return {"output": out, "mlp_intermediate": inter.reshape(-1)}


def llama_attention_sglang(
    x: torch.Tensor,
    residual: Optional[torch.Tensor],
    w: Dict[str, torch.Tensor],
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    dims: LlamaDims,
    dtype: torch.dtype = torch.float32,
    round_io: bool = True,
) -> Dict[str, torch.Tensor]:
    """The attention block the reference fuses for LLaMA (`llama_decoder_layer_sglang`): fused add + RMSNorm,
    stacked QKV projection, NeoX RoPE over the whole head, attention over every cache row plus the new token
    (the caches are not written), O projection without bias or residual
    (reference tests/test_llama.py:57-113; include/5090/llama/kernel_sglang.cuh:97-105 residual add with fp16
    rounding, :292-293 rope angles cos[d % (D/2)], :332-333 returned k / v;
    llama_kernel_sglang_dispatch.cu:40 SEQ_LEN = k_cache.size(0)).
    Weights: `rms1 [H]`, `w_qkv [3H,H]` = [Wq;Wk;Wv], `w_o [H,H]`."""
    H, nh, D = dims.hidden, dims.heads, dims.head_dim
    f = lambda t: t.detach().to("cpu").to(dtype)
    r = f(x).reshape(1, H)
    if residual is not None:
        r = _r16(r + f(residual).reshape(1, H), True)        # the sum is an fp16 value in the reference as well
    n1 = rms_norm(r, f(w["rms1"]).reshape(H), dims.eps)
    qkv = (n1 @ f(w["w_qkv"]).t()).reshape(3, nh, D)
    half = D // 2
    c = f(cos).reshape(-1)[:half]
    sn = f(sin).reshape(-1)[:half]
    c2, s2 = torch.cat([c, c]), torch.cat([sn, sn])
    q = rope_partial_neox(qkv[0], c2, s2, D)
    k_new = _r16(rope_partial_neox(qkv[1], c2, s2, D), round_io)
    v_new = _r16(qkv[2], round_io)
    S = k_cache.shape[0]
    kc = f(k_cache).reshape(S, nh, D)
    vc = f(v_cache).reshape(S, nh, D)
    keys = torch.cat([kc, k_new[None]], dim=0).permute(1, 0, 2)
    vals = torch.cat([vc, v_new[None]], dim=0).permute(1, 0, 2)
    p = torch.softmax(torch.einsum("hd,hsd->hs", q, keys) / math.sqrt(D), dim=-1)
    o = torch.einsum("hs,hsd->hd", p, vals)
    out = _r16(o.reshape(1, H) @ f(w["w_o"]).t(), round_io)
    return {"output": out, "residual": r, "k_new": k_new[None], "v_new": v_new[None], "attn_heads": o}


def rope_pairs_gptj(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """GPT-J RoPE over the whole last dim: dims (2i, 2i+1) rotate together, tables indexed by the dim
    (reference include/5090/llama/kernel.cuh:280-281,298-314; tests/test_llama.py:31-36,48-51):
    out[2i] = t[2i] cos[2i] - t[2i+1] sin[2i],  out[2i+1] = t[2i+1] cos[2i+1] + t[2i] sin[2i+1]."""
    D = t.shape[-1]
    cos = cos.reshape(-1)[:D].to(t.dtype)
    sin = sin.reshape(-1)[:D].to(t.dtype)
    partner = torch.stack((-t[..., 1::2], t[..., 0::2]), dim=-1).reshape(t.shape)
    return t * cos + partner * sin


def llama_attention_plain(
    x: torch.Tensor,
    w: Dict[str, torch.Tensor],
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    dims: LlamaDims,
    dtype: torch.dtype = torch.float32,
    round_io: bool = True,
) -> Dict[str, torch.Tensor]:
    """The reference's plain `llama_decoder_layer` op (include/5090/llama/kernel.cuh): RMSNorm (eps 1e-6, :58,131),
    q/k/v = n @ W with weights stored [in, out] (`w_qkv_t` [3H, H]: three such matrices stacked,
    llama_kernel_dispatch.cu:44-58; kernel.cuh:144,187,230), GPT-J RoPE on q and k (:298-314), attention over every
    cache row plus the new token, output = attn @ `w_o_t` ([in, out], :573), no residual, caches not written."""
    H, nh, D = dims.hidden, dims.heads, dims.head_dim
    f = lambda t: t.detach().to("cpu").to(dtype)
    n1 = rms_norm(f(x).reshape(1, H), f(w["rms1"]).reshape(H), 1e-6)
    wq, wk, wv = f(w["w_qkv_t"]).reshape(3, H, H)
    q = rope_pairs_gptj((n1 @ wq).reshape(nh, D), f(cos), f(sin))
    k_new = _r16(rope_pairs_gptj((n1 @ wk).reshape(nh, D), f(cos), f(sin)), round_io)
    v_new = _r16((n1 @ wv).reshape(nh, D), round_io)
    S = k_cache.shape[0]
    keys = torch.cat([f(k_cache).reshape(S, nh, D), k_new[None]], dim=0).permute(1, 0, 2)
    vals = torch.cat([f(v_cache).reshape(S, nh, D), v_new[None]], dim=0).permute(1, 0, 2)
    pr = torch.softmax(torch.einsum("hd,hsd->hs", q, keys) / math.sqrt(D), dim=-1)
    o = torch.einsum("hs,hsd->hd", pr, vals)
    out = _r16(o.reshape(1, H) @ f(w["w_o_t"]), round_io)
    return {"output": out, "k_new": k_new[None], "v_new": v_new[None], "attn_heads": o}


def llama_batch_decode_paged(
    x: torch.Tensor,
    residual: torch.Tensor,
    w: Dict[str, torch.Tensor],
    indptr: torch.Tensor,
    indices: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    positions: torch.Tensor,
    cos_sin: torch.Tensor,
    dims: LlamaDims,
    dtype: torch.dtype = torch.float32,
    round_io: bool = True,
) -> Dict[str, torch.Tensor]:
    """One decode step of a batch of sequences over paged caches (`llama_decoder_layer_batch_decode_sglang`,
    reference include/5090/llama/kernel_batch_sglang.cuh): sequence b owns the cache rows
    indices[indptr[b] : indptr[b+1]]; the last of them receives the new token's K/V (:367-370, end_idx =
    indptr[b+1]-1 at :120-122), the others are attended over together with the new token; RoPE angles come from
    cos_sin[positions[b]] = [cos(D/2) | sin(D/2)] (:343-346).  Per sequence this is `llama_attention_sglang` on the
    gathered rows.  `x`, `residual` [B,H]; caches [rows,H] (copies are updated and returned)."""
    B, H, D = x.shape[0], dims.hidden, dims.head_dim
    k_cache, v_cache = k_cache.clone(), v_cache.clone()
    outs, ress = [], []
    for b in range(B):
        lo, hi = int(indptr[b]), int(indptr[b + 1]) - 1
        rows = indices[lo:hi].long()
        cs = cos_sin[int(positions[b])].float()
        r = llama_attention_sglang(x[b:b + 1], residual[b:b + 1], w, k_cache[rows], v_cache[rows], cs[: D // 2], cs[D // 2:], dims, dtype, round_io)
        outs.append(r["output"]); ress.append(r["residual"])
        slot = int(indices[hi])
        k_cache[slot] = r["k_new"].reshape(H).to(k_cache.dtype)
        v_cache[slot] = r["v_new"].reshape(H).to(v_cache.dtype)
    return {"output": torch.cat(outs), "residual": torch.cat(ress), "k_cache": k_cache, "v_cache": v_cache}


def make_llama_attn_inputs(dims: LlamaDims, S: int, seed: int = 0, w_std: float = 0.02):
    """Seeded fp16 tensors for the LLaMA attention block: weights dict, input, residual, caches [S,H], cos/sin [1,D]
    (random angles per pair, duplicated halves, as reference tests/test_llama.py:24-28,140-142 builds them)."""
    H, D = dims.hidden, dims.head_dim
    g = torch.Generator().manual_seed(7000 + seed)
    rn = lambda *shape, std=1.0: (torch.randn(*shape, generator=g) * std).half()
    w = {"rms1": (1 + 0.1 * torch.randn(H, generator=g)).half(), "w_qkv": rn(3 * H, H, std=w_std), "w_o": rn(H, H, std=w_std)}
    x, res = rn(1, H), rn(1, H)
    k, v = rn(S, H), rn(S, H)
    ang = torch.rand(1, D // 2, generator=g) * (2 * math.pi)
    cos = torch.cat([torch.cos(ang), torch.cos(ang)], dim=-1).float()
    sin = torch.cat([torch.sin(ang), torch.sin(ang)], dim=-1).float()
    return w, x, res, k, v, cos, sin


def make_llama_plain_inputs(dims: LlamaDims, S: int, seed: int = 0, w_std: float = 0.02):
    """Seeded fp16 tensors for the plain LLaMA op: weights dict (`rms1`, `w_qkv_t` [3H,H] = three [in,out] matrices,
    `w_o_t` [in,out]), input [1,H], caches [S,H], cos/sin [1,D] with one random angle per (2i, 2i+1) pair."""
    H, D = dims.hidden, dims.head_dim
    g = torch.Generator().manual_seed(8200 + seed)
    rn = lambda *shape, std=1.0: (torch.randn(*shape, generator=g) * std).half()
    w = {"rms1": (1 + 0.1 * torch.randn(H, generator=g)).half(), "w_qkv_t": rn(3 * H, H, std=w_std), "w_o_t": rn(H, H, std=w_std)}
    x, k, v = rn(1, H), rn(S, H), rn(S, H)
    ang = torch.rand(1, D // 2, generator=g) * (2 * math.pi)
    cos = torch.repeat_interleave(torch.cos(ang), 2, dim=-1).float().contiguous()
    sin = torch.repeat_interleave(torch.sin(ang), 2, dim=-1).float().contiguous()
    return w, x, k, v, cos, sin


def make_llama_batch_inputs(dims: LlamaDims, lens, seed: int = 0, max_pos: int = 512, w_std: float = 0.02, layers: int = 3):
    """Seeded inputs of the paged batch op: sequences of `lens` cached tokens each, their pages scattered over a shared
    pool of cache rows (one pool per layer).  Returns (w, x [B,H], residual [B,H], indptr, indices, caches = [(k, v)] per
    layer, positions, cos_sin [max_pos, D])."""
    H, D, B = dims.hidden, dims.head_dim, len(lens)
    g = torch.Generator().manual_seed(9100 + seed)
    rn = lambda *shape, std=1.0: (torch.randn(*shape, generator=g) * std).half()
    w = {"rms1": (1 + 0.1 * torch.randn(H, generator=g)).half(), "w_qkv": rn(3 * H, H, std=w_std), "w_o": rn(H, H, std=w_std)}
    x, res = rn(B, H), rn(B, H)
    total = sum(lens) + B
    pool = total + 37
    indices = torch.randperm(pool, generator=g)[:total].to(torch.int32)
    indptr = torch.zeros(B + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(torch.tensor([n + 1 for n in lens]), 0).to(torch.int32)
    caches = [(rn(pool, H), rn(pool, H)) for _ in range(layers)]
    positions = torch.randint(0, max_pos, (B,), generator=g, dtype=torch.int64)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(max_pos).float()[:, None] * inv[None, :]
    cos_sin = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).float().contiguous()
    return w, x, res, indptr, indices, caches, positions, cos_sin


# --------------------------------------------------------------------------------------
# Seeded synthetic inputs shared by tests, smoke and the benchmark
# --------------------------------------------------------------------------------------

def make_layer_weights(dims: NeoxDims, layer: int = 0, w_std: float = 0.02, b_std: float = 0.01,
                       device: str = "cpu") -> Dict[str, torch.Tensor]:
    """fp16 weights ~N(0,w_std), biases ~N(0,b_std), LN weight 1+N(0,0.02), LN bias N(0,b_std);
    one CPU generator per tensor seeded 1000 + 16*layer + k."""
    H, F, Q = dims.hidden, dims.ffn, dims.qkv_rows

    def rn(k, shape, std, mean=0.0):
        g = torch.Generator().manual_seed(1000 + 16 * layer + k)
        return (torch.randn(shape, generator=g) * std + mean).to(torch.float16).to(device)

    return {
        "ln_w": rn(0, (H,), 0.02, 1.0), "ln_b": rn(1, (H,), b_std),
        "w_qkv": rn(2, (Q, H), w_std), "b_qkv": rn(3, (Q,), b_std),
        "w_o": rn(4, (H, H), w_std), "b_o": rn(5, (H,), b_std),
        "post_ln_w": rn(6, (H,), 0.02, 1.0), "post_ln_b": rn(7, (H,), b_std),
        "w_up": rn(8, (F, H), w_std), "b_up": rn(9, (F,), b_std),
        "w_down": rn(10, (H, F), w_std), "b_down": rn(11, (H,), b_std),
    }


def make_layer_inputs(dims: NeoxDims, seq_len: int, capacity: Optional[int] = None, seed: int = 0,
                      device: str = "cpu"):
    """x ~N(0,1) `[1,H]` fp16; K/V caches ~N(0,1) `[capacity,H]` fp16 (rows >= seq_len hold
    poison 1e4 so a kernel that reads them fails parity); cos/sin fp32 `[1,rot]` at position seq_len."""
    capacity = seq_len + 1 if capacity is None else capacity
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((1, dims.hidden), generator=g).to(torch.float16)
    k = torch.randn((capacity, dims.hidden), generator=g).to(torch.float16)
    v = torch.randn((capacity, dims.hidden), generator=g).to(torch.float16)
    k[seq_len:] = 1e4
    v[seq_len:] = 1e4
    cos, sin = rope_table(torch.tensor([seq_len]), dims.rotary_dim)
    return x.to(device), k.to(device), v.to(device), cos.to(device), sin.to(device)


def make_reference_unit_test_inputs(dims: NeoxDims, seq_len: int = 129, seed: int = 42, zero_bias_o: bool = False,
                                    pad_rope_to_head_dim: bool = False, ln_2d: bool = True):
    """The inputs of the reference's own layer unit tests, drawn in their order from one CPU generator
    (reference tests/test_pythia.py:15 seed 42, :162-164 every tensor `randn * 0.1` in fp16, :191-217 the order
    input, weight_qkv, bias_qkv, weight_o, bias_o, the four LayerNorm tensors as `[1,H]`, the four MLP tensors, one
    `[2, seqlen, H]` K/V block with exactly `seqlen` rows, :24-42 then RoPE from an independent uniform angle per
    rotary entry, padded to `[1, D]` with cos 1 / sin 0; tests/test_pythia_6b9.py:47-51,196-228 is the same recipe
    with a random bias_o and un-padded `[rot]` tables).  `zero_bias_o` / `pad_rope_to_head_dim` select the 2.8B
    script's choices.  Returns (weights dict, x, k_cache, v_cache, cos, sin): the two halves of cos / sin do NOT repeat,
    so a kernel that reads entry d mod rot/2 for dim d fails on these inputs."""
    H, F, D, rot = dims.hidden, dims.ffn, dims.head_dim, dims.rotary_dim
    g = torch.Generator().manual_seed(seed)
    rn = lambda *shape: (torch.randn(shape, generator=g) * 0.1).half()
    x = rn(1, H)
    w = {"w_qkv": rn(3 * H, H), "b_qkv": rn(3 * H), "w_o": rn(H, H)}
    w["b_o"] = torch.zeros(H, dtype=torch.float16) if zero_bias_o else rn(H)
    for name in ("ln_w", "ln_b", "post_ln_w", "post_ln_b"):
        t = rn(1, H)
        w[name] = t if ln_2d else t.reshape(H)
    w["w_up"], w["b_up"], w["w_down"], w["b_down"] = rn(F, H), rn(F), rn(H, F), rn(H)
    kv = rn(2, seq_len, H)
    ang = torch.rand((1, rot), generator=g, dtype=torch.float32) * (2 * math.pi)
    cos, sin = torch.cos(ang), torch.sin(ang)
    if pad_rope_to_head_dim:
        cos = torch.cat([cos, torch.ones((1, D - rot))], dim=-1)
        sin = torch.cat([sin, torch.zeros((1, D - rot))], dim=-1)
    else:
        cos, sin = cos.reshape(rot), sin.reshape(rot)
    return w, x, kv[0].contiguous(), kv[1].contiguous(), cos.contiguous(), sin.contiguous()
