"""Pins for the CPU oracle: each check is independent of the oracle's own formulae
(a third-party implementation, a brute-force loop, or a closed form / invariant)."""
import math

import pytest
import torch

from oracle import neox_oracle as O
from oracle.neox_oracle import NeoxDims

TINY = NeoxDims(hidden=64, heads=4, head_dim=16, rotary_dim=4, ffn=256)
SMALL = NeoxDims(hidden=256, heads=8, head_dim=32, rotary_dim=8, ffn=1024)


def _mk(dims, S, seed=0, w_std=0.05):
    w = O.make_layer_weights(dims, layer=seed, w_std=w_std, b_std=0.05)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S, capacity=S + 2, seed=seed)
    return w, x, k, v, cos, sin


# ---------------------------------------------------------------- HF GPTNeoXLayer (third party)
@pytest.mark.parametrize("dims,S", [(TINY, 5), (SMALL, 33), (SMALL, 0),
                                    (NeoxDims(320, 4, 80, 20, 1280), 17)])
def test_layer_matches_hf_gptneox_layer(dims, S):
    from oracle import hf_neox
    w, x, k, v, cos, sin = _mk(dims, S)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims, dtype=torch.float64, round_io=False)
    layer = hf_neox.build_hf_layer(dims, w, dtype=torch.float64)
    out, k_new, v_new = hf_neox.hf_layer_decode(layer, x, k, v, cos, sin, S, dims, dtype=torch.float64)
    # HF's eager attention runs its softmax in float32 even for a float64 module: ~1e-8 noise
    assert torch.allclose(r["output"], out, atol=1e-6, rtol=0)
    assert torch.allclose(r["k_new"], k_new, atol=1e-12, rtol=0)
    assert torch.allclose(r["v_new"], v_new, atol=1e-12, rtol=0)


def test_rope_table_matches_hf_rotary_embedding():
    from oracle import hf_neox
    from transformers.models.gpt_neox.modeling_gpt_neox import GPTNeoXRotaryEmbedding
    dims = NeoxDims(320, 4, 80, 20, 1280)
    rot = GPTNeoXRotaryEmbedding(hf_neox._config(dims))
    pos = torch.tensor([[0, 1, 7, 513, 4095]])
    c, s = rot(torch.zeros(1, 5, dims.hidden), pos)
    c2, s2 = O.rope_table(pos[0], dims.rotary_dim)
    assert c.shape[-1] == dims.rotary_dim
    # HF forms position*inv_freq in float32 (angle error ~ pos * 6e-8); the oracle uses float64 angles
    assert torch.allclose(c[0, :3], c2[:3], atol=2e-6) and torch.allclose(s[0, :3], s2[:3], atol=2e-6)
    assert torch.allclose(c[0], c2, atol=1e-3) and torch.allclose(s[0], s2, atol=1e-3)


def test_stack_matches_hf_causal_lm():
    from oracle import hf_neox
    from transformers import DynamicCache
    dims, L, V, S = TINY, 3, 97, 6
    layers = [O.make_layer_weights(dims, layer=i, w_std=0.08, b_std=0.05) for i in range(L)]
    g = torch.Generator().manual_seed(7)
    embed = torch.randn((V, dims.hidden), generator=g).half()
    lm = (torch.randn((V, dims.hidden), generator=g) * 0.1).half()
    fw = (1 + 0.02 * torch.randn(dims.hidden, generator=g)).half()
    fb = (0.01 * torch.randn(dims.hidden, generator=g)).half()
    kcs = [torch.randn((S + 2, dims.hidden), generator=g).half() for _ in range(L)]
    vcs = [torch.randn((S + 2, dims.hidden), generator=g).half() for _ in range(L)]
    model = hf_neox.build_hf_model(dims, layers, embed, fw, fb, lm, dtype=torch.float64)
    nh, D = dims.heads, dims.head_dim
    past = DynamicCache(ddp_cache_data=[
        (kc[:S].double().reshape(S, nh, D).permute(1, 0, 2)[None].contiguous(),
         vc[:S].double().reshape(S, nh, D).permute(1, 0, 2)[None].contiguous()) for kc, vc in zip(kcs, vcs)])
    tok = 11
    with torch.no_grad():
        hf = model(input_ids=torch.tensor([[tok]]), past_key_values=past,
                   position_ids=torch.tensor([[S]]), use_cache=True).logits[0, -1]
    r = O.neox_stack_decode(tok, embed, layers, fw, fb, lm, [k.clone() for k in kcs], [v.clone() for v in vcs],
                            S, dims, dtype=torch.float64)
    # the oracle rounds the hidden state to fp16 between layers (that is what the op API carries)
    assert torch.allclose(r["logits"], hf, atol=5e-3)
    assert r["next_token"] == int(hf.argmax())


# ---------------------------------------------------------------- brute force, pure Python float64
def _brute_force_layer(x, w, kc, vc, cos, sin, S, d):
    H, nh, D, rot, F = d.hidden, d.heads, d.head_dim, d.rotary_dim, d.ffn
    xs = [float(t) for t in x.reshape(-1)]
    mean = sum(xs) / H
    var = sum((t - mean) ** 2 for t in xs) / H
    rstd = 1.0 / math.sqrt(var + d.eps)
    L = lambda name: w[name].double().reshape(-1).tolist()
    M = lambda name: w[name].double().tolist()
    ln1 = [(xs[i] - mean) * rstd * L("ln_w")[i] + L("ln_b")[i] for i in range(H)]
    ln2 = [(xs[i] - mean) * rstd * L("post_ln_w")[i] + L("post_ln_b")[i] for i in range(H)]
    Wq, bq = M("w_qkv"), L("b_qkv")
    qkv = [sum(Wq[r][c] * ln1[c] for c in range(H)) + bq[r] for r in range(3 * H)]
    cs, sn = cos.double().reshape(-1).tolist(), sin.double().reshape(-1).tolist()

    def rope(vec):
        o = list(vec)
        for i in range(rot // 2):
            a, b = vec[i], vec[i + rot // 2]
            o[i] = a * cs[i] - b * sn[i]
            o[i + rot // 2] = b * cs[i + rot // 2] + a * sn[i + rot // 2]
        return o

    attn_in = []
    k_new, v_new = [], []
    for h in range(nh):
        base = h * 3 * D
        q = rope(qkv[base:base + D])
        k = rope(qkv[base + D:base + 2 * D])
        v = qkv[base + 2 * D:base + 3 * D]
        k_new.append(k)
        v_new.append(v)
        keys = [kc[s, h * D:(h + 1) * D].double().tolist() for s in range(S)] + [k]
        vals = [vc[s, h * D:(h + 1) * D].double().tolist() for s in range(S)] + [v]
        sc = [sum(q[i] * kk[i] for i in range(D)) / math.sqrt(D) for kk in keys]
        m = max(sc)
        e = [math.exp(t - m) for t in sc]
        z = sum(e)
        attn_in += [sum(e[s] * vals[s][i] for s in range(S + 1)) / z for i in range(D)]
    Wo, bo = M("w_o"), L("b_o")
    attn = [sum(Wo[r][c] * attn_in[c] for c in range(H)) + bo[r] for r in range(H)]
    Wu, bu = M("w_up"), L("b_up")
    up = [sum(Wu[r][c] * ln2[c] for c in range(H)) + bu[r] for r in range(F)]
    g = [0.5 * t * (1 + math.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t ** 3))) for t in up]
    Wd, bd = M("w_down"), L("b_down")
    out = [xs[r] + attn[r] + sum(Wd[r][c] * g[c] for c in range(F)) + bd[r] for r in range(H)]
    return out, k_new, v_new


def test_layer_matches_pure_python_brute_force():
    d, S = TINY, 5
    w, x, k, v, cos, sin = _mk(d, S, seed=3, w_std=0.1)
    out, k_new, v_new = _brute_force_layer(x, w, k, v, cos, sin, S, d)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, d, dtype=torch.float64, round_io=False)
    assert torch.allclose(r["output"].reshape(-1), torch.tensor(out, dtype=torch.float64), atol=1e-10)
    assert torch.allclose(r["k_new"].reshape(-1), torch.tensor(k_new, dtype=torch.float64).reshape(-1), atol=1e-12)
    assert torch.allclose(r["v_new"].reshape(-1), torch.tensor(v_new, dtype=torch.float64).reshape(-1), atol=1e-12)


# ---------------------------------------------------------------- closed forms and invariants
def test_layer_norm_against_torch_and_constant_vector():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 96, generator=g, dtype=torch.float64)
    w, b = torch.randn(96, generator=g, dtype=torch.float64), torch.randn(96, generator=g, dtype=torch.float64)
    assert torch.allclose(O.layer_norm(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (96,), w, b, 1e-5), atol=1e-12)
    assert torch.allclose(O.layer_norm(torch.full((1, 96), 3.25, dtype=torch.float64), w, b, 1e-5), b[None], atol=1e-12)


def test_gelu_against_torch():
    x = torch.linspace(-12, 12, 4001, dtype=torch.float64)
    assert torch.allclose(O.gelu_tanh(x), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-12)


def test_rope_identity_norm_and_passthrough():
    g = torch.Generator().manual_seed(2)
    t = torch.randn(4, 16, generator=g, dtype=torch.float64)
    one, zero = torch.ones(8), torch.zeros(8)
    assert torch.equal(O.rope_partial_neox(t, one, zero, 8), t)
    c0, s0 = O.rope_table(torch.tensor([0]), 8)
    assert torch.allclose(O.rope_partial_neox(t, c0, s0, 8), t, atol=1e-12)
    c, s = O.rope_table(torch.tensor([37]), 8, dtype=torch.float64)
    r = O.rope_partial_neox(t, c, s, 8)
    assert torch.equal(r[:, 8:], t[:, 8:])
    for i in range(4):   # pairs (i, i+4) are rotated: norm preserved
        assert torch.allclose(r[:, i] ** 2 + r[:, i + 4] ** 2, t[:, i] ** 2 + t[:, i + 4] ** 2, atol=1e-12)
    # sign convention: rotating e_0 by angle theta gives (cos, sin) on dims (0, rot/2)
    e = torch.zeros(1, 16, dtype=torch.float64); e[0, 0] = 1
    r = O.rope_partial_neox(e, c, s, 8)
    assert math.isclose(r[0, 0], math.cos(37.0)) and math.isclose(r[0, 4], math.sin(37.0))


def test_zero_weights_give_identity_and_bias_only():
    d, S = SMALL, 9
    w, x, k, v, cos, sin = _mk(d, S)
    z = {n: torch.zeros_like(t) for n, t in w.items()}
    z["ln_w"], z["post_ln_w"] = w["ln_w"], w["post_ln_w"]
    r = O.neox_layer_decode(x, z, k, v, cos, sin, S, d)
    assert torch.equal(r["output"].half(), x)
    z["b_o"], z["b_down"] = w["b_o"], w["b_down"]
    r = O.neox_layer_decode(x, z, k, v, cos, sin, S, d, dtype=torch.float64, round_io=False)
    assert torch.allclose(r["output"], x.double() + w["b_o"].double() + w["b_down"].double(), atol=1e-12)


def test_attention_special_cases():
    d = SMALL
    w, x, k, v, cos, sin = _mk(d, 0)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, 0, d, dtype=torch.float64, round_io=False)
    assert torch.allclose(r["attn_heads"], r["v_new"][0], atol=1e-12)          # S=0: only the new token
    S = 12
    w, x, k, v, cos, sin = _mk(d, S)
    r0 = O.neox_layer_decode(x, w, k, v, cos, sin, S, d, dtype=torch.float64, round_io=False)
    k[:S] = r0["k_new"].reshape(1, -1).half()                                  # all keys identical -> mean of V
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, d, dtype=torch.float64, round_io=True)
    mean_v = (v[:S].double().sum(0) + r["v_new"].reshape(-1)) / (S + 1)
    assert torch.allclose(r["attn_heads"].reshape(-1), mean_v, atol=1e-9)
    # permutation invariance over cache rows and independence from rows >= S
    w, x, k, v, cos, sin = _mk(d, S)
    perm = torch.randperm(S, generator=torch.Generator().manual_seed(0))
    k2, v2 = k.clone(), v.clone()
    k2[:S], v2[:S] = k[perm], v[perm]
    k2[S:], v2[S:] = -7.0, 123.0
    a = O.neox_layer_decode(x, w, k, v, cos, sin, S, d, dtype=torch.float64)["output"]
    b = O.neox_layer_decode(x, w, k2, v2, cos, sin, S, d, dtype=torch.float64)["output"]
    assert torch.allclose(a, b, atol=1e-12)
    # a dominant key selects its V row
    k3 = k.clone()
    q = r0["q"]
    k3[3] = (q.reshape(-1) * 50).half()
    r = O.neox_layer_decode(x, w, k3, v, cos, sin, S, d, dtype=torch.float64, round_io=False)
    assert torch.allclose(r["attn_heads"].reshape(-1), v[3].double(), atol=1e-6)


def test_cache_side_effect():
    d, S = SMALL, 7
    w, x, k, v, cos, sin = _mk(d, S)
    k0, v0 = k.clone(), v.clone()
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, d, write_cache=True)
    assert torch.equal(k[S], r["k_new"].reshape(-1).half()) and torch.equal(v[S], r["v_new"].reshape(-1).half())
    keep = [i for i in range(k.shape[0]) if i != S]
    assert torch.equal(k[keep], k0[keep]) and torch.equal(v[keep], v0[keep])


# ---- LLaMA ------------------------------------------------------------------------------------------

def _tiny_llama():
    dims = O.LlamaDims(hidden=64, heads=4, head_dim=16, ffn=96, eps=1e-6)
    S = 7
    w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, S, seed=1, w_std=0.2)
    g = torch.Generator().manual_seed(77)
    w["rms2"] = (1 + 0.1 * torch.randn(dims.hidden, generator=g)).half()
    w["w_gate_up"] = (0.2 * torch.randn(2 * dims.ffn, dims.hidden, generator=g)).half()
    w["w_down"] = (0.2 * torch.randn(dims.hidden, dims.ffn, generator=g)).half()
    return dims, S, w, x, res, k, v, cos, sin


def test_llama_attention_sglang_matches_hf_llama_attention():
    """fused add + RMSNorm + stacked QKV + whole-head NeoX RoPE + attention + O projection == HF LlamaRMSNorm + LlamaAttention."""
    hf = pytest.importorskip("transformers")
    from oracle import hf_neox
    dims, S, w, x, res, k, v, cos, sin = _tiny_llama()
    got = O.llama_attention_sglang(x, res, w, k, v, cos, sin, dims, dtype=torch.float64, round_io=False)
    r = (x.double() + res.double()).half().double()
    assert torch.equal(got["residual"], r)
    layer = hf_neox.build_hf_llama_layer(dims, w, dtype=torch.float64)
    want, k_new, v_new = hf_neox.hf_llama_attention(layer, r, k, v, cos, sin, dims, dtype=torch.float64)
    assert torch.allclose(got["output"], want, atol=1e-6, rtol=0)   # HF eager attention takes its softmax in float32
    # (HF's LlamaRMSNorm works in float32 whatever the module dtype: agreement to float32 rounding)
    assert torch.allclose(got["k_new"], k_new, atol=1e-6, rtol=0) and torch.allclose(got["v_new"], v_new, atol=1e-6, rtol=0)


def test_llama_layer_decode_matches_hf_llama_decoder_layer():
    hf = pytest.importorskip("transformers")
    from oracle import hf_neox
    dims, S, w, x, res, k, v, cos, sin = _tiny_llama()
    got = O.llama_layer_decode(x, w, k, v, cos, sin, S, dims, dtype=torch.float64, round_io=False)
    layer = hf_neox.build_hf_llama_layer(dims, w, dtype=torch.float64)
    want, k_new, v_new = hf_neox.hf_llama_layer_decode(layer, x, k, v, cos, sin, S, dims, dtype=torch.float64)
    assert torch.allclose(got["output"], want, atol=3e-6, rtol=0)   # HF works in float32 inside RMSNorm and softmax
    assert torch.allclose(got["k_new"], k_new, atol=1e-6, rtol=0)


def test_llama_attention_closed_forms():
    dims, S, w, x, res, k, v, cos, sin = _tiny_llama()
    # no cache rows: the only key is the new token, so the head outputs are its V
    got = O.llama_attention_sglang(x, res, w, k[:0], v[:0], cos, sin, dims, dtype=torch.float64, round_io=False)
    assert torch.allclose(got["attn_heads"], got["v_new"][0], atol=1e-12, rtol=0)
    # without a residual the norm sees the input itself
    got2 = O.llama_attention_sglang(x, None, w, k, v, cos, sin, dims, dtype=torch.float64, round_io=False)
    assert torch.equal(got2["residual"], x.double())
    # zero angles: RoPE is the identity, k_new = Wk n
    one, zero = torch.ones(1, dims.head_dim), torch.zeros(1, dims.head_dim)
    got3 = O.llama_attention_sglang(x, None, w, k, v, one, zero, dims, dtype=torch.float64, round_io=False)
    n = O.rms_norm(x.double(), w["rms1"].double(), dims.eps)
    assert torch.allclose(got3["k_new"].reshape(-1), (n @ w["w_qkv"].double().t()).reshape(3, -1)[1], atol=1e-12, rtol=0)


def test_llama_batch_decode_paged_matches_hf_per_sequence():
    """Page-table conventions of the batched op, against HF modules fed by hand: the sequence's history is the rows
    indices[indptr[b] : indptr[b+1]-1], the new K/V lands in row indices[indptr[b+1]-1], and the angles of position p
    are row p of cos_sin = [cos | sin] — here HF's own LlamaRotaryEmbedding evaluated at that position."""
    hf = pytest.importorskip("transformers")
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    from oracle import hf_neox
    dims, _, w, _, _, _, _, _, _ = _tiny_llama()
    H, D = dims.hidden, dims.head_dim
    g = torch.Generator().manual_seed(5)
    lens = [5, 0, 9]
    B, pool, max_pos = len(lens), 40, 64
    x = torch.randn(B, H, generator=g).half()
    res = torch.randn(B, H, generator=g).half()
    k = torch.randn(pool, H, generator=g).half()
    v = torch.randn(pool, H, generator=g).half()
    indices = torch.randperm(pool, generator=g)[: sum(lens) + B].to(torch.int32)
    indptr = torch.tensor([0, 6, 7, 17], dtype=torch.int32)
    positions = torch.tensor([5, 63, 20], dtype=torch.int64)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).double() / D))
    ang = torch.arange(max_pos).double()[:, None] * inv[None, :]
    cos_sin = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1)
    got = O.llama_batch_decode_paged(x, res, w, indptr, indices, k, v, positions, cos_sin, dims, dtype=torch.float64, round_io=False)

    layer = hf_neox.build_hf_llama_layer(dims, w, dtype=torch.float64)
    cfg = LlamaConfig(hidden_size=H, num_attention_heads=dims.heads, head_dim=D, max_position_embeddings=max_pos, rope_theta=10000.0)
    rotary = LlamaRotaryEmbedding(cfg)
    touched = []
    for b in range(B):
        lo, hi = int(indptr[b]), int(indptr[b + 1]) - 1
        rows = indices[lo:hi].long()
        hc, hs = rotary(torch.zeros(1, 1, H, dtype=torch.float64), positions[b].reshape(1, 1))     # [1,1,D] each
        r = (x[b:b + 1].double() + res[b:b + 1].double()).half().double()
        want, k_new, v_new = hf_neox.hf_llama_attention(layer, r, k[rows], v[rows], hc, hs, dims, dtype=torch.float64)
        assert torch.allclose(got["output"][b:b + 1].double(), want, atol=1e-6, rtol=0)      # HF takes norm and softmax in float32
        slot = int(indices[hi])
        touched.append(slot)
        # the caches hold fp16
        assert torch.equal(got["k_cache"][slot], k_new.reshape(-1).half()) or torch.allclose(got["k_cache"][slot].double(), k_new.reshape(-1), atol=0, rtol=1e-3)
        assert torch.allclose(got["v_cache"][slot].double(), v_new.reshape(-1), atol=1e-6, rtol=1e-3)
        assert torch.equal(got["residual"][b:b + 1].double(), r)
    keep = torch.ones(pool, dtype=torch.bool)
    keep[touched] = False
    assert torch.equal(got["k_cache"][keep], k[keep]) and torch.equal(got["v_cache"][keep], v[keep])


def test_rope_pairs_gptj_matches_hf_gptj_rotary():
    """Pairing and sign convention of the GPT-J rotary, against HF's GPT-J helper (tables with one angle per pair,
    repeated for the two dims of the pair, as `apply_rotary_pos_emb` of modeling_gptj builds them)."""
    hf = pytest.importorskip("transformers")
    from transformers.models.gptj.modeling_gptj import apply_rotary_pos_emb as gptj_rope
    g = torch.Generator().manual_seed(3)
    D = 16
    t = torch.randn(1, 1, 4, D, generator=g, dtype=torch.float64)        # [batch, seq, heads, dim]
    ang = torch.rand(D // 2, generator=g, dtype=torch.float64) * 6.28
    sin_h, cos_h = torch.sin(ang)[None, None, :], torch.cos(ang)[None, None, :]       # HF repeats each entry twice itself
    want = gptj_rope(t, sin_h, cos_h)
    cos = torch.repeat_interleave(torch.cos(ang), 2)
    sin = torch.repeat_interleave(torch.sin(ang), 2)
    got = O.rope_pairs_gptj(t[0, 0], cos, sin)
    assert torch.allclose(got, want[0, 0], atol=1e-12, rtol=0)
    # a rotation of each pair: norms of the pairs are kept, angle 0 is the identity
    assert torch.allclose(got.reshape(4, D // 2, 2).norm(dim=-1), t[0, 0].reshape(4, D // 2, 2).norm(dim=-1), atol=1e-12)
    assert torch.equal(O.rope_pairs_gptj(t[0, 0], torch.ones(D, dtype=torch.float64), torch.zeros(D, dtype=torch.float64)), t[0, 0])


def test_llama_attention_plain_is_the_sglang_block_with_transposed_weights_and_gptj_pairs():
    """With zero angles both ops apply no rotation: the plain op on transposed weights must equal the (HF-pinned)
    sglang block without a residual; with angles, q and k of the plain op are the GPT-J rotation of the unrotated ones."""
    dims, S, w, x, res, k, v, cos, sin = _tiny_llama()
    H, D = dims.hidden, dims.head_dim
    wt = {"rms1": w["rms1"], "w_qkv_t": w["w_qkv"].reshape(3, H, H).transpose(1, 2).contiguous().reshape(3 * H, H),
          "w_o_t": w["w_o"].t().contiguous()}
    one, zero = torch.ones(1, D), torch.zeros(1, D)
    a = O.llama_attention_plain(x, wt, k, v, one, zero, dims, dtype=torch.float64, round_io=False)
    b = O.llama_attention_sglang(x, None, w, k, v, one, zero, dims, dtype=torch.float64, round_io=False)
    assert torch.allclose(a["output"], b["output"], atol=1e-12, rtol=0)
    assert torch.allclose(a["k_new"], b["k_new"], atol=1e-12, rtol=0) and torch.allclose(a["v_new"], b["v_new"], atol=1e-12, rtol=0)
    g = torch.Generator().manual_seed(9)
    ang = torch.rand(D // 2, generator=g, dtype=torch.float64) * 6.28
    c2, s2 = torch.repeat_interleave(torch.cos(ang), 2), torch.repeat_interleave(torch.sin(ang), 2)
    r = O.llama_attention_plain(x, wt, k, v, c2, s2, dims, dtype=torch.float64, round_io=False)
    assert torch.allclose(r["k_new"][0], O.rope_pairs_gptj(a["k_new"][0], c2, s2), atol=1e-12, rtol=0)
    assert torch.equal(r["v_new"], a["v_new"])
    # S = 0: the only key is the new token
    r0 = O.llama_attention_plain(x, wt, k[:0], v[:0], c2, s2, dims, dtype=torch.float64, round_io=False)
    assert torch.allclose(r0["attn_heads"], r0["v_new"][0], atol=1e-12, rtol=0)


# ---------------------------------------------------------------- the reference's own unit-test inputs
# (tests/test_pythia.py:24-42: an independent angle per rotary entry, so entries d and d + rot/2 of cos / sin differ)
@pytest.mark.parametrize("dims,zero_bo,pad", [(TINY, True, True), (NeoxDims(320, 4, 80, 20, 1280), True, True),
                                              (SMALL, False, False)])
def test_reference_recipe_inputs_against_hf_layer_and_brute_force(dims, zero_bo, pad):
    from oracle import hf_neox
    S = 7
    w, x, k, v, cos, sin = O.make_reference_unit_test_inputs(dims, seq_len=S, zero_bias_o=zero_bo, pad_rope_to_head_dim=pad)
    rot = dims.rotary_dim
    assert cos.numel() == (dims.head_dim if pad else rot) and k.shape == (S, dims.hidden)
    assert not torch.allclose(cos.reshape(-1)[: rot // 2], cos.reshape(-1)[rot // 2: rot])      # the halves do not repeat
    if pad:
        assert torch.equal(cos.reshape(-1)[rot:], torch.ones(dims.head_dim - rot)) and float(sin.reshape(-1)[rot:].abs().max()) == 0.0
    assert (float(w["b_o"].abs().max()) == 0.0) == zero_bo and w["ln_w"].shape == (1, dims.hidden)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims, dtype=torch.float64, round_io=False)
    wf = {n: t.reshape(-1) if n.startswith(("ln_", "post_ln_")) else t for n, t in w.items()}
    layer = hf_neox.build_hf_layer(dims, wf, dtype=torch.float64)
    out, k_new, v_new = hf_neox.hf_layer_decode(layer, x, k, v, cos, sin, S, dims, dtype=torch.float64)
    assert torch.allclose(r["output"], out, atol=1e-6, rtol=0)
    assert torch.allclose(r["k_new"], k_new, atol=1e-12, rtol=0) and torch.allclose(r["v_new"], v_new, atol=1e-12, rtol=0)
    if dims.hidden <= 64:
        bo, bk, bv = _brute_force_layer(x, wf, k, v, cos, sin, S, dims)
        assert torch.allclose(r["output"].reshape(-1), torch.tensor(bo, dtype=torch.float64), atol=1e-10)
        assert torch.allclose(r["k_new"].reshape(-1), torch.tensor(bk, dtype=torch.float64).reshape(-1), atol=1e-12)
    # a table whose second half is overwritten with the first gives a different rotation: the two conventions are
    # told apart by these inputs
    c2 = cos.clone().reshape(-1); c2[rot // 2: rot] = c2[: rot // 2]
    s2 = sin.clone().reshape(-1); s2[rot // 2: rot] = s2[: rot // 2]
    other = O.neox_layer_decode(x, w, k, v, c2, s2, S, dims, dtype=torch.float64, round_io=False)
    assert float((other["k_new"] - r["k_new"]).abs().max()) > 1e-3


def test_llama_attention_plain_rotates_q_as_well():
    """q of the plain op under non-zero angles: the attention output must be that of the GPT-J-rotated q against the
    returned (rotated) keys; an unrotated q gives a different result."""
    dims, S, w, x, res, k, v, cos, sin = _tiny_llama()
    H, D, nh = dims.hidden, dims.head_dim, dims.heads
    wt = {"rms1": w["rms1"], "w_qkv_t": w["w_qkv"].reshape(3, H, H).transpose(1, 2).contiguous().reshape(3 * H, H),
          "w_o_t": w["w_o"].t().contiguous()}
    g = torch.Generator().manual_seed(10)
    ang = torch.rand(D // 2, generator=g, dtype=torch.float64) * 6.28
    c2, s2 = torch.repeat_interleave(torch.cos(ang), 2), torch.repeat_interleave(torch.sin(ang), 2)
    r = O.llama_attention_plain(x, wt, k, v, c2, s2, dims, dtype=torch.float64, round_io=False)
    n1 = O.rms_norm(x.double().reshape(1, H), w["rms1"].double(), 1e-6)
    q_raw = (n1 @ wt["w_qkv_t"].double().reshape(3, H, H)[0]).reshape(nh, D)
    keys = torch.cat([k.double().reshape(S, nh, D), r["k_new"]], dim=0).permute(1, 0, 2)
    vals = torch.cat([v.double().reshape(S, nh, D), r["v_new"]], dim=0).permute(1, 0, 2)

    def heads(q):
        p = torch.softmax(torch.einsum("hd,hsd->hs", q, keys) / math.sqrt(D), dim=-1)
        return torch.einsum("hs,hsd->hd", p, vals)
    # HF's GPT-J rotation of q (third party), as test_rope_pairs_gptj_matches_hf_gptj_rotary uses it
    from transformers.models.gptj.modeling_gptj import apply_rotary_pos_emb as gptj_rope
    q_rot = gptj_rope(q_raw[None, None], s2[None, None, 0::2], c2[None, None, 0::2])[0, 0]
    assert torch.allclose(r["attn_heads"], heads(q_rot), atol=1e-12, rtol=0)
    assert float((r["attn_heads"] - heads(q_raw)).abs().max()) > 1e-4
