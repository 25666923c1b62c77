"""GPU parity of the decoder-layer ops against the CPU oracle on identical seeded inputs.

Tolerance (fp16 I/O, fp32 accumulation): max-abs <= 2e-2 and cosine >= 0.9999 on the layer output
and on the new K / V rows; integer-like facts (cache row == returned row, untouched rows, determinism,
split == fused) are bit-exact."""
import pytest
import torch

from oracle import neox_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MIN_COS = 0.9999

MODELS = {"pythia_2b8": O.PYTHIA_2B8, "pythia_6b9": O.PYTHIA_6B9}


def _cos(a, b):
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    return float((a @ b) / (a.norm() * b.norm() + 1e-30))


def assert_close(name, got, want, max_abs=MAX_ABS):
    got, want = got.detach().cpu().float(), want.detach().cpu().float()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    err = float((got - want).abs().max())
    cs = _cos(got, want)
    print(f"  {name}: max-abs {err:.3e} cosine {cs:.7f}", flush=True)
    assert err <= max_abs, f"{name}: max-abs {err} > {max_abs}"
    assert cs >= MIN_COS, f"{name}: cosine {cs} < {MIN_COS}"


def layer_args(w, x, k, v, cos, sin, with_down=True):
    a = [x, w["w_qkv"], w["b_qkv"], w["w_o"], w["b_o"], k, v, w["ln_w"], w["ln_b"], cos, sin,
         w["post_ln_w"], w["post_ln_b"], w["w_up"], w["b_up"]]
    if with_down:
        a += [w["w_down"], w["b_down"]]
    return a


def make(model, S, capacity=None, seed=0, layer=0):
    dims = MODELS[model]
    w = O.make_layer_weights(dims, layer=layer)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S, capacity=capacity, seed=seed)
    dev = "cuda:0"
    wg = {n: t.to(dev) for n, t in w.items()}
    return dims, w, (x, k, v, cos, sin), wg, tuple(t.to(dev) for t in (x, k, v, cos, sin))


@pytest.fixture(scope="module")
def cf():
    import clusterfusion
    return clusterfusion


@pytest.mark.parametrize("model,S", [("pythia_2b8", 512), ("pythia_6b9", 2048), ("pythia_2b8", 129),
                                     ("pythia_6b9", 129), ("pythia_2b8", 0), ("pythia_6b9", 1),
                                     ("pythia_2b8", 63), ("pythia_6b9", 4097), ("pythia_6b9", 16384),
                                     ("pythia_2b8", 4096),
                                     # either side of the length up to which the fused kernel deals 80-dim heads out per chiplet
                                     ("pythia_2b8", 1228), ("pythia_2b8", 1229)])
@pytest.mark.parametrize("variant", ["decoder_layer_split", "decoder_layer"])
def test_layer_matches_oracle(cf, model, S, variant):
    print(f"\ncase {model} {variant} S={S}", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=S)
    x, k, v, cos, sin = gpu
    k0, v0 = k.clone(), v.clone()
    op = getattr(cf, f"{model}_{variant}")
    out, k_new, v_new = op(*layer_args(wg, x, k, v, cos, sin), S)
    torch.cuda.synchronize()
    assert cf.check_workspace(x, dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn) == 0
    ref = O.neox_layer_decode(*cpu[:1], w, *cpu[1:], S, dims)
    assert out.shape == (1, dims.hidden) and k_new.shape == (1, dims.heads, dims.head_dim) == v_new.shape
    assert_close("output", out, ref["output"])
    assert_close("k_new", k_new, ref["k_new"])
    assert_close("v_new", v_new, ref["v_new"])
    # the cache row is the returned row, bit for bit; every other row is untouched
    assert torch.equal(k[S], k_new.reshape(-1)) and torch.equal(v[S], v_new.reshape(-1))
    keep = torch.arange(k.shape[0], device=k.device) != S
    assert torch.equal(k[keep], k0[keep]) and torch.equal(v[keep], v0[keep])


@pytest.mark.parametrize("model,S", [("pythia_2b8", 300), ("pythia_6b9", 700)])
def test_split_equals_fused_and_is_deterministic(cf, model, S):
    print(f"\ncase {model} split-vs-fused S={S}", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=11)
    x, k, v, cos, sin = gpu
    outs = []
    for variant in ("decoder_layer", "decoder_layer_split", "decoder_layer", "decoder_layer_split"):
        kk, vv = k.clone(), v.clone()
        o, kn, vn = getattr(cf, f"{model}_{variant}")(*layer_args(wg, x, kk, vv, cos, sin), S)
        outs.append((o.clone(), kn.clone(), vn.clone(), kk, vv))
    torch.cuda.synchronize()
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)


@pytest.mark.parametrize("model", ["pythia_2b8", "pythia_6b9"])
def test_attention_only_then_mlp_only(cf, model):
    S = 200
    print(f"\ncase {model} attention_only/mlp_only S={S}", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=5)
    x, k, v, cos, sin = gpu
    attn, inter, k_new, v_new = getattr(cf, f"{model}_attention_only")(*layer_args(wg, x, k, v, cos, sin, False), S)
    out = getattr(cf, f"{model}_mlp_only")(x, attn, inter, wg["w_down"], wg["b_down"])
    torch.cuda.synchronize()
    ref = O.neox_layer_decode(*cpu[:1], w, *cpu[1:], S, dims)
    assert attn.shape == (1, dims.hidden) and inter.shape == (dims.ffn,)
    assert_close("attn_output", attn, ref["attn_output"])
    assert_close("mlp_intermediate", inter, ref["mlp_intermediate"])
    assert_close("output", out, ref["output"])
    assert_close("k_new", k_new, ref["k_new"])
    assert torch.equal(k[S], k_new.reshape(-1)) and torch.equal(v[S], v_new.reshape(-1))


def test_cache_with_exactly_seq_len_rows_skips_the_append(cf):
    model, S = "pythia_2b8", 129
    print(f"\ncase {model} capacity == S", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, capacity=S, seed=2)
    x, k, v, cos, sin = gpu
    k0, v0 = k.clone(), v.clone()
    out, k_new, v_new = cf.pythia_2b8_decoder_layer(*layer_args(wg, x, k, v, cos, sin), S)
    torch.cuda.synchronize()
    ref = O.neox_layer_decode(*cpu[:1], w, *cpu[1:], S, dims)
    assert_close("output", out, ref["output"])
    assert_close("k_new", k_new, ref["k_new"])
    assert torch.equal(k, k0) and torch.equal(v, v0)


def test_ln_tensors_may_be_2d_and_rope_padded(cf):
    # the reference's 2.8B scripts pass LN tensors as [1,H] and cos/sin padded to [1,D]
    # (tests/test_pythia.py:25-42,203-208); only the element count matters
    model, S = "pythia_2b8", 77
    print(f"\ncase {model} [1,H] LN + padded rope", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=3)
    x, k, v, cos, sin = gpu
    pad = dims.head_dim - dims.rotary_dim
    cos_p = torch.cat([cos, torch.ones(1, pad, device=cos.device)], dim=-1).contiguous()
    sin_p = torch.cat([sin, torch.zeros(1, pad, device=cos.device)], dim=-1).contiguous()
    wg2 = dict(wg)
    for n in ("ln_w", "ln_b", "post_ln_w", "post_ln_b"):
        wg2[n] = wg[n].reshape(1, -1)
    a, _, _ = cf.pythia_2b8_decoder_layer(*layer_args(wg, x, k.clone(), v.clone(), cos, sin), S)
    b, _, _ = cf.pythia_2b8_decoder_layer(*layer_args(wg2, x, k.clone(), v.clone(), cos_p, sin_p), S)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_zero_weights_return_the_input_bit_exact(cf):
    model, S = "pythia_6b9", 40
    print(f"\ncase {model} zero weights", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=4)
    x, k, v, cos, sin = gpu
    z = {n: (t if n in ("ln_w", "post_ln_w") else torch.zeros_like(t)) for n, t in wg.items()}
    out, k_new, v_new = cf.pythia_6b9_decoder_layer(*layer_args(z, x, k, v, cos, sin), S)
    torch.cuda.synchronize()
    assert torch.equal(out, x)
    assert float(k_new.abs().max()) == 0.0 and float(v_new.abs().max()) == 0.0
