"""GPU parity of `llama_decoder_layer_sglang` (fused add + RMSNorm, QKV, whole-head RoPE, attention over every
cache row plus the new token, O projection) against the CPU oracle, through the C ABI entry
`cfpp_llama_attention_decode`.  Tolerance: fp16 I/O with fp32 accumulation, max-abs <= 2e-2 and cosine >= 0.9999."""
import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cf():
    import clusterfusion
    return clusterfusion


def run(cf, dims, S, seed, w_std=0.02, split=False):
    w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, S, seed=seed, w_std=w_std)
    ref = O.llama_attention_sglang(x, res, w, k, v, cos, sin, dims)
    dev = "cuda:0"
    res_g = res.to(dev)
    kg, vg = k.to(dev), v.to(dev)
    out, res_out, kn, vn = cf.llama_decoder_layer_sglang(x.to(dev), res_g, w["w_qkv"].to(dev), w["w_o"].to(dev), kg, vg,
                                                         w["rms1"].to(dev), dims.eps, cos.to(dev), sin.to(dev), dims.heads, split)
    torch.cuda.synchronize()
    return ref, out, res_out, res_g, kn, vn, (k, v, kg, vg)


@pytest.mark.parametrize("S", [4096, 2048, 129, 1, 0])
def test_llama2_7b_attention_matches_oracle(cf, S):
    print(f"\ncase llama2-7b attention S={S}", flush=True)
    dims = O.LLAMA2_7B
    ref, out, res_out, res_g, kn, vn, (k, v, kg, vg) = run(cf, dims, S, seed=S)
    assert_close("output", out, ref["output"])
    assert_close("k_new", kn, ref["k_new"])
    assert_close("v_new", vn, ref["v_new"])
    # the residual stream is updated in place with fp16(input + residual), bit for bit
    assert res_out.data_ptr() == res_g.data_ptr()
    assert torch.equal(res_g.cpu().float(), ref["residual"].float())
    # the caches are read only (the caller appends k_new / v_new)
    assert torch.equal(kg.cpu(), k) and torch.equal(vg.cpu(), v)


def test_small_geometry_and_determinism(cf):
    """hidden 1024, 8 heads of 128, odd cache length; two calls give identical bits."""
    print("\ncase llama attention hidden=1024", flush=True)
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    ref, out, _, _, kn, vn, _ = run(cf, dims, 333, seed=5, w_std=0.05)
    assert_close("output", out, ref["output"])
    assert_close("k_new", kn, ref["k_new"])
    _, out2, _, _, kn2, _, _ = run(cf, dims, 333, seed=5, w_std=0.05)
    assert torch.equal(out, out2) and torch.equal(kn, kn2)


@pytest.mark.parametrize("S", [1024, 0])
def test_one_launch_per_stage_gives_the_same_bits(cf, S):
    """mode = split (QKV rows, attention items, O rows as three launches; gate/up rows and down rows as two): what the
    library falls back to when a device cannot hold a one-launch grid.  Same results, bit for bit."""
    print(f"\ncase llama2-7b split launches S={S}", flush=True)
    dims = O.LLAMA2_7B
    ref, out, _, res_g, kn, vn, _ = run(cf, dims, S, seed=70 + S)
    _, out_s, _, res_s, kn_s, vn_s, _ = run(cf, dims, S, seed=70 + S, split=True)
    assert torch.equal(out, out_s) and torch.equal(kn, kn_s) and torch.equal(vn, vn_s) and torch.equal(res_g, res_s)
    assert_close("output", out_s, ref["output"])
    w = _full_layer_weights(dims, seed=6)
    g = torch.Generator().manual_seed(32)
    h = torch.randn(1, dims.hidden, generator=g).half()
    dev = "cuda:0"
    a = [h.to(dev), w["rms2"].to(dev), w["w_gate_up"].to(dev), w["w_down"].to(dev), dims.eps]
    one, two = cf.llama_mlp(*a), cf.llama_mlp(*a, split=True)
    torch.cuda.synchronize()
    assert torch.equal(one, two)
    assert_close("mlp output", two, O.llama_mlp(h, w, dims)["output"])


def test_argument_errors(cf):
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, 16, seed=1)
    dev = "cuda:0"
    a = [x.to(dev), res.to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev), k.to(dev), v.to(dev), w["rms1"].to(dev), 1e-6,
         cos.to(dev), sin.to(dev), 8]
    bad = list(a); bad[2] = a[2][:-1]
    with pytest.raises(RuntimeError, match="elements"):
        cf.llama_decoder_layer_sglang(*bad)
    bad = list(a); bad[4] = a[4][:8]
    with pytest.raises(RuntimeError, match="rows"):
        cf.llama_decoder_layer_sglang(*bad)
    bad = list(a); bad[8] = a[8].half()
    with pytest.raises(RuntimeError, match="float32"):
        cf.llama_decoder_layer_sglang(*bad)
    torch.cuda.synchronize()


def _full_layer_weights(dims, seed):
    w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, 0, seed=seed)
    g = torch.Generator().manual_seed(9000 + seed)
    w["rms2"] = (1 + 0.1 * torch.randn(dims.hidden, generator=g)).half()
    w["w_gate_up"] = (0.02 * torch.randn(2 * dims.ffn, dims.hidden, generator=g)).half()
    w["w_down"] = (0.02 * torch.randn(dims.hidden, dims.ffn, generator=g)).half()
    return w


@pytest.mark.parametrize("hidden,ffn", [(4096, 11008), (1024, 2816)])
def test_llama_mlp_matches_oracle(cf, hidden, ffn):
    """output = h + W_down (silu(Wg n) * (Wu n)); ffn 11008 leaves a half-filled last 512-column chunk."""
    print(f"\ncase llama mlp hidden={hidden} ffn={ffn}", flush=True)
    dims = O.LlamaDims(hidden=hidden, heads=hidden // 128, head_dim=128, ffn=ffn)
    w = _full_layer_weights(dims, seed=3)
    g = torch.Generator().manual_seed(31)
    h = torch.randn(1, hidden, generator=g).half()
    ref = O.llama_mlp(h, w, dims)
    dev = "cuda:0"
    out = cf.llama_mlp(h.to(dev), w["rms2"].to(dev), w["w_gate_up"].to(dev), w["w_down"].to(dev), dims.eps)
    torch.cuda.synchronize()
    assert_close("output", out, ref["output"])
    # linearity in W_down: doubling it doubles the MLP term (output - h)
    out2 = cf.llama_mlp(h.to(dev), w["rms2"].to(dev), w["w_gate_up"].to(dev), (w["w_down"].float() * 2).half().to(dev), dims.eps)
    torch.cuda.synchronize()
    d1, d2 = out.cpu().float() - h.float(), out2.cpu().float() - h.float()
    assert float((d2 - 2 * d1).abs().max()) <= 2e-2


@pytest.mark.parametrize("S", [4096, 77])
def test_llama2_7b_full_layer_matches_oracle(cf, S):
    print(f"\ncase llama2-7b full layer S={S}", flush=True)
    dims = O.LLAMA2_7B
    w = _full_layer_weights(dims, seed=4)
    _, x, _, k, v, cos, sin = O.make_llama_attn_inputs(dims, S, seed=40 + S)
    ref = O.llama_layer_decode(x, w, k, v, cos, sin, S, dims)
    dev = "cuda:0"
    out, kn, vn = cf.llama_decoder_layer_full(x.to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev), k.to(dev), v.to(dev),
                                              w["rms1"].to(dev), w["rms2"].to(dev), w["w_gate_up"].to(dev), w["w_down"].to(dev),
                                              dims.eps, cos.to(dev), sin.to(dev), dims.heads)
    torch.cuda.synchronize()
    assert_close("output", out, ref["output"])
    assert_close("k_new", kn, ref["k_new"])
    assert_close("v_new", vn, ref["v_new"])
