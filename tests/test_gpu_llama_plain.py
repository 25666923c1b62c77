"""GPU parity of the plain `llama_decoder_layer` op (RMSNorm, q/k/v products with weights stored [in, out], GPT-J
rotary pairs, attention over every cache row plus the new token, O product; no residual, caches read only) against the
CPU oracle, through the C ABI entry `cfpp_llama_attention_plain`.  Tolerance: fp16 I/O with fp32 accumulation,
max-abs <= 2e-2 and cosine >= 0.9999."""
import math

import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cf():
    import clusterfusion
    return clusterfusion


def make(dims, S, seed, w_std=0.02):
    return O.make_llama_plain_inputs(dims, S, seed=seed, w_std=w_std)


def run(cf, dims, S, seed, **kw):
    w, x, k, v, cos, sin = make(dims, S, seed, **kw)
    ref = O.llama_attention_plain(x, w, k, v, cos, sin, dims)
    dev = "cuda:0"
    kg, vg = k.to(dev), v.to(dev)
    out, kn, vn = cf.llama_decoder_layer(x.to(dev), w["w_qkv_t"].to(dev), w["w_o_t"].to(dev), kg, vg, w["rms1"].to(dev),
                                         cos.to(dev), sin.to(dev), num_heads=dims.heads)
    torch.cuda.synchronize()
    assert torch.equal(kg.cpu(), k) and torch.equal(vg.cpu(), v)       # the caches are read only
    return ref, out, kn, vn


@pytest.mark.parametrize("S", [4096, 1000, 1, 0])
def test_llama2_7b_plain_op_matches_oracle(cf, S):
    print(f"\ncase llama2-7b plain op S={S}", flush=True)
    ref, out, kn, vn = run(cf, O.LLAMA2_7B, S, seed=S)
    assert_close("output", out, ref["output"])
    assert_close("k_new", kn, ref["k_new"])
    assert_close("v_new", vn, ref["v_new"])


def test_small_geometry_and_repeatable(cf):
    print("\ncase llama plain op hidden=1024", flush=True)
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    ref, out, kn, vn = run(cf, dims, 200, seed=3, w_std=0.05)
    assert_close("output", out, ref["output"])
    assert_close("k_new", kn, ref["k_new"])
    _, out2, kn2, _ = run(cf, dims, 200, seed=3, w_std=0.05)
    assert torch.equal(out, out2) and torch.equal(kn, kn2)             # fixed summation order


def test_argument_errors(cf):
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    w, x, k, v, cos, sin = make(dims, 16, seed=1)
    dev = "cuda:0"
    a = [x.to(dev), w["w_qkv_t"].to(dev), w["w_o_t"].to(dev), k.to(dev), v.to(dev), w["rms1"].to(dev), cos.to(dev), sin.to(dev)]
    with pytest.raises(RuntimeError):       # tables with one entry per pair only
        cf.llama_decoder_layer(*(a[:6] + [cos[:, :64].contiguous().to(dev), sin[:, :64].contiguous().to(dev)]), num_heads=8)
    with pytest.raises(RuntimeError):       # weight of the wrong size
        cf.llama_decoder_layer(*(a[:1] + [a[2]] + a[2:]), num_heads=8)
    with pytest.raises(RuntimeError):       # hidden size not divisible by the head count
        cf.llama_decoder_layer(*a, num_heads=7)
    cf.llama_decoder_layer(*a, num_heads=8)
    torch.cuda.synchronize()
