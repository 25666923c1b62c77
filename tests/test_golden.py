"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the pinned oracle):
the oracle must keep reproducing them on the CPU, and the HIP path must match them on the GPU."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle import neox_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
G = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(G)


def load(name):
    return {k: torch.from_numpy(v) for k, v in np.load(os.path.join(HERE, "golden", name + ".npz")).items()}


@pytest.mark.parametrize("name", ["neox_h512_s37", "pythia_2b8_s512"])
def test_oracle_reproduces_golden(name):
    dims, S, w, x, k, v, cos, sin = G.inputs(name)
    want = load(name)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims, dtype=torch.float32)
    for n in ("output", "k_new", "v_new", "attn_output", "mlp_intermediate"):
        # fp32 vs the fp64 run that wrote the fixture: a flipped fp16 rounding is one ulp at most
        assert float((r[n].float() - want[n]).abs().max()) <= 8e-3, n
        assert float((r[n].float() - want[n]).abs().mean()) <= 1e-4, n


@pytest.mark.parametrize("name", ["pythia_2b8_reference_recipe_s129"])
def test_oracle_reproduces_reference_recipe_golden(name):
    dims, w, x, k, v, cos, sin = G.reference_recipe_inputs(name)
    want = load(name)
    r = O.neox_layer_decode(x, w, k, v, cos, sin, 129, dims, dtype=torch.float32)
    for n in ("output", "k_new", "v_new"):
        # these inputs give outputs of magnitude ~10 (every tensor N(0, 0.1), LayerNorm weights included): one fp16
        # ulp there is 8e-3
        assert float((r[n].float() - want[n]).abs().max()) <= 1.6e-2, n
        assert float((r[n].float() - want[n]).abs().mean()) <= 2e-4, n


@pytest.mark.gpu
@pytest.mark.parametrize("name,op", [("neox_h512_s37", None), ("pythia_2b8_s512", "pythia_2b8_decoder_layer"),
                                     ("pythia_6b9_s2048", "pythia_6b9_decoder_layer"),
                                     ("pythia_2b8_s512", "pythia_2b8_decoder_layer_split")])
def test_hip_matches_golden(name, op):
    import clusterfusion as cf
    from tests.test_gpu_layer_parity import assert_close, layer_args
    print(f"\ncase golden {name} {op}", flush=True)
    dims, S, w, x, k, v, cos, sin = G.inputs(name)
    dev = "cuda:0"
    wg = {n: t.to(dev) for n, t in w.items()}
    a = layer_args(wg, x.to(dev), k.to(dev), v.to(dev), cos.to(dev), sin.to(dev))
    if op is None:     # a small Pythia-70M-like geometry through the generic op, fused and split
        outs = []
        for split in (False, True):
            a = layer_args(wg, x.to(dev), k.to(dev), v.to(dev), cos.to(dev), sin.to(dev))
            outs.append(cf.neox_decoder_layer(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps,
                                              split, *a, S))
        torch.cuda.synchronize()
        assert all(torch.equal(p, q) for p, q in zip(outs[0], outs[1]))
        out, k_new, v_new = outs[0]
    else:
        out, k_new, v_new = getattr(cf, op)(*a, S)
        torch.cuda.synchronize()
    want = load(name)
    assert_close("output", out, want["output"])
    assert_close("k_new", k_new, want["k_new"])
    assert_close("v_new", v_new, want["v_new"])


@pytest.mark.parametrize("name", ["llama_h1024_s333"])
def test_oracle_reproduces_llama_golden(name):
    dims, w, x, res, k, v, cos, sin = G.llama_inputs(name)
    want = load(name)
    r = O.llama_attention_sglang(x, res, w, k, v, cos, sin, dims, dtype=torch.float32)
    assert torch.equal(r["residual"].float(), want["residual"])
    for n in ("output", "k_new", "v_new"):
        assert float((r[n].float() - want[n]).abs().max()) <= 8e-3, n
        assert float((r[n].float() - want[n]).abs().mean()) <= 1e-4, n


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["llama_h1024_s333", "llama2_7b_s1024"])
def test_hip_matches_llama_golden(name):
    import clusterfusion as cf
    from tests.test_gpu_layer_parity import assert_close
    print(f"\ncase golden {name}", flush=True)
    dims, w, x, res, k, v, cos, sin = G.llama_inputs(name)
    dev = "cuda:0"
    res_g = res.to(dev)
    out, _, k_new, v_new = cf.llama_decoder_layer_sglang(x.to(dev), res_g, w["w_qkv"].to(dev), w["w_o"].to(dev), k.to(dev), v.to(dev),
                                                         w["rms1"].to(dev), dims.eps, cos.to(dev), sin.to(dev), dims.heads)
    torch.cuda.synchronize()
    want = load(name)
    assert_close("output", out, want["output"])
    assert_close("k_new", k_new, want["k_new"])
    assert_close("v_new", v_new, want["v_new"])
    assert torch.equal(res_g.cpu().float().reshape(-1), want["residual"].reshape(-1))


def test_oracle_reproduces_llama_plain_and_batch_golden():
    dims, w, x, k, v, cos, sin = G.llama_plain_inputs("llama_plain_h1024_s200")
    want = load("llama_plain_h1024_s200")
    r = O.llama_attention_plain(x, w, k, v, cos, sin, dims, dtype=torch.float32)
    for n in ("output", "k_new", "v_new"):
        assert float((r[n].float() - want[n]).abs().max()) <= 8e-3, n
        assert float((r[n].float() - want[n]).abs().mean()) <= 1e-4, n
    dims, layer_id, w, x, res, indptr, indices, caches, positions, cos_sin = G.llama_batch_inputs("llama_batch_h1024")
    want = load("llama_batch_h1024")
    r = O.llama_batch_decode_paged(x, res, w, indptr, indices, caches[layer_id][0], caches[layer_id][1], positions, cos_sin, dims)
    rows = G.new_rows(indptr, indices)
    assert torch.equal(r["residual"].float(), want["residual"])
    for got, n in ((r["output"], "output"), (r["k_cache"][rows], "k_rows"), (r["v_cache"][rows], "v_rows")):
        assert float((got.float() - want[n]).abs().max()) <= 8e-3, n
        assert float((got.float() - want[n]).abs().mean()) <= 1e-4, n


@pytest.mark.gpu
def test_hip_matches_llama_plain_and_batch_golden():
    import clusterfusion as cf
    from tests.test_gpu_layer_parity import assert_close
    print("\ncase golden llama_plain_h1024_s200 / llama_batch_h1024", flush=True)
    dev = "cuda:0"
    dims, w, x, k, v, cos, sin = G.llama_plain_inputs("llama_plain_h1024_s200")
    out, kn, vn = cf.llama_decoder_layer(x.to(dev), w["w_qkv_t"].to(dev), w["w_o_t"].to(dev), k.to(dev), v.to(dev), w["rms1"].to(dev),
                                         cos.to(dev), sin.to(dev), num_heads=dims.heads)
    torch.cuda.synchronize()
    want = load("llama_plain_h1024_s200")
    assert_close("output", out, want["output"])
    assert_close("k_new", kn, want["k_new"])
    assert_close("v_new", vn, want["v_new"])
    dims, layer_id, w, x, res, indptr, indices, caches, positions, cos_sin = G.llama_batch_inputs("llama_batch_h1024")
    gc = [(a.to(dev), b.to(dev)) for a, b in caches]
    kptr = torch.tensor([a.data_ptr() for a, _ in gc], dtype=torch.uint64, device=dev)
    vptr = torch.tensor([b.data_ptr() for _, b in gc], dtype=torch.uint64, device=dev)
    out, res_out = torch.empty_like(x, device=dev), torch.empty_like(x, device=dev)
    cf.llama_decoder_layer_batch_decode_sglang(out, res_out, x.to(dev), res.to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev), indptr.to(dev),
                                               indices.to(dev), kptr, vptr, layer_id, w["rms1"].to(dev), dims.eps, positions.to(dev),
                                               cos_sin.to(dev))
    torch.cuda.synchronize()
    want = load("llama_batch_h1024")
    rows = G.new_rows(indptr, indices)
    assert_close("output", out, want["output"])
    assert torch.equal(res_out.cpu().float(), want["residual"])
    assert_close("k rows", gc[layer_id][0][rows], want["k_rows"])
    assert_close("v rows", gc[layer_id][1][rows], want["v_rows"])
