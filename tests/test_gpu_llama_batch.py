"""GPU parity of `llama_decoder_layer_batch_decode_sglang` (a batch of sequences over paged caches: fused add +
RMSNorm, QKV, whole-head RoPE from cos_sin[position], new K/V row into the page table's last slot, attention over
the sequence's pages plus the new token, O projection) against the CPU oracle, through the C ABI entry
`cfpp_llama_batch_decode`.  Tolerance: fp16 I/O with fp32 accumulation, max-abs <= 2e-2 and cosine >= 0.9999."""
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


def make_case(dims, lens, seed, max_pos=512, w_std=0.02, layers=3, layer_id=1):
    """Sequences of `lens` cached tokens each; their pages are scattered over a shared pool of cache rows."""
    return O.make_llama_batch_inputs(dims, lens, seed=seed, max_pos=max_pos, w_std=w_std, layers=layers) + (layer_id,)


def run(cf, dims, lens, seed, **kw):
    w, x, res, indptr, indices, caches, positions, cos_sin, layer_id = make_case(dims, lens, seed, **kw)
    k, v = caches[layer_id]
    ref = O.llama_batch_decode_paged(x, res, w, indptr, indices, k, v, positions, cos_sin, dims)
    dev = "cuda:0"
    gc = [(a.to(dev), b.to(dev)) for a, b in caches]
    kptr = torch.tensor([a.data_ptr() for a, _ in gc], dtype=torch.uint64, device=dev)
    vptr = torch.tensor([b.data_ptr() for _, b in gc], dtype=torch.uint64, device=dev)
    out = torch.full_like(x, float("nan"), device=dev)
    res_out = torch.full_like(x, float("nan"), device=dev)
    xg, rg = x.to(dev), res.to(dev)
    ret = cf.llama_decoder_layer_batch_decode_sglang(out, res_out, xg, rg, w["w_qkv"].to(dev), w["w_o"].to(dev), indptr.to(dev),
                                                     indices.to(dev), kptr, vptr, layer_id, w["rms1"].to(dev), dims.eps,
                                                     positions.to(dev), cos_sin.to(dev))
    torch.cuda.synchronize()
    assert ret is None
    # inputs are read only
    assert torch.equal(xg.cpu(), x) and torch.equal(rg.cpu(), res)
    return ref, out, res_out, gc, caches, indptr, indices, layer_id


def check(ref, out, res_out, gc, caches, indptr, indices, layer_id):
    assert_close("output", out, ref["output"])
    assert torch.equal(res_out.cpu().float(), ref["residual"].float())      # fp16(input + residual), bit for bit
    B = indptr.numel() - 1
    slots = [int(indices[int(indptr[b + 1]) - 1]) for b in range(B)]
    for li, ((kg, vg), (k, v)) in enumerate(zip(gc, caches)):
        kc, vc = kg.cpu(), vg.cpu()
        if li != layer_id:
            assert torch.equal(kc, k) and torch.equal(vc, v), "a cache of another layer was touched"
            continue
        keep = torch.ones(k.shape[0], dtype=torch.bool)
        keep[slots] = False
        assert torch.equal(kc[keep], k[keep]) and torch.equal(vc[keep], v[keep]), "a row other than the new tokens' was written"
        assert_close("new k rows", kc[slots], ref["k_cache"][slots])
        assert_close("new v rows", vc[slots], ref["v_cache"][slots])


@pytest.mark.parametrize("lens", [[1024], [700, 3, 0, 129], [64] * 8, [2048, 1, 333, 17, 900, 5, 64, 1500, 31], [40] * 19,
                                  [0, 5, 1024, 33] * 4, [1, 0] * 16])
def test_llama2_7b_batch_matches_oracle(cf, lens):
    print(f"\ncase llama2-7b paged batch lens={lens}", flush=True)
    r = run(cf, O.LLAMA2_7B, lens, seed=len(lens), max_pos=4096)
    check(*r)


def test_small_geometry_repeatable_and_page_order(cf):
    """hidden 1024, 8 heads of 128; two calls give identical bits."""
    print("\ncase llama paged batch hidden=1024", flush=True)
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    r1 = run(cf, dims, [77, 5, 300], seed=4, w_std=0.05)
    check(*r1)
    r2 = run(cf, dims, [77, 5, 300], seed=4, w_std=0.05)
    assert torch.equal(r1[1], r2[1])


@pytest.mark.parametrize("lens", [[200, 0, 33, 1, 90], [17] * 20, [300] * 16])
def test_hidden_2048_geometry(cf, lens):
    """hidden 2048, 16 heads of 128: the four-wave instantiation of the pipelined row kernel; up to 16 sequences with the
    norm inside the QKV launch and the heads merged inside a workgroup, more than 16 with the norm as a launch of its own."""
    print(f"\ncase llama paged batch hidden=2048 lens={lens}", flush=True)
    dims = O.LlamaDims(hidden=2048, heads=16, head_dim=128, ffn=0)
    check(*run(cf, dims, lens, seed=7 + len(lens), w_std=0.03))


def test_batch_of_one_equals_single_sequence_op(cf):
    """With an identity page table the batched op and `llama_decoder_layer_sglang` see the same problem."""
    print("\ncase paged batch of one vs single-sequence op", flush=True)
    dims = O.LLAMA2_7B
    S, dev = 513, "cuda:0"
    w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, S, seed=11)
    D = dims.head_dim
    cos_sin = torch.cat([cos[:, : D // 2], sin[:, : D // 2]], dim=-1).contiguous()          # one position
    out1, _, kn, vn = cf.llama_decoder_layer_sglang(x.to(dev), res.clone().to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev), k.to(dev),
                                                    v.to(dev), w["rms1"].to(dev), dims.eps, cos.to(dev), sin.to(dev), dims.heads)
    kg = torch.cat([k, torch.zeros(1, dims.hidden, dtype=k.dtype)]).to(dev)
    vg = torch.cat([v, torch.zeros(1, dims.hidden, dtype=v.dtype)]).to(dev)
    out = torch.empty_like(x, device=dev)
    res_out = torch.empty_like(x, device=dev)
    cf.llama_decoder_layer_batch_decode_sglang(
        out, res_out, x.to(dev), res.to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev),
        torch.tensor([0, S + 1], dtype=torch.int32, device=dev), torch.arange(S + 1, dtype=torch.int32, device=dev),
        torch.tensor([kg.data_ptr()], dtype=torch.uint64, device=dev), torch.tensor([vg.data_ptr()], dtype=torch.uint64, device=dev),
        0, w["rms1"].to(dev), dims.eps, torch.zeros(1, dtype=torch.int64, device=dev), cos_sin.to(dev))
    torch.cuda.synchronize()
    # (different kernels, different summation order: close, not bit-equal)
    assert_close("k row", kg[S], kn.reshape(-1).cpu())
    assert_close("v row", vg[S], vn.reshape(-1).cpu())
    assert_close("output", out, out1.cpu())


def test_argument_errors(cf):
    dims = O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0)
    w, x, res, indptr, indices, caches, positions, cos_sin, layer_id = make_case(dims, [5, 9], seed=2)
    dev = "cuda:0"
    gc = [(a.to(dev), b.to(dev)) for a, b in caches]
    kptr = torch.tensor([a.data_ptr() for a, _ in gc], dtype=torch.uint64, device=dev)
    vptr = torch.tensor([b.data_ptr() for _, b in gc], dtype=torch.uint64, device=dev)
    xg, rg = x.to(dev), res.to(dev)
    out, res_out = torch.empty_like(xg), torch.empty_like(xg)
    args = [out, res_out, xg, rg, w["w_qkv"].to(dev), w["w_o"].to(dev), indptr.to(dev), indices.to(dev), kptr, vptr, layer_id,
            w["rms1"].to(dev), dims.eps, positions.to(dev), cos_sin.to(dev)]
    with pytest.raises(RuntimeError):      # the sum would be written while it is still being read
        cf.llama_decoder_layer_batch_decode_sglang(*(args[:1] + [rg] + args[2:]))
    with pytest.raises(RuntimeError):      # float16 positions
        cf.llama_decoder_layer_batch_decode_sglang(*(args[:13] + [positions.half().to(dev)] + args[14:]))
    with pytest.raises(RuntimeError):      # layer_id outside the pointer tables
        cf.llama_decoder_layer_batch_decode_sglang(*(args[:10] + [7] + args[11:]))
    with pytest.raises(RuntimeError):      # indptr on the host
        cf.llama_decoder_layer_batch_decode_sglang(*(args[:6] + [indptr] + args[7:]))
    cf.llama_decoder_layer_batch_decode_sglang(*args)
    torch.cuda.synchronize()
