"""The C ABI called the way a non-torch host would: through ctypes with raw device pointers (`tensor.data_ptr()`),
no torch extension in between.  torch only owns the device memory and the stream."""
import ctypes
import os

import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import assert_close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Dims(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int32), ("heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
                ("rotary_dim", ctypes.c_int32), ("ffn", ctypes.c_int32), ("eps", ctypes.c_float)]


class Weights(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("ln_w", "ln_b", "w_qkv", "b_qkv", "w_o", "b_o", "post_ln_w", "post_ln_b",
                                                "w_up", "b_up", "w_down", "b_down")]


class Io(ctypes.Structure):
    _fields_ = [("input", ctypes.c_void_p), ("output", ctypes.c_void_p), ("k_new", ctypes.c_void_p), ("v_new", ctypes.c_void_p),
                ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p), ("cache_rows", ctypes.c_int32),
                ("cos", ctypes.c_void_p), ("sin", ctypes.c_void_p), ("rope_stride", ctypes.c_int32), ("seq_len", ctypes.c_int32),
                ("d_seq_len", ctypes.c_void_p), ("max_seq_len", ctypes.c_int32), ("attn_output", ctypes.c_void_p),
                ("mlp_intermediate", ctypes.c_void_p)]


@pytest.mark.parametrize("mode", [0, 1])
def test_layer_decode_through_ctypes(mode):
    lib = ctypes.CDLL(os.path.join(ROOT, "clusterfusionplus_amd", "libcfpp.so"))
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    lib.cfpp_neox_layer_decode.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                           ctypes.c_size_t, ctypes.c_void_p]
    dims, S = O.PYTHIA_2B8, 200
    print(f"\ncase ctypes cfpp_neox_layer_decode mode={mode} S={S}", flush=True)
    w = O.make_layer_weights(dims, layer=3)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S, capacity=S + 1, seed=17)
    dev = "cuda:0"
    wg = {n: t.to(dev) for n, t in w.items()}
    xg, kg, vg, cg, sg = (t.to(dev) for t in (x, k, v, cos, sin))
    out = torch.empty(1, dims.hidden, dtype=torch.float16, device=dev)
    k_new, v_new = torch.empty_like(out), torch.empty_like(out)
    d = Dims(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps)
    n = lib.cfpp_neox_workspace_bytes(ctypes.byref(d))
    ws = torch.zeros(n, dtype=torch.uint8, device=dev)           # torch allocations are 256-byte aligned
    assert ws.data_ptr() % 256 == 0
    cw = Weights(**{name: wg[name].data_ptr() for name, _ in Weights._fields_})
    io = Io(input=xg.data_ptr(), output=out.data_ptr(), k_new=k_new.data_ptr(), v_new=v_new.data_ptr(), k_cache=kg.data_ptr(),
            v_cache=vg.data_ptr(), cache_rows=S + 1, cos=cg.data_ptr(), sin=sg.data_ptr(), rope_stride=0, seq_len=S,
            d_seq_len=None, max_seq_len=0, attn_output=None, mlp_intermediate=None)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    ref = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims)
    assert_close("output", out, ref["output"])
    assert_close("k_new", k_new.reshape(1, dims.heads, dims.head_dim), ref["k_new"])
    assert_close("v_new", v_new.reshape(1, dims.heads, dims.head_dim), ref["v_new"])
    assert torch.equal(kg[S], k_new.reshape(-1)) and torch.equal(vg[S], v_new.reshape(-1))
    lib.cfpp_workspace_check.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    assert lib.cfpp_workspace_check(ctypes.byref(d), ws.data_ptr(), stream) == 0
    # a position-indexed table needs the position's row: seq_len == cache_rows is refused before any launch
    io.rope_stride, io.seq_len = dims.rotary_dim, S + 1
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream) == -3


@pytest.mark.parametrize("mode", [0, 1])
def test_device_seq_len_beyond_max_seq_len_is_flagged(mode):
    """`max_seq_len` sizes the launches when the length lives in device memory (in split mode: the grid of the attention
    items).  A device-side length beyond it, though still inside the caches, must not be attended with too small a grid:
    the kernels raise the sequence flag, append nothing, and the next call reports CFPP_ERR_DEVICE."""
    import clusterfusionplus_amd as pkg
    lib = ctypes.CDLL(os.path.join(ROOT, "clusterfusionplus_amd", "libcfpp.so"))
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    lib.cfpp_neox_layer_decode.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                           ctypes.c_size_t, ctypes.c_void_p]
    dims, rows, cap = O.PYTHIA_2B8, 400, 100
    print(f"\ncase device seq_len vs max_seq_len={cap}, cache rows {rows}, mode={mode}", flush=True)
    w = O.make_layer_weights(dims, layer=4)
    x, k, v, _, _ = O.make_layer_inputs(dims, rows - 1, capacity=rows, seed=21)
    dev = "cuda:0"
    wg = {n: t.to(dev) for n, t in w.items()}
    xg, kg, vg = (t.to(dev) for t in (x, k, v))
    cos_t, sin_t = pkg.rope_tables(rows, dims.rotary_dim, device=dev)
    out = torch.empty(1, dims.hidden, dtype=torch.float16, device=dev)
    k_new, v_new = torch.empty_like(out), torch.empty_like(out)
    d = Dims(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps)
    n = lib.cfpp_neox_workspace_bytes(ctypes.byref(d))
    ws = torch.zeros(n, dtype=torch.uint8, device=dev)
    cw = Weights(**{name: wg[name].data_ptr() for name, _ in Weights._fields_})
    seq = torch.tensor([cap], dtype=torch.int32, device=dev)
    io = Io(input=xg.data_ptr(), output=out.data_ptr(), k_new=k_new.data_ptr(), v_new=v_new.data_ptr(), k_cache=kg.data_ptr(),
            v_cache=vg.data_ptr(), cache_rows=rows, cos=cos_t.data_ptr(), sin=sin_t.data_ptr(), rope_stride=dims.rotary_dim, seq_len=0,
            d_seq_len=seq.data_ptr(), max_seq_len=cap, attn_output=None, mlp_intermediate=None)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.cfpp_device_status(1) == 0
    # at the bound: attended in full, equal to the oracle
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream) == 0
    torch.cuda.synchronize()
    assert lib.cfpp_device_status(0) == 0
    ref = O.neox_layer_decode(x, w, k, v, cos_t[cap:cap + 1].cpu(), sin_t[cap:cap + 1].cpu(), cap, dims)
    assert_close("output at max_seq_len", out, ref["output"])
    assert torch.equal(kg[cap], k_new.reshape(-1))
    # beyond it (rows would allow it): flagged, nothing appended
    k0 = kg.clone()
    seq.fill_(3 * cap)
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(kg, k0)
    assert lib.cfpp_device_status(0) & 2
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream) == -7
    assert lib.cfpp_device_status(1) & 2
    lib.cfpp_workspace_check.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    assert lib.cfpp_workspace_check(ctypes.byref(d), ws.data_ptr(), stream) == -7        # the workspace's own word, then zeroed
    assert lib.cfpp_workspace_check(ctypes.byref(d), ws.data_ptr(), stream) == 0
    assert lib.cfpp_device_status(0) == 0
