"""cfpp_neox_layer_decode_static, the layer step that allocates nothing (its scratch is an array inside the library),
called through the C ABI with raw device pointers and compared, bit for bit, with cfpp_neox_layer_decode on a
caller-provided workspace: two calls in a row, the second on a smaller geometry and a shorter context, so that the
second call finds the first one's contents in the shared array."""
import ctypes
import os

import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import assert_close
from tests.test_gpu_ctypes_boundary import Dims, Io, Weights

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def _lib():
    lib = ctypes.CDLL(os.path.join(ROOT, "clusterfusionplus_amd", "libcfpp.so"))
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    lib.cfpp_static_scratch_bytes.restype = ctypes.c_size_t
    lib.cfpp_neox_layer_decode.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                           ctypes.c_size_t, ctypes.c_void_p]
    lib.cfpp_neox_layer_decode_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    return lib


def _case(dims, S, seed):
    w = O.make_layer_weights(dims, layer=seed)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S, capacity=S + 1, seed=seed)
    wg = {n: t.to(DEV) for n, t in w.items()}
    return w, (x, k, v, cos, sin), wg, [t.to(DEV) for t in (x, cos, sin)]


def _call(lib, dims, wg, xg, cg, sg, k, v, S, mode, static):
    kg, vg = k.to(DEV), v.to(DEV)
    out = torch.empty(1, dims.hidden, dtype=torch.float16, device=DEV)
    k_new, v_new = torch.empty_like(out), torch.empty_like(out)
    d = Dims(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps)
    cw = Weights(**{name: wg[name].data_ptr() for name, _ in Weights._fields_})
    io = Io(input=xg.data_ptr(), output=out.data_ptr(), k_new=k_new.data_ptr(), v_new=v_new.data_ptr(), k_cache=kg.data_ptr(),
            v_cache=vg.data_ptr(), cache_rows=S + 1, cos=cg.data_ptr(), sin=sg.data_ptr(), rope_stride=0, seq_len=S,
            d_seq_len=None, max_seq_len=0, attn_output=None, mlp_intermediate=None)
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        rc = lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, stream)
    else:
        n = lib.cfpp_neox_workspace_bytes(ctypes.byref(d))
        ws = torch.zeros(n, dtype=torch.uint8, device=DEV)
        rc = lib.cfpp_neox_layer_decode(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, ws.data_ptr(), n, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return out, k_new, v_new, kg, vg


@pytest.mark.parametrize("mode", [0, 1])
def test_static_entry_point_equals_the_workspace_one(mode):
    lib = _lib()
    assert lib.cfpp_init() == 0
    big = (O.PYTHIA_6B9, 300, 51)
    small = (O.PYTHIA_2B8, 100, 52)
    assert lib.cfpp_static_scratch_bytes() >= lib.cfpp_neox_workspace_bytes(ctypes.byref(Dims(4096, 32, 128, 32, 16384, 1e-5)))
    for dims, S, seed in (big, small, big):              # the second call is the smaller one; then back again
        print(f"\ncase static scratch mode={mode} hidden={dims.hidden} S={S}", flush=True)
        w, (x, k, v, cos, sin), wg, (xg, cg, sg) = _case(dims, S, seed)
        want = _call(lib, dims, wg, xg, cg, sg, k, v, S, mode, static=False)
        got = _call(lib, dims, wg, xg, cg, sg, k, v, S, mode, static=True)
        for name, a, b in zip(("output", "k_new", "v_new", "k_cache", "v_cache"), got, want):
            assert torch.equal(a, b), name
        ref = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims)
        assert_close("output vs oracle", got[0], ref["output"])
        assert torch.equal(got[3][S], got[1].reshape(-1))
    # a geometry whose scratch would not fit the array is refused before anything is launched
    wide = Dims(4096, 512, 8, 8, 16384, 1e-5)
    assert lib.cfpp_neox_workspace_bytes(ctypes.byref(wide)) > lib.cfpp_static_scratch_bytes()
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(wide), None, None, mode, None) == -10
    assert lib.cfpp_device_status(0) == 0
