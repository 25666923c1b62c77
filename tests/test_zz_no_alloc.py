"""cfpp_neox_layer_decode_static, the layer step that allocates nothing (its scratch is an array inside the library),
called through the C ABI with raw device pointers and compared, bit for bit, with cfpp_neox_layer_decode on a
caller-provided workspace: two calls in a row, the second on a smaller geometry and a shorter context, so that the
second call finds the first one's contents in the shared array.  Also what the entry point is for: the free device
memory does not move across its calls, a call recorded into a graph replays to the eager result, a device-side
failure of one of its launches is reported, and a process that has not run cfpp_init() is told so."""
import ctypes
import os
import subprocess
import sys

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


def _io_for(dims, out, k_new, v_new, xg, kg, vg, cg, sg, rows, S, d_seq=None, stride=0):
    return Io(input=xg.data_ptr(), output=out.data_ptr(), k_new=k_new.data_ptr(), v_new=v_new.data_ptr(), k_cache=kg.data_ptr(),
              v_cache=vg.data_ptr(), cache_rows=rows, cos=cg.data_ptr(), sin=sg.data_ptr(), rope_stride=stride, seq_len=S,
              d_seq_len=None if d_seq is None else d_seq.data_ptr(), max_seq_len=0, attn_output=None, mlp_intermediate=None)


def test_static_calls_allocate_nothing_and_replay_from_a_graph():
    """Free device memory is the same before and after the calls (no hipMalloc behind them), and one call recorded with
    torch.cuda.graph on a side stream gives the eager call's bits on every replay, with eager work in between."""
    lib = _lib()
    assert lib.cfpp_init() == 0
    dims, S = O.PYTHIA_2B8, 77
    print(f"\ncase static scratch: allocation and capture, hidden={dims.hidden} S={S}", flush=True)
    w, (x, k, v, cos, sin), wg, (xg, cg, sg) = _case(dims, S, 53)
    d = Dims(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps)
    cw = Weights(**{name: wg[name].data_ptr() for name, _ in Weights._fields_})
    kg, vg = k.to(DEV), v.to(DEV)
    out = torch.empty(1, dims.hidden, dtype=torch.float16, device=DEV)
    k_new, v_new = torch.empty_like(out), torch.empty_like(out)
    io = _io_for(dims, out, k_new, v_new, xg, kg, vg, cg, sg, S + 1, S)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), 0, stream) == 0    # first use: symbol lookup
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for mode in (0, 1, 0):
        assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "a static call changed the free device memory"
    eager = out.clone()
    ref = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims)
    assert_close("eager static output vs oracle", eager, ref["output"])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), 0, side.cuda_stream)
    assert rc == 0, rc
    for i in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
        assert torch.equal(kg[S], k_new.reshape(-1))
        # eager work between the replays, on the same static array, another geometry
        _call(lib, O.PYTHIA_6B9, *_small_6b9(), static=True)
    assert lib.cfpp_device_status(0) == 0


_6B9_CASE = {}


def _small_6b9():
    if not _6B9_CASE:
        dims = O.PYTHIA_6B9
        w, (x, k, v, cos, sin), wg, (xg, cg, sg) = _case(dims, 40, 54)
        _6B9_CASE["args"] = (wg, xg, cg, sg, k, v, 40, 0)
    return _6B9_CASE["args"]


def test_static_call_reports_a_device_side_failure():
    """A device-side length with no cache row of its own: the launch flags it, cfpp_device_status shows bit 1 and the
    next launching call returns CFPP_ERR_DEVICE, although the status word inside the static array is cleared by every
    call.  The kernels clamp the length and exit normally."""
    lib = _lib()
    assert lib.cfpp_init() == 0
    assert lib.cfpp_device_status(1) == 0
    dims, rows = O.PYTHIA_2B8, 20
    print(f"\ncase static scratch: device seq_len == cache rows ({rows})", flush=True)
    w, (x, k, v, cos, sin), wg, (xg, cg, sg) = _case(dims, rows - 1, 55)
    import clusterfusionplus_amd as pkg
    cos_t, sin_t = pkg.rope_tables(rows, dims.rotary_dim, device=DEV)
    d = Dims(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, dims.eps)
    cw = Weights(**{name: wg[name].data_ptr() for name, _ in Weights._fields_})
    kg, vg = k.to(DEV), v.to(DEV)
    k0, v0 = kg.clone(), vg.clone()
    out = torch.empty(1, dims.hidden, dtype=torch.float16, device=DEV)
    k_new, v_new = torch.empty_like(out), torch.empty_like(out)
    seq = torch.tensor([rows], dtype=torch.int32, device=DEV)
    io = _io_for(dims, out, k_new, v_new, xg, kg, vg, cos_t, sin_t, rows, 0, d_seq=seq, stride=dims.rotary_dim)
    stream = torch.cuda.current_stream().cuda_stream
    for mode in (0, 1):
        assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(kg, k0) and torch.equal(vg, v0)                   # nothing appended
        assert lib.cfpp_device_status(0) & 2
        assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), mode, stream) == -7
        assert lib.cfpp_device_status(1) & 2 and lib.cfpp_device_status(0) == 0
    # a valid length afterwards: back to normal, equal to the oracle
    seq.fill_(rows - 1)
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), ctypes.byref(cw), ctypes.byref(io), 0, stream) == 0
    torch.cuda.synchronize()
    ref = O.neox_layer_decode(x, w, k, v, cos_t[rows - 1:rows].cpu(), sin_t[rows - 1:rows].cpu(), rows - 1, dims)
    assert_close("output after the failure was cleared", out, ref["output"])
    assert lib.cfpp_device_status(0) == 0


def test_static_call_before_init_is_refused_in_a_fresh_process():
    """In a process where nothing has created the failure-flag word, the static entry point launches nothing and returns
    CFPP_ERR_NOT_INITIALISED (-11); after cfpp_init() it gets as far as its argument checks (-1 for the NULL tensors)."""
    code = (
        "import ctypes, torch\n"
        "torch.cuda.init()\n"
        f"lib = ctypes.CDLL({os.path.join(ROOT, 'clusterfusionplus_amd', 'libcfpp.so')!r})\n"
        "class D(ctypes.Structure):\n"
        "    _fields_ = [(n, ctypes.c_int32) for n in ('hidden', 'heads', 'head_dim', 'rotary_dim', 'ffn')] + [('eps', ctypes.c_float)]\n"
        "d = D(2560, 32, 80, 20, 10240, 1e-5)\n"
        "a = lib.cfpp_neox_layer_decode_static(ctypes.byref(d), None, None, 0, None)\n"
        "b = lib.cfpp_init()\n"
        "c = lib.cfpp_neox_layer_decode_static(ctypes.byref(d), None, None, 0, None)\n"
        "print('RESULT', a, b, c)\n")
    res = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    line = [l for l in res.stdout.splitlines() if l.startswith("RESULT")]
    assert line, res.stdout[-2000:]
    assert line[0].split()[1:] == ["-11", "0", "-1"], line[0]
