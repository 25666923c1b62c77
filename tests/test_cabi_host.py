"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header declares,
and rejects bad arguments with its documented status codes before anything is launched."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "clusterfusionplus_amd", "libcfpp.so")
HEADER = os.path.join(ROOT, "include", "cfpp.h")


@pytest.fixture(scope="module")
def lib():
    import torch  # noqa: F401  the HIP runtime the library binds to
    if not os.path.exists(LIB):
        pytest.fail("libcfpp.so is not built: run `python -m clusterfusionplus_amd.build`")
    return ctypes.CDLL(LIB)


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cfpp_[a-z0-9_]+)\s*\(", text)))


class Dims(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int32), ("heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
                ("rotary_dim", ctypes.c_int32), ("ffn", ctypes.c_int32), ("eps", ctypes.c_float)]


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert len(names) >= 18, names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in cfpp.h but not exported by libcfpp.so: {missing}"


def test_status_strings_and_version(lib):
    lib.cfpp_status_str.restype = ctypes.c_char_p
    lib.cfpp_version.restype = ctypes.c_char_p
    assert lib.cfpp_status_str(0) == b"ok"
    seen = {lib.cfpp_status_str(-i) for i in range(1, 12)}
    assert len(seen) == 11 and b"unknown status" not in seen
    assert lib.cfpp_status_str(-12) == b"unknown status"
    assert b"gfx950" in lib.cfpp_version()


def test_workspace_bytes_and_dims_validation(lib):
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    ok = [Dims(2560, 32, 80, 20, 10240, 1e-5), Dims(4096, 32, 128, 32, 16384, 1e-5)]
    for d in ok:
        n = lib.cfpp_neox_workspace_bytes(ctypes.byref(d))
        assert n > 0 and n % 256 == 0
    bad = [Dims(2560, 32, 81, 20, 10240, 1e-5),     # hidden != heads * head_dim
           Dims(4100, 32, 128, 32, 16384, 1e-5),
           Dims(8192, 32, 256, 32, 32768, 1e-5),    # head_dim > 128
           Dims(4096, 32, 128, 33, 16384, 1e-5),    # odd rotary_dim
           Dims(4096, 32, 128, 32, 16384, 0.0)]     # eps
    for d in bad:
        assert lib.cfpp_neox_workspace_bytes(ctypes.byref(d)) == 0
    assert lib.cfpp_neox_workspace_bytes(None) == 0


def test_null_and_mode_errors_launch_nothing(lib):
    d = Dims(4096, 32, 128, 32, 16384, 1e-5)
    # unknown mode, NULL structs: rejected before any HIP call, so this runs without a GPU
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), None, None, 7, None, ctypes.c_size_t(0), None) == -6
    assert lib.cfpp_neox_layer_decode(ctypes.byref(d), None, None, 0, None, ctypes.c_size_t(0), None) == -1
    assert lib.cfpp_neox_layer_decode(None, None, None, 0, None, ctypes.c_size_t(0), None) == -1
    assert lib.cfpp_neox_mlp_down(ctypes.byref(d), None, None, None, None, None, None, None, ctypes.c_size_t(0), None) == -1
    assert lib.cfpp_ctx_step(0, ctypes.c_int64(12345), None, None, 0, None, None) == -1
    assert lib.cfpp_ctx_destroy(0, ctypes.c_int64(12345)) == 0          # unknown id: no-op
    assert lib.cfpp_stack_create(None, None) == -1
    assert lib.cfpp_stack_destroy(None) == 0
    assert lib.cfpp_neox_lm_head(4096, 100, ctypes.c_float(1e-5), None, None, None, None, None, None) == -1
    # a vocabulary beyond what the 32-bit row shares of the kernels cover is refused (-2) before anything is launched
    buf = ctypes.create_string_buffer(64)
    ptr = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.cfpp_neox_lm_head(4096, (1 << 19) + 1, ctypes.c_float(1e-5), ptr, ptr, ptr, ptr, ctypes.cast(buf, ctypes.POINTER(ctypes.c_float)), None) == -2


def test_one_launch_rule_and_device_status_without_a_gpu(lib):
    """The routing rule of the fused mode: a grid is launched in one piece only if it fits compute units x occupancy."""
    fits = lib.cfpp_one_launch_fits
    assert fits(256, 256, 1) == 1 and fits(256, 256, 2) == 1 and fits(512, 256, 2) == 1
    assert fits(257, 256, 1) == 0 and fits(256, 128, 1) == 0 and fits(256, 255, 1) == 0
    assert fits(256, 256, 0) == 0            # the kernel does not fit a compute unit at all (or the query failed)
    assert fits(0, 256, 1) == 0 and fits(256, 0, 1) == 0 and fits(-1, 256, 1) == 0
    assert fits(1 << 30, 1 << 30, 4) == 1    # no overflow in the product
    assert lib.cfpp_device_status(0) == 0 and lib.cfpp_device_status(1) == 0
    assert lib.cfpp_ctx_check(0, ctypes.c_int64(4242), None) == -5          # unknown context
    assert lib.cfpp_stack_check(None, None) == -1
    assert lib.cfpp_stack_layers_per_launch(None) == -1


class NeoxIo(ctypes.Structure):
    _fields_ = [("input", ctypes.c_void_p), ("output", ctypes.c_void_p), ("k_new", ctypes.c_void_p), ("v_new", ctypes.c_void_p),
                ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p), ("cache_rows", ctypes.c_int32),
                ("cos", ctypes.c_void_p), ("sin", ctypes.c_void_p), ("rope_stride", ctypes.c_int32), ("seq_len", ctypes.c_int32),
                ("d_seq_len", ctypes.c_void_p), ("max_seq_len", ctypes.c_int32), ("attn_output", ctypes.c_void_p),
                ("mlp_intermediate", ctypes.c_void_p)]


def test_sequence_length_rules_are_checked_before_any_launch(lib):
    """seq_len may equal the cache rows only when the append can be skipped and cos / sin are the position's own row;
    with position-indexed tables or a device-side length the position needs a row of its own."""
    d = Dims(2560, 32, 80, 20, 10240, 1e-5)
    w = (ctypes.c_void_p * 12)(*([4096] * 12))
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    n = lib.cfpp_neox_workspace_bytes(ctypes.byref(d))
    ws = ctypes.c_void_p(1 << 20)

    def call(**kw):
        io = NeoxIo(input=4096, output=4096, k_new=4096, v_new=4096, k_cache=4096, v_cache=4096, cache_rows=10, cos=4096, sin=4096,
                    rope_stride=0, seq_len=0, d_seq_len=None, max_seq_len=0, attn_output=None, mlp_intermediate=None)
        for k, v in kw.items():
            setattr(io, k, v)
        return lib.cfpp_neox_layer_decode(ctypes.byref(d), w, ctypes.byref(io), 7 if kw.get("_mode") else 0, ws, ctypes.c_size_t(n), None)

    assert call(seq_len=11) == -3 and call(seq_len=-1) == -3 and call(cache_rows=-1) == -3
    assert call(seq_len=10, rope_stride=20) == -3            # the table has no row for position 10
    assert call(seq_len=3, rope_stride=-20) == -3
    assert call(d_seq_len=4096, cache_rows=0) == -3          # a device-side length always appends
    assert call(seq_len=3, cos=4100) == -8                   # misaligned pointer: still an argument error, nothing launched


def test_static_entry_point_argument_errors_launch_nothing(lib):
    """The allocation-free layer step: bad mode, bad geometry and a geometry beyond its built-in scratch array are
    refused before any HIP call."""
    lib.cfpp_static_scratch_bytes.restype = ctypes.c_size_t
    lib.cfpp_neox_workspace_bytes.restype = ctypes.c_size_t
    cap = lib.cfpp_static_scratch_bytes()
    assert cap == 1280 * 1024
    for d in (Dims(2560, 32, 80, 20, 10240, 1e-5), Dims(4096, 32, 128, 32, 16384, 1e-5)):
        assert lib.cfpp_neox_workspace_bytes(ctypes.byref(d)) <= cap
    d = Dims(4096, 32, 128, 32, 16384, 1e-5)
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(d), None, None, 5, None) == -6
    assert lib.cfpp_neox_layer_decode_static(None, None, None, 0, None) == -1
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(Dims(4096, 32, 128, 33, 16384, 1e-5)), None, None, 0, None) == -2
    wide = Dims(4096, 512, 8, 8, 16384, 1e-5)
    assert lib.cfpp_neox_workspace_bytes(ctypes.byref(wide)) > cap
    assert lib.cfpp_neox_layer_decode_static(ctypes.byref(wide), None, None, 0, None) == -10
    lib.cfpp_status_str.restype = ctypes.c_char_p
    assert b"static" in lib.cfpp_status_str(-10)
    assert b"cfpp_init" in lib.cfpp_status_str(-11)
    # a valid geometry gets as far as the device set-up and no further: without a GPU that is a HIP error (> 0), with
    # one it is -11 until cfpp_init() has created the failure-flag word (NULL tensors are looked at after that)
    import torch
    rc = lib.cfpp_neox_layer_decode_static(ctypes.byref(d), None, None, 0, None)
    assert (rc > 0) if not torch.cuda.is_available() else rc in (-11, -1)


def test_shapes_without_an_instantiation_are_refused(lib):
    """Only the (hidden chunks, MLP-down chunks) pairs the kernels are instantiated for are accepted; the workspace size
    is defined for any valid geometry, the launching calls refuse the others before touching the device."""
    ws = ctypes.c_void_p(1 << 20)
    w = (ctypes.c_void_p * 12)(*([4096] * 12))
    for hidden, heads, hd, ffn in ((1536, 12, 128, 6144), (3072, 24, 128, 12288), (3584, 28, 128, 14336), (4096, 32, 128, 8192)):
        d = Dims(hidden, heads, hd, 32, ffn, 1e-5)
        io = NeoxIo(input=4096, output=4096, k_new=4096, v_new=4096, k_cache=4096, v_cache=4096, cache_rows=10, cos=4096, sin=4096,
                    rope_stride=0, seq_len=0, d_seq_len=None, max_seq_len=0, attn_output=None, mlp_intermediate=None)
        assert lib.cfpp_neox_layer_decode(ctypes.byref(d), w, ctypes.byref(io), 0, ws, ctypes.c_size_t(8 << 20), None) == -2, hidden
    buf = ctypes.create_string_buffer(64)
    ptr = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.cfpp_neox_lm_head(1536, 100, ctypes.c_float(1e-5), ptr, ptr, ptr, ptr, ctypes.cast(buf, ctypes.POINTER(ctypes.c_float)), None) == -2


class LlamaBatch(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int32), ("heads", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("eps", ctypes.c_float),
                ("batch", ctypes.c_int32), ("layer_id", ctypes.c_int32)] + [(n, ctypes.c_void_p) for n in (
                    "rms_w", "w_qkv", "w_o", "input", "residual", "residual_out", "output", "paged_kv_indptr", "paged_kv_indices",
                    "k_cache_ptrs", "v_cache_ptrs", "positions", "cos_sin")]


def test_llama_batch_argument_checks_launch_nothing(lib):
    lib.cfpp_llama_batch_workspace_bytes.restype = ctypes.c_size_t
    n = lib.cfpp_llama_batch_workspace_bytes(4096, 32, 128, 16)
    assert n > 0 and n % 256 == 0
    assert lib.cfpp_llama_batch_workspace_bytes(4096, 32, 128, 32) > n           # scratch grows with the batch
    assert lib.cfpp_llama_batch_workspace_bytes(4096, 32, 128, 0) == 0
    assert lib.cfpp_llama_batch_workspace_bytes(4100, 32, 128, 4) == 0
    ws = ctypes.c_void_p(256)
    a = LlamaBatch(4096, 32, 128, 1e-6, 4, 0)
    assert lib.cfpp_llama_batch_decode(None, ws, ctypes.c_size_t(n), None) == -1
    assert lib.cfpp_llama_batch_decode(ctypes.byref(a), ws, ctypes.c_size_t(n), None) == -1          # NULL tensors
    for f in ("rms_w", "w_qkv", "w_o", "input", "residual", "residual_out", "output", "cos_sin", "paged_kv_indptr", "paged_kv_indices",
              "k_cache_ptrs", "v_cache_ptrs", "positions"):
        setattr(a, f, 4096)
    a.residual_out = 8192
    a.input = 4104                                                                                     # not 16-byte aligned
    assert lib.cfpp_llama_batch_decode(ctypes.byref(a), ws, ctypes.c_size_t(n), None) == -8
    a.input = 8192                                                                                     # sum written over a row still read
    assert lib.cfpp_llama_batch_decode(ctypes.byref(a), ws, ctypes.c_size_t(n), None) == -9
    a.input = 4096
    assert lib.cfpp_llama_batch_decode(ctypes.byref(a), ws, ctypes.c_size_t(16), None) == -4           # workspace too small
    a.batch = 0
    assert lib.cfpp_llama_batch_decode(ctypes.byref(a), ws, ctypes.c_size_t(n), None) == -2


def test_package_imports_and_exposes_reference_names():
    import clusterfusion
    want = ["pythia_2b8_decoder_layer", "pythia_2b8_decoder_layer_split", "pythia_2b8_attention_only",
            "pythia_2b8_mlp_only", "pythia_2b8_create_graph_context", "pythia_2b8_graph_decode_step",
            "pythia_2b8_destroy_graph_context", "pythia_6b9_decoder_layer", "pythia_6b9_create_graph_context",
            "pythia_6b9_graph_decode_step", "pythia_6b9_destroy_graph_context",   # reference include/pybind.cpp:284-297
            "llama_decoder_layer_sglang", "llama_decoder_layer_batch_decode_sglang"]  # :281-282
    for n in want:
        assert callable(getattr(clusterfusion, n)), n
    # CPU tensors are refused with an exception, not a crash
    import torch
    t = torch.zeros(1, 2560, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        clusterfusion.pythia_2b8_mlp_only(t, t, t, t, t)
    with pytest.raises(RuntimeError, match="not initialized"):
        clusterfusion.pythia_2b8_graph_decode_step(99, t, t, t, t, t, t, t, t, t, t, t, t, t, 0)


def test_rope_tables_match_oracle():
    from clusterfusionplus_amd.model import rope_tables
    from oracle.neox_oracle import rope_table
    import torch
    c, s = rope_tables(300, 20, device="cpu")
    c2, s2 = rope_table(torch.arange(300), 20)
    assert torch.equal(c, c2) and torch.equal(s, s2)


def test_hf_hand_off_helpers_reproduce_the_hf_layer():
    """layer_tensors_from_hf / kv_cache_from_hf: a prefill done by HuggingFace, one decode step by the oracle on the
    converted tensors == the HF layer's own decode step."""
    pytest.importorskip("transformers")
    import torch
    from transformers import DynamicCache
    from clusterfusionplus_amd.model import kv_cache_from_hf, layer_tensors_from_hf, layer_tensor_order
    from oracle import hf_neox, neox_oracle as O
    dims = O.NeoxDims(hidden=64, heads=4, head_dim=16, rotary_dim=4, ffn=256)
    w0 = O.make_layer_weights(dims, layer=3, w_std=0.2, b_std=0.1)
    layer = hf_neox.build_hf_layer(dims, w0, dtype=torch.float64)
    w = layer_tensors_from_hf(layer, dtype=torch.float64)
    assert tuple(w) == layer_tensor_order
    for k in layer_tensor_order:
        assert torch.equal(w[k].reshape(-1), w0[k].double().reshape(-1)), k
    S = 6
    g = torch.Generator().manual_seed(4)
    key = torch.randn(1, dims.heads, S, dims.head_dim, generator=g, dtype=torch.float64)
    val = torch.randn(1, dims.heads, S, dims.head_dim, generator=g, dtype=torch.float64)
    kc, vc, n = kv_cache_from_hf(key, val, rows=S + 2, dtype=torch.float64)
    assert n == S and kc.shape == (S + 2, dims.hidden) and torch.equal(kc[S:], torch.zeros(2, dims.hidden, dtype=torch.float64))
    x = torch.randn(1, dims.hidden, generator=g, dtype=torch.float64)
    cos, sin = O.rope_table(torch.tensor([S]), dims.rotary_dim)
    got = O.neox_layer_decode(x, w, kc, vc, cos, sin, S, dims, dtype=torch.float64, round_io=False)
    cache = DynamicCache(ddp_cache_data=[(key.clone(), val.clone())])
    c = cos.double().reshape(-1)[: dims.rotary_dim][None, None]
    s_ = sin.double().reshape(-1)[: dims.rotary_dim][None, None]
    with torch.no_grad():
        want = layer(x.reshape(1, 1, -1), attention_mask=None, layer_past=cache, position_embeddings=(c, s_))
    want = want[0] if isinstance(want, tuple) else want
    assert torch.allclose(got["output"], want.reshape(1, -1), atol=1e-6, rtol=0)
    with pytest.raises(ValueError):
        kv_cache_from_hf(key, val, rows=S - 1)
