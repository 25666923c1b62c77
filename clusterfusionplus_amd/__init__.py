"""MI355X (gfx950) implementation of ClusterFusion++'s fused GPT-NeoX / Pythia decode step.

The operator surface is the reference's (`clusterfusion/__init__.py:6-16` re-exports every
non-underscore name of its native module; the names are listed in include/pybind.cpp:280-297):

    pythia_2b8_decoder_layer, pythia_2b8_decoder_layer_split, pythia_2b8_attention_only,
    pythia_2b8_mlp_only, pythia_2b8_create_graph_context, pythia_2b8_graph_decode_step,
    pythia_2b8_destroy_graph_context, and the pythia_6b9_* twins
    (the 6.9B split / attention_only / mlp_only ops are additions; the reference has none).

Everything runs in the HIP library; there is no Python or CPU fallback.  Importing this package
without the built native libraries raises ImportError (build them with
`python -m clusterfusionplus_amd.build`).
"""
import importlib
import os as _os
import sys as _sys

_here = _os.path.dirname(_os.path.abspath(__file__))
_missing = [n for n in ("libcfpp.so", "_clusterfusion.so") if not _os.path.exists(_os.path.join(_here, n))]
# `python -m clusterfusionplus_amd.build` has to get past this file on a fresh checkout: for that one command
# the package imports without its operators; every other import without the libraries fails here.
_building = "clusterfusionplus_amd.build" in getattr(_sys, "orig_argv", [])

if _missing and not _building:
    raise ImportError(
        f"clusterfusionplus_amd: native library {_missing[0]} is missing from {_here}; "
        "run `python -m clusterfusionplus_amd.build` (needs hipcc for gfx950). There is no fallback path.")

__all__ = []
if not _missing:
    import torch as _torch  # noqa: F401  (loads the HIP runtime the native libraries bind to)

    _native = importlib.import_module("clusterfusionplus_amd._clusterfusion")
    __all__ = [n for n in dir(_native) if not n.startswith("_")]
    globals().update({n: getattr(_native, n) for n in __all__})

    from .model import (NeoxConfig, PYTHIA_2B8, PYTHIA_6B9, NeoxDecoder, layer_tensor_order, rope_tables,  # noqa: E402
                        layer_tensors_from_hf, kv_cache_from_hf, config_from_hf, stack_tensors_from_hf)

    __all__ += ["NeoxConfig", "PYTHIA_2B8", "PYTHIA_6B9", "NeoxDecoder", "layer_tensor_order", "rope_tables",
                "layer_tensors_from_hf", "kv_cache_from_hf", "config_from_hf", "stack_tensors_from_hf"]
