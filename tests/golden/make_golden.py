"""Writes the golden fixtures of the decode-step parity tests.

The reference repository holds no stored expected outputs (its scripts compute them live on a CUDA device),
so the fixtures are produced by this repository's CPU oracle after it has been pinned against HuggingFace
GPTNeoXLayer / LlamaAttention, a brute-force loop and closed forms (tests/test_oracle_pins.py).  Inputs are regenerated from
fixed seeds (oracle.neox_oracle.make_layer_weights / make_layer_inputs); only the expected outputs are
stored, as float32 in one .npz per case.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import neox_oracle as O  # noqa: E402

CASES = {
    # name: (dims, seq_len, seed)
    "neox_h512_s37": (O.NeoxDims(hidden=512, heads=8, head_dim=64, rotary_dim=16, ffn=2048), 37, 101),
    "pythia_2b8_s512": (O.PYTHIA_2B8, 512, 102),
    "pythia_6b9_s2048": (O.PYTHIA_6B9, 2048, 103),
}


def inputs(name):
    dims, S, seed = CASES[name]
    w = O.make_layer_weights(dims, layer=seed)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S, capacity=S + 1, seed=seed)
    return dims, S, w, x, k, v, cos, sin


# LLaMA attention block (llama_attention_sglang): dims, cache rows, seed
LLAMA_CASES = {
    "llama_h1024_s333": (O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0), 333, 7),
    "llama2_7b_s1024": (O.LLAMA2_7B, 1024, 8),
}


def llama_inputs(name):
    dims, S, seed = LLAMA_CASES[name]
    return (dims,) + tuple(O.make_llama_attn_inputs(dims, S, seed=seed))


# plain LLaMA op (llama_attention_plain): dims, cache rows, seed
LLAMA_PLAIN_CASES = {"llama_plain_h1024_s200": (O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0), 200, 3)}
# paged batch (llama_batch_decode_paged): dims, cached tokens per sequence, seed, layer whose caches are used
LLAMA_BATCH_CASES = {"llama_batch_h1024": (O.LlamaDims(hidden=1024, heads=8, head_dim=128, ffn=0), [77, 5, 300, 0, 41], 4, 1)}


def llama_plain_inputs(name):
    dims, S, seed = LLAMA_PLAIN_CASES[name]
    return (dims,) + tuple(O.make_llama_plain_inputs(dims, S, seed=seed, w_std=0.05))


def llama_batch_inputs(name):
    dims, lens, seed, layer_id = LLAMA_BATCH_CASES[name]
    return (dims, layer_id) + tuple(O.make_llama_batch_inputs(dims, lens, seed=seed, w_std=0.05))


# The reference's own unit-test inputs (oracle.make_reference_unit_test_inputs: reference tests/test_pythia.py:15,24-42,
# 162-230 and the 6.9B twin): dims, zero bias_o, RoPE tables padded to [1, D]
REFERENCE_RECIPE_CASES = {
    "pythia_2b8_reference_recipe_s129": (O.PYTHIA_2B8, True, True),
    "pythia_6b9_reference_recipe_s129": (O.PYTHIA_6B9, False, False),
}


def reference_recipe_inputs(name):
    dims, zero_bo, pad = REFERENCE_RECIPE_CASES[name]
    return (dims,) + tuple(O.make_reference_unit_test_inputs(dims, 129, zero_bias_o=zero_bo, pad_rope_to_head_dim=pad))


def new_rows(indptr, indices):
    return [int(indices[int(indptr[b + 1]) - 1]) for b in range(indptr.numel() - 1)]


def main():
    torch.set_num_threads(max(1, os.cpu_count() or 1))
    for name in REFERENCE_RECIPE_CASES:
        dims, w, x, k, v, cos, sin = reference_recipe_inputs(name)
        r = O.neox_layer_decode(x, w, k, v, cos, sin, 129, dims, dtype=torch.float64, round_io=True)
        out = {n: r[n].to(torch.float32).numpy() for n in ("output", "k_new", "v_new")}
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, {n: a.shape for n, a in out.items()}, os.path.getsize(path), "bytes")
    for name in LLAMA_PLAIN_CASES:
        dims, w, x, k, v, cos, sin = llama_plain_inputs(name)
        r = O.llama_attention_plain(x, w, k, v, cos, sin, dims, dtype=torch.float64, round_io=True)
        out = {n: r[n].to(torch.float32).numpy() for n in ("output", "k_new", "v_new")}
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, {n: a.shape for n, a in out.items()}, os.path.getsize(path), "bytes")
    for name in LLAMA_BATCH_CASES:
        dims, layer_id, w, x, res, indptr, indices, caches, positions, cos_sin = llama_batch_inputs(name)
        k, v = caches[layer_id]
        r = O.llama_batch_decode_paged(x, res, w, indptr, indices, k, v, positions, cos_sin, dims, dtype=torch.float64)
        rows = new_rows(indptr, indices)
        out = {"output": r["output"].to(torch.float32).numpy(), "residual": r["residual"].to(torch.float32).numpy(),
               "k_rows": r["k_cache"][rows].to(torch.float32).numpy(), "v_rows": r["v_cache"][rows].to(torch.float32).numpy()}
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, {n: a.shape for n, a in out.items()}, os.path.getsize(path), "bytes")
    for name in LLAMA_CASES:
        dims, w, x, res, k, v, cos, sin = llama_inputs(name)
        r = O.llama_attention_sglang(x, res, w, k, v, cos, sin, dims, dtype=torch.float64, round_io=True)
        out = {n: r[n].to(torch.float32).numpy() for n in ("output", "residual", "k_new", "v_new")}
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, {n: a.shape for n, a in out.items()}, os.path.getsize(path), "bytes")
    for name in CASES:
        dims, S, w, x, k, v, cos, sin = inputs(name)
        r = O.neox_layer_decode(x, w, k, v, cos, sin, S, dims, dtype=torch.float64, round_io=True)
        out = {n: r[n].to(torch.float32).numpy() for n in ("output", "k_new", "v_new", "attn_output", "mlp_intermediate")}
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **out)
        print(name, {n: a.shape for n, a in out.items()}, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
