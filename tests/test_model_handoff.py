"""The prefill -> decode hand-off for a whole model and the reference's end-to-end check (reference
tests/benchmark_decode.py:60-119 pulls 12 tensors x layers plus `past_key_values` out of a HuggingFace model,
:147-189 decodes token by token, :446-448 compares the generated ids with HuggingFace's own generation).

The HuggingFace model is built locally from a config with random weights (no download).  CPU part: the conversion
(`stack_tensors_from_hf`) feeds the oracle's layer step and reproduces HuggingFace's next-token logits in float64.
GPU part: HuggingFace prefills a prompt, `NeoxDecoder.from_hf` converts, the decoder generates from its captured
hipGraph, and every token is HuggingFace's greedy token (or the two logits are closer than the tolerance) with the
logits agreeing at every step."""
import pytest
import torch

from oracle import neox_oracle as O

transformers = pytest.importorskip("transformers")


def _hf_model(dims, n_layers, vocab, seed, dtype):
    from oracle import hf_neox
    g = torch.Generator().manual_seed(seed)
    layers = [O.make_layer_weights(dims, layer=seed + i, w_std=0.05, b_std=0.02) for i in range(n_layers)]
    embed = torch.randn(vocab, dims.hidden, generator=g).half()
    lm = (0.05 * torch.randn(vocab, dims.hidden, generator=g)).half()
    fw = (1 + 0.02 * torch.randn(dims.hidden, generator=g)).half()
    fb = (0.01 * torch.randn(dims.hidden, generator=g)).half()
    return hf_neox.build_hf_model(dims, layers, embed, fw, fb, lm, dtype=dtype)      # fp16-representable values in `dtype`


def _fp16_cache(cache):
    """The prefill's cache with its values rounded to fp16 (what the decode caches hold)."""
    from transformers import DynamicCache
    return DynamicCache(ddp_cache_data=[(l.keys.half().to(l.keys.dtype), l.values.half().to(l.values.dtype)) for l in cache.layers])


def test_stack_tensors_from_hf_feed_the_oracle_to_hf_logits():
    from clusterfusionplus_amd.model import config_from_hf, stack_tensors_from_hf, layer_tensor_order
    dims = O.NeoxDims(hidden=64, heads=4, head_dim=16, rotary_dim=4, ffn=256)
    L, V, P = 3, 97, 7
    model = _hf_model(dims, L, V, seed=5, dtype=torch.float64)
    cfg = config_from_hf(model.config)
    assert (cfg.hidden, cfg.heads, cfg.head_dim, cfg.rotary_dim, cfg.ffn, cfg.n_layers, cfg.vocab) == (64, 4, 16, 4, 256, L, V)
    assert cfg.eps == dims.eps and cfg.rope_base == 10000.0
    prompt = torch.randint(0, V, (1, P), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        out = model(input_ids=prompt, use_cache=True)
    t = stack_tensors_from_hf(model, out.past_key_values, max_rows=P + 4, dtype=torch.float64)
    assert t["seq_len"] == P and len(t["layers"]) == L and tuple(t["layers"][0]) == layer_tensor_order
    assert t["k_caches"][0].shape == (P + 4, 64) and torch.equal(t["k_caches"][1][P:], torch.zeros(4, 64, dtype=torch.float64))
    cache = out.past_key_values
    tok = int(out.logits[0, -1].argmax())
    for step in range(4):
        S = P + step
        cos, sin = O.rope_table(torch.tensor([S]), dims.rotary_dim)
        h = t["embed"][tok].reshape(1, -1)
        for w, kc, vc in zip(t["layers"], t["k_caches"], t["v_caches"]):
            h = O.neox_layer_decode(h, w, kc, vc, cos, sin, S, dims, dtype=torch.float64, round_io=False, write_cache=True)["output"]
        logits = (O.layer_norm(h, t["final_ln_w"], t["final_ln_b"], dims.eps) @ t["lm_head"].t()).reshape(-1)
        with torch.no_grad():
            want = model(input_ids=torch.tensor([[tok]]), past_key_values=cache, use_cache=True).logits[0, -1]
        assert torch.allclose(logits, want, atol=1e-6, rtol=0), (step, float((logits - want).abs().max()))
        tok = int(want.argmax())
    with pytest.raises(ValueError):
        stack_tensors_from_hf(model, out.past_key_values, max_rows=P)            # no row for the first generated token


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["fused", "split"])
def test_hf_prefill_then_graph_decode_matches_hf_greedy_generation(mode):
    import clusterfusionplus_amd as pkg
    dims = O.NeoxDims(hidden=1024, heads=16, head_dim=64, rotary_dim=16, ffn=4096)
    L, V, P, N = 4, 2048, 32, 16
    print(f"\ncase HF model hand-off: {L} layers, hidden {dims.hidden}, prompt {P}, {N} generated tokens, {mode}", flush=True)
    model = _hf_model(dims, L, V, seed=11, dtype=torch.float32)
    prompt = torch.randint(0, V, (1, P), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        out = model(input_ids=prompt, use_cache=True)
    first = int(out.logits[0, -1].argmax())
    dec, S = pkg.NeoxDecoder.from_hf(model, out.past_key_values, max_rows=P + N + 2, device="cuda:0", mode=mode)
    assert S == P
    cache = _fp16_cache(out.past_key_values)
    dec.set_state(first, S)
    tok, ours, worst_cos, worst_err, off = first, [], 1.0, 0.0, 0
    for step in range(N):
        dec.graph_steps(1)
        torch.cuda.synchronize()
        logits = dec.logits.cpu()
        with torch.no_grad():
            want = model(input_ids=torch.tensor([[tok]]), past_key_values=cache, use_cache=True).logits[0, -1]
        cs = float(torch.nn.functional.cosine_similarity(logits.double(), want.double(), dim=0))
        err = float((logits - want).abs().max())
        worst_cos, worst_err = min(worst_cos, cs), max(worst_err, err)
        assert cs >= 0.9999 and err <= 2e-2, (step, cs, err)
        pick = int(dec.state.cpu()[0])
        assert pick == int(torch.argmax(logits))
        hf_pick = int(want.argmax())
        # HuggingFace's greedy token, or one whose HF logit is within the logit tolerance of HF's best
        assert pick == hf_pick or float(want.max() - want[pick]) <= 2e-2, (step, pick, hf_pick)
        off += pick != hf_pick
        ours.append(pick)
        tok = pick                      # HuggingFace follows the decoder's token, so both hold the same history
    print(f"  {N} tokens, {off} picks differ from HF's within the tolerance; logits max-abs {worst_err:.3e}, worst cosine {worst_cos:.7f}",
          flush=True)
    assert dec.generated() == ours
    assert int(dec.state.cpu()[1]) == P + N
    # the appended rows are what HuggingFace's cache holds for the same tokens
    for l in (0, L - 1):
        hk = cache.layers[l].keys[0].permute(1, 0, 2).reshape(P + N, -1)
        got = dec._k_caches[l][:P + N].cpu().float()
        assert float((got - hk).abs().max()) <= 2e-2, l
