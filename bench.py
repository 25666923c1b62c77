#!/usr/bin/env python3
"""Benchmark of the whole-model decode step (TPOT) on one MI355X.

A "step" is one generated token: embedding row -> 32 fused decoder layers -> final LayerNorm ->
LM head -> argmax (two launches: all layers, then the LM head with the pick and the next embedding row),
replayed from one captured hipGraph, batch 1, fp16 weights (random init, synthetic) with fp32
accumulation, KV caches pre-filled to the given context.

Prints ONE JSON line (last line of stdout).  `value` is ms per token (TPOT); `roofline` prices the
dominant kernel (the launch that runs the decoder layers: k_fused_stack, all layers in one launch, or
k_fused, one layer, with --mode fused_layers) against the 8 TB/s HBM peak using algorithmic bytes
(weights + small vectors + KV rows [0,S), read once) over its HIP-event-timed launch duration;
`cpu_baseline` is the HuggingFace GPTNeoXLayer fp32 path timed on this box's host cores on a bounded
sample (reported, not a target).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0



def recorded_traffic(model, ctx, kernel="k_fused"):
    """HBM bytes per launch of the fused layer kernel (fetched + written) as recorded in the committed hardware-counter
    summary of this workload (two `rocprofv3 --pmc` runs of this script, FETCH_SIZE and WRITE_SIZE, scaled by the
    256 MiB calibration copy): the number on the summary's `traffic_bytes_per_launch:` line and the file it came from,
    or (None, None) when no summary exists for the workload.  A counter run cannot be part of a timed run; the
    summary states the command and the commit it was taken at."""
    rel = os.path.join("profiles", f"{kernel}_{model}_ctx{ctx}_hbm_traffic.txt")
    try:
        with open(os.path.join(ROOT, rel)) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0]), rel
    except OSError:
        pass
    return None, None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def layer_bytes(cfg, S):
    """Algorithmic bytes of one decoder layer at context S: weights + biases/LN vectors + KV rows [0,S)."""
    H, F = cfg.hidden, cfg.ffn
    weights = 2 * (3 * H * H + H * H + 2 * F * H)
    small = 2 * (3 * H + H + F + H + 4 * H)
    kv = S * 2 * H * 2
    return weights + small + kv


def step_bytes(cfg, S):
    H = cfg.hidden
    return cfg.n_layers * layer_bytes(cfg, S) + cfg.vocab * H * 2 + 2 * H * 2 + H * 2


def build_model(cfg, rows, ctx, device, mode):
    import torch
    import clusterfusionplus_amd as pkg
    torch.manual_seed(0)
    H, F = cfg.hidden, cfg.ffn

    def rn(shape, std, mean=0.0):
        return torch.empty(shape, dtype=torch.float16, device=device).normal_(mean, std)

    layers = []
    for _ in range(cfg.n_layers):
        layers.append({
            "ln_w": rn((H,), 0.02, 1.0), "ln_b": rn((H,), 0.01),
            "w_qkv": rn((3 * H, H), 0.02), "b_qkv": rn((3 * H,), 0.01),
            "w_o": rn((H, H), 0.02), "b_o": rn((H,), 0.01),
            "post_ln_w": rn((H,), 0.02, 1.0), "post_ln_b": rn((H,), 0.01),
            "w_up": rn((F, H), 0.02), "b_up": rn((F,), 0.01),
            "w_down": rn((H, F), 0.02), "b_down": rn((H,), 0.01),
        })
    embed = rn((cfg.vocab, H), 1.0)
    lm_head = rn((cfg.vocab, H), 0.02)
    fw, fb = rn((H,), 0.02, 1.0), rn((H,), 0.01)
    k_caches = [rn((rows, H), 1.0) for _ in range(cfg.n_layers)]
    v_caches = [rn((rows, H), 1.0) for _ in range(cfg.n_layers)]
    dec = pkg.NeoxDecoder(cfg, layers, embed, fw, fb, lm_head, k_caches, v_caches, mode=mode)
    dec.tensors = dict(layers=layers, embed=embed, final_ln_w=fw, final_ln_b=fb, lm_head=lm_head, k_caches=k_caches, v_caches=v_caches)
    return dec


def time_tokens(dec, stream, ctx, tokens, warm):
    """TPOT in ms of `tokens` graph replays starting at context `ctx` + `warm`, HIP events on the launch stream."""
    import torch
    dec.set_state(11, ctx)
    dec.graph_steps(warm)
    stream.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    dec.graph_steps(tokens)
    e1.record(stream)
    stream.synchronize()
    return e0.elapsed_time(e1) / tokens


def context_sweep(dec, cfg, stream, contexts, tokens=24, warm=4):
    """TPOT and fraction of the 8 TB/s roofline at several contexts, on the model that is already resident."""
    out = []
    for c in contexts:
        tpot = time_tokens(dec, stream, c, tokens, warm)
        sb = step_bytes(cfg, c + warm + tokens // 2)
        out.append({"context": c, "tokens": tokens, "tpot_ms": round(tpot, 4), "bytes": sb,
                    "hbm_gbps": round(sb / (tpot * 1e-3) / 1e9, 1), "frac_of_peak": round(sb / (tpot * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        log(f"[sweep] context {c}: {tpot:.4f} ms/token = {out[-1]['frac_of_peak'] * 100:.1f} % of peak")
    dec.check()
    return out


def drop_in_loop(model, cfg, dec, ctx, tokens=24, warm=4):
    """The reference's own per-token flow through the drop-in ops (reference tests/benchmark_decode.py:225-284): one
    context per layer, per token the embedding row, 32 x `<model>_graph_decode_step`, `F.layer_norm`, the LM head
    matmul and argmax in torch.  The reference runs that Python loop eagerly; here the position lives in a device int32
    (the step op accepts one), so the loop is captured once with torch.cuda.graph and replayed per token."""
    import torch
    import clusterfusion as cf
    t = dec.tensors
    L, H, dev = cfg.n_layers, cfg.hidden, t["embed"].device
    create, step, destroy = (getattr(cf, f"{model}_{n}") for n in ("create_graph_context", "graph_decode_step", "destroy_graph_context"))
    rows = t["k_caches"][0].shape[0]
    base = 1000
    for l, w in enumerate(t["layers"]):
        create(base + l, t["k_caches"][l], t["v_caches"][l], w["w_qkv"], w["w_o"], w["w_up"], w["w_down"], rows)
    seq = torch.tensor([ctx], dtype=torch.int32, device=dev)
    tok = torch.tensor([11], dtype=torch.int64, device=dev)

    def one_token(library_head=False):
        h = t["embed"].index_select(0, tok)
        for l, w in enumerate(t["layers"]):
            h, _, _ = step(base + l, h, w["ln_w"], w["ln_b"], w["b_qkv"], w["b_o"], dec.cos, dec.sin, t["k_caches"][l], t["v_caches"][l],
                           w["post_ln_w"], w["post_ln_b"], w["b_up"], w["b_down"], seq)
        if library_head:
            # final LayerNorm + LM head in the library (one launch), argmax in torch
            logits = cf.lm_head(h, t["final_ln_w"], t["final_ln_b"], t["lm_head"], cfg.eps)
        else:
            h = torch.nn.functional.layer_norm(h, (H,), t["final_ln_w"], t["final_ln_b"], eps=cfg.eps)
            logits = torch.matmul(h, t["lm_head"].t())
        tok.copy_(torch.argmax(logits, dim=-1).reshape(1))
        seq.add_(1)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_token()                      # warm-up outside the capture (library handles, lazy initialisation)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(4):
        one_token()                      # the reference's way: the Python loop, launched eagerly
    e1.record()
    torch.cuda.synchronize()
    eager = e0.elapsed_time(e1) / 4
    eager_wall = (time.perf_counter() - t0) * 1e3 / 4
    def captured(library_head):
        with torch.cuda.stream(side):
            one_token(library_head)      # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_token(library_head)
        seq.fill_(ctx)
        for _ in range(warm):
            graph.replay()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(tokens):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        assert int(seq.item()) == ctx + warm + tokens
        return e0.elapsed_time(e1) / tokens
    tpot = captured(False)
    tpot_lib = captured(True)
    for l in range(L):
        destroy(base + l)                # raises if a step of the context failed on the device
    sb = step_bytes(cfg, ctx + warm + tokens // 2)
    return {"workload": f"{model}: per-layer contexts, {L} x {model}_graph_decode_step per token with a device current_seq_len, final "
                        "LayerNorm + LM head + argmax in torch, captured once with torch.cuda.graph and replayed",
            "context": ctx, "tokens": tokens, "tpot_ms": round(tpot, 4), "frac_of_peak": round(sb / (tpot * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "library_lm_head_tpot_ms": round(tpot_lib, 4),
            "library_lm_head_frac_of_peak": round(sb / (tpot_lib * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "library_lm_head_note": "same loop with the final LayerNorm + LM head in the library (lm_head op), argmax in torch",
            "eager_python_loop_tpot_ms": round(max(eager, eager_wall), 4)}


def cpu_baseline(cfg, S, budget_s=12.0):
    """HF GPTNeoXLayer (fp32, eager) on the host cores: one layer at context S, repeated for a bounded
    time, scaled to a token (x n_layers) plus the fp32 LM-head matvec."""
    import torch
    from oracle import neox_oracle as O
    dims = O.NeoxDims(cfg.hidden, cfg.heads, cfg.head_dim, cfg.rotary_dim, cfg.ffn, cfg.eps)
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    w = O.make_layer_weights(dims, layer=0)
    x, k, v, cos, sin = O.make_layer_inputs(dims, S)
    impl = "HF GPTNeoXLayer"
    try:
        from oracle import hf_neox
        layer = hf_neox.build_hf_layer(dims, w, dtype=torch.float32)
        run = lambda: hf_neox.hf_layer_decode(layer, x, k, v, cos, sin, S, dims, dtype=torch.float32)
        run()
    except Exception as e:   # transformers missing or incompatible on this box
        impl = "torch restatement of the layer (oracle)"
        log(f"[cpu_baseline] HF layer unavailable ({type(e).__name__}: {e}); timing the oracle restatement")
        wf = {n: t.float() for n, t in w.items()}
        run = lambda: O.neox_layer_decode(x, wf, k.float(), v.float(), cos, sin, S, dims)
        run()
    times = []
    t_end = time.perf_counter() + budget_s * 0.8
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 40):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    layer_ms = times[len(times) // 2] * 1e3
    lm = torch.randn(cfg.vocab, cfg.hidden)
    h = torch.randn(cfg.hidden)
    lm_times = []
    for _ in range(5):
        t0 = time.perf_counter()
        torch.mv(lm, h)
        lm_times.append(time.perf_counter() - t0)
    lm_ms = sorted(lm_times)[len(lm_times) // 2] * 1e3
    return {
        "value": round(layer_ms * cfg.n_layers + lm_ms, 3), "unit": "ms/token", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{impl}, fp32 eager, 1 layer at S={S} x {len(times)} runs (median {layer_ms:.2f} ms) scaled x{cfg.n_layers}"
                  f" + fp32 LM head matvec ({lm_ms:.2f} ms)",
    }


def bench_single_layer(model, S, steps=160, warmup=16, nset=8):
    """One decoder layer through the drop-in ops (`<model>_decoder_layer` and `<model>_decoder_layer_split`), batch-1
    decode at context S, replayed from a captured graph that cycles through `nset` weight and cache sets (more than the
    256 MB Infinity Cache holds), so that every launch reads HBM-cold data.  Returns {mode: us per layer}."""
    import torch
    import clusterfusion as cf
    import clusterfusionplus_amd as pkg
    dev = "cuda:0"
    cfg = pkg.PYTHIA_2B8 if model == "pythia_2b8" else pkg.PYTHIA_6B9
    H, F = cfg.hidden, cfg.ffn
    torch.manual_seed(5)

    def rn(shape, std, mean=0.0):
        return torch.empty(shape, dtype=torch.float16, device=dev).normal_(mean, std)
    sets = []
    for _ in range(nset):
        sets.append([rn((3 * H, H), 0.02), rn((3 * H,), 0.01), rn((H, H), 0.02), rn((H,), 0.01), rn((S + 1, H), 1.0), rn((S + 1, H), 1.0),
                     rn((H,), 0.02, 1.0), rn((H,), 0.01), None, None, rn((H,), 0.02, 1.0), rn((H,), 0.01), rn((F, H), 0.02), rn((F,), 0.01),
                     rn((H, F), 0.02), rn((H,), 0.01)])
    x = rn((1, H), 1.0)
    cos_t, sin_t = pkg.rope_tables(S + 1, cfg.rotary_dim, cfg.rope_base, device=dev)
    cos, sin = cos_t[S:S + 1].contiguous(), sin_t[S:S + 1].contiguous()
    for a in sets:
        a[8], a[9] = cos, sin
    out = {}
    for mode, name in (("fused", f"{model}_decoder_layer"), ("split", f"{model}_decoder_layer_split")):
        op = getattr(cf, name)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for a in sets:
                op(x, *a, S)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = [op(x, *a, S) for a in sets]
        for _ in range(max(1, warmup // nset)):
            graph.replay()
        torch.cuda.synchronize()
        reps = max(1, steps // nset)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        out[mode] = e0.elapsed_time(e1) * 1e3 / (reps * nset)
        del graph, keep
    if cf.device_status() != 0:
        raise RuntimeError("a layer launch raised a device-side failure flag")
    return out


def bench_llama_layer(args, emit=True):
    """Extra workload (not the headline): one LLaMA-2-7B layer, batch-1 decode at context --ctx (default 4096):
    the attention block (the reference's llama_decoder_layer_sglang) followed by the MLP block, replayed from a
    captured graph over 8 weight sets so that every launch reads HBM-cold weights."""
    import torch
    import clusterfusion as cf
    from oracle import neox_oracle as O      # seeded synthetic inputs only
    dev = "cuda:0"
    dims, S, nset = O.LLAMA2_7B, args.ctx, 8
    H, F = dims.hidden, dims.ffn
    g = torch.Generator().manual_seed(1)
    sets = []
    for i in range(nset):
        w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, S, seed=i)
        gu = (0.02 * torch.randn(2 * F, H, generator=g)).half().to(dev)
        dn = (0.02 * torch.randn(H, F, generator=g)).half().to(dev)
        sets.append(dict(x=x.to(dev), qkv=w["w_qkv"].to(dev), o=w["w_o"].to(dev), k=k.to(dev), v=v.to(dev), r1=w["rms1"].to(dev),
                         gu=gu, dn=dn, cos=cos.to(dev), sin=sin.to(dev)))

    def layer(a):
        return cf.llama_decoder_layer_full(a["x"], a["qkv"], a["o"], a["k"], a["v"], a["r1"], a["r1"], a["gu"], a["dn"], dims.eps,
                                           a["cos"], a["sin"], dims.heads)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for a in sets:
            layer(a)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [layer(a) for a in sets]
    for _ in range(max(1, args.warmup // nset)):
        graph.replay()
    torch.cuda.synchronize()
    reps = max(1, args.steps // nset)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (reps * nset)
    nbytes = 2 * (3 * H * H + H * H + 3 * F * H) + 2 * 2 * H + S * 2 * H * 2
    gbps = nbytes / (us * 1e-6) / 1e9
    result = {
        "metric": "layer_latency_us", "value": round(us, 2), "unit": "us/layer", "n_gpus": 1, "steps": reps * nset, "warmup": args.warmup,
        "ms_per_step": round(us * 1e-3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"llama2_7b decoder layer (attention block + SwiGLU MLP block, 2 launches), batch-1 decode, context {S}, "
                               "graph replay over 8 weight sets", "context": S, "hidden": H, "ffn": F},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "traffic": None, "kernel": "k_fused (attention block) + k_gated_mlp", "bytes_per_launch": nbytes,
                     "launch_us": round(us, 2)},
        "cpu_baseline": None}
    if emit:
        print(json.dumps(result), flush=True)
    return result


def bench_llama_batch(args, emit=True):
    """Extra workload (not the headline): the LLaMA-2-7B attention block for --batch sequences of --ctx cached tokens
    each over paged caches (the reference's llama_decoder_layer_batch_decode_sglang), pages scattered over the pool,
    six weight sets in turn so that every call reads HBM-cold weights."""
    import torch
    import clusterfusion as cf
    from oracle import neox_oracle as O      # geometry constants only
    dev = "cuda:0"
    dims, S, B, nset = O.LLAMA2_7B, args.ctx, args.batch, 6
    H, D = dims.hidden, dims.head_dim
    g = torch.Generator().manual_seed(2)
    ws = [((0.02 * torch.randn(3 * H, H, generator=g)).half().to(dev), (0.02 * torch.randn(H, H, generator=g)).half().to(dev))
          for _ in range(nset)]
    rms = (1 + 0.1 * torch.randn(H, generator=g)).half().to(dev)
    max_pos = S + 1
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(max_pos).float()[:, None] * inv[None, :]
    cos_sin = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).float().contiguous().to(dev)
    total = B * (S + 1)
    pool = total + 64
    ncache = 4 if B * S <= 32768 else 2
    caches = [(torch.randn(pool, H, generator=g).half().to(dev), torch.randn(pool, H, generator=g).half().to(dev)) for _ in range(ncache)]
    kptr = torch.tensor([a.data_ptr() for a, _ in caches], dtype=torch.uint64, device=dev)
    vptr = torch.tensor([b.data_ptr() for _, b in caches], dtype=torch.uint64, device=dev)
    indices = torch.randperm(pool, generator=g)[:total].to(torch.int32).to(dev)
    indptr = (torch.arange(B + 1) * (S + 1)).to(torch.int32).to(dev)
    pos = torch.full((B,), S, dtype=torch.int64, device=dev)
    x = torch.randn(B, H, generator=g).half().to(dev)
    res = torch.randn(B, H, generator=g).half().to(dev)
    out, res_out = torch.empty_like(x), torch.empty_like(x)

    def call(i):
        wq, wo = ws[i % nset]
        cf.llama_decoder_layer_batch_decode_sglang(out, res_out, x, res, wq, wo, indptr, indices, kptr, vptr, i % ncache, rms, dims.eps,
                                                   pos, cos_sin)
    for i in range(max(args.warmup, nset)):
        call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(args.steps):
        call(i)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / args.steps
    nbytes = 2 * 4 * H * H + 2 * H + B * S * 2 * H * 2
    gbps = nbytes / (us * 1e-6) / 1e9
    result = {
        "metric": "batch_step_latency_us", "value": round(us, 2), "unit": "us/call", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us * 1e-3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"llama2_7b attention block, {B} sequences x {S} cached tokens over paged caches (page = 1 token, "
                               f"scattered), {3 if B <= 16 else 4} launches per call", "batch": B, "context": S, "hidden": H,
                   "tokens_per_s_per_layer": round(B / (us * 1e-6))},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "traffic": None, "kernel": ("k_batch_mfma_pipe (add + norm + QKV) + k_batch_attn + k_batch_mfma_pipe (O)" if B <= 16 else
                                                  "k_batch_norm + k_batch_mfma_pipe (QKV) + k_batch_attn + k_batch_mfma_pipe (O)"),
                     "bytes_per_launch": nbytes, "launch_us": round(us, 2)},
        "cpu_baseline": None}
    if emit:
        print(json.dumps(result), flush=True)
    return result


def other_workloads(pkg, dev, args):
    """Short measurements of the other configurations, appended to the headline line (each is also a workload of its
    own: --model pythia_2b8 / llama2_7b_layer / llama2_7b_batch).  A failure is reported, not raised."""
    import copy
    import torch
    out = []

    def attempt(name, fn):
        try:
            out.append(fn())
        except Exception as e:     # noqa: BLE001
            log(f"[other_workloads] {name} failed: {type(e).__name__}: {e}")
            out.append({"workload": name, "error": f"{type(e).__name__}: {e}"})

    def stack_2b8():
        cfg, ctx, K, W = pkg.PYTHIA_2B8, 1024, 64, 8
        dec = build_model(cfg, 4096 + 64, ctx, dev, "fused")
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            dec.set_state(11, ctx)
            per_layer, _lm, _total = dec.profile_step()
            tpot = time_tokens(dec, stream, ctx, K, W)
            sweep = context_sweep(dec, cfg, stream, [2048, 4096])
        sb = step_bytes(cfg, ctx + W + K // 2)
        lay_us = sorted(per_layer)[len(per_layer) // 2] * 1e3
        first = {"context": ctx, "tokens": K, "tpot_ms": round(tpot, 4), "bytes": sb, "hbm_gbps": round(sb / (tpot * 1e-3) / 1e9, 1),
                 "frac_of_peak": round(sb / (tpot * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
        return {"workload": "pythia_2b8 full stack, batch-1 greedy decode, hipGraph replay, context 1024", "metric": "tpot_ms",
                "value": round(tpot, 4), "unit": "ms/token", "bytes": sb, "hbm_gbps": first["hbm_gbps"],
                "frac_of_peak": first["frac_of_peak"], "layer_kernel_us": round(lay_us, 2),
                "layer_kernel_frac_of_peak": round(layer_bytes(cfg, ctx + 1) / (lay_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                "sweep": [first] + sweep}

    def brief(r):
        return {"workload": r["config"]["workload"], "metric": r["metric"], "value": r["value"], "unit": r["unit"],
                "bytes": r["roofline"]["bytes_per_launch"], "hbm_gbps": r["roofline"]["achieved"], "frac_of_peak": r["roofline"]["frac"]}

    def llama_layer():
        a = copy.copy(args)
        a.ctx, a.steps, a.warmup = 4096, 64, 8
        return brief(bench_llama_layer(a, emit=False))

    def llama_batch():
        a = copy.copy(args)
        a.ctx, a.batch, a.steps, a.warmup = 1024, 16, 60, 12
        return brief(bench_llama_batch(a, emit=False))

    def single_layer(model, S, config_no):
        cfg = pkg.PYTHIA_2B8 if model == "pythia_2b8" else pkg.PYTHIA_6B9
        us = bench_single_layer(model, S)
        lb = layer_bytes(cfg, S)
        res = {"workload": f"BASELINE config {config_no}: one {model} decoder layer, batch 1, context {S}, graph replay over 8 weight "
                           "and cache sets (HBM-cold), fused and split ops", "metric": "layer_latency_us", "unit": "us/layer",
               "bytes": lb, "roofline_us": round(lb / (HBM_PEAK_GBPS * 1e9) * 1e6, 2)}
        for mode in ("fused", "split"):
            res[f"{mode}_us"] = round(us[mode], 2)
            res[f"{mode}_frac_of_peak"] = round(lb / (us[mode] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
        res["value"] = res["fused_us"]
        res["frac_of_peak"] = res["fused_frac_of_peak"]
        return res

    def stack_2b8_own_process():
        """The 2.8B stack as the workload of its own that it also is (`--model pythia_2b8 --ctx 1024`), in a process of its
        own: measured inside this process, after the 6.9B model, the sweeps and the per-layer contexts have come and gone,
        the same kernels on the same tensors read 2-3 % slower than in a fresh process (where its tensors end up in device
        memory).  Falls back to the measurement in this process when the child cannot be run."""
        import subprocess
        cmd = [sys.executable, os.path.abspath(__file__), "--model", "pythia_2b8", "--ctx", "1024", "--steps", "64", "--warmup", "8",
               "--no-cpu-baseline"]
        try:
            out_text = subprocess.run(cmd, capture_output=True, text=True, timeout=600, check=True).stdout
            r = json.loads([ln for ln in out_text.splitlines() if ln.startswith("{\"metric\"")][-1])
        except Exception as e:     # noqa: BLE001
            log(f"[other_workloads] pythia_2b8 in a process of its own failed ({type(e).__name__}: {e}); measuring in this process")
            return stack_2b8()
        return {"workload": "pythia_2b8 full stack, batch-1 greedy decode, hipGraph replay, context 1024 (measured in a process of its "
                            "own: python bench.py --model pythia_2b8 --ctx 1024)", "metric": "tpot_ms",
                "value": r["value"], "unit": "ms/token", "bytes": r["step"]["bytes"], "hbm_gbps": r["step"]["hbm_gbps"],
                "frac_of_peak": r["step"]["frac_of_peak"], "layer_kernel_us": r["roofline"]["layer_us"],
                "layer_kernel_frac_of_peak": r["roofline"]["frac"], "sweep": r.get("sweep"),
                "launch_per_layer_mode": r.get("launch_per_layer_mode"), "split_mode": r.get("split_mode")}

    attempt("pythia_2b8 single layer (config 1)", lambda: single_layer("pythia_2b8", 512, 1))
    torch.cuda.empty_cache()
    attempt("pythia_6b9 single layer (config 3)", lambda: single_layer("pythia_6b9", 2048, 3))
    torch.cuda.empty_cache()
    attempt("pythia_2b8 full stack", stack_2b8_own_process)
    torch.cuda.empty_cache()
    attempt("llama2_7b decoder layer", llama_layer)
    torch.cuda.empty_cache()
    attempt("llama2_7b paged batch", llama_batch)
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--model", default="pythia_6b9", choices=["pythia_6b9", "pythia_2b8", "llama2_7b_layer", "llama2_7b_batch"])
    ap.add_argument("--batch", type=int, default=16, help="sequences per call (llama2_7b_batch only)")
    ap.add_argument("--ctx", type=int, default=2048, help="KV-cache rows already filled when the timed region starts")
    ap.add_argument("--mode", default="fused", choices=["fused", "split", "fused_layers"],
                    help="fused: one launch per layer, or one for all layers where the device holds the whole grid; "
                         "fused_layers: one launch per layer in any case; split: one launch per stage")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-also", dest="also", action="store_false",
                    help="skip the context sweep, the drop-in per-layer loop and the short measurements of the other configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU (the hot path is a single-GPU batch-1 decode step); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import clusterfusionplus_amd as pkg
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = "cuda:0"
    if args.model == "llama2_7b_layer":
        if args.ctx == 2048:
            args.ctx = 4096          # the context this workload is quoted at
        return bench_llama_layer(args)
    if args.model == "llama2_7b_batch":
        if args.ctx == 2048:
            args.ctx = 1024
        return bench_llama_batch(args)
    cfg = pkg.PYTHIA_6B9 if args.model == "pythia_6b9" else pkg.PYTHIA_2B8
    K, W = args.steps, args.warmup
    extras = args.also and args.mode == "fused"
    sweep_ctx = {"pythia_6b9": [1024, 4096, 8192, 16384], "pythia_2b8": [1024, 2048, 4096]}[args.model]
    sweep_ctx = [c for c in sweep_ctx if c != args.ctx]
    rows = max(args.ctx + W + K, (max(sweep_ctx) + 28) if extras else 0) + 40
    t0 = time.perf_counter()
    dec = build_model(cfg, rows, args.ctx, dev, args.mode)
    torch.cuda.synchronize()
    log(f"[bench] built {args.model} ({cfg.n_layers} layers) in {time.perf_counter() - t0:.1f} s; cache rows {rows}")

    # a plain device-to-device copy of known size (256 MiB read + 256 MiB written): the reference point
    # that hardware-counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) are scaled by
    cal_src = torch.empty(128 << 20, dtype=torch.float16, device=dev).normal_()
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        dec.set_state(11, args.ctx)
        dec.graph_steps(W)                       # captures on first use; untimed warm-up replays
        stream.synchronize()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        dec.graph_steps(K)
        e1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        state = dec.state.cpu().tolist()
        assert state[1] == args.ctx + W + K, state
        # per-kernel durations with HIP events attached to the dispatches themselves (eager launches, same stream, the
        # positions of the timed region's first steps)
        dec.set_state(11, args.ctx + W)
        layer_ms, lm_ms = [], []
        for _ in range(5):
            per_layer, lm, _total = dec.profile_step()
            layer_ms.append(sum(per_layer) / len(per_layer))
            lm_ms.append(lm)
        S_prof = args.ctx + W + 3
    ev_ms = e0.elapsed_time(e1)
    tpot = wall_ms / K
    dec.check()                       # raises if any launch of the run raised a device-side failure flag

    S_mid = args.ctx + W + K // 2
    sb = step_bytes(cfg, S_mid)
    lb = layer_bytes(cfg, S_prof)
    lay_ms = sorted(layer_ms)[len(layer_ms) // 2]
    achieved = lb / (lay_ms * 1e-3) / 1e9
    # fused mode runs all layers in one launch where the device holds the whole grid: that launch is the dominant kernel
    per_launch = dec.layers_per_launch if args.mode == "fused" else 1
    if per_launch > 1:
        kernel_name = f"k_fused_stack (all {per_launch} decoder layers in one launch)"
    else:
        kernel_name = "k_fused (one decoder layer)" if args.mode != "split" else "stage A+B+C kernels (one decoder layer)"
    traffic, traffic_source = (None, None)
    if args.mode != "split":
        traffic, traffic_source = recorded_traffic(args.model, args.ctx, "k_fused_stack" if per_launch > 1 else "k_fused")
    result = {
        "metric": "tpot_ms", "value": round(tpot, 4), "unit": "ms/token", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(tpot, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{args.model} full stack: {cfg.n_layers} layers + final LN + LM head (vocab {cfg.vocab}), "
                               f"batch-1 greedy decode, hipGraph replay, context {args.ctx}",
                   "mode": args.mode, "context": args.ctx, "hidden": cfg.hidden, "ffn": cfg.ffn, "layers": cfg.n_layers},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": kernel_name, "layers_per_launch": per_launch,
                     "bytes_per_launch": lb * per_launch, "launch_us": round(lay_ms * 1e3 * per_launch, 2),
                     "bytes_per_layer": lb, "layer_us": round(lay_ms * 1e3, 2)},
        "step": {"bytes": sb, "hbm_gbps": round(sb / (tpot * 1e-3) / 1e9, 1),
                 "frac_of_peak": round(sb / (tpot * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                 "roofline_ms": round(sb / (HBM_PEAK_GBPS * 1e9) * 1e3, 4), "event_ms_per_step": round(ev_ms / K, 4),
                 "lm_head_us": round(sorted(lm_ms)[len(lm_ms) // 2] * 1e3, 1)},
    }
    if extras:
        with torch.cuda.stream(stream):
            result["sweep"] = [{"context": args.ctx, "tokens": K, "tpot_ms": round(tpot, 4), "bytes": sb,
                                "hbm_gbps": result["step"]["hbm_gbps"], "frac_of_peak": result["step"]["frac_of_peak"]}] + \
                context_sweep(dec, cfg, stream, sweep_ctx)
        result["sweep"].sort(key=lambda r: r["context"])
        try:
            # the same model with one launch per layer (CFPP_MODE_FUSED_LAYERS): what the one launch for all layers is worth
            ldec = pkg.NeoxDecoder(cfg, dec.tensors["layers"], dec.tensors["embed"], dec.tensors["final_ln_w"], dec.tensors["final_ln_b"],
                                   dec.tensors["lm_head"], dec.tensors["k_caches"], dec.tensors["v_caches"], mode="fused_layers")
            with torch.cuda.stream(stream):
                lt = time_tokens(ldec, stream, args.ctx, 32, 6)
            ldec.check()
            lsb = step_bytes(cfg, args.ctx + 6 + 16)
            result["launch_per_layer_mode"] = {"workload": f"{args.model} full stack, one fused launch per layer instead of one for all "
                                                           f"layers, hipGraph replay, context {args.ctx}", "context": args.ctx, "tokens": 32,
                                               "tpot_ms": round(lt, 4), "bytes": lsb, "hbm_gbps": round(lsb / (lt * 1e-3) / 1e9, 1),
                                               "frac_of_peak": round(lsb / (lt * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
            log(f"[launch per layer] context {args.ctx}: {lt:.4f} ms/token = {result['launch_per_layer_mode']['frac_of_peak'] * 100:.1f} % of peak")
            del ldec
        except Exception as e:     # noqa: BLE001
            log(f"[launch_per_layer_mode] failed: {type(e).__name__}: {e}")
            result["launch_per_layer_mode"] = {"error": f"{type(e).__name__}: {e}"}
        try:
            # the same model through the per-stage launches (CFPP_MODE_SPLIT), sharing the weights and caches
            sdec = pkg.NeoxDecoder(cfg, dec.tensors["layers"], dec.tensors["embed"], dec.tensors["final_ln_w"], dec.tensors["final_ln_b"],
                                   dec.tensors["lm_head"], dec.tensors["k_caches"], dec.tensors["v_caches"], mode="split")
            with torch.cuda.stream(stream):
                st = time_tokens(sdec, stream, args.ctx, 32, 6)
            sdec.check()
            ssb = step_bytes(cfg, args.ctx + 6 + 16)
            result["split_mode"] = {"workload": f"{args.model} full stack, split mode (one launch per stage instead of one per layer), "
                                                f"hipGraph replay, context {args.ctx}", "context": args.ctx, "tokens": 32,
                                    "tpot_ms": round(st, 4), "bytes": ssb, "hbm_gbps": round(ssb / (st * 1e-3) / 1e9, 1),
                                    "frac_of_peak": round(ssb / (st * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
            log(f"[split] context {args.ctx}: {st:.4f} ms/token = {result['split_mode']['frac_of_peak'] * 100:.1f} % of peak")
            del sdec
        except Exception as e:     # noqa: BLE001
            log(f"[split_mode] failed: {type(e).__name__}: {e}")
            result["split_mode"] = {"error": f"{type(e).__name__}: {e}"}
        try:
            result["drop_in_loop"] = drop_in_loop(args.model, cfg, dec, args.ctx)
            result["drop_in_loop"]["neox_decoder_tpot_ms"] = round(tpot, 4)
        except Exception as e:     # noqa: BLE001
            log(f"[drop_in_loop] failed: {type(e).__name__}: {e}")
            result["drop_in_loop"] = {"error": f"{type(e).__name__}: {e}"}
    if args.also and args.model == "pythia_6b9":
        del dec
        torch.cuda.empty_cache()
        result["other_workloads"] = other_workloads(pkg, dev, args)
    if not args.no_cpu_baseline:
        try:
            result["cpu_baseline"] = cpu_baseline(cfg, args.ctx)
        except Exception as e:
            log(f"[cpu_baseline] failed: {type(e).__name__}: {e}")
            result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
