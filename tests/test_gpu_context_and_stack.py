"""GPU tests of the decode contexts (create / graph_decode_step / destroy), the whole-model decoder
(eager steps and hipGraph replays) and the LM head, against the CPU oracle."""
import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import MODELS, assert_close, layer_args, make

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cf():
    import clusterfusion
    return clusterfusion


def step_args(wg, x, k, v, cos, sin):
    return [x, wg["ln_w"], wg["ln_b"], wg["b_qkv"], wg["b_o"], cos, sin, k, v,
            wg["post_ln_w"], wg["post_ln_b"], wg["b_up"], wg["b_down"]]


@pytest.mark.parametrize("model,S", [("pythia_2b8", 512), ("pythia_6b9", 333)])
def test_graph_decode_step_equals_decoder_layer(cf, model, S):
    print(f"\ncase {model} graph context S={S}", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, capacity=S + 4, seed=21)
    x, k, v, cos, sin = gpu
    k2, v2 = k.clone(), v.clone()
    ref_out, ref_k, ref_v = getattr(cf, f"{model}_decoder_layer")(*layer_args(wg, x, k2, v2, cos, sin), S)
    create = getattr(cf, f"{model}_create_graph_context")
    step = getattr(cf, f"{model}_graph_decode_step")
    destroy = getattr(cf, f"{model}_destroy_graph_context")
    create(7, k, v, wg["w_qkv"], wg["w_o"], wg["w_up"], wg["w_down"], S + 4)
    out, kn, vn = step(7, *step_args(wg, x, k, v, cos, sin), S)
    torch.cuda.synchronize()
    assert torch.equal(out, ref_out) and torch.equal(kn, ref_k) and torch.equal(vn, ref_v)
    assert torch.equal(k, k2) and torch.equal(v, v2)
    # the returned tensors are the context's static buffers: the next step overwrites them
    # (reference pythia_kernel_dispatch_graph.cu:286; callers clone, tests/benchmark_decode.py:266-267)
    keep = out.clone()
    x2 = (x.float() * 0.5).half()
    out2, _, _ = step(7, *step_args(wg, x2, k, v, cos, sin), S + 1)
    torch.cuda.synchronize()
    assert out2.data_ptr() == out.data_ptr() and not torch.equal(out, keep)
    # a second context id has its own buffers
    create(8, k, v, wg["w_qkv"], wg["w_o"], wg["w_up"], wg["w_down"], S + 4)
    out3, _, _ = step(8, *step_args(wg, x, k, v, cos, sin), S)
    torch.cuda.synchronize()
    assert out3.data_ptr() != out.data_ptr() and torch.equal(out3, keep)
    destroy(7)
    destroy(8)
    destroy(8)          # unknown id: no-op, as in the reference (graph.cu:292-294)
    with pytest.raises(RuntimeError, match="not initialized"):
        step(7, *step_args(wg, x, k, v, cos, sin), S)


def test_graph_decode_step_replays_from_a_captured_graph(cf):
    """Device-resident seq_len + rope tables: one captured graph serves consecutive positions."""
    model, S0, n = "pythia_2b8", 40, 3
    print(f"\ncase {model} torch.cuda.graph replay", flush=True)
    dims, w, cpu, wg, gpu = make(model, S0, capacity=S0 + 8, seed=22)
    x, k, v, _, _ = gpu
    import clusterfusionplus_amd as pkg
    cos_t, sin_t = pkg.rope_tables(S0 + 8, dims.rotary_dim, device="cuda:0")
    seq = torch.tensor([S0], dtype=torch.int32, device="cuda:0")
    xin = x.clone()
    cf.pythia_2b8_create_graph_context(31, k, v, wg["w_qkv"], wg["w_o"], wg["w_up"], wg["w_down"], S0 + 8)
    args = lambda: step_args(wg, xin, k, v, cos_t, sin_t)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        cf.pythia_2b8_graph_decode_step(31, *args(), seq)      # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    k_eager, v_eager = k.clone(), v.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out, kn, vn = cf.pythia_2b8_graph_decode_step(31, *args(), seq)
    # eager reference on separate caches, position by position
    k_ref, v_ref = k_eager.clone(), v_eager.clone()
    for i in range(n):
        S = S0 + i
        seq.fill_(S)
        xin.copy_((x.float() * (1.0 + 0.1 * i)).half())
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        cos, sin = cos_t[S:S + 1].contiguous(), sin_t[S:S + 1].contiguous()
        want, _, _ = cf.pythia_2b8_decoder_layer(*layer_args(wg, xin, k_ref, v_ref, cos, sin), S)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i}"
        assert torch.equal(k[S], k_ref[S]) and torch.equal(v[S], v_ref[S])
    cf.pythia_2b8_destroy_graph_context(31)


def test_argument_errors_raise(cf):
    model, S = "pythia_2b8", 16
    print(f"\ncase {model} argument validation", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, seed=23)
    x, k, v, cos, sin = gpu
    good = layer_args(wg, x, k, v, cos, sin)
    op = cf.pythia_2b8_decoder_layer

    def bad(i, t, match):
        a = list(good)
        a[i] = t
        with pytest.raises(RuntimeError, match=match):
            op(*a, S)

    bad(0, x.float(), "float16")                              # wrong dtype
    bad(0, x.cpu(), "GPU")                                    # CPU tensor
    bad(1, wg["w_qkv"][:-1], "elements")                      # wrong element count
    bad(1, wg["w_qkv"].t(), "contiguous")                     # non-contiguous
    bad(9, cos.half(), "float32")                             # rope dtype
    bad(5, k[:, :-8], "contiguous|shape")                     # cache shape
    with pytest.raises(RuntimeError, match="exceeds"):
        op(*good, S + 5)                                      # seq_len beyond the cache rows
    with pytest.raises(RuntimeError, match=">= 0"):
        op(*good, -1)
    with pytest.raises(RuntimeError):
        cf.pythia_6b9_decoder_layer(*good, S)                 # 2.8B tensors into the 6.9B op
    with pytest.raises(RuntimeError, match="max_seq_len"):
        cf.pythia_2b8_create_graph_context(1, k, v, wg["w_qkv"], wg["w_o"], wg["w_up"], wg["w_down"], S + 100)
    torch.cuda.synchronize()


def _tiny_stack(L, V, rows, S, dims):
    g = torch.Generator().manual_seed(5)
    layers = [O.make_layer_weights(dims, layer=i, w_std=0.02, b_std=0.01) for i in range(L)]
    embed = torch.randn((V, dims.hidden), generator=g).half()
    lm = (torch.randn((V, dims.hidden), generator=g) * 0.02).half()
    fw = (1 + 0.02 * torch.randn(dims.hidden, generator=g)).half()
    fb = (0.01 * torch.randn(dims.hidden, generator=g)).half()
    kcs = [torch.randn((rows, dims.hidden), generator=g).half() for _ in range(L)]
    vcs = [torch.randn((rows, dims.hidden), generator=g).half() for _ in range(L)]
    for t in kcs + vcs:
        t[S:] = 1e4      # rows the decoder has not written yet must never be read
    return layers, embed, fw, fb, lm, kcs, vcs


@pytest.mark.parametrize("model,mode", [("pythia_2b8", "fused"), ("pythia_2b8", "split"), ("pythia_6b9", "fused")])
def test_stack_decode_matches_oracle(cf, model, mode):
    """3 layers + final LN + LM head: eager step, then hipGraph replays, against the oracle stack."""
    import clusterfusionplus_amd as pkg
    dims = MODELS[model]
    L, V, rows, S = 3, 1000, 48, 20
    print(f"\ncase {model} stack {mode} L={L} V={V} S={S}", flush=True)
    layers, embed, fw, fb, lm, kcs, vcs = _tiny_stack(L, V, rows, S, dims)
    dev = "cuda:0"
    cfg = pkg.NeoxConfig(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, L, V)
    g_layers = [{n: t.to(dev) for n, t in w.items()} for w in layers]
    g_k, g_v = [t.to(dev) for t in kcs], [t.to(dev) for t in vcs]
    dec = pkg.NeoxDecoder(cfg, g_layers, embed.to(dev), fw.to(dev), fb.to(dev), lm.to(dev), g_k, g_v, mode=mode)
    # fused mode runs the model's layers in one launch on a device that holds the whole grid; split mode never does
    assert dec.layers_per_launch == (L if mode == "fused" else 1)
    tok = 17
    dec.set_state(tok, S)
    o_k, o_v = [t.clone() for t in kcs], [t.clone() for t in vcs]
    seq = S
    for step in range(4):
        ref = O.neox_stack_decode(tok, embed, layers, fw, fb, lm, o_k, o_v, seq, dims)
        if step == 0:
            dec.step()              # eager launches
        else:
            dec.graph_steps(1)      # captured once, then replayed
        torch.cuda.synchronize()
        logits = dec.logits.clone()
        cs = float(torch.nn.functional.cosine_similarity(logits.cpu().double(), ref["logits"].double(), dim=0))
        err = float((logits.cpu() - ref["logits"].float()).abs().max())
        print(f"  step {step}: logits max-abs {err:.3e} cosine {cs:.7f}", flush=True)
        assert cs >= 0.9999 and err <= 2e-2
        assert_close("hidden", dec.hidden, ref["hiddens"][-1])
        st = dec.state.cpu().tolist()
        # greedy pick == argmax of the device logits (ties broken towards the lower index)
        assert st[0] == int(torch.argmax(logits)) and st[1] == seq + 1 and st[2] == step + 1
        for l in range(L):
            assert_close(f"k_cache[{l}][{seq}]", g_k[l][seq], o_k[l][seq])
            assert torch.equal(g_k[l][seq + 1:].cpu(), kcs[l][seq + 1:])   # later rows untouched
        # keep the oracle on the device's token so both walk the same path
        tok = st[0]
        seq += 1
    assert len(dec.generated()) == 4


@pytest.mark.parametrize("model,L", [("pythia_2b8", 1), ("pythia_2b8", 2), ("pythia_6b9", 5), ("pythia_160m", 3)])
def test_layers_in_one_launch_equal_layers_in_launches_of_their_own(cf, model, L):
    """The launch that runs all layers of a stack hands rows from layer to layer inside the launch; one launch per layer
    (fused_layers) and the per-stage launches (split mode) hand them over at launch boundaries.  Same arithmetic: logits, hidden state, picks and cache rows must be
    equal bit for bit, for one layer (no hand-over), two, and more, over several tokens (eager, then graph replays)."""
    import clusterfusionplus_amd as pkg
    dims = MODELS[model] if model in MODELS else O.NeoxDims(hidden=768, heads=12, head_dim=64, rotary_dim=16, ffn=3072)
    V, rows, S, N = 500, 40, 9, 5
    print(f"\ncase one launch == per stage, {model} L={L}", flush=True)
    layers, embed, fw, fb, lm, kcs, vcs = _tiny_stack(L, V, rows, S, dims)
    dev = "cuda:0"
    cfg = pkg.NeoxConfig(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, L, V)
    g_layers = [{n: t.to(dev) for n, t in w.items()} for w in layers]
    out = {}
    for mode in ("fused", "fused_layers", "split"):
        g_k, g_v = [t.to(dev) for t in kcs], [t.to(dev) for t in vcs]
        dec = pkg.NeoxDecoder(cfg, g_layers, embed.to(dev), fw.to(dev), fb.to(dev), lm.to(dev), g_k, g_v, mode=mode)
        if mode == "fused":
            # hidden sizes that are not whole 512-column chunks (768) keep one launch per layer
            assert dec.layers_per_launch == (L if dims.hidden % 512 == 0 else 1)
        else:
            assert dec.layers_per_launch == 1
        dec.set_state(3, S)
        seen = []
        for step in range(N):
            if step == 0:
                dec.step()
            else:
                dec.graph_steps(1)
            torch.cuda.synchronize()
            seen.append((dec.logits.clone(), dec.hidden.clone()))
        dec.check()
        out[mode] = (seen, dec.generated(), [t.clone() for t in g_k], [t.clone() for t in g_v])
    for other in ("fused_layers", "split"):
        assert out["fused"][1] == out[other][1]
        for (la, ha), (lb, hb) in zip(out["fused"][0], out[other][0]):
            assert torch.equal(la, lb) and torch.equal(ha, hb)
        for a, b in zip(out["fused"][2] + out["fused"][3], out[other][2] + out[other][3]):
            assert torch.equal(a, b)


def test_lm_head_matches_torch(cf):
    print("\ncase lm_head", flush=True)
    g = torch.Generator().manual_seed(9)
    H, V = 4096, 3001
    x = torch.randn(1, H, generator=g).half()
    w = (torch.randn(V, H, generator=g) * 0.02).half()
    lw = (1 + 0.02 * torch.randn(H, generator=g)).half()
    lb = (0.01 * torch.randn(H, generator=g)).half()
    got = cf.lm_head(x.cuda(), lw.cuda(), lb.cuda(), w.cuda(), 1e-5).cpu()
    want = torch.nn.functional.layer_norm(x.float(), (H,), lw.float(), lb.float(), 1e-5) @ w.float().t()
    assert_close("logits", got, want.reshape(-1))
