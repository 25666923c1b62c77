"""Phase timeline of the fused decoder-layer kernel inside a whole-model decode step.

Needs a profiling build of the HIP library, kept at a path of its own (it never replaces the product library): its
fused kernel stores a 100 MHz timestamp per wave at every phase boundary.  This script loads that build before the
package (both carry the same library name, so the binding resolves to the one already loaded), runs a synthetic model
of the given shape, records one eager step, and prints per phase the median over the layers of the mean / earliest /
latest time (microseconds from the kernel's first wave) over all workgroups.  Run it as a script, not with -m (the
package import would load the product library first):

    python -m clusterfusionplus_amd.build --trace-lib /tmp/libcfpp_trace.so
    python clusterfusionplus_amd/phase_trace.py --trace-lib /tmp/libcfpp_trace.so --model pythia_2b8 --ctx 1024

With --stack the step goes through the launch that runs all layers of the model (the whole-model decoder's own path):
the same table per layer of that launch, and the hand-over from layer to layer inside it.
"""
import argparse
import ctypes
import os
import sys

import numpy as np
import torch

if __package__ in (None, ""):            # run as a script: make the package importable, but do not import it yet
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def load_trace_library(path):
    """Loads the profiling build globally, before anything has loaded the product library."""
    if "clusterfusionplus_amd" in sys.modules:
        raise RuntimeError("the package is already imported (its product library is loaded): run this file as a script, "
                           "python clusterfusionplus_amd/phase_trace.py --trace-lib PATH ...")
    lib = ctypes.CDLL(os.path.abspath(path), mode=ctypes.RTLD_GLOBAL)
    if not hasattr(lib, "cfpp_debug_set_trace"):
        raise RuntimeError(f"{path} is not a profiling build (python -m clusterfusionplus_amd.build --trace-lib PATH)")
    return lib

# slot -> (label, which waves report it)
SLOTS = [(0, "kernel entry", "all"), (14, "LayerNorm inputs and first weight tile requested", "all"), (15, "own chunk of the input row arrived", "all"),
         (1, "LayerNorm done", "all"), (2, "own QKV rows stored, QKV arrival counted", "streaming"),
         (2, "own QKV rows stored, QKV arrival counted", "attention"),
         (3, "QKV event seen, attention item begins", "attention"), (8, "item's q back and rotated (cache items)", "attention"),
         (11, "item's partial published, head counter answered", "attention"),
         (4, "attention item done (head merged by its last split)", "attention"),
         (12, "own MLP-up phase 0 rows stored", "streaming"), (5, "own MLP-up phase 1 rows stored", "streaming"),
         (6, "MLP-up phase 0 event seen (down phase 0 may read)", "streaming"), (13, "MLP-up phase 1 event seen (down phase 1 may read)", "streaming"),
         (7, "heads event seen (O rows may read)", "attention"), (9, "stage C begins", "all"), (10, "stage C done: rows reduced and stored", "all")]


def synthetic_decoder(cfg, rows, device):
    from clusterfusionplus_amd import NeoxDecoder
    torch.manual_seed(0)
    H, F = cfg.hidden, cfg.ffn

    def rn(shape, std, mean=0.0):
        return torch.empty(shape, dtype=torch.float16, device=device).normal_(mean, std)
    layers = [{"ln_w": rn((H,), 0.02, 1.0), "ln_b": rn((H,), 0.01), "w_qkv": rn((3 * H, H), 0.02), "b_qkv": rn((3 * H,), 0.01),
               "w_o": rn((H, H), 0.02), "b_o": rn((H,), 0.01), "post_ln_w": rn((H,), 0.02, 1.0), "post_ln_b": rn((H,), 0.01),
               "w_up": rn((F, H), 0.02), "b_up": rn((F,), 0.01), "w_down": rn((H, F), 0.02), "b_down": rn((H,), 0.01)}
              for _ in range(cfg.n_layers)]
    return NeoxDecoder(cfg, layers, rn((cfg.vocab, H), 1.0), rn((H,), 0.02, 1.0), rn((H,), 0.01), rn((cfg.vocab, H), 0.02),
                       [rn((rows, H), 1.0) for _ in range(cfg.n_layers)], [rn((rows, H), 1.0) for _ in range(cfg.n_layers)])


def main():
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--trace-lib", required=True, metavar="PATH", help="the profiling build of the HIP library to load")
    ap.add_argument("--model", default="pythia_6b9", choices=["pythia_6b9", "pythia_2b8", "llama2_7b_attention"])
    ap.add_argument("--ctx", type=int, default=2048)
    ap.add_argument("--raw", help="also save the raw timestamps of every layer ([layer][workgroup][wave][slot]) as .npy")
    ap.add_argument("--stack", action="store_true",
                    help="trace the launch that runs all layers of the model (one eager step): the phases of every layer, "
                         "and how the rows pass from layer to layer inside the launch")
    a = ap.parse_args()
    load_trace_library(a.trace_lib)
    from clusterfusionplus_amd import PYTHIA_2B8, PYTHIA_6B9, debug_set_trace
    dev = "cuda:0"
    if a.model == "llama2_7b_attention":
        return llama_attention(a, dev)
    cfg = PYTHIA_6B9 if a.model == "pythia_6b9" else PYTHIA_2B8
    dec = synthetic_decoder(cfg, a.ctx + 64, dev)
    dec.set_state(11, a.ctx)
    for _ in range(3):
        dec.step()
    torch.cuda.synchronize()
    lay, _lm, _tot = dec.profile_step()
    if a.stack:
        return stack_launch(a, dec, cfg, lay, dev)
    print(f"{a.model}, context {a.ctx}: fused layer kernel {np.median(lay) * 1e3:.1f} us (median of {len(lay)} layers, HIP events, "
          "profiling build)")
    # the trace buffer holds one launch: record the layers of one step one at a time through the per-layer op
    tr = torch.zeros(1024 * 16 * 16, dtype=torch.int64, device=dev)
    debug_set_trace(tr)          # raises unless the library is a profiling build
    per_layer = []
    import clusterfusionplus_amd as pkg
    op = pkg.neox_decoder_layer
    # re-run single layers with their own weights (cold: 32 different weight sets in turn)
    x = torch.randn(1, cfg.hidden, device=dev).half()
    cos, sin = dec.cos[a.ctx:a.ctx + 1].contiguous(), dec.sin[a.ctx:a.ctx + 1].contiguous()
    for l, w in enumerate(dec._layers):
        tr.zero_()
        op(cfg.hidden, cfg.heads, cfg.head_dim, cfg.rotary_dim, cfg.ffn, cfg.eps, False, x, w["w_qkv"], w["b_qkv"], w["w_o"], w["b_o"],
           dec._k_caches[l], dec._v_caches[l], w["ln_w"], w["ln_b"], cos, sin, w["post_ln_w"], w["post_ln_b"], w["w_up"], w["b_up"],
           w["w_down"], w["b_down"], a.ctx)
        torch.cuda.synchronize()
        per_layer.append(tr.cpu().numpy().reshape(1024, 16, 16)[:256, :8].astype(np.float64))
    debug_set_trace(None)
    if a.raw:
        np.save(a.raw, np.stack(per_layer))
    report(per_layer[2:])
    return 0


def stack_launch(a, dec, cfg, lay, dev):
    """One eager step through the launch that runs all layers; layer l stamps into block l of the trace buffer."""
    from clusterfusionplus_amd import debug_set_trace
    L = cfg.n_layers
    if dec.layers_per_launch != L:
        raise RuntimeError("this stack runs one launch per layer (see NeoxDecoder.layers_per_launch): nothing to trace with --stack")
    print(f"{a.model}, context {a.ctx}: all {L} layers in one launch, {sum(lay) * 1e3:.0f} us = {np.mean(lay) * 1e3:.1f} us per layer "
          "(HIP events, profiling build)")
    block = 1024 * 16 * 16
    tr = torch.zeros(L * block, dtype=torch.int64, device=dev)
    debug_set_trace(tr)
    dec.step()
    torch.cuda.synchronize()
    debug_set_trace(None)
    dec.step()                       # (the table forgets the buffer before it is freed)
    torch.cuda.synchronize()
    raw = tr.cpu().numpy().reshape(L, 1024, 16, 16)[:, :256, :8].astype(np.float64)
    if a.raw:
        np.save(a.raw, raw)
    report(list(raw[2:]))
    # the hand-over: from the last output row of layer l to the norm of layer l + 1
    def stamps(l, slot):
        v = raw[l][:, :, slot]
        return v[v > 0]
    rows = []
    for l in range(2, L - 1):
        done = stamps(l, 10)                 # stage C done, per wave
        end = done.max()
        seen, norm, entry = stamps(l + 1, 14), stamps(l + 1, 1), stamps(l + 1, 0)
        rows.append(((end - done.min()) / 100, (np.median(done) - end) / 100, (np.median(entry) - end) / 100, (entry.max() - end) / 100,
                     (np.median(seen) - end) / 100, (seen.max() - end) / 100, (np.median(norm) - end) / 100, (norm.max() - end) / 100))
    m = np.median(np.array(rows), axis=0)
    print("hand-over between layers (us relative to the moment the last wave of layer l has stored its output rows; median over layers)")
    print(f"  first wave of layer l done                                         {-m[0]:8.2f}")
    print(f"  median wave of layer l done                                        {m[1]:8.2f}")
    print(f"  layer l+1 entered (median / last wave)                             {m[2]:8.2f} {m[3]:8.2f}")
    print(f"  layer l complete seen, input row requested (median / last wave)    {m[4]:8.2f} {m[5]:8.2f}")
    print(f"  norm of layer l+1 done (median / last wave)                        {m[6]:8.2f} {m[7]:8.2f}")
    return 0


def llama_attention(a, dev):
    """The LLaMA-2-7B attention block (fused add + RMSNorm, QKV, attention, O: the fused kernel without an MLP) over eight
    weight sets in turn."""
    import clusterfusion as cf
    from clusterfusionplus_amd import debug_set_trace
    H, heads, S = 4096, 32, a.ctx
    torch.manual_seed(0)

    def rn(shape, std, mean=0.0):
        return torch.empty(shape, dtype=torch.float16, device=dev).normal_(mean, std)
    sets = [(rn((3 * H, H), 0.02), rn((H, H), 0.02), rn((S + 1, H), 1.0), rn((S + 1, H), 1.0), rn((H,), 0.02, 1.0)) for _ in range(8)]
    x, res = rn((1, H), 1.0), rn((1, H), 1.0)
    ang = torch.rand(1, 64, device=dev) * 6.28
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1).float(), torch.cat([ang.sin(), ang.sin()], -1).float()
    tr = torch.zeros(1024 * 16 * 16, dtype=torch.int64, device=dev)
    debug_set_trace(tr)
    per_launch = []
    for it in range(24):
        wq, wo, k, v, rms = sets[it % 8]
        tr.zero_()
        cf.llama_decoder_layer_sglang(x, res.clone(), wq, wo, k[:S], v[:S], rms, 1e-5, cos, sin, heads)
        torch.cuda.synchronize()
        per_launch.append(tr.cpu().numpy().reshape(1024, 16, 16)[:256, :8].astype(np.float64))
    debug_set_trace(None)
    if a.raw:
        np.save(a.raw, np.stack(per_launch))
    print(f"llama2_7b attention block, context {S}: phase stamps of the fused kernel (profiling build)")
    report(per_launch[8:])
    return 0


def report(launches):
    rows = {}
    for raw in launches:
        t0 = raw[:, :, 0][raw[:, :, 0] > 0].min()
        us = (raw - t0) / 100.0
        for slot, label, who in SLOTS:
            sl = {"all": slice(0, 8), "streaming": slice(0, 4), "attention": slice(4, 8)}[who]
            col = us[:, sl, slot][raw[:, sl, slot] >= t0]        # waves that do not pass a boundary leave its slot at zero
            if col.size:
                rows.setdefault((slot, who), []).append((col.mean(), col.min(), np.percentile(col, 50), col.max()))
    print(f"{'phase boundary (us from the first wave; median over layers of ...)':84s} {'mean':>7s} {'first':>7s} {'median':>7s} {'last':>7s}")
    for slot, label, who in SLOTS:
        if (slot, who) in rows:
            m = np.median(np.array(rows[(slot, who)]), axis=0)
            print(f"{label + ' [' + who + ' waves]':84s} {m[0]:7.2f} {m[1]:7.2f} {m[2]:7.2f} {m[3]:7.2f}")


if __name__ == "__main__":
    sys.exit(main())
