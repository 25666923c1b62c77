"""Boundaries and failure reporting of the decode ops on the GPU: positions at the last cache row, a device-side
current_seq_len beyond the caches (the kernels flag it, clamp, do not append, and the next call reports it), the
whole-model decoder refusing to step past its caches, and scratch buffers that are never shared between two
geometries.  No test makes a kernel wait expire: every launch here exits normally."""
import pytest
import torch

from oracle import neox_oracle as O
from tests.test_gpu_layer_parity import assert_close, layer_args, make
from tests.test_gpu_context_and_stack import step_args, _tiny_stack

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cf():
    import clusterfusion
    return clusterfusion


def test_device_seq_len_at_the_last_row_and_beyond(cf):
    import clusterfusionplus_amd as pkg
    model, rows = "pythia_2b8", 24
    S = rows - 1
    print(f"\ncase {model} device seq_len = rows - 1, then rows", flush=True)
    dims, w, cpu, wg, gpu = make(model, S, capacity=rows, seed=31)
    x, k, v, _, _ = gpu
    cos_t, sin_t = pkg.rope_tables(rows, dims.rotary_dim, device="cuda:0")
    assert cf.device_status(True) == 0
    cf.pythia_2b8_create_graph_context(41, k, v, wg["w_qkv"], wg["w_o"], wg["w_up"], wg["w_down"], rows)
    seq = torch.tensor([S], dtype=torch.int32, device="cuda:0")
    out, kn, vn = cf.pythia_2b8_graph_decode_step(41, *step_args(wg, x, k, v, cos_t, sin_t), seq)
    torch.cuda.synchronize()
    assert cf.device_status() == 0
    ref = O.neox_layer_decode(cpu[0], w, cpu[1], cpu[2], cos_t[S:S + 1].cpu(), sin_t[S:S + 1].cpu(), S, dims)
    assert_close("output at the last row", out, ref["output"])
    assert torch.equal(k[S], kn.reshape(-1))
    # one position further there is no row to append to and no table row to read: flagged, nothing written
    k0, v0 = k.clone(), v.clone()
    seq.fill_(rows)
    cf.pythia_2b8_graph_decode_step(41, *step_args(wg, x, k, v, cos_t, sin_t), seq)
    torch.cuda.synchronize()
    assert torch.equal(k, k0) and torch.equal(v, v0)
    assert cf.device_status() & 2
    with pytest.raises(RuntimeError, match="failure flag"):
        cf.pythia_2b8_graph_decode_step(41, *step_args(wg, x, k, v, cos_t, sin_t), seq)
    assert cf.device_status() == 0                       # reported once, then cleared
    # the context's own status word still remembers it: destroy reports it too
    with pytest.raises(RuntimeError, match="failure flag"):
        cf.pythia_2b8_destroy_graph_context(41)
    assert cf.device_status(True) == 0
    # and the device works as before
    out2, _, _ = cf.pythia_2b8_decoder_layer(*layer_args(wg, x, k0.clone(), v0.clone(), cos_t[S:S + 1].contiguous(),
                                                         sin_t[S:S + 1].contiguous()), S)
    torch.cuda.synchronize()
    assert_close("output after the failure was cleared", out2, ref["output"])
    assert cf.check_workspace(x, dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn) == 0


def test_decoder_refuses_to_step_past_its_caches(cf):
    import clusterfusionplus_amd as pkg
    dims = O.PYTHIA_2B8
    L, V, rows, S = 2, 300, 12, 9
    print(f"\ncase stack bounds rows={rows} S={S}", flush=True)
    layers, embed, fw, fb, lm, kcs, vcs = _tiny_stack(L, V, rows, S, dims)
    dev = "cuda:0"
    cfg = pkg.NeoxConfig(dims.hidden, dims.heads, dims.head_dim, dims.rotary_dim, dims.ffn, L, V)
    dec = pkg.NeoxDecoder(cfg, [{n: t.to(dev) for n, t in w.items()} for w in layers], embed.to(dev), fw.to(dev), fb.to(dev),
                          lm.to(dev), [t.to(dev) for t in kcs], [t.to(dev) for t in vcs])
    with pytest.raises(RuntimeError):
        dec.set_state(3, rows)                           # the next step would append row `rows`
    dec.set_state(3, S)
    with pytest.raises(RuntimeError):
        dec.graph_steps(rows - S + 1)                    # one step too many: nothing is launched
    dec.graph_steps(rows - S)                            # exactly up to the last row
    torch.cuda.synchronize()
    assert dec.state.cpu().tolist()[1:3] == [rows, rows - S]
    with pytest.raises(RuntimeError):
        dec.step()
    with pytest.raises(RuntimeError):
        dec.graph_steps(1)
    assert len(dec.generated()) == rows - S              # generated() checks the stack's status word
    assert cf.device_status() == 0


def test_scratch_is_not_shared_between_geometries(cf):
    """Same hidden size, different head counts (and the Pythia-6.9B op in between, whose scratch has the same hidden
    and ffn): every geometry gets its own zero-initialised buffer."""
    dev = "cuda:0"
    print("\ncase scratch per geometry: hidden 4096 with 32 / 64 / 32 heads", flush=True)

    def llama(heads, seed):
        dims = O.LlamaDims(hidden=4096, heads=heads, head_dim=4096 // heads, ffn=0)
        w, x, res, k, v, cos, sin = O.make_llama_attn_inputs(dims, 70, seed=seed)
        ref = O.llama_attention_sglang(x, res, w, k, v, cos, sin, dims)
        out, _, kn, _ = cf.llama_decoder_layer_sglang(x.to(dev), res.to(dev), w["w_qkv"].to(dev), w["w_o"].to(dev), k.to(dev), v.to(dev),
                                                      w["rms1"].to(dev), dims.eps, cos.to(dev), sin.to(dev), heads)
        torch.cuda.synchronize()
        assert_close(f"output, {heads} heads", out, ref["output"])
        assert_close(f"k_new, {heads} heads", kn, ref["k_new"])

    llama(32, 1)
    dims, w, cpu, wg, gpu = make("pythia_6b9", 50, seed=2)
    out, _, _ = cf.pythia_6b9_decoder_layer(*layer_args(wg, *gpu), 50)
    torch.cuda.synchronize()
    assert_close("pythia_6b9 output", out, O.neox_layer_decode(cpu[0], w, *cpu[1:], 50, dims)["output"])
    llama(64, 3)
    llama(32, 4)
    assert cf.device_status() == 0
