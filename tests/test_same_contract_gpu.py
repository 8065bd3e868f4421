"""Device layers against the same-contract CPU model (tests/same_contract.py: the oracle's arithmetic with a rounding at every point
where the device stores a tensor in 8 or 16 bits), layer by layer on the device's own stored inputs.  Inside an attention layer the
attention core (bf16 probabilities on the device, fp32 in the model) is compared on its own - output and the three gradients within
1e-2 - and the model then continues from the device's copies, so that the rest of the layer is compared on identical inputs too.

Why per layer: the 8-bit rounding of the residual state turns the 1e-3 differences an attention layer legitimately has (bf16
probabilities on the device, fp32 in the model) into flipped codes - about 2 % of the codes after one attention layer, a quarter after
four - so a whole step run twice end to end differs by the storage noise itself, however exact each layer is.  Given the same stored
inputs (the layer's 8-bit input and tile scales, the incoming fp32 state gradient) nothing chaotic is left, and the contract's tolerance
applies: the state increment, the outgoing state gradient and every packed delta within 1e-2 of the tensor's maximum.  The whole step is
compared with the fp32 oracle statistically (unbiased scale, correlation) in test_model_gpu.py."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from model_harness import E4M3, I8, Harness, rel_err, scale_fit  # noqa: E402
from same_contract import SameContract, rep  # noqa: E402

TOL_MAX = 1e-2   # max |device - model| / max |model| per tensor
TOL_RMS = 5e-3   # rms of the difference / rms of the tensor
# e4m3 mode: the MFMA fp32 accumulation carries about 4e-5 relative noise (the int8 sums are exact), which flips about 1 % of the bf16
# activations by an ulp and through them about 0.1 % of the e4m3 codes (steps of 6 %): isolated elements that inherit one flipped code.
# The contract stays 1e-2 of the tensor's maximum; what is allowed beyond it is counted: at most 0.2 % of a tensor's elements may exceed
# it, none may exceed 3e-2 (one flipped code of a large element; two would), and the rms and the scale fit must not move.
TOL_MAX_E4M3 = 3e-2
TOL_OUTLIERS_E4M3 = 2e-3
TOL_RMS_E4M3 = 8e-3


def dev_values(h, raw):
    return raw.astype(np.float32) if h.mode == I8 else h.orc.e4m3_table(hw=True)[raw]


def check_layers(h, k_tile=0):
    s = SameContract(h, k_tile)
    m = h.device_model(k_tile=k_tile)
    bad = []
    tol_max_layer = TOL_MAX if h.mode == I8 else TOL_MAX_E4M3
    tol_rms_layer = TOL_RMS if h.mode == I8 else TOL_RMS_E4M3
    Q = h.heads * 128

    def f32(name, index, cols):
        return m.array(name, index).float().cpu().numpy()[:h.n, :cols]

    def cmp(what, got, ref, tol_max=TOL_MAX, tol_rms=TOL_RMS):
        rms, mx = rel_err(got, ref)
        fit, _ = scale_fit(got, ref)
        # elements beyond the contract's 1e-2 of the maximum (only the e4m3 layers' tensors are allowed any)
        over = float((np.abs(got.astype(np.float64) - ref) > TOL_MAX * (np.abs(ref).max() + 1e-30)).mean())
        print(f"{what}: rms {rms:.2e} max {mx:.2e} beyond 1e-2: {over:.2e} fit {fit:.6f}", flush=True)
        if not (mx <= tol_max and rms <= tol_rms and abs(fit - 1) <= 1e-3 and over <= (TOL_OUTLIERS_E4M3 if tol_max > TOL_MAX else 0)):
            bad.append((what, rms, mx, over, fit))
    try:
        m.backprop()  # a real step: realistic state and state gradient to feed every layer with
        torch.cuda.synchronize()
        n, depth = h.n, h.depth
        state = m.array("state"); sgrad = m.array("stateGrad"); gmax = m.array("gradMaxNorm")
        S = state.clone(); G = sgrad.clone()
        Sh = S.cpu().numpy()[:n]; Gh = G.cpu().numpy()[:n]
        # ---- final layer on the device's own last norm state
        fn8 = dev_values(h, m.read("normState", depth)[:n]); fsc = np.ascontiguousarray(m.read("stateScale", depth)[:, :n].T)
        sim_n8, sim_sc = s.normalize_state(Sh)
        print("final norm state: codes that differ", float((sim_n8 != fn8).mean()), flush=True)
        assert (sim_n8 != fn8).mean() < 1e-3 and np.abs(sim_sc - fsc).max() <= 1e-5 * fsc.max()
        s.final_backward(fn8, fsc)
        loss = m.loss_sum() / (h.target >= 0).sum()
        print("loss", loss, s.loss)
        if abs(loss - s.loss) > 2e-4 * abs(s.loss):
            bad.append(("loss", loss, s.loss))
        cmp("soft-max gradient", m.array("finalGrad").float().cpu().numpy()[:n, :h.vocab], s.grad_v, tol_rms=3e-3)
        cmp("final delta", m.get_delta(-2, 0, h.vocab, h.dim), s.delta_final)
        cmp("embed delta", m.get_delta(-1, 0, h.label_count, h.dim), s.embedding_delta(Gh), tol_max=1e-5, tol_rms=1e-5)
        # ---- every layer in isolation, forward and backward, on the same inputs
        for d in range(depth):
            state.copy_(S)
            m.layer_forward(d)
            torch.cuda.synchronize()
            add = (state - S).cpu().numpy()[:n]
            n8 = dev_values(h, m.read("normState", d)[:n]); sc = np.ascontiguousarray(m.read("stateScale", d)[:, :n].T)
            assert (sim_n8 != n8).mean() < 1e-3
            tag = f"layer {d} type {int(h.lt[d])}"
            att = int(h.lt[d]) == 0
            if att:
                s.force[d] = {"val16": f32("act.val", d, Q)}
            sim_add = s.layer_forward(d, n8)
            if att:
                cmp(tag + " attention output", s.force[d]["val16"], s.core["val16"])
            cmp(tag + " state increment", add, sim_add, tol_max=tol_max_layer, tol_rms=tol_rms_layer)
            sgrad.copy_(G)
            gmax[0, 0] = G[:n].abs().max()
            m.layer_backward(d)
            torch.cuda.synchronize()
            if att:
                s.force[d].update(dq=f32("act.val", d, Q), dk=f32("scratch.g2", Q, Q), dv=f32("scratch.g3", Q, Q))
            sim_grad = s.layer_backward(d, n8, sc, Gh)
            if att:
                cmp(tag + " dVal into the attention backward", f32("scratch.g1", Q, Q), s.core["dval16"], tol_max=tol_max_layer, tol_rms=tol_rms_layer)
                for nm in ("dq", "dk", "dv"):
                    cmp(tag + " attention " + nm, s.force[d][nm], s.core[nm])
            cmp(tag + " outgoing state gradient", sgrad.cpu().numpy()[:n], sim_grad, tol_max=tol_max_layer, tol_rms=tol_rms_layer)
            for i, q in enumerate(h.layers[d]):
                cmp(tag + f" delta {i}", m.get_delta(d, i, *q.fast.shape), s.delta[d][i], tol_max=tol_max_layer, tol_rms=tol_rms_layer)
        assert not bad, bad
    finally:
        m.close()


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_layers_same_contract(mode):
    print("case same contract per layer: 2 attention + 2 ffn layers (window 1 / 64, slopes 0 / 0.5)", mode, flush=True)
    check_layers(Harness(mode, dim=256, heads=2, ffn_tiles=4, depth=2, vocab=256, frag_count=4, frag_len=64, wide_window=64, seed=9, bias_std=0.5))


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_layers_same_contract_sharp_attention(mode):
    print("case same contract per layer: sharp attention, large vocabulary bias", mode, flush=True)
    check_layers(Harness(mode, dim=256, heads=2, ffn_tiles=4, depth=1, vocab=256, frag_count=3, frag_len=100, wide_window=64, seed=4, std=0.05,
                         k_std=1.0, bias_std=1.0))


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_layers_same_contract_large_tile_branches(mode):
    """8192 tokens, dim 512, 4 heads, ffn 2048: the 256x256 ring kernel with the fused normalise / RoPE epilogue, the token-axis
    slices of the small deltas, the stacked Q/K/V/gate delta and the grouped dX products all run inside the layer backward here"""
    print("case same contract per layer: large-tile branches", mode, flush=True)
    check_layers(Harness(mode, dim=512, heads=4, ffn_tiles=16, depth=1, vocab=256, frag_count=16, frag_len=512, wide_window=512, seed=12))


def test_layers_same_contract_moe():
    """the reference's depth-3 schedule with experts (att ffn att ffn att moe att moe), expert width 256: each MoE layer alone on the
    device's own stored input - routing, gather, grouped expand / gate / contract products, combine, the gate and norm backward over
    grouped rows, routing backward, grouped dX products and the per-expert deltas - against the model that rounds where the device does.
    Both sides route from the same 8-bit input, so they pick the same experts (the fp32 oracle does not: a few per cent of the tokens
    change experts under 8-bit state noise, which is why the whole-step comparison of MoE models is loose)"""
    print("case same contract per layer: MoE", flush=True)
    check_layers(Harness(E4M3, dim=256, heads=2, ffn_tiles=2, depth=3, vocab=256, frag_count=4, frag_len=96, wide_window=64, experts=8,
                         selected=2, xp=256, seed=16, std=0.05))


def test_layers_same_contract_moe_64_experts_width_512():
    """the expert count and expert width of the MoE benchmark (64 experts, top-2, width 512 = four norm tiles per expert slab, which
    runs the second pass of the gate / norm backward's tile loop and 64-way routing tables), on 768 tokens: 8192 grouped rows"""
    print("case same contract per layer: MoE, 64 experts x 512", flush=True)
    check_layers(Harness(E4M3, dim=512, heads=4, ffn_tiles=4, depth=3, vocab=256, frag_count=4, frag_len=192, wide_window=64, experts=64,
                         selected=2, xp=512, seed=17, std=0.05))
