"""Whole-step parity: forward + backward of a small dense model on the GPU step driver against the CPU oracle's
orc_model_step (the reference's ComputeBackprop, src/gpt/compute/cpu_transformer.cpp:128-198), fed identical quantised weights.
Tolerances are per tensor, relative to its rms / maximum; they are set by the 8-bit storage of states (1/24 steps) and gradients."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
from model_harness import E4M3, I8, Harness, rel_err  # noqa: E402


def check_model(h, tol_state, tol_grad, tol_delta):
    failures = []

    def expect(cond, what):
        if not cond:
            failures.append(what)
    h.oracle_step()
    m = h.device_model()
    try:
        m.backprop()
        torch.cuda.synchronize()
        st = m.array("state").float().cpu().numpy()[:h.n]
        rms, mx = rel_err(st, h.states[-1])
        print("final state rel err rms/max", rms, mx)
        expect(rms <= tol_state, 'state')
        g0 = m.array("stateGrad").float().cpu().numpy()[:h.n]
        rms, mx = rel_err(g0, h.ref_grad0)
        print("embedding-level state gradient rel err rms/max", rms, mx)
        expect(rms <= tol_grad, 'stateGrad')
        loss = m.loss_sum() / (h.target >= 0).sum()
        print("loss", loss, h.ref_loss)
        expect(abs(loss - h.ref_loss) <= 2e-3 * abs(h.ref_loss), 'loss')
        worst = 0
        for d in range(h.depth):
            for i, q in enumerate(h.layers[d]):
                got = m.get_delta(d, i, *q.fast.shape)
                rms, mx = rel_err(got, h.ref_delta[d][i])
                worst = max(worst, rms)
                print(f"layer {d} type {h.lt[d]} matrix {i}: delta rel err rms/max {rms:.4f} {mx:.4f}")
                expect(rms <= tol_delta, ('delta', d, i))
        got = m.get_delta(-2, 0, h.vocab, h.dim)
        rms, mx = rel_err(got, h.ref_delta_final)
        print("final layer delta rel err", rms, mx)
        expect(rms <= tol_delta, 'final delta')
        got = m.get_delta(-1, 0, h.label_count, h.dim)
        rms, mx = rel_err(got, h.ref_delta_embed)
        print("embedding delta rel err", rms, mx)
        expect(rms <= tol_grad, 'embed delta')
        print("worst layer delta rms rel err", worst)
        assert not failures, failures
    finally:
        m.close()


def test_tiny_dense_int8_step():
    """BASELINE config[0]: e256 h2 d4 ffn8 w64 (8 layers), byte vocab, 8 fragments of 64 tokens, weights N(0, 0.02)"""
    print("case tiny dense int8", flush=True)
    h = Harness(I8, dim=256, heads=2, ffn_tiles=8, depth=4, vocab=256, frag_count=8, frag_len=64, wide_window=64, seed=3)
    check_model(h, tol_state=4e-2, tol_grad=5e-2, tol_delta=1e-1)


def test_tiny_dense_int8_step_sharp_attention():
    print("case tiny dense int8 sharp", flush=True)
    h = Harness(I8, dim=256, heads=2, ffn_tiles=4, depth=2, vocab=256, frag_count=3, frag_len=100, wide_window=64, seed=4, std=0.05, k_std=1.0)
    check_model(h, tol_state=4e-2, tol_grad=5e-2, tol_delta=1e-1)


def test_tiny_dense_fp8_step():
    print("case tiny dense fp8", flush=True)
    h = Harness(E4M3, dim=256, heads=2, ffn_tiles=8, depth=4, vocab=256, frag_count=8, frag_len=64, wide_window=64, seed=5)
    check_model(h, tol_state=5e-2, tol_grad=1.5e-1, tol_delta=2e-1)
