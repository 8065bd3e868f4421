"""Pins the same-contract CPU model (tests/same_contract.py) without a GPU: its quantisers against the oracle's scalar converters and
torch's bfloat16, and its whole step against the fp32 oracle step - the two differ by the 8-bit storage noise only, which is unbiased:
per tensor the least-squares scale is 1 within 6e-3 and the correlation at least 0.995.  A dropped term, a wrong factor or a
transposed operand in the model fails these the same way it would in the device code."""
import numpy as np
import pytest

from model_harness import E4M3, I8, Harness, rel_err, scale_fit
from oracle_lib import Oracle
from same_contract import SameContract, bf16, e4m3, e4m3_numpy, f16


def test_quantisers_of_the_model_match_the_scalar_converters():
    orc = Oracle()
    r = np.random.default_rng(0)
    tab = orc.e4m3_table(hw=True)
    pos = np.sort(np.unique(np.abs(tab[np.isfinite(tab) & ((np.arange(256) & 0x7f) != 0x7f)])))
    mids = (pos[1:] + pos[:-1]) / 2
    x = np.concatenate([r.standard_normal(2000) * s for s in (1e-3, 0.02, 1, 30, 300)] + [pos, -pos, mids, -mids, [0.0, 448, 464, 465, 1e9, -1e9]])
    x = x.astype(np.float32)
    want = np.array([tab[orc.lib.orc_cvt_e4m3_rne(float(v))] for v in x], np.float32)
    assert np.array_equal(e4m3(x), want) and np.array_equal(e4m3_numpy(x), want)
    torch = pytest.importorskip("torch")
    y = (r.standard_normal(5000) * 10.0 ** r.integers(-10, 10, 5000)).astype(np.float32)
    assert np.array_equal(bf16(y), torch.from_numpy(y).bfloat16().float().numpy())
    assert np.array_equal(f16(y[np.abs(y) < 6e4]), torch.from_numpy(y[np.abs(y) < 6e4]).half().float().numpy())


@pytest.mark.parametrize("mode", [I8, E4M3])
def test_same_contract_step_is_the_oracle_step_plus_unbiased_storage_noise(mode):
    h = Harness(mode, dim=256, heads=2, ffn_tiles=4, depth=2, vocab=256, frag_count=4, frag_len=64, wide_window=64, seed=9, bias_std=0.5)
    h.oracle_step()
    s = SameContract(h).run()
    assert abs(s.loss - h.ref_loss) <= 2e-3 * abs(h.ref_loss)
    pairs = [("state", s.state, h.states[-1]), ("stateGrad", s.state_grad, h.ref_grad0), ("final", s.delta_final, h.ref_delta_final),
             ("embed", s.delta_embed, h.ref_delta_embed)]
    for d in range(h.depth):
        for i in range(len(h.layers[d])):
            pairs.append((("delta", d, i), s.delta[d][i], h.ref_delta[d][i]))
    for what, got, ref in pairs:
        rms, _ = rel_err(got, ref)
        fit, corr = scale_fit(got, ref)
        # e4m3 fast gradients flush what lies more than 17 binary orders below their maximum: a slight shrink (measured down to 0.9936)
        assert rms <= 0.12 and abs(fit - 1) <= (6e-3 if mode == I8 else 1e-2) and corr >= 0.995, (what, rms, fit, corr)


def test_same_contract_moe_step_follows_the_oracle_step():
    """attention + MoE (e4m3): the model's MoE layer against the fp32 oracle's.  Looser than the dense case: besides the storage noise a
    few per cent of the tokens pick another expert once their select logits come from 8-bit states"""
    h = Harness(E4M3, dim=256, heads=2, ffn_tiles=2, depth=1, vocab=256, frag_count=4, frag_len=96, wide_window=64, experts=8, selected=2, xp=256,
                seed=16, std=0.05)
    h.oracle_step()
    s = SameContract(h).run()
    assert abs(s.loss - h.ref_loss) <= 2e-3 * abs(h.ref_loss)
    pairs = [("state", s.state, h.states[-1]), ("stateGrad", s.state_grad, h.ref_grad0), ("final", s.delta_final, h.ref_delta_final)]
    for d in range(h.depth):
        for i in range(len(h.layers[d])):
            pairs.append((("delta", d, i), s.delta[d][i], h.ref_delta[d][i]))
    for what, got, ref in pairs:
        rms, _ = rel_err(got, ref)
        fit, corr = scale_fit(got, ref)
        assert rms <= 0.25 and abs(fit - 1) <= 2e-2 and corr >= 0.97, (what, rms, fit, corr)
