"""What storing W and the momentum in fp16 only costs against the reference's fp32 master weights and
fp32 optimizer state (dl_base.py:185, main.py:178-179), and that the layer's `master_weights` mode is
the reference's regime.

The CPU part emulates both storage regimes over a few hundred steps of a small problem with the
reference's kind of schedule (lr1 = 0.0025, cosine with warm-up from 0, dl_base.py:397): every step's
arithmetic is the oracle's fp32 update; the fp16-resident regime rounds W and M to fp16 after each step
(what xfc_dw_update stores), the master regime rounds only the copy the GEMMs read.  It records how many
updates the fp16 store drops (|lr * M| below half an ulp of W) and bounds the drift of the trained
weights."""
import math

import pytest
import torch

from oracle import xfc_oracle as O
from renee_amd import cosine_schedule_with_warmup, synth


def _run(regime: str, steps: int, B=64, L=2048, d=64, base_lr=0.0025, mu=0.9, seed=3):
    X_all = [synth.make_X(B, d, seed + s) for s in range(8)]
    P_all = [synth.make_positives(B, L, 8, 2.3, 1.1, seed + s).coo() for s in range(8)]
    W = synth.make_W(L, d, seed)               # fp32 master, N(0, 0.02)
    M = torch.zeros_like(W)
    if regime == "fp16":
        W = W.half().float()
    dropped = total = 0
    for s in range(steps):
        lr = cosine_schedule_with_warmup(s, steps // 10, steps, base_lr)
        X = X_all[s % 8].half().float()
        px, py = P_all[s % 8]
        W16 = W.half().float()                 # what the GEMMs read in either regime
        G = O.grad_logits(O.logits(X, W16), px, py).half().float()
        dW = O.dw(G, X)
        W_new, M_new = O.sgd_momentum(W, M, dW, lr, mu, 0.0)
        if regime == "fp16":
            M_new = M_new.half().float()
            W_st = (W - lr * M_new).half().float()   # fp32 arithmetic, one rounding on store
            moved = (lr * M_new).abs() > 0
            dropped += int(((W_st == W) & moved).sum())
            total += int(moved.sum())
            W_new = W_st
        W, M = W_new, M_new
    return W, M, dropped / max(total, 1)


def test_fp16_resident_weights_drop_small_updates_and_master_weights_do_not():
    steps = 300
    W_ref, M_ref, _ = _run("fp32", steps)      # the reference's regime = the oracle's fp32 state
    W_16, M_16, dropped = _run("fp16", steps)
    rel = lambda a, b: float((a - b).norm() / b.norm())
    moved_ref = float((W_ref - synth.make_W(2048, 64, 3)).norm())
    drift = float((W_16 - W_ref).norm())
    print(f"fp16-resident after {steps} steps at lr1=0.0025: {dropped:.1%} of the non-zero updates left W unchanged; "
          f"|W16 - Wref| / |Wref - W0| = {drift / moved_ref:.3f}; rel(W) = {rel(W_16, W_ref):.2e}; rel(M) = {rel(M_16, M_ref):.2e}")
    # the effect exists and is bounded: a visible share of the updates is lost, yet the trained weights stay
    # within a few per cent of the distance the reference regime has moved them
    assert dropped > 0.02
    assert drift / moved_ref < 0.10
    assert rel(M_16, M_ref) < 2e-2


def test_half_ulp_rule():
    """An update below half an ulp of the stored fp16 weight is lost; the same update applied to an fp32
    master accumulates and surfaces in the fp16 copy later."""
    w0 = torch.tensor([0.02], dtype=torch.float16)
    ulp = 2.0 ** -16                                     # fp16 spacing in [2^-6, 2^-5)
    step = 0.3 * ulp
    w16, w32 = w0.clone(), w0.float().clone()
    for _ in range(10):
        w16 = (w16.float() - step).half()
        w32 = w32 - step
    assert float(w16) == float(w0)                       # every one of the ten updates was rounded away
    assert abs(float(w32.half()) - (float(w0) - 10 * step)) <= ulp / 2
    assert float(w32.half()) != float(w0)


@pytest.mark.gpu
def test_master_weights_mode_follows_the_fp32_oracle_where_fp16_resident_stalls(dev):
    """50 steps with lr * |M| below half an fp16 ulp of |W| for most weights: the fp32-master layer tracks
    the fp32 oracle, the fp16-resident layer barely moves (its deviation is recorded, not hidden)."""
    from renee_amd import XFCLayer

    B, L, d, steps, lr, mu = 64, 4096, 64, 50, 2e-5, 0.9
    W0 = synth.make_W(L, d, 9)
    Xs = [synth.make_X(B, d, 20 + s).half() for s in range(4)]
    Ps = [synth.make_positives(B, L, 8, 2.3, 1.1, 20 + s).coo() for s in range(4)]
    master = XFCLayer(L, d, B, dev, lr=lr, momentum=mu, weight=W0, master_weights=True)
    resident = XFCLayer(L, d, B, dev, lr=lr, momentum=mu, weight=W0)
    Wo, Mo = W0.clone(), torch.zeros(L, d)
    for s in range(steps):
        X, (px, py) = Xs[s % 4], Ps[s % 4]
        for lay in (master, resident):
            lay.fwd_grad(X.to(dev), px, py)
            lay.dx(B)
            lay.dw_update(X.to(dev))
        G = O.grad_logits(O.logits(X.float(), Wo.half().float()), px, py).half().float()
        Wo, Mo = O.sgd_momentum(Wo, Mo, O.dw(G, X.float()), lr, mu, 0.0)
    torch.cuda.synchronize()
    rel = lambda a, b: float((a.double().cpu() - b.double()).norm() / b.double().norm())
    moved = Wo - W0
    m_err = float((master.xfc_weight_master.cpu() - Wo).norm() / moved.norm())
    r_err = float((resident.xfc_weight.float().cpu() - Wo).norm() / moved.norm())
    print(f"after {steps} steps at lr={lr}: error / distance moved: master {m_err:.3e}, fp16-resident {r_err:.3e}; "
          f"rel(M) master {rel(master.momentum_buffer, Mo):.2e} resident {rel(resident.momentum_buffer, Mo):.2e}")
    assert master.xfc_weight_master.dtype == torch.float32 and master.momentum_buffer.dtype == torch.float32
    assert m_err <= 1e-2                                  # the master follows the oracle's trajectory
    assert rel(master.momentum_buffer, Mo) <= 1e-3
    assert torch.equal(master.xfc_weight, master.xfc_weight_master.half())   # the fp16 copy is the master, rounded
    assert r_err > 10 * m_err                             # ...where the fp16-resident weights visibly lag
