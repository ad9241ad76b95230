"""Pins oracle/xfc_oracle.py against things it was not derived from: float64
brute force, autograd of the reference's own baseline loss, torch.optim.SGD,
sorting, closed forms, and the committed golden vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import xfc_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _tiny(B=5, L=11, d=7, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(B, d, generator=g, dtype=dtype)
    W = torch.randn(L, d, generator=g, dtype=dtype) * 0.3
    return X, W


def test_logits_dx_dw_bruteforce():
    X, W = _tiny()
    B, d = X.shape
    L = W.shape[0]
    Z = O.logits(X, W)
    G = torch.randn(B, L, dtype=torch.float64)
    dX, dW = O.dx(G, W, 3.0), O.dw(G, X)
    for b in range(B):
        for l in range(L):
            assert abs(Z[b, l] - sum(X[b, k] * W[l, k] for k in range(d))) < 1e-12
    for b in range(B):
        for k in range(d):
            assert abs(dX[b, k] - 3.0 * sum(G[b, l] * W[l, k] for l in range(L))) < 1e-12
    for l in range(L):
        for k in range(d):
            assert abs(dW[l, k] - sum(G[b, l] * X[b, k] for b in range(B))) < 1e-12
    # a transposed operand or a dropped scale would not survive these
    assert not torch.allclose(O.dx(G, W, 3.0), O.dx(G, W, 1.0))
    assert torch.allclose(O.dw(G, X, acc=dW), 2 * dW)


def test_grad_matches_autograd_of_bce_sum():
    X, W = _tiny(B=6, L=13, d=5, seed=1)
    pos_x = torch.tensor([0, 0, 2, 5, 5, 5])
    pos_y = torch.tensor([1, 12, 0, 3, 4, 12])
    Y = torch.zeros(6, 13, dtype=torch.float64)
    Y[pos_x, pos_y] = 1.0
    Xp, Wp = X.clone().requires_grad_(True), W.clone().requires_grad_(True)
    Z = Xp @ Wp.t()
    Z.retain_grad()
    torch.nn.BCEWithLogitsLoss(reduction="sum")(Z, Y).backward()  # dl_base.py:171,282-283
    r = O.step(X, W, torch.zeros_like(W), pos_x, pos_y, lr=0.1, momentum=0.9, scale=5.0)
    assert torch.allclose(r["G"], Z.grad, atol=1e-12)
    assert torch.allclose(r["dW"], Wp.grad, atol=1e-12)
    assert torch.allclose(r["dX"], 5.0 * Xp.grad, atol=1e-12)
    # closed form and sign invariants
    z = O.logits(X, W)
    assert torch.allclose(r["G"], 1 / (1 + torch.exp(-z)) - Y, atol=1e-12)
    assert ((r["G"] < 0) == (Y > 0)).all()
    assert (r["G"].abs() < 1).all()


def test_positive_set_semantics_on_duplicates():
    Z = torch.zeros(2, 4, dtype=torch.float64)
    G = O.grad_logits(Z.clone(), torch.tensor([0, 0, 0, 1]), torch.tensor([2, 2, 2, 0]))
    expect = torch.full((2, 4), 0.5, dtype=torch.float64)
    expect[0, 2] = -0.5  # listed three times, lowered once
    expect[1, 0] = -0.5
    assert torch.equal(G, expect)
    assert torch.equal(O.grad_logits(Z.clone(), torch.zeros(0, dtype=torch.long), torch.zeros(0, dtype=torch.long)),
                       torch.full((2, 4), 0.5, dtype=torch.float64))


@pytest.mark.parametrize("wd", [0.0, 1e-2])
def test_sgd_momentum_matches_torch_optim(wd):
    torch.manual_seed(3)
    W0 = torch.randn(9, 4, dtype=torch.float64)
    grads = [torch.randn(9, 4, dtype=torch.float64) for _ in range(4)]
    p = torch.nn.Parameter(W0.clone())
    opt = torch.optim.SGD([p], lr=0.05, momentum=0.9, weight_decay=wd)
    W, M = W0.clone(), torch.zeros_like(W0)
    for g in grads:
        p.grad = g.clone()
        opt.step()
        W, M = O.sgd_momentum(W, M, g, 0.05, 0.9, wd)
        assert torch.allclose(W, p.detach(), atol=1e-13)
        assert torch.allclose(M, opt.state[p]["momentum_buffer"], atol=1e-13)
    # closed form, steps 1 and 2, wd = 0
    W1, M1 = O.sgd_momentum(W0, torch.zeros_like(W0), grads[0], 0.05, 0.9)
    W2, M2 = O.sgd_momentum(W1, M1, grads[1], 0.05, 0.9)
    assert torch.allclose(M1, grads[0]) and torch.allclose(W1, W0 - 0.05 * grads[0])
    assert torch.allclose(M2, 0.9 * grads[0] + grads[1])
    assert torch.allclose(W2, W0 - 0.05 * grads[0] - 0.05 * (0.9 * grads[0] + grads[1]))
    # lr = 0 (first step of a warm-up schedule) still advances the momentum
    W3, M3 = O.sgd_momentum(W0, torch.zeros_like(W0), grads[0], 0.0, 0.9)
    assert torch.equal(W3, W0) and torch.allclose(M3, grads[0])


def test_step_uses_old_weights_for_dx():
    X, W = _tiny(seed=4)
    px, py = torch.tensor([1]), torch.tensor([2])
    r = O.step(X, W, torch.zeros_like(W), px, py, lr=0.5, momentum=0.9)
    assert torch.allclose(r["dX"], r["G"] @ W)
    assert not torch.allclose(r["dX"], r["G"] @ r["W"])


def test_step_accum_equals_step():
    X, W = _tiny(B=7, L=9, d=4, seed=5)
    # rows 0-2 | 3-5 | 6 ; pos_x local to each micro-batch (dl_base.py:939-959)
    px_full = torch.tensor([0, 2, 3, 3, 6])
    py = torch.tensor([1, 8, 0, 4, 2])
    px_local = torch.tensor([0, 2, 0, 0, 0])
    index = torch.tensor([0, 2, 4, 5])
    a = O.step(X, W, torch.zeros_like(W), px_full, py, 0.05, 0.9, 1e-3, 2.0)
    b = O.step_accum(X, W, torch.zeros_like(W), px_local, py, index, 3, 0.05, 0.9, 1e-3, 2.0)
    for k in ("dX", "dW", "W", "M"):
        assert torch.allclose(a[k], b[k], atol=1e-12), k


def test_topk_against_sort_and_tie_rule():
    X, W = _tiny(B=8, L=40, d=6, seed=6, dtype=torch.float32)
    v, i = O.topk(X, W, 5)
    Z = O.logits(X, W)
    sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
    assert torch.equal(v, sv[:, :5]) and torch.equal(i, si[:, :5])
    v7, i7 = O.topk(X, W, 7)  # K > 5 goes through torch.topk
    assert torch.equal(v7, sv[:, :7])
    # exact ties: lowest label id first
    Xt = torch.zeros(1, 2)
    Xt[0, 0] = 1.0
    Wt = torch.tensor([[0.5, 0], [0.9, 0], [0.9, 0], [0.1, 0], [0.9, 0], [0.5, 0]])
    v, i = O.topk(Xt, Wt, 5)
    assert i.tolist() == [[1, 2, 4, 0, 5]]
    # padded labels are clamped (dl_base.py:782)
    v, i = O.topk(Xt, Wt, 5, numy=3)
    assert i.tolist() == [[1, 2, 2, 0, 2]]


def test_xfc_gemm_modes():
    torch.manual_seed(7)
    B, L, d = 6, 10, 4
    X, W = torch.randn(B, d), torch.randn(L, d) * 0.3
    out = torch.full((B, L), float("nan"))
    O.xfc_gemm(X, W.t(), out, 1.0, 0.0, True)  # dl_base.py:591
    assert torch.allclose(out, torch.sigmoid(O.logits(X, W)), atol=1e-6)
    G = out.clone()
    grad = torch.full((L, d), float("nan"))
    O.xfc_gemm(G.t(), X, grad, 1.0, 0.0, False)  # dl_base.py:623, beta = 0 never reads out
    assert torch.allclose(grad, O.dw(G, X), atol=1e-5)
    O.xfc_gemm(G.t(), X, grad, 1.0, 1.0, False)  # dl_base.py:629
    assert torch.allclose(grad, 2 * O.dw(G, X), atol=1e-5)
    gi = torch.empty(B, d)
    O.xfc_gemm(G, W, gi, 4.0, 0.0, False)  # dl_base.py:604
    assert torch.allclose(gi, O.dx(G, W, 4.0), atol=1e-5)
    with pytest.raises(RuntimeError):
        O.xfc_gemm(X, W.t().contiguous(), out, 1.0, 0.0, True)  # row x row is not a sigmoid mode
    with pytest.raises(RuntimeError):
        O.xfc_gemm(X.unsqueeze(0), W.t(), out, 1.0, 0.0, True)


def test_sampled_loss_is_bce_sum():
    X, W = _tiny(B=4, L=9, d=3, seed=8, dtype=torch.float32)
    px, py = torch.tensor([0, 1, 3]), torch.tensor([2, 2, 8])
    Y = torch.zeros(4, 9)
    Y[px, py] = 1
    Z = O.logits(X, W) * 5
    want = torch.nn.BCEWithLogitsLoss(reduction="sum")(Z, Y)
    assert torch.allclose(O.sampled_loss(Z, px, py), want, rtol=1e-5)


def test_pad_numy():
    assert O.pad_numy(131073) == 131088          # LF-AmazonTitles-131K on one GPU
    assert O.pad_numy(2812281) == 2812288
    assert O.pad_numy(131072) == 131072
    assert O.pad_numy(100, 8) == 128             # 100 -> 104 (x8) -> 13/GPU -> 16/GPU
    assert O.pad_numy(1310720, 4) == 1310720


def test_golden_vectors():
    z = np.load(os.path.join(GOLD, "xfc_step_small.npz"))
    lr, mu, wd, scale = [float(v) for v in z["hyper"]]
    X, W = torch.from_numpy(z["X"]), torch.from_numpy(z["W0"])
    px, py = torch.from_numpy(z["pos_x"]), torch.from_numpy(z["pos_y"])
    M = torch.zeros_like(W)
    for s in (1, 2):
        r = O.step(X, W, M, px, py, lr, mu, wd, scale)
        for k in ("G", "dW", "dX", "W", "M"):
            assert np.allclose(r[k].numpy(), z[f"{k}{s}"], atol=1e-12), (k, s)
        loss = O.sampled_loss(O.logits(X, W), *torch.unique(torch.stack([px, py]), dim=1))
        assert abs(float(loss) - float(z[f"loss{s}"])) < 1e-3 * abs(float(z[f"loss{s}"]))
        W, M = r["W"], r["M"]
