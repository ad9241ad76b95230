"""Parity of the HIP path (called through the C ABI) with the CPU oracle on the
same seeded inputs.  The oracle receives the fp16-rounded X and W upcast to
fp32, so input quantisation is not charged to the kernels.

Tolerance (stated by the task): relative Frobenius error <= 1e-3 on G, dW and
dX; the same bound is used for W and M after the update (one fp16 rounding of
each per step)."""
import os

import numpy as np
import pytest
import torch

from oracle import xfc_oracle as O
from renee_amd import XFCLayer, coo_to_csr, synth, xfc_gemm
from renee_amd._lib import XfcError

pytestmark = pytest.mark.gpu
TOL = 1e-3
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def rel(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm())


def worst(a, b):
    """Largest single error as a fraction of the largest reference magnitude.  The Frobenius norm hides a few
    wrong rows or columns in a large matrix (seven wrong label rows of 3001 stay under 1e-3); this does not."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


def _problem(B, L, d, kmax=8, kmean=2.3, zipf=1.1, seed=0):
    X = synth.make_X(B, d, seed).half()
    W = synth.make_W(L, d, seed).half()
    P = synth.make_positives(B, L, kmax, kmean, zipf, seed)
    return X, W, P


def _check_step(dev, X, W, px, py, lr=0.05, mu=0.9, wd=0.0, scale=1.0, steps=1, csr=None):
    B, d = X.shape
    L = W.shape[0]
    lay = XFCLayer(L, d, B, dev, lr=lr, momentum=mu, weight_decay=wd, weight=W)
    Xd = X.to(dev)
    Wo, Mo = W.float(), torch.zeros(L, d)
    for s in range(steps):
        print(f"step {s}: B={B} L={L} d={d} nnz={len(px)}", flush=True)
        ref = O.step(X.float(), Wo, Mo, px, py, lr, mu, wd, scale)
        if csr is not None:
            G = lay.fwd_grad(Xd, rowptr=csr[0].to(dev), colidx=csr[1].to(dev))
        else:
            G = lay.fwd_grad(Xd, px.to(dev), py.to(dev))
        assert rel(G, ref["G"]) <= TOL
        assert float((G.float().cpu() - ref["G"]).abs().max()) <= 1e-3   # |G| < 1: half an fp16 step is 2.4e-4
        if L % 8:  # the pad columns up to the next multiple of 8 are written as zero
            assert float(lay.outsoft[:B, L:(L + 7) // 8 * 8].abs().max()) == 0.0
        # every positive is negative in G, everything else is in (0, 1)
        Gc = G.float().cpu()
        mask = torch.zeros(B, L, dtype=torch.bool)
        if len(px):
            ok = (px >= 0) & (px < B) & (py >= 0) & (py < L)
            mask[px[ok], py[ok]] = True
        assert (Gc[mask] <= 0).all() and (Gc[~mask] >= 0).all()
        dX = lay.dx(B, scale=scale)
        assert rel(dX, ref["dX"]) <= TOL and worst(dX, ref["dX"]) <= 5e-3
        dW = torch.empty(L, d, device=dev, dtype=torch.float32)
        lay.dw_update(Xd, dW_out=dW)
        assert rel(dW, ref["dW"]) <= TOL and worst(dW, ref["dW"]) <= 5e-3
        # update parity is judged from the same starting point: the oracle is advanced from the
        # device's fp16 state so that per-step rounding does not compound in the comparison
        assert rel(lay.xfc_weight, ref["W"]) <= TOL and worst(lay.xfc_weight, ref["W"]) <= 3e-3
        assert rel(lay.momentum_buffer, ref["M"]) <= TOL and worst(lay.momentum_buffer, ref["M"]) <= 3e-3
        Wo, Mo = lay.xfc_weight.float().cpu(), lay.momentum_buffer.float().cpu()
    return lay


def test_cfg0_shape(dev):
    c = synth.CONFIGS[0]
    X, W, P = _problem(c["B"], c["L"], 768, c["kmax"], c["kmean"], c["zipf"])
    px, py = P.coo()
    _check_step(dev, X, W, px, py, steps=2)


def test_cfg1_shape_csr(dev):
    c = synth.CONFIGS[1]
    X, W, P = _problem(c["B"], c["L"], 768, c["kmax"], c["kmean"], c["zipf"], seed=1)
    px, py = P.coo()
    _check_step(dev, X, W, px, py, csr=(torch.from_numpy(P.rowptr), torch.from_numpy(P.colidx)), scale=4096.0)


@pytest.mark.parametrize("B,L,d", [(1, 9, 8), (7, 1000, 64), (100, 4097, 128), (264, 12345, 384), (513, 2049, 1024),
                                   (512, 8313, 768)])
def test_ragged_shapes(dev, B, L, d):
    X, W, P = _problem(B, L, d, seed=B)
    px, py = P.coo()
    _check_step(dev, X, W, px, py, wd=1e-3, scale=3.0)


def test_adversarial_label_sets(dev):
    B, L, d = 300, 1000 + 121, 64
    X, W, _ = _problem(B, L, d, seed=9)
    rows, cols = [], []
    rows += [5, 5, 5]; cols += [17, 17, 17]                  # duplicated pair counts once
    rows += list(range(B)); cols += [0] * B                   # a head label positive for every row
    rows += [0, 299, 256, 255]; cols += [L - 1, L - 1, L - 1, 1024]  # last ragged label tile, tile edges
    rows += [10, 11]; cols += [127, 128]
    perm = np.random.default_rng(0).permutation(len(rows))    # unsorted COO
    px = torch.tensor(rows)[perm]
    py = torch.tensor(cols)[perm]
    _check_step(dev, X, W, px, py)
    # out-of-range pairs are ignored
    px2 = torch.cat([px, torch.tensor([B, -1, 3])])
    py2 = torch.cat([py, torch.tensor([0, 0, L])])
    lay = XFCLayer(L, d, B, dev, weight=W)
    G2 = lay.fwd_grad(X.to(dev), px2.to(dev), py2.to(dev)).clone()
    G1 = lay.fwd_grad(X.to(dev), px.to(dev), py.to(dev))
    assert torch.equal(G1, G2)
    # row pointers that are not a CSR (not monotone, negative, past the list): nothing outside colidx[0 .. nnz) is
    # read and no entry counts twice, so at most nnz entries of G are below zero and the rest is sigmoid(Z)
    rp, ci = coo_to_csr(px, py, B)
    bad = rp.clone()
    bad[1:-1] = torch.from_numpy(np.random.default_rng(1).integers(-5, len(ci) + 50, size=B - 1).astype(np.int32))
    Gb = lay.fwd_grad(X.to(dev), rowptr=bad.to(dev), colidx=ci.to(dev)).float().cpu()
    S = torch.sigmoid(O.logits(X.float(), W.float()))
    neg = Gb < 0
    assert int(neg.sum()) <= len(ci) and rel(Gb[~neg], S[~neg]) <= TOL
    assert float((Gb[neg] - (S[neg] - 1.0)).abs().max()) <= 1e-3
    # no positives at all: G = sigmoid(Z)
    G0 = lay.fwd_grad(X.to(dev))
    assert rel(G0, torch.sigmoid(O.logits(X.float(), W.float()))) <= TOL


def test_golden_vectors(dev):
    z = np.load(os.path.join(GOLD, "xfc_step_small.npz"))
    lr, mu, wd, scale = [float(v) for v in z["hyper"]]
    X, W = torch.from_numpy(z["X"]).half(), torch.from_numpy(z["W0"]).half()
    px, py = torch.from_numpy(z["pos_x"]), torch.from_numpy(z["pos_y"])
    B, d = X.shape
    L = W.shape[0]
    lay = XFCLayer(L, d, B, dev, lr=lr, momentum=mu, weight_decay=wd, weight=W)
    G = lay.fwd_grad(X.to(dev), px.to(dev), py.to(dev))
    assert rel(G, torch.from_numpy(z["G1"])) <= TOL
    assert rel(lay.dx(B, scale=scale), torch.from_numpy(z["dX1"])) <= TOL
    dW = torch.empty(L, d, device=dev)
    lay.dw_update(X.to(dev), dW_out=dW)
    assert rel(dW, torch.from_numpy(z["dW1"])) <= TOL
    assert rel(lay.xfc_weight, torch.from_numpy(z["W1"])) <= TOL
    assert rel(lay.momentum_buffer, torch.from_numpy(z["M1"])) <= TOL
    # second step: compounding of two fp16-stored updates stays inside the same bound here
    lay.xfc_backward(X.to(dev), px.to(dev), py.to(dev), scale=scale)
    assert rel(lay.xfc_weight, torch.from_numpy(z["W2"])) <= 2 * TOL
    assert rel(lay.momentum_buffer, torch.from_numpy(z["M2"])) <= 2 * TOL


def test_real_label_distribution(dev):
    """First 256 rows of the reference's LF-AmazonTitles-131K test label matrix
    (L = 131,073, not a multiple of 8)."""
    lines = open(os.path.join(GOLD, "lf_amazontitles_131k_tst_first256.txt")).read().splitlines()
    B, L = [int(v) for v in lines[0].split()]
    rows, cols = [], []
    for b, line in enumerate(lines[1:]):
        for tok in line.split():
            rows.append(b)
            cols.append(int(tok.split(":")[0]))
    px, py = torch.tensor(rows), torch.tensor(cols)
    assert B == 256 and L == 131073 and len(px) > 256
    X, W = synth.make_X(B, 768, 5).half(), synth.make_W(L, 768, 5).half()
    rp, ci = coo_to_csr(px, py, B)
    _check_step(dev, X, W, px, py, csr=(rp, ci))


def test_step_entry_point_and_linearity(dev):
    B, L, d = 128, 5000, 256
    X, W, P = _problem(B, L, d, seed=4)
    rp, ci = torch.from_numpy(P.rowptr).to(dev), torch.from_numpy(P.colidx).to(dev)
    a = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=1e-4, weight=W)
    b = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=1e-4, weight=W)
    px, py = P.coo()
    for _ in range(3):
        ga = a.step_csr(X.to(dev), rp, ci, scale=2.0).clone()
        gb = b.xfc_backward(X.to(dev), px.to(dev), py.to(dev), scale=1.0)
        assert torch.equal(a.xfc_weight, b.xfc_weight) and torch.equal(a.momentum_buffer, b.momentum_buffer)
        assert torch.allclose(ga, 2.0 * gb, rtol=1e-6, atol=0)  # dX is linear in the loss scale


def test_split_accumulation(dev):
    """--accum: micro-batches of rows, dW accumulated in fp32, one optimizer step (dl_base.py:318-344)."""
    B, L, d, xfcz = 200, 3000, 128, 64
    X, W, P = _problem(B, L, d, seed=6)
    px, py = P.coo()
    lay = XFCLayer(L, d, xfcz, dev, lr=0.05, momentum=0.9, weight_decay=1e-3, weight=W)
    # the collator's layout: pos_x local to each micro-batch, `index` the nnz offsets
    index, px_local = [0], px.clone()
    for s in range(0, B, xfcz):
        e = min(B, s + xfcz)
        index.append(int(P.rowptr[e]))
        px_local[index[-2]:index[-1]] -= s
    gi = torch.empty(B, d, device=dev)
    for i, s in enumerate(range(0, B, xfcz)):
        e = min(B, s + xfcz)
        sl = slice(index[i], index[i + 1])
        lay.xfc_backward(X[s:e].to(dev), px_local[sl].to(dev), py[sl].to(dev), grad_input=gi[s:e], scale=2.0,
                         accumulate=True)
    grad = lay.xfc_weight_grad.clone()
    lay.optimizer_step()
    ref = O.step_accum(X.float(), W.float(), torch.zeros(L, d), px_local, py, torch.tensor(index), xfcz,
                       0.05, 0.9, 1e-3, 2.0)
    assert rel(gi, ref["dX"]) <= TOL and rel(grad, ref["dW"]) <= TOL
    assert rel(lay.xfc_weight, ref["W"]) <= TOL and rel(lay.momentum_buffer, ref["M"]) <= TOL
    assert lay.xfc_weight_grad is None


def test_lr_zero_still_updates_momentum(dev):
    B, L, d = 64, 512, 64
    X, W, P = _problem(B, L, d, seed=2)
    px, py = P.coo()
    lay = XFCLayer(L, d, B, dev, lr=0.0, momentum=0.9, weight=W)
    lay.xfc_backward(X.to(dev), px.to(dev), py.to(dev))
    assert torch.equal(lay.xfc_weight.cpu(), W)
    assert float(lay.momentum_buffer.abs().sum()) > 0


def test_xfc_gemm_three_modes(dev):
    """The reference's call sites: dl_base.py:591, :623, :629 and the dead :604."""
    B, L, d = 256, 4096, 768
    X, W, _ = _problem(B, L, d, seed=3)
    Xd, Wd = X.to(dev), W.to(dev)
    out = torch.full((B, L), float("nan"), device=dev, dtype=torch.float16)  # beta = 0 must not read it
    xfc_gemm(Xd, Wd.t(), out, 1.0, 0.0, True)
    ref = X.float().clone(), W.float().clone()
    want = torch.sigmoid(O.logits(*ref))
    assert rel(out, want) <= TOL
    G = out
    grad = torch.full((L, d), float("nan"), device=dev)
    xfc_gemm(G.t(), Xd, grad, 1.0, 0.0, False)
    want_dw = O.dw(G.float().cpu(), X.float())
    assert rel(grad, want_dw) <= TOL
    xfc_gemm(G.t(), Xd, grad, 1.0, 1.0, False)
    assert rel(grad, 2 * want_dw) <= TOL
    gi = torch.full((B, d), float("nan"), device=dev)
    xfc_gemm(G, Wd, gi, 4096.0, 0.0, False)
    assert rel(gi, O.dx(G.float().cpu(), W.float(), 4096.0)) <= TOL
    # alpha / beta on the sigmoid mode
    prev = (torch.randn(B, L) * 0.5).half()
    out2 = prev.to(dev)
    xfc_gemm(Xd, Wd.t(), out2, 2.0, 0.5, True)
    assert rel(out2, torch.sigmoid(2.0 * O.logits(*ref) + 0.5 * prev.float())) <= TOL


def test_xfc_gemm_alpha_beta_off_the_reference_call_sites(dev):
    """Argument values the reference's three call sites never pass but its kernels accept
    (xfc_gemm_kernel.cu:76-81, :137-142, :215-220 hand alpha and beta straight to the epilogue): beta != 0 in
    the row x row mode, beta outside {0, 1} in the column x row mode and in xfc_dw, and an output whose
    column stride is not 1 at a shape of many tiles."""
    from renee_amd._lib import check, lib

    B, L, d = 200, 4104, 72
    g = torch.Generator().manual_seed(11)
    G = (torch.rand(B, L, generator=g) - 0.3).half()
    W = (torch.randn(L, d, generator=g) * 0.05).half()
    X = torch.randn(B, d, generator=g).half()
    Gd, Wd, Xd = G.to(dev), W.to(dev), X.to(dev)
    # row x row (the dX mode), beta != 0: the split partial sums are reduced onto beta * out
    prev = torch.randn(B, d, generator=g)
    gi = prev.to(dev)
    xfc_gemm(Gd, Wd, gi, 3.0, -0.5, False)
    assert rel(gi, 3.0 * (G.float() @ W.float()) - 0.5 * prev) <= TOL
    # column x row (the dW mode), alpha and beta arbitrary
    prev = torch.randn(L, d, generator=g)
    grad = prev.to(dev)
    xfc_gemm(Gd.t(), Xd, grad, 2.0, -0.25, False)
    assert rel(grad, 2.0 * (G.float().t() @ X.float()) - 0.25 * prev) <= TOL
    # xfc_dw (split accumulation entry point) with a beta that is neither 0 nor 1
    grad = prev.to(dev)
    check(lib().xfc_dw(Gd.data_ptr(), Gd.stride(0), Xd.data_ptr(), Xd.stride(0), grad.data_ptr(), d, B, L, d, 0.5,
                       torch.cuda.current_stream().cuda_stream), "xfc_dw")
    assert rel(grad, G.float().t() @ X.float() + 0.5 * prev) <= TOL
    # outputs with a column stride other than 1 (any-stride kernel), several hundred thousand elements
    out_t = torch.full((L, B), float("nan"), device=dev, dtype=torch.float16)
    xfc_gemm(Xd, Wd.t(), out_t.t(), 1.0, 0.0, True)  # out is (B, L) with strides (1, B)
    assert rel(out_t.t(), torch.sigmoid(X.float() @ W.float().t())) <= TOL
    wide = torch.zeros(L, 2 * d, device=dev)
    xfc_gemm(Gd.t(), Xd, wide[:, ::2], 1.0, 0.0, False)  # column stride 2
    assert rel(wide[:, ::2], G.float().t() @ X.float()) <= TOL
    assert float(wide[:, 1::2].abs().max()) == 0.0
    wide = torch.zeros(B, 2 * d, device=dev)
    xfc_gemm(Gd, Wd, wide[:, ::2], 1.0, 0.0, False)
    assert rel(wide[:, ::2], G.float() @ W.float()) <= TOL
    assert float(wide[:, 1::2].abs().max()) == 0.0


def test_dx_and_topk_accept_a_workspace_smaller_than_their_fastest_plan(dev):
    """xfc_dx cuts the label axis into as many slices as the workspace holds (8 at least) and xfc_topk (K <= 8)
    uses as many label groups as fit (8 at least): the result does not depend on it; below the minimum the
    calls report XFC_ERR_WORKSPACE."""
    from renee_amd._lib import check, lib

    h = lib()
    st = torch.cuda.current_stream().cuda_stream
    B, L, d = 96, 40000, 64
    g = torch.Generator().manual_seed(12)
    G = (torch.rand(B, L, generator=g) - 0.3).half().to(dev)
    W = (torch.randn(L, d, generator=g) * 0.05).half().to(dev)
    want = G.float() @ W.float()
    full = h.xfc_dx_workspace_bytes(B, L, d)
    least = 8 * B * d * 4
    assert full > least
    for nbytes in (full, (full + least) // 2, least):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        dX = torch.full((B, d), float("nan"), device=dev)
        check(h.xfc_dx(G.data_ptr(), L, W.data_ptr(), d, dX.data_ptr(), d, B, L, d, 1.0, ws.data_ptr(), nbytes, st), "xfc_dx")
        assert rel(dX, want) <= TOL
    ws = torch.empty(least, dtype=torch.uint8, device=dev)
    assert h.xfc_dx(G.data_ptr(), L, W.data_ptr(), d, dX.data_ptr(), d, B, L, d, 1.0, ws.data_ptr(), least - 16, st) == 4
    X = torch.randn(B, d, generator=g).half().to(dev)
    Z = X.float() @ W.float().t()
    sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
    full = h.xfc_topk_workspace_bytes(B, L, 5)
    least = 8 * B * 5 * 8 + 4 * B
    assert full > 2 * least
    for nbytes in (full, full // 2, least):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        v = torch.empty(B, 5, device=dev)
        i = torch.empty(B, 5, device=dev, dtype=torch.int64)
        check(h.xfc_topk(X.data_ptr(), d, W.data_ptr(), d, B, L, d, L, 5, v.data_ptr(), i.data_ptr(), ws.data_ptr(), nbytes, st),
              "xfc_topk")
        assert torch.allclose(v, sv[:, :5], rtol=0, atol=2e-5 * float(sv.abs().max()))
        assert float((i == si[:, :5]).float().mean()) > 0.99
    assert h.xfc_topk(X.data_ptr(), d, W.data_ptr(), d, B, L, d, L, 5, v.data_ptr(), i.data_ptr(), ws.data_ptr(), least - 16, st) == 4


def test_xfc_gemm_any_stride_fallback_and_errors(dev):
    B, L, d = 9, 37, 20  # nothing is a multiple of 8
    g = torch.Generator().manual_seed(0)
    X, W = torch.randn(B, d, generator=g).half(), (torch.randn(L, d, generator=g) * 0.2).half()
    Xd, Wd = X.to(dev), W.to(dev)
    out = torch.empty(B, L, device=dev, dtype=torch.float16)
    xfc_gemm(Xd, Wd.t(), out, 1.0, 0.0, True)
    assert rel(out, torch.sigmoid(O.logits(X.float(), W.float()))) <= TOL
    grad = torch.empty(L, d, device=dev)
    xfc_gemm(out.t(), Xd, grad, 1.0, 0.0, False)
    assert rel(grad, O.dw(out.float().cpu(), X.float())) <= TOL
    gi = torch.empty(B, d, device=dev)
    xfc_gemm(out, Wd, gi, 2.0, 0.0, False)
    assert rel(gi, O.dx(out.float().cpu(), W.float(), 2.0)) <= TOL
    # several tiles of the fallback kernel with ragged edges on every axis and beta != 0, in the three layouts
    M, N, K = 130, 201, 77
    A, Bm = (torch.randn(M, K, generator=g) * 0.3).half(), (torch.randn(K, N, generator=g) * 0.3).half()
    prev = torch.randn(M, N, generator=g)
    want = 1.5 * (A.float() @ Bm.float()) - 0.5 * prev
    for a_dev in (A.to(dev), A.t().contiguous().to(dev).t()):  # row x row, column x row
        acc = prev.to(dev)
        xfc_gemm(a_dev, Bm.to(dev), acc, 1.5, -0.5, False)
        assert rel(acc, want) <= TOL and worst(acc, want) <= 2e-3 * float(want.abs().max())
    acc = prev.half().to(dev)
    xfc_gemm(A.to(dev), Bm.t().contiguous().to(dev).t(), acc, 1.5, -0.5, True)  # row x column, sigmoid
    want = torch.sigmoid(1.5 * (A.float() @ Bm.float()) - 0.5 * prev.half().float())
    assert rel(acc, want) <= TOL and worst(acc, want) <= 1e-3
    with pytest.raises(XfcError):  # row x row with apply_sigmoid: the reference exits the process here
        xfc_gemm(Xd, Wd.t().contiguous(), out, 1.0, 0.0, True)
    with pytest.raises(XfcError):  # inner dimensions disagree
        xfc_gemm(Xd[:, :8], Wd.t(), out, 1.0, 0.0, True)
    with pytest.raises(TypeError):
        xfc_gemm(Xd.float(), Wd.t(), out, 1.0, 0.0, True)


def test_logits(dev):
    B, L, d = 130, 3001, 768
    X, W, _ = _problem(B, L, d, seed=8)
    lay = XFCLayer(L, d, B, dev, weight=W)
    Z = lay.xfc_forward(X.to(dev))
    assert rel(Z, O.logits(X.float(), W.float())) <= TOL


def test_step_under_graph_capture(dev):
    """The entry points enqueue on the caller's stream and neither allocate nor synchronise, so a whole
    step can be captured in a HIP graph.  Every replay must reproduce the eager step bit for bit."""
    B, L, d = 256, 20000, 256
    X, W, P = _problem(B, L, d, seed=11)
    rp, ci = torch.from_numpy(P.rowptr).to(dev), torch.from_numpy(P.colidx).to(dev)
    Xd = X.to(dev)
    eager = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=1e-4, weight=W)
    graphed = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=1e-4, weight=W)
    # no sizing pass for the captured layer: its buffers, workspace included, exist since construction
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            graphed.step_csr(Xd, rp, ci, scale=2.0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # the captured call did not run; replay and compare with eager steps, with eager work in between
    for _ in range(4):
        g.replay()
        ge = eager.step_csr(Xd, rp, ci, scale=2.0).clone()
        torch.cuda.synchronize()
        assert torch.equal(graphed.xfc_weight, eager.xfc_weight)
        assert torch.equal(graphed.momentum_buffer, eager.momentum_buffer)
        assert torch.equal(graphed.grad_input[:B], ge)


@pytest.mark.parametrize("B,L,d", [(64, 1000, 64), (300, 70001, 128), (512, 8192, 768)])
def test_fused_loss(dev, B, L, d):
    """Summed BCE-with-logits loss from the forward pass (dl_base.py:578-583) against the oracle and
    against BCEWithLogitsLoss(reduction='sum'); G must be unchanged by asking for the loss."""
    X, W, P = _problem(B, L, d, seed=3)
    px, py = P.coo()
    lay = XFCLayer(L, d, B, dev, weight=W)
    loss = torch.zeros(1, device=dev)
    G1 = lay.fwd_grad(X.to(dev), px.to(dev), py.to(dev), loss_out=loss).clone()
    G0 = lay.fwd_grad(X.to(dev), px.to(dev), py.to(dev))
    assert torch.equal(G0, G1)
    Z = O.logits(X.float(), W.float())
    want = float(O.sampled_loss(Z.double(), px, py))
    Y = torch.zeros(B, L, dtype=torch.float64)
    Y[px, py] = 1.0
    bce = float(torch.nn.BCEWithLogitsLoss(reduction="sum")(Z.double(), Y))
    assert abs(want - bce) <= 1e-6 * abs(bce)  # the oracle follows the reference and sums in float32
    assert abs(float(loss) - bce) <= 1e-5 * abs(bce)


def test_state_dict_round_trip(dev):
    B, L, d = 64, 1000, 64
    X, W, P = _problem(B, L, d, seed=5)
    px, py = P.coo()
    a = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    a.xfc_backward(X.to(dev), px.to(dev), py.to(dev))
    st = a.state_dict()
    b = XFCLayer(L, d, B, dev, lr=0.01, momentum=0.5, seed=9)
    b.load_state_dict(st)
    a.xfc_backward(X.to(dev), px.to(dev), py.to(dev))
    b.xfc_backward(X.to(dev), px.to(dev), py.to(dev))
    assert torch.equal(a.xfc_weight, b.xfc_weight) and torch.equal(a.momentum_buffer, b.momentum_buffer)
    # a reference checkpoint holds fp32 weights and may have no momentum yet
    c = XFCLayer(L, d, B, dev, seed=1)
    c.load_state_dict({"xfc_weight": W.float()})
    assert torch.equal(c.xfc_weight.cpu(), W) and float(c.momentum_buffer.abs().sum()) == 0.0


def test_fp32_embeddings_are_cast_once_as_the_reference_casts_them(dev):
    """The encoder hands over fp32 embeddings and the reference casts them to fp16 before the XFC GEMMs
    (dl_base.py:561).  An fp32 `embed` (also one on the CPU) must give the bits the fp16 one gives, and
    stay within tolerance of the oracle evaluated on the fp16-rounded embeddings."""
    B, L, d = 96, 3000, 128
    X32 = synth.make_X(B, d, 31)                      # fp32, not representable in fp16
    W = synth.make_W(L, d, 31).half()
    P = synth.make_positives(B, L, 8, 2.3, 1.1, 31)
    px, py = P.coo()
    a = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    b = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    c = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    dXa = a.xfc_backward(X32.to(dev), px, py).clone()           # fp32 on the GPU
    dXb = b.xfc_backward(X32.half().to(dev), px, py).clone()    # already fp16
    dXc = c.xfc_backward(X32, px, py).clone()                   # fp32 on the CPU
    for other, dXo in ((b, dXb), (c, dXc)):
        assert torch.equal(dXa, dXo) and torch.equal(a.xfc_weight, other.xfc_weight)
        assert torch.equal(a.momentum_buffer, other.momentum_buffer)
    ref = O.step(X32.half().float(), W.float(), torch.zeros(L, d), px, py, 0.05, 0.9, 0.0, 1.0)
    assert rel(dXa[:B], ref["dX"]) <= TOL and rel(a.xfc_weight, ref["W"]) <= TOL


def test_seeded_shape_sweep(dev):
    """Sixteen seeded shapes off every tile boundary (batch 1..520, labels 8..6000, d a multiple of 8 up
    to 384), X handed over as a strided view, random weight decay and loss scale: one whole step each."""
    rng = np.random.default_rng(123)
    for case in range(16):
        B = int(rng.integers(1, 521))
        L = int(rng.integers(8, 6001))
        d = 8 * int(rng.integers(1, 49))
        wd = float(rng.choice([0.0, 1e-4, 1e-2]))
        scale = float(rng.choice([1.0, 4096.0, 0.5]))
        X, W, P = _problem(B, L, d, kmax=min(8, L), seed=1000 + case)
        px, py = P.coo()
        wide = torch.zeros(B, d + 8 * int(rng.integers(0, 3)), dtype=torch.float16)
        wide[:, :d] = X
        print(f"sweep case {case}: B={B} L={L} d={d} ld={wide.shape[1]} wd={wd} scale={scale}", flush=True)
        lay = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=wd, weight=W)
        Xd = wide.to(dev)[:, :d]
        ref = O.step(X.float(), W.float(), torch.zeros(L, d), px, py, 0.05, 0.9, wd, scale)
        dX = lay.xfc_backward(Xd, px.to(dev), py.to(dev), scale=scale)
        assert rel(lay.outsoft[:B, :L], ref["G"]) <= TOL and worst(lay.outsoft[:B, :L], ref["G"]) <= 2e-3
        assert rel(dX[:B], ref["dX"]) <= TOL and worst(dX[:B], ref["dX"]) <= 5e-3
        assert rel(lay.xfc_weight, ref["W"]) <= TOL and worst(lay.xfc_weight, ref["W"]) <= 3e-3
        assert rel(lay.momentum_buffer, ref["M"]) <= TOL and worst(lay.momentum_buffer, ref["M"]) <= 3e-3


@pytest.mark.parametrize("B,L,d", [(1030, 2500, 256), (2500, 1999, 128), (4100, 1024, 64)])
def test_batches_above_1024(dev, B, L, d):
    """More rows than any BASELINE configuration has: five to seventeen row tiles in the forward pass and dX, a
    contraction over up to 4100 rows in dW."""
    X, W, P = _problem(B, L, d, seed=B)
    px, py = P.coo()
    _check_step(dev, X, W, px, py, wd=1e-4, scale=2.0)


@pytest.mark.parametrize("B,L,d,csr", [(16, 3_200_000, 8, False), (16, 3_200_000, 8, True), (15000, 520, 8, True)])
def test_bucket_pass_variants(dev, B, L, d, csr):
    """The pass that groups the positives by label tile keeps its per-tile counters in LDS up to 12,288 label tiles
    and in global memory above (3.2 M labels: 12,500 tiles), and walks a CSR list by entry with the row pointers in
    LDS while they fit next to the counters (15,000 rows do not: one row per thread then)."""
    X, W, P = _problem(B, L, d, kmax=6, kmean=3.0, seed=77)
    px, py = P.coo()
    _check_step(dev, X, W, px, py, csr=(torch.from_numpy(P.rowptr), torch.from_numpy(P.colidx)) if csr else None)


def test_index_tensors_are_checked_and_moved_before_any_launch(dev):
    """Label tensors arrive from the collator on the CPU (dl_base.py:934-936).  They are copied to the
    layer's GPU, never dereferenced where they are; a wrong dtype or length raises before a launch."""
    B, L, d = 64, 3000, 64
    X, W, P = _problem(B, L, d, seed=21)
    px, py = P.coo()
    rp, ci = torch.from_numpy(P.rowptr), torch.from_numpy(P.colidx)
    lay = XFCLayer(L, d, B, dev, weight=W)
    Xd = X.to(dev)
    G_dev = lay.fwd_grad(Xd, px.to(dev), py.to(dev)).clone()
    G_cpu = lay.fwd_grad(Xd, px, py).clone()                      # CPU COO: moved, same result
    assert torch.equal(G_dev, G_cpu)
    G_csr = lay.fwd_grad(Xd, rowptr=rp, colidx=ci).clone()        # CPU CSR
    assert torch.equal(G_dev, G_csr)
    marker = lay.outsoft[:B, :L].clone()  # columns past the labels are never written (and may hold NaN)
    with pytest.raises(TypeError):
        lay.fwd_grad(Xd, rowptr=rp.long(), colidx=ci)             # int64 CSR is not silently misread
    with pytest.raises(TypeError):
        lay.step_csr(Xd, rp.to(dev), ci.long().to(dev))
    with pytest.raises(TypeError):
        lay.fwd_grad(Xd, px.int(), py.int())
    with pytest.raises(RuntimeError):
        lay.step_csr(Xd, rp[:-1], ci)                             # rowptr must have B + 1 entries
    with pytest.raises(RuntimeError):
        lay.fwd_grad(Xd, px[:-1], py)
    small = XFCLayer(L, d, B, dev, weight=W, max_positives=4)
    with pytest.raises(ValueError):
        small.fwd_grad(Xd, px, py)
    torch.cuda.synchronize()
    assert torch.equal(lay.outsoft[:B, :L], marker)                   # nothing ran for the rejected calls
    gi = lay.step_csr(Xd, rp, ci)                                 # CPU CSR through the one-call step
    ref = O.step(X.float(), W.float(), torch.zeros(L, d), px, py, 0.05, 0.9, 0.0, 1.0)
    assert rel(gi, ref["dX"]) <= TOL and rel(lay.xfc_weight, ref["W"]) <= TOL


def test_two_layers_on_two_streams(dev):
    """Each layer owns its scratch, so two layers may run on two streams at once: the results are
    bit-identical to the same steps run one after the other."""
    B, L, d = 256, 40000, 256
    X, W, P = _problem(B, L, d, seed=22)
    X2, W2, P2 = _problem(B, L, d, seed=23)
    rp, ci = torch.from_numpy(P.rowptr).to(dev), torch.from_numpy(P.colidx).to(dev)
    rp2, ci2 = torch.from_numpy(P2.rowptr).to(dev), torch.from_numpy(P2.colidx).to(dev)
    Xd, X2d = X.to(dev), X2.to(dev)

    def build():
        return (XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W),
                XFCLayer(L, d, B, dev, lr=0.02, momentum=0.8, weight=W2))

    sa, sb = build()
    for _ in range(3):
        sa.step_csr(Xd, rp, ci, scale=2.0)
        sb.step_csr(X2d, rp2, ci2, scale=0.5)
    torch.cuda.synchronize()
    ca, cb = build()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(3):
        with torch.cuda.stream(s1):
            ca.step_csr(Xd, rp, ci, scale=2.0)
        with torch.cuda.stream(s2):
            cb.step_csr(X2d, rp2, ci2, scale=0.5)
    torch.cuda.synchronize()
    for serial, conc in ((sa, ca), (sb, cb)):
        assert torch.equal(serial.xfc_weight, conc.xfc_weight)
        assert torch.equal(serial.momentum_buffer, conc.momentum_buffer)
        assert torch.equal(serial.grad_input[:B], conc.grad_input[:B])


def test_empty_batch_and_reference_optimizer_state(dev):
    """B = 0 launches nothing and leaves W and M alone; a reference checkpoint's optimizer state
    (torch layout, fp32 momentum_buffer) is taken over by load_state_dict."""
    from renee_amd._lib import lib
    L, d = 1000, 64
    W = synth.make_W(L, d, 5).half()
    lay = XFCLayer(L, d, 8, dev, weight=W)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib().xfc_dw_update(lay.outsoft.data_ptr(), lay.ldg, lay.outsoft.data_ptr(), d, lay.xfc_weight.data_ptr(), d,
                             lay.momentum_buffer.data_ptr(), d, 0, L, d, 0.05, 0.9, 0.0, None, 0, st)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(lay.xfc_weight.cpu(), W) and float(lay.momentum_buffer.abs().max()) == 0.0
    m32 = torch.randn(L, d) * 0.1
    lay.load_state_dict({"xfc_weight": W.float()},
                        optimizer_state={"state": {0: {"momentum_buffer": m32}}, "param_groups": [{"lr": 0.05}]})
    assert torch.equal(lay.momentum_buffer.cpu(), m32.half())


@pytest.mark.parametrize("B,L,d,wd", [(256, 4097, 768, 0.0), (100, 3001, 64, 1e-3)])
def test_master_weights_update_matches_fp32_oracle(dev, B, L, d, wd):
    """xfc_dw_update_master: the reference's optimizer regime (fp32 W and momentum, dl_base.py:185,
    main.py:178-179) with the fp16 copy of W written by the same pass; two steps, then the split
    accumulation path (xfc_dw + xfc_sgd_momentum_master)."""
    X, W, P = _problem(B, L, d, seed=51)
    W32 = synth.make_W(L, d, 51)                    # an fp32 weight that is not fp16-representable
    px, py = P.coo()
    Xd = X.to(dev)
    lay = XFCLayer(L, d, B, dev, lr=0.01, momentum=0.9, weight_decay=wd, weight=W32, master_weights=True)
    assert torch.equal(lay.xfc_weight_master.cpu(), W32) and torch.equal(lay.xfc_weight.cpu(), W32.half())
    Wo, Mo = W32.clone(), torch.zeros(L, d)
    for s in range(2):
        print(f"master step {s}: B={B} L={L} d={d}", flush=True)
        G = lay.fwd_grad(Xd, px, py)
        Gref = O.grad_logits(O.logits(X.float(), Wo.half().float()), px, py)
        assert rel(G, Gref) <= TOL
        dW = torch.empty(L, d, device=dev, dtype=torch.float32)
        lay.dw_update(Xd, dW_out=dW)
        # the oracle is fed the device's own fp16 G so that only the update is compared
        Gd = lay.outsoft[:B, :L].float().cpu()
        dWo = O.dw(Gd, X.float())
        assert rel(dW, dWo) <= TOL
        Wn, Mn = O.sgd_momentum(Wo, Mo, dW.cpu(), 0.01, 0.9, wd)
        assert rel(lay.xfc_weight_master, Wn) <= 1e-6 and rel(lay.momentum_buffer, Mn) <= 1e-6
        assert torch.equal(lay.xfc_weight, lay.xfc_weight_master.half())
        Wo, Mo = lay.xfc_weight_master.cpu().clone(), lay.momentum_buffer.cpu().clone()
    # split accumulation: two micro-batches, then one optimizer step on the fp32 state
    half = B // 2 // 8 * 8 or B
    lay.fwd_grad(Xd[:half], *[t[px < half] for t in (px, py)])
    lay.dw_accumulate(Xd[:half])
    acc = lay.xfc_weight_grad.clone()
    lay.optimizer_step()
    Wn, Mn = O.sgd_momentum(Wo, Mo, acc.cpu(), 0.01, 0.9, wd)
    assert rel(lay.xfc_weight_master, Wn) <= 1e-6 and rel(lay.momentum_buffer, Mn) <= 1e-6
    assert torch.equal(lay.xfc_weight, lay.xfc_weight_master.half())
    st = lay.state_dict()
    assert st["xfc_weight"].dtype == torch.float32 and st["momentum_buffer"].dtype == torch.float32


@pytest.mark.parametrize("B", [1, 32, 64, 100, 128, 129])
def test_small_batches_take_the_small_row_tiles(dev, B):
    """Batches of up to 64 and up to 128 rows run 64- and 128-row tiles in the forward, dX and top-K kernels
    (the reference's B = 32 plumbing case, --accum micro-batches dl_base.py:318-340, partial last batches):
    the whole step and the top-5 against the oracle."""
    L, d = 5001, 768
    X, W, P = _problem(B, L, d, kmax=6, kmean=2.0, seed=60 + B)
    px, py = P.coo()
    lay = _check_step(dev, X, W, px, py, lr=0.05, mu=0.9, wd=1e-4, scale=4.0, steps=2)
    v, i = lay.topk(X.to(dev), 5)
    ov, oi = O.topk(X.float(), lay.xfc_weight.float().cpu(), 5)
    assert torch.allclose(v.cpu(), ov, rtol=0, atol=1e-3 * float(ov.abs().max()))
    gap = (ov[:, :-1] - ov[:, 1:]).abs().min(dim=1).values                  # rows whose top-5 is clearly separated
    sure = gap > 1e-4 * float(ov.abs().max())
    assert torch.equal(i.cpu()[sure], oi[sure])


def test_reference_loss_module_interface(dev):
    """renee_amd.BCELossMultiNode has the reference class's call signature (dl_base.py:576); the XFC
    block of fit (dl_base.py:303-344) written against it, with the reference's own `out` and
    `grad_input` views, matches the oracle over two steps, with and without a preceding xfc_forward,
    the sampled loss on step 0, and under split accumulation."""
    from renee_amd import BCELossMultiNode

    class Scaler:                       # the part of torch.cuda.amp.GradScaler the path uses (dl_base.py:599)
        def get_scale(self):
            return 4096.0

    B, L, d = 96, 4112, 128             # numy padded to a multiple of 16 as main.py:83-87 does
    X, W, P = _problem(B, L, d, seed=71)
    z = torch.stack(P.coo())            # the collator's 'z' (2 x nnz LongTensor on the CPU)
    lay = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    lm = BCELossMultiNode(lay, compute_loss=True, scaler=Scaler())
    Wo, Mo = W.float(), torch.zeros(L, d)
    for step in range(2):
        embed_out = lm.gather_embed(X.float().to(dev), None)
        do_forward = step == 0          # a loss step: the reference runs xfc_forward first (dl_base.py:311)
        out = lay.outsoft[0:B, :]
        if do_forward:
            lm.xfc_forward(embed_out, out)
        loss = lm.xfc_backward(embed_out, out, z[0], z[1], lay.grad_input[0:B, :], not do_forward)
        lm.xfc_optimizer.step()
        lm.count += 1
        ref = O.step(X.float(), Wo, Mo, z[0], z[1], 0.05, 0.9, 0.0, 4096.0)
        assert rel(lay.grad_input[:B], ref["dX"]) <= TOL
        assert rel(lay.xfc_weight, ref["W"]) <= TOL and rel(lay.momentum_buffer, ref["M"]) <= TOL
        if step == 0:
            want = O.sampled_loss(O.logits(X.float(), Wo), z[0], z[1])
            assert abs(float(loss) - float(want)) <= 1e-3 * abs(float(want))
        Wo, Mo = lay.xfc_weight.float().cpu(), lay.momentum_buffer.float().cpu()
    # --accum 2: two micro-batches into the fp32 grad, then one optimizer step (dl_base.py:318-343)
    lm2 = BCELossMultiNode(lay, compute_loss=False, scaler=Scaler(), accum=2)
    half = B // 2
    idx = [0, int((z[0] < half).sum()), z.shape[1]]
    for i, (r0, r1) in enumerate(((0, half), (half, B))):
        e = lm2.gather_embed(X[r0:r1].float().to(dev))
        lm2.xfc_backward(e, lay.outsoft[0:r1 - r0, :], z[0, idx[i]:idx[i + 1]] - r0, z[1, idx[i]:idx[i + 1]],
                         lay.grad_input[r0:r1, :], True)
    lm2.xfc_optimizer.step()
    ref = O.step(X.float(), Wo, Mo, z[0], z[1], 0.05, 0.9, 0.0, 4096.0)
    assert rel(lay.grad_input[:B], ref["dX"]) <= TOL
    assert rel(lay.xfc_weight, ref["W"]) <= TOL and rel(lay.momentum_buffer, ref["M"]) <= TOL


def test_autograd_wrapper_sends_grad_input_into_the_encoder_graph(dev):
    """loss.backward() through xfc_loss gives the encoder what the reference hands to embed.backward
    (dl_base.py:360): scale * G . W with the weights before the update, and the step's update is applied."""
    from renee_amd import xfc_loss

    B, L, d = 96, 3000, 64
    X, W, P = _problem(B, L, d, seed=21)
    px, py = P.coo()
    ref = O.step(X.float(), W.float(), torch.zeros(L, d), px, py, 0.05, 0.9, 0.0, 8.0)
    lay = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight=W)
    enc = torch.nn.Linear(d, d, bias=False).to(dev)   # stands for the encoder
    with torch.no_grad():
        enc.weight.copy_(torch.eye(d))
    inp = X.float().to(dev)
    embed = enc(inp)
    loss = xfc_loss(embed, lay, px, py, scale=8.0, compute_loss=True)
    loss.backward()
    assert rel(enc.weight.grad, ref["dX"].t() @ X.float()) <= TOL    # d loss / d enc.weight = dX^T . inp
    assert rel(lay.xfc_weight, ref["W"]) <= TOL
    want_loss = torch.nn.functional.binary_cross_entropy_with_logits(
        O.logits(X.float(), W.float()), (ref["G"] < 0).float(), reduction="sum")
    got_loss = float(loss.detach())
    assert abs(got_loss - float(want_loss)) <= 1e-4 * float(want_loss), (got_loss, float(want_loss))


def test_training_loop_learns_and_topk_finds_the_labels(dev):
    """A trainer loop as the reference's fit runs it (dl_base.py:295-376): encoder forward, classifier step with
    the update inside, grad_input into the encoder's backward, encoder optimizer step; then the predictor's
    top-5 (dl_base.py:736-756).  512 labels with one prototype input each: recall@5 goes from chance to most."""
    from renee_amd import xfc_loss

    torch.manual_seed(0)
    B, L, d, din, n = 256, 512, 64, 32, 4096
    protos = torch.nn.functional.normalize(torch.randn(L, din), dim=1)
    lab = torch.randint(0, L, (n,))
    xs = (protos[lab] + 0.02 * torch.randn(n, din)).to(dev)
    lab_d = lab.to(dev)
    enc = torch.nn.Linear(din, d, bias=False).to(dev)
    opt = torch.optim.SGD(enc.parameters(), lr=2e-3)
    lay = XFCLayer(L, d, B, dev, lr=2e-3, momentum=0.9, seed=3)

    def recall():
        hit = 0
        with torch.no_grad():
            for i in range(0, n, B):
                _, top = lay.topk(enc(xs[i:i + B]), 5)
                hit += int((top == lab_d[i:i + B, None]).any(1).sum())
        return hit / n

    before = recall()
    rows = torch.arange(B, device=dev)
    for step in range(400):
        idx = torch.randint(0, n, (B,), device=dev)
        loss = xfc_loss(enc(xs[idx]), lay, rows, lab_d[idx])
        opt.zero_grad()
        loss.backward()
        opt.step()
    after = recall()
    print(f"recall@5 {before:.3f} -> {after:.3f}", flush=True)
    assert before < 0.05 and after > 0.6
