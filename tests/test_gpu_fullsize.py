"""Full BASELINE sizes, every element checked.  The CPU oracle cannot finish these in
seconds, so the reference is the same fp32 formulation (dl_base.py:572, :593-594, :606,
:625, main.py:178-179) evaluated with torch fp32 ops on the GPU in label chunks, built
from X, W, M and the label list only -- never from a kernel's own output: G, dX, and W
and M after the update are each compared in full (relative Frobenius error over the whole
array, and a bound on the largest single error so that one wrong tile in tens of thousands
cannot hide in the norm), plus the size-independent properties (one negative entry of G
per positive, zeroed pad columns, linearity of dX in the loss scale)."""
import pytest
import torch

from renee_amd import XFCLayer, synth

pytestmark = pytest.mark.gpu
TOL = 1e-3
CHUNK = 1 << 16  # labels per reference chunk: B x CHUNK fp32 = 256 MB at batch 1024


class _Err:
    """Running relative Frobenius error and largest absolute error over chunks."""

    def __init__(self):
        self.num = self.den = 0.0
        self.max_abs = 0.0

    def add(self, got, ref):
        diff = got.double() - ref.double()
        self.num += float((diff * diff).sum())
        self.den += float((ref.double() * ref.double()).sum())
        self.max_abs = max(self.max_abs, float(diff.abs().max()))

    @property
    def rel(self):
        return (self.num / self.den) ** 0.5


def _fullsize_step(dev, cfg, lr=0.05, mu=0.9, wd=1e-4, scale=2.0):
    c = synth.CONFIGS[cfg]
    B, L, d = c["B"], c["L"], synth.D_MODEL
    print(f"cfg{cfg}: B={B} L={L}", flush=True)
    lay = XFCLayer(L, d, B, dev, lr=lr, momentum=mu, weight_decay=wd, seed=cfg)
    # a momentum that is not zero, so that the update's mu * M term is exercised at every element
    g = torch.Generator(device=dev).manual_seed(100 + cfg)
    for r0 in range(0, L, 1 << 20):
        r1 = min(L, r0 + (1 << 20))
        lay.momentum_buffer[r0:r1] = (torch.randn(r1 - r0, d, generator=g, device=dev) * 0.01).half()
    X = synth.make_X(B, d, cfg, dev).half()
    P = synth.make_positives(B, L, c["kmax"], c["kmean"], c["zipf"], cfg)
    rp, ci = torch.from_numpy(P.rowptr).to(dev), torch.from_numpy(P.colidx).to(dev)
    px, py = (t.to(dev) for t in P.coo())
    W0, M0 = lay.xfc_weight.clone(), lay.momentum_buffer.clone()
    Xf = X.float()

    G = lay.fwd_grad(X, rowptr=rp, colidx=ci)
    dX = lay.dx(B, scale=scale).clone()
    assert torch.allclose(lay.dx(B, scale=1.0) * scale, dX, rtol=1e-6, atol=0)
    lay.dw_update(X)
    torch.cuda.synchronize()
    if L % 8:
        assert float(lay.outsoft[:B, L:(L + 7) // 8 * 8].abs().max()) == 0.0

    eG, eW, eM = _Err(), _Err(), _Err()
    dX_ref = torch.zeros(B, d, device=dev)
    negatives = 0
    for l0 in range(0, L, CHUNK):
        l1 = min(L, l0 + CHUNK)
        Wc, Mc = W0[l0:l1].float(), M0[l0:l1].float()
        Gr = torch.sigmoid(Xf @ Wc.t())                              # dl_base.py:572, :593
        m = (py >= l0) & (py < l1)
        Gr[px[m], py[m] - l0] -= 1.0                                 # dl_base.py:594 (non-accumulating)
        Gk = G[:, l0:l1]
        eG.add(Gk, Gr)
        negatives += int((Gk < 0).sum())
        dX_ref += Gr @ Wc                                            # dl_base.py:606
        dWr = Gr.t() @ Xf                                            # dl_base.py:625
        Mr = mu * Mc + dWr + wd * Wc                                 # main.py:178-179 (FusedSGD: wd, momentum)
        Wr = Wc - lr * Mr
        eM.add(lay.momentum_buffer[l0:l1], Mr)
        eW.add(lay.xfc_weight[l0:l1], Wr)
        del Gr, dWr, Mr, Wr, Wc, Mc
    print(f"cfg{cfg}: G {eG.rel:.2e} (max {eG.max_abs:.2e})  W {eW.rel:.2e} (max {eW.max_abs:.2e})  "
          f"M {eM.rel:.2e} (max {eM.max_abs:.2e})", flush=True)
    assert negatives == P.nnz  # one entry below zero per (row, label) pair, nowhere else
    assert eG.rel <= TOL and eG.max_abs <= 1e-3   # half an fp16 step of a value below 1 is 2.4e-4
    dX_ref *= scale
    assert float((dX - dX_ref).norm() / dX_ref.norm()) <= TOL
    assert float((dX - dX_ref).abs().max()) <= 5e-3 * float(dX_ref.abs().max())
    assert eM.rel <= TOL and eW.rel <= TOL
    # one fp16 rounding of M (|M| up to a few times 0.01 plus dW) and of W: well below these bounds,
    # which a tile updated twice, skipped, or written to the wrong rows would exceed
    assert eM.max_abs <= 2e-3 * float(M0.abs().max() + 1.0) and eW.max_abs <= 2e-3 * float(W0.abs().max() + lr)
    del W0, M0
    return lay, X


def test_config2_headline_shape(dev):
    _fullsize_step(dev, 2)


def test_config3_ragged_labels_and_top5(dev):
    lay, X = _fullsize_step(dev, 3)
    B, L = X.shape[0], lay.numy
    v, i = lay.topk(X, 5)
    # reference: fp32 logits on the GPU in label chunks, running top-5 with a stable sort (lowest id first);
    # the same chunks, rounded to fp16, are kept as the reference logits of the K = 100 check below
    best_v = torch.full((B, 5), float("-inf"), device=dev)
    best_i = torch.zeros(B, 5, dtype=torch.int64, device=dev)
    Zref = torch.empty(B, L, device=dev, dtype=torch.float16)
    step = 1 << 17
    for l0 in range(0, L, step):
        l1 = min(L, l0 + step)
        Z = X.float() @ lay.xfc_weight[l0:l1].float().t()
        Zref[:, l0:l1] = Z.half()
        cv = torch.cat([best_v, Z], 1)
        cidx = torch.cat([best_i, torch.arange(l0, l1, device=dev).expand(B, -1)], 1)
        sv, sp = torch.sort(cv, dim=1, descending=True, stable=True)
        best_v, best_i = sv[:, :5], torch.gather(cidx, 1, sp[:, :5])
    scale = float(best_v.abs().max())
    assert torch.allclose(v, best_v, rtol=0, atol=2e-5 * scale)
    mism = (i != best_i)
    # the two fp32 evaluations differ in summation order: allow swaps only between near-equal scores
    if mism.any():
        for b, j in mism.nonzero().tolist():
            other = best_v[b, min(j + 1, 4)] if j < 4 else best_v[b, j - 1]
            gap = min(abs(float(best_v[b, j] - other)), abs(float(best_v[b, max(j - 1, 0)] - best_v[b, j])) or 1e9)
            assert gap <= 1e-5 * scale, (b, j)
    assert float(mism.float().mean()) < 0.01
    # the final evaluation's K = 100 (dl_base.py:817-818) at the same size
    torch.cuda.synchronize()
    print("top-100 at configs[3] size", flush=True)
    v100, i100 = lay.topk(X, 100)
    # (a) against the reference logits (fp32 chunks rounded to fp16, nothing of the kernels in them): the
    # values agree to one fp16 step (the two fp32 sums differ in order, so a rounding may fall either way),
    # and the labels returned hold those values in the reference logits
    tv, _ = torch.topk(Zref.float(), 100, dim=1)
    ulp = 2.0 ** -10 * scale  # one fp16 step at the largest score is at most this
    assert float((v100 - tv).abs().max()) <= ulp
    assert float((torch.gather(Zref, 1, i100).float() - v100).abs().max()) <= ulp
    del Zref
    # (b) the selection itself is exact on the logits it was given: torch.topk of the library's own fp16
    # logits gives identical values; indices point at those values, ascending within equal values, distinct
    Zg = lay.xfc_forward(X)
    tv, _ = torch.topk(Zg, 100, dim=1)
    assert torch.equal(v100, tv.float())
    assert torch.equal(torch.gather(Zg, 1, i100).float(), v100)
    same = v100[:, 1:] == v100[:, :-1]
    assert bool((i100[:, 1:] > i100[:, :-1])[same].all())
    srt, _ = torch.sort(i100, dim=1)
    assert bool((srt[:, 1:] != srt[:, :-1]).all())
    # the fused K = 5 scorer and the selection agree on the leaders (fp16 rounding can swap near-equal ones)
    assert float((i100[:, :5] == i).float().mean()) > 0.95


def test_config4_streaming_shape(dev):
    _fullsize_step(dev, 4)


def test_smaller_batches_fit_a_layer_sized_for_max_batch(dev):
    """A layer built for max_batch serves every smaller batch on the workspace it allocated once
    (dl_base.py:175-187, :318-340), also where the smaller batch's own plan needs more scratch than
    max_batch's: dX at 260 rows of a 512-row layer (more label slices than 512 rows take), and the fused
    top-5 at 256 rows of a 300-row layer with few feature dims (more label groups)."""
    L, d = 1310720, 768
    lay = XFCLayer(L, d, 512, dev, seed=5)
    B = 260
    X = synth.make_X(B, d, 5, dev).half()
    P = synth.make_positives(B, L, 20, 5.0, 1.0, 5)
    px, py = (t.to(dev) for t in P.coo())
    W0 = lay.xfc_weight.clone()
    dX = lay.xfc_backward(X, px, py, scale=1.0).clone()
    ref = torch.zeros(B, d, device=dev)
    for l0 in range(0, L, CHUNK):
        l1 = min(L, l0 + CHUNK)
        Wc = W0[l0:l1].float()
        Gr = torch.sigmoid(X.float() @ Wc.t())
        m = (py >= l0) & (py < l1)
        Gr[px[m], py[m] - l0] -= 1.0
        ref += Gr @ Wc
    assert float((dX - ref).norm() / ref.norm()) <= TOL
    del lay, W0
    torch.cuda.empty_cache()
    L, d = 70001, 16
    W = synth.make_W(L, d, 6).half()
    lay = XFCLayer(L, d, 300, dev, weight=W)
    X = synth.make_X(256, d, 6, dev).half()
    v, i = lay.topk(X, 5)
    Z = X.float() @ lay.xfc_weight.float().t()
    sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
    assert torch.allclose(v, sv[:, :5], rtol=0, atol=2e-5 * float(sv.abs().max()))
    assert float((i == si[:, :5]).float().mean()) > 0.99
