"""Top-K scoring kernel against the oracle's iterated-max restatement
(dl_base.py:736-756, :782).  Indices must agree except where the oracle's own
neighbouring scores are closer than the accumulation-order noise of an fp32 dot
product of 768 fp16 products (relative 1e-5 here); exact ties must resolve to
the lower label id."""
import pytest
import torch

from oracle import xfc_oracle as O
from renee_amd import XFCLayer, synth

pytestmark = pytest.mark.gpu
NEAR = 1e-5


def _check(dev, X, W, K, numy=None):
    B, d = X.shape
    L = W.shape[0]
    lay = XFCLayer(L, d, B, dev, weight=W)
    print(f"topk: B={B} L={L} d={d} K={K} numy={numy}", flush=True)
    v, i = lay.topk(X.to(dev), K, numy)
    v, i = v.cpu(), i.cpu()
    Z = O.logits(X.float(), W.float())
    rv, ri = O.topk(X.float(), W.float(), K if K <= 5 else K, numy)
    if K > 5:  # the oracle's K > 5 branch is torch.topk, whose tie order is unspecified: sort explicitly
        sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
        rv, ri = sv[:, :K], si[:, :K]
        if numy is not None:
            ri = torch.where(ri >= numy, torch.full_like(ri, numy - 1), ri)
    scale = float(Z.abs().max())
    assert torch.allclose(v, rv, rtol=0, atol=2e-5 * scale)
    mism = (i != ri)
    if mism.any():
        # a mismatch is only acceptable between labels whose oracle scores are (nearly) equal
        sv, _ = torch.sort(Z, dim=1, descending=True)
        for b, j in mism.nonzero().tolist():
            lo, hi = float(sv[b, min(j + 1, L - 1)]), float(sv[b, max(j - 1, 0)])
            here = float(sv[b, j])
            assert min(abs(here - lo), abs(hi - here)) <= NEAR * scale, (b, j, i[b], ri[b])
    return i, ri


@pytest.mark.parametrize("B,L,d,K", [(37, 1000, 64, 5), (256, 4096, 768, 5), (300, 70001, 128, 3), (8, 9, 8, 8),
                                     (64, 5000, 64, 1)])
def test_topk_matches_oracle(dev, B, L, d, K):
    X = synth.make_X(B, d, 1).half()
    W = synth.make_W(L, d, 1).half()
    _check(dev, X, W, K)


def test_topk_config3_like(dev):
    """Batch 1024 and a label count that is not a multiple of the tile (as configs[3]), top-5."""
    B, L, d = 1024, 131072 + 121, 768
    X = synth.make_X(B, d, 2).half()
    W = synth.make_W(L, d, 2).half()
    _check(dev, X, W, 5)


def test_topk_exact_ties_and_pad_clamp(dev):
    B, L, d = 16, 2000, 64
    X = synth.make_X(B, d, 3).half()
    W = synth.make_W(L, d, 3).half()
    # identical label rows give bit-identical scores: the lower id must come first
    W[1500] = W[7]
    W[300] = W[7]
    W[1999] = W[7]
    W[7] *= 0  # make the group easy to find: set all four rows to a large common vector
    big = (X[0] * 4).half()
    for r in (7, 300, 1500, 1999):
        W[r] = big
    i, ri = _check(dev, X, W, 5)
    assert i[0, :4].tolist() == [7, 300, 1500, 1999]
    # padded labels (ids >= numy) are clamped to numy-1
    i2, ri2 = _check(dev, X, W, 5, numy=1990)
    assert i2[0, :4].tolist() == [7, 300, 1500, 1989]
    assert int(i2.max()) <= 1989


def test_topk_heavy_ties_across_label_groups(dev):
    """Integer-valued scores: thousands of exact ties per row, spread over all the label groups that
    share a row's score bound.  Ties with a published bound must still be admitted (a tying label of
    lower id ranks first), so indices and values must equal a stable descending sort exactly; the
    all-zero matrix is the extreme case (every score ties, and the bound is zero)."""
    g = torch.Generator().manual_seed(11)
    B, L, d = 70, 20011, 64
    X = torch.randint(0, 2, (B, d), generator=g).half()
    for W in (torch.randint(-1, 2, (L, d), generator=g).half(), torch.zeros(L, d).half()):
        Z = X.float() @ W.float().T  # small integers, exact in fp16 products and fp32 sums
        sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
        lay = XFCLayer(L, d, B, dev, weight=W)
        for K in (1, 5, 8):
            print(f"topk ties: B={B} L={L} K={K} zero={bool((W == 0).all())}", flush=True)
            v, i = lay.topk(X.to(dev), K)
            assert torch.equal(i.cpu(), si[:, :K])
            assert torch.equal(v.cpu(), sv[:, :K])


def test_topk_bounds_seeded_from_the_label_sample(dev):
    """Label counts large enough for the bounds to start from the K-th score over the first 2048 labels.
    The seed only has to be a lower bound: rows whose best labels all lie inside the sample (the seed
    then equals their K-th score up to the safety margin, and ties with it must survive), rows whose
    sample holds nothing but their worst scores, and a sample of equal scores."""
    g = torch.Generator().manual_seed(9)
    L, K = 600000, 5
    base = (torch.rand(L, generator=g) - 0.5).half()
    cases = []
    s = base.clone()
    s[:2048] = (1.0 + torch.rand(2048, generator=g)).half()          # the best labels are the sampled ones
    s[1000] = s[7] = s[2047] = s[:2048].max()                          # and the best score is shared
    cases.append(s)
    s = base.clone()
    s[:2048] = -4.0                                                    # the sample is useless
    s[599990] = s[300000] = 3.0
    cases.append(s)
    s = base.clone()
    s[:2048] = 0.25                                                    # a flat sample inside the range
    s[5000:5004] = 0.25                                                # later ties with the seed's score
    cases.append(s)
    for s in cases:
        X, W = _axis_problem(s, B=2)                                   # rows: 1 x and 2 x the scores
        lay = XFCLayer(L, 8, 2, dev, weight=W)
        v, i = lay.topk(X.to(dev), K)
        Z = X.float() @ W.float().T
        sv, si = torch.sort(Z, dim=1, descending=True, stable=True)
        assert torch.equal(i.cpu(), si[:, :K]) and torch.equal(v.cpu(), sv[:, :K])


def test_topk_rising_scores_exact_rescan(dev):
    """Scores that keep rising with the label id beat every threshold in every tile: the per-row
    candidate buffers overflow and the exact rescan path must produce the answer."""
    B, L, d = 40, 3000, 64
    X = synth.make_X(B, d, 4).half()
    base = X.float().mean(0)
    base = base / base.norm()
    ramp = torch.linspace(0.1, 4.0, L).unsqueeze(1)
    W = (ramp * base.unsqueeze(0) + 0.001 * synth.make_W(L, d, 4)).half()
    X = (X.float() * 0 + base.unsqueeze(0) + 0.05 * synth.make_X(B, d, 5)).half()
    _check(dev, X, W, 5)
    _check(dev, X, W, 8)


# ---- 8 < K <= 128: exact selection over fp16 logits (the final evaluation's K = 100, dl_base.py:817-818) ----
def _check_select(dev, X, W, K, numy=None, max_ws=None, vs_oracle=True):
    B, d = X.shape
    L = W.shape[0]
    lay = XFCLayer(L, d, B, dev, weight=W)
    print(f"topk-select: B={B} L={L} d={d} K={K} numy={numy} max_ws={max_ws}", flush=True)
    if max_ws is None:
        v, i = lay.topk(X.to(dev), K, numy)
    else:
        # a caller workspace smaller than all rows' logits, straight through the C ABI
        from renee_amd._lib import check, lib
        Xd = X.to(dev)
        ws = torch.empty(max_ws, dtype=torch.uint8, device=dev)
        v = torch.empty(B, K, device=dev, dtype=torch.float32)
        i = torch.empty(B, K, device=dev, dtype=torch.int64)
        check(lib().xfc_topk(Xd.data_ptr(), Xd.stride(0), lay.xfc_weight.data_ptr(), d, B, L, d,
                             L if numy is None else numy, K, v.data_ptr(), i.data_ptr(), ws.data_ptr(), ws.numel(),
                             torch.cuda.current_stream().cuda_stream), "xfc_topk")
    v, i = v.cpu(), i.cpu()
    # (a) the selection itself, against a stable sort of the same fp16 logits: exact
    Zg = lay.xfc_forward(X.to(dev)).float().cpu()
    sv, si = torch.sort(Zg, dim=1, descending=True, stable=True)
    ev, ei = sv[:, :K], si[:, :K]
    if numy is not None:
        ei = torch.where(ei >= numy, torch.full_like(ei, numy - 1), ei)
    assert torch.equal(v, ev)
    assert torch.equal(i, ei)
    if not vs_oracle:
        return i
    # (b) against the oracle's fp32 scores: values to fp16 rounding, indices except between near-equal scores
    Z = O.logits(X.float(), W.float())
    ov, oi = torch.sort(Z, dim=1, descending=True, stable=True)
    scale = float(Z.abs().max())
    assert torch.allclose(v, ov[:, :K], rtol=0, atol=1e-3 * scale)
    near = 1.5e-3 * scale
    kth = ov[:, K - 1]
    chosen = torch.gather(Z, 1, si[:, :K])
    assert bool((chosen >= kth[:, None] - near).all())          # nothing clearly below the K-th was taken
    must = Z > (kth[:, None] + near)                            # everything clearly above it was
    took = torch.zeros_like(must)
    took.scatter_(1, si[:, :K], True)
    assert bool((took | ~must).all())
    return i


@pytest.mark.parametrize("B,L,d,K", [(37, 1000, 64, 100), (256, 4096, 768, 100), (64, 70001, 128, 9),
                                     (5, 128, 8, 128), (3, 100, 8, 100), (9, 5000, 64, 500), (4, 1024, 8, 1024),
                                     (6, 30000, 32, 1024),
                                     # above 1024 the selection runs on its larger sort buffer (up to 8192)
                                     (5, 9000, 32, 1025), (3, 8192, 8, 8192), (4, 200003, 64, 5000), (2, 70001, 16, 8192)])
def test_topk_select_matches_sort_and_oracle(dev, B, L, d, K):
    X = synth.make_X(B, d, 4).half()
    W = synth.make_W(L, d, 4).half()
    _check_select(dev, X, W, K)


def test_topk_select_row_blocks_and_pad_clamp(dev):
    """A workspace smaller than all rows' logits: rows go in blocks of 256 (600 -> 256 + 256 + 88)."""
    B, L, d = 600, 3001, 64
    X = synth.make_X(B, d, 5).half()
    W = synth.make_W(L, d, 5).half()
    i = _check_select(dev, X, W, 100, numy=2990, max_ws=300 * 3008 * 2)
    assert int(i.max()) <= 2989


def _axis_problem(scores, B=3):
    """Logits that are exactly the given fp16 numbers: X rows are multiples of e_0, W[:, 0] = scores."""
    L = scores.numel()
    X = torch.zeros(B, 8, dtype=torch.float16)
    X[:, 0] = torch.tensor([1.0, 2.0, 0.5][:B], dtype=torch.float16)
    W = torch.zeros(L, 8, dtype=torch.float16)
    W[:, 0] = scores
    return X, W


def test_topk_select_crowded_bin_takes_the_refining_pass(dev):
    """4000 labels whose scores are the 32 fp16 numbers of one histogram bin [1, 1+32/1024): more than the
    sort capacity lie in the K-th value's bin, so its low key bits are histogrammed as well."""
    g = torch.Generator().manual_seed(6)
    L = 6000
    scores = (torch.rand(L, generator=g) * 0.5).half()
    crowd = torch.randperm(L, generator=g)[:4000]
    scores[crowd] = (1.0 + torch.randint(0, 32, (4000,), generator=g).float() / 1024).half()
    X, W = _axis_problem(scores)
    _check_select(dev, X, W, 100, vs_oracle=False)
    _check_select(dev, X, W, 128, vs_oracle=False)


def test_topk_select_sampled_bound_and_its_fallback(dev):
    """Rows long enough for the sampled first pass (every 8th 16 KB block at K = 100).  The sample's K-th
    score only has to be a lower bound: rows whose large scores all sit in the sampled blocks, rows whose
    sampled blocks hold only small scores (so that far more than the sort buffer lie above the bound and
    the full passes must take over), and a crowd of equal top scores must all give the exact answer."""
    g = torch.Generator().manual_seed(8)
    L, K, blk = 300000, 100, 8192
    in_sample = ((torch.arange(L) // blk) % 8 == 0)
    base = (torch.rand(L, generator=g) * 0.5).half()
    # (a) plain random scores
    X, W = _axis_problem(base.clone())
    _check_select(dev, X, W, K, vs_oracle=False)
    # (b) everything large lies in the sampled blocks: the bound is tight, few candidates
    s = base.clone()
    s[in_sample] = (1.0 + torch.rand(int(in_sample.sum()), generator=g)).half()
    X, W = _axis_problem(s)
    _check_select(dev, X, W, K, vs_oracle=False)
    # (c) the sampled blocks hold only small scores: the bound is loose and 200,000+ elements lie above it
    s = base.clone()
    s[~in_sample] = (1.0 + torch.rand(int((~in_sample).sum()), generator=g)).half()
    X, W = _axis_problem(s)
    _check_select(dev, X, W, K, vs_oracle=False)
    # (d) 5000 copies of the largest score, spread everywhere
    s = base.clone()
    s[torch.randperm(L, generator=g)[:5000]] = 2.0
    X, W = _axis_problem(s)
    i = _check_select(dev, X, W, K, vs_oracle=False)
    assert i[0].tolist() == sorted(i[0].tolist())  # equal scores come in label order


def test_topk_select_many_copies_of_the_kth_value(dev):
    """3000 labels share the K-th largest score (more than can be sorted): they are taken in label order;
    also a constant row, signed zeros and negative scores."""
    g = torch.Generator().manual_seed(7)
    L = 9000
    scores = (torch.rand(L, generator=g) * 0.5 - 1.0).half()      # negative background
    same = torch.randperm(L, generator=g)[:3000]
    scores[same] = 0.75
    top = torch.randperm(L, generator=g)[:40]
    scores[top] = (1.0 + torch.arange(40).float() / 64).half()    # 40 distinct larger scores (some overwrite 0.75)
    X, W = _axis_problem(scores)
    i = _check_select(dev, X, W, 100, vs_oracle=False)
    ties = sorted(set(same.tolist()) - set(top.tolist()))
    assert i[0, 40:].tolist() == ties[:60]
    # every logit equal (zero weights): the first K labels, in order; -0 and +0 are one value
    Wz = torch.zeros(L, 8, dtype=torch.float16)
    Xz = torch.zeros(2, 8, dtype=torch.float16)
    Xz[0, 0], Xz[1, 0] = 1.0, -1.0
    Wz[::2, 0] = -0.0
    iz = _check_select(dev, Xz, Wz, 100, vs_oracle=False)
    assert iz[0].tolist() == list(range(100)) and iz[1].tolist() == list(range(100))


def test_topk_select_large_k_with_heavy_ties(dev):
    """K above 1024 on rows that hold few distinct scores: the K-th value's copies outnumber the sort buffer and
    are taken in label order; the result is still the stable sort's."""
    B, L, d = 3, 60000, 8
    g = torch.Generator().manual_seed(9)
    X = torch.zeros(B, d)
    X[:, 0] = 1.0
    W = torch.zeros(L, d)
    W[:, 0] = torch.randint(0, 3, (L,), generator=g).float() * 0.25     # three distinct scores, ~20,000 copies each
    _check_select(dev, X.half(), W.half(), 6000, vs_oracle=False)
    _check_select(dev, X.half(), W.half(), 1500, vs_oracle=False)
