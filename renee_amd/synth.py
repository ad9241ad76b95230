"""Seeded synthetic inputs for the XFC step, in the shapes the benchmark names.

X   : B x d, i.i.d. N(0,1), each row L2-normalised.
W   : L x d, i.i.d. N(0, 0.02^2)  (the reference's init, dl_base.py:185-187).
Y   : sparse positives.  Row b gets k_b labels, k_b in [1, kmax] from a truncated
      geometric distribution whose parameter is solved for the requested mean;
      label ids are i.i.d. draws from the finite-support Zipf law p(r) ~ r^-s,
      r = 1..L (inverse CDF on the normalised cumulative sum; id = r-1), then
      de-duplicated and sorted within the row.  Stored both as CSR (rowptr,
      colidx, int32) and as the reference's row-sorted COO pair (pos_x, pos_y,
      int64; dl_base.py:934-936).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

# (B, L, kmax, mean positives, Zipf exponent) of the five benchmark configurations; d = 768.
CONFIGS = {
    0: dict(B=32, L=131072, kmax=8, kmean=2.3, zipf=1.1),
    1: dict(B=512, L=131072, kmax=8, kmean=2.3, zipf=1.1),
    2: dict(B=512, L=1310720, kmax=20, kmean=5.0, zipf=1.0),
    3: dict(B=1024, L=2812281, kmax=30, kmean=8.0, zipf=0.9),
    4: dict(B=1024, L=16777216, kmax=50, kmean=5.0, zipf=1.0),
}
D_MODEL = 768


@dataclass
class Positives:
    rowptr: np.ndarray  # int32 [B+1]
    colidx: np.ndarray  # int32 [nnz]

    @property
    def nnz(self) -> int:
        return int(self.colidx.shape[0])

    def coo(self):
        """Row-sorted COO (pos_x, pos_y) as int64 torch tensors."""
        counts = np.diff(self.rowptr)
        rows = np.repeat(np.arange(counts.shape[0], dtype=np.int64), counts)
        return torch.from_numpy(rows), torch.from_numpy(self.colidx.astype(np.int64))


def _geometric_q(kmax: int, mean: float) -> float:
    """q such that P(k) ~ q^(k-1), k = 1..kmax, has the given mean."""
    ks = np.arange(1, kmax + 1, dtype=np.float64)

    def m(q):
        p = q ** (ks - 1)
        return float((ks * p).sum() / p.sum())

    lo, hi = 1e-9, 1.0
    if mean >= m(hi):
        return 1.0
    for _ in range(200):
        mid = 0.5 * (lo + hi)
        if m(mid) < mean:
            lo = mid
        else:
            hi = mid
    return 0.5 * (lo + hi)


def make_positives(B: int, L: int, kmax: int, kmean: float, zipf: float, seed: int = 0) -> Positives:
    rng = np.random.default_rng(seed)
    ks = np.arange(1, kmax + 1)
    pk = _geometric_q(kmax, kmean) ** (ks - 1.0)
    pk /= pk.sum()
    k = rng.choice(ks, size=B, p=pk)
    cdf = np.cumsum(np.arange(1, L + 1, dtype=np.float64) ** (-zipf))
    cdf /= cdf[-1]
    rowptr = np.zeros(B + 1, dtype=np.int32)
    cols = []
    for b in range(B):
        ids = np.searchsorted(cdf, rng.random(int(k[b])), side="left")
        ids = np.unique(np.minimum(ids, L - 1)).astype(np.int32)
        cols.append(ids)
        rowptr[b + 1] = rowptr[b] + ids.shape[0]
    return Positives(rowptr=rowptr, colidx=np.concatenate(cols) if cols else np.zeros(0, np.int32))


def make_X(B: int, d: int = D_MODEL, seed: int = 0, device="cpu", dtype=torch.float32) -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed(1000 + seed)
    X = torch.randn(B, d, generator=g, device=device, dtype=torch.float32)
    X = X / X.norm(dim=1, keepdim=True)
    return X.to(dtype)


def make_W(L: int, d: int = D_MODEL, seed: int = 0, device="cpu", dtype=torch.float32,
           chunk_rows: int = 1 << 20) -> torch.Tensor:
    """N(0, 0.02^2) label matrix, generated in row chunks so that the fp32
    temporaries stay small next to a 25 GB fp16 matrix."""
    g = torch.Generator(device=device)
    g.manual_seed(2000 + seed)
    W = torch.empty(L, d, device=device, dtype=dtype)
    for r0 in range(0, L, chunk_rows):
        r1 = min(L, r0 + chunk_rows)
        W[r0:r1] = (torch.randn(r1 - r0, d, generator=g, device=device, dtype=torch.float32) * 0.02).to(dtype)
    return W


def make_config(cfg: int, seed: int = 0, device="cpu", dtype=torch.float32, d: int = D_MODEL):
    """(X, W, Positives) for one of the benchmark configurations."""
    c = CONFIGS[cfg]
    X = make_X(c["B"], d, seed, device, dtype)
    W = make_W(c["L"], d, seed, device, dtype)
    P = make_positives(c["B"], c["L"], c["kmax"], c["kmean"], c["zipf"], seed)
    return X, W, P
