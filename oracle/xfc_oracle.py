"""CPU oracle for Renee's XFC (extreme fully-connected classifier) layer step.

TEST INFRASTRUCTURE ONLY.  This file restates, in plain torch CPU arithmetic
(float32 by default, float64 on request), the formulation that the reference
runs on the GPU.  Only the test-suite, the smoke check and the CPU-baseline leg
of the benchmark may import it; the product never does.

Each function cites the reference lines it follows (paths are relative to the
reference checkout):

  logits            dl_base.py:568-573     out = X @ W.T
  grad_logits       dl_base.py:590-594     sigmoid in place, then out[pos_x,pos_y] -= 1
  dx                dl_base.py:602-608     grad_input = scale * (G @ W)
  dw                dl_base.py:620-634     grad = G.T @ X  (beta=1 accumulates)
  sgd_momentum      main.py:178-179 (apex FusedSGD, momentum, weight_decay,
                    dampening 0, no Nesterov, wd before momentum) stepped at
                    dl_base.py:343
  step              dl_base.py:303-344     the sequence above for one batch
  step_accum        dl_base.py:318-340     same with row micro-batches ('--accum')
  topk              dl_base.py:736-756,782 iterative max (K<=5) / topk, pad clamp
  xfc_gemm          xfc_gemm_kernel.cu:49-51,59-65,113,151 and xfc_gemm.cpp:17-40
                    the six-argument native call: stride dispatch, alpha/beta
  sampled_loss      dl_base.py:578-583     sparse BCE loss (off under --noloss)
  pad_numy          main.py:76-89          label-count padding rule

How each one is pinned (see tests/test_oracle.py):
  logits/dw/dx      float64 brute-force loops on tiny shapes; torch.mm
  grad_logits       autograd of BCEWithLogitsLoss(reduction='sum') on a dense
                    target matrix (the reference's own default implementation,
                    dl_base.py:280-283), closed form 1/(1+e^-z)-y, set
                    semantics on duplicated positives vs a dense boolean mask
  sgd_momentum      torch.optim.SGD over several steps; closed form for steps
                    1 and 2.  apex FusedSGD itself (commit 5c9625c, install2.sh)
                    is not installed here: PARITY UNPINNED against apex, pinned
                    against torch.optim.SGD which apex documents it matches.
  topk              torch.sort with explicit tie handling; lowest-index rule
  xfc_gemm          the three call sites' algebra vs logits/dw/dx; CUTLASS's
                    own rounding (fp16 sigmoid output) is PARITY UNPINNED
                    bit-for-bit (CUTLASS is not vendored), pinned to 1e-3.
  sampled_loss      BCEWithLogitsLoss(reduction='sum') value
"""
from __future__ import annotations

import torch


def logits(X: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
    """Z = X . W^T  (dl_base.py:572)."""
    return X @ W.t()


def grad_logits(Z: torch.Tensor, pos_x: torch.Tensor, pos_y: torch.Tensor) -> torch.Tensor:
    """G = sigmoid(Z); G[pos_x, pos_y] -= 1  (dl_base.py:593-594).

    The indexed subtraction is a gather / subtract / non-accumulating scatter:
    a (row, col) pair listed twice is lowered by 1 once.
    """
    G = torch.sigmoid(Z)
    if pos_x.numel():
        G[pos_x.long(), pos_y.long()] -= 1.0
    return G


def dx(G: torch.Tensor, W: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """grad_input = scale * G . W  (dl_base.py:606/608, alpha = loss scale)."""
    return scale * (G @ W)


def dw(G: torch.Tensor, X: torch.Tensor, acc: torch.Tensor | None = None) -> torch.Tensor:
    """grad = G^T . X, optionally added to an earlier micro-batch's grad
    (dl_base.py:623-633)."""
    g = G.t() @ X
    return g if acc is None else acc + g


def sgd_momentum(W, M, dW, lr: float, momentum: float, weight_decay: float = 0.0):
    """One SGD-momentum step, returning (W_new, M_new).

    g = dW + wd*W ; M = mu*M + g ; W = W - lr*M   (main.py:178-179, dl_base.py:343;
    dampening 0, no Nesterov, weight decay applied before momentum).  With M
    preallocated as zeros the first step gives M = g, which is what the
    optimizer's "no buffer yet" branch produces.
    """
    g = dW + weight_decay * W if weight_decay != 0.0 else dW
    M_new = momentum * M + g
    W_new = W - lr * M_new
    return W_new, M_new


def step(X, W, M, pos_x, pos_y, lr, momentum, weight_decay=0.0, scale=1.0):
    """One XFC step (dl_base.py:303-344, accum == 1).  Returns a dict with
    G, dX, dW, W_new, M_new.  dX uses W before the update."""
    Z = logits(X, W)
    G = grad_logits(Z, pos_x, pos_y)
    dX = dx(G, W, scale)
    dW = dw(G, X)
    W_new, M_new = sgd_momentum(W, M, dW, lr, momentum, weight_decay)
    return {"G": G, "dX": dX, "dW": dW, "W": W_new, "M": M_new}


def step_accum(X, W, M, pos_x, pos_y, index, xfc_batch_size, lr, momentum,
               weight_decay=0.0, scale=1.0):
    """Split gradient accumulation (dl_base.py:318-340): rows are processed
    xfc_batch_size at a time; `index` holds the nnz offsets of each micro-batch
    and pos_x is local to its micro-batch (dl_base.py:939-959).  dW accumulates,
    the optimizer steps once."""
    bsz = X.shape[0]
    dX = torch.empty(bsz, W.shape[1], dtype=X.dtype)
    grad = None
    start, i = 0, 0
    while start < bsz:
        end = min(start + xfc_batch_size, bsz)
        sl = slice(int(index[i]), int(index[i + 1]))
        G = grad_logits(logits(X[start:end], W), pos_x[sl], pos_y[sl])
        dX[start:end] = dx(G, W, scale)
        grad = dw(G, X[start:end], grad)
        start, i = end, i + 1
    W_new, M_new = sgd_momentum(W, M, grad, lr, momentum, weight_decay)
    return {"dX": dX, "dW": grad, "W": W_new, "M": M_new}


def topk(X, W, K: int = 5, numy: int | None = None):
    """Exact top-K labels per row (dl_base.py:736-756): for K <= 5 the maximum
    is taken K times, overwriting each winner with the dtype's lowest value;
    torch.max returns the first (lowest-index) maximum.  Indices at or past
    `numy` (padded labels) are clamped to numy-1 (dl_base.py:782)."""
    out = logits(X, W).clone()
    if K <= 5:
        vals, inds = [], []
        rows = torch.arange(out.shape[0])
        lowest = torch.finfo(out.dtype).min
        for _ in range(K):
            v, i = torch.max(out, 1)
            vals.append(v)
            inds.append(i)
            out[rows, i] = lowest
        top_v, top_i = torch.stack(vals, 1), torch.stack(inds, 1)
    else:
        top_v, top_i = torch.topk(out, K)
    if numy is not None:
        top_i = torch.where(top_i >= numy, torch.full_like(top_i, numy - 1), top_i)
    return top_v, top_i


def xfc_gemm(mat_in1, mat_in2, mat_out, alpha: float, beta: float, apply_sigmoid: bool) -> None:
    """The native six-argument call, in place on mat_out.

    M, N come from mat_out, K from mat_in2.size(0) (xfc_gemm_kernel.cu:49-51).
    The layout is chosen from the strides of the views the caller passes:
      apply_sigmoid, in1 row-major, in2 column-major  -> out = sigmoid(a*in1@in2 + b*out)   (:59-100)
      in1 column-major, in2 row-major                 -> out = a*in1@in2 + b*out  (fp32 out) (:113-150)
      in1 row-major, in2 row-major                    -> same algebra, split-K               (:151-241)
    Anything else is rejected (:102-103, :243-244).  With beta == 0 the old
    contents of mat_out are not read.
    """
    for t in (mat_in1, mat_in2, mat_out):
        if t.dim() != 2:
            raise RuntimeError("expected 2D tensor")  # xfc_gemm.cpp:28-30
    s1, s2 = mat_in1.stride(), mat_in2.stride()
    if apply_sigmoid:
        ok = s1[1] == 1 and s2[0] == 1
    else:
        ok = (s1[0] == 1 and s2[1] == 1) or (s1[1] == 1 and s2[1] == 1)
    if not ok:
        raise RuntimeError("unsupported operand layout")
    acc = alpha * (mat_in1.float() @ mat_in2.float())
    if beta != 0.0:
        acc = acc + beta * mat_out.float()
    if apply_sigmoid:
        acc = torch.sigmoid(acc)
    mat_out.copy_(acc.to(mat_out.dtype))


def sampled_loss(Z, pos_x, pos_y) -> torch.Tensor:
    """Sparse BCE-with-logits loss, summed (dl_base.py:578-583):
    sum(max(z,0)) - sum(z[pos]) + sum(log(1+exp(-|z|)))."""
    loss = Z.clamp(min=0.0).sum(dtype=torch.float32)
    loss = loss - Z[pos_x.long(), pos_y.long()].sum(dtype=torch.float32)
    loss = loss + (1 + (-torch.abs(Z.float())).exp()).log().sum(dtype=torch.float32)
    return loss


def pad_numy(numy: int, world_size: int = 1) -> int:
    """Label-count padding (main.py:76-89): up to a multiple of world_size, then
    so that the per-GPU share is a multiple of 16."""
    padded = numy
    if padded % world_size != 0:
        padded = world_size * ((numy + world_size - 1) // world_size)
    per_gpu = padded // world_size
    if per_gpu % 16 != 0:
        padded = world_size * 16 * ((per_gpu + 15) // 16)
    return padded
