"""Writes tests/golden/xfc_step_small.npz: inputs and expected outputs of two
XFC steps on a tiny problem.

The expected values do NOT come from oracle/xfc_oracle.py.  They come from the
formulation the reference itself offers as its baseline (`--default-impl`,
dl_base.py:274-295, :519-522): logits by matmul, a dense 0/1 target matrix,
BCEWithLogitsLoss(reduction='sum'), autograd for dZ, dW and dX, and
torch.optim.SGD(momentum, weight_decay) for the update (the optimizer apex
FusedSGD is documented to match, main.py:178-179) -- all in float64.
Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    torch.manual_seed(1234)
    B, L, d = 20, 75, 32
    lr, mu, wd, scale = 0.05, 0.9, 1e-3, 8.0
    X = torch.randn(B, d, dtype=torch.float64)
    X = (X / X.norm(dim=1, keepdim=True)).half().double()  # exactly representable in fp16
    W0 = (torch.randn(L, d, dtype=torch.float64) * 0.02).half().double()
    rng = np.random.default_rng(7)
    rows, cols = [], []
    for b in range(B):
        k = int(rng.integers(0, 5))  # some rows have no positives
        c = np.unique(rng.integers(0, L, size=k))
        rows += [b] * len(c)
        cols += list(c)
    rows += [3, 3]            # a duplicated pair: must count once
    cols += [L - 1, L - 1]    # ... in the last (ragged) label column
    pos_x = torch.tensor(rows, dtype=torch.int64)
    pos_y = torch.tensor(cols, dtype=torch.int64)
    Y = torch.zeros(B, L, dtype=torch.float64)
    Y[pos_x, pos_y] = 1.0

    W = torch.nn.Parameter(W0.clone())
    opt = torch.optim.SGD([W], lr=lr, momentum=mu, weight_decay=wd)
    out = {}
    for step in (1, 2):
        Xp = X.clone().requires_grad_(True)
        Z = Xp @ W.t()
        Z.retain_grad()
        loss = torch.nn.BCEWithLogitsLoss(reduction="sum")(Z, Y)
        opt.zero_grad()
        loss.backward()
        out[f"G{step}"] = Z.grad.numpy().copy()
        out[f"dW{step}"] = W.grad.numpy().copy()
        out[f"dX{step}"] = (scale * Xp.grad).numpy().copy()
        out[f"loss{step}"] = np.array(loss.item())
        opt.step()
        out[f"W{step}"] = W.detach().numpy().copy()
        out[f"M{step}"] = opt.state[W]["momentum_buffer"].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "xfc_step_small.npz"), X=X.numpy(), W0=W0.numpy(),
                        pos_x=pos_x.numpy(), pos_y=pos_y.numpy(),
                        hyper=np.array([lr, mu, wd, scale]), **out)
    print("wrote xfc_step_small.npz")


if __name__ == "__main__":
    main()
