"""The reference's loss-module interface for the classifier on one GPU.

`BCELossMultiNode` here has the methods GenericModel.fit calls on the reference's class of that name
(dl_base.py:525-642): gather_embed, xfc_forward(embed, out) and
xfc_backward(embed_out, out, pos_x, pos_y, grad_input, use_custom), with the same argument meaning, so
that the XFC block of fit (dl_base.py:303-344) runs on an XFCLayer without being rewritten:

    loss_model = BCELossMultiNode(layer, compute_loss=not args.noloss, scaler=model.scaler)
    embed_out = loss_model.gather_embed(embed, batch_data)
    if do_forward: loss_model.xfc_forward(embed_out, layer.outsoft[0:bsz, :layer.numy])
    loss += loss_model.xfc_backward(embed_out, layer.outsoft[0:bsz, :layer.numy], z[0], z[1],
                                    layer.grad_input[0:bsz, :], not do_forward)
    loss_model.xfc_optimizer.step()        # a no-op when the update was fused into the dW pass

What differs from the reference, all of it behind the same calls: the sigmoid, the subtraction of the
positives and (on the reference's one step in LOSS_SAMPLE_FREQ) the sampled loss come out of one fused
pass over embed . W^T whether or not `out` already holds logits; grad_input is written in fp32 directly;
with accum == 1 the optimizer step happens inside the dW pass.  One GPU only: the collectives of the
reference's gather_embed and loss/grad all-reduces have no counterpart here.
"""
from __future__ import annotations

import torch

from .xfc import XFCLayer

LOSS_SAMPLE_FREQ = 100  # dl_base.py:144


class _FusedStep:
    """Stands where fit holds `self.xfc_optimizer` (dl_base.py:343): step() applies an accumulated
    gradient if there is one and does nothing when the update already ran inside the dW pass."""

    def __init__(self, owner: "BCELossMultiNode"):
        self._owner = owner

    def step(self) -> None:
        lay = self._owner.layer
        if lay.xfc_weight_grad is not None:
            lay.optimizer_step(lr=self._owner.lr)

    def zero_grad(self, set_to_none: bool = True) -> None:
        self._owner.layer.xfc_weight_grad = None


class BCELossMultiNode:
    def __init__(self, layer: XFCLayer, compute_loss: bool = False, scaler=None, accum: int = 1,
                 loss_sample_freq: int = LOSS_SAMPLE_FREQ):
        self.layer = layer
        self.compute_loss = bool(compute_loss)   # not args.noloss, dl_base.py:167
        self.scaler = scaler                     # anything with get_scale(), e.g. torch's GradScaler (dl_base.py:158)
        self.accum = int(accum)
        self.loss_sample_freq = int(loss_sample_freq)
        self.count = 0                           # the trainer's step counter (dl_base.py:172, :366)
        self.lr: float | None = None             # set per step from the schedule; None = the layer's lr
        self.loss = torch.zeros(1, device=layer.device, dtype=torch.float32)
        self.scale_bwd = 1.0
        self.xfc_optimizer = _FusedStep(self)

    # dl_base.py:535-566 with world_size == 1: only the fp16 conversion of the embeddings is left (the
    # weights are already resident in fp16)
    def gather_embed(self, embed: torch.Tensor, batch_data=None) -> torch.Tensor:
        return embed.to(device=self.layer.device, dtype=torch.float16)

    # dl_base.py:568-573
    def xfc_forward(self, embed: torch.Tensor, out: torch.Tensor) -> None:
        self.layer.xfc_forward(embed, out if out.shape[1] == self.layer.numy else out[:, : self.layer.numy])

    # dl_base.py:576-642
    def xfc_backward(self, embed_out: torch.Tensor, out: torch.Tensor, pos_x: torch.Tensor, pos_y: torch.Tensor,
                     grad_input: torch.Tensor, use_custom: bool = True) -> torch.Tensor:
        lay = self.layer
        sample = self.compute_loss and self.count % self.loss_sample_freq == 0
        # sigmoid(embed . W^T) - Y into `out` in one pass (use_custom or not: logits that xfc_forward may
        # have left in `out` are recomputed, not read), with the summed loss on the sampled steps (:578-583)
        lay.fwd_grad(embed_out, pos_x, pos_y, loss_out=self.loss if sample else None, out=out)
        if lay.xfc_weight_grad is None and self.scaler is not None:   # first micro-batch of a step (:598-600)
            self.scale_bwd = float(self.scaler.get_scale())
        bsz = embed_out.shape[0]
        lay.dx(bsz, grad_input, self.scale_bwd, out=out)              # :602-608
        if self.accum == 1:
            lay.dw_update(embed_out, lr=self.lr, out=out)             # :620-634 and the optimizer step of :343
        else:
            lay.dw_accumulate(embed_out, out=out)                     # :623 / :629
        return self.loss
