"""The classifier step as a differentiable scalar, for trainers that drive the encoder with
`loss.backward()` instead of handing grad_input to `embed.backward` by hand (dl_base.py:360).

    loss = xfc_loss(embed, layer, pos_x, pos_y, scale=scaler.get_scale(), lr=current_lr)
    loss.backward()          # embed.grad += scale * G . W, the reference's grad_input

The forward call runs the whole XFC step on the layer (G, grad_input, dW fused with the SGD-momentum
update: dl_base.py:576-642 and :343), exactly as XFCLayer.xfc_backward does; the returned tensor is the
summed BCE-with-logits loss of the batch when compute_loss is set (dl_base.py:578-583) and zero under
--noloss, where the loss is never formed.  Its gradient with respect to `embed` is grad_input either way.
The label matrix is not a torch parameter: it is updated inside the call, as in the reference, whose
classifier runs under no_grad (dl_base.py:303).
"""
from __future__ import annotations

import torch

from .xfc import XFCLayer


class _XFCStep(torch.autograd.Function):
    @staticmethod
    def forward(ctx, embed, layer, pos_x, pos_y, scale, lr, compute_loss, accumulate):
        bsz = embed.shape[0]
        loss = torch.zeros(1, device=layer.device, dtype=torch.float32)
        layer.fwd_grad(embed, pos_x, pos_y, loss_out=loss if compute_loss else None)
        gi = layer.dx(bsz, None, scale)
        if accumulate:
            layer.dw_accumulate(embed)
        else:
            layer.dw_update(embed, lr=lr)
        # the layer's grad_input buffer is reused by the next step: keep this step's values
        ctx.save_for_backward(gi.clone())
        ctx.embed_dtype, ctx.embed_device = embed.dtype, embed.device
        return loss.reshape(())

    @staticmethod
    def backward(ctx, grad_out):
        (gi,) = ctx.saved_tensors
        g = (gi * grad_out.to(gi.device)).to(device=ctx.embed_device, dtype=ctx.embed_dtype)
        return g, None, None, None, None, None, None, None


def xfc_loss(embed: torch.Tensor, layer: XFCLayer, pos_x: torch.Tensor, pos_y: torch.Tensor, scale: float = 1.0,
             lr: float | None = None, compute_loss: bool = False, accumulate: bool = False) -> torch.Tensor:
    """One classifier step on `layer` for the batch `embed` (batch, dims) with positives (pos_x, pos_y);
    returns a scalar whose backward() sends scale * G . W into embed's graph."""
    return _XFCStep.apply(embed, layer, pos_x, pos_y, float(scale), lr, bool(compute_loss), bool(accumulate))
