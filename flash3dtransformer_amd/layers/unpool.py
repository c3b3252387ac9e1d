"""Additive unpooling layer (reference: flash3dxfmr/layers/unpool.py)."""
import torch
from torch import nn
from torch.autograd import Function

from ..lib import pshattn
from ..psh.subbuck import SubbuckBuffers, UnpoolBuffers, UnpoolGradients


class AdditiveUnpoolFunction(Function):
    """up[r] = down[i] + residual[r] for every point r that pooled into row i (unpool_ind)"""

    @staticmethod
    def forward(ctx, residual_feat, down_feat, buffers: SubbuckBuffers, subbuck_size: int) -> torch.Tensor:
        buf = UnpoolBuffers.create_unpool_buff(residual_feat)
        pshattn.additive_unpool_fwd(residual_feat, down_feat, buf.up_add_feat, buffers.unpool_ind, subbuck_size)
        ctx.subbuck_size = subbuck_size
        ctx.subbuck_buffers = buffers
        ctx.down_len = down_feat.shape[0]
        return buf.up_add_feat

    @staticmethod
    def backward(ctx, grad_up_add_feat):
        """grad_res = the output gradient (identity branch), grad_down[i] = sum over the points pooled into row i
        (reference: layers/unpool.py:50-77)"""
        g = grad_up_add_feat if grad_up_add_feat.dtype == torch.bfloat16 else grad_up_add_feat.to(torch.bfloat16)
        g = g.contiguous()
        grads = UnpoolGradients.create_unpool_grad(g, ctx.subbuck_buffers, ctx.down_len)
        pshattn.additive_unpool_bwd(grads.grad_res, grads.grad_down, g, ctx.subbuck_buffers.unpool_ind, ctx.subbuck_size)
        return grads.grad_res, grads.grad_down, None, None


class AdditiveUnpoolLayer(nn.Module):
    def __init__(self, subbuck_size: int = 2) -> None:
        super().__init__()
        assert 1 <= subbuck_size <= 1024, f"subbuck_size must be in [1, 1024], input is {subbuck_size}"
        self.subbuck_size = subbuck_size

    def forward(self, residual_feat, down_feat, buffers: SubbuckBuffers, norms=None) -> torch.Tensor:
        """norms: (descriptor of the residual branch, descriptor of the down branch, activation name), descriptors from
        nn_ops.fused_row_norm: the two tensors are then normalised by the unpooling kernel as it reads them (inference
        only: no autograd graph is recorded)"""
        to = lambda t: (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)).contiguous()
        if norms is None:
            return AdditiveUnpoolFunction.apply(to(residual_feat), to(down_feat), buffers, self.subbuck_size)
        res = to(residual_feat)
        buf = UnpoolBuffers.create_unpool_buff(res)
        pshattn.additive_unpool_norm_fwd(res, to(down_feat), buf.up_add_feat, buffers.unpool_ind, self.subbuck_size,
                                         norms[0], norms[1], norms[2])
        return buf.up_add_feat
