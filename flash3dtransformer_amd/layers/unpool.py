"""Additive unpooling layer (reference: flash3dxfmr/layers/unpool.py)."""
import torch
from torch import nn
from torch.autograd import Function

from ..lib import pshattn
from ..psh.subbuck import SubbuckBuffers, UnpoolBuffers


class AdditiveUnpoolFunction(Function):
    """up[r] = down[i] + residual[r] for every point r that pooled into row i (unpool_ind)"""

    @staticmethod
    def forward(ctx, residual_feat, down_feat, buffers: SubbuckBuffers, subbuck_size: int) -> torch.Tensor:
        buf = UnpoolBuffers.create_unpool_buff(residual_feat)
        pshattn.additive_unpool_fwd(residual_feat, down_feat, buf.up_add_feat, buffers.unpool_ind, subbuck_size)
        ctx.subbuck_size = subbuck_size
        return buf.up_add_feat

    @staticmethod
    def backward(ctx, grad_up_add_feat):
        raise NotImplementedError("additive_unpool_bwd: the gfx950 library implements the forward pass only")


class AdditiveUnpoolLayer(nn.Module):
    def __init__(self, subbuck_size: int = 2) -> None:
        super().__init__()
        assert 1 <= subbuck_size <= 1024, f"subbuck_size must be in [1, 1024], input is {subbuck_size}"
        self.subbuck_size = subbuck_size

    def forward(self, residual_feat, down_feat, buffers: SubbuckBuffers) -> torch.Tensor:
        to = lambda t: (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)).contiguous()
        return AdditiveUnpoolFunction.apply(to(residual_feat), to(down_feat), buffers, self.subbuck_size)
