"""In-bucket pooling layer (reference: flash3dxfmr/layers/pooling.py)."""
import torch
from torch import nn
from torch.autograd import Function

from ..lib import pshattn
from ..psh import batching as f3dbatch
from ..psh import subbuck as f3dsubbuck

NUM_VOX = 0xFFFF


class SubbuckReduceFunction(Function):
    """(coords, feat, seps) -> (reduced_feat, SubbuckBuffers): groups of `subbuck_size` spatially
    close points of every cloud are reduced to one row (0 mean, 1 sum, 2 min, 3 max).  The buffers
    carry reduced_coord, reduced_sep and unpool_ind for the next level and for unpooling."""

    @staticmethod
    def forward(ctx, coords, input_feat, seps, subbuck_size, reduction_op, out_alignment=1):
        max_n = f3dbatch.max_inslen_from_seps(seps)
        sb = f3dsubbuck.SubbuckBuffers.create_subbuck_buff(coords, input_feat, seps, subbuck_size,
                                                           out_alignment=out_alignment)
        pshattn.batch_subbuck_reduce(coords, input_feat, seps, max_n, subbuck_size, NUM_VOX, sb.bbox_min, sb.bbox_max,
                                     sb.subbuck_id, sb.subbuck_off, sb.reduced_sep, sb.reduced_coord, sb.reduced_feat,
                                     sb.unpool_ind, 1, reduction_op)
        ctx.save_for_backward(input_feat, sb.unpool_ind)
        ctx.subbuck_size, ctx.reduction_op = subbuck_size, reduction_op
        sb.remove_unused_buffers()
        ctx.mark_non_differentiable(sb.reduced_coord)
        return sb.reduced_feat, sb

    @staticmethod
    def backward(ctx, grad_reduced_feat, grad_buffers):
        """only input_feat is differentiable (reference: layers/pooling.py:87-116)"""
        input_feat, unpool_ind = ctx.saved_tensors
        g = grad_reduced_feat if grad_reduced_feat.dtype == torch.bfloat16 else grad_reduced_feat.to(torch.bfloat16)
        grad_input_feat = torch.zeros_like(input_feat)
        pshattn.batch_subbuck_reduce_backward(g.contiguous(), input_feat, unpool_ind, grad_input_feat, ctx.subbuck_size,
                                              ctx.reduction_op)
        return None, grad_input_feat, None, None, None, None


class InbucketPoolingLayer(nn.Module):
    REDOP_MAP = {"mean": 0, "sum": 1, "min": 2, "max": 3}

    def __init__(self, reduction_op, out_alignment=1024, subbuck_size=2):
        """The reference restricts subbuck_size to 2 (pooling.py:159); the kernels here take any size
        from 1 to 1024, e.g. 8 for a 2x2x2-like reduction."""
        super().__init__()
        assert 1 <= subbuck_size <= 1024, f"subbuck_size must be in [1, 1024], input is {subbuck_size}"
        if isinstance(reduction_op, str):
            assert reduction_op in self.REDOP_MAP, f"Unsupported reduction op name:{reduction_op}"
            reduction_op = self.REDOP_MAP[reduction_op]
        self.reduction_op = int(reduction_op)
        self.out_align = out_alignment
        self.subbuck_size = subbuck_size

    def forward(self, coords, input_feat, seps, post=None):
        """post: (descriptor, activation name) from nn_ops.fused_row_norm: the norm / activation that follows the
        pooling is then applied by the reduce kernel itself (inference only: no autograd graph is recorded)"""
        feat = input_feat if input_feat.dtype == torch.bfloat16 else input_feat.to(torch.bfloat16)
        if post is None:
            return SubbuckReduceFunction.apply(coords, feat.contiguous(), seps, self.subbuck_size, self.reduction_op,
                                               self.out_align)
        feat = feat.contiguous()
        max_n = f3dbatch.max_inslen_from_seps(seps)
        sb = f3dsubbuck.SubbuckBuffers.create_subbuck_buff(coords, feat, seps, self.subbuck_size,
                                                           out_alignment=self.out_align)
        pshattn.subbuck_build(coords, seps, max_n, self.subbuck_size, NUM_VOX, sb.subbuck_id, sb.subbuck_off,
                              sb.reduced_sep, sb.reduced_coord, sb.unpool_ind)
        pshattn.reduce_feat_norm(feat, coords.shape[0], sb.unpool_ind, sb.reduced_feat, self.subbuck_size,
                                 self.reduction_op, post[0], post[1])
        sb.remove_unused_buffers()
        return sb.reduced_feat, sb
