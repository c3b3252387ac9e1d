"""Pooling wrapper, additive-unpooling wrapper and the hourglass that joins them around a submodule
(reference: flash3dxfmr/layers/hourglass.py)."""
from typing import Tuple

import torch
import torch.cuda.nvtx as nvtx
from torch import nn

from ..psh import batching as f3dbatch
from ..psh import dev_context as f3ddev
from ..psh import subbuck as f3dsubbuck
from . import pooling, unpool
from .nn_ops import Linear, apply_norm_act, fused_row_norm


class PoolingWrapper(nn.Module):
    """proj (Linear) -> in-bucket pooling -> optional norm -> optional activation.
    Returns (reduced_feat, projected_feat, buffers); projected_feat is the skip connection."""
    NVTX_SCOPE = "PoolingWrapper"

    def __init__(self, in_channels: int, out_channels: int, red_op, out_align, norm_layer: callable = None,
                 act_layer: callable = None, subbuck_size: int = 2):
        super().__init__()
        self.proj = Linear(in_channels, out_channels)
        self.pooling = pooling.InbucketPoolingLayer(red_op, out_alignment=out_align, subbuck_size=subbuck_size)
        self.norm = norm_layer(out_channels) if norm_layer is not None else None
        self.act = act_layer() if act_layer is not None else None

    def forward(self, coords, input_feat, seps) -> Tuple[torch.Tensor, torch.Tensor, f3dsubbuck.SubbuckBuffers]:
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        projected = self.proj(input_feat)
        post = fused_row_norm(self.norm, self.act, projected)
        if post is not None:     # inference: the norm (and activation) runs inside the reduce kernel
            reduced_feat, subbuffers = self.pooling(coords, projected, seps, post=post)
        else:
            reduced_feat, subbuffers = self.pooling(coords, projected, seps)
            reduced_feat = apply_norm_act(self.norm, self.act, reduced_feat)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return reduced_feat, projected, subbuffers


class AdditiveUnpoolingWrapper(nn.Module):
    """proj(down) and proj_skip(residual) (Linear -> norm -> act each), then additive unpooling"""
    NVTX_SCOPE = "AdditiveUnpoolingWrapper"

    def __init__(self, in_channels: int, skip_channels: int, out_channels: int, subbuck_size: int = 2,
                 norm_layer: callable = None, act_layer: callable = None):
        super().__init__()
        self.proj = nn.Sequential(Linear(in_channels, out_channels))
        self.proj_skip = nn.Sequential(Linear(skip_channels, out_channels))
        if norm_layer is not None:
            self.proj.add_module("norm", norm_layer(out_channels))
            self.proj_skip.add_module("norm", norm_layer(out_channels))
        if act_layer is not None:
            self.proj.add_module("act", act_layer())
            self.proj_skip.add_module("act", act_layer())
        self.unpool = unpool.AdditiveUnpoolLayer(subbuck_size)

    @staticmethod
    def _branch(seq: nn.Sequential, x):
        y = seq[0](x)
        return apply_norm_act(getattr(seq, "norm", None), getattr(seq, "act", None), y)

    def forward(self, residual, down, buffers: f3dsubbuck.SubbuckBuffers) -> torch.Tensor:
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        raw_down, raw_skip = self.proj[0](down), self.proj_skip[0](residual)
        nd = fused_row_norm(getattr(self.proj, "norm", None), getattr(self.proj, "act", None), raw_down)
        ns = fused_row_norm(getattr(self.proj_skip, "norm", None), getattr(self.proj_skip, "act", None), raw_skip)
        if nd is not None and ns is not None and nd[0][0] == ns[0][0] and nd[1] == ns[1]:
            # inference: both branches' norm (and activation) run inside the unpooling kernel
            output = self.unpool(raw_skip, raw_down, buffers, norms=(ns[0], nd[0], nd[1]))
        else:
            proj_down = apply_norm_act(getattr(self.proj, "norm", None), getattr(self.proj, "act", None), raw_down)
            proj_skip = apply_norm_act(getattr(self.proj_skip, "norm", None), getattr(self.proj_skip, "act", None), raw_skip)
            output = self.unpool(proj_skip, proj_down, buffers)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return output


class HourglassModule(nn.Module):
    """pool -> submodule(reduced_coord, reduced_feat, reduced_sep) -> unpool(skip, submodule output)"""
    NVTX_SCOPE = "HourglassModule"

    def __init__(self, pooling_in_channels: int, pooling_out_channels: int, pooling_reduction_op,
                 pooling_length_alignment: int, unpooling_in_channels: int, unpooling_out_channels: int,
                 pooling_norm_layer: callable = None, pooling_act_layer: callable = None,
                 unpooling_norm_layer: callable = None, unpooling_act_layer: callable = None,
                 submodule: nn.Module = None, subbuck_size: int = 2):
        super().__init__()
        if submodule is None:
            raise ValueError("A submodule must be provided for HourglassModule.")
        self.pooling = PoolingWrapper(pooling_in_channels, pooling_out_channels, pooling_reduction_op,
                                      pooling_length_alignment, pooling_norm_layer, pooling_act_layer, subbuck_size)
        self.unpooling = AdditiveUnpoolingWrapper(unpooling_in_channels, pooling_out_channels, unpooling_out_channels,
                                                  subbuck_size, unpooling_norm_layer, unpooling_act_layer)
        self.submodule = submodule

    def forward(self, coords, input_feat, seps) -> torch.Tensor:
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        reduced_feat, residual_feat, buffers = self.pooling(coords, input_feat, seps)
        # The reduced length is rounded up for the next level's attention buckets; the extra
        # (zero-filled) rows are handed on as part of the last cloud so that every row of every
        # level belongs to a cloud and is written by the unpooling on the way back.
        sub_sep = buffers.reduced_sep
        if buffers.reduced_feat.shape[0] != buffers.unpool_ind.shape[0]:
            sub_sep = f3dbatch.with_last_separator(sub_sep, buffers.reduced_feat.shape[0])
        sub_out = self.submodule(buffers.reduced_coord, reduced_feat, sub_sep)
        output = self.unpooling(residual_feat, sub_out, buffers)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return output
