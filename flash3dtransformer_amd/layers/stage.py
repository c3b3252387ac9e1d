"""Transformer block and stage (reference: flash3dxfmr/layers/stage.py)."""
from dataclasses import dataclass
from typing import List

import torch
import torch.cuda.nvtx as nvtx
from torch import nn

from ..psh import bucket_scope
from ..psh import dev_context as f3ddev
from . import buck_swin, elem_wise
from .nn_ops import CoordEmbedding, apply_norm, is_fusable_layernorm, materialize


@dataclass(slots=True)
class XFMRSpecs:
    channels: int
    hid_channels: int
    num_heads: int
    qkv_bias: bool
    swin_plan: bucket_scope.SwinPlan
    norm_layer: callable


class XFMR(nn.Module):
    """mid = proj(attention(qkv(norm(x)))) + x;  out = MLP(mid) + mid   (stage.py:71-102 of the reference).
    Takes the (coord, feat, sep) triplet of the submodule interface and uses only `feat`."""
    NVTX_SCOPE = "XFMR"

    def __init__(self, channels: int, hid_chann: int, num_heads: int, buck_size: int, qkv_bias: bool,
                 swin_plan: bucket_scope.SwinPlan, norm_layer: callable, mlp_activation: str = "swiglu"):
        super().__init__()
        self.set_chnn = channels
        self.swin_plan = swin_plan
        self.norm = norm_layer(channels)
        self.bwa = buck_swin.BucketSwinAttentionModule(channels, num_heads, buck_size, qkv_bias)
        self.mlp = elem_wise.MLP(channels, hid_chann, mlp_activation)

    def forward(self, reduced_coord, reduced_feat: torch.Tensor, reduced_sep) -> torch.Tensor:
        assert reduced_feat.dim() == 2, f"Expect input features have two axes [N, C], but got shape={reduced_feat.shape}"
        N, C = reduced_feat.shape
        assert C == self.set_chnn, f"Expect input feat_dim={self.set_chnn}, but got {C}"
        scope_bucks = self.swin_plan.gen_scopes_from_plan(N, reduced_feat.device)
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        fused_ln = is_fusable_layernorm(self.norm, C)   # norm -> qkv in one kernel
        if isinstance(reduced_feat, CoordEmbedding) and not (fused_ln and self.mlp.mlp.takes_projection(N)):
            reduced_feat = reduced_feat.materialize()   # an unstored embedding needs both of the block's kernels that form it
        x = reduced_feat if fused_ln else apply_norm(self.norm, reduced_feat)
        pre = self.norm if fused_ln else None
        out = None
        if not torch.is_grad_enabled() and reduced_feat.dtype == torch.bfloat16:
            # inference: out-projection + residual + MLP + residual in one kernel where it applies
            x_in = x if isinstance(x, CoordEmbedding) else x.view(1, N, C)
            attn = self.bwa(x_in, scope_bucks, pre_norm=pre, skip_proj=True).view(N, C)
            out = self.mlp.mlp.after_projection(attn, self.bwa.proj, reduced_feat)
            if out is None:
                mid = self.bwa.proj(attn, residual=materialize(reduced_feat))
                out = self.mlp(mid, residual=mid)
        else:
            mid = self.bwa(x.view(1, N, C), scope_bucks, residual=reduced_feat.view(1, N, C), pre_norm=pre).view(N, C)
            out = self.mlp(mid, residual=mid)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return out


class Stage(nn.Module):
    """encoder blocks -> middle submodule -> decoder blocks, all on the (coord, feat, sep) triplet"""
    NVTX_SCOPE = "Stage"

    def __init__(self, encoder_specs: List[XFMRSpecs], buck_size: int, submodule: nn.Module,
                 decoder_specs: List[XFMRSpecs]):
        super().__init__()
        if submodule is None:
            raise ValueError("A submodule must be provided for a Stage.")

        def blocks(specs):
            return nn.ModuleList([XFMR(s.channels, s.hid_channels, s.num_heads, buck_size, s.qkv_bias, s.swin_plan,
                                       s.norm_layer) for s in specs])
        self.encoder_blocks = blocks(encoder_specs)
        self.middle = submodule
        self.decoder_blocks = blocks(decoder_specs)

    def forward(self, reduced_coord, reduced_feat, reduced_sep) -> torch.Tensor:
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        x = reduced_feat
        for block in self.encoder_blocks:
            x = block(reduced_coord, x, reduced_sep)
        x = self.middle(reduced_coord, materialize(x), reduced_sep)
        for block in self.decoder_blocks:
            x = block(reduced_coord, x, reduced_sep)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return x
