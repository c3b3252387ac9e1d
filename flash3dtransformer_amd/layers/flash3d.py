"""Top-level Flash3D model (reference: flash3dxfmr/layers/flash3d.py)."""
from dataclasses import dataclass
from typing import List, Union

import torch
import torch.cuda.nvtx as nvtx
from torch import nn

from ..psh import batching as f3dbatch
from ..psh import dev_context as f3ddev
from ..psh import psh_main as pm
from . import hourglass as f3dhourglass
from . import psh_ops
from . import stage as f3dstage
from .nn_ops import Linear


class LeafModule(nn.Module):
    """Deepest level's middle: a linear map from the last encoder width to the first decoder width"""

    def __init__(self, in_dim, out_dim):
        super().__init__()
        self.proj = Linear(in_dim, out_dim)

    def forward(self, reduced_coord, reduced_feat, reduced_sep) -> torch.Tensor:
        return self.proj(reduced_feat)


@dataclass(slots=True)
class F3DLevelSpecs:
    encoder_specs: List[f3dstage.XFMRSpecs]
    decoder_specs: List[f3dstage.XFMRSpecs]
    reduction_op: Union[int, str]
    pool_align: int
    pool_norm: callable
    pool_act: callable
    unpool_norm: callable
    unpool_act: callable


class Flash3D(nn.Module):
    """Recursive hourglass of Stages: level i = Stage(encoders_i, Hourglass(pool, level i+1, unpool),
    decoders_i); the last level's middle is a LeafModule.

    forward(coords [N,3] fp16, input_feat, seps [B] uint32) -> [pad_to, C_out] bf16, rows in PSH
    (scattered) order, pad_to = N rounded up to buck_size * scope_size * 6.

    By default, as in the reference, `input_feat` is accepted and not used: the first-level features are
    the embedded scattered coordinates.  With `in_feat_dim` set, `input_feat` [N, in_feat_dim] is moved to
    PSH order by the scatter's permutation index, projected by `input_proj` (a parameter the reference does
    not have) and added to the coordinate embedding.  Unlike the reference, which hands the UNSCATTERED
    coordinates to the tree next to scattered features (flash3d.py:162-163), the tree receives the
    scattered coordinates, with the pad rows counted into the last cloud, so that pooling groups the rows
    it actually pools.  `to_input_order(out)` brings per-point rows of the last forward back to the order
    the points came in."""
    NVTX_SCOPE = "Flash3D"

    def __init__(self, level_specs: List[F3DLevelSpecs], buck_size: int, scope_size: int, top_level_hash,
                 subbuck_size: int = 2, in_feat_dim: int = None):
        super().__init__()
        f3ddev.set_sync_stream(False)
        emb_chann = level_specs[0].encoder_specs[0].channels
        self.first_hashtype = top_level_hash
        self.psh_scatter = psh_ops.PSH3DCoordEmbedding(emb_chann, buck_size, buck_size * scope_size * 6)
        self.level_specs = level_specs
        self.buck_size = buck_size
        self.scope_size = scope_size
        self.subbuck_size = subbuck_size
        self.module_tree = self.build_module(0)
        self.in_feat_dim = in_feat_dim
        self._in_feat_pad = 0
        if in_feat_dim is not None:
            # the matrix-core linear takes inner widths in multiples of 8: narrower point features are zero-padded
            self._in_feat_pad = -in_feat_dim % 8
            self.input_proj = Linear(in_feat_dim + self._in_feat_pad, emb_chann)
        self._last_index = None
        self._last_n = 0
        self._last_seps = None

    def build_module(self, level: int) -> nn.Module:
        if level >= len(self.level_specs):
            raise ValueError("Level exceeds level_specs length.")
        spec = self.level_specs[level]
        last_enc, first_dec = spec.encoder_specs[-1], spec.decoder_specs[0]
        if level + 1 >= len(self.level_specs):
            middle = LeafModule(last_enc.channels, first_dec.channels)
        else:
            nxt = self.level_specs[level + 1]
            middle = f3dhourglass.HourglassModule(
                pooling_in_channels=last_enc.channels,
                pooling_out_channels=nxt.encoder_specs[0].channels,
                pooling_reduction_op=spec.reduction_op,
                pooling_length_alignment=spec.pool_align,
                unpooling_in_channels=nxt.decoder_specs[-1].channels,
                unpooling_out_channels=first_dec.channels,
                pooling_norm_layer=spec.pool_norm,
                pooling_act_layer=spec.pool_act,
                unpooling_norm_layer=spec.unpool_norm,
                unpooling_act_layer=spec.unpool_act,
                submodule=self.build_module(level + 1),
                subbuck_size=self.subbuck_size,
            )
        return f3dstage.Stage(encoder_specs=spec.encoder_specs, buck_size=self.buck_size, submodule=middle,
                              decoder_specs=spec.decoder_specs)

    def forward(self, coords: torch.Tensor, input_feat: torch.Tensor, seps: torch.Tensor) -> torch.Tensor:
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        # at inference without input features the embedding is not stored: the first block forms it inside its kernels
        psh_feat = self.psh_scatter(coords, seps, self.first_hashtype, lazy=self.in_feat_dim is None)
        scattered = self.psh_scatter.last_scattered_coord
        self._last_index, self._last_n, self._last_seps = None, coords.shape[0], seps
        if self.in_feat_dim is not None:
            if input_feat is None or input_feat.shape != (coords.shape[0], self.in_feat_dim):
                raise RuntimeError(f"input_feat must be [{coords.shape[0]}, {self.in_feat_dim}]")
            feat = input_feat.to(torch.bfloat16)
            if self._in_feat_pad:
                feat = torch.nn.functional.pad(feat, (0, self._in_feat_pad))
            if feat.requires_grad:
                index, _ = pm.batch_scatter_index(self.psh_scatter.last_buffers, seps)
                feat = psh_ops.to_psh_order(feat, index)
            else:
                index, feat = pm.batch_scatter_index(self.psh_scatter.last_buffers, seps, feat)
            self._last_index = index
            psh_feat = psh_feat + self.input_proj(feat)
        tree_seps = seps
        if scattered.shape[0] != coords.shape[0]:
            tree_seps = f3dbatch.with_last_separator(seps, scattered.shape[0])
        out = self.module_tree(scattered, psh_feat, tree_seps)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return out

    def to_input_order(self, out: torch.Tensor) -> torch.Tensor:
        """Rows of a per-point tensor of the last forward ([pad_to, ...], PSH order) in the order the points
        came in ([N, ...]); differentiable."""
        if self._last_index is None:
            if self._last_seps is None:
                raise RuntimeError("to_input_order needs a forward call first")
            self._last_index, _ = pm.batch_scatter_index(self.psh_scatter.last_buffers, self._last_seps)
        return psh_ops.to_input_order(out, self._last_index, self._last_n)
