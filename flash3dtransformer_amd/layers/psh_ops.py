"""PSH scatter layer and coordinate embedding (reference: flash3dxfmr/layers/psh_ops.py)."""
from typing import Tuple

import torch
from torch import nn

from ..lib import pshattn
from ..psh import arithmatic as f3darith
from ..psh import psh_main as pm
from .nn_ops import CoordEmbedding, Linear, torch_backward


class _PermuteRows(torch.autograd.Function):
    """Row permutation by a PSH out-to-in index; the gradient of one direction is the other direction."""

    @staticmethod
    def forward(ctx, x, index, n_out: int, gather: bool):
        out = torch.empty((n_out,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
        if not gather:
            out.zero_()      # rows that the index does not name
        pshattn.permute_rows(index, x.contiguous(), out, gather)
        ctx.index, ctx.n_in, ctx.gather = index, x.shape[0], gather
        return out

    @staticmethod
    def backward(ctx, grad):
        g = torch.empty((ctx.n_in,) + tuple(grad.shape[1:]), dtype=grad.dtype, device=grad.device)
        if ctx.gather:
            g.zero_()
        pshattn.permute_rows(ctx.index, grad.contiguous(), g, not ctx.gather)
        return g, None, None, None


def to_psh_order(x: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """x [N, ...] in input order -> [pad_to, ...] in PSH (scattered) order, pad rows zero; index: the out-to-in
    index of psh_main.batch_scatter_index"""
    return _PermuteRows.apply(x, index, index.shape[0], True)


def to_input_order(y: torch.Tensor, index: torch.Tensor, n: int) -> torch.Tensor:
    """y [pad_to, ...] in PSH order -> [n, ...] in the order the points came in (pad rows dropped)"""
    return _PermuteRows.apply(y, index, n, False)


class PSHScatterLayer(nn.Module):
    def __init__(self, bucket_size: int = 512) -> None:
        super().__init__()
        self.bucket_size = bucket_size

    def forward(self, coords, seps, hash_op: int) -> Tuple[torch.Tensor, pm.BucketScatterBuffers]:
        pad_to = f3darith.cdiv(coords.shape[0], self.bucket_size) * self.bucket_size
        return pm.batch_bucket_scatter(coords, seps, self.bucket_size, pad_to, hash_op)


class _CoordEmbedGrad(torch.autograd.Function):
    """emb = bf16(coord) @ w.T + b computed by the HIP forward; the coordinates carry no gradient, the weights take
    theirs from the weight-gradient kernel over the coordinates padded to 8 columns (its inner sizes are multiples of 8)"""

    @staticmethod
    def forward(ctx, emb, weight, bias, coord):
        ctx.save_for_backward(weight, bias, coord)
        return emb.view_as(emb)

    @staticmethod
    def backward(ctx, dy):
        weight, bias, coord = ctx.saved_tensors
        dy2 = dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)
        if dy2.stride(-1) != 1:
            dy2 = dy2.contiguous()
        c8 = torch.zeros(coord.shape[0], 8, dtype=torch.bfloat16, device=coord.device)
        c8[:, :3] = coord
        dw8 = torch.empty(weight.shape[0], 8, dtype=torch.float32, device=coord.device)
        db = torch.empty(weight.shape[0], dtype=torch.float32, device=coord.device) if bias is not None else None
        pshattn.linear_wgrad_bf16(dy2, c8, dw8, db)
        return (None, dw8[:, :3].to(weight.dtype) if ctx.needs_input_grad[1] else None,
                db.to(bias.dtype) if bias is not None and ctx.needs_input_grad[2] else None, None)


class PSH3DCoordEmbedding(nn.Module):
    """PSH-scatter the coordinates (padded to `alignment` rows) and embed them with a 3 -> emb_dim
    linear layer.  Returns the embedding; the scattered coordinates of the last call are kept in
    `last_scattered_coord` for the caller that needs them (the model routes them down the tree)."""

    def __init__(self, emb_dim: int, bucket_size, alignment, feat_dtype=torch.bfloat16):
        super().__init__()
        self.bucket_size = bucket_size
        self.alignment = alignment
        self.feat_dtype = feat_dtype
        self.lin = Linear(3, emb_dim)
        self.last_scattered_coord = None
        self.last_buffers = None

    def forward(self, coords, seps, hash_op, lazy: bool = False):
        """lazy (inference only): return a CoordEmbedding, which the first block turns into its input inside its own
        kernels, instead of storing the [rows, emb_dim] tensor"""
        pad_to = f3darith.cdiv(coords.shape[0], self.alignment) * self.alignment
        scattered, buffers = pm.batch_bucket_scatter(coords, seps, self.bucket_size, pad_to, hash_op)
        self.last_scattered_coord = scattered
        self.last_buffers = buffers
        if lazy and not torch.is_grad_enabled() and self.lin.out_features in CoordEmbedding.EMBED_WIDTHS:
            return CoordEmbedding(scattered, self.lin)
        emb = torch.empty(pad_to, self.lin.out_features, dtype=torch.bfloat16, device=coords.device)
        lin = self.lin
        pshattn.coord_embed_bf16(scattered, lin._w.get(lin.weight, lin.training), lin._b.get(lin.bias, lin.training), emb)
        # the coordinates carry no gradient; the embedding's weights do (bf16 view of the fp16 coordinates, as the kernel reads them)
        if not (torch.is_grad_enabled() and (lin.weight.requires_grad or (lin.bias is not None and lin.bias.requires_grad))):
            return emb
        if lin.out_features % 8 == 0:
            return _CoordEmbedGrad.apply(emb, lin.weight, lin.bias, scattered)
        coord_f = scattered
        ref = lambda w, b: torch.nn.functional.linear(coord_f.to(torch.bfloat16).float(), w, b)
        return torch_backward(emb, ref, lin.weight, lin.bias)
