"""Bucketed (scoped) multi-head self-attention (reference: flash3dxfmr/layers/buck_swin.py)."""
from typing import Tuple

import torch
import torch.cuda.nvtx as nvtx
from torch import nn
from torch.autograd import Function

from ..lib import pshattn
from ..psh import dev_context as f3ddev
from ..psh import swin_attn as sa
from .nn_ops import CoordEmbedding, LayerNorm, Linear, _DerivedCache, norm_params_bf16


class BuckSwinFwdFunction(Function):
    """O = attention(Q, K, V) inside every scope of buckets; keeps (Q, K, V, O, LSE) for the backward
    pass (buck_swin.py:20-95 of the reference)."""

    @staticmethod
    def forward(ctx, Q, K, V, scope_buckets, buck_size: int) -> torch.Tensor:
        buff = sa.BuckSwinFwdBuffers.create_buckswin_fwd_buff(Q)
        pshattn.buck_swin_fwd(Q, K, V, buff.O, buff.LSE, scope_buckets, buck_size)
        ctx.save_for_backward(Q, K, V, buff.O, buff.LSE)
        ctx.scope_buckets, ctx.buck_size = scope_buckets, buck_size
        return buff.O

    @staticmethod
    def backward(ctx, grad_output) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, None, None]:
        Q, K, V, O, lse = ctx.saved_tensors
        dO = grad_output if grad_output.dtype == torch.bfloat16 else grad_output.to(torch.bfloat16)
        bwd = sa.BuckSwinBwdBuffers.create_buckswin_buffers(O, ctx.scope_buckets, ctx.buck_size)
        pshattn.buck_swin_bwd(Q, K, V, O, dO.contiguous(), lse, bwd.Delta, bwd.dQ, bwd.dK, bwd.dV, ctx.scope_buckets,
                              ctx.buck_size)
        return bwd.dQ, bwd.dK, bwd.dV, None, None


def _covers(scope_buckets, buck_size: int, L: int) -> bool:
    """the planner vouches that its table covers all rows, and the table was made for a tensor of this length"""
    return bool(getattr(scope_buckets, "covers_all_rows", False)) and scope_buckets.numel() * buck_size == L


class BuckSwinQKVFunction(Function):
    """The same attention over the three thirds of one projection output qkv [B, L, 3 H D] (the kernel reads Q, K, V
    as column slices).  The backward writes dQ, dK, dV straight into the thirds of one [B, L, 3 H D] gradient, so
    autograd neither splits the projection output nor concatenates three gradients."""

    @staticmethod
    def forward(ctx, qkv, scope_buckets, buck_size: int, num_heads: int) -> torch.Tensor:
        B, L, C3 = qkv.shape
        D = C3 // 3 // num_heads
        Q, K, V = (t.view(B, L, num_heads, D) for t in torch.chunk(qkv, 3, dim=-1))
        buff = sa.BuckSwinFwdBuffers.create_buckswin_fwd_buff(Q, _covers(scope_buckets, buck_size, L))
        pshattn.buck_swin_fwd(Q, K, V, buff.O, buff.LSE, scope_buckets, buck_size)
        ctx.save_for_backward(qkv, buff.O, buff.LSE)
        ctx.scope_buckets, ctx.buck_size, ctx.num_heads = scope_buckets, buck_size, num_heads
        return buff.O

    @staticmethod
    def backward(ctx, grad_output):
        qkv, O, lse = ctx.saved_tensors
        B, L, H, D = O.shape
        Q, K, V = (t.view(B, L, H, D) for t in torch.chunk(qkv, 3, dim=-1))
        dO = grad_output if grad_output.dtype == torch.bfloat16 else grad_output.to(torch.bfloat16)
        # rows that no scope covers are not written: zero-filled unless the planner vouches that its table covers all
        # ... for THIS tensor: a table made for another length leaves rows out
        dqkv = torch.empty_like(qkv) if _covers(ctx.scope_buckets, ctx.buck_size, L) else torch.zeros_like(qkv)
        dQ, dK, dV = (t.view(B, L, H, D) for t in torch.chunk(dqkv, 3, dim=-1))
        delta = torch.zeros(B, L, H, dtype=torch.float32, device=O.device)
        pshattn.buck_swin_bwd(Q, K, V, O, dO.contiguous(), lse, delta, dQ, dK, dV, ctx.scope_buckets, ctx.buck_size)
        return dqkv, None, None, None


class BucketSwinAttention(nn.Module):
    def __init__(self, buck_size: int) -> None:
        super().__init__()
        self.buck_size = buck_size

    def forward(self, Q, K, V, scope_buckets) -> torch.Tensor:
        assert Q.dim() == 4, f"Expect Q with four axes [B, L, H, D], but got shape={Q.shape}"
        return BuckSwinFwdFunction.apply(Q, K, V, scope_buckets, self.buck_size)


class BucketSwinAttentionModule(nn.Module):
    NVTX_SCOPE = "BucketSwinAttention"

    def __init__(self, channels: int, num_heads: int, buck_size: int, qkv_bias: bool = True):
        super().__init__()
        assert channels % num_heads == 0, f"Channels={channels} NOT divisible by num_heads={num_heads}"
        self.num_heads = num_heads
        self.head_dim = channels // num_heads
        self.qkv = Linear(channels, channels * 3, bias=qkv_bias)
        self.attn = BucketSwinAttention(buck_size)
        self.proj = Linear(channels, channels)
        self.qkv._fold = _DerivedCache()      # (table, chol): LayerNorm + QKV of a coordinate embedding, folded

    def _attention_of_embedding(self, emb: CoordEmbedding, pre_norm, scope_buckets):
        """The attention output [1, L, H, D] of an unstored coordinate embedding with Q, K and V formed inside the
        attention kernel: LayerNorm and the QKV projection of the rank-4 embedding fold into four numbers per output
        feature (prepared once per set of weights).  None where no kernel covers the shape (32-wide heads, scopes of
        256 or 512 tokens, LayerNorm in front): the caller then runs the projection kernel on the embedding."""
        tokens = scope_buckets.shape[1] * self.attn.buck_size
        if (torch.is_grad_enabled() or not isinstance(pre_norm, LayerNorm) or self.head_dim != 32 or tokens not in (256, 512)
                or scope_buckets.shape[1] > 4):
            return None
        lin, qkv = emb.lin, self.qkv

        def build():
            training = self.training or pre_norm.training or lin.training
            g, be = norm_params_bf16(pre_norm)
            return pshattn.embed_qkv_fold(lin._w.get(lin.weight, training), lin._b.get(lin.bias, training), g, be, pre_norm.eps,
                                          qkv._w.get(qkv.weight, training), qkv._b.get(qkv.bias, training), self.num_heads)

        fold = qkv._fold.get_or_build((lin.weight, lin.bias, pre_norm.weight, pre_norm.bias, qkv.weight, qkv.bias),
                                      (float(pre_norm.eps), self.num_heads), build)
        if fold is None:
            return None
        table, chol = fold
        L = emb.shape[0]
        O = torch.empty(1, L, self.num_heads, self.head_dim, dtype=torch.bfloat16, device=emb.device)
        lse = (torch.empty if _covers(scope_buckets, self.attn.buck_size, L) else torch.zeros)(
            1, L, self.num_heads, dtype=torch.float32, device=emb.device)
        if not pshattn.embed_buck_swin_fwd(emb.coord, table, chol, O, lse, scope_buckets, self.attn.buck_size):
            return None
        return O

    def forward(self, x: torch.Tensor, scope_buckets: torch.Tensor, residual: torch.Tensor = None,
                pre_norm=None, skip_proj: bool = False) -> torch.Tensor:
        """x [B, L, C] -> [B, L, C].  Q, K and V are read by the attention kernel straight out of the
        [B, L, 3C] projection output (the reference makes three contiguous copies, :187-190); the
        residual, when given, is added in the out-projection's epilogue.  skip_proj: return the attention output
        itself (the caller applies `self.proj`, e.g. inside the kernel of the MLP that follows)."""
        if isinstance(x, CoordEmbedding):      # [L, C], not stored: one batch element
            B, (L, C) = 1, x.shape
        else:
            assert x.dim() == 3, f"Expect input features with three axes [B, L, C], but got shape={x.shape}"
            B, L, C = x.shape
        assert C == self.num_heads * self.head_dim, f"Expect input channels are {self.num_heads * self.head_dim}, but got {C}"
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        attn_out = self._attention_of_embedding(x, pre_norm, scope_buckets) if isinstance(x, CoordEmbedding) else None
        if attn_out is None:
            # pre_norm: LayerNorm applied inside the projection kernel; a CoordEmbedding is formed there too
            qkv = self.qkv.embedded(x, pre_norm).view(B, L, -1) if isinstance(x, CoordEmbedding) else self.qkv(x, pre_norm=pre_norm)
            if qkv.dtype == torch.bfloat16 and qkv.is_contiguous():
                attn_out = BuckSwinQKVFunction.apply(qkv, scope_buckets, self.attn.buck_size, self.num_heads)
            else:
                q, k, v = (t.view(B, L, self.num_heads, self.head_dim) for t in torch.chunk(qkv, 3, dim=-1))
                attn_out = self.attn(q, k, v, scope_buckets)
        out = attn_out.view(B, L, C) if skip_proj else self.proj(attn_out.view(B, L, C), residual=residual)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return out
