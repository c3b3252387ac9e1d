"""Output buffers of the bucketed attention ops (reference: flash3dxfmr/psh/swin_attn.py:13-43)."""
from dataclasses import dataclass

import torch


@dataclass(slots=True)
class BuckSwinFwdBuffers:
    O: torch.Tensor
    LSE: torch.Tensor

    @staticmethod
    def create_buckswin_fwd_buff(Q: torch.Tensor, all_rows_covered: bool = False):
        B, L, H, D = Q.shape
        # rows outside every scope keep these values (LSE 0, O uninitialised), as in the reference.
        # `all_rows_covered`: the caller vouches that the scope table covers every row of THIS tensor (every plan of
        # bucket_scope.py does); the kernel then writes every LSE value and the zero fill is left out
        lse = (torch.empty if all_rows_covered else torch.zeros)(B, L, H, dtype=torch.float32, device=Q.device)
        return BuckSwinFwdBuffers(torch.empty(B, L, H, D, dtype=Q.dtype, device=Q.device), lse)


@dataclass(slots=True)
class BuckSwinBwdBuffers:
    """gradient buffers of the backward op (reference: psh/swin_attn.py:26-43): zero-filled, because rows that no
    scope covers are not written; dense [B, L, H, D] whatever the layout of O"""
    O: torch.Tensor
    dQ: torch.Tensor
    dK: torch.Tensor
    dV: torch.Tensor
    Scope_buckets: torch.Tensor
    Delta: torch.Tensor
    buck_size: int

    @staticmethod
    def create_buckswin_buffers(O: torch.Tensor, Scope_buckets: torch.Tensor, buck_size: int):
        B, L, H, D = O.shape
        Delta = torch.zeros(B, L, H, dtype=torch.float32, device=O.device)
        mk = lambda: torch.zeros(B, L, H, D, dtype=O.dtype, device=O.device)
        return BuckSwinBwdBuffers(O, mk(), mk(), mk(), Scope_buckets, Delta, buck_size)
