"""Output buffers of the bucketed attention op (reference: flash3dxfmr/psh/swin_attn.py:13-24)."""
from dataclasses import dataclass

import torch


@dataclass(slots=True)
class BuckSwinFwdBuffers:
    O: torch.Tensor
    LSE: torch.Tensor

    @staticmethod
    def create_buckswin_fwd_buff(Q: torch.Tensor):
        B, L, H, D = Q.shape
        # rows outside every scope keep these values (LSE 0, O uninitialised), as in the reference;
        # every plan of bucket_scope.py covers all rows, so the model path never reads such a row
        return BuckSwinFwdBuffers(torch.empty(B, L, H, D, dtype=Q.dtype, device=Q.device),
                                  torch.zeros(B, L, H, dtype=torch.float32, device=Q.device))
