"""MLP block (reference: flash3dxfmr/layers/elem_wise.py:19-33)."""
import torch.cuda.nvtx as nvtx
from torch import nn

from ..psh import dev_context as f3ddev
from .nn_ops import LayerNormMLP


class MLP(nn.Module):
    NVTX_SCOPE = "MLP"

    def __init__(self, in_dim, hidden_dim, activation: str = "swiglu"):
        super().__init__()
        self.mlp = LayerNormMLP(hidden_size=in_dim, ffn_hidden_size=in_dim if hidden_dim is None else hidden_dim,
                                activation=activation)

    def forward(self, x, residual=None):
        """LayerNorm -> fc1 -> act -> fc2 (+ residual fused into the fc2 epilogue when given)"""
        if f3ddev.get_nvtx():
            nvtx.range_push(self.NVTX_SCOPE)
        res = self.mlp(x, residual)
        if f3ddev.get_nvtx():
            nvtx.range_pop()
        return res
