"""PSH scatter layer and coordinate embedding (reference: flash3dxfmr/layers/psh_ops.py)."""
from typing import Tuple

import torch
from torch import nn

from ..lib import pshattn
from ..psh import arithmatic as f3darith
from ..psh import psh_main as pm
from .nn_ops import Linear, torch_backward


class PSHScatterLayer(nn.Module):
    def __init__(self, bucket_size: int = 512) -> None:
        super().__init__()
        self.bucket_size = bucket_size

    def forward(self, coords, seps, hash_op: int) -> Tuple[torch.Tensor, pm.BucketScatterBuffers]:
        pad_to = f3darith.cdiv(coords.shape[0], self.bucket_size) * self.bucket_size
        return pm.batch_bucket_scatter(coords, seps, self.bucket_size, pad_to, hash_op)


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

    def forward(self, coords, seps, hash_op):
        pad_to = f3darith.cdiv(coords.shape[0], self.alignment) * self.alignment
        scattered, _ = pm.batch_bucket_scatter(coords, seps, self.bucket_size, pad_to, hash_op)
        self.last_scattered_coord = scattered
        emb = torch.empty(pad_to, self.lin.out_features, dtype=torch.bfloat16, device=coords.device)
        lin = self.lin
        pshattn.coord_embed_bf16(scattered, lin._w.get(lin.weight), lin._b.get(lin.bias), emb)
        # the coordinates carry no gradient; the embedding's weights do (bf16 view of the fp16 coordinates, as the kernel reads them)
        coord_f = scattered
        ref = lambda w, b: torch.nn.functional.linear(coord_f.to(torch.bfloat16).float(), w, b)
        return torch_backward(emb, ref, lin.weight, lin.bias)
