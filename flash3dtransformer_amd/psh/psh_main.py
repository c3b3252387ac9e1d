"""PSH bucket scatter: buffer contract and the Python entry of the op
(reference: flash3dxfmr/psh/psh_main.py:21-125)."""
import math
from dataclasses import dataclass
from typing import Tuple, Optional

import torch

from . import arithmatic as f3darith
from . import batching as f3dbatch
from . import bucket as f3dbuck
from . import dev_context as f3ddev
from ..lib import pshattn

NUM_VOX = 0xFFFF


def bucket_geometry(seps: torch.Tensor, bucket_size: int, num_vox: int = NUM_VOX):
    """(num_buck, divisor, longest cloud) from the cloud sizes, psh_main.py:47-49,100-104: the number
    of hash buckets is the mean cloud size (fp32 mean) over the bucket size, floored, rounded up to
    a power of two; the divisor maps the 16-bit hash range onto them."""
    sizes = f3dbatch.host_sizes(seps)
    mean_n = float(torch.tensor(sizes, dtype=torch.float32).mean())
    num_buck = f3darith.round_next_two_power(int(mean_n / bucket_size))
    if num_buck == 0:
        raise RuntimeError(f"mean cloud size {mean_n:.0f} is smaller than bucket_size={bucket_size}: no hash bucket")
    return num_buck, int(math.ceil(num_vox / num_buck)), int(max(sizes))


@dataclass(slots=True)
class BucketScatterBuffers:
    bucket_id: torch.Tensor
    bucket_cntr: torch.Tensor
    bucket_offs: torch.Tensor
    bucket_cumsum: torch.Tensor
    probe_offs: torch.Tensor
    scattered_coord: torch.Tensor
    scatter_index: Optional[torch.Tensor] = None   # filled by batch_scatter_index

    @staticmethod
    def create_buffers(coords: torch.Tensor, seps: torch.Tensor, bucket_size: int, pad_to: int, num_buck: int = None,
                       debug_prefill: bool = True):
        """Allocation contract of the op (psh_main.py:31-67).  Prefills the kernels rely on:
        bucket_cntr = 0 (slots are counted up from it).  bucket_id = 1 and scattered_coord = NaN are the
        reference's debugging prefills (its tests look for surviving NaNs); `debug_prefill=False` skips
        them, which is safe here because the scatter kernel writes every row of both."""
        total_n, d = coords.shape
        dev = coords.device
        if num_buck is None:
            num_buck, _, _ = bucket_geometry(seps, bucket_size)
        b = seps.shape[0]
        zeros = torch.zeros(2, b, num_buck, dtype=torch.uint32, device=dev)   # one fill for both counters
        if debug_prefill:
            bucket_id = torch.ones(total_n, dtype=torch.uint16, device=dev)
            scattered = torch.full((pad_to, d), float("nan"), dtype=torch.float16, device=dev)
        else:
            bucket_id = torch.empty(total_n, dtype=torch.uint16, device=dev)
            scattered = torch.empty(pad_to, d, dtype=torch.float16, device=dev)
        return BucketScatterBuffers(
            bucket_id=bucket_id,
            bucket_cntr=zeros[0],
            bucket_offs=torch.empty(total_n, dtype=torch.uint32, device=dev),
            bucket_cumsum=zeros[1],
            probe_offs=f3dbuck.generate_probe_offsets(dev, row_major=True),
            scattered_coord=scattered,
        )


def batch_bucket_scatter(coords: torch.Tensor, seps: torch.Tensor, bucket_size: int, pad_to: int, hash_op: int,
                         debug_prefill: bool = False) -> Tuple[torch.Tensor, BucketScatterBuffers]:
    """coords [N,3] fp16 (clouds concatenated, `seps` inclusive cumulative sizes, uint32) ->
    scattered_coord [pad_to,3]: every cloud's points grouped by hash bucket (hash_op: 1 ZORDER_DIV,
    2 XORSUM_DIV, 3 ZORDER_MOD, 4 XORSUM_MOD), rows [N, pad_to) = 0.

    Same call sequence as psh_main.py:70-125, with one host sync instead of three and the whole-batch
    bounding box from one fused kernel instead of two torch reductions."""
    f3ddev.init_dev(coords.get_device())
    num_buck, divisor, max_n = bucket_geometry(seps, bucket_size)
    buffers = BucketScatterBuffers.create_buffers(coords, seps, bucket_size, pad_to, num_buck, debug_prefill)
    bbox = torch.empty(2, 3, dtype=torch.float16, device=coords.device)
    pshattn.coord_bbox(coords, bbox[0], bbox[1])
    pshattn.batch_psh_scatter_pad_hash(
        coords, buffers.bucket_id, buffers.bucket_cntr, buffers.bucket_offs, seps, max_n, num_buck, divisor,
        bucket_size, NUM_VOX, bbox[0], bbox[1], buffers.probe_offs, buffers.bucket_cumsum,
        buffers.scattered_coord, 0.0, hash_op)
    return buffers.scattered_coord, buffers


def batch_scatter_index(buffers: BucketScatterBuffers, seps: torch.Tensor,
                        feat: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Out-to-in permutation index of a finished batch_bucket_scatter, uint32 [pad_to]: row r of the scattered
    layout holds input row index[r]; the pad rows hold N + 3 (batch_psh_bucket.cuh:678, :735).  With `feat`
    [N, ...] also returns the features in scattered order with zero pad rows, moved in the same pass (the step
    batch_psh_cumsum_scatter_feat_index_postpad_ker, batch_psh_bucket.cuh:617-753, announces and never reaches).
    The index is kept in `buffers.scatter_index`."""
    pad_to = buffers.scattered_coord.shape[0]
    dev = buffers.scattered_coord.device
    index = torch.empty(pad_to, dtype=torch.uint32, device=dev)
    out = None
    if feat is not None:
        feat = feat.contiguous()
        out = torch.empty((pad_to,) + tuple(feat.shape[1:]), dtype=feat.dtype, device=dev)
    pshattn.psh_scatter_feat_index(buffers.bucket_id, buffers.bucket_cntr, buffers.bucket_offs, seps,
                                   buffers.bucket_cumsum, index, feat, out)
    buffers.scatter_index = index
    return index, out
