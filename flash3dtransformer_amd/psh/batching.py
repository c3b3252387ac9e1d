"""Batch bookkeeping: clouds are concatenated along the point axis and described by `seps`, the
inclusive cumulative point counts (reference: flash3dxfmr/psh/batching.py:13-40)."""
from typing import List, Sequence

import torch


def collate_coords_flat_sep(coords: Sequence[torch.Tensor], coord_dtype=None, sep_dtype=None):
    """[N_i, >=3] tensors -> (xyz [sum N_i, 3] contiguous, seps [B])"""
    sizes = torch.tensor([int(c.shape[0]) for c in coords], dtype=torch.int32)
    flat = torch.cat(list(coords), dim=0)
    if coord_dtype is not None:
        flat = flat.to(coord_dtype)
    seps = torch.cumsum(sizes, dim=0)
    if sep_dtype is not None:
        seps = seps.to(sep_dtype)
    return flat[:, :3].contiguous(), seps


def sep2sizes(seps: torch.Tensor) -> torch.Tensor:
    wide = seps.to(torch.int64)
    return torch.diff(wide, prepend=wide.new_zeros(1)).to(seps.dtype)


def max_inslen_from_seps(seps: torch.Tensor) -> int:
    return int(sep2sizes(seps.to(torch.int64)).max())


def bulk_to(ts: List[torch.Tensor], dest):
    return [t.to(dest) for t in ts]


def cdiv_int(a: torch.Tensor, b):
    return (a + (b - 1)) / b


_HOST_SIZES = {}   # (data_ptr, shape, version) of the last separator tensors seen -> their sizes on the host


def host_sizes(seps: torch.Tensor):
    """Cloud sizes as a Python list with a single device->host copy (the reference pays one
    `.item()` sync per statistic, psh_main.py:47,102).  The copy is a host-device synchronisation, so
    the answer is remembered per separator tensor: the same tensor (same storage, unchanged since)
    costs nothing the next time, and the host can queue a whole step ahead of the GPU."""
    key = (seps.data_ptr(), tuple(seps.shape), seps._version, str(seps.device))
    hit = _HOST_SIZES.get(key)
    if hit is not None:
        return hit
    wide = seps.to(torch.int64).cpu()
    sizes = torch.diff(wide, prepend=wide.new_zeros(1)).tolist()
    if len(_HOST_SIZES) > 64:
        _HOST_SIZES.clear()
    _HOST_SIZES[key] = sizes
    return sizes
