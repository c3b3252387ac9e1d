"""Batch bookkeeping: clouds are concatenated along the point axis and described by `seps`, the
inclusive cumulative point counts (reference: flash3dxfmr/psh/batching.py:13-40)."""
from typing import List, Sequence

import weakref

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
    """largest cloud of the batch, from the host-side sizes (one device->host copy per separator tensor, then none)"""
    return max(host_sizes(seps))


def with_last_separator(seps: torch.Tensor, total: int) -> torch.Tensor:
    """A copy of `seps` whose last entry is `total` (rows appended for alignment are counted into the last cloud).
    The copy is made once per separator tensor and length, and the host-side sizes of the copy are derived from those
    of `seps`, so handing it on costs no host synchronisation."""
    facts = host_facts(seps)
    key = ("with_last", int(total))
    if key not in facts:
        out = seps.clone()
        out.view(torch.int32)[-1] = int(total)
        if "sizes" in facts:
            sizes = list(facts["sizes"])
            sizes[-1] += int(total) - sum(sizes)
            host_facts(out)["sizes"] = sizes
        facts[key] = out
    return facts[key]


def bulk_to(ts: List[torch.Tensor], dest):
    return [t.to(dest) for t in ts]


def cdiv_int(a: torch.Tensor, b):
    return (a + (b - 1)) / b


_HOST_FACTS = {}   # id(separator tensor) -> (weak reference, tensor version, facts known on the host)


def host_facts(seps: torch.Tensor) -> dict:
    """Per-tensor memo for values derived from a separator tensor that live on the host.  Keyed by the
    tensor OBJECT (a weak reference proves it is still the same one: a new tensor that happens to reuse
    the address is a different object) and its version counter (in-place torch ops bump it)."""
    key = id(seps)
    hit = _HOST_FACTS.get(key)
    if hit is not None and hit[0]() is seps and hit[1] == seps._version:
        return hit[2]
    facts = {}
    _HOST_FACTS[key] = (weakref.ref(seps, lambda _r, k=key, d=_HOST_FACTS: d.pop(k, None)), seps._version, facts)
    return facts


def host_sizes(seps: torch.Tensor):
    """Cloud sizes as a Python list with a single device->host copy (the reference pays one
    `.item()` sync per statistic, psh_main.py:47,102).  The copy is a host-device synchronisation, so
    the answer is remembered per separator tensor: the same tensor object, unchanged since, costs nothing
    the next time, and the host can queue a whole step ahead of the GPU."""
    facts = host_facts(seps)
    if "sizes" not in facts:
        wide = seps.to(torch.int64).cpu()
        facts["sizes"] = torch.diff(wide, prepend=wide.new_zeros(1)).tolist()
    return facts["sizes"]
