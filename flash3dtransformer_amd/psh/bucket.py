"""Probe-offset table of the overflow rebalancer (reference: flash3dxfmr/psh/bucket.py:19-40):
the 124 non-zero offsets of {-2..2}^3 plus four +-3 corners, as int16 [128, 3]."""
import random

import torch

_CORNERS = ((3, 3, 3), (3, -3, 3), (-3, 3, -3), (-3, -3, -3))


def probe_offset_list(shuffle_seed=None):
    r = range(-2, 3)
    offs = [(i, j, k) for i in r for j in r for k in r if (i, j, k) != (0, 0, 0)] + list(_CORNERS)
    if shuffle_seed is None:
        random.shuffle(offs)          # reference behaviour: unseeded shuffle per call
    else:
        random.Random(shuffle_seed).shuffle(offs)
    return offs


_PROBE_CACHE = {}   # (device, row_major, shuffle_seed) -> table on the device (read-only for every consumer)


def generate_probe_offsets(device, row_major=True, shuffle_seed=None):
    key = (str(device), bool(row_major), shuffle_seed)
    hit = _PROBE_CACHE.get(key)
    if hit is not None:
        return hit
    t = torch.tensor(probe_offset_list(shuffle_seed), dtype=torch.int16)
    if not row_major:
        t = t.t()
    t = t.contiguous().to(device)
    _PROBE_CACHE[key] = t
    return t
