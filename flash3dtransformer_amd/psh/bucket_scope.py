"""Attention scope planning (reference: flash3dxfmr/psh/bucket_scope.py).

An attention bucket is a fixed run of `buck_size` rows of the flattened, scattered point array; a
scope is the list of buckets that attend to each other.  Both reference plans ("swin", "stride")
reduce to consecutive groups of `scope_size_in_buck` buckets when the length is aligned and to ONE
global scope otherwise (bucket_scope.py:58-82) — the same mapping is produced here, as a closed
form, and cached per (length, plan, device) so that a forward pass uploads each scope table once.
"""
import math
import warnings
from dataclasses import dataclass
from typing import List

import torch


def minimal_alignment(buck_size: int, scope_size_in_buck: int) -> int:
    return buck_size


def swinable_alignment(buck_size: int, scope_size_in_buck: int) -> int:
    return buck_size * scope_size_in_buck


def stridable_alignment(buck_size: int, scope_size_in_buck: int) -> int:
    # 6 = lcm(1, 2, 3): lengths stay aligned for strides 1..3
    return buck_size * scope_size_in_buck * 6


def generate_single_scope(total_N: int, buck_size: int, scope_size: int) -> List[List[int]]:
    return [list(range(total_N // buck_size))]


def generate_swin_scopes(total_N: int, buck_size: int, scope_size: int, offset: int = 0) -> List[List[int]]:
    n = int(math.ceil(total_N / buck_size))
    assert scope_size <= n, "scope_size must be less than or equal to the number of buckets (N)"
    assert n % scope_size == 0, "For non-overlapping scopes, the number of buckets N must be divisible by scope_size"
    return [[(offset + s * scope_size + j) % n for j in range(scope_size)] for s in range(n // scope_size)]


def generate_stride_scopes(total_N: int, buck_size: int, scope_size: int, stride: int = 1) -> List[List[int]]:
    n = int(math.ceil(total_N / buck_size))
    assert n % stride == 0, f"num_bucket={n} must be divisible by stride={stride}"
    out = []
    for chunk in range(0, n, scope_size * stride):
        for s in range(stride):
            idx = [chunk + s + stride * k for k in range(scope_size)]
            if all(i < n for i in idx):
                out.append(idx)
    return out


_SCOPE_CACHE = {}


@dataclass
class SwinPlan:
    plan_name: str
    buck_size: int
    scope_size_in_buck: int
    offset_or_stride: int

    def scope_shape(self, total_N: int):
        """(num_scopes, scope_size) the plan yields for a buffer of total_N rows"""
        assert self.plan_name in ["swin", "stride"], f"Unsupported scoping plan name: {self.plan_name}"
        bs, sc = self.buck_size, self.scope_size_in_buck
        assert total_N % minimal_alignment(bs, sc) == 0, \
            f"Input buffer length must be divisible by minimal alignment = {bs}, but got {total_N}"
        align = stridable_alignment(bs, sc) if self.plan_name == "stride" else swinable_alignment(bs, sc)
        nbuck = total_N // bs
        if total_N % align == 0:
            return nbuck // sc, sc
        return 1, nbuck

    def gen_scopes_from_plan(self, total_N, device):
        ns, sz = self.scope_shape(total_N)
        key = (int(total_N), self.buck_size, ns, sz, str(device))
        hit = _SCOPE_CACHE.get(key)
        if hit is None:
            if ns == 1 and sz > self.scope_size_in_buck:
                warnings.warn(
                    f"buffer length {total_N} is not aligned for plan '{self.plan_name}' "
                    f"(bucket {self.buck_size} x scope {self.scope_size_in_buck}): falling back to ONE global "
                    f"attention scope of {sz} buckets (quadratic cost)")
            hit = torch.arange(ns * sz, dtype=torch.int32).view(ns, sz).to(device).view(torch.uint32)
            # every bucket of the buffer sits in exactly one scope: ops that write only covered rows write all rows
            hit.covers_all_rows = True
            _SCOPE_CACHE[key] = hit
        return hit
