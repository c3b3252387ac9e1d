"""Sub-bucket pooling buffers (reference: flash3dxfmr/psh/subbuck.py:40-132)."""
import dataclasses as dcls

import torch

from .arithmatic import cdiv
from . import batching as f3dbatch


def calc_red_sep_sizes(seps: torch.Tensor, subbuck_size: int):
    """Every cloud of n points pools to ceil(n / subbuck_size) rows: (total rows, per-cloud rows,
    cumulative rows) with the dtype of `seps` (subbuck.py:40-53).  Computed on the host from the cloud
    sizes (known there after one copy per separator tensor) and remembered per tensor, so a repeated
    forward on the same batch neither synchronises nor uploads anything; the returned cumulative tensor
    already carries its own sizes for the next level."""
    assert seps.dim() == 1, f"Seps dimension is expected to be 1, got {seps.dim()} instead"
    facts = f3dbatch.host_facts(seps)
    key = ("reduced", int(subbuck_size))
    if key not in facts:
        sizes = f3dbatch.host_sizes(seps)
        red = [(n + subbuck_size - 1) // subbuck_size for n in sizes]
        cum, acc = [], 0
        for r in red:
            acc += r
            cum.append(acc)
        as_dev = lambda v: torch.tensor(v, dtype=torch.int64).to(seps.dtype).to(seps.device)
        red_sizes, red_cum = as_dev(red), as_dev(cum)
        f3dbatch.host_facts(red_cum)["sizes"] = red
        facts[key] = (acc, red_sizes, red_cum)
    return facts[key]


@dcls.dataclass(slots=True)
class SubbuckBuffers:
    bbox_min: torch.Tensor
    bbox_max: torch.Tensor
    expect_sep: torch.Tensor
    subbuck_id: torch.Tensor
    subbuck_off: torch.Tensor
    reduced_sep: torch.Tensor
    reduced_coord: torch.Tensor
    reduced_feat: torch.Tensor
    unpool_ind: torch.Tensor

    @staticmethod
    def create_subbuck_buff(coords: torch.Tensor, input_feat: torch.Tensor, seps: torch.Tensor,
                            subbuck_size=2, out_alignment=1):
        """Allocation contract of batch_subbuck_reduce (subbuck.py:68-102).  `unpool_ind` MUST be
        prefilled with an index >= N: that marks a slot no point was mapped to.  The reduced length is
        rounded up to `out_alignment` so the next level's attention buckets divide it; the op
        zero-fills the extra rows (the reference leaves them uninitialised)."""
        total_n, d = coords.shape
        dev = coords.device
        # The op quantises inside each tile's own box; the whole-batch box is part of the reference
        # signature only.  It is kept cheap: no reduction pass, just the representable range.
        bbox_min = torch.full((d,), -65504.0, dtype=torch.float16, device=dev)
        bbox_max = torch.full((d,), 65504.0, dtype=torch.float16, device=dev)
        red_len, _, red_sep = calc_red_sep_sizes(seps, subbuck_size)
        aligned = cdiv(red_len, out_alignment) * out_alignment
        return SubbuckBuffers(
            bbox_min, bbox_max, red_sep,
            torch.zeros(total_n, dtype=torch.uint32, device=dev),
            torch.empty(total_n, dtype=torch.uint16, device=dev),
            red_sep,
            torch.empty(aligned, d, dtype=torch.float16, device=dev),
            torch.empty(aligned, input_feat.shape[1], dtype=input_feat.dtype, device=dev),
            torch.full((red_len, subbuck_size), total_n + 3, dtype=torch.int32, device=dev).view(torch.uint32),
        )

    def remove_unused_buffers(self):
        del self.subbuck_id
        del self.subbuck_off


@dcls.dataclass(slots=True)
class UnpoolBuffers:
    up_add_feat: torch.Tensor

    @staticmethod
    def create_unpool_buff(residual_feat: torch.Tensor):
        return UnpoolBuffers(torch.empty_like(residual_feat))


@dcls.dataclass(slots=True)
class UnpoolGradients:
    """gradient buffers of additive unpooling (reference: psh/subbuck.py:119-132): grad_res like the output
    gradient, grad_down with the aligned row count of the pooled features; both start from zero because the
    kernel leaves rows that no slot refers to untouched"""
    grad_res: torch.Tensor
    grad_down: torch.Tensor

    @staticmethod
    def create_unpool_grad(grad_up_added: torch.Tensor, sb: "SubbuckBuffers", down_len: int = None):
        feat_dim = grad_up_added.shape[-1]
        if down_len is None:
            down_len = sb.reduced_feat.shape[0]
        grad_res = torch.zeros_like(grad_up_added)
        grad_down = torch.zeros(down_len, feat_dim, dtype=grad_up_added.dtype, device=grad_up_added.device)
        return UnpoolGradients(grad_res, grad_down)
