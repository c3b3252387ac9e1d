"""Point-cloud ingress: KITTI velodyne sweeps -> the (coords, seps) batch the PSH ops take.

The reference reads sweeps in its tests only (tests/test_psh.py:31-44: ``np.fromfile(f, float32).reshape(-1, 4)``,
keep the first ``n // down_sample_ratio`` points, ``collate_coords_flat_sep`` to fp16 coordinates and uint32
separators).  This module gives that path a home in the package; a sweep file holds float32 records
(x, y, z, reflectance), little endian, without a header.
"""
import glob
import os
from typing import Iterable, Iterator, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import batching as f3dbatch

RECORD_FLOATS = 4  # x, y, z, reflectance


def kitti_sweep_files(kitti_root: str) -> Iterator[str]:
    """sweep files of every sequence under ``<root>/dataset/sequences/*/velodyne/*.bin``, in sorted order
    (the reference iterates the same pattern in directory order, tests/test_psh.py:31-32)"""
    return iter(sorted(glob.glob(os.path.join(kitti_root, "dataset", "sequences", "*", "velodyne", "*.bin"))))


def load_velodyne_bin(path: str, mmap: bool = True) -> np.ndarray:
    """one sweep as float32 [n, 4]; memory-mapped by default so that a large sequence is not read eagerly"""
    size = os.path.getsize(path)
    if size % (4 * RECORD_FLOATS) != 0:
        raise ValueError(f"{path}: {size} bytes is not a whole number of (x, y, z, reflectance) float32 records")
    if size == 0:
        return np.empty((0, RECORD_FLOATS), dtype=np.float32)
    if mmap:
        return np.memmap(path, dtype="<f4", mode="r").reshape(-1, RECORD_FLOATS)
    return np.fromfile(path, dtype="<f4").reshape(-1, RECORD_FLOATS)


def build_batch(files: Iterable[str], num_samples: Optional[int] = None, down_sample_ratio: int = 2,
                coord_dtype=torch.float16, sep_dtype=torch.uint32,
                with_reflectance: bool = False) -> Tuple[torch.Tensor, ...]:
    """(coords [N, 3], seps [B]) from the first ``num_samples`` files, keeping the first
    ``n // down_sample_ratio`` points of every sweep (tests/test_psh.py:34-44); with ``with_reflectance`` also
    the reflectance column [N, 1] float32 as a third value (an input feature the reference's tests drop)"""
    assert down_sample_ratio >= 1
    sweeps: List[torch.Tensor] = []
    for i, f in enumerate(files):
        if num_samples is not None and i >= num_samples:
            break
        rec = load_velodyne_bin(f)
        keep = rec.shape[0] // down_sample_ratio
        sweeps.append(torch.from_numpy(np.ascontiguousarray(rec[:keep])))
    if not sweeps:
        raise ValueError("no sweep files given")
    coords, seps = f3dbatch.collate_coords_flat_sep(sweeps, coord_dtype=coord_dtype, sep_dtype=sep_dtype)
    if with_reflectance:
        return coords, seps, torch.cat([s[:, 3:4] for s in sweeps], dim=0).contiguous()
    return coords, seps


def write_velodyne_bin(path: str, points_xyzr: np.ndarray) -> None:
    """inverse of ``load_velodyne_bin`` (synthetic sweeps for tests and demos)"""
    a = np.ascontiguousarray(points_xyzr, dtype="<f4")
    assert a.ndim == 2 and a.shape[1] == RECORD_FLOATS
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    a.tofile(path)
