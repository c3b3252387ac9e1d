"""KITTI velodyne ingress (reference: tests/test_psh.py:31-44, psh/batching.py:13-28) on synthetic sweep files."""
import os

import numpy as np
import pytest
import torch


def _write_tree(tmp_path, sizes):
    from flash3dtransformer_amd.psh import ingress
    rng = np.random.default_rng(5)
    sweeps = []
    for i, n in enumerate(sizes):
        pts = np.concatenate([rng.normal(0, 20, (n, 3)), rng.uniform(0, 1, (n, 1))], axis=1).astype(np.float32)
        ingress.write_velodyne_bin(str(tmp_path / "dataset" / "sequences" / f"{i // 2:02d}" / "velodyne" / f"{i:06d}.bin"), pts)
        sweeps.append(pts)
    return sweeps


def test_build_batch_matches_reference_recipe(tmp_path):
    from flash3dtransformer_amd.psh import ingress
    sizes = [1001, 64, 7, 2500]
    sweeps = _write_tree(tmp_path, sizes)
    files = list(ingress.kitti_sweep_files(str(tmp_path)))
    assert [os.path.basename(f) for f in files] == [f"{i:06d}.bin" for i in range(4)]
    coords, seps = ingress.build_batch(files, down_sample_ratio=2)
    kept = [n // 2 for n in sizes]
    assert coords.dtype == torch.float16 and seps.dtype == torch.uint32
    assert seps.view(torch.int32).tolist() == np.cumsum(kept).tolist()
    want = np.concatenate([s[:k, :3] for s, k in zip(sweeps, kept)]).astype(np.float16)
    assert np.array_equal(coords.numpy().view(np.uint16), want.view(np.uint16))
    c3, s3, refl = ingress.build_batch(files, num_samples=3, down_sample_ratio=1, with_reflectance=True)
    assert c3.shape[0] == sum(sizes[:3]) == refl.shape[0] and s3.shape[0] == 3
    assert np.array_equal(refl.numpy()[:, 0], np.concatenate([s[:, 3] for s in sweeps[:3]]))


def test_malformed_and_empty_files(tmp_path):
    from flash3dtransformer_amd.psh import ingress
    bad = tmp_path / "bad.bin"
    bad.write_bytes(b"\x00" * 20)                      # not a multiple of 16 bytes
    with pytest.raises(ValueError):
        ingress.load_velodyne_bin(str(bad))
    empty = tmp_path / "empty.bin"
    empty.write_bytes(b"")
    assert ingress.load_velodyne_bin(str(empty)).shape == (0, 4)
    with pytest.raises(ValueError):
        ingress.build_batch([])
