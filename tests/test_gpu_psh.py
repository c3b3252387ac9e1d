"""GPU parity of PSH bucketing (rows A1-A3, A5) against the CPU oracle, through the C ABI
(pshattn -> libf3d_hip.so).  Bit-exact: bucket ids, histograms, slots (stable order), cumsum and
every scattered coordinate row.  Also the reference's own invariants (tests/test_psh.py:117-129 of
the reference): no NaN left, cumsum identity, scoreboard."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV, n_f16, n_u16, n_u32, t_f16, t_u32

pytestmark = pytest.mark.gpu


def _run_psh(coords, seps, bucket_size, hash_op, pad_align, oracle, rebalance=0):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import bucket as f3dbuck
    nb, div, max_n = oracle.psh_params(seps, bucket_size)
    n = coords.shape[0]
    pad_to = -(-n // pad_align) * pad_align
    c, s = t_f16(coords), t_u32(seps)
    bucket_id = torch.ones(n, dtype=torch.uint16, device=DEV)
    cntr = torch.zeros(len(seps), nb, dtype=torch.uint32, device=DEV)
    offs = torch.empty(n, dtype=torch.uint32, device=DEV)
    cumsum = torch.zeros_like(cntr)
    probes = f3dbuck.generate_probe_offsets(DEV, shuffle_seed=0)
    scat = torch.full((pad_to, 3), float("nan"), dtype=torch.float16, device=DEV)
    bmin, bmax = torch.min(c, dim=0)[0], torch.max(c, dim=0)[0]
    mgr = pshattn.DeviceManagerSingleton.instance()
    mgr.init_dev_info(0)
    mgr.set_sync_stream(True)
    mgr.set_psh_rebalance(rebalance)
    pshattn.batch_psh_scatter_pad_hash(c, bucket_id, cntr, offs, s, max_n, nb, div, bucket_size, 0xFFFF, bmin, bmax,
                                       probes, cumsum, scat, 0.0, hash_op)
    torch.cuda.synchronize()
    return dict(nb=nb, div=div, pad_to=pad_to, ids=n_u16(bucket_id), cnt=n_u32(cntr), off=n_u32(offs),
                cumsum=n_u32(cumsum), scat=n_f16(scat), bmin=n_f16(bmin), bmax=n_f16(bmax),
                t=(bucket_id, cntr, offs, s), t_cumsum=cumsum)


def _check_against_oracle(coords, seps, out, hash_op, oracle, rebalance=0, bucket_size=512):
    ids, cnt, off = oracle.psh_claim(coords, seps, out["bmin"], out["bmax"], 0xFFFF, out["div"], out["nb"], hash_op)
    if rebalance:
        ids, cnt, off = oracle.psh_rebalance(ids, cnt, off, seps, bucket_size)
    cumsum, scat = oracle.cumsum_scatter_pad(coords, seps, out["nb"], ids, cnt, off, out["pad_to"], 0.0)
    assert np.array_equal(out["ids"], ids), "bucket ids differ"
    assert np.array_equal(out["cnt"], cnt), "bucket histograms differ"
    assert np.array_equal(out["off"], off), "slots differ (stable order expected)"
    assert np.array_equal(out["cumsum"], cumsum)
    assert np.array_equal(out["scat"].view(np.uint16), scat.view(np.uint16)), "scattered rows differ"


@pytest.mark.parametrize("hash_op", [1, 2, 3, 4])
def test_c1_uniform_cube_bit_exact(oracle, hash_op):
    """BASELINE config 1: 1 x 32,768 points uniform in a 51.2 m cube, bucket 512 -> 64 buckets"""
    import bench_workloads as synth
    coords, seps = synth.batch_of([synth.uniform_cube(32768, 51.2, 1001)])
    out = _run_psh(coords, seps, 512, hash_op, 512, oracle)
    assert out["nb"] == 64 and out["div"] == 1024
    _check_against_oracle(coords, seps, out, hash_op, oracle)
    assert not np.isnan(out["scat"]).any()
    rc, _ = oracle.scoreboard(out["ids"], out["cnt"], out["off"], seps)
    assert rc == 0


def test_quantiser_division_mode_bit_exact(oracle):
    """f3d_set_quantiser(1): IEEE division in the voxel quantiser (src/psh/hash_fns.cuh:23-33 as written), for a user
    whose CUDA build of the reference was not a fast-math one.  Every fp16 pattern as a coordinate (so every rounding
    case of the quotient is in the batch) plus config 1's cloud; ids, counts, slots and scattered rows against the
    oracle in the same mode; the two modes differ on this input, so the switch is seen to act; the sub-bucket
    builder follows the same switch."""
    import bench_workloads as synth
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import subbuck
    mgr = pshattn.DeviceManagerSingleton.instance()
    bits = np.arange(65536, dtype=np.uint16).view(np.float16)
    bits = bits[np.isfinite(bits) & (np.abs(bits.astype(np.float32)) <= 80.0)]
    rng = np.random.default_rng(11)
    every = np.stack([bits, rng.permutation(bits), rng.permutation(bits)], axis=1)
    cube, _ = synth.batch_of([synth.uniform_cube(32768, 51.2, 1001)])
    coords = np.concatenate([every, cube]).astype(np.float16)
    seps = np.array([every.shape[0], coords.shape[0]], dtype=np.uint32)
    assert mgr.get_quantiser() == 0
    base = _run_psh(coords, seps, 512, 1, 512, oracle)
    try:
        mgr.set_quantiser(1)
        oracle.set_quantiser(1)
        assert mgr.get_quantiser() == 1
        for hash_op in (1, 2, 3, 4):
            out = _run_psh(coords, seps, 512, hash_op, 512, oracle, rebalance=hash_op % 2)
            _check_against_oracle(coords, seps, out, hash_op, oracle, rebalance=hash_op % 2)
            if hash_op == 1:
                assert (out["ids"] != base["ids"]).any() or (out["off"] != base["off"]).any()
        # sub-bucket builder in the same mode
        S = 4
        c, s = t_f16(coords), t_u32(seps)
        f = torch.zeros(coords.shape[0], 8, dtype=torch.bfloat16, device=DEV)
        sb = subbuck.SubbuckBuffers.create_subbuck_buff(c, f, s, S, out_alignment=1)
        max_n = int(np.diff(np.concatenate([[0], seps.astype(np.int64)])).max())
        pshattn.batch_subbuck_reduce(c, f, s, max_n, S, 0xFFFF, sb.bbox_min, sb.bbox_max, sb.subbuck_id, sb.subbuck_off,
                                     sb.reduced_sep, sb.reduced_coord, sb.reduced_feat, sb.unpool_ind, 1, 0)
        torch.cuda.synchronize()
        sid, soff, unpool, red_coord, _ = oracle.subbuck_build(coords, seps, S)
        assert np.array_equal(n_u32(sb.unpool_ind), unpool) and np.array_equal(n_u32(sb.subbuck_id), sid)
        assert np.array_equal(n_f16(sb.reduced_coord).view(np.uint16), red_coord.view(np.uint16))
    finally:
        mgr.set_quantiser(0)
        oracle.set_quantiser(0)
    with pytest.raises(RuntimeError, match="quantiser mode"):
        mgr.set_quantiser(3)


@pytest.mark.parametrize("sizes,bucket_size", [
    ([20000, 17001, 23456], 512),          # ragged batch, partial tail tiles
    ([70000, 300, 65000, 1], 512),         # tiny and single-point clouds next to large ones
    ([9000, 0, 8000], 256),                # an empty cloud in the middle
    ([300000, 280000], 512),               # 512 buckets, multi-item tiles
])
def test_ragged_batches_bit_exact(oracle, sizes, bucket_size):
    rng = np.random.default_rng(sum(sizes))
    pts = np.concatenate([rng.normal(0, 20, (n, 3)) + rng.uniform(-5, 5, 3) for n in sizes]).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    for hash_op in (1, 4):
        out = _run_psh(pts, seps, bucket_size, hash_op, bucket_size * 6, oracle)
        _check_against_oracle(pts, seps, out, hash_op, oracle)
        n = pts.shape[0]
        assert (out["scat"][n:] == 0).all() and not np.isnan(out["scat"]).any()


@pytest.mark.parametrize("sizes,bucket_size", [
    ([5000, 8192, 1, 0, 777], 64),         # clouds of at most 8192 points, an empty and a one-point cloud
    ([16384, 12000, 3], 512),              # exactly 16,384
    ([32768, 16385, 20000, 0], 512),       # exactly 32,768, one point more than 16,384, an empty last cloud
])
@pytest.mark.parametrize("rebalance", [0, 1])
def test_small_clouds_bit_exact(oracle, sizes, bucket_size, rebalance):
    """Small clouds at the tile-size boundaries, half of each cloud clustered so that buckets overflow and the
    rebalance plan is in use, empty and one-point clouds, pad rows, all four hash types; ids, counts, slots and
    scattered rows bit-exact vs the oracle."""
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(sum(sizes) + rebalance)
    pts = np.concatenate([np.concatenate([rng.normal(0, 2.0, (n // 2, 3)), rng.uniform(-30, 30, (n - n // 2, 3))])
                          for n in sizes]).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    for hash_op in (1, 2, 3, 4):
        out = _run_psh(pts, seps, bucket_size, hash_op, bucket_size * 6, oracle, rebalance=rebalance)
        _check_against_oracle(pts, seps, out, hash_op, oracle, rebalance=rebalance, bucket_size=bucket_size)
        n = pts.shape[0]
        assert (out["scat"][n:] == 0).all() and not np.isnan(out["scat"]).any()
        if rebalance:
            assert (out["cnt"][:, 1:] <= bucket_size).all()
    pshattn.DeviceManagerSingleton.instance().set_psh_rebalance(1)


def test_lidar_batch_reference_invariants(oracle):
    """4 synthetic sweeps (heavily clustered): the reference's three checks, through its own
    sanitizer entry point"""
    import bench_workloads as synth
    from flash3dtransformer_amd.lib import pshattn
    clouds = [synth.lidar_sweep(30000, 1004 + i, oversample=2) for i in range(4)]
    coords, seps = synth.batch_of(clouds)
    for hash_op in (1, 2, 3, 4):
        out = _run_psh(coords, seps, 512, hash_op, 512, oracle)
        _check_against_oracle(coords, seps, out, hash_op, oracle)
        bucket_id, cntr, offs, s = out["t"]
        assert not np.isnan(out["scat"]).any()
        assert np.array_equal(np.cumsum(out["cnt"], axis=1), out["cumsum"])
        maxc = int(out["cnt"].max())
        table = torch.zeros((4, out["nb"], maxc), dtype=torch.int8, device=DEV)
        res = cntr.clone()
        maxcnt = torch.from_numpy(out["cnt"].max(1).astype(np.int32)).to(DEV).view(torch.uint32)
        pshattn.batch_bucket_sanitizer_cpu(bucket_id, cntr, offs, table, res, s, maxcnt, 4, out["nb"])
        assert int(res.view(torch.int32).abs().sum()) == 0


def test_degenerate_axis_and_special_values(oracle):
    """flat cloud (z constant -> 0/0 in the quantiser) and points outside the given box"""
    rng = np.random.default_rng(1)
    pts = rng.uniform(-10, 10, (20000, 3)).astype(np.float16)
    pts[:, 2] = np.float16(1.5)
    seps = np.array([20000], np.uint32)
    out = _run_psh(pts, seps, 512, 1, 512, oracle)
    _check_against_oracle(pts, seps, out, 1, oracle)


def test_bbox_kernel_matches_torch():
    from flash3dtransformer_amd.lib import pshattn
    g = torch.Generator().manual_seed(3)
    for n in (1, 63, 4097, 500001):
        c = (torch.randn(n, 3, generator=g) * 30).to(torch.float16).to(DEV)
        bb = torch.empty(2, 3, dtype=torch.float16, device=DEV)
        pshattn.coord_bbox(c, bb[0], bb[1])
        assert torch.equal(bb[0], c.min(0)[0]) and torch.equal(bb[1], c.max(0)[0])


def test_python_wrapper_and_saturating_size_properties(oracle):
    """psh_main.batch_bucket_scatter on 16 x 262,144 points: size-independent properties only
    (multiset of rows preserved, rows sorted by bucket id inside each cloud, pads zero)"""
    from flash3dtransformer_amd.psh import psh_main
    n_c, b = 262144, 16
    g = torch.Generator().manual_seed(5)
    coords = (torch.rand(n_c * b, 3, generator=g) * 51.2).to(torch.float16).to(DEV)
    seps = (torch.arange(1, b + 1, dtype=torch.int32) * n_c).to(DEV).view(torch.uint32)
    pad_to = -(-coords.shape[0] // 3072) * 3072
    scat, buf = psh_main.batch_bucket_scatter(coords, seps, 512, pad_to, 2)
    torch.cuda.synchronize()
    assert not torch.isnan(scat).any()
    cnt = buf.bucket_cntr.view(torch.int32).long()
    assert torch.equal(torch.cumsum(cnt, 1), buf.bucket_cumsum.view(torch.int32).long())
    assert int(cnt.sum()) == n_c * b
    # checksum of rows is permutation invariant per cloud
    key = lambda t: (t.view(torch.int16).long() & 0xFFFF).mul(torch.tensor([1, 65536, 65536 ** 2], device=DEV)).sum(1)
    kin, kout = key(coords).view(b, n_c), key(scat[:n_c * b]).view(b, n_c)
    assert torch.equal(kin.sort(1)[0], kout.sort(1)[0])
    # recompute bucket ids of the scattered rows: must be non-decreasing inside each cloud
    ids = buf.bucket_id.view(torch.int16).long() & 0xFFFF
    excl = torch.cumsum(cnt, 1) - cnt
    dst = (torch.arange(b, device=DEV).repeat_interleave(n_c) * n_c
           + excl.view(-1)[torch.arange(b, device=DEV).repeat_interleave(n_c) * cnt.shape[1] + ids]
           + buf.bucket_offs.view(torch.int32).long())
    assert torch.equal(scat[dst], coords)
    assert dst.unique().numel() == n_c * b


@pytest.mark.parametrize("rebalance", [0, 1])
def test_large_tile_configuration_bit_exact(oracle, rebalance):
    """Batches big enough for the 8192-point tiles (LDS-staged scatter): 72 ragged clouds, 4.5 M points, half of
    them clustered so that buckets overflow; ids, counts, slots and scattered rows bit-exact vs the oracle"""
    import bench_workloads as synth
    rng = np.random.default_rng(77)
    clouds = []
    for i in range(72):
        n = int(rng.integers(56000, 70000))
        if i % 2:
            clouds.append((rng.normal(0, 8.0, (n, 3)) * np.array([1.0, 1.0, 0.1])).astype(np.float32))
        else:
            clouds.append(rng.uniform(0, 51.2, (n, 3)).astype(np.float32))
    clouds[5] = clouds[5][:8191]        # one tile minus one point
    clouds[6] = clouds[6][:8193]        # one tile plus one point
    coords, seps = synth.batch_of(clouds)
    assert -(-max(len(c) for c in clouds) // 8192) * len(clouds) >= 512
    out = _run_psh(coords, seps, 512, 2, 3072, oracle, rebalance=rebalance)
    _check_against_oracle(coords, seps, out, 2, oracle, rebalance=rebalance)
    assert not np.isnan(out["scat"]).any()
    from flash3dtransformer_amd.lib import pshattn
    pshattn.DeviceManagerSingleton.instance().set_psh_rebalance(1)


@pytest.mark.parametrize("case", ["lidar", "uniform_exact_capacity", "ragged"])
def test_rebalance_bit_exact_and_reference_invariants(oracle, case):
    """A4 (deterministic overflow rebalance + recycle): final ids, counts, slots and scattered rows
    bit-exact vs the oracle, and the reference's three checks on the result"""
    import bench_workloads as synth
    from flash3dtransformer_amd.lib import pshattn
    if case == "lidar":
        clouds = [synth.lidar_sweep(40000, 1004 + i, oversample=2) for i in range(3)]
    elif case == "uniform_exact_capacity":
        clouds = [synth.uniform_cube(65536, 51.2, 1002), synth.uniform_cube(65536, 51.2, 1003)]
    else:
        rng = np.random.default_rng(5)
        clouds = [rng.normal(0, s, (n, 3)).astype(np.float32) for n, s in ((50000, 3.0), (700, 30.0), (90001, 12.0))]
    coords, seps = synth.batch_of(clouds)
    for hash_op in (1, 2):
        out = _run_psh(coords, seps, 512, hash_op, 3072, oracle, rebalance=1)
        _check_against_oracle(coords, seps, out, hash_op, oracle, rebalance=1)
        assert not np.isnan(out["scat"]).any()
        assert np.array_equal(np.cumsum(out["cnt"], axis=1), out["cumsum"])
        assert (out["cnt"][:, 1:] <= 512).all()
        bucket_id, cntr, offs, s = out["t"]
        b = len(seps)
        table = torch.zeros((b, out["nb"], int(out["cnt"].max())), dtype=torch.int8, device=DEV)
        res = cntr.clone()
        maxcnt = torch.from_numpy(out["cnt"].max(1).astype(np.int32)).to(DEV).view(torch.uint32)
        pshattn.batch_bucket_sanitizer_cpu(bucket_id, cntr, offs, table, res, s, maxcnt, b, out["nb"])
    pshattn.DeviceManagerSingleton.instance().set_psh_rebalance(1)


@pytest.mark.parametrize("sizes,bucket_size,rebalance,feat_shape,feat_dtype", [
    ([20000, 17001, 23456], 512, 1, (64,), torch.bfloat16),     # 128-byte rows: 8 lanes x 16 B
    ([9000, 0, 8000], 256, 0, (1,), torch.bfloat16),            # 2-byte rows, an empty cloud
    ([70000, 300, 65000, 1], 512, 1, (4,), torch.float32),      # KITTI-style [n, 4] float rows
    ([33000, 31000], 512, 1, (3, 5), torch.float16),            # 30-byte rows: 2-byte units, 16 lanes
    ([300000, 280000], 512, 1, (256,), torch.bfloat16),         # 512-byte rows at the large-tile configuration
])
def test_scatter_index_and_features_bit_exact(oracle, sizes, bucket_size, rebalance, feat_shape, feat_dtype):
    """Permutation index + feature scatter (batch_psh_bucket.cuh:617-753) against the oracle, bit for bit; the
    index must also reproduce the coordinate scatter of the bucketing call itself, and permute_rows must move rows
    both ways."""
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(sum(sizes) + 1)
    pts = np.concatenate([rng.normal(0, 20, (n, 3)) + rng.uniform(-5, 5, 3) for n in sizes]).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    n = pts.shape[0]
    out = _run_psh(pts, seps, bucket_size, 2, bucket_size * 6, oracle, rebalance=rebalance)
    bucket_id, cntr, offs, s = out["t"]
    pad_to = out["pad_to"]
    g = torch.Generator().manual_seed(7)
    feat = torch.randn((n,) + feat_shape, generator=g).to(feat_dtype).to(DEV)
    index = torch.full((pad_to,), 0xFFFFFFF, dtype=torch.int32, device=DEV).view(torch.uint32)
    sfeat = torch.full((pad_to,) + feat_shape, 7.0, dtype=feat_dtype, device=DEV)
    pshattn.psh_scatter_feat_index(bucket_id, cntr, offs, s, out["t_cumsum"], index, feat, sfeat)
    index_only = torch.empty_like(index)
    pshattn.psh_scatter_feat_index(bucket_id, cntr, offs, s, out["t_cumsum"], index_only)
    torch.cuda.synchronize()
    bits = {2: torch.int16, 4: torch.int32}[feat.element_size()]
    feat_np = feat.cpu().view(bits).numpy()
    ref_idx, ref_feat = oracle.scatter_feat_index(seps, out["nb"], out["ids"], out["off"], out["cumsum"], pad_to, feat_np)
    idx = n_u32(index)
    assert np.array_equal(idx, ref_idx) and np.array_equal(n_u32(index_only), ref_idx)
    assert np.array_equal(sfeat.cpu().view(bits).numpy(), ref_feat)
    # independent of the oracle: the index reproduces the bucketing call's own coordinate scatter
    assert np.array_equal(pts[idx[:n]].view(np.uint16), out["scat"][:n].view(np.uint16))
    assert (idx[n:] == n + 3).all()
    # permute_rows: gather by the index = the fused feature scatter; the other direction restores the input
    gathered = torch.full_like(sfeat, 3.0)
    pshattn.permute_rows(index, feat, gathered, True)
    restored = torch.full_like(feat, 5.0)
    pshattn.permute_rows(index, gathered, restored, False)
    torch.cuda.synchronize()
    assert torch.equal(gathered.view(bits), sfeat.view(bits))
    assert torch.equal(restored.view(bits), feat.view(bits))


def test_scatter_index_misaligned_rows_and_errors():
    """Rows whose base address is only 2-byte aligned fall back to narrower units; bad arguments raise."""
    from flash3dtransformer_amd.lib import pshattn
    n, c = 1000, 24
    g = torch.Generator().manual_seed(3)
    perm = torch.randperm(n, generator=g).to(torch.int32)
    index = torch.cat([perm, torch.full((24,), n + 3, dtype=torch.int32)]).to(DEV).view(torch.uint32)
    base = torch.randn(n * c + 1, generator=g).to(torch.bfloat16).to(DEV)
    src = base[1:].view(n, c)                       # 2-byte aligned rows
    dst = torch.full((n + 24, c), 9.0, dtype=torch.bfloat16, device=DEV)
    pshattn.permute_rows(index, src, dst, True)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src[perm.to(DEV).long()]) and (dst[n:] == 0).all()
    with pytest.raises(RuntimeError, match="row shape or dtype"):
        pshattn.permute_rows(index, src, dst.float(), True)
    with pytest.raises(RuntimeError, match="entries"):
        pshattn.permute_rows(index[:10], src, dst, True)


def test_layer_permutation_is_differentiable_and_model_takes_features():
    """to_psh_order / to_input_order are each other's gradient; Flash3D with in_feat_dim consumes input_feat
    and to_input_order returns per-point rows in the order the points came in."""
    import bench_workloads as synth
    from flash3dtransformer_amd.layers import psh_ops
    from flash3dtransformer_amd.psh import psh_main as pm
    coords, seps = synth.batch_of([synth.uniform_cube(9000, 40.0, 5), synth.uniform_cube(8200, 40.0, 6)])
    c, s = t_f16(coords), t_u32(seps)
    n = coords.shape[0]
    pad_to = -(-n // 1536) * 1536
    scattered, buffers = pm.batch_bucket_scatter(c, s, 256, pad_to, 2)
    index, _ = pm.batch_scatter_index(buffers, s)
    x = torch.randn(n, 16, device=DEV).to(torch.bfloat16).requires_grad_(True)
    y = psh_ops.to_psh_order(x, index)
    w = torch.randn(pad_to, 16, device=DEV).to(torch.bfloat16)
    (y.float() * w.float()).sum().backward()
    idx = index.view(torch.int32)[:n].long()
    assert torch.equal(y[:n], x.detach()[idx]) and (y[n:] == 0).all()
    expect = torch.zeros(n, 16, dtype=torch.bfloat16, device=DEV)
    expect[idx] = w[:n]
    assert torch.equal(x.grad, expect)
    back = psh_ops.to_input_order(y.detach(), index, n)
    assert torch.equal(back, x.detach())
    # coordinates gathered by the index are the scattered coordinates
    assert torch.equal(psh_ops.to_psh_order(c, index)[:n], scattered[:n])
