"""Workloads that bench.py, the parity tests and the smoke test share; not part of the library.

Synthetic point clouds (numpy, seeded; no dataset is needed):
uniform_cube  points ~ U[0, side)^3
lidar_sweep   a spinning-LiDAR-like sweep: 64 elevation rings from -25 deg to +2 deg, 2048 azimuth
              steps, rays cast from the origin against a ground plane z = -1.7 m and random
              axis-aligned boxes, ranges kept in [2, 80] m, then thinned to the requested size with
              acceptance proportional to 1/r^2.

Model-level workloads: the encoder stage (4 LiDAR sweeps x 120,000 points, C = 256, 8 heads x 32, gated MLP with
1024 hidden features) and the 5-level hourglass (channels 32 / 64 / 128 / 256 / 512, 32-wide heads, bucket 512).
Weights are random from a seed, rounded to bf16; modules come back on the CPU in eval mode."""
import math

import numpy as np
import torch


def uniform_cube(n: int, side: float = 51.2, seed: int = 1001) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.uniform(0.0, side, (n, 3)).astype(np.float32)


def _ray_box(dirs, lo, hi):
    """slab test for rays from the origin; returns hit distance (inf when missed)"""
    with np.errstate(divide="ignore", invalid="ignore"):
        t1 = lo[None, :] / dirs
        t2 = hi[None, :] / dirs
    tmin = np.nanmax(np.minimum(t1, t2), axis=1)
    tmax = np.nanmin(np.maximum(t1, t2), axis=1)
    hit = (tmax >= np.maximum(tmin, 0.0)) & (tmin > 0.0)
    return np.where(hit, tmin, np.inf)


def lidar_sweep(n_points: int = 120_000, seed: int = 1004, n_rings: int = 64, n_azimuth: int = 2048,
                n_boxes: int = 30, oversample: int = 4) -> np.ndarray:
    """float32 [n_points, 4]: x, y, z, intensity ~ U[0, 1)"""
    rng = np.random.default_rng(seed)
    elev = np.deg2rad(np.linspace(-25.0, 2.0, n_rings))
    centres = rng.uniform(-60.0, 60.0, (n_boxes, 2))
    sizes = rng.uniform(1.0, 6.0, (n_boxes, 3))
    ground = -1.7
    pts = []
    for _ in range(oversample):
        az = (np.arange(n_azimuth) + rng.uniform(0.0, 1.0, n_azimuth)) * (2.0 * np.pi / n_azimuth)
        e, a = np.meshgrid(elev, az, indexing="ij")
        e = e + rng.normal(0.0, np.deg2rad(0.05), e.shape)
        dirs = np.stack([np.cos(e) * np.cos(a), np.cos(e) * np.sin(a), np.sin(e)], axis=-1).reshape(-1, 3)
        with np.errstate(divide="ignore"):
            t = np.where(dirs[:, 2] < 0, ground / dirs[:, 2], np.inf)
        for c, s in zip(centres, sizes):
            lo = np.array([c[0] - s[0] / 2, c[1] - s[1] / 2, ground])
            hi = np.array([c[0] + s[0] / 2, c[1] + s[1] / 2, ground + s[2]])
            t = np.minimum(t, _ray_box(dirs, lo, hi))
        keep = (t >= 2.0) & (t <= 80.0)
        pts.append(dirs[keep] * t[keep, None])
    pts = np.concatenate(pts, axis=0)
    r2 = (pts ** 2).sum(1)
    w = 1.0 / r2
    w /= w.sum()
    if pts.shape[0] < n_points:
        raise ValueError(f"only {pts.shape[0]} returns for {n_points} requested points; raise `oversample`")
    # weighted sampling without replacement (Efraimidis-Spirakis keys), O(n log n) and seed-stable
    keys = rng.uniform(0.0, 1.0, pts.shape[0]) ** (1.0 / (w * pts.shape[0]))
    idx = np.sort(np.argpartition(-keys, n_points - 1)[:n_points])   # keep sweep (ring-major) order
    out = np.empty((n_points, 4), dtype=np.float32)
    out[:, :3] = pts[idx]
    out[:, 3] = rng.uniform(0.0, 1.0, n_points)
    return out


def batch_of(clouds):
    """list of [n_i, >=3] arrays -> (fp16 xyz [N, 3], uint32 inclusive cumulative sizes [B])"""
    xyz = np.concatenate([c[:, :3] for c in clouds], axis=0).astype(np.float16)
    seps = np.cumsum([c.shape[0] for c in clouds]).astype(np.uint32)
    return np.ascontiguousarray(xyz), seps


ENCODER_STAGE = dict(channels=256, hidden=1024, heads=8, bucket_size=512, scope_size=1, hash_type=2)
HOURGLASS = dict(channels=(32, 64, 128, 256, 512), bucket_size=512, scope_size=1, hash_type=2, subbuck_size=2)


def _xavier_bf16_(modules, seed):
    g = torch.Generator().manual_seed(seed)
    for m in modules:
        for _, p in m.named_parameters(recurse=False):
            if p.dim() == 2:
                bound = math.sqrt(6.0 / (p.shape[0] + p.shape[1]))
                p.data = ((torch.rand(p.shape, generator=g) * 2 - 1) * bound).to(torch.bfloat16).float()


def encoder_stage(activation="swiglu", seed=1004, scope_size=None):
    """(PSH3DCoordEmbedding, XFMR) of the encoder-stage workload, Xavier-uniform bf16-rounded weights"""
    from flash3dtransformer_amd import layers as L
    from flash3dtransformer_amd.psh.bucket_scope import SwinPlan
    c = ENCODER_STAGE
    scope = c["scope_size"] if scope_size is None else scope_size
    torch.manual_seed(seed)
    emb = L.PSH3DCoordEmbedding(c["channels"], c["bucket_size"], c["bucket_size"] * scope * 6)
    blk = L.XFMR(c["channels"], c["hidden"], c["heads"], c["bucket_size"], True,
                 SwinPlan("swin", c["bucket_size"], scope, 0), lambda ch: L.LayerNorm(ch), activation)
    _xavier_bf16_(list(emb.modules()) + list(blk.modules()), seed)
    return emb.eval(), blk.eval()


def hourglass(seed=1005, channels=None, bucket_size=None, subbuck_size=None):
    """Flash3D with one encoder and one decoder block per level, heads = C / 32, gated MLP with 4 C hidden features,
    mean pooling over `subbuck_size` points, LayerNorm around pooling / unpooling, pooled lengths aligned to a bucket"""
    from flash3dtransformer_amd import layers as L
    from flash3dtransformer_amd.psh.bucket_scope import SwinPlan
    c = HOURGLASS
    chans = list(channels or c["channels"])
    bs = bucket_size or c["bucket_size"]
    scope, S = c["scope_size"], subbuck_size or c["subbuck_size"]
    torch.manual_seed(seed)
    ln = lambda ch: L.LayerNorm(ch)
    spec = lambda ch: L.XFMRSpecs(ch, 4 * ch, ch // 32, True, SwinPlan("swin", bs, scope, 0), ln)
    levels = [L.F3DLevelSpecs([spec(ch)], [spec(ch)], "mean", bs * scope, ln if i + 1 < len(chans) else None, None,
                              ln if i + 1 < len(chans) else None, None) for i, ch in enumerate(chans)]
    model = L.Flash3D(levels, bs, scope, c["hash_type"], subbuck_size=S)
    # weights rounded to bf16 so that a CPU restatement reads the same numbers
    for p in model.parameters():
        p.data = p.data.to(torch.bfloat16).float()
    return model.eval()


HOURGLASS_REF_SHAPE = dict(channels=(32, 64, 128, 256, 512), bucket_size=512, scope_size=8, hash_type=2, subbuck_size=2)


def hourglass_ref_shape(seed=1005, channels=None):
    """Flash3D in the shape of the reference's own model test (tests/test_psh_hourglass.py:55-150 of the reference),
    extended to five levels: scopes of 8 buckets of 512, two encoder and two decoder blocks per level (the first
    encoder block of the first level on the "stride" plan, the others on "swin"), BatchNorm1d(eps=1e-3, momentum=0.01) +
    GELU around pooling and unpooling, pooled lengths aligned to bucket x scope, mean pooling over 2 points, gated MLP
    with 4 C hidden features.  Heads = C / 32 (the benchmark's head width; the reference's test uses 16-wide heads)."""
    from functools import partial
    from flash3dtransformer_amd import layers as L
    from flash3dtransformer_amd.psh.bucket_scope import SwinPlan, swinable_alignment
    c = HOURGLASS_REF_SHAPE
    chans = list(channels or c["channels"])
    bs, scope, S = c["bucket_size"], c["scope_size"], c["subbuck_size"]
    torch.manual_seed(seed)
    ln = lambda ch: L.LayerNorm(ch)
    bn = partial(torch.nn.BatchNorm1d, eps=1e-3, momentum=0.01)
    spec = lambda ch, plan, k: L.XFMRSpecs(ch, 4 * ch, ch // 32, True, SwinPlan(plan, bs, scope, k), ln)
    levels = []
    for i, ch in enumerate(chans):
        last = i + 1 == len(chans)
        levels.append(L.F3DLevelSpecs([spec(ch, "stride" if i == 0 else "swin", 1), spec(ch, "swin", 2)],
                                      [spec(ch, "swin", 3), spec(ch, "swin", 4)], "mean", swinable_alignment(bs, scope),
                                      None if last else bn, None if last else torch.nn.GELU,
                                      None if last else bn, None if last else torch.nn.GELU))
    model = L.Flash3D(levels, bs, scope, c["hash_type"], subbuck_size=S)
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():                      # running statistics and affine parameters that matter
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.1)
            m.running_var.copy_(torch.rand(m.num_features, generator=g) + 0.5)
            m.weight.data.copy_(torch.rand(m.num_features, generator=g) + 0.5)
            m.bias.data.copy_(torch.randn(m.num_features, generator=g) * 0.1)
    for p in model.parameters():
        p.data = p.data.to(torch.bfloat16).float()
    return model.eval()


def _act_name(act):
    return {None: None, torch.nn.GELU: "gelu", torch.nn.ReLU: "relu"}[act]


def hourglass_oracle_levels(model):
    """the per-level description oracle-side restatements of the model take (heads, block counts, pooling)"""
    out = []
    for spec in model.level_specs:
        out.append(dict(heads=spec.encoder_specs[0].num_heads, n_enc=len(spec.encoder_specs),
                        n_dec=len(spec.decoder_specs), red_op={"mean": 0, "sum": 1, "min": 2, "max": 3}.get(
                            spec.reduction_op, spec.reduction_op), pool_align=spec.pool_align,
                        pool_act=_act_name(spec.pool_act), unpool_act=_act_name(spec.unpool_act)))
    return out


def lidar_batch(n_clouds, points_per_cloud, seed):
    """(coords fp16 [N, 3], seps uint32 [B], list of float32 [n, 4] sweeps) of synthetic LiDAR sweeps"""
    clouds = [lidar_sweep(points_per_cloud, seed + i) for i in range(n_clouds)]
    coords, seps = batch_of(clouds)
    return coords, seps, clouds


def to_device(coords: np.ndarray, seps: np.ndarray, dev="cuda:0"):
    return (torch.from_numpy(coords).to(dev),
            torch.from_numpy(np.ascontiguousarray(seps).view(np.int32)).to(dev).view(torch.uint32))
