"""The two model-level workloads the benchmark and the parity tests share: the encoder stage (4 LiDAR sweeps x
120,000 points, C = 256, 8 heads x 32, gated MLP with 1024 hidden features) and the 5-level hourglass (channels
32 / 64 / 128 / 256 / 512, 32-wide heads, bucket 512).  Weights are random from a seed, rounded to bf16; modules come
back on the CPU in eval mode."""
import math

import numpy as np
import torch

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
    from . import layers as L
    from .psh.bucket_scope import SwinPlan
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
    from . import layers as L
    from .psh.bucket_scope import SwinPlan
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


def hourglass_oracle_levels(model):
    """the per-level description oracle-side restatements of the model take (heads, block counts, pooling)"""
    out = []
    for spec in model.level_specs:
        out.append(dict(heads=spec.encoder_specs[0].num_heads, n_enc=len(spec.encoder_specs),
                        n_dec=len(spec.decoder_specs), red_op={"mean": 0, "sum": 1, "min": 2, "max": 3}.get(
                            spec.reduction_op, spec.reduction_op), pool_align=spec.pool_align,
                        pool_act=None, unpool_act=None))
    return out


def lidar_batch(n_clouds, points_per_cloud, seed):
    """(coords fp16 [N, 3], seps uint32 [B], list of float32 [n, 4] sweeps) of synthetic LiDAR sweeps"""
    from . import synth
    clouds = [synth.lidar_sweep(points_per_cloud, seed + i) for i in range(n_clouds)]
    coords, seps = synth.batch_of(clouds)
    return coords, seps, clouds


def to_device(coords: np.ndarray, seps: np.ndarray, dev="cuda:0"):
    return (torch.from_numpy(coords).to(dev),
            torch.from_numpy(np.ascontiguousarray(seps).view(np.int32)).to(dev).view(torch.uint32))
