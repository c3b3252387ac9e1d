"""Writes the small known-answer fixtures of this folder (`*.npz`, tens of KB each).

The reference holds no golden vectors on disk (its tests draw `torch.randn` on the GPU or read KITTI
files), so the fixtures are produced by the CPU oracle of this repository, after the oracle itself
has been pinned by closed forms, brute force and library routines (tests/test_oracle_*.py).  They
freeze those answers: a later change to the oracle or to the kernels that moves any of them fails
tests/test_golden.py (CPU, oracle vs fixture) or tests/test_gpu_golden.py (HIP path vs fixture, no
oracle in the loop).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import f3d_oracle as orc  # noqa: E402


def bf16_bits(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def psh_fixture():
    """two clouds (150 + 106 points), bucket size 4 -> 32 buckets (the smallest bucket count the op accepts);
    all four hashes, rebalance off and on"""
    rng = np.random.default_rng(20240601)
    sizes = [150, 106]
    coords = np.concatenate([rng.normal(0, 8, (n, 3)) + rng.uniform(-3, 3, 3) for n in sizes]).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    bucket_size, pad_to = 4, 288
    nb, div, max_n = orc.psh_params(seps, bucket_size)
    bmin, bmax = coords.min(0), coords.max(0)
    out = dict(coords=coords.view(np.uint16), seps=seps, bucket_size=np.uint32(bucket_size), pad_to=np.uint32(pad_to),
               num_bucket=np.uint32(nb), divisor=np.uint32(div), max_n=np.uint32(max_n),
               bbox_min=bmin.view(np.uint16), bbox_max=bmax.view(np.uint16),
               vox=orc.vox_coord(coords, bmin, bmax))
    for h in (1, 2, 3, 4):
        ids, cnt, off = orc.psh_claim(coords, seps, bmin, bmax, 0xFFFF, div, nb, h)
        cumsum, scat = orc.cumsum_scatter_pad(coords, seps, nb, ids, cnt, off, pad_to, 0.0)
        out.update({f"h{h}_ids": ids, f"h{h}_cnt": cnt, f"h{h}_off": off, f"h{h}_cumsum": cumsum,
                    f"h{h}_scat": scat.view(np.uint16)})
        rid, rcnt, roff = orc.psh_rebalance(ids, cnt, off, seps, bucket_size)
        rcumsum, rscat = orc.cumsum_scatter_pad(coords, seps, nb, rid, rcnt, roff, pad_to, 0.0)
        out.update({f"h{h}_reb_ids": rid, f"h{h}_reb_cnt": rcnt, f"h{h}_reb_off": roff, f"h{h}_reb_cumsum": rcumsum,
                    f"h{h}_reb_scat": rscat.view(np.uint16)})
    np.savez_compressed(os.path.join(HERE, "psh_256pts.npz"), **out)


def pool_fixture():
    """sub-bucket pooling of 2 clouds (90 + 61 points), S=2 and S=3, 8 channels; all reduce ops; unpool"""
    rng = np.random.default_rng(20240602)
    sizes = [90, 61]
    coords = rng.uniform(-20, 20, (sum(sizes), 3)).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    feat = bf16_bits(rng.normal(0, 1, (sum(sizes), 8)))
    out = dict(coords=coords.view(np.uint16), seps=seps, feat=feat)
    for S in (2, 3):
        sub_id, sub_off, unpool, red_coord, red_sep = orc.subbuck_build(coords, seps, S, out_align=16)
        out.update({f"s{S}_sub_id": sub_id, f"s{S}_sub_off": sub_off, f"s{S}_unpool": unpool,
                    f"s{S}_red_coord": red_coord.view(np.uint16), f"s{S}_red_sep": red_sep})
        for op in (0, 1, 2, 3):
            out[f"s{S}_red_op{op}"] = orc.reduce_feat(feat, unpool, op, r_aligned=red_coord.shape[0])
        down = bf16_bits(rng.normal(0, 1, (red_coord.shape[0], 8)))
        out[f"s{S}_down"] = down
        out[f"s{S}_up"] = orc.additive_unpool(feat, down, unpool)
    np.savez_compressed(os.path.join(HERE, "pool_151pts.npz"), **out)


def attn_fixture():
    """2 buckets x 128 tokens per scope (the smallest bucket the op accepts), 2 scopes, 2 heads, head dim 16;
    fp32 reference output and LSE;
    a second case masks the tail of every bucket (kv_len)"""
    g = torch.Generator().manual_seed(20240603)
    B, L, H, D, bs = 1, 512, 2, 16, 128
    Q, K, V = [(torch.randn(B, L, H, D, generator=g)).to(torch.bfloat16) for _ in range(3)]
    scopes = np.array([[1, 0], [2, 3]], dtype=np.uint32)     # first scope lists its buckets in swapped order
    kv_len = np.array([128, 70, 1, 128], dtype=np.int32)
    O, LSE = orc.buck_swin_fwd(Q, K, V, scopes, bs)
    Om, LSEm = orc.buck_swin_fwd(Q, K, V, scopes, bs, kv_len=kv_len)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "attn_2x128.npz"), Q=bits(Q), K=bits(K), V=bits(V), scopes=scopes,
                        bucket_size=np.uint32(bs), kv_len=kv_len,
                        O=np.asarray(O, dtype=np.float32), LSE=np.asarray(LSE, dtype=np.float32),
                        O_masked=np.asarray(Om, dtype=np.float32), LSE_masked=np.asarray(LSEm, dtype=np.float32))


def dense_fixture():
    """one transformer block's dense path on 64 rows x 32 channels: LayerNorm -> linear, linear + residual,
    LayerNorm -> fc1 -> swiglu -> fc2 + residual (bf16 parameters, fp32 reference values)"""
    g = torch.Generator().manual_seed(20240604)
    r = lambda *s: torch.randn(*s, generator=g)
    bf = lambda t: t.to(torch.bfloat16)
    x = bf(r(64, 32))
    ln_w, ln_b = bf(1 + 0.1 * r(32)), bf(0.1 * r(32))
    w_qkv, b_qkv = bf(r(96, 32) * 0.2), bf(r(96) * 0.1)
    w1, b1 = bf(r(128, 32) * 0.2), bf(r(128) * 0.1)
    w2, b2 = bf(r(32, 64) * 0.2), bf(r(32) * 0.1)
    xf = x.float()
    ln = orc.layernorm(xf, ln_w.float(), ln_b.float())
    qkv = orc.linear(orc._r(ln), w_qkv.float(), b_qkv.float())
    h = orc.linear(orc._r(ln), w1.float(), b1.float())
    act = orc.swiglu(orc._r(h))
    y = orc.linear(orc._r(act), w2.float(), b2.float()) + xf
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "dense_64x32.npz"), x=bits(x), ln_w=bits(ln_w), ln_b=bits(ln_b),
                        w_qkv=bits(w_qkv), b_qkv=bits(b_qkv), w1=bits(w1), b1=bits(b1), w2=bits(w2), b2=bits(b2),
                        ln=ln.numpy(), qkv=qkv.numpy(), act=act.numpy(), y=y.numpy())


if __name__ == "__main__":
    orc.build()
    psh_fixture()
    pool_fixture()
    attn_fixture()
    dense_fixture()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
