"""The CPU oracle against the committed known-answer fixtures of tests/golden (written by
tests/golden/make_fixtures.py).  Integer structures must match bit for bit; floating-point
references to 1e-6 (they are fp32 torch results of the same formulas, so only library-version
noise is allowed)."""
import os

import numpy as np
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def _bf(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)


def test_psh_fixture(oracle):
    g = load("psh_256pts.npz")
    coords, seps = g["coords"].view(np.float16), g["seps"]
    bs, pad_to = int(g["bucket_size"]), int(g["pad_to"])
    nb, div, max_n = oracle.psh_params(seps, bs)
    assert (nb, div, max_n) == (int(g["num_bucket"]), int(g["divisor"]), int(g["max_n"])) == (32, 2048, 150)
    bmin, bmax = g["bbox_min"].view(np.float16), g["bbox_max"].view(np.float16)
    assert np.array_equal(coords.min(0).view(np.uint16), g["bbox_min"])
    assert np.array_equal(oracle.vox_coord(coords, bmin, bmax), g["vox"])
    for h in (1, 2, 3, 4):
        ids, cnt, off = oracle.psh_claim(coords, seps, bmin, bmax, 0xFFFF, div, nb, h)
        for reb in ("", "reb_"):
            if reb:
                ids, cnt, off = oracle.psh_rebalance(ids, cnt, off, seps, bs)
            cumsum, scat = oracle.cumsum_scatter_pad(coords, seps, nb, ids, cnt, off, pad_to, 0.0)
            k = f"h{h}_{reb}"
            assert np.array_equal(ids, g[k + "ids"]) and np.array_equal(cnt, g[k + "cnt"])
            assert np.array_equal(off, g[k + "off"]) and np.array_equal(cumsum, g[k + "cumsum"])
            assert np.array_equal(scat.view(np.uint16), g[k + "scat"])
            # what the fixture itself must satisfy, whoever wrote it
            assert g[k + "cnt"].sum(1).tolist() == [150, 106]
            rows = g[k + "scat"][:256]
            assert sorted(map(tuple, rows)) == sorted(map(tuple, g["coords"])), "scatter is not a permutation"
            assert not g[k + "scat"][256:].any()
        assert int(g[f"h{h}_reb_cnt"][:, 1:].max()) <= bs, "rebalance left a bucket other than 0 above the bucket size"


def test_pool_fixture(oracle):
    g = load("pool_151pts.npz")
    coords, seps, feat = g["coords"].view(np.float16), g["seps"], g["feat"]
    for S in (2, 3):
        sub_id, sub_off, unpool, red_coord, red_sep = oracle.subbuck_build(coords, seps, S, out_align=16)
        k = f"s{S}_"
        assert np.array_equal(sub_id, g[k + "sub_id"]) and np.array_equal(sub_off, g[k + "sub_off"])
        assert np.array_equal(unpool, g[k + "unpool"]) and np.array_equal(red_sep, g[k + "red_sep"])
        assert np.array_equal(red_coord.view(np.uint16), g[k + "red_coord"])
        for op in (0, 1, 2, 3):
            assert np.array_equal(oracle.reduce_feat(feat, unpool, op, r_aligned=red_coord.shape[0]), g[k + f"red_op{op}"])
        assert np.array_equal(oracle.additive_unpool(feat, g[k + "down"], unpool), g[k + "up"])
        # the fixture's own structure: every point appears in exactly one slot of the inverse map
        u = g[k + "unpool"].reshape(-1)
        assert sorted(u[u < 151].tolist()) == list(range(151))
        assert g[k + "red_sep"].tolist() == np.cumsum([-(-90 // S), -(-61 // S)]).tolist()


def test_attention_fixture(oracle):
    g = load("attn_2x128.npz")
    shape = (1, 512, 2, 16)
    Q, K, V = [_bf(g[n]).reshape(shape) for n in "QKV"]
    O, LSE = oracle.buck_swin_fwd(Q, K, V, g["scopes"], int(g["bucket_size"]))
    assert np.allclose(O.numpy(), g["O"], atol=1e-6) and np.allclose(LSE.numpy(), g["LSE"], atol=1e-6)
    Om, LSEm = oracle.buck_swin_fwd(Q, K, V, g["scopes"], int(g["bucket_size"]), kv_len=g["kv_len"])
    assert np.allclose(Om.numpy(), g["O_masked"], atol=1e-6) and np.allclose(LSEm.numpy(), g["LSE_masked"], atol=1e-6)
    # independent restatement for the second scope (buckets 2, 3 = rows 256..511): library SDPA
    q, k, v = [t[:, 256:].permute(0, 2, 1, 3).float() for t in (Q, K, V)]
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v).permute(0, 2, 1, 3)
    assert np.allclose(g["O"][:, 256:], want.numpy(), atol=2e-6)
    # masked rows of the fixture are zero: bucket 1 keeps 70 keys, bucket 2 keeps one
    assert not g["O_masked"][:, 128 + 70:256].any() and not g["O_masked"][:, 257:384].any()
    # row 256 (the one valid row of bucket 2) attends to itself and to the 128 rows of bucket 3
    keys = [256] + list(range(384, 512))
    q1 = Q[:, 256:257].permute(0, 2, 1, 3).float()
    k1, v1 = [t[:, keys].permute(0, 2, 1, 3).float() for t in (K, V)]
    want1 = torch.nn.functional.scaled_dot_product_attention(q1, k1, v1).permute(0, 2, 1, 3)
    assert np.allclose(g["O_masked"][:, 256:257], want1.numpy(), atol=2e-6)


def test_dense_fixture(oracle):
    g = load("dense_64x32.npz")
    x, ln_w, ln_b = _bf(g["x"]).float(), _bf(g["ln_w"]).float(), _bf(g["ln_b"]).float()
    ln = oracle.layernorm(x, ln_w, ln_b)
    assert np.allclose(ln.numpy(), g["ln"], atol=1e-6)
    h = oracle._r(ln)
    assert np.allclose(oracle.linear(h, _bf(g["w_qkv"]), _bf(g["b_qkv"])).numpy(), g["qkv"], atol=1e-5)
    act = oracle.swiglu(oracle._r(oracle.linear(h, _bf(g["w1"]), _bf(g["b1"]))))
    assert np.allclose(act.numpy(), g["act"], atol=1e-5)
    y = oracle.linear(oracle._r(act), _bf(g["w2"]), _bf(g["b2"])) + x
    assert np.allclose(y.numpy(), g["y"], atol=1e-5)
    # the fixture's LayerNorm rows have zero mean / unit variance once the affine part is undone
    z = (g["ln"] - ln_b.numpy()) / ln_w.numpy()
    assert np.abs(z.mean(1)).max() < 1e-4 and np.abs(z.var(1) - 1).max() < 1e-3
