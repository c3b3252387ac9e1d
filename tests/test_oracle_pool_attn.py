"""Pins for the pooling / unpooling / sub-bucket / attention parts of the CPU oracle.

reduce and unpool are checked against numpy / torch library reductions on the same bf16 inputs
(the formulas of the reference's tests/test_subbuck_reduce.py:131-147 and tests/test_unpooling.py:
127-134); the sub-bucket builder against the structural invariants of
tests/test_subbuck_reduce.py:486-631; attention against torch's scaled_dot_product_attention,
closed-form special cases and permutation invariance (tests/test_attn_fwd.py:185-190, 418-452).
"""
import math

import numpy as np
import pytest
import torch


def _bf16(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)


def _bits(t):
    return t.contiguous().view(torch.uint16).numpy()


@pytest.mark.parametrize("S,op", [(3, 0), (2, 1), (2, 2), (2, 3), (8, 0), (8, 3)])
def test_reduce_feat_vs_torch(oracle, S, op):
    rng = np.random.default_rng(40 + S + op)
    n, c = 1000, 24
    feat = _bf16(rng.normal(0, 1, (n, c)))
    r = -(-n // S)
    perm = rng.permutation(n)
    unpool = np.full((r, S), n + 3, dtype=np.uint32)
    unpool.reshape(-1)[:n] = perm                 # last row partially empty
    unpool[3, :] = n + 3                          # one fully empty row -> zeros
    got = oracle.reduce_feat(_bits(feat), unpool, op, r_aligned=r + 5)
    f32 = feat.float()
    want = torch.zeros(r + 5, c)
    for i in range(r):
        rows = [int(x) for x in unpool[i] if x < n]
        if not rows:
            continue
        g = f32[rows]
        want[i] = [g.mean(0), g.sum(0), g.amin(0), g.amax(0)][op]
    got_f = torch.from_numpy(oracle.bf16_bits_to_f32(got))
    # library mean may associate differently from the slot-order sum: one bf16 ulp of slack
    assert torch.allclose(got_f, want.to(torch.bfloat16).float(), atol=2 ** -6, rtol=2 ** -7)
    if op in (2, 3):
        assert torch.equal(got_f, want.to(torch.bfloat16).float())   # min / max are exact
    assert (got[r:] == 0).all() and (got[3] == 0).all()


def test_additive_unpool_vs_torch(oracle):
    rng = np.random.default_rng(9)
    n, c, S = 777, 40, 2
    r = -(-n // S)
    res = _bf16(rng.normal(0, 1, (n, c)))
    down = _bf16(rng.normal(0, 1, (r + 4, c)))
    unpool = np.full((r, S), n + 3, dtype=np.uint32)
    unpool.reshape(-1)[:n] = rng.permutation(n)
    up = oracle.additive_unpool(_bits(res), _bits(down), unpool)
    want = torch.zeros(n, c, dtype=torch.bfloat16)
    for i in range(r):
        for s in range(S):
            row = int(unpool[i, s])
            if row < n:
                want[row] = down[i] + res[row]       # bf16 + bf16 in torch rounds the fp32 sum once
    assert np.array_equal(up, _bits(want))


@pytest.mark.parametrize("S", [2, 3, 4, 8])
def test_subbuck_structure_invariants(oracle, S):
    rng = np.random.default_rng(S)
    sizes = [1300, 1024, 2051, 7]
    coords = rng.uniform(-30, 30, (sum(sizes), 3)).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    sub_id, sub_off, unpool, red_coord, red_sep = oracle.subbuck_build(coords, seps, S, out_align=16)
    n = coords.shape[0]
    start = rstart = 0
    for b, end in enumerate(seps):
        end, rend = int(end), int(red_sep[b])
        ids, offs = sub_id[start:end].astype(np.int64), sub_off[start:end].astype(np.int64)
        nred = rend - rstart
        assert nred == -(-(end - start) // S)
        assert len(np.unique(ids)) == nred and ids.min() == 0 and ids.max() == nred - 1
        assert offs.max() < S
        codes = ids * S + offs
        assert len(np.unique(codes)) == end - start          # (id, off) unique
        # slots inside a sub-bucket are packed from 0
        for sid in np.unique(ids)[:50]:
            o = np.sort(offs[ids == sid])
            assert np.array_equal(o, np.arange(len(o)))
        # unpool_ind is the inverse map
        assert np.array_equal(unpool[rstart + ids, offs], np.arange(start, end))
        # reduced coordinate = mean of the members
        c32 = coords.astype(np.float32)
        for sid in range(0, nred, max(1, nred // 40)):
            members = unpool[rstart + sid]
            members = members[members < n]
            assert np.abs(c32[members].mean(0) - red_coord[rstart + sid].astype(np.float32)).max() < 0.2
        start, rstart = end, rend
    assert (unpool[unpool >= n] == n + 3).all()
    assert (red_coord[rstart:].view(np.uint16) == 0).all()
    # determinism: same seed same answer, other seed other grouping
    again = oracle.subbuck_build(coords, seps, S, out_align=16)
    assert np.array_equal(again[2], unpool)
    other = oracle.subbuck_build(coords, seps, S, seed=1, out_align=16)
    assert not np.array_equal(other[2], unpool)


def test_subbuck_groups_are_spatially_local(oracle):
    """grouping by z-order cell must beat grouping by input order on mean intra-group spread"""
    rng = np.random.default_rng(77)
    coords = rng.uniform(0, 50, (4096, 3)).astype(np.float16)
    seps = np.array([4096], np.uint32)
    _, _, unpool, _, _ = oracle.subbuck_build(coords, seps, 8)
    c32 = coords.astype(np.float32)
    spread = np.mean([c32[g].std(0).mean() for g in unpool])
    naive = np.mean([c32[i:i + 8].std(0).mean() for i in range(0, 4096, 8)])
    assert spread < 0.7 * naive


def test_tile_quat_is_unit_and_in_range(oracle):
    import ctypes
    q = (ctypes.c_float * 4)()
    for t in range(20):
        oracle.lib().f3d_or_tile_quat(3407, 1, t, q)
        v = np.array(list(q), dtype=np.float64)
        assert abs(np.linalg.norm(v) - 1.0) < 1e-6 and (v > 0).all()
    u = np.array([oracle.lib().f3d_or_rng_u01(3407, 0, 0, i) for i in range(4000)])
    assert 0 <= u.min() and u.max() < 1 and abs(u.mean() - 0.5) < 0.03


# ------------------------------------------------------------------------------------------------

def _qkv(rng, B, L, H, D, scale=1.0):
    mk = lambda: _bf16(rng.normal(0, scale, (B, L, H, D)))
    return mk(), mk(), mk()


def test_attention_single_scope_equals_sdpa(oracle):
    rng = np.random.default_rng(2)
    B, L, H, D, bs = 2, 256, 3, 16, 64
    Q, K, V = _qkv(rng, B, L, H, D)
    scopes = np.arange(L // bs, dtype=np.uint32)[None, :]
    O, LSE = oracle.buck_swin_fwd(Q, K, V, scopes, bs)
    want = torch.nn.functional.scaled_dot_product_attention(
        Q.float().transpose(1, 2), K.float().transpose(1, 2), V.float().transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(O, want, atol=2e-5, rtol=1e-5)
    logits = torch.einsum("blhd,bmhd->bhlm", Q.float(), K.float()) / math.sqrt(D)
    assert torch.allclose(LSE, torch.logsumexp(logits, -1).permute(0, 2, 1), atol=1e-5)


def test_attention_block_diagonal_and_permutation_invariance(oracle):
    rng = np.random.default_rng(3)
    B, L, H, D, bs = 1, 512, 2, 32, 64
    Q, K, V = _qkv(rng, B, L, H, D)
    scopes = oracle.gen_scopes(L, bs, 2)
    O, LSE = oracle.buck_swin_fwd(Q, K, V, scopes, bs)
    # scope = contiguous 128-row block -> block-diagonal attention
    for s in range(L // 128):
        sl = slice(128 * s, 128 * (s + 1))
        want = torch.nn.functional.scaled_dot_product_attention(
            Q[:, sl].float().transpose(1, 2), K[:, sl].float().transpose(1, 2),
            V[:, sl].float().transpose(1, 2)).transpose(1, 2)
        assert torch.allclose(O[:, sl], want, atol=2e-5, rtol=1e-5)
    # bucket order inside a scope does not matter
    O2, LSE2 = oracle.buck_swin_fwd(Q, K, V, scopes[:, ::-1].copy(), bs)
    assert torch.allclose(O, O2, atol=1e-6) and torch.allclose(LSE, LSE2, atol=1e-6)


def test_attention_closed_forms_and_masks(oracle):
    rng = np.random.default_rng(4)
    B, L, H, D, bs = 1, 256, 2, 16, 128
    _, _, V = _qkv(rng, B, L, H, D)
    Z = torch.zeros_like(V)
    scopes = oracle.gen_scopes(L, bs, 1)
    O, LSE = oracle.buck_swin_fwd(Z, Z, V, scopes, bs)
    for s in range(2):
        sl = slice(bs * s, bs * (s + 1))
        assert torch.allclose(O[:, sl], V[:, sl].float().mean(1, keepdim=True).expand(-1, bs, -1, -1), atol=1e-6)
    assert torch.allclose(LSE, torch.full_like(LSE, math.log(bs)), atol=1e-6)
    # masks: kv_len == bucket size changes nothing; shorter lengths equal attention over the prefix
    Q, K, V = _qkv(rng, B, L, H, D)
    full = oracle.buck_swin_fwd(Q, K, V, scopes, bs)
    same = oracle.buck_swin_fwd(Q, K, V, scopes, bs, kv_len=np.array([bs, bs]))
    assert torch.equal(full[0], same[0]) and torch.equal(full[1], same[1])
    kl = np.array([100, 37])
    O, LSE = oracle.buck_swin_fwd(Q, K, V, scopes, bs, kv_len=kl)
    for s in range(2):
        sl = slice(bs * s, bs * s + int(kl[s]))
        want = torch.nn.functional.scaled_dot_product_attention(
            Q[:, sl].float().transpose(1, 2), K[:, sl].float().transpose(1, 2),
            V[:, sl].float().transpose(1, 2)).transpose(1, 2)
        assert torch.allclose(O[:, sl], want, atol=2e-5, rtol=1e-5)
        assert (O[:, bs * s + int(kl[s]):bs * (s + 1)] == 0).all()
        assert (LSE[:, bs * s + int(kl[s]):bs * (s + 1)] == 0).all()
    # rows outside every scope keep their initial content
    init = torch.full((B, L, H, D), 7.0)
    O, _ = oracle.buck_swin_fwd(Q, K, V, scopes[:1], bs, O_init=init)
    assert (O[:, bs:] == 7.0).all()
