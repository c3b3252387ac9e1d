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


# ---------------------------------------------------------------------------------------------
# backward of the feature reduce and of additive unpooling
# ---------------------------------------------------------------------------------------------

def _random_inverse_map(rng, n, S, holes):
    """an unpool_ind [R, S] in which every point appears once; `holes` extra empty slots are spread at random"""
    r = -(-(n + holes) // S)
    flat = np.full(r * S, n + 3, dtype=np.uint32)
    pos = rng.permutation(r * S)[:n]
    flat[pos] = rng.permutation(n).astype(np.uint32)
    return flat.reshape(r, S)


@pytest.mark.parametrize("S,op", [(2, 0), (3, 0), (8, 0), (4, 1), (2, 2), (8, 2), (3, 3), (8, 3)])
def test_reduce_feat_bwd_vs_torch_autograd(oracle, S, op):
    """gradient of gather + mean / sum / amin / amax (the forward formula of reference
    tests/test_subbuck_reduce.py:131-147) by torch autograd in fp32, on inputs without ties (for which
    amin / amax send the whole gradient to the single winner, as the reference kernel does)"""
    rng = np.random.default_rng(100 * S + op)
    n, C = 203, 12
    unpool = _random_inverse_map(rng, n, S, holes=17)
    # distinct bf16 values per column so that min / max have no ties
    x = torch.stack([torch.from_numpy(rng.permutation(n).astype(np.float32)) * 0.25 - 20 for _ in range(C)], 1)
    x = x.to(torch.bfloat16)
    assert all(len(set(x[:, c].tolist())) == n for c in range(C))
    g = torch.from_numpy(rng.normal(0, 1, (unpool.shape[0], C)).astype(np.float32)).to(torch.bfloat16)
    got = oracle.reduce_feat_bwd(_bits(g), _bits(x), unpool, op)
    # torch: masked gather, reduce, backward
    xf = x.float().requires_grad_(True)
    idx = torch.from_numpy(unpool.astype(np.int64))
    valid = idx < n
    gathered = xf[idx.clamp(max=n - 1)]                                  # [R, S, C]
    if op <= 1:
        red = (gathered * valid[..., None]).sum(1)
        if op == 0:
            red = red / valid.sum(1).clamp(min=1)[:, None]
    else:
        fill = float("inf") if op == 2 else float("-inf")
        masked = torch.where(valid[..., None], gathered, torch.full_like(gathered, fill))
        red = masked.amin(1) if op == 2 else masked.amax(1)
        red = torch.where(valid.any(1)[:, None], red, torch.zeros_like(red))
    red.backward(g.float())
    want = xf.grad.to(torch.bfloat16)
    assert np.array_equal(got, _bits(want))


def test_reduce_feat_bwd_first_winner_on_ties_and_untouched_rows(oracle):
    """ties go to the first slot that reaches the extreme (reference loop, strict comparison,
    batch_psh_subbuck_reduce_bwd.cuh:96-104); rows that no slot refers to keep the prefill"""
    x = _bits(torch.tensor([[1.0], [5.0], [5.0], [2.0], [7.0]], dtype=torch.bfloat16))
    unpool = np.array([[3, 1, 2, 0]], dtype=np.uint32)            # values 2, 5, 5, 1 ; row 4 is never referred to
    g = _bits(torch.tensor([[3.0]], dtype=torch.bfloat16))
    prefill = _bits(torch.full((5, 1), 9.0, dtype=torch.bfloat16))
    mx = oracle.reduce_feat_bwd(g, x, unpool, 3, grad_in_init=prefill)
    f = lambda b: oracle.bf16_bits_to_f32(b).reshape(-1).tolist()
    assert f(mx) == [0.0, 3.0, 0.0, 0.0, 9.0]                     # slot 1 (row 1) wins the tie against slot 2 (row 2)
    mn = oracle.reduce_feat_bwd(g, x, unpool, 2, grad_in_init=prefill)
    assert f(mn) == [3.0, 0.0, 0.0, 0.0, 9.0]
    mean = oracle.reduce_feat_bwd(g, x, np.array([[3, 1, 2, 77]], dtype=np.uint32), 0, grad_in_init=prefill)
    assert f(mean) == [9.0, 1.0, 1.0, 1.0, 9.0]                   # 3 valid slots share the gradient


@pytest.mark.parametrize("S,C", [(2, 16), (3, 5), (8, 8)])
def test_additive_unpool_bwd_vs_torch_autograd(oracle, S, C):
    """up[r] = down[i] + res[r] (reference tests/test_unpooling.py:127-134) differentiated by torch in fp32:
    grad_res is the output gradient on the pooled rows, grad_down the per-row sum rounded once to bf16"""
    rng = np.random.default_rng(S * 10 + C)
    n = 157
    unpool = _random_inverse_map(rng, n, S, holes=9)
    r = unpool.shape[0]
    g = torch.from_numpy(rng.normal(0, 1, (n, C)).astype(np.float32)).to(torch.bfloat16)
    grad_res, grad_down = oracle.additive_unpool_bwd(_bits(g), unpool, down_rows=r + 3)
    res = torch.zeros(n, C, requires_grad=True)
    down = torch.zeros(r + 3, C, requires_grad=True)
    idx = torch.from_numpy(unpool.astype(np.int64))
    rows = idx[idx < n]
    src = torch.arange(r)[:, None].expand(r, S)[idx < n]
    up = torch.zeros(n, C).index_add(0, rows, down[src]) + res      # every point appears exactly once
    up.backward(g.float())
    assert np.array_equal(grad_res, _bits(res.grad.to(torch.bfloat16)))
    assert np.array_equal(grad_down, _bits(down.grad.to(torch.bfloat16)))
    assert not grad_down[r:].any()


def test_attention_bwd_formulas_vs_autograd(oracle):
    """the explicit backward formulas against torch autograd through the oracle's forward (the reference's own
    tests differentiate an SDPA / FA2 oracle the same way, tests/test_attn_bwd.py)"""
    rng = np.random.default_rng(11)
    B, L, H, D, bs = 2, 512, 3, 16, 128
    Q, K, V = [t.float().requires_grad_(True) for t in _qkv(rng, B, L, H, D)]
    scopes = np.array([[1, 0], [3, 2]], dtype=np.uint32)
    dO = torch.from_numpy(rng.normal(0, 1, (B, L, H, D)).astype(np.float32))
    O, _ = oracle.buck_swin_fwd(Q, K, V, scopes, bs)
    O.backward(dO)
    dQ, dK, dV, Delta = oracle.buck_swin_bwd(Q.detach(), K.detach(), V.detach(), dO, scopes, bs)
    for got, want in ((dQ, Q.grad), (dK, K.grad), (dV, V.grad)):
        assert (got - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())
    assert (Delta - (dO * O.detach()).sum(-1)).abs().max().item() <= 1e-5
    # a scope table that leaves buckets out: their rows get zero gradients
    dQ2, dK2, dV2, _ = oracle.buck_swin_bwd(Q.detach(), K.detach(), V.detach(), dO, np.array([[1, 0]], dtype=np.uint32), bs)
    assert not dQ2[:, 256:].any() and not dK2[:, 256:].any() and not dV2[:, 256:].any()
    assert torch.equal(dQ2[:, :256], dQ[:, :256])


def test_attention_bwd_with_valid_lengths_vs_autograd(oracle):
    """the masked backward against autograd through the oracle's masked forward (whose masks the forward tests pin):
    a full bucket, a ragged one, a one-key bucket, and an empty bucket sharing a scope with a valid one"""
    rng = np.random.default_rng(12)
    B, L, H, D, bs = 1, 512, 2, 16, 128
    Q, K, V = [t.float().requires_grad_(True) for t in _qkv(rng, B, L, H, D)]
    scopes = np.array([[1, 0], [3, 2]], dtype=np.uint32)
    kv_len = np.array([128, 77, 1, 0])
    dO = torch.from_numpy(rng.normal(0, 1, (B, L, H, D)).astype(np.float32))
    O, _ = oracle.buck_swin_fwd(Q, K, V, scopes, bs, kv_len=kv_len)
    O.backward(dO)
    dQ, dK, dV, Delta = oracle.buck_swin_bwd(Q.detach(), K.detach(), V.detach(), dO, scopes, bs, kv_len=kv_len)
    for got, want in ((dQ, Q.grad), (dK, K.grad), (dV, V.grad)):
        assert torch.isfinite(want).all()
        assert (got - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item())
    assert (Delta - (dO * O.detach()).sum(-1)).abs().max().item() <= 1e-5
    for t in (dQ, dK, dV):
        assert not t[:, 128 + 77:256].any() and not t[:, 257:].any() and t[:, :128 + 77].any()
    assert torch.equal(dV[:, 256], dO[:, 256])      # the one-key bucket: P = 1
    # lengths equal to the bucket size change nothing
    same = oracle.buck_swin_bwd(Q.detach(), K.detach(), V.detach(), dO, scopes, bs, kv_len=np.full(4, bs))
    plain = oracle.buck_swin_bwd(Q.detach(), K.detach(), V.detach(), dO, scopes, bs)
    assert all(torch.equal(a, b) for a, b in zip(same, plain))


@pytest.mark.parametrize("act", [None, "gelu", "relu"])
def test_bn_act_vs_torch_batch_norm(oracle, act):
    """eval-mode BatchNorm1d (+ GELU / ReLU) of the oracle against torch.nn.functional.batch_norm(training=False) and the
    library activations on random statistics (the reference's pool_norm / unpool_norm callables,
    tests/test_psh_hourglass.py:103-106: BatchNorm1d(eps=1e-3) then GELU)"""
    g = torch.Generator().manual_seed(17)
    n, c = 513, 40
    x = (torch.randn(n, c, generator=g) * 2).to(torch.bfloat16).float()
    bn = {"weight": torch.rand(c, generator=g) + 0.5, "bias": torch.randn(c, generator=g) * 0.3,
          "mean": torch.randn(c, generator=g) * 0.5, "var": torch.rand(c, generator=g) * 2 + 0.1, "eps": 1e-3}
    got = oracle.bn_act(x, bn, act)
    want = torch.nn.functional.batch_norm(x, bn["mean"], bn["var"], bn["weight"], bn["bias"], False, 0.0, bn["eps"])
    # the library may associate (x - mean) * rstd * w + b differently: at most one bf16 step before the activation
    want_r = want.to(torch.bfloat16).float()
    pre = oracle.bn_act(x, bn, None)
    assert (pre - want).abs().max().item() <= 2 ** -8 * max(1.0, want.abs().max().item())
    assert (pre != want_r).float().mean().item() < 0.01
    if act == "gelu":
        want_a = torch.nn.functional.gelu(pre).to(torch.bfloat16).float()
    elif act == "relu":
        want_a = torch.relu(pre)
    else:
        want_a = pre
    assert torch.equal(got, want_a)
    # a module says the same: nn.BatchNorm1d in eval mode with those statistics
    m = torch.nn.BatchNorm1d(c, eps=1e-3).eval()
    with torch.no_grad():
        m.weight.copy_(bn["weight"]); m.bias.copy_(bn["bias"])
        m.running_mean.copy_(bn["mean"]); m.running_var.copy_(bn["var"])
        assert torch.allclose(m(x), want, atol=1e-6, rtol=1e-6)
    # a dropped shift, a forgotten eps or var used as std would all fail the comparison above; make sure of one
    wrong = (x - bn["mean"]) / torch.sqrt(bn["var"]) * bn["weight"] + bn["bias"]
    assert (wrong - want).abs().max().item() > 2 ** -8 * max(1.0, want.abs().max().item())


def test_norm_act_layernorm_vs_torch(oracle):
    g = torch.Generator().manual_seed(18)
    x = torch.randn(100, 64, generator=g).to(torch.bfloat16).float()
    p = {"weight": torch.rand(64, generator=g) + 0.5, "bias": torch.randn(64, generator=g) * 0.1, "eps": 1e-5}
    want = torch.nn.functional.layer_norm(x, (64,), p["weight"], p["bias"], 1e-5).to(torch.bfloat16).float()
    assert torch.equal(oracle.norm_act(x, p, None), want)
    assert torch.equal(oracle.norm_act(x, p, "gelu"), torch.nn.functional.gelu(want).to(torch.bfloat16).float())
    assert torch.equal(oracle.norm_act(x, None, None), x)


def test_swiglu_half_order_closed_forms(oracle):
    """The gate of te.LayerNormMLP(activation="swiglu") as the reference calls it (layers/elem_wise.py:22-26):
    the activation acts on the FIRST half of the fc1 output and the second half multiplies it.  Closed
    forms that a swapped-halves restatement fails: a unit multiplier leaves silu of the first half, a zero
    first half gives zero whatever the multiplier (silu(0) = 0, while silu(g)*0 would too, so the converse
    case is checked as well: a zero second half gives zero), silu of the second half never appears, and
    swapping the halves changes the result."""
    g = torch.Generator().manual_seed(5)
    a = torch.randn(37, 48, generator=g) * 3
    m = torch.randn(37, 48, generator=g) * 3
    silu = a / (1 + torch.exp(-a))                       # written out, not the library call the oracle uses
    assert torch.allclose(oracle.swiglu(torch.cat([a, torch.ones_like(a)], -1)), silu, atol=1e-6, rtol=1e-6)
    assert (oracle.swiglu(torch.cat([torch.zeros_like(m), m], -1)) == 0).all()
    assert (oracle.swiglu(torch.cat([a, torch.zeros_like(a)], -1)) == 0).all()
    # first half = 1 gives silu(1) * m = 0.731058... * m, not silu(m)
    got = oracle.swiglu(torch.cat([torch.ones_like(m), m], -1))
    assert torch.allclose(got, m * (1 / (1 + math.exp(-1.0))), atol=1e-6, rtol=1e-6)
    both = oracle.swiglu(torch.cat([a, m], -1))
    assert torch.allclose(both, silu * m, atol=1e-5, rtol=1e-5)
    assert not torch.allclose(both, oracle.swiglu(torch.cat([m, a], -1)), atol=1e-3)
    # bf16 input is computed in fp32 and the output has half the width
    hb = torch.cat([a, m], -1).to(torch.bfloat16)
    out = oracle.swiglu(hb)
    assert out.dtype == torch.float32 and out.shape == (37, 48)
