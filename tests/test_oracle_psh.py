"""Pins for the PSH part of the CPU oracle (voxel quantiser, hashes, slot claim, scatter).

Each check is chosen so that a plausible slip in oracle/f3d_oracle.c (dropped term, wrong shift,
swapped axis, exclusive-vs-inclusive scan) fails at least one of them.  None re-types the oracle's
own formula: they use numpy's float16/float32 casts, bit loops, closed forms and the reference's
scoreboard invariant (tests/test_psh.py:117-129 of the reference).
"""
import numpy as np
import pytest


def test_half_to_float_all_patterns(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.f3d_or_half_to_float(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_rne(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(7)
    # random floats over the half range, plus exact ties, subnormals and overflow edges
    xs = np.concatenate([
        rng.normal(0, 100, 4000), rng.normal(0, 1e-5, 2000), rng.uniform(-70000, 70000, 2000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5,
                  1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2049.0, 2051.0, np.inf, -np.inf]),
    ]).astype(np.float32)
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.f3d_or_float_to_half(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_conversions_match_torch(oracle):
    import torch
    L = oracle.lib()
    rng = np.random.default_rng(8)
    xs = np.concatenate([rng.normal(0, 3, 5000), [1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 0.0, -0.0, 3.4e38]]).astype(np.float32)
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.uint16).numpy()
    got = np.array([L.f3d_or_float_to_bf16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.f32_to_bf16_bits(xs), want)
    back = np.array([L.f3d_or_bf16_to_float(int(b)) for b in want], dtype=np.float32)
    assert np.array_equal(back, torch.from_numpy(want).view(torch.bfloat16).float().numpy())


def test_vox_known_answers(oracle):
    L = oracle.lib()
    nv = 0xFFFF
    assert L.f3d_or_vox1(0.0, 0.0, 51.2, nv) == 0            # c == min -> 0
    assert L.f3d_or_vox1(51.2, 0.0, 51.2, nv) == nv - 1      # c == max -> clamp to num_vox-1
    assert L.f3d_or_vox1(25.6, 0.0, 51.2, nv) == 32767       # midpoint: floor(65535/2)
    assert L.f3d_or_vox1(-1.0, 0.0, 51.2, nv) == 0           # below the box clamps to 0
    assert L.f3d_or_vox1(99.0, 0.0, 51.2, nv) == nv - 1      # above the box clamps high
    assert L.f3d_or_vox1(3.0, 3.0, 3.0, nv) == nv - 1        # degenerate axis: 0/0 = NaN -> hi
    assert L.f3d_or_vox1(1.0, 0.0, 4.0, 16) == 4             # small grid by hand: 1*16/4


def test_vox_bruteforce_all_fp16(oracle):
    """every finite fp16 pattern inside a fixed bbox vs an independent numpy float32 evaluation"""
    bits = np.arange(65536, dtype=np.uint16)
    c = bits.view(np.float16)
    mn, mx = np.float16(-40.5), np.float16(51.19)
    keep = np.isfinite(c)
    c = c[keep]
    coords = np.stack([c, c, c], axis=1)
    got = oracle.vox_coord(coords, np.array([mn] * 3, np.float16), np.array([mx] * 3, np.float16))
    c32 = c.astype(np.float32)
    with np.errstate(all="ignore"):
        inv = np.float32(1.0) / (np.float32(mx) - np.float32(mn))
        q = ((c32 - np.float32(mn)) * np.float32(65535.0)) * inv
        q_div = ((c32 - np.float32(mn)) * np.float32(65535.0)) / (np.float32(mx) - np.float32(mn))
    # the reciprocal form may differ from true division only by landing on the other side of an
    # integer boundary, i.e. by one cell, and only rarely
    d = np.abs(np.clip(np.floor(q), 0, 65534) - np.clip(np.floor(q_div), 0, 65534))
    assert d.max() <= 1 and (d > 0).mean() < 0.01
    want = np.clip(np.floor(q), 0, 65534).astype(np.uint16)
    assert np.array_equal(got[:, 0], want)
    assert np.array_equal(got[:, 2], want)


def test_vox_division_mode_bruteforce_all_fp16(oracle):
    """mode 1 of the quantiser (IEEE division, hash_fns.cuh:23-33 as written): every finite fp16 pattern against the
    quotient computed in float64 and rounded once to float32 (for two float32 operands that is the correctly rounded
    float32 quotient: 53 >= 2 * 24 + 2 bits), in two boxes; known answers keep their values; mode 0 comes back"""
    bits = np.arange(65536, dtype=np.uint16)
    c = bits.view(np.float16)
    c = c[np.isfinite(c)]
    coords = np.stack([c, c, c], axis=1)
    try:
        oracle.set_quantiser(1)
        for mn, mx in ((np.float16(-40.5), np.float16(51.19)), (np.float16(-79.9), np.float16(80.0))):
            got = oracle.vox_coord(coords, np.array([mn] * 3, np.float16), np.array([mx] * 3, np.float16))
            num = ((c.astype(np.float32) - np.float32(mn)) * np.float32(65535.0)).astype(np.float64)
            den = np.float64(np.float32(mx) - np.float32(mn))
            with np.errstate(all="ignore"):
                q = (num / den).astype(np.float32)
            want = np.clip(np.floor(q), 0, 65534).astype(np.uint16)
            assert np.array_equal(got[:, 0], want) and np.array_equal(got[:, 1], want)
        L = oracle.lib()
        assert L.f3d_or_vox1(25.6, 0.0, 51.2, 0xFFFF) == 32767 and L.f3d_or_vox1(3.0, 3.0, 3.0, 0xFFFF) == 0xFFFE
        assert L.f3d_or_vox1(1.0, 0.0, 4.0, 16) == 4
        # a case on which the two modes differ: 19.546875 in the box [-40.5, 51.1875]: the rounded reciprocal
        # puts the quotient on the other side of an integer than the division does
        got1 = oracle.vox_coord(coords, np.array([-40.5] * 3, np.float16), np.array([51.19] * 3, np.float16))
        oracle.set_quantiser(0)
        got0 = oracle.vox_coord(coords, np.array([-40.5] * 3, np.float16), np.array([51.19] * 3, np.float16))
        assert 0 < (got0 != got1).mean() < 0.01
        assert np.abs(got0.astype(np.int32) - got1.astype(np.int32)).max() == 1
    finally:
        oracle.set_quantiser(0)
    with pytest.raises(ValueError):
        oracle.set_quantiser(2)


def test_morton_spread_bit_loop(oracle):
    L = oracle.lib()
    for k in range(16):
        assert L.f3d_or_space_out_bit_3d(1 << k) == 1 << (3 * k)
    rng = np.random.default_rng(3)
    for v in rng.integers(0, 65536, 200):
        want = 0
        for k in range(16):
            want |= ((int(v) >> k) & 1) << (3 * k)
        assert L.f3d_or_space_out_bit_3d(int(v)) == want


def test_zorder16_bit_positions(oracle):
    """bit i of the 16-bit z-order word is, in order, y10 z10 x11 y11 z11 ... x15 y15; z15 is dropped"""
    L = oracle.lib()
    names = []
    for pos in range(31, 47):           # morton bit positions kept by (>> 31) & 0xFFFF
        names.append(("xyz"[pos % 3], pos // 3))
    assert names[0] == ("y", 10) and names[1] == ("z", 10) and names[-1] == ("y", 15)
    for axis in "xyz":
        for k in range(16):
            v = {"x": 0, "y": 0, "z": 0}
            v[axis] = 1 << k
            want = 0
            if (axis, k) in names:
                want = 1 << names.index((axis, k))
            assert L.f3d_or_zorder16(v["x"], v["y"], v["z"]) == want, (axis, k)
    assert L.f3d_or_zorder16(0xFFFF, 0xFFFF, 0xFFFF) == 0xFFFF
    assert L.f3d_or_hash(0xFFFF, 0xFFFF, 0xFFFF, 1, 1024, 64) == 63
    assert L.f3d_or_hash(0, 0, 0x8000, 1, 1024, 64) == 0     # z15 alone does not move the bucket


def test_hash_c_vs_numpy_all_types(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(11)
    vox = rng.integers(0, 65535, (3000, 3)).astype(np.uint16)
    for nb in (32, 64, 128, 256, 512):
        div = -(-65535 // nb)
        for ht in (1, 2, 3, 4):
            want = oracle.hash_ids(vox, ht, div, nb)
            got = np.array([L.f3d_or_hash(int(a), int(b), int(c), ht, div, nb) for a, b, c in vox[:400]], np.uint16)
            assert np.array_equal(got, want[:400])
            assert want.max() < nb
    # xorsum closed form on hand-picked values
    assert L.f3d_or_hash(0x00FF, 0x0F0F, 0x3333, 2, 1024, 64) == (0x00FF ^ 0x0F0F ^ 0x3333) // 1024
    assert L.f3d_or_hash(0x00FF, 0x0F0F, 0x3333, 4, 1024, 64) == (0x00FF ^ 0x0F0F ^ 0x3333) % 64


def _cloud(rng, sizes):
    pts = rng.uniform(0, 51.2, (int(sum(sizes)), 3)).astype(np.float16)
    return pts, np.cumsum(sizes).astype(np.uint32)


@pytest.mark.parametrize("hash_type", [1, 2, 3, 4])
def test_claim_scoreboard_and_histogram(oracle, hash_type):
    rng = np.random.default_rng(100 + hash_type)
    coords, seps = _cloud(rng, [20000, 17001, 23456])
    nb, div, _ = oracle.psh_params(seps, 512)
    assert nb == 64      # int(20152.3 / 512) = 39 -> next power of two
    mn, mx = coords.min(0), coords.max(0)
    ids, cnt, off = oracle.psh_claim(coords, seps, mn, mx, 0xFFFF, div, nb, hash_type)
    # ids agree with the vectorised numpy hash of the C quantiser's voxels
    assert np.array_equal(ids, oracle.hash_ids(oracle.vox_coord(coords, mn, mx), hash_type, div, nb))
    start = 0
    for b, end in enumerate(seps):
        assert np.array_equal(cnt[b], np.bincount(ids[start:end], minlength=nb))
        start = int(end)
    assert cnt.sum() == coords.shape[0]
    rc, _ = oracle.scoreboard(ids, cnt, off, seps)
    assert rc == 0
    # the scoreboard must catch a duplicated slot, an out-of-range id and a wrong count
    off2 = off.copy()
    same = np.where(ids[:20000] == ids[5])[0]
    off2[same[0]] = off2[same[1]]
    assert oracle.scoreboard(ids, cnt, off2, seps)[0] == 2
    ids2 = ids.copy(); ids2[7] = nb
    assert oracle.scoreboard(ids2, cnt, off, seps)[0] == 1
    cnt2 = cnt.copy(); cnt2[1, 3] += 1
    assert oracle.scoreboard(ids, cnt2, off, seps)[0] in (2, 3)


def test_scatter_cumsum_multiset_and_positions(oracle):
    rng = np.random.default_rng(5)
    coords, seps = _cloud(rng, [17000, 16500])
    nb, div, _ = oracle.psh_params(seps, 512)
    mn, mx = coords.min(0), coords.max(0)
    ids, cnt, off = oracle.psh_claim(coords, seps, mn, mx, 0xFFFF, div, nb, 1)
    pad_to = -(-coords.shape[0] // 512) * 512
    cumsum, scat = oracle.cumsum_scatter_pad(coords, seps, nb, ids, cnt, off, pad_to, 0.0)
    assert np.array_equal(cumsum, np.cumsum(cnt, axis=1))
    assert not np.isnan(scat).any()
    assert (scat[coords.shape[0]:] == 0).all()
    # every point sits at cloud_start + exclusive_cumsum[id] + slot
    excl = np.cumsum(cnt, axis=1) - cnt
    start = 0
    for b, end in enumerate(seps):
        i = np.arange(start, end)
        dst = start + excl[b][ids[i]] + off[i]
        assert np.array_equal(scat[dst].view(np.uint16), coords[i].view(np.uint16))
        # stable order: inside one cloud the scattered rows are the points stably sorted by id
        order = np.argsort(ids[i], kind="stable")
        assert np.array_equal(scat[start:end].view(np.uint16), coords[i][order].view(np.uint16))
        start = int(end)


@pytest.mark.parametrize("rebalance", [False, True])
def test_scatter_index_is_the_scatter_permutation(oracle, rebalance):
    """Pins the permutation index (batch_psh_bucket.cuh:617-753) by what fixes it without restating its formula:
    it is a bijection on every cloud's row range, the input coordinates gathered by it are the scatter step's
    output bit for bit, without rebalance it is the stable argsort by bucket id, and features ride along."""
    rng = np.random.default_rng(11)
    coords, seps = _cloud(rng, [9000, 0, 7777, 8300])
    n = coords.shape[0]
    nb, div, _ = oracle.psh_params(seps, 256)
    mn, mx = coords.min(0), coords.max(0)
    ids, cnt, off = oracle.psh_claim(coords, seps, mn, mx, 0xFFFF, div, nb, 2)
    if rebalance:
        ids, cnt, off = oracle.psh_rebalance(ids, cnt, off, seps, 256)
    pad_to = -(-n // 1536) * 1536
    cumsum, scat = oracle.cumsum_scatter_pad(coords, seps, nb, ids, cnt, off, pad_to, 0.0)
    feat = rng.integers(0, 2 ** 16, (n, 5), dtype=np.uint16)
    idx, sfeat = oracle.scatter_feat_index(seps, nb, ids, off, cumsum, pad_to, feat)
    assert np.array_equal(idx, oracle.scatter_feat_index(seps, nb, ids, off, cumsum, pad_to))
    assert (idx[n:] == n + 3).all() and (sfeat[n:] == 0).all()
    start = 0
    for end in seps:
        end = int(end)
        assert np.array_equal(np.sort(idx[start:end]), np.arange(start, end, dtype=np.uint32))
        if not rebalance:
            order = np.argsort(ids[start:end], kind="stable")
            assert np.array_equal(idx[start:end], start + order)
        start = end
    assert np.array_equal(coords[idx[:n]].view(np.uint16), scat[:n].view(np.uint16))
    assert np.array_equal(feat[idx[:n]], sfeat[:n])


def test_helpers_closed_forms(oracle):
    for v in range(1, 3000):
        p = oracle.round_next_two_power(v)
        assert p >= v and p & (p - 1) == 0 and (p // 2 < v)
    assert oracle.psh_params([32768], 512) == (64, 1024, 32768)
    assert oracle.psh_params([65536, 131072], 512)[0] == 128
    assert oracle.psh_params(np.cumsum([120000] * 4), 512)[0] == 256
    assert oracle.psh_params(np.cumsum([250000] * 4), 512)[0] == 512
    n, sizes, sep = oracle.calc_red_sep_sizes([5, 12, 20], 3)
    assert n == 2 + 3 + 3 and list(sizes) == [2, 3, 3] and list(sep) == [2, 5, 8]
    s = oracle.gen_scopes(512 * 8, 512, 2, "swin")
    assert s.tolist() == [[0, 1], [2, 3], [4, 5], [6, 7]]
    assert oracle.gen_scopes(512 * 7, 512, 2, "swin").tolist() == [list(range(7))]
    assert oracle.gen_scopes(512 * 8, 512, 2, "stride").tolist() == [list(range(8))]   # 8 % 12 != 0
    assert oracle.gen_scopes(512 * 12, 512, 2, "stride").shape == (6, 2)


@pytest.mark.parametrize("case", ["lidar", "uniform_exact_capacity", "uniform_spare"])
def test_rebalance_invariants(oracle, case):
    """A4: the invariants the reference's own checks rest on (tests/test_psh.py:117-129) plus the
    properties that define a rebalance: conservation, dense unique slots, bounded occupancy wherever
    capacity exists, untouched buckets stay put, leftovers go to bucket 0 only."""
    import bench_workloads as synth
    bs = 512
    if case == "lidar":
        clouds = [synth.lidar_sweep(30000, 7 + i, oversample=2) for i in range(2)]
    elif case == "uniform_exact_capacity":
        clouds = [synth.uniform_cube(65536, 51.2, 3)]          # 128 buckets x 512 == N
    else:
        clouds = [synth.uniform_cube(60000, 51.2, 4), synth.uniform_cube(50000, 20.0, 5)]
    coords, seps = synth.batch_of(clouds)
    nb, div, _ = oracle.psh_params(seps, bs)
    ids0, cnt0, off0 = oracle.psh_claim(coords, seps, coords.min(0), coords.max(0), 0xFFFF, div, nb, 1)
    ids, cnt, off = oracle.psh_rebalance(ids0, cnt0, off0, seps, bs)
    assert oracle.scoreboard(ids, cnt, off, seps)[0] == 0
    assert ids.max() < nb
    start = 0
    for b, end in enumerate(seps):
        end = int(end)
        n = end - start
        assert cnt[b].sum() == n
        assert np.array_equal(cnt[b], np.bincount(ids[start:end], minlength=nb))
        over = np.maximum(cnt0[b][1:].astype(np.int64) - bs, 0).sum()
        free = np.maximum(bs - cnt0[b][1:].astype(np.int64), 0).sum()
        assert (cnt[b][1:] <= bs).all()                                   # buckets != 0 are bounded
        assert cnt[b][0] == cnt0[b][0] + max(0, over - free)              # leftovers land in bucket 0 only
        moved = ids[start:end] != ids0[start:end]
        assert moved.sum() == over
        # only points that overflowed move; everyone else keeps id and slot
        was_over = (off0[start:end] >= bs) & (ids0[start:end] != 0)
        assert np.array_equal(moved, was_over)
        assert np.array_equal(off[start:end][~moved], off0[start:end][~moved])
        # order-preserving transport: destinations are non-decreasing in (source bucket, slot) order
        src_order = np.lexsort((off0[start:end][moved], ids0[start:end][moved]))
        dst = ids[start:end][moved][src_order].astype(np.int64)
        dst[dst == 0] = nb                                                # recycle bucket comes last
        assert (np.diff(dst) >= 0).all()
        start = end


def test_one_multiply_division_of_16_bit_numbers_is_exact():
    """the hashing kernel divides the 16-bit hash by the bucket divisor with q = (x * (2^32 // d + 1)) >> 32
    (csrc/f3d_device.h:div16); exact for every 16-bit x and every divisor a bucket geometry can produce"""
    x = np.arange(65536, dtype=np.uint64)
    for d in list(range(2, 70)) + [127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049,
                                   4095, 4096, 21845, 32767, 32768, 65534, 65535]:
        magic = np.uint64((1 << 32) // d + 1)
        q = (x * magic) >> np.uint64(32)
        assert np.array_equal(q, x // np.uint64(d)), d
