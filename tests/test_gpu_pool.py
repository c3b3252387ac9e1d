"""GPU parity of sub-bucket pooling and additive unpooling (rows A6-A8) against the CPU oracle,
through the C ABI.  The builder, the reduce and the unpool are all bit-exact: the oracle sums in
slot order in fp32 and rounds to bf16 / fp16 once, exactly what the kernels do.  The tolerance the
task states (max-abs <= 2e-2 bf16, <= 1e-4 fp32 accumulate) is therefore met with zero error."""
import numpy as np
import pytest
import torch

from tests.gpu_util import (DEV, bf16_bits, n_bf16_bits, n_f16, n_u16, n_u32, t_bf16_bits, t_f16, t_u32)

pytestmark = pytest.mark.gpu


def _pool(coords, seps, feat_bits, S, op, out_align, oracle):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import subbuck
    c, s, f = t_f16(coords), t_u32(seps), t_bf16_bits(feat_bits)
    sb = subbuck.SubbuckBuffers.create_subbuck_buff(c, f, s, S, out_alignment=out_align)
    max_n = int(np.diff(np.concatenate([[0], seps.astype(np.int64)])).max())
    pshattn.batch_subbuck_reduce(c, f, s, max_n, S, 0xFFFF, sb.bbox_min, sb.bbox_max, sb.subbuck_id, sb.subbuck_off,
                                 sb.reduced_sep, sb.reduced_coord, sb.reduced_feat, sb.unpool_ind, 1, op)
    torch.cuda.synchronize()
    return sb


@pytest.mark.parametrize("S,op,sizes,C", [
    (2, 0, [1300, 1024, 2051, 7], 256),
    (3, 0, [1300, 1400, 1023], 256),       # S does not divide 1024: 1023-point tiles
    (4, 3, [5000, 1], 64),
    (8, 2, [4096], 128),
    (16, 0, [3000, 1029], 64),             # the widest group that is summed through row shifts
    (32, 0, [2100, 33], 64),               # groups of two lane rows
    (2, 1, [3000, 2999], 40),              # 40 channels: 5 chunks per row
    (2, 0, [2000], 20),                    # channel count not a multiple of 8: scalar path
])
def test_builder_and_reduce_bit_exact(oracle, S, op, sizes, C):
    rng = np.random.default_rng(S * 100 + op)
    coords = rng.uniform(-30, 30, (sum(sizes), 3)).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    feat = bf16_bits(rng.normal(0, 1, (sum(sizes), C)))
    sb = _pool(coords, seps, feat, S, op, 16, oracle)
    sub_id, sub_off, unpool, red_coord, red_sep = oracle.subbuck_build(coords, seps, S, out_align=16)
    assert np.array_equal(n_u32(sb.unpool_ind), unpool), "inverse map differs"
    assert np.array_equal(n_u32(sb.subbuck_id), sub_id)
    assert np.array_equal(n_u16(sb.subbuck_off), sub_off)
    assert np.array_equal(n_f16(sb.reduced_coord).view(np.uint16), red_coord.view(np.uint16))
    want = oracle.reduce_feat(feat, unpool, op, r_aligned=sb.reduced_feat.shape[0])
    assert np.array_equal(n_bf16_bits(sb.reduced_feat), want), "reduced features differ"


def test_builder_long_runs_of_one_cell_bit_exact(oracle):
    """Clouds whose points share few distinct positions (one position only; three; a 2000-point cloud of 40 positions):
    whole tiles fall into one or a few cells of the counting sort, so the order inside a cell's run (input order) is
    what decides every output."""
    rng = np.random.default_rng(77)
    same = np.tile(np.array([[1.5, -2.25, 0.75]]), (1500, 1))
    three = np.array([[0.0, 0.0, 0.0], [10.0, -3.0, 2.0], [-7.0, 4.0, 1.0]])[rng.integers(0, 3, 1100)]
    forty = rng.uniform(-20, 20, (40, 3))[rng.integers(0, 40, 2000)]
    coords = np.concatenate([same, three, forty]).astype(np.float16)
    seps = np.cumsum([1500, 1100, 2000]).astype(np.uint32)
    feat = bf16_bits(rng.normal(0, 1, (coords.shape[0], 16)))
    for S in (2, 8):
        sb = _pool(coords, seps, feat, S, 0, 1, oracle)
        sub_id, sub_off, unpool, red_coord, _ = oracle.subbuck_build(coords, seps, S)
        assert np.array_equal(n_u32(sb.unpool_ind), unpool), "inverse map differs"
        assert np.array_equal(n_u32(sb.subbuck_id), sub_id) and np.array_equal(n_u16(sb.subbuck_off), sub_off)
        assert np.array_equal(n_f16(sb.reduced_coord).view(np.uint16), red_coord.view(np.uint16))
        # one position only: the cloud's rows come out in input order
        assert np.array_equal(unpool[:1500 // S].reshape(-1), np.arange(1500 // S * S))


def test_c3_pool_unpool_full_size(oracle):
    """BASELINE config 3: 262,144 points x 128 channels, S=8 (2x2x2), mean and max, then unpool"""
    import bench_workloads as synth
    from flash3dtransformer_amd.lib import pshattn
    n, C, S = 262144, 128, 8
    coords, seps = synth.batch_of([synth.uniform_cube(n // 4, 51.2, 1003 + i) for i in range(4)])
    rng = np.random.default_rng(1003)
    feat = bf16_bits(rng.normal(0, 1, (n, C)).astype(np.float32))
    res = bf16_bits(rng.normal(0, 1, (n, C)).astype(np.float32))
    _, _, unpool, red_coord, _ = oracle.subbuck_build(coords, seps, S)
    assert unpool.shape == (n // 8, 8)
    for op in (0, 3):
        sb = _pool(coords, seps, feat, S, op, 1, oracle)
        assert np.array_equal(n_u32(sb.unpool_ind), unpool)
        want = oracle.reduce_feat(feat, unpool, op)
        got = n_bf16_bits(sb.reduced_feat)
        assert np.array_equal(got, want)
        # stated tolerance, for the record: max-abs error of the bf16 output vs an fp64 reduction
        f64 = oracle.bf16_bits_to_f32(feat).astype(np.float64)[unpool]
        ref = f64.mean(1) if op == 0 else f64.max(1)
        assert np.abs(oracle.bf16_bits_to_f32(got) - ref).max() <= 2e-2
    up = torch.empty(n, C, dtype=torch.bfloat16, device=DEV)
    pshattn.additive_unpool_fwd(t_bf16_bits(res), sb.reduced_feat, up, sb.unpool_ind, S)
    torch.cuda.synchronize()
    want_up = oracle.additive_unpool(res, n_bf16_bits(sb.reduced_feat), unpool)
    assert np.array_equal(n_bf16_bits(up), want_up)


@pytest.mark.parametrize("S,C", [(2, 64), (3, 24), (2, 12)])
def test_unpool_bit_exact_with_empty_slots(oracle, S, C):
    """expected[r] = down[i] + res[r] (reference tests/test_unpooling.py:127-134); rows that no slot
    references keep the caller's prefill"""
    rng = np.random.default_rng(S + C)
    n = 1501
    r = -(-n // S)
    unpool = np.full((r, S), n + 3, dtype=np.uint32)
    keep = rng.permutation(n)[: n - 40]                 # 40 rows are referenced by no slot
    unpool.reshape(-1)[: keep.size] = keep
    res, down = bf16_bits(rng.normal(0, 1, (n, C))), bf16_bits(rng.normal(0, 1, (r + 7, C)))
    from flash3dtransformer_amd.lib import pshattn
    up = torch.full((n, C), 5.0, dtype=torch.bfloat16, device=DEV)
    pshattn.additive_unpool_fwd(t_bf16_bits(res), t_bf16_bits(down), up, t_u32(unpool), S)
    torch.cuda.synchronize()
    want = oracle.additive_unpool(res, down, unpool, up_init=bf16_bits(np.full((n, C), 5.0)))
    assert np.array_equal(n_bf16_bits(up), want)


def test_reference_structure_invariants_on_gpu_output():
    """the reference's sub-bucket checks (tests/test_subbuck_reduce.py:486-631) on the kernel output"""
    rng = np.random.default_rng(12)
    sizes = [1350] * 8
    S = 2
    coords = rng.normal(0, 15, (sum(sizes), 3)).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    feat = bf16_bits(rng.normal(0, 1, (sum(sizes), 32)))
    sb = _pool(coords, seps, feat, S, 0, 1, None)
    ids, offs = n_u32(sb.subbuck_id).astype(np.int64), n_u16(sb.subbuck_off).astype(np.int64)
    unpool, red_sep = n_u32(sb.unpool_ind), n_u32(sb.reduced_sep)
    red_coord = n_f16(sb.reduced_coord).astype(np.float32)
    c32 = coords.astype(np.float32)
    start = rstart = 0
    for b, end in enumerate(seps):
        end, rend = int(end), int(red_sep[b])
        i, o = ids[start:end], offs[start:end]
        assert len(np.unique(i)) == rend - rstart and i.min() == 0 and i.max() == rend - rstart - 1
        assert o.max() < S and len(np.unique(i * S + o)) == end - start
        assert np.array_equal(unpool[rstart + i, o], np.arange(start, end))
        for sid in range(0, rend - rstart, 37):
            mem = unpool[rstart + sid]
            mem = mem[mem < coords.shape[0]]
            assert np.abs(c32[mem].mean(0) - red_coord[rstart + sid]).max() < 0.2
        start, rstart = end, rend


def test_pool_argument_errors():
    from flash3dtransformer_amd.lib import pshattn
    c = torch.zeros(10, 3, dtype=torch.float16, device=DEV)
    f = torch.zeros(10, 8, dtype=torch.bfloat16, device=DEV)
    s = torch.tensor([10], dtype=torch.int32, device=DEV).view(torch.uint32)
    from flash3dtransformer_amd.psh import subbuck
    sb = subbuck.SubbuckBuffers.create_subbuck_buff(c, f, s, 2)
    args = lambda **k: dict(dict(coord=c, feat=f, red_feat=sb.reduced_feat, unpool=sb.unpool_ind, S=2, op=0), **k)

    def call(a):
        pshattn.batch_subbuck_reduce(a["coord"], a["feat"], s, 10, a["S"], 0xFFFF, sb.bbox_min, sb.bbox_max,
                                     sb.subbuck_id, sb.subbuck_off, sb.reduced_sep, sb.reduced_coord, a["red_feat"],
                                     a["unpool"], 1, a["op"])
    with pytest.raises(RuntimeError, match="Unsupported reduction"):
        call(args(op=4))
    with pytest.raises(RuntimeError, match="subbucket_size"):
        call(args(S=3))
    with pytest.raises(RuntimeError, match="feature dim"):
        call(args(red_feat=torch.zeros(5, 16, dtype=torch.bfloat16, device=DEV)))
    with pytest.raises(RuntimeError, match="dtype"):
        call(args(feat=f.float()))
    with pytest.raises(RuntimeError, match="not contiguous"):
        call(args(feat=torch.zeros(10, 16, dtype=torch.bfloat16, device=DEV)[:, ::2]))


# ---------------------------------------------------------------------------------------------
# backward ops (reference: additive_unpool_bwd, batch_subbuck_reduce_backward)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("S,op,n,C", [
    (2, 0, 5000, 64), (3, 0, 4097, 24), (8, 0, 30000, 128), (4, 1, 1000, 40),
    (2, 2, 3001, 16), (8, 3, 20000, 32), (3, 3, 999, 12),       # 12 channels: scalar path
])
def test_reduce_backward_bit_exact(oracle, S, op, n, C):
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(S * 1000 + op * 10 + C)
    coords = rng.uniform(-30, 30, (n, 3)).astype(np.float16)
    seps = np.array([n // 3, n], dtype=np.uint32)
    _, _, unpool, _, _ = oracle.subbuck_build(coords, seps, S, out_align=16)
    r_al = -(-unpool.shape[0] // 16) * 16
    x = bf16_bits(np.round(rng.normal(0, 1, (n, C)) * 4) / 4)           # coarse values: plenty of ties for min / max
    g = bf16_bits(rng.normal(0, 1, (r_al, C)))
    grad_in = torch.full((n, C), 7.0, dtype=torch.bfloat16, device=DEV)
    pshattn.batch_subbuck_reduce_backward(t_bf16_bits(g), t_bf16_bits(x), t_u32(unpool), grad_in, S, op)
    torch.cuda.synchronize()
    want = oracle.reduce_feat_bwd(g, x, unpool, op, grad_in_init=bf16_bits(np.full((n, C), 7.0)))
    assert np.array_equal(n_bf16_bits(grad_in), want)


@pytest.mark.parametrize("S,n,C", [(2, 6000, 64), (3, 4099, 24), (8, 40000, 128), (2, 777, 12)])
def test_unpool_backward_bit_exact(oracle, S, n, C):
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(S + n + C)
    r = -(-n // S) + 5
    unpool = np.full((r, S), n + 3, dtype=np.uint32)
    keep = rng.permutation(n)[: n - 30]                    # 30 rows are referred to by no slot
    unpool.reshape(-1)[rng.permutation(r * S)[: keep.size]] = keep
    g = bf16_bits(rng.normal(0, 1, (n, C)))
    grad_res = torch.full((n, C), 3.0, dtype=torch.bfloat16, device=DEV)
    grad_down = torch.full((r + 11, C), 5.0, dtype=torch.bfloat16, device=DEV)
    pshattn.additive_unpool_bwd(grad_res, grad_down, t_bf16_bits(g), t_u32(unpool), S)
    torch.cuda.synchronize()
    want_res, want_down = oracle.additive_unpool_bwd(g, unpool, grad_res_init=bf16_bits(np.full((n, C), 3.0)))
    assert np.array_equal(n_bf16_bits(grad_res), want_res)
    got_down = n_bf16_bits(grad_down)
    assert np.array_equal(got_down[:r], want_down)
    assert np.array_equal(got_down[r:], bf16_bits(np.full((11, C), 5.0)))      # rows past the map are not written


def test_pool_unpool_layers_backpropagate(oracle):
    """gradients flow through InbucketPoolingLayer and AdditiveUnpoolLayer (reference autograd functions
    layers/pooling.py:18-116, layers/unpool.py:18-77) and equal the oracle's composition"""
    from flash3dtransformer_amd.layers.pooling import InbucketPoolingLayer
    from flash3dtransformer_amd.layers.unpool import AdditiveUnpoolLayer
    rng = np.random.default_rng(77)
    n, C, S = 3000, 32, 2
    coords = rng.uniform(-20, 20, (n, 3)).astype(np.float16)
    seps = np.array([1700, n], dtype=np.uint32)
    feat = torch.from_numpy(rng.normal(0, 1, (n, C)).astype(np.float32)).to(torch.bfloat16).to(DEV).requires_grad_(True)
    res = torch.from_numpy(rng.normal(0, 1, (n, C)).astype(np.float32)).to(torch.bfloat16).to(DEV).requires_grad_(True)
    pool, unpool_layer = InbucketPoolingLayer("mean", out_alignment=16, subbuck_size=S), AdditiveUnpoolLayer(S)
    red, sb = pool(t_f16(coords), feat, t_u32(seps))
    up = unpool_layer(res, red, sb)
    w = torch.from_numpy(rng.normal(0, 1, (n, C)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    (up.float() * w.float()).sum().backward()
    torch.cuda.synchronize()
    # oracle: d up = w ; unpool bwd -> (grad_res, grad_down) ; reduce bwd(mean) of grad_down -> grad_feat
    unpool = n_u32(sb.unpool_ind)
    g_res, g_down = oracle.additive_unpool_bwd(n_bf16_bits(w), unpool, down_rows=red.shape[0])
    g_feat = oracle.reduce_feat_bwd(g_down, n_bf16_bits(feat.detach()), unpool, 0)
    assert np.array_equal(n_bf16_bits(res.grad), g_res)
    assert np.array_equal(n_bf16_bits(feat.grad), g_feat)


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _norm_reference(x_bits, kind, params, act):
    """fp64 restatement of the two layers: LayerNorm over the channels, or act(bf16(x * scale + shift))"""
    x = _bf16_to_f32(x_bits).astype(np.float64)
    if kind == "layer":
        g, b, eps = params
        mu = x.mean(1, keepdims=True)
        var = ((x - mu) ** 2).mean(1, keepdims=True)
        return (x - mu) / np.sqrt(var + eps) * g + b
    scale, shift = params
    y = x * scale + shift
    y = _bf16_to_f32(bf16_bits(y.astype(np.float32))).astype(np.float64)     # the norm's output is a bf16 tensor
    if act == "gelu":
        from math import erf
        y = 0.5 * y * (1.0 + np.vectorize(erf)(y / np.sqrt(2.0)))
    elif act == "relu":
        y = np.maximum(y, 0.0)
    elif act == "silu":
        y = y / (1.0 + np.exp(-y))
    return y


def _norm_case(kind, C, rng):
    """(descriptor for pshattn, parameters for _norm_reference)"""
    if kind == "layer":
        g = _bf16_to_f32(bf16_bits(rng.uniform(0.5, 1.5, C).astype(np.float32)))
        b = _bf16_to_f32(bf16_bits(rng.normal(0, 0.3, C).astype(np.float32)))
        desc = ("layer", t_bf16_bits(bf16_bits(g)), t_bf16_bits(bf16_bits(b)), 1e-5)
        return desc, (g.astype(np.float64), b.astype(np.float64), 1e-5)
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    shift = rng.normal(0, 0.3, C).astype(np.float32)
    desc = ("affine", torch.from_numpy(scale).to(DEV), torch.from_numpy(shift).to(DEV))
    return desc, (scale.astype(np.float64), shift.astype(np.float64))


@pytest.mark.parametrize("S,op,sizes,C,kind,act", [
    (2, 0, [1300, 1024, 2051, 7], 32, "layer", None),
    (2, 0, [3000, 2999], 64, "layer", None),
    (8, 3, [4096, 100], 128, "layer", None),
    (2, 0, [2500], 256, "layer", None),
    (4, 0, [1500, 3], 512, "layer", None),
    (2, 0, [1300, 1024], 64, "affine", "gelu"),
    (2, 1, [2000, 7], 40, "affine", None),          # 40 channels: 5 lanes per row
    (8, 2, [4100], 256, "affine", "relu"),
    (2, 0, [999], 32, "affine", "silu"),
])
def test_reduce_with_fused_norm(oracle, S, op, sizes, C, kind, act):
    """subbuck_build + reduce_feat_norm against the oracle's reduce followed by the norm in fp64 (a bf16 rounding of
    slack), and against the library's own two kernels (reduce, then LayerNorm / affine + activation): at most one bf16
    step apart"""
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import subbuck
    rng = np.random.default_rng(S * 100 + op + C)
    coords = rng.uniform(-30, 30, (sum(sizes), 3)).astype(np.float16)
    seps = np.cumsum(sizes).astype(np.uint32)
    feat = bf16_bits(rng.normal(0.3, 1.0, (sum(sizes), C)))
    desc, ref_params = _norm_case(kind, C, rng)
    plain = _pool(coords, seps, feat, S, op, 16, oracle)          # builder + plain reduce
    c, s, f = t_f16(coords), t_u32(seps), t_bf16_bits(feat)
    sb = subbuck.SubbuckBuffers.create_subbuck_buff(c, f, s, S, out_alignment=16)
    max_n = int(np.diff(np.concatenate([[0], seps.astype(np.int64)])).max())
    pshattn.subbuck_build(c, s, max_n, S, 0xFFFF, sb.subbuck_id, sb.subbuck_off, sb.reduced_sep, sb.reduced_coord, sb.unpool_ind)
    pshattn.reduce_feat_norm(f, coords.shape[0], sb.unpool_ind, sb.reduced_feat, S, op, desc, act)
    torch.cuda.synchronize()
    assert np.array_equal(n_u32(sb.unpool_ind), n_u32(plain.unpool_ind))
    assert np.array_equal(n_f16(sb.reduced_coord).view(np.uint16), n_f16(plain.reduced_coord).view(np.uint16))
    got = _bf16_to_f32(n_bf16_bits(sb.reduced_feat)).astype(np.float64)
    want = _norm_reference(n_bf16_bits(plain.reduced_feat), kind, ref_params, act)       # alignment rows included
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-6), np.abs(got - want).max()
    # the two-kernel path of the library
    two = torch.empty_like(plain.reduced_feat)
    if kind == "layer":
        pshattn.layernorm_bf16(plain.reduced_feat, desc[1], desc[2], two, 1e-5)
    else:
        pshattn.affine_act_bf16(plain.reduced_feat, desc[1], desc[2], two, act)
    torch.cuda.synchronize()
    two = _bf16_to_f32(n_bf16_bits(two)).astype(np.float64)
    assert np.all(np.abs(got - two) <= 2.0 ** -7 * np.abs(two) + 1e-6), np.abs(got - two).max()


@pytest.mark.parametrize("S,C,kind,act", [(2, 64, "layer", None), (2, 32, "layer", None), (8, 256, "layer", None),
                                          (3, 128, "layer", None), (2, 64, "affine", "gelu"), (3, 24, "affine", None),
                                          (2, 512, "affine", "relu")])
def test_unpool_with_fused_norm(oracle, S, C, kind, act):
    """up[r] = norm_down(down[i]) + norm_res(res[r]) for r = unpool_ind[i, s]; rows that no slot references keep the
    caller's prefill"""
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(S + C + len(kind))
    n = 1501
    r = -(-n // S)
    unpool = np.full((r, S), n + 3, dtype=np.uint32)
    keep = rng.permutation(n)[: n - 20]                        # 20 rows are referred to by no slot
    unpool.reshape(-1)[: keep.size] = keep
    res, down = bf16_bits(rng.normal(0.2, 1, (n, C))), bf16_bits(rng.normal(-0.1, 1, (r + 2, C)))
    dr, pr = _norm_case(kind, C, rng)
    dd, pd = _norm_case(kind, C, rng)
    up = torch.full((n, C), 7.0, dtype=torch.bfloat16, device=DEV)
    pshattn.additive_unpool_norm_fwd(t_bf16_bits(res), t_bf16_bits(down), up, t_u32(unpool), S, dr, dd, act)
    torch.cuda.synchronize()
    got = _bf16_to_f32(n_bf16_bits(up)).astype(np.float64)
    nres = _bf16_to_f32(bf16_bits(_norm_reference(res, kind, pr, act).astype(np.float32))).astype(np.float64)
    ndown = _bf16_to_f32(bf16_bits(_norm_reference(down, kind, pd, act).astype(np.float32))).astype(np.float64)
    want = np.full((n, C), 7.0)
    for i in range(r):
        for s in range(S):
            t = unpool[i, s]
            if t < n:
                want[t] = nres[t] + ndown[i]
    # each operand may be one bf16 step off its fp64 value, and the sum is rounded once more
    tol = 2.0 ** -7 * (np.abs(nres) + np.abs(ndown[0:1]).max() + np.abs(want)) + 1e-6
    assert np.all(np.abs(got - want) <= tol), np.abs(got - want).max()
    untouched = np.setdiff1d(np.arange(n), keep)
    assert np.all(got[untouched] == 7.0)


def test_fused_norm_argument_errors():
    from flash3dtransformer_amd.lib import pshattn
    C = 24          # LayerNorm over 3 lanes per row is not covered
    feat = torch.zeros(64, C, dtype=torch.bfloat16, device=DEV)
    ind = torch.zeros(32, 2, dtype=torch.int32, device=DEV).view(torch.uint32)
    out = torch.zeros(32, C, dtype=torch.bfloat16, device=DEV)
    g = torch.ones(C, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="No fused normalisation"):
        pshattn.reduce_feat_norm(feat, 64, ind, out, 2, 0, ("layer", g, None, 1e-5))
    with pytest.raises(RuntimeError, match="unsupported activation"):
        pshattn.reduce_feat_norm(torch.zeros(64, 32, dtype=torch.bfloat16, device=DEV), 64, ind,
                                 torch.zeros(32, 32, dtype=torch.bfloat16, device=DEV), 2, 0,
                                 ("layer", torch.ones(32, dtype=torch.bfloat16, device=DEV), None, 1e-5), "gelu")
