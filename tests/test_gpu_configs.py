"""The two model-level workloads at their stated shapes.

encoder stage: 4 synthetic LiDAR sweeps x 120,000 points, C = 256, 8 heads x 32, gated MLP 256 -> 1024 -> 256, bucket
512, hash 2: PSH3DCoordEmbedding + XFMR on the GPU against the oracle's restatement of the same op sequence, full size
(the benchmark's own step).

hourglass: 5 levels 32 / 64 / 128 / 256 / 512, 32-wide heads, bucket 512: against the oracle pipeline at a size the CPU
covers (4 x 20,000 points), and at full size (4 x 250,000 points) through properties that do not depend on size.

The reference's own model-level test asserts nothing about numbers (tests/test_psh_hourglass.py:159-163 of the
reference: a forward and a backward that must not raise); integer structures are bit-exact in the per-op tests, so what
is left here is the accumulation of bf16 roundings over the layers, held inside the bands below."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _state_dict_cpu(*modules_with_prefix):
    sd = {}
    for prefix, m in modules_with_prefix:
        for k, v in m.state_dict().items():
            sd[prefix + k] = v.detach().float().cpu().to(torch.bfloat16).float() if "running_" not in k \
                else v.detach().float().cpu()
    return sd


def _bands(got, want, mean_tol, bulk_tol, max_tol):
    """mean error <= mean_tol * scale, 99 % of the entries within bulk_tol * scale, largest error <= max_tol * max|ref|
    (scale = mean |ref|, at least 1).  The callers' values leave 3 to 4 times the measured error as headroom."""
    err = (got - want).abs()
    scale = want.abs().mean().item()
    assert scale > 0.05, "degenerate case: output too small to mean anything"
    assert torch.isfinite(got).all()
    assert err.mean().item() <= mean_tol * max(1.0, scale), f"mean err {err.mean().item()} at scale {scale}"
    assert err.max().item() <= max_tol * max(1.0, want.abs().max().item()), f"max err {err.max().item()}"
    print(f"bands: mean err {err.mean().item():.5f} max err {err.max().item():.4f} scale {scale:.4f} "
          f"ref max {want.abs().max().item():.3f} p99 {err.flatten().kthvalue(int(err.numel() * 0.99)).values.item():.4f}")
    assert (err <= bulk_tol * max(1.0, scale)).float().mean().item() >= 0.99
    return err.mean().item(), err.max().item(), scale


def test_encoder_stage_4x120k_full_size_vs_oracle(oracle):
    import bench_workloads as configs
    cfg = configs.ENCODER_STAGE
    C, H, bs, scope, hash_op = cfg["channels"], cfg["heads"], cfg["bucket_size"], cfg["scope_size"], cfg["hash_type"]
    coords, seps, _ = configs.lidar_batch(4, 120_000, 1004)
    emb, blk = configs.encoder_stage("swiglu", 1004)
    emb, blk = emb.to(DEV), blk.to(DEV)
    c, s = configs.to_device(coords, seps, DEV)
    with torch.no_grad():
        feat = emb(c, s, hash_op)
        out = blk(None, feat, None)
        # the same with the embedding not stored: the block forms it inside its kernels (what bench.py times)
        lazy = emb(c, s, hash_op, lazy=True)
        assert not isinstance(lazy, torch.Tensor)
        out_lazy = blk(None, lazy, None)
    torch.cuda.synchronize()
    n = coords.shape[0]
    pad_to = -(-n // (bs * scope * 6)) * (bs * scope * 6)
    assert out.shape == (pad_to, C)
    # PSH: every scattered row bit for bit
    scat = oracle.psh_scatter_coords(coords, seps, bs, pad_to, hash_op)
    assert np.array_equal(emb.last_scattered_coord.cpu().numpy().view(np.uint16), scat.view(np.uint16))
    sd = _state_dict_cpu(("emb.", emb), ("blk.", blk))
    torch.set_num_threads(max(1, min(16, torch.get_num_threads())))
    x = oracle._r(oracle.linear(torch.from_numpy(scat.astype(np.float32)).to(torch.bfloat16), sd["emb.lin.weight"],
                                sd["emb.lin.bias"]))
    assert (feat.float().cpu() - x).abs().max().item() <= 2e-2 * max(1.0, x.abs().max().item())
    w = {k: sd["blk." + v] for k, v in oracle.XFMR_KEYS.items()}
    want = oracle.xfmr_block(x, w, oracle.gen_scopes(pad_to, bs, scope), bs, H, "swiglu")
    # measured: mean 0.0009 at scale 0.73, 99th percentile 0.008, max 0.094 at max|ref| 15.6
    _bands(out.float().cpu(), want, mean_tol=0.004, bulk_tol=0.03, max_tol=0.03)
    _bands(out_lazy.float().cpu(), want, mean_tol=0.004, bulk_tol=0.03, max_tol=0.03)
    d = (out_lazy.float() - out.float()).abs()
    assert d.mean().item() <= 0.004 and d.max().item() <= 0.5, (d.mean().item(), d.max().item())


def test_first_block_follows_weight_changes_with_unstored_embedding():
    """the folded LayerNorm + QKV table of the first block is rebuilt when a parameter it was made from changes"""
    import bench_workloads as configs
    cfg = configs.ENCODER_STAGE
    coords, seps, _ = configs.lidar_batch(2, 20_000, 77)
    emb, blk = configs.encoder_stage("swiglu", 77)
    emb, blk = emb.to(DEV), blk.to(DEV)
    c, s = configs.to_device(coords, seps, DEV)

    def both():
        with torch.no_grad():
            stored = blk(None, emb(c, s, cfg["hash_type"]), None)
            lazy = blk(None, emb(c, s, cfg["hash_type"], lazy=True), None)
        return stored.float(), lazy.float()

    s0, l0 = both()
    assert blk.bwa.qkv._fold._val is not None, "the first block did not take the attention kernel that forms its own rows"
    assert (s0 - l0).abs().mean().item() <= 0.004
    with torch.no_grad():
        blk.bwa.qkv.weight.mul_(-0.5)
        blk.norm.bias.add_(0.3)
        emb.lin.weight.mul_(1.5)
    s1, l1 = both()
    assert (s1 - s0).abs().mean().item() > 0.05          # the change matters ...
    assert (s1 - l1).abs().mean().item() <= 0.004        # ... and the unstored path follows it


def _hook_pooling_buffers(model):
    from flash3dtransformer_amd.layers.hourglass import PoolingWrapper
    seen = []
    hooks = [m.register_forward_hook(lambda mod, inp, outp: seen.append((inp[0], inp[2], outp[2])))
             for m in model.modules() if isinstance(m, PoolingWrapper)]
    return seen, hooks


def test_hourglass_five_levels_vs_oracle_pipeline(oracle):
    import bench_workloads as configs
    cfg = configs.HOURGLASS
    bs, scope, S, hash_op = cfg["bucket_size"], cfg["scope_size"], cfg["subbuck_size"], cfg["hash_type"]
    model = configs.hourglass(1005)
    g = torch.Generator().manual_seed(7)
    for name, p in model.named_parameters():
        if p.dim() == 2:                     # make attention logits and MLP outputs matter
            p.data = (p.data * 2.0).to(torch.bfloat16).float()
        elif "norm" in name and name.endswith("weight"):
            p.data = (p.data + torch.randn(p.shape, generator=g) * 0.1).to(torch.bfloat16).float()
    model = model.to(DEV).eval()
    coords, seps, _ = configs.lidar_batch(4, 20_000, 1005)
    c, s = configs.to_device(coords, seps, DEV)
    seen, hooks = _hook_pooling_buffers(model)
    with torch.no_grad():
        out = model(c, None, s)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    sd = _state_dict_cpu(("", model))
    trace = []
    want, scat = oracle.flash3d_forward(sd, coords, seps, configs.hourglass_oracle_levels(model), bs, scope, hash_op, S,
                                        trace)
    assert np.array_equal(model.psh_scatter.last_scattered_coord.cpu().numpy().view(np.uint16), scat.view(np.uint16))
    # every level's pooling map and pooled coordinates are integer / fp16 work: bit for bit
    pools = [t for t in trace if t[0] == "pool"]
    assert len(pools) == len(seen) == 4
    for (_, level, unpool, red_coord), (_, _, buf) in zip(pools, seen):
        got_u = buf.unpool_ind.cpu().view(torch.int32).numpy().view(np.uint32)
        assert np.array_equal(got_u, unpool), f"level {level}: pooling map differs"
        assert np.array_equal(buf.reduced_coord.cpu().numpy().view(np.uint16), red_coord.view(np.uint16)), level
    assert out.shape == want.shape
    # ten transformer blocks, four poolings and four unpoolings deep; measured: mean 0.009 at scale 1.5, 99th
    # percentile 0.031, max 0.094 at max|ref| 6.3
    _bands(out.float().cpu(), want, mean_tol=0.025, bulk_tol=0.08, max_tol=0.06)


def test_hourglass_reference_shape_vs_oracle_pipeline(oracle):
    """The reference's own model shape (tests/test_psh_hourglass.py:55-150 of the reference: scopes of 8 buckets, two
    encoder + two decoder blocks per level, eval-mode BatchNorm1d(eps=1e-3) + GELU around pooling / unpooling, pooled
    lengths aligned to bucket x scope) on three levels 32 / 64 / 128 at 4 x 20,000 points against the oracle pipeline:
    scattered coordinates, every pooling map and pooled coordinates bit for bit; the output inside bands."""
    import bench_workloads as configs
    cfg = configs.HOURGLASS_REF_SHAPE
    bs, scope, S, hash_op = cfg["bucket_size"], cfg["scope_size"], cfg["subbuck_size"], cfg["hash_type"]
    model = configs.hourglass_ref_shape(1005, channels=(32, 64, 128))
    for name, p in model.named_parameters():
        if p.dim() == 2:                     # make attention logits and MLP outputs matter
            p.data = (p.data * 2.0).to(torch.bfloat16).float()
    model = model.to(DEV).eval()
    coords, seps, _ = configs.lidar_batch(4, 20_000, 1005)
    c, s = configs.to_device(coords, seps, DEV)
    seen, hooks = _hook_pooling_buffers(model)
    with torch.no_grad():
        out = model(c, None, s)
        again = model(c, None, s)            # second forward: prepared weights are reused
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    assert torch.equal(out, again)
    sd = _state_dict_cpu(("", model))
    trace = []
    want, scat = oracle.flash3d_forward(sd, coords, seps, configs.hourglass_oracle_levels(model), bs, scope, hash_op, S,
                                        trace)
    assert np.array_equal(model.psh_scatter.last_scattered_coord.cpu().numpy().view(np.uint16), scat.view(np.uint16))
    pools = [t for t in trace if t[0] == "pool"]
    assert len(pools) == 2 and len(seen) == 4          # two poolings per forward, two forwards
    for (_, level, unpool, red_coord), (_, _, buf) in zip(pools, seen):
        assert buf.reduced_coord.shape[0] % (bs * scope) == 0
        assert np.array_equal(buf.unpool_ind.cpu().view(torch.int32).numpy().view(np.uint32), unpool), level
        assert np.array_equal(buf.reduced_coord.cpu().numpy().view(np.uint16), red_coord.view(np.uint16)), level
    assert out.shape == want.shape
    # measured: mean 0.029 at scale 5.9, 99th percentile 0.25, max 1.0 at max|ref| 247
    _bands(out.float().cpu(), want, mean_tol=0.02, bulk_tol=0.15, max_tol=0.02)


def test_hourglass_reference_shape_4x250k_properties():
    """the same shape on five levels 32 ... 512 at 4 x 250,000 points: finite, bit-reproducible, every level's length a
    multiple of bucket x scope (so that no level falls back to one global scope), pooling maps bijective"""
    import bench_workloads as configs
    import warnings
    model = configs.hourglass_ref_shape(1005).to(DEV).eval()
    coords, seps, _ = configs.lidar_batch(4, 250_000, 1005)
    c, s = configs.to_device(coords, seps, DEV)
    seen, hooks = _hook_pooling_buffers(model)
    with torch.no_grad(), warnings.catch_warnings():
        warnings.simplefilter("error")       # the planner warns when a length falls back to one global scope
        out = model(c, None, s)
        again = model(c, None, s)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    bs, scope = configs.HOURGLASS_REF_SHAPE["bucket_size"], configs.HOURGLASS_REF_SHAPE["scope_size"]
    n = coords.shape[0]
    pad_to = -(-n // (bs * scope * 6)) * (bs * scope * 6)
    assert out.shape == (pad_to, 32) and torch.isfinite(out.float()).all() and torch.equal(out, again)
    assert out.float().abs().mean().item() > 1e-3
    rows = pad_to
    for _, _, buf in seen[:4]:
        u = buf.unpool_ind.cpu().view(torch.int32).numpy().view(np.uint32)
        filled = u[u < rows]
        assert filled.size == rows and np.array_equal(np.sort(filled), np.arange(rows, dtype=np.uint32))
        rows = buf.reduced_coord.shape[0]
        assert rows % (bs * scope) == 0


def test_hourglass_4x250k_full_size_properties():
    """config 5 at full size: finite output of the right shape; every level's pooling map is a bijection between the
    level's rows and the filled slots; restoring the input order inverts the PSH permutation"""
    import bench_workloads as configs
    model = configs.hourglass(1005).to(DEV).eval()
    coords, seps, _ = configs.lidar_batch(4, 250_000, 1005)
    c, s = configs.to_device(coords, seps, DEV)
    seen, hooks = _hook_pooling_buffers(model)
    with torch.no_grad():
        out = model(c, None, s)
        again = model(c, None, s)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    n = coords.shape[0]
    bs = configs.HOURGLASS["bucket_size"]
    pad_to = -(-n // (bs * 6)) * (bs * 6)
    assert out.shape == (pad_to, 32) and torch.isfinite(out.float()).all()
    assert out.float().abs().mean().item() > 1e-3
    assert torch.equal(out, again), "the forward is a pure function of its input"
    assert len(seen) == 8
    rows = pad_to
    for level, (lvl_coords, lvl_seps, buf) in enumerate(seen[:4]):
        assert lvl_coords.shape[0] == rows
        u = buf.unpool_ind.view(torch.int32).long().reshape(-1)
        filled = u[u < rows]
        assert filled.numel() == rows, f"level {level}: {filled.numel()} filled slots for {rows} rows"
        assert torch.equal(torch.sort(filled)[0], torch.arange(rows, device=DEV)), f"level {level}: not a bijection"
        sizes = torch.diff(lvl_seps.view(torch.int32).long(), prepend=torch.zeros(1, dtype=torch.long, device=DEV))
        want_rows = int(((sizes + 1) // 2).sum())
        assert buf.unpool_ind.shape[0] == want_rows
        assert buf.reduced_feat.shape[0] % bs == 0 and buf.reduced_feat.shape[0] - want_rows < bs
        rows = buf.reduced_feat.shape[0]
    # input order: the scattered coordinates come back as the input coordinates, and rows map through the index
    with torch.no_grad():
        assert torch.equal(model.to_input_order(model.psh_scatter.last_scattered_coord), c)
        per_point = model.to_input_order(out)
    idx = model._last_index.view(torch.int32)[:n].long()
    assert per_point.shape == (n, 32) and torch.equal(out[:n], per_point[idx])


def test_encoder_stage_4x120k_backward_full_size_properties():
    """config 4 at full size through loss.backward(): every gradient is finite and not identically zero; a second run
    gives the same bits (no atomics anywhere in the backward); and the backward is linear in the upstream gradient:
    doubling it doubles every gradient exactly (a power of two commutes with every bf16 / fp32 rounding on the way)"""
    import bench_workloads as configs
    cfg = configs.ENCODER_STAGE
    hash_op = cfg["hash_type"]
    coords, seps, _ = configs.lidar_batch(4, 120_000, 1004)
    emb, blk = configs.encoder_stage("swiglu", 1004)
    emb, blk = emb.to(DEV).train(), blk.to(DEV).train()
    c, s = configs.to_device(coords, seps, DEV)
    params = [p for p in list(emb.parameters()) + list(blk.parameters())]
    g = torch.Generator(device="cpu").manual_seed(77)

    def grads(scale):
        for p in params:
            p.grad = None
        feat = emb(c, s, hash_op)
        out = blk(None, feat, None)
        if grads.dy is None:
            grads.dy = (torch.randn(out.shape, generator=g) * 0.25).to(torch.bfloat16).to(DEV)
        out.backward(grads.dy * scale)
        torch.cuda.synchronize()
        return [p.grad.detach().clone() for p in params]
    grads.dy = None
    g1, g1b, g2 = grads(1.0), grads(1.0), grads(2.0)
    for p, a, b, d in zip(params, g1, g1b, g2):
        assert torch.isfinite(a).all() and a.abs().max().item() > 0, tuple(p.shape)
        assert torch.equal(a, b), f"gradient of a {tuple(p.shape)} parameter differs between two runs"
        assert torch.equal(a * 2, d), f"gradient of a {tuple(p.shape)} parameter is not linear in the upstream gradient"


def test_hourglass_4x250k_backward_full_size_properties():
    """config 5 at full size through loss.backward(): PSH embedding, five levels of blocks, pooling and unpooling.  Every
    parameter receives a finite, not identically zero gradient; a second run gives the same bits; doubling the upstream
    gradient doubles every gradient exactly"""
    import bench_workloads as configs
    model = configs.hourglass(1005).to(DEV).train()
    coords, seps, _ = configs.lidar_batch(4, 250_000, 1005)
    c, s = configs.to_device(coords, seps, DEV)
    params = list(model.parameters())
    g = torch.Generator(device="cpu").manual_seed(78)

    def grads(scale):
        for p in params:
            p.grad = None
        out = model(c, None, s)
        if grads.dy is None:
            grads.dy = (torch.randn(out.shape, generator=g) * 0.25).to(torch.bfloat16).to(DEV)
        out.backward(grads.dy * scale)
        torch.cuda.synchronize()
        return [p.grad.detach().clone() for p in params]
    grads.dy = None
    g1, g1b, g2 = grads(1.0), grads(1.0), grads(2.0)
    names = [n for n, _ in model.named_parameters()]
    for n, a, b, d in zip(names, g1, g1b, g2):
        assert torch.isfinite(a).all() and a.abs().max().item() > 0, n
        assert torch.equal(a, b), f"{n}: gradient differs between two runs"
        assert torch.equal(a * 2, d), f"{n}: gradient is not linear in the upstream gradient"
