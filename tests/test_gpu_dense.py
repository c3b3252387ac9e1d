"""GPU parity of the dense layers (rows A11, A12): MFMA linear with fused epilogues, LayerNorm,
coordinate embedding, affine+activation, and the gemm_sm_bf16 op (reference tests/test_gemm.py:26-43:
M,N,K = 128,256,128, allclose(atol=rtol=1e-2)).  Floating-point ops: compared with fp32 torch on the
same bf16-rounded inputs; tolerance is one bf16 rounding of the result plus accumulation noise,
|err| <= 2e-2 * max(1, |ref|)."""
import math

import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _rand(shape, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _close(got, ref, tol=2e-2):
    err = (got.float().cpu() - ref).abs()
    assert (err <= tol * ref.abs().clamp(min=1.0)).all(), f"max err {err.max().item()}"


def test_gemm_sm_bf16_reference_case():
    from flash3dtransformer_amd.lib import pshattn
    M, N, K = 128, 256, 128
    a, b = _rand((M, K), 2).to(DEV), _rand((K, N), 3).to(DEV)
    o = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    pshattn.gemm_sm_bf16(a, b, o)
    ref = a.float().cpu() @ b.float().cpu()
    # the reference's own bar for this op (tests/test_gemm.py:35 of the reference)
    assert torch.allclose(o.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    # general shapes, which the reference op rejects
    for (M, N, K) in [(300, 72, 40), (1, 8, 8), (1000, 520, 264)]:
        a, b = _rand((M, K), M).to(DEV), _rand((K, N), N).to(DEV)
        o = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        pshattn.gemm_sm_bf16(a, b, o)
        _close(o, a.float().cpu() @ b.float().cpu(), tol=2e-2 * max(1.0, K ** 0.5 / 4))


@pytest.mark.parametrize("M,N,K,act,use_bias,use_res", [
    (4096, 768, 256, None, True, False),       # QKV projection of the C=256 block
    (4096, 256, 256, None, True, True),        # out-projection + residual
    (4096, 2048, 256, "swiglu", True, False),  # fc1 of the swiglu MLP, hid = 1024
    (4096, 256, 1024, None, True, True),       # fc2 + residual
    (1000, 1024, 256, "gelu", True, False),    # plain-GELU MLP variant, ragged M
    (777, 96, 64, "relu", False, False),
    (130, 136, 72, "silu", True, True),        # edges in M, N and K
    (3000, 32, 128, None, True, True),         # half-full last chunk of the row-panel kernel (fc2 of a C=32 level)
    (140000, 96, 32, None, True, False),       # the same in the 512-row configuration (qkv of a C=32 level)
    (140000, 32, 32, "gelu", True, True),
    (3001, 1536, 512, None, True, False),      # qkv of a C=512 level: 512 inner features in the row-panel kernel, ragged M
    (2500, 512, 512, None, True, True),        # out-projection + residual of that level
    (2100, 96, 512, None, True, True),         # 512 inner features, residual, 32 columns in the last chunk
    (120000, 32, 256, "silu", True, True),     # activation + residual on a single 32-column chunk, 512-row configuration
    (2100, 2048, 512, "swiglu", True, False),  # its fc1
    (700, 256, 512, "gelu", False, True),      # fc2 of a C=256 level
    (40000, 256, 1024, None, True, True),      # fc2 + residual of the C=256 block at a size the output-panel kernel takes
    (33001, 128, 640, None, False, False),     # the same kernel: 128 outputs, ragged M, 20 chunks, no bias, no residual
    (35000, 256, 544, None, True, False),      # 17 chunks
])
def test_linear_epilogues(oracle, M, N, K, act, use_bias, use_res):
    from flash3dtransformer_amd.lib import pshattn
    x, w = _rand((M, K), 1), _rand((N, K), 2, scale=1 / math.sqrt(K))
    bias = _rand((N,), 3) if use_bias else None
    n_out = N // 2 if act == "swiglu" else N
    res = _rand((M, n_out), 4) if use_res else None
    y = torch.full((M, n_out), 9.0, dtype=torch.bfloat16, device=DEV)
    pshattn.linear_bf16(x.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV),
                        None if res is None else res.to(DEV), y, act)
    torch.cuda.synchronize()
    lin = oracle.linear(x, w, bias).to(torch.bfloat16).float()       # a Linear rounds its output to bf16
    if act == "swiglu":
        ref = oracle.swiglu(lin)
    elif act == "gelu":
        ref = oracle.gelu(lin)
    elif act == "relu":
        ref = torch.relu(lin)
    elif act == "silu":
        ref = torch.nn.functional.silu(lin)
    else:
        ref = lin
    if res is not None:
        ref = ref.to(torch.bfloat16).float() + res.float()
    _close(y, ref)


@pytest.mark.parametrize("M,N,K,act,use_res", [
    (5000, 768, 256, None, False),       # norm -> qkv of the C=256 block
    (5000, 2048, 256, "swiglu", False),  # LayerNormMLP front half
    (333, 96, 32, "gelu", True),
    (133000, 96, 32, None, False),       # norm -> qkv of a C=32 level, 512-row configuration, half-full chunk
    (1000, 192, 64, None, True),
    (2049, 256, 128, "relu", False),
    (1900, 1536, 512, None, False),      # norm -> qkv of a C=512 level
    (1300, 2048, 512, "swiglu", True),   # norm -> fc1 -> gate of that level
])
def test_layernorm_fused_linear(oracle, M, N, K, act, use_res):
    from flash3dtransformer_amd.lib import pshattn
    x, w = _rand((M, K), 1, scale=2.0) + 0.3, _rand((N, K), 2, scale=1 / math.sqrt(K))
    g, b, bias = _rand((K,), 3) + 1.0, _rand((K,), 4, scale=0.2), _rand((N,), 5)
    n_out = N // 2 if act == "swiglu" else N
    res = _rand((M, n_out), 6) if use_res else None
    y = torch.full((M, n_out), 9.0, dtype=torch.bfloat16, device=DEV)
    pshattn.ln_linear_bf16(x.to(DEV), g.to(DEV), b.to(DEV), 1e-5, w.to(DEV), bias.to(DEV),
                           None if res is None else res.to(DEV), y, act)
    torch.cuda.synchronize()
    acts = {"swiglu": oracle.swiglu, "gelu": oracle.gelu, "relu": torch.relu, None: lambda t: t}
    # the reference's sequence of bf16 roundings (LayerNorm output, Linear output) ...
    ln = oracle.layernorm(x, g, b, 1e-5).to(torch.bfloat16).float()
    lin = oracle.linear(ln, w, bias).to(torch.bfloat16).float()
    ref = acts[act](lin)
    # ... and the same mathematics without any intermediate rounding
    exact = acts[act](oracle.linear(oracle.layernorm(x, g, b, 1e-5), w, bias))
    if res is not None:
        ref = ref.to(torch.bfloat16).float() + res.float()
        exact = exact + res.float()
    # The kernel folds LayerNorm into the weights (w * gamma rounded to bf16, statistics applied to the fp32
    # accumulators), so its roundings fall in other places than the reference's.  It must sit as close to the
    # exact result as the reference's own rounding sequence does (bf16 output rounding included in both).
    yf = y.float().cpu()
    err_ref = (ref.to(torch.bfloat16).float() - exact).abs()
    err_us = (yf - exact).abs()
    scale = exact.abs().clamp(min=1.0)
    assert (err_us / scale).max() <= 1.5 * (err_ref / scale).max() + 4e-3, (err_us.max(), err_ref.max())
    assert err_us.mean() <= 1.25 * err_ref.mean() + 1e-4, (err_us.mean(), err_ref.mean())


def test_linear_strided_views():
    """x and y may be column slices of wider buffers (row stride > width)"""
    from flash3dtransformer_amd.lib import pshattn
    M, N, K = 512, 128, 64
    xb, w = _rand((M, 3 * K), 5).to(DEV), _rand((N, K), 6, scale=0.1).to(DEV)
    yb = torch.zeros(M, 2 * N, dtype=torch.bfloat16, device=DEV)
    pshattn.linear_bf16(xb[:, K:2 * K], w, None, None, yb[:, N:], None)
    torch.cuda.synchronize()
    _close(yb[:, N:], xb[:, K:2 * K].float().cpu() @ w.float().cpu().t())
    assert (yb[:, :N] == 0).all()


@pytest.mark.parametrize("M,C", [(1000, 256), (33, 32), (257, 1024), (64, 520), (5, 4096)])
def test_layernorm(oracle, M, C):
    from flash3dtransformer_amd.lib import pshattn
    x, g, b = _rand((M, C), 1, scale=3.0), _rand((C,), 2), _rand((C,), 3)
    y = torch.empty(M, C, dtype=torch.bfloat16, device=DEV)
    pshattn.layernorm_bf16(x.to(DEV), g.to(DEV), b.to(DEV), y, 1e-5)
    torch.cuda.synchronize()
    _close(y, oracle.layernorm(x, g, b, 1e-5))


def test_coord_embed_and_affine(oracle):
    from flash3dtransformer_amd.lib import pshattn
    M, C = 5000, 256
    coord = _rand((M, 3), 1, scale=30.0, dtype=torch.float16)
    w, b = _rand((C, 3), 2, scale=0.3), _rand((C,), 3)
    y = torch.empty(M, C, dtype=torch.bfloat16, device=DEV)
    pshattn.coord_embed_bf16(coord.to(DEV), w.to(DEV), b.to(DEV), y)
    torch.cuda.synchronize()
    _close(y, oracle.linear(coord.to(torch.bfloat16), w, b))
    x = _rand((M, C), 4)
    scale, shift = torch.rand(C) + 0.5, torch.randn(C)
    for act, fn in (("gelu", oracle.gelu), (None, lambda t: t), ("relu", torch.relu)):
        pshattn.affine_act_bf16(x.to(DEV), scale.to(DEV), shift.to(DEV), y, act)
        torch.cuda.synchronize()
        _close(y, fn((x.float() * scale + shift).to(torch.bfloat16).float()))


def test_dense_argument_errors():
    from flash3dtransformer_amd.lib import pshattn
    mk = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        pshattn.linear_bf16(mk(16, 12), mk(8, 12), None, None, mk(16, 8))
    with pytest.raises(RuntimeError, match="shape mismatch"):
        pshattn.linear_bf16(mk(16, 16), mk(8, 24), None, None, mk(16, 8))
    with pytest.raises(RuntimeError, match="LayerNorm width"):
        pshattn.layernorm_bf16(mk(4, 12), mk(12), mk(12), mk(4, 12))
    with pytest.raises(RuntimeError, match="gemm shape mismatch"):
        pshattn.gemm_sm_bf16(mk(8, 16), mk(8, 16), mk(8, 16))


@pytest.mark.parametrize("M,C,H,use_res,use_bias", [
    (4096, 256, 1024, True, True),      # the C = 256 block's MLP
    (1000, 256, 512, False, True),      # ragged M, no residual
    (777, 128, 512, True, False),       # C = 128, no biases
    (300, 256, 32, True, True),         # a single hidden chunk
    (70000, 128, 256, True, True),      # many workgroups
    (5000, 32, 128, True, True),        # narrow layers: all weights resident in LDS, waves walk the row tiles
    (100000, 64, 256, True, True),      # ... more tiles than resident waves
    (333, 64, 64, False, False),        # ... ragged M, no residual, no biases
    (1000, 32, 640, True, True),        # ... the largest hidden width that fits at C = 32
    (40, 64, 288, True, False),         # ... and at C = 64; fewer rows than one workgroup's waves
])
def test_fused_mlp_matches_two_kernel_path(oracle, M, C, H, use_res, use_bias):
    """The one-kernel gated MLP against (a) the LayerNorm+fc1+swiglu kernel followed by the fc2+residual kernel, whose
    roundings it reproduces (same folded weights, hidden activations rounded to bf16; only the fp32 summation order
    of fc2 differs), and (b) the unrounded mathematics, next to the reference's own rounding sequence."""
    from flash3dtransformer_amd.lib import pshattn
    x = (_rand((M, C), 1, scale=2.0) + 0.3).to(DEV)
    g, b = (_rand((C,), 3) + 1.0).to(DEV), _rand((C,), 4, scale=0.2).to(DEV)
    w1, w2 = _rand((2 * H, C), 2, scale=1 / math.sqrt(C)).to(DEV), _rand((C, H), 5, scale=1 / math.sqrt(H)).to(DEV)
    b1 = _rand((2 * H,), 6).to(DEV) if use_bias else None
    b2 = _rand((C,), 7).to(DEV) if use_bias else None
    res = _rand((M, C), 8).to(DEV) if use_res else None
    y = torch.full((M, C), 9.0, dtype=torch.bfloat16, device=DEV)
    assert pshattn.ln_mlp_swiglu_bf16(x, g, b, 1e-5, w1, b1, w2, b2, res, y)
    hid = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    y2 = torch.empty_like(y)
    pshattn.ln_linear_bf16(x, g, b, 1e-5, w1, b1, None, hid, "swiglu")
    pshattn.linear_bf16(hid, w2, b2, res, y2, None)
    torch.cuda.synchronize()
    d = (y.float() - y2.float()).abs()
    scale = y2.float().abs().clamp(min=1.0)
    # a hidden value that rounds the other way (the two paths sum fc1 in different orders: the fused kernel starts its
    # accumulators from b', the other adds it last) moves an output by a step or two before the final rounding: at most
    # four bf16 steps apart
    assert (d / scale).max().item() <= 2 ** -5, (d / scale).max().item()
    assert (d > 0).float().mean().item() < 0.02                                     # and almost always equal
    # (b) against the unrounded mathematics: at least as close as the reference's own sequence of bf16 roundings
    # (LayerNorm output, fc1 output, gated product, fc2 output, residual sum)
    xc, gc, bc, w1c, w2c = x.cpu(), g.cpu(), b.cpu(), w1.cpu(), w2.cpu()
    b1c, b2c = (None if b1 is None else b1.cpu()), (None if b2 is None else b2.cpu())
    rb = lambda t: t.to(torch.bfloat16).float()
    exact = oracle.linear(oracle.swiglu(oracle.linear(oracle.layernorm(xc, gc, bc, 1e-5), w1c, b1c)), w2c, b2c)
    ref = rb(oracle.linear(rb(oracle.swiglu(rb(oracle.linear(rb(oracle.layernorm(xc, gc, bc, 1e-5)), w1c, b1c)))), w2c, b2c))
    if res is not None:
        exact = exact + res.float().cpu()
        ref = rb(ref + res.float().cpu())
    scale = exact.abs().clamp(min=1.0)
    err_us, err_ref = (y.float().cpu() - exact).abs() / scale, (ref - exact).abs() / scale
    assert err_us.max() <= 1.5 * err_ref.max() + 4e-3, (err_us.max(), err_ref.max())
    assert err_us.mean() <= 1.25 * err_ref.mean() + 1e-4, (err_us.mean(), err_ref.mean())


@pytest.mark.parametrize("M,C,H,use_bias", [
    (4096, 256, 1024, True),       # the C = 256 block
    (1000, 256, 512, True),        # ragged M
    (777, 128, 512, False),        # C = 128 (two projection chunks), no biases
    (300, 256, 32, True),          # a single hidden chunk behind the projection
    (70000, 128, 256, True),       # many workgroups
    (66000, 256, 64, True),        # more panels than CUs: shorter panels in the last turn
    (5000, 32, 128, True),         # narrow layers: the projection weight resident in LDS with the others
    (100000, 64, 256, True),       # ... more tiles than resident waves
    (333, 64, 64, False),          # ... ragged M, no biases
    (40, 32, 512, True),           # ... fewer rows than one workgroup's waves
])
def test_proj_residual_mlp_in_one_kernel(oracle, M, C, H, use_bias):
    """out-projection + residual + gated MLP + residual in one kernel against (a) the projection kernel followed by the
    one-kernel MLP (the one kernel rounds x1 once, from the fp32 sum of projection and block input, and the final sum
    once: results a bf16 step or two apart, never more), and (b) the unrounded mathematics next to the reference's
    rounding sequence."""
    from flash3dtransformer_amd.lib import pshattn
    a = _rand((M, C), 11, scale=1.5).to(DEV)
    x = (_rand((M, C), 1, scale=2.0) + 0.3).to(DEV)
    wp = _rand((C, C), 12, scale=1 / math.sqrt(C)).to(DEV)
    bp = _rand((C,), 13).to(DEV) if use_bias else None
    g, b = (_rand((C,), 3) + 1.0).to(DEV), _rand((C,), 4, scale=0.2).to(DEV)
    w1, w2 = _rand((2 * H, C), 2, scale=1 / math.sqrt(C)).to(DEV), _rand((C, H), 5, scale=1 / math.sqrt(H)).to(DEV)
    b1 = _rand((2 * H,), 6).to(DEV) if use_bias else None
    b2 = _rand((C,), 7).to(DEV) if use_bias else None
    y = torch.full((M, C), 9.0, dtype=torch.bfloat16, device=DEV)
    assert pshattn.proj_ln_mlp_swiglu_bf16(a, wp, bp, x, g, b, 1e-5, w1, b1, w2, b2, y)
    x1 = torch.empty_like(x)
    y2 = torch.empty_like(y)
    pshattn.linear_bf16(a, wp, bp, x, x1, None)
    assert pshattn.ln_mlp_swiglu_bf16(x1, g, b, 1e-5, w1, b1, w2, b2, x1, y2)
    torch.cuda.synchronize()
    d = (y.float() - y2.float()).abs()
    scale = y2.float().abs().clamp(min=1.0)
    # x1 differs by a bf16 step wherever the two roundings of the separate kernels fall the other way than the single
    # one; behind the LayerNorm, the gate and the long sums that leaves the two results about one bf16 step apart on
    # average (each about one step from the unrounded mathematics, see below) and a few steps at most
    assert (d / scale).max().item() <= 0.25, (d / scale).max().item()
    assert (d / scale).mean().item() <= 6e-3, (d / scale).mean().item()
    ac, xc, wpc, gc, bc, w1c, w2c = a.cpu(), x.cpu(), wp.cpu(), g.cpu(), b.cpu(), w1.cpu(), w2.cpu()
    cpu = lambda t: None if t is None else t.cpu()
    rb = lambda t: t.to(torch.bfloat16).float()
    mlp = lambda t, r: oracle.linear(r(oracle.swiglu(r(oracle.linear(r(oracle.layernorm(t, gc, bc, 1e-5)), w1c, cpu(b1))))), w2c, cpu(b2))
    same = lambda t: t
    x1e = oracle.linear(ac, wpc, cpu(bp)) + xc.float()
    exact = x1e + mlp(x1e, same)
    x1r = rb(rb(oracle.linear(ac, wpc, cpu(bp))) + xc.float())
    ref = rb(x1r + rb(mlp(x1r, rb)))
    scale = exact.abs().clamp(min=1.0)
    err_us, err_ref = (y.float().cpu() - exact).abs() / scale, (ref - exact).abs() / scale
    assert err_us.max() <= 1.5 * err_ref.max() + 4e-3, (err_us.max(), err_ref.max())
    assert err_us.mean() <= 1.25 * err_ref.mean() + 1e-4, (err_us.mean(), err_ref.mean())


def test_proj_residual_mlp_unsupported_width_is_reported():
    from flash3dtransformer_amd.lib import pshattn
    mk = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    y = torch.full((64, 64), 3.0, dtype=torch.bfloat16, device=DEV)
    # C = 64 with a hidden width whose weights do not fit into LDS; C = 512
    assert not pshattn.proj_ln_mlp_swiglu_bf16(mk(64, 64), mk(64, 64), None, mk(64, 64), mk(64), mk(64), 1e-5, mk(640, 64),
                                               None, mk(64, 320), None, y)
    assert (y == 3.0).all()
    y5 = torch.full((64, 512), 3.0, dtype=torch.bfloat16, device=DEV)
    assert not pshattn.proj_ln_mlp_swiglu_bf16(mk(64, 512), mk(512, 512), None, mk(64, 512), mk(512), mk(512), 1e-5,
                                               mk(128, 512), None, mk(512, 64), None, y5)
    assert (y5 == 3.0).all()


@pytest.mark.parametrize("M,K,N", [(70000, 256, 768), (5000, 32, 96), (333, 64, 192), (200000, 128, 384), (1, 256, 32)])
def test_embedding_inside_layernorm_linear(oracle, M, K, N):
    """LayerNorm + Linear on the coordinate embedding formed inside the kernel against the embedding kernel followed by
    the LayerNorm + Linear kernel (the embedding is summed in another order on the matrix core: a bf16 step apart in
    a few places), and against fp32 mathematics."""
    from flash3dtransformer_amd.lib import pshattn
    g = torch.Generator().manual_seed(21)
    coord = ((torch.rand(M, 3, generator=g) - 0.5) * 80.0).to(torch.float16).to(DEV)
    we, be = _rand((K, 3), 22, scale=0.5).to(DEV), _rand((K,), 23).to(DEV)
    gam, bet = (_rand((K,), 3) + 1.0).to(DEV), _rand((K,), 4, scale=0.2).to(DEV)
    w, b = _rand((N, K), 2, scale=1 / math.sqrt(K)).to(DEV), _rand((N,), 6).to(DEV)
    y = torch.full((M, N), 9.0, dtype=torch.bfloat16, device=DEV)
    assert pshattn.embed_ln_linear_bf16(coord, pshattn.embed_table(we, be), gam, bet, 1e-5, w, b, y)
    x = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    y2 = torch.empty_like(y)
    pshattn.coord_embed_bf16(coord, we, be, x)
    pshattn.ln_linear_bf16(x, gam, bet, 1e-5, w, b, None, y2, None)
    torch.cuda.synchronize()
    d = (y.float() - y2.float()).abs() / y2.float().abs().clamp(min=1.0)
    assert d.max().item() <= 2 ** -4, d.max().item()
    assert (d > 0).float().mean().item() < 0.05
    xe = oracle.linear(coord.cpu().to(torch.bfloat16), we.cpu(), be.cpu()).to(torch.bfloat16)
    ref = oracle.linear(oracle.layernorm(xe, gam.cpu(), bet.cpu(), 1e-5), w.cpu(), b.cpu())
    _close(y.float().cpu(), ref)


@pytest.mark.parametrize("M,C,H", [(70000, 256, 1024), (5000, 32, 128), (333, 64, 64), (66000, 128, 256)])
def test_embedding_as_block_input_of_proj_residual_mlp(oracle, M, C, H):
    """the one-kernel second half of a block with its block input formed from the coordinates against the same kernel
    reading the stored embedding (the embedding enters unrounded: a bf16 step apart in places), and against the
    unrounded mathematics"""
    from flash3dtransformer_amd.lib import pshattn
    g = torch.Generator().manual_seed(31)
    coord = ((torch.rand(M, 3, generator=g) - 0.5) * 8.0).to(torch.float16).to(DEV)
    we, be = _rand((C, 3), 22, scale=0.5).to(DEV), _rand((C,), 23).to(DEV)
    a = _rand((M, C), 11, scale=1.5).to(DEV)
    wp, bp = _rand((C, C), 12, scale=1 / math.sqrt(C)).to(DEV), _rand((C,), 13).to(DEV)
    gam, bet = (_rand((C,), 3) + 1.0).to(DEV), _rand((C,), 4, scale=0.2).to(DEV)
    w1, w2 = _rand((2 * H, C), 2, scale=1 / math.sqrt(C)).to(DEV), _rand((C, H), 5, scale=1 / math.sqrt(H)).to(DEV)
    b1, b2 = _rand((2 * H,), 6).to(DEV), _rand((C,), 7).to(DEV)
    y = torch.full((M, C), 9.0, dtype=torch.bfloat16, device=DEV)
    assert pshattn.embed_proj_ln_mlp_swiglu_bf16(a, wp, bp, coord, pshattn.embed_table(we, be), gam, bet, 1e-5, w1, b1, w2, b2, y)
    x = torch.empty(M, C, dtype=torch.bfloat16, device=DEV)
    y2 = torch.empty_like(y)
    pshattn.coord_embed_bf16(coord, we, be, x)
    assert pshattn.proj_ln_mlp_swiglu_bf16(a, wp, bp, x, gam, bet, 1e-5, w1, b1, w2, b2, y2)
    torch.cuda.synchronize()
    d = (y.float() - y2.float()).abs() / y2.float().abs().clamp(min=1.0)
    assert d.max().item() <= 0.25 and d.mean().item() <= 4e-3, (d.max().item(), d.mean().item())
    c = lambda t: t.cpu()
    xe = oracle.linear(c(coord).to(torch.bfloat16), c(we), c(be))
    x1 = oracle.linear(c(a), c(wp), c(bp)) + xe
    exact = x1 + oracle.linear(oracle.swiglu(oracle.linear(oracle.layernorm(x1, c(gam), c(bet), 1e-5), c(w1), c(b1))), c(w2), c(b2))
    scale = exact.abs().clamp(min=1.0)
    err_us, err_ref = (y.float().cpu() - exact).abs() / scale, (y2.float().cpu() - exact).abs() / scale
    assert err_us.max() <= 1.5 * err_ref.max() + 4e-3 and err_us.mean() <= 1.25 * err_ref.mean() + 1e-4


def test_embedding_inside_layernorm_linear_unsupported_width_is_reported():
    from flash3dtransformer_amd.lib import pshattn
    mk = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    y = torch.full((64, 64), 3.0, dtype=torch.bfloat16, device=DEV)
    coord = torch.zeros(64, 3, dtype=torch.float16, device=DEV)
    assert not pshattn.embed_ln_linear_bf16(coord, mk(512, 8), mk(512), mk(512), 1e-5, mk(64, 512), None, y)
    assert (y == 3.0).all()


def test_fused_mlp_unsupported_width_is_reported():
    from flash3dtransformer_amd.lib import pshattn
    mk = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    y = torch.full((64, 64), 3.0, dtype=torch.bfloat16, device=DEV)
    # C = 64 with a hidden width whose weights do not fit into LDS; C = 512
    assert not pshattn.ln_mlp_swiglu_bf16(mk(64, 64), mk(64), mk(64), 1e-5, mk(640, 64), None, mk(64, 320), None, None, y)
    assert (y == 3.0).all()
    y5 = torch.full((64, 512), 3.0, dtype=torch.bfloat16, device=DEV)
    assert not pshattn.ln_mlp_swiglu_bf16(mk(64, 512), mk(512), mk(512), 1e-5, mk(128, 512), None, mk(512, 64), None, None, y5)
    assert (y5 == 3.0).all()


def test_layernorm_mlp_layer_one_kernel_and_two_kernel_paths():
    """LayerNormMLP(fused=True) routes through the one-kernel gated MLP, fused=False through LayerNorm+fc1+gate and
    fc2+residual; the default picks by size and equals one of them bit for bit; gradients flow through either."""
    from flash3dtransformer_amd.layers.nn_ops import LayerNormMLP
    torch.manual_seed(5)
    a, b, auto = LayerNormMLP(256, 512, fused=False).to(DEV), LayerNormMLP(256, 512, fused=True).to(DEV), LayerNormMLP(256, 512).to(DEV)
    b.load_state_dict(a.state_dict())
    auto.load_state_dict(a.state_dict())
    x = torch.randn(3000, 256, device=DEV).to(torch.bfloat16)
    ya, yb = a(x, residual=x), b(x, residual=x)
    d = (ya.float() - yb.float()).abs() / ya.float().abs().clamp(min=1.0)
    assert d.max().item() <= 2 ** -5
    assert torch.equal(auto(x, residual=x), ya)                       # 3,000 rows of width 256: two kernels
    big = torch.randn(70000, 256, device=DEV).to(torch.bfloat16)
    assert torch.equal(auto(big, residual=big), b(big, residual=big))   # 70,000 rows: one kernel
    xg = x.clone().requires_grad_(True)
    b(xg, residual=xg).float().square().mean().backward()
    assert xg.grad is not None and torch.isfinite(xg.grad.float()).all() and xg.grad.abs().max().item() > 0
    assert b.fc2_weight.grad.abs().max().item() > 0


def test_fused_mlp_and_output_panel_kernel_at_bench_size(oracle):
    """482,304 rows x 256 channels, hidden 1024 (the bench's MLP): the one-kernel MLP against LayerNorm+fc1+gate
    followed by fc2+residual (which at this size runs the output-panel kernel), and the output-panel kernel against
    the tiled GEMM on a row slice small enough to fall back to it."""
    from flash3dtransformer_amd.lib import pshattn
    M, C, H = 482304, 256, 1024
    x = (_rand((M, C), 11, scale=1.5)).to(DEV)
    g, b = (_rand((C,), 3) + 1.0).to(DEV), _rand((C,), 4, scale=0.2).to(DEV)
    w1, w2 = _rand((2 * H, C), 2, scale=1 / math.sqrt(C)).to(DEV), _rand((C, H), 5, scale=1 / math.sqrt(H)).to(DEV)
    b1, b2 = _rand((2 * H,), 6).to(DEV), _rand((C,), 7).to(DEV)
    y = torch.empty(M, C, dtype=torch.bfloat16, device=DEV)
    assert pshattn.ln_mlp_swiglu_bf16(x, g, b, 1e-5, w1, b1, w2, b2, x, y)
    hid = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    y2 = torch.empty_like(y)
    pshattn.ln_linear_bf16(x, g, b, 1e-5, w1, b1, None, hid, "swiglu")
    pshattn.linear_bf16(hid, w2, b2, x, y2, None)                     # output-panel kernel (K = 1024 > 512, many rows)
    torch.cuda.synchronize()
    # one bf16 step of the fc2 output before the residual add, whose magnitude is at most |y| + |residual|
    d = (y.float() - y2.float()).abs() / (y2.float().abs() + x.float().abs()).clamp(min=1.0)
    assert d.max().item() <= 2 ** -6 and (d > 0).float().mean().item() < 0.02
    # against the fp32 oracle on 4,096 rows spread over the launch (first panel, interior, the short panels of the
    # last turn of the chip, the very last rows): as close to the unrounded mathematics as the reference's own
    # sequence of bf16 roundings
    rows = torch.cat([torch.arange(0, 1024), torch.arange(200_000, 201_024), torch.arange(481_000, 482_024),
                      torch.arange(M - 1024, M)]).to(DEV)
    xc, gc, bc, w1c, w2c, b1c, b2c = [t.cpu() for t in (x[rows], g, b, w1, w2, b1, b2)]
    rb = lambda t: t.to(torch.bfloat16).float()
    exact = oracle.linear(oracle.swiglu(oracle.linear(oracle.layernorm(xc, gc, bc, 1e-5), w1c, b1c)), w2c, b2c) + xc.float()
    ref = rb(rb(oracle.linear(rb(oracle.swiglu(rb(oracle.linear(rb(oracle.layernorm(xc, gc, bc, 1e-5)), w1c, b1c)))),
                              w2c, b2c)) + xc.float())
    scale = exact.abs().clamp(min=1.0)
    for got in (y[rows], y2[rows]):
        err_us, err_ref = (got.float().cpu() - exact).abs() / scale, (ref - exact).abs() / scale
        assert err_us.max() <= 1.5 * err_ref.max() + 4e-3, (err_us.max(), err_ref.max())
        assert err_us.mean() <= 1.25 * err_ref.mean() + 1e-4, (err_us.mean(), err_ref.mean())
        assert (got.float().cpu() - exact).abs().max() <= 2e-2 * exact.abs().max().clamp(min=1.0)
    n_small = 20000                                                   # fewer rows than the output-panel kernel takes
    y3 = torch.empty(n_small, C, dtype=torch.bfloat16, device=DEV)
    pshattn.linear_bf16(hid[-n_small:], w2, b2, x[-n_small:], y3, None)   # tiled GEMM
    torch.cuda.synchronize()
    d = (y2[-n_small:].float() - y3.float()).abs() / (y3.float().abs() + x[-n_small:].float().abs()).clamp(min=1.0)
    assert d.max().item() <= 2 ** -6 and (d > 0).float().mean().item() < 0.02


def test_staged_weights_are_reused_and_refreshed():
    """Eval-mode forwards under no_grad keep the prepared weights (LayerNorm fold, fragment-major copies) between calls:
    the second call must give the first call's bits, a changed parameter must show in the next output, and a buffer
    that is too small is refused with a message."""
    from flash3dtransformer_amd import layers as L
    from flash3dtransformer_amd.lib import pshattn
    torch.manual_seed(3)
    ln = L.LayerNorm(256).to(DEV).eval()
    lin = L.Linear(256, 768).to(DEV).eval()
    mlp = L.LayerNormMLP(256, 1024).to(DEV).eval()
    wide = L.LayerNormMLP(512, 2048).to(DEV).eval()          # two-kernel path: fc1 fold and the re-laid fc2 weight
    x = torch.randn(40000, 256, device=DEV).to(torch.bfloat16)
    xw = torch.randn(40000, 512, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        ln.weight.add_(torch.randn_like(ln.weight) * 0.1)
        first = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]
        assert lin._staged._key is not None and mlp._staged[0]._key is not None and wide._staged[1]._key is not None
        second = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]
        for a, b in zip(first, second):
            assert torch.equal(a, b)
        # the same layers without staging (training mode prepares per call): identical bits
        for m in (ln, lin, mlp, wide):
            m.train()
        third = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]
        for a, b in zip(first, third):
            assert torch.equal(a, b)
        for m in (ln, lin, mlp, wide):
            m.eval()
        fourth = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]       # staged again after train() / eval()
        for a, b in zip(first, fourth):
            assert torch.equal(a, b)
        # a parameter update (version bump) is seen
        ln.bias.add_(0.5)
        mlp.fc2_bias.add_(1.0)
        wide.fc2_weight.mul_(2.0)
        fifth = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]
        for a, b in zip(first, fifth):
            assert not torch.equal(a, b)
        for m in (ln, lin, mlp, wide):
            m.train()
        sixth = [lin(x, pre_norm=ln), mlp(x, residual=x), wide(xw)]
        for a, b in zip(fifth, sixth):
            assert torch.equal(a, b)
    small = torch.empty(1024, dtype=torch.uint8, device=DEV)
    pshattn.stage_weights(small, False)
    y = torch.empty(64, 768, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(768, 256, dtype=torch.bfloat16, device=DEV)
    g = torch.ones(256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="f3d_stage_weights"):
        pshattn.ln_linear_bf16(x[:64], g, g, 1e-5, w, None, None, y, None)
    pshattn.ln_linear_bf16(x[:64], g, g, 1e-5, w, None, None, y, None)     # the staging ended with the failed call
