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
    assert torch.allclose(o.float().cpu(), ref, atol=1e-2 * K ** 0.5, rtol=1e-2)
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
    (2100, 2048, 512, "swiglu", True, False),  # its fc1
    (700, 256, 512, "gelu", False, True),      # fc2 of a C=256 level
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
