"""GPU checks of the dense layers' backward kernels: weight / bias gradient of a linear layer (transposing MFMA kernel),
LayerNorm backward, gated-activation backward.  The reference has no source for these (torch / TransformerEngine
autograd supply them: flash3dxfmr/layers/buck_swin.py:159-163, elem_wise.py:22-26), so the yardstick is torch itself:
fp64 / fp32 torch on the same bf16-rounded inputs.  Tolerances: the weight gradient is an fp32 sum of exact bf16
products, so it matches the fp64 result to fp32 accumulation noise (1e-5 of the largest entry); bf16 outputs carry one
bf16 rounding (2^-8 relative) on top of fp32 arithmetic."""
import numpy as np
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


@pytest.mark.parametrize("M,N,K", [
    (4133, 768, 256),     # qkv of the C=256 block, ragged rows
    (70001, 256, 1024),   # fc2: four k-tiles, slabs of several stages
    (3000, 2048, 256),    # fc1: sixteen n-tiles
    (1000, 96, 32),       # narrow level: one partly filled tile
    (5, 8, 8),            # smaller than one stage
    (64, 136, 264),       # edges in n and k, exactly one stage
    (200000, 256, 256),   # out-projection at a row count that gives every compute unit a slab
])
def test_linear_wgrad_matches_fp64(M, N, K):
    from flash3dtransformer_amd.lib import pshattn
    dy, x = _rand((M, N), M + N, 0.5).to(DEV), _rand((M, K), M + K).to(DEV)
    dw = torch.full((N, K), float("nan"), dtype=torch.float32, device=DEV)
    db = torch.full((N,), float("nan"), dtype=torch.float32, device=DEV)
    pshattn.linear_wgrad_bf16(dy, x, dw, db)
    ref_w = dy.double().t() @ x.double()
    ref_b = dy.double().sum(0)
    assert (dw.double() - ref_w).abs().max().item() <= 1e-5 * ref_w.abs().max().item() + 1e-6
    assert (db.double() - ref_b).abs().max().item() <= 1e-5 * ref_b.abs().max().item() + 1e-6
    # a second call gives the same bits (fixed summation order), accumulate adds to what is there
    dw2 = torch.empty_like(dw)
    pshattn.linear_wgrad_bf16(dy, x, dw2, None)
    assert torch.equal(dw, dw2)
    pshattn.linear_wgrad_bf16(dy, x, dw2, db, accumulate=True)
    assert (dw2.double() - 2 * ref_w).abs().max().item() <= 2e-5 * ref_w.abs().max().item() + 1e-6
    assert (db.double() - 2 * ref_b).abs().max().item() <= 2e-5 * ref_b.abs().max().item() + 1e-6


def test_linear_wgrad_random_shapes():
    """shapes drawn at random (multiples of 8 in n and k, any row count), one of the operands a column slice"""
    from flash3dtransformer_amd.lib import pshattn
    rng = np.random.default_rng(2024)
    for it in range(16):
        M = int(rng.integers(1, 40000))
        N, K = int(rng.integers(1, 80)) * 8, int(rng.integers(1, 80)) * 8
        dy = _rand((M, N + 8), it, 0.5).to(DEV)[:, 8:]
        x = _rand((M, K), 100 + it).to(DEV)
        dw = torch.full((N, K), float("nan"), dtype=torch.float32, device=DEV)
        db = torch.full((N,), float("nan"), dtype=torch.float32, device=DEV)
        pshattn.linear_wgrad_bf16(dy, x, dw, db)
        ref_w, ref_b = dy.double().t() @ x.double(), dy.double().sum(0)
        assert (dw.double() - ref_w).abs().max().item() <= 1e-5 * ref_w.abs().max().item() + 1e-6, (M, N, K)
        assert (db.double() - ref_b).abs().max().item() <= 1e-5 * ref_b.abs().max().item() + 1e-6, (M, N, K)


def test_linear_wgrad_strided_operands_and_empty_input():
    """dy and x as column slices of wider tensors (the three thirds of a qkv gradient); zero rows give zeros"""
    from flash3dtransformer_amd.lib import pshattn
    M, C = 2500, 128
    big_dy, big_x = _rand((M, 3 * C), 1).to(DEV), _rand((M, 2 * C), 2).to(DEV)
    dy, x = big_dy[:, C:2 * C], big_x[:, C:]
    dw = torch.empty(C, C, dtype=torch.float32, device=DEV)
    pshattn.linear_wgrad_bf16(dy, x, dw)
    ref = dy.double().t() @ x.double()
    assert (dw.double() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()
    dw.fill_(7.0)
    db = torch.full((C,), 7.0, dtype=torch.float32, device=DEV)
    pshattn.linear_wgrad_bf16(big_dy[:0, :C], big_x[:0, :C], dw, db)
    assert (dw == 0).all() and (db == 0).all()
    with pytest.raises(RuntimeError):
        pshattn.linear_wgrad_bf16(big_dy[:, :C], big_x[:, :C], torch.empty(C, C + 8, dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("M,C", [(3001, 256), (700, 32), (1030, 64), (4096, 128), (2500, 512), (1, 256)])
@pytest.mark.parametrize("with_res", [False, True])
def test_layernorm_backward_matches_autograd(M, C, with_res):
    from flash3dtransformer_amd.lib import pshattn
    x, dh = _rand((M, C), C + M, 2.0).to(DEV), _rand((M, C), 2 * C + M).to(DEV)
    gamma = (1.0 + 0.2 * _rand((C,), 3).float()).to(torch.bfloat16).to(DEV)
    dres = _rand((M, C), 5).to(DEV) if with_res else None
    dx = torch.empty_like(x)
    dg = torch.full((C,), float("nan"), dtype=torch.float32, device=DEV)
    db = torch.full((C,), float("nan"), dtype=torch.float32, device=DEV)
    pshattn.layernorm_bwd_bf16(x, dh, gamma, dres, dx, dg, db, 1e-5)
    xr = x.float().requires_grad_(True)
    gr = gamma.float().requires_grad_(True)
    br = torch.zeros(C, device=DEV, requires_grad=True)
    y = torch.nn.functional.layer_norm(xr, (C,), gr, br, 1e-5)
    y.backward(dh.float())
    want_dx = xr.grad + (dres.float() if with_res else 0.0)
    err = (dx.float() - want_dx).abs()
    assert (err <= 1e-2 * want_dx.abs().clamp(min=1.0)).all(), err.max().item()
    assert (dg - gr.grad).abs().max().item() <= 1e-4 * max(1.0, gr.grad.abs().max().item())
    assert (db - br.grad).abs().max().item() <= 1e-4 * max(1.0, br.grad.abs().max().item())
    # accumulate, and dx written over dh
    pshattn.layernorm_bwd_bf16(x, dh, gamma, dres, dh, dg, db, 1e-5, accumulate=True)
    assert torch.equal(dh, dx)
    assert (dg - 2 * gr.grad).abs().max().item() <= 2e-4 * max(1.0, gr.grad.abs().max().item())


def test_layernorm_backward_unsupported_width_says_so():
    from flash3dtransformer_amd.lib import pshattn
    C = 96
    x = _rand((10, C), 1).to(DEV)
    f = lambda: torch.empty(C, dtype=torch.float32, device=DEV)
    with pytest.raises(NotImplementedError):
        pshattn.layernorm_bwd_bf16(x, x.clone(), _rand((C,), 2).to(DEV), None, torch.empty_like(x), f(), f())


@pytest.mark.parametrize("M,H", [(3001, 1024), (77, 8), (2048, 128)])
def test_swiglu_backward_matches_autograd(M, H):
    from flash3dtransformer_amd.lib import pshattn
    z, da = _rand((M, 2 * H), M, 2.0).to(DEV), _rand((M, H), H).to(DEV)
    dz, a = torch.empty_like(z), torch.empty_like(da)
    pshattn.swiglu_bwd_bf16(z, da, dz, a)
    zr = z.float().requires_grad_(True)
    ar = torch.nn.functional.silu(zr[:, :H]) * zr[:, H:]
    ar.backward(da.float())
    for got, want in ((a, ar.detach()), (dz, zr.grad)):
        err = (got.float() - want).abs()
        assert (err <= 1e-2 * want.abs().clamp(min=1.0)).all(), err.max().item()
    # in place: dz over z, a over da
    z2, da2 = z.clone(), da.clone()
    pshattn.swiglu_bwd_bf16(z2, da2, z2, da2)
    assert torch.equal(z2, dz) and torch.equal(da2, a)


@pytest.mark.parametrize("M,C,H", [(3001, 256, 1024), (70000, 256, 512), (777, 128, 96), (20000, 128, 512), (256, 256, 32),
                                   (50001, 64, 256), (1000, 64, 32), (90000, 32, 128), (333, 32, 64)])
def test_fused_gate_backward_matches_autograd(M, C, H):
    """fc1 recomputed + da = dy w2 + gate backward in one kernel, against fp32 autograd of a = silu(z1) * z2 with
    z = h w1^T + b1 and the upstream gradient da = dy w2 (bf16 outputs: one rounding on top of fp32 arithmetic)"""
    from flash3dtransformer_amd.lib import pshattn
    h, dy = _rand((M, C), M + C).to(DEV), _rand((M, C), 2 * M + C, 0.5).to(DEV)
    w1, w2 = _rand((2 * H, C), C + H, C ** -0.5).to(DEV), _rand((C, H), C + 2 * H, H ** -0.5).to(DEV)
    b1 = _rand((2 * H,), 7, 0.5).to(DEV)
    dz = torch.full((M, 2 * H), float("nan"), dtype=torch.bfloat16, device=DEV)
    a = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert pshattn.mlp_gate_bwd_bf16(h, dy, w1, b1, w2.t().contiguous(), dz, a)
    zr = (h.float() @ w1.float().t() + b1.float()).requires_grad_(True)
    ar = torch.nn.functional.silu(zr[:, :H]) * zr[:, H:]
    ar.backward(dy.float() @ w2.float())
    for got, want in ((a, ar.detach()), (dz, zr.grad)):
        err = (got.float() - want).abs()
        assert (err <= 2e-2 * want.abs().clamp(min=1.0)).all(), err.max().item()
    # no bias; widths outside the kernel are refused without touching the outputs
    assert pshattn.mlp_gate_bwd_bf16(h, dy, w1, None, w2.t().contiguous(), dz, a)
    zr = (h.float() @ w1.float().t()).requires_grad_(True)
    (torch.nn.functional.silu(zr[:, :H]) * zr[:, H:]).backward(dy.float() @ w2.float())
    err = (dz.float() - zr.grad).abs()
    assert (err <= 2e-2 * zr.grad.abs().clamp(min=1.0)).all(), err.max().item()
    a.fill_(5.0)
    assert not pshattn.mlp_gate_bwd_bf16(h[:, :16].contiguous(), dy[:, :16].contiguous(), w1[:, :16].contiguous(), b1,
                                         w2[:16].t().contiguous(), dz, a)
    assert (a == 5.0).all()


@pytest.mark.parametrize("M,C,hid", [(5000, 64, 256), (3000, 256, 512), (2000, 512, 1024), (1500, 32, 96)])
def test_gated_mlp_layer_gradients_vs_autograd(M, C, hid):
    """LayerNormMLP with the residual taken from its own input (the way a block calls it): every gradient against
    fp32 torch autograd of the same formula.  The gradient tensors handed from kernel to kernel (da, dz, dh) are bf16 as
    in TransformerEngine, 2^-8 relative each, which leaves the parameter gradients within 1e-2 of the largest entry
    (measured: 4e-3 for the LayerNorm weight, under 1e-3 for the fc weights); an indexing mistake would show as O(1)"""
    from flash3dtransformer_amd import layers as L
    torch.manual_seed(11)
    mlp = L.LayerNormMLP(C, hid).to(DEV)   # width 512 takes the three-kernel middle, the others the one-kernel gate backward
    with torch.no_grad():
        for p in mlp.parameters():
            p.add_(torch.randn_like(p) * 0.05)
    x = torch.randn(M, C, device=DEV).to(torch.bfloat16).requires_grad_(True)
    w_out = torch.randn(M, C, device=DEV).to(torch.bfloat16).float()
    y = mlp(x, residual=x)
    (y.float() * w_out).sum().backward()
    ps = {k: v.detach().clone().requires_grad_(True) for k, v in mlp.named_parameters()}
    xr = x.detach().float().requires_grad_(True)
    h = torch.nn.functional.layer_norm(xr, (C,), ps["layer_norm_weight"], ps["layer_norm_bias"], mlp.eps)
    zz = torch.nn.functional.linear(h, ps["fc1_weight"], ps["fc1_bias"])
    yr = torch.nn.functional.linear(torch.nn.functional.silu(zz[:, :hid]) * zz[:, hid:], ps["fc2_weight"], ps["fc2_bias"]) + xr
    (yr * w_out).sum().backward()
    rel = lambda a, b: (a.float() - b).abs().max().item() / max(1e-6, b.abs().max().item())
    assert rel(x.grad, xr.grad) <= 1e-2
    for k, p in mlp.named_parameters():
        assert rel(p.grad, ps[k].grad) <= 1e-2, (k, rel(p.grad, ps[k].grad))
