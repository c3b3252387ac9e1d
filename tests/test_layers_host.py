"""Host-side logic of the layer modules that needs no GPU: when the bf16 weight copies the kernels read are made anew,
and loading a checkpoint that carries TransformerEngine's per-module `_extra_state` entries."""
import torch

from flash3dtransformer_amd import layers as L
from flash3dtransformer_amd.layers import nn_ops


def test_bf16_weight_copy_follows_the_parameter():
    lin = L.Linear(8, 4)
    w0 = lin._w.get(lin.weight, lin.training)
    # training mode or enabled gradients: every call casts again, so an edit through .data is seen at once
    lin.weight.data.mul_(0)
    assert lin._w.get(lin.weight, lin.training).abs().max().item() == 0 and w0.abs().max().item() > 0
    lin.weight.data.normal_()
    lin.eval()
    with torch.no_grad():
        a = lin._w.get(lin.weight, lin.training)
        assert lin._w.get(lin.weight, lin.training) is a                 # kept between eval-mode forwards
        lin.weight.mul_(2.0)                                             # ordinary in-place edit: version moves
        b = lin._w.get(lin.weight, lin.training)
        assert b is not a and torch.equal(b, lin.weight.to(torch.bfloat16))
        lin.weight.data.zero_()                                          # through .data: invisible ...
        assert lin._w.get(lin.weight, lin.training) is b
        L.refresh_weights(lin)                                           # ... until the copies are dropped
        assert lin._w.get(lin.weight, lin.training).abs().max().item() == 0
        lin.weight.data.fill_(1.0)
        lin.eval()                                                       # a mode call drops them too
        assert lin._w.get(lin.weight, lin.training).min().item() == 1.0
    # a bf16 parameter is handed over itself
    lin16 = L.Linear(8, 4).to(torch.bfloat16).eval()
    with torch.no_grad():
        assert lin16._w.get(lin16.weight, False).data_ptr() == lin16.weight.data_ptr()


def test_load_state_dict_drops_copies_and_accepts_extra_state():
    mlp = L.LayerNormMLP(32, 64).eval()
    with torch.no_grad():
        old = mlp._c[2].get(mlp.fc1_weight, False)
        sd = {k: torch.zeros_like(v) for k, v in mlp.state_dict().items()}
        sd["_extra_state"] = None           # what te.LayerNormMLP stores beside its parameters
        mlp.load_state_dict(sd, strict=True)
        new = mlp._c[2].get(mlp.fc1_weight, False)
    assert new.abs().max().item() == 0 and old.abs().max().item() > 0
    # nested: the reference's MLP wrapper holds te.LayerNormMLP as `.mlp`, te.Linear as the leaf `.proj`
    blk = L.MLP(32, 64)
    sd = dict(blk.state_dict())
    sd["mlp._extra_state"] = torch.zeros(1)
    blk.load_state_dict(sd, strict=True)
    lin = L.Linear(8, 4)
    sd = dict(lin.state_dict())
    sd["_extra_state"] = None
    lin.load_state_dict(sd, strict=True)
    assert isinstance(lin, nn_ops._CachedParamModule)


def test_planner_tables_cover_every_bucket_and_say_so():
    """every plan of bucket_scope.py puts each bucket of the buffer into exactly one scope (reference:
    flash3dxfmr/psh/bucket_scope.py:58-82); the cached table carries that fact for ops that write only covered rows"""
    from flash3dtransformer_amd.psh.bucket_scope import SwinPlan
    for plan, total, bs, sc in (("swin", 8192, 512, 1), ("swin", 16384, 512, 8), ("swin", 5 * 512, 512, 2),
                                ("stride", 12 * 256, 256, 2)):
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            t = SwinPlan(plan, bs, sc, 0 if plan == "swin" else 1).gen_scopes_from_plan(total, torch.device("cpu"))
        assert getattr(t, "covers_all_rows", False)
        ids = t.view(torch.int32).flatten().tolist()
        assert sorted(ids) == list(range(total // bs))


def test_layernorm_qkv_of_a_rank4_embedding_folds_to_four_numbers_per_feature():
    """The identity behind the first block's attention kernel that forms Q, K, V from coordinates (float64, no GPU):
    for x = E c with c = (x, y, z, 1),  W (gamma * (x - mean x) / sqrt(var x + eps) + beta) + b
    = rstd (M c) + b'  with  M = W diag(gamma) E',  b' = W beta + b,  rstd = 1 / sqrt(|L c|^2 + eps),
    E' = E minus its column means and L the upper Cholesky factor of E'^T E' / C -- checked against LayerNorm and the
    two linear layers evaluated as the reference's module sequence writes them (psh_ops.py:64-68, stage.py:94-96)."""
    import torch
    g = torch.Generator().manual_seed(3)
    C, N, eps = 96, 500, 1e-5
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    ew, eb, gamma, beta, w, b = rnd(C, 3), rnd(C), 1 + 0.2 * rnd(C), 0.3 * rnd(C), rnd(3 * C, C) / C ** 0.5, rnd(3 * C)
    c3 = rnd(N, 3) * torch.tensor([40.0, 40.0, 3.0], dtype=torch.float64)
    x = torch.nn.functional.linear(c3, ew, eb)
    want = torch.nn.functional.linear(torch.nn.functional.layer_norm(x, (C,), gamma, beta, eps), w, b)
    E = torch.cat([ew, eb[:, None]], 1)
    Ep = E - E.mean(0, keepdim=True)
    L = torch.linalg.cholesky(Ep.T @ Ep / C).T
    M, bp = (w * gamma[None, :]) @ Ep, w @ beta + b
    c = torch.cat([c3, torch.ones(N, 1, dtype=torch.float64)], 1)
    rstd = 1.0 / torch.sqrt((c @ L.T).pow(2).sum(1, keepdim=True) + eps)
    got = rstd * (c @ M.T) + bp
    assert (got - want).abs().max().item() <= 1e-9 * max(1.0, want.abs().max().item())
    # a dropped mean, a missing gamma or the uncentred Gram matrix are not the same function
    assert ((rstd * (c @ ((w * gamma[None, :]) @ E).T) + bp) - want).abs().max().item() > 1e-3
    assert ((rstd * (c @ (w @ Ep).T) + bp) - want).abs().max().item() > 1e-3
