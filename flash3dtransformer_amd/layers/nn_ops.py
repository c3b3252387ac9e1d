"""HIP-backed building blocks of the layer API: Linear, LayerNorm, LayerNormMLP and the fused
norm + activation used around pooling.  Parameters are ordinary nn.Parameters (fp32 by default, so
a checkpoint of the reference's torch / TransformerEngine modules loads by name); the kernels run on
bf16 copies: made anew on every training-mode or gradient-enabled forward, kept between eval-mode forwards
under no_grad (see _Bf16Cache for when such a copy is dropped).

Forward runs on the HIP kernels.  So does the backward of Linear (optionally with a LayerNorm in front and a
residual), LayerNorm and the gated LayerNormMLP on bf16 activations: weight / bias gradients from the transposing
MFMA kernel, input gradients from the forward linear kernels on the transposed weight, LayerNorm and gate backward
as one pass each (`_LinearGrad`, `_LayerNormGrad`, `_GatedMLPGrad`).  What those kernels do not cover (other
activations inside a Linear, widths that are not a multiple of 8, LayerNorm widths other than 32 ... 512, fp32
activations) differentiates a torch restatement of the same formula on the GPU instead (`_TorchBackward`), which
is where the reference gets all of it (torch / TransformerEngine autograd).  The forward value never comes from a
restatement.
"""
import math
import weakref

import torch
from torch import nn

from ..lib import pshattn


class _TorchBackward(torch.autograd.Function):
    """Output of a HIP forward kernel whose gradient is taken through `ref_fn`, a torch restatement of the op
    over the same inputs (None entries are passed through).  Inputs are re-read in fp32 for the backward."""

    @staticmethod
    def forward(ctx, out, ref_fn, *inputs):
        ctx.ref_fn = ref_fn
        ctx.is_tensor = [isinstance(t, torch.Tensor) for t in inputs]
        ctx.save_for_backward(*[t for t in inputs if isinstance(t, torch.Tensor)])
        return out.view_as(out)

    @staticmethod
    def backward(ctx, grad):
        saved = list(ctx.saved_tensors)
        ins, leaves = [], []
        for is_t in ctx.is_tensor:
            if not is_t:
                ins.append(None)
                continue
            t = saved.pop(0)
            leaf = t.detach().float().requires_grad_(True)
            ins.append(leaf)
            leaves.append((leaf, t))
        with torch.enable_grad():
            y = ctx.ref_fn(*ins)
            grads = torch.autograd.grad(y, [l for l, _ in leaves], grad.float().reshape(y.shape), allow_unused=True)
        out, gi = [None, None], iter(zip(grads, leaves))
        for is_t in ctx.is_tensor:
            if not is_t:
                out.append(None)
                continue
            g, (_, orig) = next(gi)
            out.append(None if g is None or not orig.requires_grad else g.to(orig.dtype).reshape(orig.shape))
        return tuple(out)


def torch_backward(out: torch.Tensor, ref_fn, *inputs) -> torch.Tensor:
    """`out` = value from the HIP kernels; gradients flow to `inputs` through `ref_fn(*inputs)`"""
    if torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in inputs):
        return _TorchBackward.apply(out, ref_fn, *inputs)
    return out


def _act_ref(z: torch.Tensor, act):
    if act is None:
        return z
    if act == "swiglu":
        h = z.shape[-1] // 2
        return torch.nn.functional.silu(z[..., :h]) * z[..., h:]
    return {"gelu": torch.nn.functional.gelu, "relu": torch.relu, "silu": torch.nn.functional.silu}[act](z)


def _linear_ref(act, eps):
    """torch restatement of Linear.forward: (x, w, b, residual, ln_w, ln_b) -> y"""
    def ref(x, w, b, residual, ln_w, ln_b):
        h = x if ln_w is None else torch.nn.functional.layer_norm(x, (x.shape[-1],), ln_w, ln_b, eps)
        y = _act_ref(torch.nn.functional.linear(h, w, b), act)
        return y if residual is None else y + residual
    return ref


class _Bf16Cache:
    """bf16 device copy of a parameter for the kernels.

    A parameter that already is bf16 is handed over as it is (always current).  An fp32 master parameter is cast
    again on every forward while gradients are enabled or the owning module is in training mode, which is what the
    reference's autocast forward does; only an eval-mode forward under no_grad keeps the copy between calls.  That
    copy is dropped when the parameter's address or version changes, on train() / eval(), on load_state_dict and by
    refresh_weights().  In-place edits through `.data` leave address and version alone: after one of those in eval
    mode call refresh_weights(model)."""

    def __init__(self):
        self._key = None
        self._val = None

    def clear(self):
        self._key = self._val = None

    def get(self, p: torch.Tensor, training: bool = False) -> torch.Tensor:
        if p is None:
            return None
        if p.dtype == torch.bfloat16 and p.is_contiguous():
            return p.detach()
        if training or torch.is_grad_enabled():
            self.clear()
            return p.detach().to(torch.bfloat16).contiguous()
        key = (p.data_ptr(), p._version, p.dtype, p.device)
        if key != self._key:
            self._val = p.detach().to(torch.bfloat16).contiguous()
            self._key = key
        return self._val


class _StagedWeights:
    """Device buffer in which a dense kernel keeps the weights it prepares per call (LayerNorm folded into the weight
    and bias, fragment-major copies) between eval-mode forwards under no_grad.  The buffer is current while the bf16
    tensors it was made from are the same storage at the same version (the entry holds them, so their memory cannot
    be handed out again meanwhile); dropped together with the bf16 copies (train() / eval(), load_state_dict,
    refresh_weights())."""

    def __init__(self):
        self._key = None
        self._src = None
        self._buf = None

    def clear(self):
        self._key = self._src = None

    def arm(self, training: bool, rows: int, cols: int, *tensors, tag=None):
        """call right before the dense op: stages the buffer for it (no-op while weights may change)"""
        if training or torch.is_grad_enabled():
            self.clear()
            return
        live = [t for t in tensors if t is not None]
        key = (tag, rows, cols) + tuple((t.data_ptr(), t._version, tuple(t.shape)) for t in live)
        need = 3 * rows * cols + 4 * rows + 2 * cols + 512
        dev = live[0].device
        if self._buf is None or self._buf.numel() < need or self._buf.device != dev:
            self._buf = torch.empty(need, dtype=torch.uint8, device=dev)
            self._key = None
        ready = key == self._key
        pshattn.stage_weights(self._buf, ready)
        self._key, self._src = key, live


class _DerivedCache(_Bf16Cache):
    """something computed from several parameters (a folded table), kept while their addresses and versions stay;
    dropped with the owning module's bf16 copies (train() / eval(), load_state_dict, refresh_weights())"""

    def get_or_build(self, params, extra, build):
        key = tuple(None if p is None else (p.data_ptr(), p._version, p.dtype, p.device) for p in params) + tuple(extra)
        if key != self._key:
            self._val = build()
            self._key = key if self._val is not None else None
        return self._val


class _CachedParamModule(nn.Module):
    """nn.Module whose kernels read bf16 copies of its parameters (`_Bf16Cache` attributes or lists of them)"""

    def _bf16_caches(self):
        for v in self.__dict__.values():
            if isinstance(v, (_Bf16Cache, _StagedWeights)):
                yield v
            elif isinstance(v, (list, tuple)):
                for c in v:
                    if isinstance(c, (_Bf16Cache, _StagedWeights)):
                        yield c

    def refresh_weights(self):
        for c in self._bf16_caches():
            c.clear()

    def train(self, mode: bool = True):
        self.refresh_weights()
        return super().train(mode)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # TransformerEngine modules of the reference store one `_extra_state` entry each (fp8 recipe state, of no use
        # to a bf16 kernel): dropped, so that such a checkpoint loads with strict=True
        state_dict.pop(prefix + "_extra_state", None)
        self.refresh_weights()
        return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)


def refresh_weights(module: nn.Module) -> None:
    """Drops every cached bf16 weight copy under `module`; needed only after in-place edits through `.data`
    (EMA swaps, manual re-initialisation) on a model that stays in eval mode under no_grad."""
    for m in module.modules():
        if isinstance(m, _CachedParamModule):
            m.refresh_weights()
        _BN_AFFINE.pop(m, None)


def as_bf16_2d(x: torch.Tensor) -> torch.Tensor:
    if x.dtype != torch.bfloat16:
        x = x.to(torch.bfloat16)
    if x.stride(-1) != 1:
        x = x.contiguous()
    return x


def _grad_out(g, like):
    """a gradient tensor in the dtype and shape autograd expects for `like`"""
    return g.to(like.dtype).reshape(like.shape)


def _transposed_bf16(w16: torch.Tensor) -> torch.Tensor:
    return w16.t().contiguous()


def _ln_backward(x2, dh, g16, dres, eps, need_dx=True):
    """(dx bf16, dgamma fp32, dbeta fp32) of LayerNorm at rows x2 for the output gradient dh (+ dres added to dx)"""
    c = x2.shape[1]
    dx = torch.empty(x2.shape, dtype=torch.bfloat16, device=x2.device)
    dg = torch.empty(c, dtype=torch.float32, device=x2.device)
    db = torch.empty(c, dtype=torch.float32, device=x2.device)
    pshattn.layernorm_bwd_bf16(x2, dh, g16, dres, dx, dg, db, eps)
    return dx, dg, db


class _LayerNormGrad(torch.autograd.Function):
    """y = LayerNorm(x) computed by the HIP forward; gradient by f3d_layernorm_bwd_bf16"""

    @staticmethod
    def forward(ctx, y, x, weight, bias, eps, g16):
        ctx.save_for_backward(x, weight, bias, g16)
        ctx.eps = eps
        return y.view_as(y)

    @staticmethod
    def backward(ctx, dy):
        x, weight, bias, g16 = ctx.saved_tensors
        dx, dg, db = _ln_backward(as_bf16_2d(x), as_bf16_2d(dy.reshape(x.shape)), g16, None, ctx.eps)
        return (None, _grad_out(dx, x) if ctx.needs_input_grad[1] else None,
                _grad_out(dg, weight) if ctx.needs_input_grad[2] else None,
                _grad_out(db, bias) if bias is not None and ctx.needs_input_grad[3] else None, None, None)


class _LinearGrad(torch.autograd.Function):
    """y = [LayerNorm](x) @ w.T + b (+ residual) computed by the HIP forward; gradient by the HIP backward kernels:
    dw, db = f3d_linear_wgrad_bf16(dy, h), dh = f3d_linear_bf16(dy, w.T), then LayerNorm backward if there is one"""

    @staticmethod
    def forward(ctx, y, x, weight, bias, residual, ln_w, ln_b, eps, w16, g16, b16):
        ctx.save_for_backward(x, weight, bias, residual, ln_w, ln_b, w16, g16, b16)
        ctx.eps = eps
        return y.view_as(y)

    @staticmethod
    def backward(ctx, dy):
        x, weight, bias, residual, ln_w, ln_b, w16, g16, b16 = ctx.saved_tensors
        need = ctx.needs_input_grad
        dy2 = as_bf16_2d(dy)
        x2 = as_bf16_2d(x)
        m, k = x2.shape
        n = dy2.shape[1]
        dev = x2.device
        if ln_w is not None:
            h = torch.empty(m, k, dtype=torch.bfloat16, device=dev)
            pshattn.layernorm_bf16(x2.contiguous(), g16, b16, h, ctx.eps)
        else:
            h = x2
        dw = db = dx = dg = dbeta = None
        if need[2] or (bias is not None and need[3]):
            dw = torch.empty(n, k, dtype=torch.float32, device=dev)
            db = torch.empty(n, dtype=torch.float32, device=dev) if bias is not None else None
            pshattn.linear_wgrad_bf16(dy2, h, dw, db)
        if need[1] or (ln_w is not None and (need[5] or need[6])):
            dh = torch.empty(m, k, dtype=torch.bfloat16, device=dev)
            pshattn.linear_bf16(dy2, _transposed_bf16(w16), None, None, dh, None)
            if ln_w is not None:
                dx, dg, dbeta = _ln_backward(x2, dh, g16, None, ctx.eps)
            else:
                dx = dh
        return (None, _grad_out(dx, x) if need[1] else None, _grad_out(dw, weight) if need[2] else None,
                _grad_out(db, bias) if bias is not None and need[3] else None,
                _grad_out(dy2, residual) if residual is not None and need[4] else None,
                _grad_out(dg, ln_w) if ln_w is not None and need[5] else None,
                _grad_out(dbeta, ln_b) if ln_b is not None and need[6] else None, None, None, None, None)


class _GatedMLPGrad(torch.autograd.Function):
    """y = fc2(silu(z1) * z2) + b2 (+ residual), [z1 | z2] = LayerNorm(x) @ w1.T + b1, computed by the HIP forward.
    The backward recomputes LayerNorm(x) and z (the forward keeps neither), then runs
    da = dy @ w2, (dz, a) = gate backward (these three in one kernel at widths 32 to 256), dw2 = dy.T a, dw1 = dz.T h,
    dh = dz @ w1, LayerNorm backward.
    When the residual is the layer's own input, its gradient dy is added to dx inside the LayerNorm backward."""

    @staticmethod
    def forward(ctx, y, x, residual, ln_w, ln_b, w1, b1, w2, b2, eps, g16, be16, w1_16, b1_16, w2_16):
        ctx.save_for_backward(x, residual, ln_w, ln_b, w1, b1, w2, b2, g16, be16, w1_16, b1_16, w2_16)
        ctx.eps = eps
        return y.view_as(y)

    @staticmethod
    def backward(ctx, dy):
        x, residual, ln_w, ln_b, w1, b1, w2, b2, g16, be16, w1_16, b1_16, w2_16 = ctx.saved_tensors
        need = ctx.needs_input_grad
        dy2 = as_bf16_2d(dy)
        x2 = as_bf16_2d(x).contiguous()
        m, c = x2.shape
        hid = w2_16.shape[1]
        dev = x2.device
        bf = dict(dtype=torch.bfloat16, device=dev)
        f32 = dict(dtype=torch.float32, device=dev)
        h = torch.empty(m, c, **bf)
        pshattn.layernorm_bf16(x2, g16, be16, h, ctx.eps)
        dz, a = torch.empty(m, 2 * hid, **bf), torch.empty(m, hid, **bf)
        w2t = _transposed_bf16(w2_16)
        # one kernel where it exists (fc1 recomputed, da = dy @ w2 and the gate backward; neither z nor da is stored) ...
        if not pshattn.mlp_gate_bwd_bf16(h, dy2, w1_16, b1_16, w2t, dz, a):
            # ... otherwise fc1, da, then the gate backward in place (dz over z, a over da)
            pshattn.linear_bf16(h, w1_16, b1_16, None, dz, None)
            pshattn.linear_bf16(dy2, w2t, None, None, a, None)
            pshattn.swiglu_bwd_bf16(dz, a, dz, a)
        dw2, db2 = torch.empty(c, hid, **f32), torch.empty(c, **f32)
        pshattn.linear_wgrad_bf16(dy2, a, dw2, db2)
        dw1, db1 = torch.empty(2 * hid, c, **f32), torch.empty(2 * hid, **f32)
        pshattn.linear_wgrad_bf16(dz, h, dw1, db1)
        pshattn.linear_bf16(dz, _transposed_bf16(w1_16), None, None, h, None)     # h <- dh
        # a residual that is the input itself: one gradient tensor for both routes
        shared = (residual is not None and need[1] and need[2] and residual.data_ptr() == x.data_ptr()
                  and residual.shape == x.shape and residual.dtype == x.dtype and residual.stride() == x.stride())
        dx, dg, dbeta = _ln_backward(x2, h, g16, dy2 if shared else None, ctx.eps)
        d_res = None
        if residual is not None and need[2] and not shared:
            d_res = _grad_out(dy2, residual)
        return (None, _grad_out(dx, x) if need[1] else None, d_res,
                _grad_out(dg, ln_w) if need[3] else None, _grad_out(dbeta, ln_b) if ln_b is not None and need[4] else None,
                _grad_out(dw1, w1) if need[5] else None, _grad_out(db1, b1) if b1 is not None and need[6] else None,
                _grad_out(dw2, w2) if need[7] else None, _grad_out(db2, b2) if b2 is not None and need[8] else None,
                None, None, None, None, None, None)


def _grad_wanted(*tensors) -> bool:
    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def _hip_backward_covers(x: torch.Tensor, *widths) -> bool:
    """bf16 activations on the GPU and widths the backward kernels take"""
    return x.is_cuda and x.dtype == torch.bfloat16 and all(w % 8 == 0 for w in widths)


class Linear(_CachedParamModule):
    """y = act(x W^T + b) (+ residual) on MFMA; parameter names match torch.nn.Linear / te.Linear"""

    def __init__(self, in_features: int, out_features: int, bias: bool = True):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        self.bias = nn.Parameter(torch.empty(out_features)) if bias else None
        self._w, self._b = _Bf16Cache(), _Bf16Cache()
        self._staged = _StagedWeights()
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            bound = 1.0 / math.sqrt(self.in_features)
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x: torch.Tensor, residual: torch.Tensor = None, act=None, out: torch.Tensor = None,
                pre_norm=None):
        """`pre_norm`: a LayerNorm-like module (weight, bias, eps) applied to x inside the same kernel"""
        lead = x.shape[:-1]
        x2 = as_bf16_2d(x.reshape(-1, x.shape[-1]))
        n_out = self.out_features // 2 if act == "swiglu" else self.out_features
        y = out if out is not None else torch.empty(x2.shape[0], n_out, dtype=torch.bfloat16, device=x.device)
        r2 = None if residual is None else as_bf16_2d(residual.reshape(-1, n_out))
        w16, b16 = self._w.get(self.weight, self.training), self._b.get(self.bias, self.training)
        g = b = None
        if pre_norm is not None:
            g, b = norm_params_bf16(pre_norm)
            if isinstance(pre_norm, LayerNorm):     # its bf16 copies are kept between calls, a torch norm's are not
                self._staged.arm(self.training or pre_norm.training, self.out_features, self.in_features, w16, b16, g, b,
                                 tag=("ln", float(pre_norm.eps)))
            pshattn.ln_linear_bf16(x2, g, b, pre_norm.eps, w16, b16, r2, y, act)
        else:
            if self.in_features > 512:     # long inner dimension: the output-panel kernel re-lays the weight
                self._staged.arm(self.training, self.out_features, self.in_features, w16, b16, tag="ys")
            pshattn.linear_bf16(x2, w16, b16, r2, y, act)
        ln_w = None if pre_norm is None else pre_norm.weight
        ln_b = None if pre_norm is None else pre_norm.bias
        eps = 0.0 if pre_norm is None else pre_norm.eps
        x_in = x.reshape(-1, x.shape[-1])
        res_in = None if residual is None else residual.reshape(-1, n_out)
        if not _grad_wanted(x_in, self.weight, self.bias, res_in, ln_w, ln_b):
            return y.view(*lead, n_out)
        if act is None and _hip_backward_covers(x_in, self.in_features, self.out_features) and (
                pre_norm is None or (self.in_features in pshattn.LN_BWD_WIDTHS and g is not None)):
            out = _LinearGrad.apply(y, x_in, self.weight, self.bias, res_in, ln_w, ln_b, eps, w16, g, b)
        else:
            out = torch_backward(y, _linear_ref(act, eps), x_in, self.weight, self.bias, res_in, ln_w, ln_b)
        return out.view(*lead, n_out)

    def embedded(self, emb: "CoordEmbedding", pre_norm):
        """forward(emb.materialize(), pre_norm=pre_norm) without storing the embedding: inference only"""
        if isinstance(pre_norm, LayerNorm) and self.in_features in CoordEmbedding.EMBED_WIDTHS and self.out_features % 32 == 0:
            w16, b16 = self._w.get(self.weight, self.training), self._b.get(self.bias, self.training)
            g, b = norm_params_bf16(pre_norm)
            y = torch.empty(emb.shape[0], self.out_features, dtype=torch.bfloat16, device=emb.device)
            self._staged.arm(self.training or pre_norm.training, self.out_features, self.in_features, w16, b16, g, b,
                             tag=("ln", float(pre_norm.eps)))
            if pshattn.embed_ln_linear_bf16(emb.coord, emb.table(), g, b, pre_norm.eps, w16, b16, y):
                return y
        return self.forward(emb.materialize(), pre_norm=pre_norm)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}"


class CoordEmbedding:
    """The coordinate embedding `lin(coord.bf16())` of PSH-scattered points that has NOT been stored: at inference the
    first block forms it inside its own kernels (LayerNorm + QKV; out-projection + MLP) from the coordinates, and the
    [rows, channels] tensor is neither written nor read.  Anything else calls materialize()."""
    EMBED_WIDTHS = (32, 64, 128, 256)

    def __init__(self, coord: torch.Tensor, lin: "Linear"):
        self.coord, self.lin = coord, lin
        self.shape = torch.Size((coord.shape[0], lin.out_features))
        self.dtype, self.device = torch.bfloat16, coord.device
        self._tensor = None

    def dim(self):
        return 2

    def table(self) -> torch.Tensor:
        """[channels, 8] bf16 rows (wx, wy, wz, b, 0, 0, 0, 0), rebuilt when the layer's parameters change"""
        lin = self.lin
        key = (lin.weight._version, lin.weight.data_ptr(), None if lin.bias is None else (lin.bias._version, lin.bias.data_ptr()))
        cached = getattr(lin, "_embed_table", None)
        if cached is None or cached[0] != key or cached[1].device != self.device:
            cached = (key, pshattn.embed_table(lin.weight, lin.bias))
            lin._embed_table = cached
        return cached[1]

    def materialize(self) -> torch.Tensor:
        if self._tensor is None:
            lin = self.lin
            out = torch.empty(self.shape[0], lin.out_features, dtype=torch.bfloat16, device=self.device)
            pshattn.coord_embed_bf16(self.coord, lin._w.get(lin.weight, lin.training), lin._b.get(lin.bias, lin.training), out)
            self._tensor = out
        return self._tensor


def materialize(feat):
    """a feature tensor as a tensor (a CoordEmbedding is stored first)"""
    return feat.materialize() if isinstance(feat, CoordEmbedding) else feat


class LayerNorm(_CachedParamModule):
    """LayerNorm over the last axis with fp32 statistics; parameter names match nn.LayerNorm / te.LayerNorm"""

    def __init__(self, normalized_shape: int, eps: float = 1e-5):
        super().__init__()
        self.normalized_shape, self.eps = int(normalized_shape), eps
        self.weight = nn.Parameter(torch.ones(self.normalized_shape))
        self.bias = nn.Parameter(torch.zeros(self.normalized_shape))
        self._w, self._b = _Bf16Cache(), _Bf16Cache()

    def forward(self, x: torch.Tensor):
        x2 = as_bf16_2d(x.reshape(-1, x.shape[-1])).contiguous()
        y = torch.empty_like(x2)
        g16 = self._w.get(self.weight, self.training)
        pshattn.layernorm_bf16(x2, g16, self._b.get(self.bias, self.training), y, self.eps)
        x_in = x.reshape(-1, x.shape[-1])
        if _grad_wanted(x_in, self.weight, self.bias) and _hip_backward_covers(x_in) \
                and self.normalized_shape in pshattn.LN_BWD_WIDTHS:
            return _LayerNormGrad.apply(y, x_in, self.weight, self.bias, self.eps, g16).view(x.shape)
        eps = self.eps
        ref = lambda xx, w, b: torch.nn.functional.layer_norm(xx, (xx.shape[-1],), w, b, eps)
        return torch_backward(y, ref, x_in, self.weight, self.bias).view(x.shape)


FUSABLE_LN_WIDTHS = (32, 64, 128, 256, 512)
FUSED_MLP_WIDTHS = (32, 64, 128, 256)      # widths the one-kernel gated MLP covers (32 / 64: while the weights fit into LDS)
PROJ_MLP_WIDTHS = (32, 64, 128, 256)       # widths at which it also takes the out-projection and its residual in front


def is_fusable_layernorm(norm, width: int) -> bool:
    """LayerNorm over one axis with affine weights, at a width the fused LayerNorm+Linear kernel covers"""
    if width not in FUSABLE_LN_WIDTHS:
        return False
    if isinstance(norm, LayerNorm):
        return True
    return isinstance(norm, nn.LayerNorm) and norm.elementwise_affine and len(norm.normalized_shape) == 1


def norm_params_bf16(norm):
    if isinstance(norm, LayerNorm):
        return norm._w.get(norm.weight, norm.training), norm._b.get(norm.bias, norm.training)
    b = None if norm.bias is None else norm.bias.detach().to(torch.bfloat16).contiguous()
    return norm.weight.detach().to(torch.bfloat16).contiguous(), b


def apply_norm(norm: nn.Module, x: torch.Tensor) -> torch.Tensor:
    """Runs a norm module the user passed as a callable: LayerNorm flavours go to the HIP kernel,
    eval-mode BatchNorm1d folds into one affine kernel, anything else runs as given."""
    if isinstance(norm, LayerNorm):
        return norm(x)
    if isinstance(norm, nn.LayerNorm) and norm.elementwise_affine and len(norm.normalized_shape) == 1 \
            and x.is_cuda and x.shape[-1] % 8 == 0:
        x2 = as_bf16_2d(x.reshape(-1, x.shape[-1])).contiguous()
        y = torch.empty_like(x2)
        b = None if norm.bias is None else norm.bias.detach().to(torch.bfloat16)
        g16 = norm.weight.detach().to(torch.bfloat16)
        pshattn.layernorm_bf16(x2, g16, b, y, norm.eps)
        x_in = x.reshape(-1, x.shape[-1])
        if _grad_wanted(x_in, norm.weight, norm.bias) and _hip_backward_covers(x_in) \
                and x.shape[-1] in pshattn.LN_BWD_WIDTHS:
            return _LayerNormGrad.apply(y, x_in, norm.weight, norm.bias, norm.eps, g16).view(x.shape)
        eps = norm.eps
        ref = lambda xx, w, bb: torch.nn.functional.layer_norm(xx, (xx.shape[-1],), w, bb, eps)
        return torch_backward(y, ref, x.reshape(-1, x.shape[-1]), norm.weight, norm.bias).view(x.shape)
    return norm(x)


_BN_AFFINE = weakref.WeakKeyDictionary()      # eval-mode BatchNorm1d -> (key, scale, shift)


def _bn_affine(bn: nn.BatchNorm1d):
    """scale and shift of an eval-mode BatchNorm1d (running statistics folded with the affine parameters), fp32; kept per
    module while its statistics and parameters stay at the same address and version"""
    src = [bn.running_mean, bn.running_var] + ([bn.weight, bn.bias] if bn.affine else [])
    key = (bn.eps,) + tuple((t.data_ptr(), t._version) for t in src)
    hit = _BN_AFFINE.get(bn)
    if hit is not None and hit[0] == key and not torch.is_grad_enabled():
        return hit[1], hit[2]
    rstd = torch.rsqrt(bn.running_var.float() + bn.eps)
    g = bn.weight.detach().float() if bn.affine else torch.ones_like(rstd)
    b = bn.bias.detach().float() if bn.affine else torch.zeros_like(rstd)
    scale, shift = (g * rstd).contiguous(), (b - bn.running_mean.float() * g * rstd).contiguous()
    _BN_AFFINE[bn] = (key, scale, shift)
    return scale, shift


_ACT_NAMES = {nn.GELU: "gelu", nn.ReLU: "relu", nn.SiLU: "silu"}


def apply_norm_act(norm, act, x: torch.Tensor) -> torch.Tensor:
    """norm followed by activation as used around pooling / unpooling (hourglass.py:104-109, 152-159
    of the reference).  Eval-mode BatchNorm1d + GELU/ReLU/SiLU is one fused kernel."""
    act_name = None
    if act is not None:
        act_name = _ACT_NAMES.get(type(act))
        if isinstance(act, nn.GELU) and act.approximate != "none":
            act_name = None
    fusable_act = act is None or act_name is not None
    if isinstance(norm, nn.BatchNorm1d) and not norm.training and norm.track_running_stats and fusable_act \
            and x.is_cuda and x.shape[-1] % 8 == 0:
        scale, shift = _bn_affine(norm)
        x2 = as_bf16_2d(x).contiguous()
        y = torch.empty_like(x2)
        pshattn.affine_act_bf16(x2, scale, shift, y, act_name)
        mean, var, bn_eps = norm.running_mean, norm.running_var, norm.eps

        def ref(xx, w, b):   # eval-mode BatchNorm1d (running statistics are constants) then the activation
            return _act_ref(torch.nn.functional.batch_norm(xx, mean.float(), var.float(), w, b, False, 0.0, bn_eps), act_name)
        return torch_backward(y, ref, x, norm.weight if norm.affine else None, norm.bias if norm.affine else None)
    if norm is not None:
        x = apply_norm(norm, x)
    if act is not None:
        x = act(x)
    return x


def fused_row_norm(norm, act, x: torch.Tensor):
    """What the pooling / unpooling kernels can apply to their rows in place of `apply_norm_act(norm, act, .)` on the
    tensor afterwards: (descriptor, activation name) or None.  Inference only (no autograd graph), bf16 rows on the
    GPU: a LayerNorm over the channels without activation at the widths 32 .. 512, or an eval-mode BatchNorm1d with
    no activation / GELU / ReLU / SiLU at a multiple of 8 channels."""
    if torch.is_grad_enabled() or norm is None or not x.is_cuda or x.dtype != torch.bfloat16:
        return None
    c = x.shape[-1]
    if act is None and is_fusable_layernorm(norm, c):
        g, b = norm_params_bf16(norm)
        return ("layer", g, b, norm.eps), None
    if isinstance(norm, nn.BatchNorm1d) and not norm.training and norm.track_running_stats and c % 8 == 0:
        act_name = None
        if act is not None:
            act_name = _ACT_NAMES.get(type(act))
            if act_name is None or (isinstance(act, nn.GELU) and act.approximate != "none"):
                return None
        scale, shift = _bn_affine(norm)
        return ("affine", scale, shift), act_name
    return None


class LayerNormMLP(_CachedParamModule):
    """LayerNorm -> fc1 -> activation -> fc2, the role te.LayerNormMLP plays in the reference
    (flash3dxfmr/layers/elem_wise.py:22-26).  Parameter names follow TransformerEngine
    (layer_norm_weight/bias, fc1_weight/bias, fc2_weight/bias).  activation "swiglu": fc1 has
    2 * ffn_hidden_size outputs and the hidden state is silu(h[:, :ffn]) * h[:, ffn:]; "gelu": plain
    fc1 -> GELU -> fc2."""

    def __init__(self, hidden_size: int, ffn_hidden_size: int, activation: str = "swiglu", eps: float = 1e-5,
                 fused: bool = None):
        super().__init__()
        # fused: run the whole gated MLP as one kernel where one exists (widths 32 / 64 / 128 / 256): the hidden
        # activations [rows, ffn_hidden_size] are then never allocated.  None (default): where it is the faster path on
        # MI355X (measured against LayerNorm+fc1+gate followed by fc2+residual, hidden = 4 x width: widths 32 and 64
        # at every row count, 27 % faster at 3 k rows and 2.2 to 2.9 x at 0.5 to 1 M rows; width 128 at every row
        # count, 19 to 41 % faster; width 256 from 32 k rows up, 6 to 23 % faster, and 11 % slower at 16 k rows)
        self.fused = fused
        assert activation in ("swiglu", "gelu")
        self.hidden_size, self.ffn_hidden_size, self.activation, self.eps = hidden_size, ffn_hidden_size, activation, eps
        fc1_out = 2 * ffn_hidden_size if activation == "swiglu" else ffn_hidden_size
        self.layer_norm_weight = nn.Parameter(torch.ones(hidden_size))
        self.layer_norm_bias = nn.Parameter(torch.zeros(hidden_size))
        self.fc1_weight = nn.Parameter(torch.empty(fc1_out, hidden_size))
        self.fc1_bias = nn.Parameter(torch.zeros(fc1_out))
        self.fc2_weight = nn.Parameter(torch.empty(hidden_size, ffn_hidden_size))
        self.fc2_bias = nn.Parameter(torch.zeros(hidden_size))
        nn.init.normal_(self.fc1_weight, std=0.023)
        nn.init.normal_(self.fc2_weight, std=0.023)
        self._c = [_Bf16Cache() for _ in range(6)]
        self._staged = [_StagedWeights(), _StagedWeights()]      # fused kernel / fc1 of the two-kernel path; fc2

    def after_projection(self, a: torch.Tensor, proj: "Linear", x: torch.Tensor):
        """x1 = proj(a) + x;  x1 + MLP(x1) in one kernel (x1 is never stored): the second half of a transformer block
        (flash3dxfmr/layers/stage.py:92-102) at inference.  a, x [rows, hidden_size] bf16 (x may be a CoordEmbedding: the
        kernel then forms the block input from the coordinates).  Returns None where that
        kernel does not apply (autograd on, other widths or activation, few rows): the caller then runs `proj` with its
        residual and this module."""
        if not self.takes_projection(a.shape[0]) or proj.in_features != self.hidden_size \
                or proj.out_features != self.hidden_size or not a.is_cuda or a.dtype != torch.bfloat16 \
                or x.dtype != torch.bfloat16:
            return None
        lazy = x if isinstance(x, CoordEmbedding) else None
        a2 = a.reshape(-1, self.hidden_size)
        x2 = None if lazy is not None else x.reshape(-1, self.hidden_size)
        if a2.stride(1) != 1 or (x2 is not None and x2.stride(1) != 1):
            return None
        params = (self.layer_norm_weight, self.layer_norm_bias, self.fc1_weight, self.fc1_bias, self.fc2_weight, self.fc2_bias)
        g16, be16, w1_16, b1_16, w2_16, b2_16 = (c.get(p, self.training) for c, p in zip(self._c, params))
        wp16, bp16 = proj._w.get(proj.weight, proj.training), proj._b.get(proj.bias, proj.training)
        y = torch.empty(a2.shape[0], self.hidden_size, dtype=torch.bfloat16, device=a.device)
        self._staged[0].arm(self.training, w1_16.shape[0], self.hidden_size, g16, be16, w1_16, b1_16, w2_16, b2_16,
                            tag=("mlp", float(self.eps)))
        if lazy is not None:
            ok = pshattn.embed_proj_ln_mlp_swiglu_bf16(a2, wp16, bp16, lazy.coord, lazy.table(), g16, be16, self.eps, w1_16,
                                                       b1_16, w2_16, b2_16, y)
        else:
            ok = pshattn.proj_ln_mlp_swiglu_bf16(a2, wp16, bp16, x2, g16, be16, self.eps, w1_16, b1_16, w2_16, b2_16, y)
        return y.view(x.shape) if ok else None

    def takes_projection(self, rows: int) -> bool:
        """whether after_projection() has a kernel for this layer at `rows` rows (inference only)"""
        return not (torch.is_grad_enabled() or self.activation != "swiglu" or self.hidden_size not in PROJ_MLP_WIDTHS
                    or self.ffn_hidden_size % 32 != 0 or self.fused is False or (self.hidden_size == 256 and rows < 30000))

    def forward(self, x: torch.Tensor, residual: torch.Tensor = None):
        x2 = as_bf16_2d(x.reshape(-1, self.hidden_size)).contiguous()
        params = (self.layer_norm_weight, self.layer_norm_bias, self.fc1_weight, self.fc1_bias, self.fc2_weight, self.fc2_bias)
        g16, be16, w1_16, b1_16, w2_16, b2_16 = (c.get(p, self.training) for c, p in zip(self._c, params))
        r2 = None if residual is None else as_bf16_2d(residual.reshape(-1, self.hidden_size))
        y = torch.empty_like(x2)
        # on request, the whole gated MLP in one kernel where one exists (hidden activations stay in registers) ...
        want_fused = self.fused if self.fused is not None else (self.hidden_size <= 128 or x2.shape[0] >= 30000)
        fused = (want_fused and self.activation == "swiglu" and self.hidden_size in FUSED_MLP_WIDTHS
                 and self.ffn_hidden_size % 32 == 0)
        if fused:
            self._staged[0].arm(self.training, w1_16.shape[0], self.hidden_size, g16, be16, w1_16, b1_16, w2_16, b2_16,
                                tag=("mlp", float(self.eps)))
            fused = pshattn.ln_mlp_swiglu_bf16(x2, g16, be16, self.eps, w1_16, b1_16, w2_16, b2_16, r2, y)
        if not fused:
            # ... otherwise LayerNorm + fc1 + activation, then fc2 + residual
            h = torch.empty(x2.shape[0], self.ffn_hidden_size, dtype=torch.bfloat16, device=x.device)
            if self.hidden_size in FUSABLE_LN_WIDTHS:
                self._staged[0].arm(self.training, w1_16.shape[0], self.hidden_size, g16, be16, w1_16, b1_16,
                                    tag=("fc1", float(self.eps)))
                pshattn.ln_linear_bf16(x2, g16, be16, self.eps, w1_16, b1_16, None, h, self.activation)
            else:
                ln = torch.empty_like(x2)
                pshattn.layernorm_bf16(x2, g16, be16, ln, self.eps)
                pshattn.linear_bf16(ln, w1_16, b1_16, None, h, self.activation)
            if self.ffn_hidden_size > 512:
                self._staged[1].arm(self.training, self.hidden_size, self.ffn_hidden_size, w2_16, b2_16, tag="ys")
            pshattn.linear_bf16(h, w2_16, b2_16, r2, y, None)
        x_in = x.reshape(-1, self.hidden_size)
        res_in = None if residual is None else residual.reshape(-1, self.hidden_size)
        if not _grad_wanted(x_in, res_in, *params):
            return y.view(x.shape)
        if self.activation == "swiglu" and self.hidden_size in pshattn.LN_BWD_WIDTHS \
                and _hip_backward_covers(x_in, self.ffn_hidden_size) and (res_in is None or res_in.dtype == torch.bfloat16):
            out = _GatedMLPGrad.apply(y, x_in, res_in, *params, self.eps, g16, be16, w1_16, b1_16, w2_16)
            return out.view(x.shape)
        act, eps = self.activation, self.eps

        def ref(xx, res, ln_w, ln_b, w1, b1, w2, b2):
            hh = torch.nn.functional.layer_norm(xx, (xx.shape[-1],), ln_w, ln_b, eps)
            out = torch.nn.functional.linear(_act_ref(torch.nn.functional.linear(hh, w1, b1), act), w2, b2)
            return out if res is None else out + res
        out = torch_backward(y, ref, x_in, res_in, *params)
        return out.view(x.shape)
