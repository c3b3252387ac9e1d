"""CPU oracle for the Flash3D forward hot path.  TEST INFRASTRUCTURE ONLY.

Python face of ``oracle/f3d_oracle.c`` (integer / byte arithmetic, loaded through ctypes) plus fp32
torch restatements of the floating-point ops (bucketed attention, linear, LayerNorm, MLP).  Only
tests, the smoke test and the benchmark's CPU-baseline leg import this module; the product package
never does.

Arrays are numpy: fp16 coordinates as ``np.float16``, bf16 features as raw ``np.uint16`` bit
patterns, counters as ``np.uint32`` / ``np.uint16`` (the reference's CounterT / HashT).

Pins (tests/test_oracle_*.py, tests/test_golden.py): every function below is held to known answers, brute force or
a numpy / torch library routine of the same quantity, except one.  PARITY UNPINNED: ``swiglu`` -- which half of
fc1's output te.LayerNormMLP(activation="swiglu") gates is fixed by TransformerEngine, which is not in this image
and which no test of the reference checks; the function itself (silu of the first half times the second) is held
to torch.nn.functional.silu.  The model-level functions (xfmr_block, stage_forward, flash3d_forward) only compose
pinned functions in the order of the reference's layer files, cited at each.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libf3d_oracle.so")


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds).  Returns the library path."""
    src = os.path.join(_HERE, "f3d_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libf3d_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.f3d_or_half_to_float.restype = ctypes.c_float
        _lib.f3d_or_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.f3d_or_float_to_half.restype = ctypes.c_uint16
        _lib.f3d_or_float_to_half.argtypes = [ctypes.c_float]
        _lib.f3d_or_bf16_to_float.restype = ctypes.c_float
        _lib.f3d_or_bf16_to_float.argtypes = [ctypes.c_uint16]
        _lib.f3d_or_float_to_bf16.restype = ctypes.c_uint16
        _lib.f3d_or_float_to_bf16.argtypes = [ctypes.c_float]
        _lib.f3d_or_vox1.restype = ctypes.c_uint16
        _lib.f3d_or_vox1.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_uint32]
        _lib.f3d_or_space_out_bit_3d.restype = ctypes.c_uint64
        _lib.f3d_or_space_out_bit_3d.argtypes = [ctypes.c_uint64]
        _lib.f3d_or_zorder16.restype = ctypes.c_uint16
        _lib.f3d_or_zorder16.argtypes = [ctypes.c_uint16] * 3
        _lib.f3d_or_hash.restype = ctypes.c_uint16
        _lib.f3d_or_hash.argtypes = [ctypes.c_uint16] * 3 + [ctypes.c_uint32] * 3
        _lib.f3d_or_rng_u32.restype = ctypes.c_uint32
        _lib.f3d_or_rng_u32.argtypes = [ctypes.c_uint32] * 4
        _lib.f3d_or_rng_u01.restype = ctypes.c_float
        _lib.f3d_or_rng_u01.argtypes = [ctypes.c_uint32] * 4
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return ctypes.c_void_p(a.ctypes.data)


def _u16(a):
    """fp16 / bf16-bits / u16 array -> uint16 view"""
    a = np.ascontiguousarray(a)
    return a.view(np.uint16) if a.dtype == np.float16 else a.astype(np.uint16, copy=False)


# ---------------------------------------------------------------------------------------------
# helpers restated from flash3dxfmr/psh/{arithmatic,batching,subbuck,bucket_scope}.py
# ---------------------------------------------------------------------------------------------

def round_next_two_power(v: int) -> int:
    """flash3dxfmr/psh/arithmatic.py:12-19"""
    v -= 1
    for s in (1, 2, 4, 8, 16):
        v |= v >> s
    return v + 1


def psh_params(seps, bucket_size: int, num_vox: int = 0xFFFF):
    """num_bucket / divisor heuristics of flash3dxfmr/psh/psh_main.py:100-104: mean cloud size (fp32
    mean), floor-divided by the bucket size, next power of two; divisor = ceil(num_vox / NB)."""
    seps = np.asarray(seps, dtype=np.int64)
    sizes = np.diff(np.concatenate([[0], seps]))
    mean_n = float(np.float32(sizes.astype(np.float32).mean()))
    nb = round_next_two_power(int(mean_n / bucket_size))
    div = int(math.ceil(num_vox / nb)) if nb > 0 else 0
    return nb, div, int(sizes.max())


def calc_red_sep_sizes(seps, subbuck_size: int):
    """flash3dxfmr/psh/subbuck.py:40-53"""
    seps = np.asarray(seps, dtype=np.int64)
    sizes = np.diff(np.concatenate([[0], seps]))
    red_sizes = (sizes + subbuck_size - 1) // subbuck_size
    return int(red_sizes.sum()), red_sizes.astype(np.uint32), np.cumsum(red_sizes).astype(np.uint32)


def gen_scopes(total_n: int, buck_size: int, scope_size: int, plan: str = "swin"):
    """flash3dxfmr/psh/bucket_scope.py:58-140 — consecutive groups of ``scope_size`` buckets when the
    length is aligned (swin: buck*scope; stride: buck*scope*6), one global scope otherwise."""
    assert plan in ("swin", "stride")
    assert total_n % buck_size == 0
    nbuck = total_n // buck_size
    align = buck_size * scope_size * (6 if plan == "stride" else 1)
    if total_n % align == 0:
        return np.arange(nbuck, dtype=np.uint32).reshape(nbuck // scope_size, scope_size)
    return np.arange(nbuck, dtype=np.uint32).reshape(1, nbuck)


# ---------------------------------------------------------------------------------------------
# A1 / A2
# ---------------------------------------------------------------------------------------------

def set_quantiser(mode: int):
    """0: the quantiser's quotient as a multiply by the rounded reciprocal (a fast-math build of the reference, default);
    1: IEEE division (src/psh/hash_fns.cuh:23-33 as written).  Applies to every later call of this module."""
    if lib().f3d_or_set_quantiser(ctypes.c_int(mode)) != 0:
        raise ValueError(f"quantiser mode must be 0 or 1, got {mode}")


def vox_coord(coord_h, bbox_min_h, bbox_max_h, num_vox: int = 0xFFFF):
    c = _u16(coord_h).reshape(-1, 3)
    out = np.empty_like(c)
    lib().f3d_or_vox_coord(_p(c), ctypes.c_uint32(c.shape[0]), _p(_u16(bbox_min_h)), _p(_u16(bbox_max_h)),
                           ctypes.c_uint32(num_vox), _p(out))
    return out


def hash_ids(vox, hash_type: int, divisor: int, num_bucket: int):
    """vectorised numpy restatement of f3d_or_hash (kept separate from the C code on purpose: the
    two are checked against each other in the oracle tests)"""
    v = vox.astype(np.uint64)

    def spread(x):
        x = (x | x << np.uint64(32)) & np.uint64(0x1f00000000ffff)
        x = (x | x << np.uint64(16)) & np.uint64(0x1f0000ff0000ff)
        x = (x | x << np.uint64(8)) & np.uint64(0x100f00f00f00f00f)
        x = (x | x << np.uint64(4)) & np.uint64(0x10c30c30c30c30c3)
        x = (x | x << np.uint64(2)) & np.uint64(0x1249249249249249)
        return x

    if hash_type in (1, 3):
        m = spread(v[:, 0]) | spread(v[:, 1]) << np.uint64(1) | spread(v[:, 2]) << np.uint64(2)
        h = ((m >> np.uint64(31)) & np.uint64(0xFFFF)).astype(np.uint32)
    else:
        h = (vox[:, 0] ^ vox[:, 1] ^ vox[:, 2]).astype(np.uint32)
    if hash_type in (1, 2):
        return (h // np.uint32(divisor & 0xFFFF)).astype(np.uint16)
    return (h % np.uint32(num_bucket & 0xFFFF)).astype(np.uint16)


# ---------------------------------------------------------------------------------------------
# A3 / A5 / scoreboard
# ---------------------------------------------------------------------------------------------

def psh_claim(coord_h, seps, bbox_min_h, bbox_max_h, num_vox, divisor, num_bucket, hash_type):
    c = _u16(coord_h).reshape(-1, 3)
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    n, b = c.shape[0], seps.shape[0]
    bucket_id = np.ones(n, dtype=np.uint16)
    counter = np.zeros((b, num_bucket), dtype=np.uint32)
    offset = np.zeros(n, dtype=np.uint32)
    rc = lib().f3d_or_psh_claim(_p(c), ctypes.c_uint32(n), _p(seps), ctypes.c_uint32(b), _p(_u16(bbox_min_h)),
                                _p(_u16(bbox_max_h)), ctypes.c_uint32(num_vox), ctypes.c_uint32(divisor),
                                ctypes.c_uint32(num_bucket), ctypes.c_uint32(hash_type), _p(bucket_id),
                                _p(counter), _p(offset))
    if rc != 0:
        raise RuntimeError(f"oracle psh_claim failed rc={rc}")
    return bucket_id, counter, offset


def psh_rebalance(bucket_id, counter, offset, seps, bucket_size):
    """deterministic overflow rebalance + recycle (A4); returns new (ids, counts, slots)"""
    ids = np.ascontiguousarray(bucket_id, dtype=np.uint16).copy()
    cnt = np.ascontiguousarray(counter, dtype=np.uint32).copy()
    off = np.ascontiguousarray(offset, dtype=np.uint32).copy()
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    rc = lib().f3d_or_psh_rebalance(_p(ids), _p(cnt), _p(off), _p(seps), ctypes.c_uint32(seps.shape[0]),
                                    ctypes.c_uint32(cnt.shape[1]), ctypes.c_uint32(bucket_size))
    assert rc == 0
    return ids, cnt, off


def cumsum_scatter_pad(coord_h, seps, num_bucket, bucket_id, counter, offset, pad_to, pad_num=0.0,
                       prefill_nan=True):
    c = _u16(coord_h).reshape(-1, 3)
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    n, b = c.shape[0], seps.shape[0]
    cumsum = np.zeros((b, num_bucket), dtype=np.uint32)
    scattered = np.full((pad_to, 3), 0x7E00 if prefill_nan else 0, dtype=np.uint16)
    rc = lib().f3d_or_cumsum_scatter_pad(_p(c), ctypes.c_uint32(n), _p(seps), ctypes.c_uint32(b),
                                         ctypes.c_uint32(num_bucket), _p(bucket_id), _p(counter), _p(offset),
                                         _p(cumsum), _p(scattered), ctypes.c_uint32(pad_to),
                                         ctypes.c_float(pad_num))
    if rc != 0:
        raise RuntimeError(f"oracle cumsum_scatter_pad failed rc={rc}")
    return cumsum, scattered.view(np.float16)


def scatter_feat_index(seps, num_bucket, bucket_id, offset, cumsum, pad_to, feat=None):
    """out-to-in permutation index of the PSH scatter (pad rows: N + 3) and, with `feat` [N, ...], the features in
    PSH order with zero pad rows (src/psh/batch_psh_bucket.cuh:617-753)"""
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    bid = np.ascontiguousarray(bucket_id, dtype=np.uint16)
    n, b = bid.shape[0], seps.shape[0]
    idx = np.full(pad_to, 0xFFFFFFFF, dtype=np.uint32)
    f = out = None
    row_bytes = 0
    if feat is not None:
        f = np.ascontiguousarray(feat)
        row_bytes = f.dtype.itemsize * int(np.prod(f.shape[1:], dtype=np.int64))
        out = np.full((pad_to,) + f.shape[1:], 0, dtype=f.dtype)
        out.view(np.uint8)[...] = 0xA5
    rc = lib().f3d_or_scatter_feat_index(
        ctypes.c_uint32(n), _p(seps), ctypes.c_uint32(b), ctypes.c_uint32(num_bucket), _p(bid),
        _p(np.ascontiguousarray(offset, dtype=np.uint32)), _p(np.ascontiguousarray(cumsum, dtype=np.uint32)),
        _p(f) if f is not None else None, ctypes.c_uint32(row_bytes), _p(idx),
        _p(out) if out is not None else None, ctypes.c_uint32(pad_to))
    if rc != 0:
        raise RuntimeError(f"oracle scatter_feat_index failed rc={rc}")
    return (idx, out) if feat is not None else idx


def scoreboard(bucket_id, counter, offset, seps):
    """0 when every (cloud, bucket, slot < count) is claimed exactly once (bucket_sanitizer_cpu.cpp:92-176)"""
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    counter = np.ascontiguousarray(counter, dtype=np.uint32)
    bad = ctypes.c_int64(-1)
    rc = lib().f3d_or_scoreboard(_p(np.ascontiguousarray(bucket_id, dtype=np.uint16)), _p(counter),
                                 _p(np.ascontiguousarray(offset, dtype=np.uint32)), _p(seps),
                                 ctypes.c_uint32(seps.shape[0]), ctypes.c_uint32(counter.shape[1]),
                                 ctypes.byref(bad))
    return rc, bad.value


# ---------------------------------------------------------------------------------------------
# A6 / A7 / A8
# ---------------------------------------------------------------------------------------------

def subbuck_build(coord_h, seps, subbuck_size, num_vox=0xFFFF, seed=3407, out_align=1):
    c = _u16(coord_h).reshape(-1, 3)
    seps = np.ascontiguousarray(seps, dtype=np.uint32)
    n = c.shape[0]
    red_len, _, red_sep = calc_red_sep_sizes(seps, subbuck_size)
    r_aligned = -(-red_len // out_align) * out_align
    sub_id = np.zeros(n, dtype=np.uint32)
    sub_off = np.zeros(n, dtype=np.uint16)
    unpool = np.full((red_len, subbuck_size), n + 3, dtype=np.uint32)
    red_coord = np.zeros((r_aligned, 3), dtype=np.uint16)
    rc = lib().f3d_or_subbuck_build(_p(c), ctypes.c_uint32(n), _p(seps), _p(red_sep),
                                    ctypes.c_uint32(seps.shape[0]), ctypes.c_uint32(subbuck_size),
                                    ctypes.c_uint32(num_vox), ctypes.c_uint32(seed), _p(sub_id), _p(sub_off),
                                    _p(unpool), _p(red_coord), ctypes.c_uint32(r_aligned))
    if rc != 0:
        raise RuntimeError(f"oracle subbuck_build failed rc={rc}")
    return sub_id, sub_off, unpool, red_coord.view(np.float16), red_sep


def reduce_feat(feat_bf, unpool_ind, red_op, r_aligned=None):
    f = np.ascontiguousarray(feat_bf, dtype=np.uint16)
    u = np.ascontiguousarray(unpool_ind, dtype=np.uint32)
    n, c = f.shape
    r, s = u.shape
    ra = r if r_aligned is None else r_aligned
    out = np.zeros((ra, c), dtype=np.uint16)
    rc = lib().f3d_or_reduce_feat(_p(f), ctypes.c_uint32(n), ctypes.c_uint32(c), _p(u), ctypes.c_uint32(r),
                                  ctypes.c_uint32(s), ctypes.c_uint32(red_op), _p(out), ctypes.c_uint32(ra))
    if rc != 0:
        raise RuntimeError(f"oracle reduce_feat failed rc={rc}")
    return out


def additive_unpool(res_bf, down_bf, unpool_ind, up_init=None):
    res = np.ascontiguousarray(res_bf, dtype=np.uint16)
    down = np.ascontiguousarray(down_bf, dtype=np.uint16)
    u = np.ascontiguousarray(unpool_ind, dtype=np.uint32)
    up = np.zeros_like(res) if up_init is None else np.ascontiguousarray(up_init, dtype=np.uint16).copy()
    rc = lib().f3d_or_additive_unpool(_p(res), _p(down), _p(up), _p(u), ctypes.c_uint32(res.shape[0]),
                                      ctypes.c_uint32(u.shape[0]), ctypes.c_uint32(res.shape[1]),
                                      ctypes.c_uint32(u.shape[1]))
    assert rc == 0
    return up


def additive_unpool_bwd(grad_up_bf, unpool_ind, down_rows=None, grad_res_init=None):
    """backward of additive_unpool: returns (grad_res, grad_down) as bf16 bit patterns
    (src/psh/additive_unpool.cuh:90-137); rows of grad_res that no slot refers to keep ``grad_res_init`` (zeros)."""
    g = np.ascontiguousarray(grad_up_bf, dtype=np.uint16)
    u = np.ascontiguousarray(unpool_ind, dtype=np.uint32)
    n, c = g.shape
    r, s = u.shape
    grad_res = np.zeros_like(g) if grad_res_init is None else np.ascontiguousarray(grad_res_init, dtype=np.uint16).copy()
    grad_down = np.zeros((r if down_rows is None else down_rows, c), dtype=np.uint16)
    rc = lib().f3d_or_additive_unpool_bwd(_p(grad_res), _p(grad_down), _p(g), _p(u), ctypes.c_uint32(n),
                                          ctypes.c_uint32(r), ctypes.c_uint32(c), ctypes.c_uint32(s))
    assert rc == 0
    return grad_res, grad_down


def reduce_feat_bwd(grad_red_bf, input_bf, unpool_ind, red_op, grad_in_init=None):
    """backward of reduce_feat (src/psh/batch_psh_subbuck_reduce_bwd.cuh:39-126): grad_input as bf16 bits"""
    g = np.ascontiguousarray(grad_red_bf, dtype=np.uint16)
    x = np.ascontiguousarray(input_bf, dtype=np.uint16)
    u = np.ascontiguousarray(unpool_ind, dtype=np.uint32)
    n, c = x.shape
    r, s = u.shape
    grad_in = np.zeros_like(x) if grad_in_init is None else np.ascontiguousarray(grad_in_init, dtype=np.uint16).copy()
    rc = lib().f3d_or_reduce_feat_bwd(_p(g), _p(x), _p(u), _p(grad_in), ctypes.c_uint32(n), ctypes.c_uint32(r),
                                      ctypes.c_uint32(c), ctypes.c_uint32(s), ctypes.c_uint32(red_op))
    if rc != 0:
        raise RuntimeError(f"oracle reduce_feat_bwd failed rc={rc}")
    return grad_in


# ---------------------------------------------------------------------------------------------
# bf16 bit helpers (numpy)
# ---------------------------------------------------------------------------------------------

def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    return np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), r)


# ---------------------------------------------------------------------------------------------
# A9 / A9m bucketed attention, A11 / A12 dense layers — fp32 torch on bf16-rounded inputs
# ---------------------------------------------------------------------------------------------

def buck_swin_fwd(Q, K, V, scope_buckets, bucket_size, kv_len=None, O_init=None, LSE_init=None):
    """Definition of pshattn.buck_swin_fwd (declared src/f3d_frontend.cu:90-92; semantics pinned by
    tests/test_attn_fwd.py:167-190, 404-452): for every batch row and every scope (row of
    ``scope_buckets``), full softmax attention among the rows of the scope's buckets, per head,
    scale 1/sqrt(D); LSE is the natural-log sum of exponentials.  Rows no scope covers keep
    ``O_init`` / ``LSE_init``.

    ``kv_len`` (extension, int per bucket): keys at in-bucket position >= kv_len are masked out;
    query rows at such positions produce O = 0, LSE = 0.

    Q, K, V: torch tensors [B, L, H, D] (any float dtype; computed in fp32).  Returns (O, LSE) fp32.
    """
    import torch

    B, L, H, D = Q.shape
    scopes = torch.as_tensor(np.asarray(scope_buckets).astype(np.int64))
    Qf, Kf, Vf = Q.float(), K.float(), V.float()
    O = torch.zeros(B, L, H, D, dtype=torch.float32) if O_init is None else O_init.float().clone()
    LSE = torch.zeros(B, L, H, dtype=torch.float32) if LSE_init is None else LSE_init.float().clone()
    ar = torch.arange(bucket_size)
    scale = 1.0 / math.sqrt(D)
    for s in range(scopes.shape[0]):
        rows = (scopes[s][:, None] * bucket_size + ar[None, :]).reshape(-1)
        if kv_len is not None:
            kl = torch.as_tensor(np.asarray(kv_len).astype(np.int64))[scopes[s]]
            valid = (ar[None, :] < kl[:, None]).reshape(-1)
        else:
            valid = torch.ones(rows.shape[0], dtype=torch.bool)
        q = Qf[:, rows].permute(0, 2, 1, 3)  # [B,H,T,D]
        k = Kf[:, rows].permute(0, 2, 1, 3)
        v = Vf[:, rows].permute(0, 2, 1, 3)
        logits = torch.matmul(q, k.transpose(-1, -2)) * scale
        logits = logits.masked_fill(~valid[None, None, None, :], float("-inf"))
        lse = torch.logsumexp(logits, dim=-1)  # [B,H,T]
        p = torch.exp(logits - lse[..., None])
        o = torch.matmul(p, v)  # [B,H,T,D]
        o = torch.where(valid[None, None, :, None], o, torch.zeros_like(o))
        lse = torch.where(valid[None, None, :], lse, torch.zeros_like(lse))
        O[:, rows] = o.permute(0, 2, 1, 3)
        LSE[:, rows] = lse.permute(0, 2, 1)
    return O, LSE


def buck_swin_bwd(Q, K, V, dO, scope_buckets, bucket_size, kv_len=None):
    """Backward of buck_swin_fwd (pshattn.buck_swin_bwd, declared src/f3d_frontend.cu:94-97; the formulas are the
    ones the reference's tests take from autograd, tests/test_attn_bwd.py): per scope and head, with
    P = softmax(Q Kt / sqrt(D)),  Delta = rowsum(dO * O),  dV = Pt dO,  dP = dO Vt,  dS = P * (dP - Delta),
    dQ = dS K / sqrt(D),  dK = dSt Q / sqrt(D).  Rows no scope covers get zero gradients.
    ``kv_len`` (the forward's extension): P is the softmax over the valid keys, and zero on masked query rows, so
    masked rows get zero gradients and Delta = 0.
    Returns (dQ, dK, dV, Delta) in fp32."""
    import torch

    B, L, H, D = Q.shape
    scopes = torch.as_tensor(np.asarray(scope_buckets).astype(np.int64))
    Qf, Kf, Vf, dOf = Q.float(), K.float(), V.float(), dO.float()
    dQ, dK, dV = torch.zeros_like(Qf), torch.zeros_like(Kf), torch.zeros_like(Vf)
    Delta = torch.zeros(B, L, H, dtype=torch.float32)
    ar = torch.arange(bucket_size)
    scale = 1.0 / math.sqrt(D)
    for s in range(scopes.shape[0]):
        rows = (scopes[s][:, None] * bucket_size + ar[None, :]).reshape(-1)
        q, k, v, do = [t[:, rows].permute(0, 2, 1, 3) for t in (Qf, Kf, Vf, dOf)]   # [B,H,T,D]
        logits = torch.matmul(q, k.transpose(-1, -2)) * scale
        if kv_len is not None:
            kl = torch.as_tensor(np.asarray(kv_len).astype(np.int64))[scopes[s]]
            valid = (ar[None, :] < kl[:, None]).reshape(-1)
            logits = logits.masked_fill(~valid[None, None, None, :], float("-inf"))
            p = torch.softmax(logits, dim=-1) if valid.any() else torch.zeros_like(logits)
            p = torch.where(valid[None, None, :, None], p, torch.zeros_like(p))
        else:
            p = torch.softmax(logits, dim=-1)
        o = torch.matmul(p, v)
        delta = (do * o).sum(-1)                                                    # [B,H,T]
        dp = torch.matmul(do, v.transpose(-1, -2))
        ds = p * (dp - delta[..., None])
        dQ[:, rows] = (torch.matmul(ds, k) * scale).permute(0, 2, 1, 3)
        dK[:, rows] = (torch.matmul(ds.transpose(-1, -2), q) * scale).permute(0, 2, 1, 3)
        dV[:, rows] = torch.matmul(p.transpose(-1, -2), do).permute(0, 2, 1, 3)
        Delta[:, rows] = delta.permute(0, 2, 1)
    return dQ, dK, dV, Delta


def linear(x, w, b=None):
    """y = x @ w.T + b in fp32 (torch.nn.Linear semantics; layers/buck_swin.py:159,163)"""
    import torch
    y = x.float() @ w.float().t()
    return y + b.float() if b is not None else y


def layernorm(x, g, b, eps=1e-5):
    import torch
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), g.float(), b.float(), eps)


def gelu(x):
    import torch
    return torch.nn.functional.gelu(x.float())


def swiglu(h):
    """silu(h[:, :hid]) * h[:, hid:] — the definition this build gives te.LayerNormMLP(activation="swiglu")
    (layers/elem_wise.py:22-26); TransformerEngine itself is absent, so this ordering is parity-unpinned."""
    import torch
    hid = h.shape[-1] // 2
    return torch.nn.functional.silu(h[..., :hid].float()) * h[..., hid:].float()


# ---------------------------------------------------------------------------------------------
# model-level restatement: the op sequence of flash3dxfmr/layers (flash3d.py:148-166,
# stage.py:71-102, hourglass.py:79-112, 165-188, 268-293), every layer output rounded to bf16 as
# the bf16 modules of the reference do
# ---------------------------------------------------------------------------------------------

def _r(t):
    """round an fp32 torch tensor to bf16 and back"""
    import torch
    return t.to(torch.bfloat16).float()


def psh_scatter_coords(coord_h, seps, bucket_size, pad_to, hash_op, num_vox=0xFFFF, rebalance=True):
    """psh_main.batch_bucket_scatter: whole-batch bbox, geometry heuristics, claim, rebalance, scatter, pad"""
    nb, div, _ = psh_params(seps, bucket_size, num_vox)
    c = np.ascontiguousarray(coord_h, dtype=np.float16)
    ids, cnt, off = psh_claim(c, seps, c.min(0), c.max(0), num_vox, div, nb, hash_op)
    if rebalance:
        ids, cnt, off = psh_rebalance(ids, cnt, off, seps, bucket_size)
    _, scat = cumsum_scatter_pad(c, seps, nb, ids, cnt, off, pad_to, 0.0)
    return scat


def xfmr_block(x, w, scopes, bucket_size, num_heads, activation="swiglu"):
    """x [N,C] fp32 holding bf16 values; w: dict of fp32 tensors (bf16-rounded weights) with keys
    norm.weight/bias, qkv.weight/bias, proj.weight/bias, ln.weight/bias, fc1.weight/bias, fc2.weight/bias"""
    import torch
    n, c = x.shape
    h = _r(layernorm(x, w["norm.weight"], w["norm.bias"]))
    qkv = _r(linear(h, w["qkv.weight"], w.get("qkv.bias")))
    q, k, v = [t.reshape(1, n, num_heads, c // num_heads) for t in qkv.chunk(3, dim=-1)]
    o, _ = buck_swin_fwd(q, k, v, scopes, bucket_size)
    o = _r(o).reshape(n, c)
    mid = _r(_r(linear(o, w["proj.weight"], w["proj.bias"])) + x)
    h2 = _r(layernorm(mid, w["ln.weight"], w["ln.bias"]))
    f1 = _r(linear(h2, w["fc1.weight"], w["fc1.bias"]))
    hid = _r(swiglu(f1)) if activation == "swiglu" else _r(gelu(f1))
    return _r(_r(linear(hid, w["fc2.weight"], w["fc2.bias"])) + mid)


def bn_act(x, bn, act):
    """eval-mode BatchNorm1d (dict weight, bias, mean, var, eps) then activation name"""
    import torch
    if bn is not None:
        x = _r((x - bn["mean"]) * torch.rsqrt(bn["var"] + bn["eps"]) * bn["weight"] + bn["bias"])
    if act == "gelu":
        x = _r(gelu(x))
    elif act == "relu":
        x = _r(torch.relu(x))
    return x


def norm_act(x, p, act):
    """optional norm then optional activation, each rounded to bf16.  `p` is None, a LayerNorm dict
    (weight, bias, eps) or an eval-mode BatchNorm1d dict (weight, bias, mean, var, eps): the callables the
    reference passes as pool_norm / unpool_norm (tests/test_psh_hourglass.py:103-106)"""
    import torch
    if p is not None and "mean" in p:
        return bn_act(x, p, act)
    if p is not None:
        x = _r(torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), p["weight"], p["bias"], p.get("eps", 1e-5)))
    return bn_act(x, None, act)


XFMR_KEYS = {"norm.weight": "norm.weight", "norm.bias": "norm.bias", "qkv.weight": "bwa.qkv.weight",
             "qkv.bias": "bwa.qkv.bias", "proj.weight": "bwa.proj.weight", "proj.bias": "bwa.proj.bias",
             "ln.weight": "mlp.mlp.layer_norm_weight", "ln.bias": "mlp.mlp.layer_norm_bias",
             "fc1.weight": "mlp.mlp.fc1_weight", "fc1.bias": "mlp.mlp.fc1_bias",
             "fc2.weight": "mlp.mlp.fc2_weight", "fc2.bias": "mlp.mlp.fc2_bias"}


def _norm_params(sd, prefix, eps_bn=1e-3):
    if prefix + "weight" not in sd:
        return None
    p = {"weight": sd[prefix + "weight"], "bias": sd[prefix + "bias"]}
    if prefix + "running_mean" in sd:
        p.update(mean=sd[prefix + "running_mean"], var=sd[prefix + "running_var"], eps=eps_bn)
    return p


def stage_forward(sd, prefix, coord_h, x, seps, levels, level, bs, scope, S, trace=None):
    """Stage.forward (layers/stage.py:171-197) around HourglassModule.forward (layers/hourglass.py:268-293) or the
    LeafModule (layers/flash3d.py:25-38), recursively.  `sd`: state dict of fp32 CPU tensors holding bf16 values
    (norm statistics fp32); `levels[level]`: dict(heads, n_enc, n_dec, red_op, pool_align, pool_act, unpool_act,
    bn_eps).  x [n, C] fp32 holding bf16 values, coord_h [n, 3] fp16, seps inclusive cumulative sizes whose last
    entry is n."""
    import torch
    cfg = levels[level]
    n = x.shape[0]
    scopes = gen_scopes(n, bs, scope)
    w = lambda pre: {k: sd[pre + v] for k, v in XFMR_KEYS.items() if pre + v in sd}
    for i in range(cfg["n_enc"]):
        x = xfmr_block(x, w(f"{prefix}encoder_blocks.{i}."), scopes, bs, cfg["heads"], cfg.get("activation", "swiglu"))
    if trace is not None:
        trace.append(("enc", level, x))
    mid = prefix + "middle."
    if level + 1 == len(levels):
        x = _r(linear(x, sd[mid + "proj.weight"], sd[mid + "proj.bias"]))
    else:
        proj = _r(linear(x, sd[mid + "pooling.proj.weight"], sd[mid + "pooling.proj.bias"]))
        _, _, unpool, red_coord, red_sep = subbuck_build(coord_h, seps, S, out_align=cfg["pool_align"])
        r_al = red_coord.shape[0]
        red = torch.from_numpy(bf16_bits_to_f32(reduce_feat(f32_to_bf16_bits(proj.numpy()), unpool, cfg["red_op"],
                                                              r_aligned=r_al)))
        red = norm_act(red, _norm_params(sd, mid + "pooling.norm.", cfg.get("bn_eps", 1e-3)), cfg.get("pool_act"))
        sub_sep = np.array(red_sep, dtype=np.uint32).copy()
        sub_sep[-1] = r_al
        if trace is not None:
            trace.append(("pool", level, unpool, red_coord))
        sub = stage_forward(sd, mid + "submodule.", red_coord, red, sub_sep, levels, level + 1, bs, scope, S, trace)
        un = mid + "unpooling."
        pd = norm_act(_r(linear(sub, sd[un + "proj.0.weight"], sd[un + "proj.0.bias"])),
                      _norm_params(sd, un + "proj.norm.", cfg.get("bn_eps", 1e-3)), cfg.get("unpool_act"))
        ps = norm_act(_r(linear(proj, sd[un + "proj_skip.0.weight"], sd[un + "proj_skip.0.bias"])),
                      _norm_params(sd, un + "proj_skip.norm.", cfg.get("bn_eps", 1e-3)), cfg.get("unpool_act"))
        up = additive_unpool(f32_to_bf16_bits(ps.numpy()), f32_to_bf16_bits(pd.numpy()), unpool)
        x = torch.from_numpy(bf16_bits_to_f32(up))
    for i in range(cfg["n_dec"]):
        x = xfmr_block(x, w(f"{prefix}decoder_blocks.{i}."), scopes, bs, cfg["heads"], cfg.get("activation", "swiglu"))
    return x


def flash3d_forward(sd, coord_h, seps, levels, bs, scope, hash_op, S, trace=None):
    """Flash3D.forward (layers/flash3d.py:148-166) with the scattered coordinates routed down the tree and the pad
    rows counted into the last cloud.  Returns (output [pad_to, C] fp32 holding bf16 values, scattered coords)."""
    import torch
    n = coord_h.shape[0]
    align = bs * scope * 6
    pad_to = -(-n // align) * align
    scat = psh_scatter_coords(coord_h, seps, bs, pad_to, hash_op)
    x = _r(linear(torch.from_numpy(scat.astype(np.float32)).to(torch.bfloat16), sd["psh_scatter.lin.weight"],
                  sd["psh_scatter.lin.bias"]))
    tree_seps = np.array(seps, dtype=np.uint32).copy()
    tree_seps[-1] = pad_to
    return stage_forward(sd, "module_tree.", scat, x, tree_seps, levels, 0, bs, scope, S, trace), scat
