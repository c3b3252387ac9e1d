"""`pshattn` — the custom-op surface of the reference (pybind module built from
src/f3d_frontend.cu:112-138), re-created over the C ABI of ``libf3d_hip.so``.

Same function names and positional argument order as the reference module, so the layer code and
tests that call ``pshattn.<op>(tensors..., scalars...)`` read the same.  Every function mutates
caller-allocated output tensors in place and returns ``None``.  Tensor-level checks (contiguity,
device, dtype) live here because the C ABI only sees pointers; value checks live in the library and
come back as ``RuntimeError`` with the library's message — the reference's
``throw std::runtime_error`` behaviour (src/common/runtime.h:36-86).

There is no CPU fallback: if the HIP library is missing this module raises on import of the first op.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libf3d_hip.so")
_lib = None

_u32, _i32, _f32, _vp = ctypes.c_uint32, ctypes.c_int, ctypes.c_float, ctypes.c_void_p


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m flash3dtransformer_amd.csrc.build` "
                "(hipcc, gfx950). There is no CPU fallback for the Flash3D ops.")
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.f3d_last_error.restype = ctypes.c_char_p
        _lib.f3d_get_seed.restype = ctypes.c_uint32
    return _lib


def library_path() -> str:
    return _LIB_PATH


def _check(rc: int):
    if rc != 0:
        raise RuntimeError(_load().f3d_last_error().decode("utf-8", "replace"))


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else _vp(0)


def _stream(dev_index: int):
    return _vp(torch.cuda.current_stream(dev_index).cuda_stream)


def assert_contiguous(tensors):
    """src/common/runtime.h assert_contiguous"""
    for i, t in enumerate(tensors):
        if not t.is_contiguous():
            raise RuntimeError(f"Tensor #{i} is not contiguous.")


def assert_same_device(tensors):
    dev = tensors[0].device
    for i, t in enumerate(tensors):
        if t.device != dev:
            raise RuntimeError(f"Tensor #{i} is on {t.device}, expected {dev}.")
    if dev.type != "cuda":
        raise RuntimeError(f"Flash3D ops need tensors on a GPU device, got {dev}.")
    return dev.index if dev.index is not None else torch.cuda.current_device()


def assert_dtype(tensors, dtype):
    for i, t in enumerate(tensors):
        if t.dtype != dtype:
            raise RuntimeError(f"Tensor #{i} has dtype {t.dtype}, expected {dtype}.")


def _check_vectors(dev_ref, tensors, dtype=torch.bfloat16):
    """optional 1-D operands (bias, beta, ...): same device as the call, the wire dtype, contiguous"""
    ts = [t for t in tensors if t is not None]
    if ts:
        assert_same_device([dev_ref] + ts)
        assert_dtype(ts, dtype)
        assert_contiguous(ts)


class DeviceManagerSingleton:
    """src/common/device_manager.{cuh,cu}; bound at src/f3d_frontend.cu:115-120"""
    _inst = None

    @staticmethod
    def instance():
        if DeviceManagerSingleton._inst is None:
            DeviceManagerSingleton._inst = DeviceManagerSingleton()
        return DeviceManagerSingleton._inst

    def init_dev_info(self, dev_id: int):
        _check(_load().f3d_init_dev_info(_i32(dev_id)))

    def init_dispatchers(self):
        _load()  # kernels are selected at call time; loading the library is all there is to do

    def set_sync_stream(self, is_syncing: bool) -> bool:
        return bool(_load().f3d_set_sync_stream(_i32(1 if is_syncing else 0)))

    def get_sync_stream(self) -> bool:
        return bool(_load().f3d_get_sync_stream())

    # extensions -----------------------------------------------------------------------------
    def set_seed(self, seed: int):
        _check(_load().f3d_set_seed(_u32(seed)))

    def get_seed(self) -> int:
        return int(_load().f3d_get_seed())

    def set_psh_rebalance(self, mode: int):
        _check(_load().f3d_set_psh_rebalance(_i32(mode)))

    def get_psh_rebalance(self) -> int:
        return int(_load().f3d_get_psh_rebalance())

    def set_quantiser(self, mode: int):
        """0: quotient of the voxel quantiser as a multiply by the rounded reciprocal (a fast-math build of the
        reference, default); 1: IEEE division (src/psh/hash_fns.cuh:23-33 as written)"""
        _check(_load().f3d_set_quantiser(_i32(mode)))

    def get_quantiser(self) -> int:
        return int(_load().f3d_get_quantiser())


# ---------------------------------------------------------------------------------------------
# PSH bucketing
# ---------------------------------------------------------------------------------------------

def batch_psh_scatter_pad_hash(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, instance_max_N,
                               num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max,
                               probe_offsets, cumsum_counter, scatter_coord, pad_num, hash_type, no_alloc=False):
    """src/f3d_frontend.cu:52-58 -> src/psh/batch_psh_bucket_dispatcher.cu:221-326.
    no_alloc=True takes the entry point that allocates nothing (fixed scratch array in the library, no
    counterpart in the reference; bbox_min / bbox_max must then be contiguous already)."""
    ts = [coord, bucket_id, bucket_counter, bucket_offset, batch_sep, probe_offsets, cumsum_counter, scatter_coord]
    assert_contiguous(ts)
    dev = assert_same_device(ts + [bbox_min, bbox_max])
    assert_dtype([coord, bbox_min, bbox_max, scatter_coord], torch.float16)
    assert_dtype([bucket_counter, bucket_offset, batch_sep, cumsum_counter], torch.uint32)
    assert_dtype([bucket_id], torch.uint16)
    if no_alloc:
        assert_contiguous([bbox_min, bbox_max])
    bbox_min, bbox_max = bbox_min.contiguous(), bbox_max.contiguous()
    fn = _load().f3d_batch_psh_scatter_pad_hash_noalloc if no_alloc else _load().f3d_batch_psh_scatter_pad_hash
    _check(fn(
        _ptr(coord), _ptr(bucket_id), _ptr(bucket_counter), _ptr(bucket_offset), _ptr(batch_sep),
        _u32(batch_sep.shape[0]), _u32(coord.shape[0]), _u32(instance_max_N), _u32(num_bucket),
        _u32(bucket_divisor), _u32(bucket_size), _u32(num_vox), _ptr(bbox_min), _ptr(bbox_max),
        _ptr(probe_offsets), _ptr(cumsum_counter), _ptr(scatter_coord), _u32(scatter_coord.shape[0]),
        _f32(pad_num), _u32(hash_type), _i32(dev), _stream(dev)))


def batch_psh_scatter_pad(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, instance_max_N,
                          num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max,
                          probe_offsets, cumsum_counter, scatter_coord, pad_num):
    """src/f3d_frontend.cu:45-50; hash fixed to H_ZORDER_MOD (batch_psh_bucket_dispatcher.cu:161-163)"""
    batch_psh_scatter_pad_hash(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, instance_max_N,
                               num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max,
                               probe_offsets, cumsum_counter, scatter_coord, pad_num, 3)


def batch_psh_scatter(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, instance_max_N, num_bucket,
                      bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max, probe_offsets, cumsum_counter,
                      scatter_coord, hash_dtype=None, coord_dtype=None, block_size_N=1024):
    """src/f3d_frontend.cu:38-43: no tail padding (scatter_coord has exactly N rows); the dtype objects
    and block size of the reference signature are accepted and unused (types are fixed on the wire)."""
    if scatter_coord.shape[0] != coord.shape[0]:
        raise RuntimeError(
            f"Output coord buffer length({scatter_coord.shape[0]}) must equal the input length({coord.shape[0]}).")
    batch_psh_scatter_pad_hash(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, instance_max_N,
                               num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max,
                               probe_offsets, cumsum_counter, scatter_coord, 0.0, 3)


def _row_bytes(t) -> int:
    n = t.element_size()
    for d in t.shape[1:]:
        n *= d
    return n


def psh_scatter_feat_index(bucket_id, bucket_counter, bucket_offset, batch_sep, cumsum_counter, scatter_idx_out2in,
                           feat=None, scattered_feat=None):
    """Completes src/psh/batch_psh_bucket.cuh:617-753: after a batch_psh_scatter* call on the same buffers,
    scatter_idx_out2in[dst] = src (pad rows: N + 3) and, with `feat`, scattered_feat[dst] = feat[src] (pad rows
    zero).  feat [N, ...] and scattered_feat [pad_to, ...] of one dtype and trailing shape."""
    ts = [bucket_id, bucket_counter, bucket_offset, batch_sep, cumsum_counter, scatter_idx_out2in]
    if (feat is None) != (scattered_feat is None):
        raise RuntimeError("feat and scattered_feat come together")
    if feat is not None:
        ts += [feat, scattered_feat]
        if feat.dtype != scattered_feat.dtype or feat.shape[1:] != scattered_feat.shape[1:]:
            raise RuntimeError(f"feat {tuple(feat.shape)} {feat.dtype} and scattered_feat "
                               f"{tuple(scattered_feat.shape)} {scattered_feat.dtype} differ in row shape or dtype")
        if feat.shape[0] != bucket_id.shape[0] or scattered_feat.shape[0] != scatter_idx_out2in.shape[0]:
            raise RuntimeError("feat needs one row per point and scattered_feat one per index entry")
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([bucket_counter, bucket_offset, batch_sep, cumsum_counter, scatter_idx_out2in], torch.uint32)
    assert_dtype([bucket_id], torch.uint16)
    if bucket_counter.shape != cumsum_counter.shape or bucket_counter.shape[0] != batch_sep.shape[0]:
        raise RuntimeError("bucket_counter and cumsum_counter must both be [batch, num_bucket]")
    row_bytes = 0 if feat is None else _row_bytes(feat)
    _check(_load().f3d_psh_scatter_feat_index(
        _ptr(bucket_id), _ptr(bucket_offset), _ptr(bucket_counter), _ptr(cumsum_counter), _ptr(batch_sep),
        _u32(batch_sep.shape[0]), _u32(bucket_id.shape[0]), _u32(bucket_counter.shape[1]),
        _ptr(feat), _u32(row_bytes), _ptr(scatter_idx_out2in), _ptr(scattered_feat),
        _u32(scatter_idx_out2in.shape[0]), _i32(dev), _stream(dev)))


def permute_rows(index, src, dst, gather: bool):
    """Row permutation by a PSH index.  gather: dst[r] = src[index[r]] (zero where index[r] >= len(src)), dst has
    len(index) rows.  not gather: dst[index[r]] = src[r] where index[r] < len(dst), src has len(index) rows."""
    ts = [index, src, dst]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([index], torch.uint32)
    if src.dtype != dst.dtype or src.shape[1:] != dst.shape[1:]:
        raise RuntimeError(f"src {tuple(src.shape)} {src.dtype} and dst {tuple(dst.shape)} {dst.dtype} differ in row "
                           f"shape or dtype")
    n_index, n_other = ((dst.shape[0], src.shape[0]) if gather else (src.shape[0], dst.shape[0]))
    if index.shape[0] != n_index:
        raise RuntimeError(f"index has {index.shape[0]} entries, the indexed side {n_index} rows")
    if n_index == 0:
        return
    if n_other == 0:
        if gather:
            dst.zero_()
        return
    _check(_load().f3d_permute_rows(_ptr(index), _ptr(src), _ptr(dst), _u32(n_index), _u32(n_other),
                                    _u32(_row_bytes(src)), _u32(1 if gather else 0), _i32(dev),
                                    _stream(dev)))


def coord_bbox(coord, bbox_min, bbox_max):
    """extension: one-pass whole-batch bounding box (replaces torch.min/max of psh_main.py:117-118)"""
    assert_contiguous([coord, bbox_min, bbox_max])
    dev = assert_same_device([coord, bbox_min, bbox_max])
    assert_dtype([coord, bbox_min, bbox_max], torch.float16)
    _check(_load().f3d_coord_bbox(_ptr(coord), _u32(coord.shape[0]), _ptr(bbox_min), _ptr(bbox_max), _i32(dev),
                                  _stream(dev)))


def batch_bucket_sanitizer_cpu(bucket_id, bucket_counter, bucket_offset, offset_check_table, bucket_residual,
                               batch_sep, offset_maxcnt, batch_size, num_bucket):
    """src/psh/bucket_sanitizer_cpu.cpp:92-176 — host-side scoreboard: every (cloud, bucket,
    slot < count) must be claimed exactly once.  Raises RuntimeError on the first violation and
    writes the residual counts / hit table back, like the reference."""
    ids = bucket_id.cpu().to(torch.int64)
    cnt = bucket_counter.cpu().to(torch.int64)
    off = bucket_offset.cpu().to(torch.int64)
    seps = batch_sep.cpu().to(torch.int64)
    maxcnt = offset_maxcnt.cpu().to(torch.int64)
    table = offset_check_table.cpu().to(torch.int64)
    res = bucket_residual.cpu().to(torch.int64)
    start = 0
    for b in range(batch_size):
        end = int(seps[b])
        i, o = ids[start:end], off[start:end]
        bad = (i >= num_bucket) | (o >= maxcnt[b])
        if bool(bad.any()):
            c = int(torch.nonzero(bad)[0]) + start
            raise RuntimeError(f"col={c}: buckid={int(ids[c])}|num_bucket={num_bucket}, "
                               f"buckoff={int(off[c])}|offset_maxcnt={int(maxcnt[b])}, overflow ")
        res[b] -= torch.bincount(i, minlength=num_bucket)[:num_bucket]
        flat = table[b].reshape(-1)
        flat += torch.bincount(i * table.shape[2] + o, minlength=flat.numel())
        start = end
    for b in range(batch_size):
        slot = torch.arange(table.shape[2])[None, :]
        wrong = (slot < cnt[b][:, None]) & (table[b] != 1)
        if bool(wrong.any()):
            k, s = [int(x) for x in torch.nonzero(wrong)[0]]
            raise RuntimeError(f"Wrong scoreboard, batchid={b} buck={k},[Slot={s}|MaxCnt={int(cnt[b, k])}],"
                               f"Score={int(table[b, k, s])}")
    bucket_residual.copy_(res.to(bucket_residual.dtype))
    offset_check_table.copy_(table.to(offset_check_table.dtype))


# ---------------------------------------------------------------------------------------------
# sub-bucket pooling / additive unpool
# ---------------------------------------------------------------------------------------------

def batch_subbuck_reduce(scattered_coord, scattered_feat, batch_sep, instance_max_N, subbuck_size, num_vox,
                         bbox_min, bbox_max, subbuck_id, subbuck_off, reduced_batch_sep, reduced_coord,
                         reduced_feat, unpool_ind, hash_type, red_op):
    """src/f3d_frontend.cu:60-66 -> src/psh/batch_subbuck_pooling_dispatcher.cu:35-144"""
    ts = [scattered_coord, scattered_feat, batch_sep, subbuck_id, subbuck_off, reduced_batch_sep, reduced_coord,
          reduced_feat]
    assert_contiguous(ts + [unpool_ind])
    dev = assert_same_device(ts + [unpool_ind])
    assert_dtype([scattered_feat, reduced_feat], torch.bfloat16)
    assert_dtype([scattered_coord, reduced_coord, bbox_min, bbox_max], torch.float16)
    assert_dtype([batch_sep, subbuck_id, reduced_batch_sep, unpool_ind], torch.uint32)
    assert_dtype([subbuck_off], torch.uint16)
    if scattered_feat.shape[1] != reduced_feat.shape[1]:
        raise RuntimeError(f"Input feature dim({scattered_feat.shape[1]}) != output feature dim({reduced_feat.shape[1]}).")
    if reduced_coord.shape[0] != reduced_feat.shape[0]:
        raise RuntimeError(f"Reduced coordinate length({reduced_coord.shape[0]}) != reduced feature length({reduced_feat.shape[0]}).")
    if scattered_coord.shape[1] != 3 or reduced_coord.shape[1] != 3:
        raise RuntimeError(f"Input coordinates dim({scattered_coord.shape[1]}) or reduced coordinates "
                           f"dim({reduced_coord.shape[1]}) are NOT 3D.")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"Unpool_ind last dimension({unpool_ind.shape[1]}) != subbucket_size({subbuck_size})")
    # Rows of the feature tensor beyond the coordinate count are ignored, as in the reference
    # (total_N is taken from the coordinates, dispatcher :43).
    _check(_load().f3d_batch_subbuck_reduce(
        _ptr(scattered_coord), _ptr(scattered_feat), _ptr(batch_sep), _u32(batch_sep.shape[0]),
        _u32(scattered_coord.shape[0]), _u32(instance_max_N), _u32(scattered_feat.shape[1]), _u32(subbuck_size),
        _u32(num_vox), _ptr(bbox_min.contiguous()), _ptr(bbox_max.contiguous()), _ptr(subbuck_id), _ptr(subbuck_off),
        _ptr(reduced_batch_sep), _ptr(reduced_coord), _ptr(reduced_feat), _u32(reduced_feat.shape[0]),
        _ptr(unpool_ind), _u32(unpool_ind.shape[0]), _u32(hash_type), _u32(red_op), _i32(dev), _stream(dev)))


def batch_subbuck_reduce_backward(grad_red_feat, input_feat, unpool_ind, grad_input_feat, subbuck_size, red_op):
    """src/f3d_frontend.cu:68-71 -> src/psh/batch_subbuck_pooling_bwd_dispatcher.cu: gradient of the feature reduce.
    grad_red_feat [>= R, C], input_feat / grad_input_feat [N, C] bf16, unpool_ind [R, S] uint32.  Rows of
    grad_input_feat that no slot refers to keep the caller's content (the reference passes zeros)."""
    ts = [grad_red_feat, input_feat, unpool_ind, grad_input_feat]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([grad_red_feat, input_feat, grad_input_feat], torch.bfloat16)
    assert_dtype([unpool_ind], torch.uint32)
    if input_feat.shape != grad_input_feat.shape:
        raise RuntimeError(f"input_feat shape {tuple(input_feat.shape)} != grad_input_feat shape {tuple(grad_input_feat.shape)}")
    if grad_red_feat.shape[1] != input_feat.shape[1] or grad_red_feat.shape[0] < unpool_ind.shape[0]:
        raise RuntimeError(f"grad_red_feat shape {tuple(grad_red_feat.shape)} does not cover unpool_ind {tuple(unpool_ind.shape)}")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"unpool_ind width {unpool_ind.shape[1]} != subbuck_size {subbuck_size}")
    _check(_load().f3d_subbuck_reduce_bwd(
        _ptr(grad_red_feat), _ptr(input_feat), _ptr(unpool_ind), _ptr(grad_input_feat), _u32(input_feat.shape[0]),
        _u32(unpool_ind.shape[0]), _u32(input_feat.shape[1]), _u32(subbuck_size), _u32(red_op), _i32(dev), _stream(dev)))


def additive_unpool_fwd(res_feat, down_feat, up_add_feat, unpool_ind, subbuck_size):
    """src/f3d_frontend.cu:99-101 -> src/psh/additive_unpool_dispatcher.cu:26-79"""
    ts = [res_feat, down_feat, up_add_feat, unpool_ind]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([res_feat, down_feat, up_add_feat], torch.bfloat16)
    assert_dtype([unpool_ind], torch.uint32)
    if res_feat.shape != up_add_feat.shape:
        raise RuntimeError(f"res_feat shape {tuple(res_feat.shape)} != up_add_feat shape {tuple(up_add_feat.shape)}")
    if res_feat.shape[1] != down_feat.shape[1]:
        raise RuntimeError(f"Feature dim mismatch: res({res_feat.shape[1]}) vs down({down_feat.shape[1]})")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"Unpool_ind last dimension({unpool_ind.shape[1]}) != subbucket_size({subbuck_size})")
    if down_feat.shape[0] < unpool_ind.shape[0]:
        raise RuntimeError(f"down_feat has {down_feat.shape[0]} rows, unpool_ind needs {unpool_ind.shape[0]}")
    _check(_load().f3d_additive_unpool_fwd(
        _ptr(res_feat), _ptr(down_feat), _ptr(up_add_feat), _ptr(unpool_ind), _u32(res_feat.shape[0]),
        _u32(unpool_ind.shape[0]), _u32(res_feat.shape[1]), _u32(subbuck_size), _i32(dev), _stream(dev)))


ROW_NORM_LAYER, ROW_NORM_AFFINE = 1, 2


def _row_norm_args(norm, c):
    """(mode, gamma, beta, scale, shift, eps) of one branch -> ctypes arguments; norm = ("layer", gamma16, beta16 | None,
    eps) or ("affine", scale32, shift32)"""
    if norm[0] == "layer":
        _, g, b, eps = norm
        assert_dtype([g] + ([b] if b is not None else []), torch.bfloat16)
        if g.numel() != c or (b is not None and b.numel() != c):
            raise RuntimeError(f"LayerNorm parameters must hold {c} values")
        return ROW_NORM_LAYER, [_ptr(g), _ptr(b), _vp(0), _vp(0), _f32(eps)]
    _, sc, sh = norm
    assert_dtype([sc, sh], torch.float32)
    if sc.numel() != c or sh.numel() != c:
        raise RuntimeError(f"scale / shift must hold {c} values")
    return ROW_NORM_AFFINE, [_vp(0), _vp(0), _ptr(sc), _ptr(sh), _f32(0.0)]


def subbuck_build(scattered_coord, batch_sep, instance_max_N, subbuck_size, num_vox, subbuck_id, subbuck_off,
                  reduced_batch_sep, reduced_coord, unpool_ind):
    """the first half of batch_subbuck_reduce alone (local_subbuck_ker, src/psh/batch_psh_subbuck_reduce.cuh:104-298):
    sub-bucket ids / offsets, the inverse map and the reduced coordinates"""
    ts = [scattered_coord, batch_sep, subbuck_id, subbuck_off, reduced_batch_sep, reduced_coord, unpool_ind]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([scattered_coord, reduced_coord], torch.float16)
    assert_dtype([batch_sep, subbuck_id, reduced_batch_sep, unpool_ind], torch.uint32)
    assert_dtype([subbuck_off], torch.uint16)
    if scattered_coord.shape[1] != 3 or reduced_coord.shape[1] != 3:
        raise RuntimeError(f"Input coordinates dim({scattered_coord.shape[1]}) or reduced coordinates "
                           f"dim({reduced_coord.shape[1]}) are NOT 3D.")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"Unpool_ind last dimension({unpool_ind.shape[1]}) != subbucket_size({subbuck_size})")
    _check(_load().f3d_subbuck_build(
        _ptr(scattered_coord), _ptr(batch_sep), _u32(batch_sep.shape[0]), _u32(scattered_coord.shape[0]),
        _u32(instance_max_N), _u32(subbuck_size), _u32(num_vox), _ptr(subbuck_id), _ptr(subbuck_off),
        _ptr(reduced_batch_sep), _ptr(reduced_coord), _u32(reduced_coord.shape[0]), _ptr(unpool_ind),
        _u32(unpool_ind.shape[0]), _i32(dev), _stream(dev)))


def reduce_feat_norm(feat, total_n, unpool_ind, reduced_feat, subbuck_size, red_op, norm, act=None):
    """extension: the feature reduce of batch_subbuck_reduce (reduce_feat_ker, src/psh/batch_psh_subbuck_reduce.cuh:300-359)
    with the pooling wrapper's norm (and activation) applied to every reduced row before it is stored; total_n = number of
    points (rows of feat beyond it are ignored).  norm = ("layer", gamma bf16, beta bf16 | None, eps) or
    ("affine", scale fp32, shift fp32)"""
    if total_n > feat.shape[0]:
        raise RuntimeError(f"feat has {feat.shape[0]} rows, total_n is {total_n}")
    assert_contiguous([feat, unpool_ind, reduced_feat])
    dev = assert_same_device([feat, unpool_ind, reduced_feat])
    assert_dtype([feat, reduced_feat], torch.bfloat16)
    assert_dtype([unpool_ind], torch.uint32)
    if feat.shape[1] != reduced_feat.shape[1]:
        raise RuntimeError(f"Input feature dim({feat.shape[1]}) != output feature dim({reduced_feat.shape[1]}).")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"Unpool_ind last dimension({unpool_ind.shape[1]}) != subbucket_size({subbuck_size})")
    mode, nargs = _row_norm_args(norm, feat.shape[1])
    a = ACT[act] if not isinstance(act, int) else act
    _check(_load().f3d_reduce_feat_norm(
        _ptr(feat), _u32(total_n), _u32(feat.shape[1]), _ptr(unpool_ind), _u32(unpool_ind.shape[0]), _u32(subbuck_size),
        _u32(red_op), _ptr(reduced_feat), _u32(reduced_feat.shape[0]), _u32(mode), *nargs, _u32(a), _i32(dev),
        _stream(dev)))


def additive_unpool_norm_fwd(res_feat, down_feat, up_add_feat, unpool_ind, subbuck_size, norm_res, norm_down, act=None):
    """extension: additive_unpool_fwd with both operands normalised on the way in (the unpooling wrapper's
    Linear -> norm -> activation branches, flash3dxfmr/layers/hourglass.py:152-159); norm_* as in reduce_feat_norm,
    both of the same kind"""
    ts = [res_feat, down_feat, up_add_feat, unpool_ind]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([res_feat, down_feat, up_add_feat], torch.bfloat16)
    assert_dtype([unpool_ind], torch.uint32)
    if res_feat.shape != up_add_feat.shape:
        raise RuntimeError(f"res_feat shape {tuple(res_feat.shape)} != up_add_feat shape {tuple(up_add_feat.shape)}")
    if res_feat.shape[1] != down_feat.shape[1]:
        raise RuntimeError(f"Feature dim mismatch: res({res_feat.shape[1]}) vs down({down_feat.shape[1]})")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"Unpool_ind last dimension({unpool_ind.shape[1]}) != subbucket_size({subbuck_size})")
    if down_feat.shape[0] < unpool_ind.shape[0]:
        raise RuntimeError(f"down_feat has {down_feat.shape[0]} rows, unpool_ind needs {unpool_ind.shape[0]}")
    if norm_res[0] != norm_down[0]:
        raise RuntimeError("both branches must use the same kind of normalisation")
    mode, ra = _row_norm_args(norm_res, res_feat.shape[1])
    _, da = _row_norm_args(norm_down, res_feat.shape[1])
    a = ACT[act] if not isinstance(act, int) else act
    _check(_load().f3d_additive_unpool_norm_fwd(
        _ptr(res_feat), _ptr(down_feat), _ptr(up_add_feat), _ptr(unpool_ind), _u32(res_feat.shape[0]),
        _u32(unpool_ind.shape[0]), _u32(res_feat.shape[1]), _u32(subbuck_size), _u32(mode), *ra, *da, _u32(a), _i32(dev),
        _stream(dev)))


def additive_unpool_bwd(grad_res, grad_down, grad_up_added, unpool_ind, subbuck_size):
    """src/f3d_frontend.cu:103-105 -> src/psh/additive_unpool_dispatcher.cu:81-134: grad_res[r] = grad_up_added[r]
    for every pooled point r, grad_down[i] = sum over the points pooled into row i.  Rows of grad_res that no slot
    refers to keep the caller's content (the reference passes zeros)."""
    ts = [grad_res, grad_down, grad_up_added, unpool_ind]
    assert_contiguous(ts)
    dev = assert_same_device(ts)
    assert_dtype([grad_res, grad_down, grad_up_added], torch.bfloat16)
    assert_dtype([unpool_ind], torch.uint32)
    if grad_res.shape != grad_up_added.shape:
        raise RuntimeError(f"grad_res shape {tuple(grad_res.shape)} != grad_up_added shape {tuple(grad_up_added.shape)}")
    if grad_down.shape[1] != grad_res.shape[1] or grad_down.shape[0] < unpool_ind.shape[0]:
        raise RuntimeError(f"grad_down shape {tuple(grad_down.shape)} does not cover unpool_ind {tuple(unpool_ind.shape)}")
    if unpool_ind.shape[1] != subbuck_size:
        raise RuntimeError(f"unpool_ind width {unpool_ind.shape[1]} != subbuck_size {subbuck_size}")
    _check(_load().f3d_additive_unpool_bwd(
        _ptr(grad_res), _ptr(grad_down), _ptr(grad_up_added), _ptr(unpool_ind), _u32(grad_res.shape[0]),
        _u32(unpool_ind.shape[0]), _u32(grad_res.shape[1]), _u32(subbuck_size), _i32(dev), _stream(dev)))


# ---------------------------------------------------------------------------------------------
# bucketed attention
# ---------------------------------------------------------------------------------------------

def buck_swin_fwd(Q, K, V, O, L, Scope_buckets, bucket_size, kv_len=None):
    """declared src/f3d_frontend.cu:90-92, called at flash3dxfmr/layers/buck_swin.py:57.
    Q,K,V,O [B,L,H,D] bf16; L (LSE) [B,L,H] fp32; Scope_buckets [n_scope, scope_size] uint32.
    Q/K/V may be column slices of one [B,L,3*H*D] projection output (equal row strides, dense last
    two axes); O and L must be contiguous.  ``kv_len`` (extension) int32 [L/bucket_size]."""
    dev = assert_same_device([Q, K, V, O, L, Scope_buckets])
    assert_dtype([Q, K, V, O], torch.bfloat16)
    assert_dtype([L], torch.float32)
    assert_dtype([Scope_buckets], torch.uint32)
    assert_contiguous([O, L, Scope_buckets])
    if Q.dim() != 4 or Q.shape != K.shape or Q.shape != V.shape or Q.shape != O.shape:
        raise RuntimeError(f"Q/K/V/O must share one [B,L,H,D] shape, got {tuple(Q.shape)} {tuple(K.shape)} "
                           f"{tuple(V.shape)} {tuple(O.shape)}")
    B, Ls, H, D = Q.shape
    if tuple(L.shape) != (B, Ls, H):
        raise RuntimeError(f"LSE shape {tuple(L.shape)} != {(B, Ls, H)}")
    if Scope_buckets.dim() != 2:
        raise RuntimeError("Scope_buckets must be [num_scopes, scope_size]")
    for t in (Q, K, V):
        if t.stride(3) != 1 or t.stride(2) != D or t.stride(0) != t.stride(1) * Ls or t.stride() != Q.stride():
            raise RuntimeError("Q/K/V must be dense over (H, D) with identical strides")
    if kv_len is not None:
        assert_dtype([kv_len], torch.int32)
        assert_contiguous([kv_len])
    _check(_load().f3d_buck_swin_fwd_strided(
        _ptr(Q), _ptr(K), _ptr(V), _u32(Q.stride(1)), _ptr(O), _ptr(L), _ptr(Scope_buckets),
        _u32(Scope_buckets.shape[0]), _u32(Scope_buckets.shape[1]), _u32(bucket_size), _u32(B), _u32(Ls), _u32(H),
        _u32(D), _ptr(kv_len), _i32(dev), _stream(dev)))


def buck_swin_bwd(Q, K, V, O, dO, LSE, Delta, dQ, dK, dV, Scope_buckets, bucket_size, kv_len=None):
    """declared src/f3d_frontend.cu:94-97, called at flash3dxfmr/layers/buck_swin.py:90-92.
    Q, K, V [B,L,H,D] bf16 (may be column slices of one projection output, equal strides); O, dO dense [B,L,H,D]
    bf16; dQ, dK, dV [B,L,H,D] bf16, dense or (extension) column slices of one [B,L,3HD] gradient tensor with equal
    strides; LSE (from the forward), Delta (written here: rowsum(dO * O)) [B,L,H] fp32.  Rows that no scope
    covers are not written (pass zero-filled dQ / dK / dV).  head_dim 16, 32, 64 or 128; scopes of any number of
    buckets.  kv_len (extension, as in the forward): int32 [L / bucket_size] valid rows per bucket."""
    dev = assert_same_device([Q, K, V, O, dO, LSE, Delta, dQ, dK, dV, Scope_buckets] +
                             ([kv_len] if kv_len is not None else []))
    if kv_len is not None:
        assert_dtype([kv_len], torch.int32)
        assert_contiguous([kv_len])
        if kv_len.numel() != Q.shape[1] // bucket_size:
            raise RuntimeError(f"kv_len must have L / bucket_size = {Q.shape[1] // bucket_size} entries")
    assert_dtype([Q, K, V, O, dO, dQ, dK, dV], torch.bfloat16)
    assert_dtype([LSE, Delta], torch.float32)
    assert_dtype([Scope_buckets], torch.uint32)
    assert_contiguous([O, dO, LSE, Delta, Scope_buckets])
    if Q.dim() != 4 or any(t.shape != Q.shape for t in (K, V, O, dO, dQ, dK, dV)):
        raise RuntimeError("Q/K/V/O/dO/dQ/dK/dV must share one [B,L,H,D] shape")
    B, Ls, H, D = Q.shape
    if tuple(LSE.shape) != (B, Ls, H) or tuple(Delta.shape) != (B, Ls, H):
        raise RuntimeError(f"LSE / Delta shape must be {(B, Ls, H)}")
    if Scope_buckets.dim() != 2:
        raise RuntimeError("Scope_buckets must be [num_scopes, scope_size]")
    for t in (Q, K, V):
        if t.stride(3) != 1 or t.stride(2) != D or t.stride(0) != t.stride(1) * Ls or t.stride() != Q.stride():
            raise RuntimeError("Q/K/V must be dense over (H, D) with identical strides")
    for t in (dQ, dK, dV):
        if t.stride(3) != 1 or t.stride(2) != D or t.stride(0) != t.stride(1) * Ls or t.stride() != dQ.stride():
            raise RuntimeError("dQ/dK/dV must be dense over (H, D) with identical strides")
    rc = _load().f3d_buck_swin_bwd_strided(
        _ptr(Q), _ptr(K), _ptr(V), _u32(Q.stride(1)), _ptr(O), _ptr(dO), _ptr(LSE), _ptr(Delta), _ptr(dQ), _ptr(dK),
        _ptr(dV), _u32(dQ.stride(1)), _ptr(Scope_buckets), _u32(Scope_buckets.shape[0]), _u32(Scope_buckets.shape[1]), _u32(bucket_size),
        _u32(B), _u32(Ls), _u32(H), _u32(D), _ptr(kv_len), _i32(dev), _stream(dev))
    if rc == 2:   # F3D_ERR_UNSUPPORTED: a shape outside the backward kernels
        raise NotImplementedError(_load().f3d_last_error().decode("utf-8", "replace"))
    _check(rc)


# ---------------------------------------------------------------------------------------------
# dense layers
# ---------------------------------------------------------------------------------------------

def gemm_sm_bf16(A, B, O):
    """src/f3d_frontend.cu:87-88: O[M,N] = A[M,K] @ B[K,N], bf16 in/out, fp32 accumulate"""
    assert_contiguous([A, B, O])
    dev = assert_same_device([A, B, O])
    assert_dtype([A, B, O], torch.bfloat16)
    M, K = A.shape
    K2, N = B.shape
    if K != K2 or tuple(O.shape) != (M, N):
        raise RuntimeError(f"gemm shape mismatch: A{tuple(A.shape)} B{tuple(B.shape)} O{tuple(O.shape)}")
    _check(_load().f3d_gemm_sm_bf16(_ptr(A), _ptr(B), _ptr(O), _u32(M), _u32(N), _u32(K), _i32(dev), _stream(dev)))
    torch.cuda.current_stream(dev).synchronize()  # the reference op always synchronises (gemm_dispatcher.cu:77)


ACT = {None: 0, "none": 0, "gelu": 1, "swiglu": 2, "silu": 3, "relu": 4}


def linear_bf16(x, w, bias, residual, y, act=None):
    """extension: y = act(x @ w.T + bias) + residual on MFMA (the nn.Linear / te.Linear sites)"""
    dev = assert_same_device([x, w, y])
    assert_dtype([x, w, y], torch.bfloat16)
    assert_contiguous([w])
    if x.dim() != 2 or y.dim() != 2 or x.stride(1) != 1 or y.stride(1) != 1:
        raise RuntimeError("linear_bf16 expects 2-D row-major x and y")
    m, k = x.shape
    n = w.shape[0]
    a = ACT[act] if not isinstance(act, int) else act
    n_out = n // 2 if a == 2 else n
    if w.shape[1] != k or tuple(y.shape) != (m, n_out):
        raise RuntimeError(f"linear shape mismatch: x{tuple(x.shape)} w{tuple(w.shape)} y{tuple(y.shape)}")
    _check_vectors(x, [bias])
    ldr = 0
    if residual is not None:
        assert_same_device([x, residual])
        assert_dtype([residual], torch.bfloat16)
        if tuple(residual.shape) != (m, n_out) or residual.stride(1) != 1:
            raise RuntimeError("residual must be [m, n_out] row-major")
        ldr = residual.stride(0)
    _check(_load().f3d_linear_bf16(_ptr(x), _u32(x.stride(0)), _ptr(w), _ptr(bias), _ptr(residual), _u32(ldr),
                                   _ptr(y), _u32(y.stride(0)), _u32(m), _u32(n), _u32(k), _u32(a), _i32(dev),
                                   _stream(dev)))


def ln_linear_bf16(x, gamma, beta, eps, w, bias, residual, y, act=None):
    """extension: y = act(LayerNorm(x) @ w.T + bias) + residual in one kernel (K in 32..512)"""
    dev = assert_same_device([x, gamma, w, y])
    assert_dtype([x, gamma, w, y], torch.bfloat16)
    assert_contiguous([w, gamma])
    if x.dim() != 2 or y.dim() != 2 or x.stride(1) != 1 or y.stride(1) != 1:
        raise RuntimeError("ln_linear_bf16 expects 2-D row-major x and y")
    m, k = x.shape
    n = w.shape[0]
    a = ACT[act] if not isinstance(act, int) else act
    n_out = n // 2 if a == 2 else n
    if w.shape[1] != k or tuple(y.shape) != (m, n_out) or gamma.shape[0] != k:
        raise RuntimeError(f"ln_linear shape mismatch: x{tuple(x.shape)} w{tuple(w.shape)} y{tuple(y.shape)}")
    _check_vectors(x, [beta, bias])
    ldr = 0
    if residual is not None:
        assert_same_device([x, residual])
        assert_dtype([residual], torch.bfloat16)
        if tuple(residual.shape) != (m, n_out) or residual.stride(1) != 1:
            raise RuntimeError("residual must be [m, n_out] row-major")
        ldr = residual.stride(0)
    _check(_load().f3d_ln_linear_bf16(_ptr(x), _u32(x.stride(0)), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w),
                                      _ptr(bias), _ptr(residual), _u32(ldr), _ptr(y), _u32(y.stride(0)), _u32(m),
                                      _u32(n), _u32(k), _u32(a), _i32(dev), _stream(dev)))


def ln_mlp_swiglu_bf16(x, gamma, beta, eps, w1, b1, w2, b2, residual, y) -> bool:
    """extension: y = (silu(LN(x) w1[:h].T + b1[:h]) * (LN(x) w1[h:].T + b1[h:])) w2.T + b2 (+ residual) in one kernel
    (te.LayerNormMLP with swiglu + the residual add, elem_wise.py:22-26, stage.py:94-97).  Returns False, leaving y
    untouched, when no fused kernel covers the widths (the caller then runs ln_linear_bf16 + linear_bf16)."""
    dev = assert_same_device([x, gamma, w1, w2, y])
    assert_dtype([x, gamma, w1, w2, y], torch.bfloat16)
    assert_contiguous([w1, w2, gamma])
    _check_vectors(x, [beta, b1, b2])
    if x.dim() != 2 or y.dim() != 2 or x.stride(1) != 1 or y.stride(1) != 1:
        raise RuntimeError("ln_mlp_swiglu_bf16 expects 2-D row-major x and y")
    m, c = x.shape
    hidden = w2.shape[1]
    if tuple(w1.shape) != (2 * hidden, c) or w2.shape[0] != c or tuple(y.shape) != (m, c) or gamma.shape[0] != c:
        raise RuntimeError(f"ln_mlp shape mismatch: x{tuple(x.shape)} w1{tuple(w1.shape)} w2{tuple(w2.shape)} "
                           f"y{tuple(y.shape)}")
    ldr = 0
    if residual is not None:
        assert_dtype([residual], torch.bfloat16)
        if tuple(residual.shape) != (m, c) or residual.stride(1) != 1:
            raise RuntimeError("residual must be [m, c] row-major")
        ldr = residual.stride(0)
    rc = _load().f3d_ln_mlp_swiglu_bf16(_ptr(x), _u32(x.stride(0)), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w1),
                                        _ptr(b1), _ptr(w2), _ptr(b2), _ptr(residual), _u32(ldr), _ptr(y),
                                        _u32(y.stride(0)), _u32(m), _u32(c), _u32(hidden), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def embed_table(w: torch.Tensor, bias) -> torch.Tensor:
    """[c, 8] bf16 rows (w[c,0], w[c,1], w[c,2], bias[c], 0, 0, 0, 0): the coordinate embedding's parameters as the
    kernels that form the embedding themselves read them"""
    c = w.shape[0]
    t = torch.zeros(c, 8, dtype=torch.bfloat16, device=w.device)
    t[:, :3] = w.detach().to(torch.bfloat16)
    if bias is not None:
        t[:, 3] = bias.detach().to(torch.bfloat16)
    return t


def embed_ln_linear_bf16(coord, table, gamma, beta, eps, w, bias, y) -> bool:
    """extension: y = LayerNorm(embed(coord)) w.T + bias with the coordinate embedding (psh_ops.py:64-68) formed inside
    the kernel instead of read from memory; `table` from embed_table().  Returns False, leaving y untouched, when no
    kernel covers the widths (the caller then runs coord_embed_bf16 + ln_linear_bf16)."""
    dev = assert_same_device([coord, table, gamma, w, y])
    assert_dtype([coord], torch.float16)
    assert_dtype([table, gamma, w, y], torch.bfloat16)
    assert_contiguous([coord, table, gamma, w])
    _check_vectors(y, [beta, bias])
    m = coord.shape[0]
    n, k = w.shape
    if (coord.dim() != 2 or coord.shape[1] != 3 or tuple(table.shape) != (k, 8) or gamma.shape[0] != k
            or tuple(y.shape) != (m, n) or y.stride(1) != 1):
        raise RuntimeError(f"embed_ln_linear shape mismatch: coord{tuple(coord.shape)} table{tuple(table.shape)} "
                           f"w{tuple(w.shape)} y{tuple(y.shape)}")
    rc = _load().f3d_embed_ln_linear_bf16(_ptr(coord), _ptr(table), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w), _ptr(bias),
                                          _ptr(y), _u32(y.stride(0)), _u32(m), _u32(n), _u32(k), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def embed_qkv_fold(embed_w, embed_b, gamma, beta, eps, w_qkv, b_qkv, num_heads: int):
    """extension: LayerNorm + QKV projection of the coordinate embedding (psh_ops.py:64-68 -> stage.py:94-96) folded
    into what embed_buck_swin_fwd reads: a table [num_heads, 4, 32, 16] bf16 (per head the Q tile in the exponent's
    units, K, V, and Q unscaled) and 16 floats (Cholesky factor of the embedding's centred Gram matrix, eps).
    Returns None when no kernel covers the head width."""
    dev = assert_same_device([embed_w, gamma, w_qkv])
    assert_dtype([embed_w, gamma, w_qkv], torch.bfloat16)
    assert_contiguous([embed_w, gamma, w_qkv])
    c = embed_w.shape[0]
    if tuple(embed_w.shape) != (c, 3) or tuple(w_qkv.shape) != (3 * c, c) or gamma.shape[0] != c or c % num_heads:
        raise RuntimeError(f"embed_qkv_fold shape mismatch: embed_w{tuple(embed_w.shape)} w_qkv{tuple(w_qkv.shape)}")
    for v, n in ((embed_b, c), (beta, c), (b_qkv, 3 * c)):
        if v is not None:
            assert_dtype([v], torch.bfloat16)
            assert_contiguous([v])
            if v.numel() != n:
                raise RuntimeError("embed_qkv_fold: bias / beta length mismatch")
    table = torch.empty(num_heads, 4, 32, 16, dtype=torch.bfloat16, device=embed_w.device)
    chol = torch.empty(16, dtype=torch.float32, device=embed_w.device)
    rc = _load().f3d_embed_qkv_fold_bf16(_ptr(embed_w), _ptr(embed_b), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w_qkv),
                                         _ptr(b_qkv), _u32(c), _u32(num_heads), _u32(c // num_heads), _ptr(table),
                                         _ptr(chol), _i32(dev), _stream(dev))
    if rc == 2:
        return None
    _check(rc)
    return table, chol


def embed_buck_swin_fwd(coord, table, chol, O, L, Scope_buckets, bucket_size) -> bool:
    """extension: buck_swin_fwd of the first block with Q, K and V formed inside the kernel from the rows' coordinates
    (coord [B * L, 3] fp16, table / chol from embed_qkv_fold) instead of read from a projection output.  O [B,L,H,32]
    bf16, L (LSE) [B,L,H] fp32.  Returns False, leaving O untouched, when no kernel covers the shape (scopes of 256 or
    512 tokens, 32-wide heads)."""
    dev = assert_same_device([coord, table, chol, O, L, Scope_buckets])
    assert_dtype([coord], torch.float16)
    assert_dtype([table, O], torch.bfloat16)
    assert_dtype([chol, L], torch.float32)
    assert_dtype([Scope_buckets], torch.uint32)
    assert_contiguous([coord, table, chol, O, L, Scope_buckets])
    if O.dim() != 4:
        raise RuntimeError(f"O must be [B,L,H,D], got {tuple(O.shape)}")
    B, Ls, H, D = O.shape
    if (coord.dim() != 2 or tuple(coord.shape) != (B * Ls, 3) or tuple(table.shape) != (H, 4, 32, 16) or chol.numel() != 16
            or tuple(L.shape) != (B, Ls, H) or Scope_buckets.dim() != 2):
        raise RuntimeError(f"embed_buck_swin_fwd shape mismatch: coord{tuple(coord.shape)} table{tuple(table.shape)} "
                           f"O{tuple(O.shape)} L{tuple(L.shape)}")
    rc = _load().f3d_embed_buck_swin_fwd(_ptr(coord), _ptr(table), _ptr(chol), _ptr(O), _ptr(L), _ptr(Scope_buckets),
                                         _u32(Scope_buckets.shape[0]), _u32(Scope_buckets.shape[1]), _u32(bucket_size),
                                         _u32(B), _u32(Ls), _u32(H), _u32(D), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def proj_ln_mlp_swiglu_bf16(a, w_proj, b_proj, x, gamma, beta, eps, w1, b1, w2, b2, y) -> bool:
    """extension: the second half of a block in one kernel (stage.py:92-102): x1 = a w_proj.T + b_proj + x, then
    y = x1 + MLP(LayerNorm(x1)) with the gated MLP of ln_mlp_swiglu_bf16; x1 never reaches memory.  Returns False,
    leaving y untouched, when no kernel covers the widths (the caller then runs linear_bf16 + ln_mlp_swiglu_bf16)."""
    dev = assert_same_device([a, w_proj, x, gamma, w1, w2, y])
    assert_dtype([a, w_proj, x, gamma, w1, w2, y], torch.bfloat16)
    assert_contiguous([w_proj, w1, w2, gamma])
    _check_vectors(x, [b_proj, beta, b1, b2])
    if any(t.dim() != 2 or t.stride(1) != 1 for t in (a, x, y)):
        raise RuntimeError("proj_ln_mlp_swiglu_bf16 expects 2-D row-major a, x and y")
    m, c = x.shape
    hidden = w2.shape[1]
    if (tuple(a.shape) != (m, c) or tuple(w_proj.shape) != (c, c) or tuple(w1.shape) != (2 * hidden, c) or w2.shape[0] != c
            or tuple(y.shape) != (m, c) or gamma.shape[0] != c):
        raise RuntimeError(f"proj_ln_mlp shape mismatch: a{tuple(a.shape)} x{tuple(x.shape)} w_proj{tuple(w_proj.shape)} "
                           f"w1{tuple(w1.shape)} w2{tuple(w2.shape)} y{tuple(y.shape)}")
    rc = _load().f3d_proj_ln_mlp_swiglu_bf16(_ptr(a), _u32(a.stride(0)), _ptr(w_proj), _ptr(b_proj), _ptr(x),
                                             _u32(x.stride(0)), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w1), _ptr(b1),
                                             _ptr(w2), _ptr(b2), _ptr(y), _u32(y.stride(0)), _u32(m), _u32(c),
                                             _u32(hidden), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def embed_proj_ln_mlp_swiglu_bf16(a, w_proj, b_proj, coord, table, gamma, beta, eps, w1, b1, w2, b2, y) -> bool:
    """extension: proj_ln_mlp_swiglu_bf16 with the block input x = embed(coord) formed inside the kernel (the first block
    behind PSH3DCoordEmbedding, psh_ops.py:64-68); `table` from embed_table().  Returns False, leaving y untouched, when
    no kernel covers the widths."""
    dev = assert_same_device([a, w_proj, coord, table, gamma, w1, w2, y])
    assert_dtype([coord], torch.float16)
    assert_dtype([a, w_proj, table, gamma, w1, w2, y], torch.bfloat16)
    assert_contiguous([w_proj, w1, w2, gamma, coord, table])
    _check_vectors(y, [b_proj, beta, b1, b2])
    if any(t.dim() != 2 or t.stride(1) != 1 for t in (a, y)):
        raise RuntimeError("embed_proj_ln_mlp_swiglu_bf16 expects 2-D row-major a and y")
    m, c = a.shape
    hidden = w2.shape[1]
    if (tuple(coord.shape) != (m, 3) or tuple(table.shape) != (c, 8) or tuple(w_proj.shape) != (c, c)
            or tuple(w1.shape) != (2 * hidden, c) or w2.shape[0] != c or tuple(y.shape) != (m, c) or gamma.shape[0] != c):
        raise RuntimeError(f"embed_proj_ln_mlp shape mismatch: a{tuple(a.shape)} coord{tuple(coord.shape)} "
                           f"table{tuple(table.shape)} w_proj{tuple(w_proj.shape)} w1{tuple(w1.shape)} w2{tuple(w2.shape)} "
                           f"y{tuple(y.shape)}")
    rc = _load().f3d_embed_proj_ln_mlp_swiglu_bf16(_ptr(a), _u32(a.stride(0)), _ptr(w_proj), _ptr(b_proj), _ptr(coord),
                                                   _ptr(table), _ptr(gamma), _ptr(beta), _f32(eps), _ptr(w1), _ptr(b1),
                                                   _ptr(w2), _ptr(b2), _ptr(y), _u32(y.stride(0)), _u32(m), _u32(c),
                                                   _u32(hidden), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def stage_weights(buf: torch.Tensor, ready: bool):
    """extension: the next dense call on this thread keeps the weights it prepares (LayerNorm fold, fragment-major
    copies) in `buf` (uint8 device tensor, 256-byte aligned), or with `ready` reuses what an earlier call with the same
    weights left there and skips the preparation launch"""
    assert_dtype([buf], torch.uint8)
    _check(_load().f3d_stage_weights(_ptr(buf), ctypes.c_size_t(buf.numel()), _i32(1 if ready else 0)))


def layernorm_bf16(x, gamma, beta, y, eps=1e-5):
    """extension: LayerNorm over the last axis, fp32 statistics"""
    assert_contiguous([x, gamma, y])
    dev = assert_same_device([x, gamma, y])
    assert_dtype([x, gamma, y], torch.bfloat16)
    _check_vectors(x, [beta])
    m, c = x.shape
    _check(_load().f3d_layernorm_bf16(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _u32(m), _u32(c), _f32(eps),
                                      _i32(dev), _stream(dev)))


def _rows2d(ts, dtype=torch.bfloat16):
    for t in ts:
        if t.dim() != 2 or t.stride(1) != 1:
            raise RuntimeError("expected 2-D row-major tensors")
    assert_dtype(ts, dtype)


def linear_wgrad_bf16(dy, x, dw, db=None, accumulate=False):
    """extension: dw[n,k] (+)= dy.T @ x, db[n] (+)= dy.sum(0), fp32 outputs (gradient of y = x @ w.T + b)"""
    dev = assert_same_device([dy, x, dw])
    _rows2d([dy, x])
    assert_dtype([dw], torch.float32)
    assert_contiguous([dw])
    m, n = dy.shape
    k = x.shape[1]
    if x.shape[0] != m or tuple(dw.shape) != (n, k):
        raise RuntimeError(f"wgrad shape mismatch: dy{tuple(dy.shape)} x{tuple(x.shape)} dw{tuple(dw.shape)}")
    if db is not None:
        _check_vectors(dy, [db], torch.float32)
        if tuple(db.shape) != (n,):
            raise RuntimeError("db must be [n]")
    _check(_load().f3d_linear_wgrad_bf16(_ptr(dy), _u32(dy.stride(0)), _ptr(x), _u32(x.stride(0)), _ptr(dw), _ptr(db),
                                         _u32(m), _u32(n), _u32(k), _u32(1 if accumulate else 0), _i32(dev),
                                         _stream(dev)))


LN_BWD_WIDTHS = (32, 64, 128, 256, 512)


def layernorm_bwd_bf16(x, dh, gamma, dres, dx, dgamma, dbeta, eps=1e-5, accumulate=False):
    """extension: LayerNorm backward (dx, dgamma, dbeta) with an optional extra gradient `dres` added to dx"""
    dev = assert_same_device([x, dh, gamma, dx, dgamma, dbeta])
    _rows2d([x, dh, dx] + ([dres] if dres is not None else []))
    _check_vectors(x, [gamma])
    _check_vectors(x, [dgamma, dbeta], torch.float32)
    m, c = x.shape
    for t in (dh, dx, dres):
        if t is not None and tuple(t.shape) != (m, c):
            raise RuntimeError("layernorm_bwd: x, dh, dx, dres must share one shape")
    if tuple(gamma.shape) != (c,) or tuple(dgamma.shape) != (c,) or tuple(dbeta.shape) != (c,):
        raise RuntimeError("layernorm_bwd: gamma, dgamma, dbeta must be [c]")
    rc = _load().f3d_layernorm_bwd_bf16(_ptr(x), _u32(x.stride(0)), _ptr(dh), _u32(dh.stride(0)), _ptr(gamma),
                                        _ptr(dres), _u32(dres.stride(0) if dres is not None else 0), _ptr(dx),
                                        _u32(dx.stride(0)), _ptr(dgamma), _ptr(dbeta), _u32(m), _u32(c), _f32(eps),
                                        _u32(1 if accumulate else 0), _i32(dev), _stream(dev))
    if rc == 2:
        raise NotImplementedError(_load().f3d_last_error().decode("utf-8", "replace"))
    _check(rc)


def swiglu_bwd_bf16(z, da, dz, a=None):
    """extension: backward of a = silu(z[:, :h]) * z[:, h:]; dz may be z itself and a may be da itself"""
    dev = assert_same_device([z, da, dz])
    _rows2d([z, da, dz] + ([a] if a is not None else []))
    m, h = da.shape
    if tuple(z.shape) != (m, 2 * h) or tuple(dz.shape) != (m, 2 * h) or (a is not None and tuple(a.shape) != (m, h)):
        raise RuntimeError("swiglu_bwd shape mismatch")
    _check(_load().f3d_swiglu_bwd_bf16(_ptr(z), _u32(z.stride(0)), _ptr(da), _u32(da.stride(0)), _ptr(dz),
                                       _u32(dz.stride(0)), _ptr(a), _u32(a.stride(0) if a is not None else 0),
                                       _u32(m), _u32(h), _i32(dev), _stream(dev)))


def mlp_gate_bwd_bf16(h, dy, w1, b1, w2t, dz, a):
    """extension: (dz, a) of the gated MLP's backward from h = LayerNorm(x), dy, w1 [2 hidden, c], b1, w2t = w2.T
    [hidden, c]: fc1 recomputed, da = dy @ w2 and the gate backward in one kernel.  Returns False (nothing written)
    when that kernel does not cover the shape."""
    dev = assert_same_device([h, dy, w1, w2t, dz, a])
    _rows2d([h, dy, dz, a])
    assert_dtype([w1, w2t], torch.bfloat16)
    assert_contiguous([w1, w2t])
    _check_vectors(h, [b1])
    m, c = h.shape
    hid = w2t.shape[0]
    if tuple(dy.shape) != (m, c) or tuple(w1.shape) != (2 * hid, c) or tuple(w2t.shape) != (hid, c) \
            or tuple(dz.shape) != (m, 2 * hid) or tuple(a.shape) != (m, hid) or (b1 is not None and tuple(b1.shape) != (2 * hid,)):
        raise RuntimeError("mlp_gate_bwd shape mismatch")
    rc = _load().f3d_mlp_gate_bwd_bf16(_ptr(h), _u32(h.stride(0)), _ptr(dy), _u32(dy.stride(0)), _ptr(w1), _ptr(b1),
                                       _ptr(w2t), _ptr(dz), _u32(dz.stride(0)), _ptr(a), _u32(a.stride(0)), _u32(m),
                                       _u32(c), _u32(hid), _i32(dev), _stream(dev))
    if rc == 2:
        return False
    _check(rc)
    return True


def coord_embed_bf16(coord, w, bias, y):
    """extension: y = bf16(coord) @ w.T + bias for w [C,3] (PSH3DCoordEmbedding, psh_ops.py:64-67)"""
    assert_contiguous([coord, w, y])
    dev = assert_same_device([coord, w, y])
    assert_dtype([coord], torch.float16)
    assert_dtype([w, y], torch.bfloat16)
    _check_vectors(coord, [bias])
    _check(_load().f3d_coord_embed_bf16(_ptr(coord), _ptr(w), _ptr(bias), _ptr(y), _u32(coord.shape[0]),
                                        _u32(w.shape[0]), _i32(dev), _stream(dev)))


def affine_act_bf16(x, scale, shift, y, act=None):
    """extension: y = act(x * scale + shift) per channel (eval BatchNorm1d folded + GELU/ReLU)"""
    assert_contiguous([x, scale, shift, y])
    dev = assert_same_device([x, scale, shift, y])
    assert_dtype([x, y], torch.bfloat16)
    assert_dtype([scale, shift], torch.float32)
    a = ACT[act] if not isinstance(act, int) else act
    _check(_load().f3d_affine_act_bf16(_ptr(x), _ptr(scale), _ptr(shift), _ptr(y), _u32(x.shape[0]),
                                       _u32(x.shape[1]), _u32(a), _i32(dev), _stream(dev)))
