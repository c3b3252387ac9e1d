// Sub-bucket pooling for gfx950: the sub-bucket builder (ids, slots, inverse map, mean coordinates)
// and the per-row feature reduce.  Counterpart of local_subbuck_ker and reduce_feat_ker,
// src/psh/batch_psh_subbuck_reduce.cuh:104-298 and :300-359, launched by
// src/psh/batch_subbuck_pooling_dispatcher.cu:119-138.
//
// Builder design: one 1024-thread workgroup per tile of tile_pts = (1024 / S) * S consecutive points
// of one cloud.  The tile is rotated by a per-tile unit quaternion (stateless RNG), quantised inside
// its own bounding box, keyed by the 13-bit z-order cell, and sorted by (cell, position) with a
// register/LDS bitonic network — a deterministic stand-in for the reference's LDS counting sort,
// whose tie order depends on atomic arbitration.  Consecutive runs of S sorted points form a
// sub-bucket.  Tile t owns output rows [t * tile_pts / S, ...) of its cloud, so no global counter
// is needed.  Every output is a pure function of (coords, seps, S, seed).
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

constexpr int kSubThreads = 1024;

__device__ __forceinline__ void tile_quat(uint32_t seed, uint32_t cloud, uint32_t tile, float q[4]) {
  float acc = 0.f;
#pragma unroll
  for (uint32_t i = 0; i < 4; ++i) {
    q[i] = __fadd_rn(0.1f, __fmul_rn(rng_u01(seed, cloud, tile, i), 0.9f));
    acc = __fadd_rn(acc, __fmul_rn(q[i], q[i]));
  }
  const float nrm = __fsqrt_rn(acc);
#pragma unroll
  for (int i = 0; i < 4; ++i) q[i] = __fdiv_rn(q[i], nrm);
}

// rotation by unit quaternion (w, x, y, z); every product and sum rounded separately
__device__ __forceinline__ void quat_rotate(const float q[4], const float p[3], float out[3]) {
  const float w = q[0], x = q[1], y = q[2], z = q[3];
  const float n1 = __fmul_rn(x, 2.0f), n2 = __fmul_rn(y, 2.0f), n3 = __fmul_rn(z, 2.0f);
  const float n4 = __fmul_rn(x, n1), n5 = __fmul_rn(y, n2), n6 = __fmul_rn(z, n3);
  const float n7 = __fmul_rn(x, n2), n8 = __fmul_rn(x, n3), n9 = __fmul_rn(y, n3);
  const float n10 = __fmul_rn(w, n1), n11 = __fmul_rn(w, n2), n12 = __fmul_rn(w, n3);
  const float a0 = __fmul_rn(__fsub_rn(1.0f, __fadd_rn(n5, n6)), p[0]);
  const float a1 = __fmul_rn(__fsub_rn(n7, n12), p[1]);
  const float a2 = __fmul_rn(__fadd_rn(n8, n11), p[2]);
  const float b0 = __fmul_rn(__fadd_rn(n7, n12), p[0]);
  const float b1 = __fmul_rn(__fsub_rn(1.0f, __fadd_rn(n4, n6)), p[1]);
  const float b2 = __fmul_rn(__fsub_rn(n9, n10), p[2]);
  const float c0 = __fmul_rn(__fsub_rn(n8, n11), p[0]);
  const float c1 = __fmul_rn(__fadd_rn(n9, n10), p[1]);
  const float c2 = __fmul_rn(__fsub_rn(1.0f, __fadd_rn(n4, n5)), p[2]);
  out[0] = __fadd_rn(__fadd_rn(a0, a1), a2);
  out[1] = __fadd_rn(__fadd_rn(b0, b1), b2);
  out[2] = __fadd_rn(__fadd_rn(c0, c1), c2);
}

__global__ __launch_bounds__(kSubThreads) void subbuck_build_kernel(
    const uint16_t* __restrict__ coord, const uint32_t* __restrict__ batch_sep,
    const uint32_t* __restrict__ reduced_batch_sep, uint32_t batch_size, uint32_t subbuck_size, uint32_t tile_pts,
    uint32_t num_vox, uint32_t seed, uint32_t* __restrict__ subbuck_id, uint16_t* __restrict__ subbuck_off,
    uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced_coord, uint32_t reduced_n,
    uint32_t reduced_aligned_n) {
  __shared__ uint32_t s_key[kSubThreads];
  __shared__ uint16_t s_xyz[kSubThreads][3];
  __shared__ float s_red[6][kSubThreads / kWave];
  __shared__ float s_bb[6];
  const uint32_t tid = threadIdx.x, cloud = blockIdx.y, tile = blockIdx.x;

  if (cloud == batch_size) {  // zero the alignment rows [reduced_n, reduced_aligned_n)
    const uint32_t r = reduced_n + tile * kSubThreads + tid;
    if (r < reduced_aligned_n) {
      uint16_t* q = reduced_coord + 3 * (size_t)r;
      q[0] = 0; q[1] = 0; q[2] = 0;
    }
    return;
  }

  const uint32_t start = cloud ? batch_sep[cloud - 1] : 0u;
  const uint32_t n = batch_sep[cloud] - start;
  const uint32_t rstart = cloud ? reduced_batch_sep[cloud - 1] : 0u;
  const uint32_t t0 = tile * tile_pts;
  if (t0 >= n) return;
  const uint32_t m = min(tile_pts, n - t0);
  const bool valid = tid < m;
  const size_t g = (size_t)start + t0 + tid;

  float p[3] = {0.f, 0.f, 0.f};
  if (valid) {
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      const uint16_t h = coord[3 * g + d];
      s_xyz[tid][d] = h;
      p[d] = half_bits_to_float(h);
    }
  }
  float q[4], r[3], rh[3];
  tile_quat(seed, cloud, tile, q);
  quat_rotate(q, p, r);
  float mn[3], mx[3];
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    rh[d] = half_bits_to_float(float_to_half_bits(r[d]));  // the rotated coordinate is an fp16 value
    mn[d] = valid ? rh[d] : INFINITY;
    mx[d] = valid ? rh[d] : -INFINITY;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mn[d] = fminf(mn[d], __shfl_xor(mn[d], off, kWave));
      mx[d] = fmaxf(mx[d], __shfl_xor(mx[d], off, kWave));
    }
  }
  const uint32_t w = tid / kWave, l = tid % kWave;
  if (l == 0) {
#pragma unroll
    for (int d = 0; d < 3; ++d) { s_red[d][w] = mn[d]; s_red[3 + d][w] = mx[d]; }
  }
  __syncthreads();
  if (tid < 6) {
    float a = s_red[tid][0];
    for (int i = 1; i < kSubThreads / kWave; ++i) a = tid < 3 ? fminf(a, s_red[tid][i]) : fmaxf(a, s_red[tid][i]);
    s_bb[tid] = a;
  }
  __syncthreads();

  uint32_t key = 0xFFFFFFFFu;
  if (valid) {
    uint32_t v[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) v[d] = vox1(rh[d], make_vox_axis_f(s_bb[d], s_bb[3 + d], num_vox));
    const uint32_t cell = zorder16(v[0], v[1], v[2]) >> 3;  // H_ZORDER_DIV with divisor 65536 / 8192
    key = (cell << 10) | tid;
  }

  // bitonic sort of one key per thread, ascending over the workgroup: partner distances below a
  // wave go through lane exchange, larger ones through LDS
  for (uint32_t k = 2; k <= kSubThreads; k <<= 1) {
    for (uint32_t j = k >> 1; j > 0; j >>= 1) {
      uint32_t other;
      if (j >= kWave) {
        s_key[tid] = key;
        __syncthreads();
        other = s_key[tid ^ j];
        __syncthreads();
      } else {
        other = __shfl_xor(key, j, kWave);
      }
      const bool up = (tid & k) == 0;
      const bool lower = (tid & j) == 0;
      key = (lower == up) ? min(key, other) : max(key, other);
    }
  }
  s_key[tid] = key;
  __syncthreads();

  // thread `tid` now owns rank `tid`
  const uint32_t S = subbuck_size;
  const uint32_t rows_per_tile = tile_pts / S;
  const uint32_t row_base = rstart + tile * rows_per_tile;
  if (valid) {
    const uint32_t j = key & 1023u;
    const size_t gp = (size_t)start + t0 + j;
    const uint32_t sub = tid / S, off = tid - sub * S;
    subbuck_id[gp] = tile * rows_per_tile + sub;
    subbuck_off[gp] = (uint16_t)off;
    unpool_ind[(size_t)row_base * S + tid] = (uint32_t)gp;
  }
  // mean coordinate of every sub-bucket, members summed in rank order
  const uint32_t nrow = (m + S - 1) / S;
  if (tid < nrow) {
    const uint32_t cnt = min(S, m - tid * S);
    float acc[3] = {0.f, 0.f, 0.f};
    for (uint32_t s = 0; s < cnt; ++s) {
      const uint32_t j = s_key[tid * S + s] & 1023u;
#pragma unroll
      for (int d = 0; d < 3; ++d) acc[d] = __fadd_rn(acc[d], half_bits_to_float(s_xyz[j][d]));
    }
    uint16_t* out = reduced_coord + 3 * (size_t)(row_base + tid);
#pragma unroll
    for (int d = 0; d < 3; ++d) out[d] = float_to_half_bits(__fdiv_rn(acc[d], (float)cnt));
  }
}

// ---- feature reduce ------------------------------------------------------------------------------
// One thread per (reduced row, 8-channel chunk): S gathered 16-byte loads, fp32 accumulate in slot
// order, one 16-byte store.  A row of C channels is covered by C/8 neighbouring lanes, so every
// gathered row is read as one contiguous burst.

struct alignas(16) Bf16x8 {
  uint16_t v[8];
};

template <int OP>
__device__ __forceinline__ float red_init() {
  return OP == F3D_O_MIN ? INFINITY : OP == F3D_O_MAX ? -INFINITY : 0.f;
}

template <int OP>
__device__ __forceinline__ float red_step(float acc, float v) {
  if (OP == F3D_O_MIN) return (v < acc) ? v : acc;
  if (OP == F3D_O_MAX) return (v > acc) ? v : acc;
  return __fadd_rn(acc, v);
}

template <int OP>
__global__ __launch_bounds__(256) void reduce_feat_vec8_kernel(
    const uint16_t* __restrict__ feat, const uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced,
    uint32_t total_n, uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t chunks_per_row, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / chunks_per_row);
  const uint32_t chunk = (uint32_t)(gid - (size_t)row * chunks_per_row);
  if (row >= reduced_aligned_n) return;
  const uint32_t C = chunks_per_row * 8;
  Bf16x8 out;
  if (row >= reduced_n) {
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = 0;
  } else {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = red_init<OP>();
    uint32_t cnt = 0;
    const uint32_t* ind = unpool_ind + (size_t)row * S;
    for (uint32_t s = 0; s < S; ++s) {
      const uint32_t src = ind[s];
      if (src < total_n) {
        ++cnt;
        const Bf16x8 x = *reinterpret_cast<const Bf16x8*>(feat + (size_t)src * C + chunk * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = red_step<OP>(acc[i], bf16_bits_to_float(x.v[i]));
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float a = acc[i];
      if (OP == F3D_O_MEAN) a = __fdiv_rn(a, (float)cnt);
      if (cnt == 0) a = 0.f;
      out.v[i] = float_to_bf16_bits(a);
    }
  }
  *reinterpret_cast<Bf16x8*>(reduced + (size_t)row * C + chunk * 8) = out;
}

// any channel count: one thread per (row, channel)
template <int OP>
__global__ __launch_bounds__(256) void reduce_feat_scalar_kernel(
    const uint16_t* __restrict__ feat, const uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced,
    uint32_t total_n, uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t C, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / C);
  const uint32_t c = (uint32_t)(gid - (size_t)row * C);
  if (row >= reduced_aligned_n) return;
  float a = 0.f;
  if (row < reduced_n) {
    a = red_init<OP>();
    uint32_t cnt = 0;
    for (uint32_t s = 0; s < S; ++s) {
      const uint32_t src = unpool_ind[(size_t)row * S + s];
      if (src < total_n) {
        ++cnt;
        a = red_step<OP>(a, bf16_bits_to_float(feat[(size_t)src * C + c]));
      }
    }
    if (OP == F3D_O_MEAN) a = __fdiv_rn(a, (float)cnt);
    if (cnt == 0) a = 0.f;
  }
  reduced[(size_t)row * C + c] = float_to_bf16_bits(a);
}

template <int OP>
static void launch_reduce(const uint16_t* feat, const uint32_t* unpool_ind, uint16_t* reduced, uint32_t total_n,
                          uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t C, uint32_t S, hipStream_t s) {
  const bool vec = (C % 8 == 0) && (((uintptr_t)feat | (uintptr_t)reduced) % 16 == 0);
  if (vec) {
    const size_t total = (size_t)reduced_aligned_n * (C / 8);
    hipLaunchKernelGGL(reduce_feat_vec8_kernel<OP>, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, feat,
                       unpool_ind, reduced, total_n, reduced_n, reduced_aligned_n, C / 8, S);
  } else {
    const size_t total = (size_t)reduced_aligned_n * C;
    hipLaunchKernelGGL(reduce_feat_scalar_kernel<OP>, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, feat,
                       unpool_ind, reduced, total_n, reduced_n, reduced_aligned_n, C, S);
  }
}

}  // namespace f3d

extern "C" {

int f3d_subbuck_build(const f3d_half_t* coord, const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n,
                      uint32_t instance_max_n, uint32_t subbuck_size, uint32_t num_vox, uint32_t* subbuck_id,
                      uint16_t* subbuck_off, const uint32_t* reduced_batch_sep, f3d_half_t* reduced_coord,
                      uint32_t reduced_aligned_n, uint32_t* unpool_ind, uint32_t reduced_n, int device,
                      void* stream) {
  using namespace f3d;
  (void)total_n;
  F3D_CHECK_ARG(subbuck_size >= 1 && subbuck_size <= 1024, "subbuck_size=%u outside [1, 1024]", subbuck_size);
  F3D_CHECK_ARG(num_vox >= 2 && num_vox <= 0x10000u, "num_vox=%u does not fit the 16-bit voxel type", num_vox);
  F3D_CHECK_ARG(reduced_aligned_n >= reduced_n, "reduced buffer length(%u) is smaller than the reduced row count(%u)",
                reduced_aligned_n, reduced_n);
  F3D_CHECK_ARG(coord && batch_sep && subbuck_id && subbuck_off && reduced_batch_sep && reduced_coord && unpool_ind,
                "null tensor pointer");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  const uint32_t tile_pts = (1024u / subbuck_size) * subbuck_size;
  const uint32_t max_tiles = cdiv_u32(instance_max_n, tile_pts);
  const uint32_t pad_tiles = cdiv_u32(reduced_aligned_n - reduced_n, kSubThreads);
  const uint32_t gx = max_tiles > pad_tiles ? max_tiles : pad_tiles;
  if (gx == 0 || (batch_size == 0 && pad_tiles == 0)) return F3D_OK;
  SyncBracket sync(s);
  hipLaunchKernelGGL(subbuck_build_kernel, dim3(gx, batch_size + (pad_tiles ? 1 : 0)), dim3(kSubThreads), 0, s, coord,
                     batch_sep, reduced_batch_sep, batch_size, subbuck_size, tile_pts, num_vox | quantiser_bit(), global_seed(),
                     subbuck_id, subbuck_off, unpool_ind, reduced_coord, reduced_n, reduced_aligned_n);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_reduce_feat(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                    uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                    uint32_t reduced_aligned_n, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(red_op <= 3, "Unsupported reduction operation id-%u", red_op);
  F3D_CHECK_ARG(reduced_aligned_n >= reduced_n, "reduced buffer length(%u) is smaller than the reduced row count(%u)",
                reduced_aligned_n, reduced_n);
  F3D_CHECK_ARG(feat && unpool_ind && reduced_feat, "null tensor pointer");
  if (reduced_aligned_n == 0 || feat_dim == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  switch (red_op) {
    case F3D_O_MEAN: launch_reduce<F3D_O_MEAN>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, s); break;
    case F3D_O_SUM: launch_reduce<F3D_O_SUM>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, s); break;
    case F3D_O_MIN: launch_reduce<F3D_O_MIN>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, s); break;
    default: launch_reduce<F3D_O_MAX>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, s); break;
  }
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_batch_subbuck_reduce(const f3d_half_t* scattered_coord, const f3d_bf16_t* scattered_feat,
                             const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n,
                             uint32_t instance_max_n, uint32_t feat_dim, uint32_t subbuck_size, uint32_t num_vox,
                             const f3d_half_t* bbox_min, const f3d_half_t* bbox_max, uint32_t* subbuck_id,
                             uint16_t* subbuck_off, const uint32_t* reduced_batch_sep, f3d_half_t* reduced_coord,
                             f3d_bf16_t* reduced_feat, uint32_t reduced_aligned_n, uint32_t* unpool_ind,
                             uint32_t reduced_n, uint32_t hash_type, uint32_t red_op, int device, void* stream) {
  // bbox_* and hash_type are part of the reference signature; its kernel quantises inside each
  // block's own box with the z-order hash regardless of them (dispatcher :108-109).
  (void)bbox_min; (void)bbox_max; (void)hash_type;
  F3D_CHECK_ARG(red_op <= 3, "Unsupported reduction operation id-%u", red_op);
  int rc = f3d_subbuck_build(scattered_coord, batch_sep, batch_size, total_n, instance_max_n, subbuck_size, num_vox,
                             subbuck_id, subbuck_off, reduced_batch_sep, reduced_coord, reduced_aligned_n, unpool_ind,
                             reduced_n, device, stream);
  if (rc != F3D_OK) return rc;
  return f3d_reduce_feat(scattered_feat, total_n, feat_dim, unpool_ind, reduced_n, subbuck_size, red_op, reduced_feat,
                         reduced_aligned_n, device, stream);
}

}  // extern "C"
