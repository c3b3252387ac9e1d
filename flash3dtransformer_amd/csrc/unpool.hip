// Additive unpooling for gfx950: up[r, :] = bf16(float(down[i, :]) + float(res[r, :])) for every
// valid r = unpool_ind[i, s].  Counterpart of additive_unpool_fwd_ker,
// src/psh/additive_unpool.cuh:43-86 (dispatcher src/psh/additive_unpool_dispatcher.cu:26-79).
//
// One thread per (down row, 8-channel chunk): the down chunk is read once (16 bytes) and added to
// each of the S gathered residual chunks; loads and stores are 128-bit and a row is covered by
// neighbouring lanes, so every row moves as one contiguous burst.
#include "f3d_device.h"
#include "f3d_internal.h"
#include "row_norm.h"

namespace f3d {

struct alignas(16) Bf16x8 {
  uint16_t v[8];
};

// NORM: both operands are normalised on the way in (row_norm.h): up[r] = norm_res(res[r]) + norm_down(down[i]),
// where the reference runs norm (and activation) layers on both tensors before the op.
template <bool NORM>
__global__ __launch_bounds__(256) void additive_unpool_vec8_kernel(
    const uint16_t* __restrict__ res, const uint16_t* __restrict__ down, uint16_t* __restrict__ up,
    const uint32_t* __restrict__ unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t chunks_per_row, uint32_t S,
    RowNorm norm_res, RowNorm norm_down) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / chunks_per_row);
  const uint32_t chunk = (uint32_t)(gid - (size_t)row * chunks_per_row);
  if (row >= down_n) return;
  const uint32_t C = chunks_per_row * 8;
  Bf16x8 d = *reinterpret_cast<const Bf16x8*>(down + (size_t)row * C + chunk * 8);
  if (NORM) d = __builtin_bit_cast(Bf16x8, row_norm_chunk(__builtin_bit_cast(u32x4_t, d), norm_down, chunk, chunks_per_row));
  float df[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) df[i] = bf16_bits_to_float(d.v[i]);
  const uint32_t* ind = unpool_ind + (size_t)row * S;
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = ind[s];
    if (r >= up_n) continue;
    const size_t o = (size_t)r * C + chunk * 8;
    Bf16x8 x = *reinterpret_cast<const Bf16x8*>(res + o);
    if (NORM) x = __builtin_bit_cast(Bf16x8, row_norm_chunk(__builtin_bit_cast(u32x4_t, x), norm_res, chunk, chunks_per_row));
    Bf16x8 y;
#pragma unroll
    for (int i = 0; i < 8; ++i) y.v[i] = float_to_bf16_bits(__fadd_rn(df[i], bf16_bits_to_float(x.v[i])));
    *reinterpret_cast<Bf16x8*>(up + o) = y;
  }
}

__global__ __launch_bounds__(256) void additive_unpool_scalar_kernel(
    const uint16_t* __restrict__ res, const uint16_t* __restrict__ down, uint16_t* __restrict__ up,
    const uint32_t* __restrict__ unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t C, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / C);
  const uint32_t c = (uint32_t)(gid - (size_t)row * C);
  if (row >= down_n) return;
  const float d = bf16_bits_to_float(down[(size_t)row * C + c]);
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = unpool_ind[(size_t)row * S + s];
    if (r >= up_n) continue;
    const size_t o = (size_t)r * C + c;
    up[o] = float_to_bf16_bits(__fadd_rn(d, bf16_bits_to_float(res[o])));
  }
}

}  // namespace f3d

static int additive_unpool_impl(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat, f3d_bf16_t* up_add_feat,
                                const uint32_t* unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t feat_dim,
                                uint32_t subbuck_size, const f3d::RowNorm* norm_res, const f3d::RowNorm* norm_down,
                                int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(res_feat && down_feat && up_add_feat && unpool_ind, "null tensor pointer");
  if (down_n == 0 || feat_dim == 0 || subbuck_size == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const bool vec = (feat_dim % 8 == 0) &&
                   (((uintptr_t)res_feat | (uintptr_t)down_feat | (uintptr_t)up_add_feat) % 16 == 0);
  if (vec) {
    const size_t total = (size_t)down_n * (feat_dim / 8);
    if (norm_res)
      hipLaunchKernelGGL(additive_unpool_vec8_kernel<true>, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, res_feat,
                         down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim / 8, subbuck_size, *norm_res, *norm_down);
    else
      hipLaunchKernelGGL(additive_unpool_vec8_kernel<false>, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, res_feat,
                         down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim / 8, subbuck_size, RowNorm{}, RowNorm{});
  } else {
    const size_t total = (size_t)down_n * feat_dim;
    hipLaunchKernelGGL(additive_unpool_scalar_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, res_feat,
                       down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim, subbuck_size);
  }
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

extern "C" int f3d_additive_unpool_fwd(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat,
                                       f3d_bf16_t* up_add_feat, const uint32_t* unpool_ind, uint32_t up_n,
                                       uint32_t down_n, uint32_t feat_dim, uint32_t subbuck_size, int device,
                                       void* stream) {
  return additive_unpool_impl(res_feat, down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim, subbuck_size, nullptr,
                              nullptr, device, stream);
}

extern "C" int f3d_additive_unpool_norm_fwd(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat,
                                            f3d_bf16_t* up_add_feat, const uint32_t* unpool_ind, uint32_t up_n,
                                            uint32_t down_n, uint32_t feat_dim, uint32_t subbuck_size, uint32_t norm_mode,
                                            const f3d_bf16_t* res_gamma, const f3d_bf16_t* res_beta, const float* res_scale,
                                            const float* res_shift, float res_eps, const f3d_bf16_t* down_gamma,
                                            const f3d_bf16_t* down_beta, const float* down_scale, const float* down_shift,
                                            float down_eps, uint32_t act, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(norm_mode == kRowNormLayer || norm_mode == kRowNormAffine, "unknown row normalisation %u", norm_mode);
  F3D_CHECK_ARG(norm_mode == kRowNormLayer ? (res_gamma && down_gamma) : (res_scale && res_shift && down_scale && down_shift),
                "null normalisation parameter");
  F3D_CHECK_ARG(act <= F3D_ACT_RELU && act != F3D_ACT_SWIGLU && (norm_mode == kRowNormAffine || act == F3D_ACT_NONE),
                "unsupported activation id %u for normalisation %u", act, norm_mode);
  const uintptr_t all = (uintptr_t)res_feat | (uintptr_t)down_feat | (uintptr_t)up_add_feat | (uintptr_t)res_gamma |
                        (uintptr_t)res_beta | (uintptr_t)res_scale | (uintptr_t)res_shift | (uintptr_t)down_gamma |
                        (uintptr_t)down_beta | (uintptr_t)down_scale | (uintptr_t)down_shift;
  if (!row_norm_supported(norm_mode, feat_dim) || (all & 15u)) {
    set_error("No fused normalisation for %u channels (a multiple of 8; LayerNorm: 8 x a power of two up to 512; "
              "16-byte aligned tensors)", feat_dim);
    return F3D_ERR_UNSUPPORTED;
  }
  const RowNorm nr{norm_mode, res_gamma, res_beta, res_scale, res_shift, res_eps, act};
  const RowNorm nd{norm_mode, down_gamma, down_beta, down_scale, down_shift, down_eps, act};
  return additive_unpool_impl(res_feat, down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim, subbuck_size, &nr, &nd,
                              device, stream);
}
