// Additive unpooling for gfx950: up[r, :] = bf16(float(down[i, :]) + float(res[r, :])) for every
// valid r = unpool_ind[i, s].  Counterpart of additive_unpool_fwd_ker,
// src/psh/additive_unpool.cuh:43-86 (dispatcher src/psh/additive_unpool_dispatcher.cu:26-79).
//
// One thread per (down row, 8-channel chunk): the down chunk is read once (16 bytes) and added to
// each of the S gathered residual chunks; loads and stores are 128-bit and a row is covered by
// neighbouring lanes, so every row moves as one contiguous burst.
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

struct alignas(16) Bf16x8 {
  uint16_t v[8];
};

__global__ __launch_bounds__(256) void additive_unpool_vec8_kernel(
    const uint16_t* __restrict__ res, const uint16_t* __restrict__ down, uint16_t* __restrict__ up,
    const uint32_t* __restrict__ unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t chunks_per_row, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / chunks_per_row);
  const uint32_t chunk = (uint32_t)(gid - (size_t)row * chunks_per_row);
  if (row >= down_n) return;
  const uint32_t C = chunks_per_row * 8;
  const Bf16x8 d = *reinterpret_cast<const Bf16x8*>(down + (size_t)row * C + chunk * 8);
  float df[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) df[i] = bf16_bits_to_float(d.v[i]);
  const uint32_t* ind = unpool_ind + (size_t)row * S;
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = ind[s];
    if (r >= up_n) continue;
    const size_t o = (size_t)r * C + chunk * 8;
    const Bf16x8 x = *reinterpret_cast<const Bf16x8*>(res + o);
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

extern "C" int f3d_additive_unpool_fwd(const f3d_bf16_t* res_feat, const f3d_bf16_t* down_feat,
                                       f3d_bf16_t* up_add_feat, const uint32_t* unpool_ind, uint32_t up_n,
                                       uint32_t down_n, uint32_t feat_dim, uint32_t subbuck_size, int device,
                                       void* stream) {
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
    hipLaunchKernelGGL(additive_unpool_vec8_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, res_feat,
                       down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim / 8, subbuck_size);
  } else {
    const size_t total = (size_t)down_n * feat_dim;
    hipLaunchKernelGGL(additive_unpool_scalar_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, res_feat,
                       down_feat, up_add_feat, unpool_ind, up_n, down_n, feat_dim, subbuck_size);
  }
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}
