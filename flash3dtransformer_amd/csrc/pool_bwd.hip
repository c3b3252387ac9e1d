// Backward of additive unpooling and of the sub-bucket feature reduce for gfx950.
// Counterparts of additive_unpool_bwd_ker (src/psh/additive_unpool.cuh:90-137, dispatcher
// src/psh/additive_unpool_dispatcher.cu:81-134) and reduce_feat_backward_ker
// (src/psh/batch_psh_subbuck_reduce_bwd.cuh:39-126, dispatcher
// src/psh/batch_subbuck_pooling_bwd_dispatcher.cu).
//
// Both walk the inverse map unpool_ind [R, S] (row indices >= N mark empty slots) exactly once.
// One thread per (reduced row, W-channel unit), W = 8 (128-bit loads and stores; a row moves as one
// contiguous burst over neighbouring lanes) or 1 (channel counts that are not multiples of 8).
// HBM bound; algorithmic bytes per launch:
//   unpool bwd : read grad_up N C 2, write grad_res N C 2 + grad_down R C 2, indices R S 4
//   reduce bwd : read grad_red R C 2 (+ input N C 2 for min / max), write grad_in N C 2, indices R S 4
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

template <int W>
struct alignas(2 * W) BfVec {
  uint16_t v[W];
};

// grad_res[r] = grad_up[r] for every row r some slot refers to; grad_down[i] = bf16(sum over the valid
// slots of row i, in slot order, fp32).  Rows of grad_res that no slot refers to are left as they are.
template <int W>
__global__ __launch_bounds__(256) void additive_unpool_bwd_kernel(
    uint16_t* __restrict__ grad_res, uint16_t* __restrict__ grad_down, const uint16_t* __restrict__ grad_up,
    const uint32_t* __restrict__ unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t units_per_row, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / units_per_row);
  const uint32_t unit = (uint32_t)(gid - (size_t)row * units_per_row);
  if (row >= down_n) return;
  const uint32_t C = units_per_row * W;
  float acc[W];
#pragma unroll
  for (int i = 0; i < W; ++i) acc[i] = 0.f;
  const uint32_t* ind = unpool_ind + (size_t)row * S;
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = ind[s];
    if (r >= up_n) continue;
    const size_t o = (size_t)r * C + unit * W;
    const BfVec<W> g = *reinterpret_cast<const BfVec<W>*>(grad_up + o);
    *reinterpret_cast<BfVec<W>*>(grad_res + o) = g;   // the residual branch passes the gradient through
#pragma unroll
    for (int i = 0; i < W; ++i) acc[i] = __fadd_rn(acc[i], bf16_bits_to_float(g.v[i]));
  }
  BfVec<W> d;
#pragma unroll
  for (int i = 0; i < W; ++i) d.v[i] = float_to_bf16_bits(acc[i]);
  *reinterpret_cast<BfVec<W>*>(grad_down + (size_t)row * C + unit * W) = d;
}

// red_op 0 mean: grad / max(count, 1) to every valid slot; 1 sum: grad to every valid slot;
// 2 min / 3 max: grad to the first slot (in slot order) that holds the strict winner, zero to the other
// valid slots.  A row without a strict winner (all values +-inf or NaN) credits slot 0, as the reference's
// loop does with its initial winner index.
template <int W>
__global__ __launch_bounds__(256) void reduce_feat_bwd_kernel(
    const uint16_t* __restrict__ grad_red, const uint16_t* __restrict__ input_feat,
    const uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ grad_in, uint32_t total_n, uint32_t reduced_n,
    uint32_t units_per_row, uint32_t S, uint32_t red_op) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / units_per_row);
  const uint32_t unit = (uint32_t)(gid - (size_t)row * units_per_row);
  if (row >= reduced_n) return;
  const uint32_t C = units_per_row * W;
  const uint32_t* ind = unpool_ind + (size_t)row * S;
  const BfVec<W> g = *reinterpret_cast<const BfVec<W>*>(grad_red + (size_t)row * C + unit * W);
  if (red_op <= 1) {
    uint32_t cnt = 0;
    for (uint32_t s = 0; s < S; ++s) cnt += ind[s] < total_n ? 1u : 0u;
    BfVec<W> out = g;
    if (red_op == 0) {
      const float c = (float)(cnt > 1u ? cnt : 1u);
#pragma unroll
      for (int i = 0; i < W; ++i) out.v[i] = float_to_bf16_bits(__fdiv_rn(bf16_bits_to_float(g.v[i]), c));
    }
    for (uint32_t s = 0; s < S; ++s) {
      const uint32_t r = ind[s];
      if (r < total_n) *reinterpret_cast<BfVec<W>*>(grad_in + (size_t)r * C + unit * W) = out;
    }
    return;
  }
  const bool is_max = red_op == 3;
  float best[W];
  uint32_t win[W];
#pragma unroll
  for (int i = 0; i < W; ++i) {
    best[i] = is_max ? -INFINITY : INFINITY;
    win[i] = 0u;
  }
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = ind[s];
    if (r >= total_n) continue;
    const BfVec<W> x = *reinterpret_cast<const BfVec<W>*>(input_feat + (size_t)r * C + unit * W);
#pragma unroll
    for (int i = 0; i < W; ++i) {
      const float v = bf16_bits_to_float(x.v[i]);
      const bool better = is_max ? (v > best[i]) : (v < best[i]);
      if (better) {
        best[i] = v;
        win[i] = s;
      }
    }
  }
  for (uint32_t s = 0; s < S; ++s) {
    const uint32_t r = ind[s];
    if (r >= total_n) continue;
    BfVec<W> out;
#pragma unroll
    for (int i = 0; i < W; ++i) out.v[i] = win[i] == s ? g.v[i] : (uint16_t)0;
    *reinterpret_cast<BfVec<W>*>(grad_in + (size_t)r * C + unit * W) = out;
  }
}

}  // namespace f3d

extern "C" int f3d_additive_unpool_bwd(f3d_bf16_t* grad_res, f3d_bf16_t* grad_down, const f3d_bf16_t* grad_up_added,
                                       const uint32_t* unpool_ind, uint32_t up_n, uint32_t down_n, uint32_t feat_dim,
                                       uint32_t subbuck_size, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(grad_res && grad_down && grad_up_added && unpool_ind, "null tensor pointer");
  if (down_n == 0 || feat_dim == 0 || subbuck_size == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const bool vec = (feat_dim % 8 == 0) &&
                   (((uintptr_t)grad_res | (uintptr_t)grad_down | (uintptr_t)grad_up_added) % 16 == 0);
  const uint32_t units = vec ? feat_dim / 8 : feat_dim;
  const size_t total = (size_t)down_n * units;
  F3D_CHECK_ARG((total + 255) / 256 <= 0x7FFFFFFFu, "problem too large for one launch");
  const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
  if (vec)
    hipLaunchKernelGGL(additive_unpool_bwd_kernel<8>, grid, block, 0, s, grad_res, grad_down, grad_up_added,
                       unpool_ind, up_n, down_n, units, subbuck_size);
  else
    hipLaunchKernelGGL(additive_unpool_bwd_kernel<1>, grid, block, 0, s, grad_res, grad_down, grad_up_added,
                       unpool_ind, up_n, down_n, units, subbuck_size);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

extern "C" int f3d_subbuck_reduce_bwd(const f3d_bf16_t* grad_red_feat, const f3d_bf16_t* input_feat,
                                      const uint32_t* unpool_ind, f3d_bf16_t* grad_input_feat, uint32_t total_n,
                                      uint32_t reduced_n, uint32_t feat_dim, uint32_t subbuck_size, uint32_t red_op,
                                      int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(grad_red_feat && input_feat && unpool_ind && grad_input_feat, "null tensor pointer");
  F3D_CHECK_ARG(red_op <= 3, "unknown reduction op %u", red_op);
  if (reduced_n == 0 || feat_dim == 0 || subbuck_size == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const bool vec = (feat_dim % 8 == 0) &&
                   (((uintptr_t)grad_red_feat | (uintptr_t)input_feat | (uintptr_t)grad_input_feat) % 16 == 0);
  const uint32_t units = vec ? feat_dim / 8 : feat_dim;
  const size_t total = (size_t)reduced_n * units;
  F3D_CHECK_ARG((total + 255) / 256 <= 0x7FFFFFFFu, "problem too large for one launch");
  const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
  if (vec)
    hipLaunchKernelGGL(reduce_feat_bwd_kernel<8>, grid, block, 0, s, grad_red_feat, input_feat, unpool_ind,
                       grad_input_feat, total_n, reduced_n, units, subbuck_size, red_op);
  else
    hipLaunchKernelGGL(reduce_feat_bwd_kernel<1>, grid, block, 0, s, grad_red_feat, input_feat, unpool_ind,
                       grad_input_feat, total_n, reduced_n, units, subbuck_size, red_op);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}
