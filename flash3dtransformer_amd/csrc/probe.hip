// Measurement aid, not part of the hot path: the rate at which the matrix cores of this GPU retire dense
// v_mfma_f32_32x32x16_bf16 products when nothing else runs (operands in registers, eight independent accumulators per
// wave, four waves per SIMD).  With random operands the chip's power budget, not the issue rate, sets the clock; with
// a zero operand the multipliers do not toggle and the rate is the 2.5 PFLOP/s of the data sheet.  bench.py reports
// both next to the kernels' figures, which are priced against the data-sheet number.
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ sink, uint32_t iters, uint32_t random_a,
                                                         uint32_t random_b) {
  uint32_t h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h = h * 1664525u + 1013904223u;
      a[i][e] = (__bf16)(random_a ? ((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f : 0.f);
      h = h * 1664525u + 1013904223u;
      b[i][e] = (__bf16)(random_b ? ((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f : 0.f);
    }
  f32x16_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j & 3], b[(j + 1) & 3], acc[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[j][i];
  if (s == 123.456f) sink[0] = s;   // keeps the products alive; never true for these operands
}

}  // namespace f3d

extern "C" {

int f3d_probe_mfma_bf16(uint32_t workgroups, uint32_t iters, uint32_t random_a, uint32_t random_b, float* sink,
                        int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(sink != nullptr, "null sink pointer");
  F3D_CHECK_ARG(workgroups > 0 && workgroups <= 65536u && iters <= (1u << 24), "probe size out of range");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, sink, iters, random_a, random_b);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
