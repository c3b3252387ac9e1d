// Pieces shared by the row-panel linear kernels.
#pragma once
#include "f3d_device.h"
#include "f3d_internal.h"
#include <stdlib.h>
#include <type_traits>

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kXsChunk = 64;   // w rows per chunk (two 32-wide MFMA tiles)
constexpr int kXsBufs = 3;     // w chunk buffers in LDS
constexpr int kXsBiasSlots = 3;  // per-chunk bias slots in LDS (256 bytes each)
constexpr int kPatchRow = 40;  // epilogue patch: 32 output columns + 8 pad (80-byte pitch keeps 16-byte alignment)
constexpr int kPatchRow2 = 72;  // the same for 64 output columns (144-byte pitch)

__device__ __forceinline__ float fast_silu(float a) {
  // a * sigmoid(a) with the hardware exp2 / rcp
  return a * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * a));
}

__device__ __forceinline__ float xs_act(float v, uint32_t act) {
  switch (act) {
    case F3D_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    case F3D_ACT_SILU: return fast_silu(v);
    case F3D_ACT_RELU: return v > 0.f ? v : 0.f;
    default: return v;
  }
}

// sum over the two lanes (l, l ^ 32) that share a row
__device__ __forceinline__ float pair_sum(float v) { return v + __shfl_xor(v, 32, kWave); }

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds + 16 l.
// gbase and lds are wave-uniform, voff is the lane's byte offset from gbase.  Inline assembly on
// purpose: the compiler keeps no record of these loads, so it never guards LDS reads of OTHER buffers
// with a full vmcnt wait; the waits that matter are written out below.
__device__ __forceinline__ void xs_lds_dma16(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

// the same with 4 bytes per lane (lane l lands at lds + 4 l) and with 2 bytes per lane, zero-extended to 4
__device__ __forceinline__ void xs_lds_dma4(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}
__device__ __forceinline__ void xs_lds_dma2(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

// s_waitcnt vmcnt(n) for a small run-time n (the instruction takes an immediate)
__device__ __forceinline__ void xs_wait_vm(uint32_t n) {
  // vmcnt is split over bits 3:0 and 15:14 of the immediate; expcnt and lgkmcnt stay at "no wait"
#define F3D_VM(N) case N: __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14)); break;
  switch (__builtin_amdgcn_readfirstlane(n)) {     // n is the same in every lane: branch on the scalar unit
    F3D_VM(0) F3D_VM(1) F3D_VM(2) F3D_VM(3) F3D_VM(4) F3D_VM(5) F3D_VM(6) F3D_VM(7) F3D_VM(8) F3D_VM(9) F3D_VM(10)
    F3D_VM(11) F3D_VM(12) F3D_VM(13) F3D_VM(14) F3D_VM(15) F3D_VM(16) F3D_VM(17) F3D_VM(18) F3D_VM(19) F3D_VM(20)
    F3D_VM(21) F3D_VM(22) F3D_VM(23) F3D_VM(24) F3D_VM(25) F3D_VM(26) F3D_VM(27) F3D_VM(28) F3D_VM(29) F3D_VM(30)
    F3D_VM(31) F3D_VM(32) F3D_VM(33) F3D_VM(34) F3D_VM(35) F3D_VM(36) F3D_VM(37) F3D_VM(38) F3D_VM(39) F3D_VM(40)
    F3D_VM(41) F3D_VM(42) F3D_VM(43) F3D_VM(44) F3D_VM(45) F3D_VM(46) F3D_VM(47) F3D_VM(48) F3D_VM(49) F3D_VM(50)
    F3D_VM(51) F3D_VM(52) F3D_VM(53) F3D_VM(54) F3D_VM(55) F3D_VM(56) F3D_VM(57) F3D_VM(58) F3D_VM(59) F3D_VM(60)
    F3D_VM(61) F3D_VM(62) F3D_VM(63)
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
#undef F3D_VM
}

template <int K>
struct XsGeom {
  static constexpr int CPR = K / 8;                       // 16-byte pieces per w row
  static constexpr int ROWB = K * 2;                      // bytes per w row
  static constexpr int CHUNK_BYTES = kXsChunk * ROWB;
  static constexpr int RP = CPR >= 16 ? 1 : 16 / CPR;     // rows sharing one swizzle value
  static constexpr int SWZ_MASK = (CPR < 16 ? CPR : 16) - 1;
  static constexpr int N_DMA = CPR;                       // direct-load instructions per chunk (64 pieces each)
  static constexpr int KP = K < 128 ? K : 128;            // columns per transposition pass of the x prologue
  __host__ __device__ static constexpr uint32_t swz(uint32_t row) { return (row / RP) & SWZ_MASK; }
};

// One wave folds one output feature n of a LayerNorm into the Linear behind it: w'[n][:] = bf16(w[n][:] * gamma) and
// b'[n] = bias[n] + sum_k w[n][k] * beta[k] as fp32.
__device__ __forceinline__ void ln_fold_row(const uint16_t* __restrict__ w, const uint16_t* __restrict__ gamma,
                                            const uint16_t* __restrict__ beta, const uint16_t* __restrict__ bias,
                                            uint16_t* __restrict__ wp, float* __restrict__ bias32, uint32_t K, uint32_t n,
                                            uint32_t lane) {
  float t = 0.f;
  for (uint32_t k = lane; k < K; k += kWave) {
    const float wv = bf16_bits_to_float(w[(size_t)n * K + k]);
    wp[(size_t)n * K + k] = float_to_bf16_bits(wv * bf16_bits_to_float(gamma[k]));
    if (beta) t = __builtin_fmaf(wv, bf16_bits_to_float(beta[k]), t);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) t += __shfl_xor(t, o, kWave);
  if (lane == 0) bias32[n] = t + (bias ? bf16_bits_to_float(bias[n]) : 0.f);
}

// w' = bf16(w * gamma) and b' = b + w beta as fp32 (defined with the linear kernels)
void launch_ln_fold(const uint16_t* w, const uint16_t* gamma, const uint16_t* beta, const uint16_t* bias, uint16_t* wp,
                    float* bias32, uint32_t N, uint32_t K, hipStream_t s);

}  // namespace f3d
