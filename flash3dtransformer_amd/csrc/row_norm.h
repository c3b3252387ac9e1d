// Normalisation of a row that is spread over neighbouring lanes, 8 bf16 channels per lane: what the pooling and
// unpooling kernels apply to a row they hold anyway, where the reference runs a norm layer (and an activation) on
// the tensor afterwards (flash3dxfmr/layers/hourglass.py:104-109, 152-159).
#pragma once
#include "xstat_common.h"

namespace f3d {

enum : uint32_t { kRowNormNone = 0, kRowNormLayer = 1, kRowNormAffine = 2 };

// kRowNormLayer: LayerNorm over the row (gamma, beta bf16 [C]; beta may be null), statistics in fp32 in two passes as
// layernorm_kernel computes them.  kRowNormAffine: act(x * scale[c] + shift[c]) (scale, shift fp32 [C]: an eval-mode
// BatchNorm1d folded), rounded to bf16 before the activation as affine_act_kernel does.
struct RowNorm {
  uint32_t mode;
  const uint16_t* gamma;
  const uint16_t* beta;
  const float* scale;
  const float* shift;
  float eps;
  uint32_t act;
};

// v: the lane's 8 channels (chunk `chunk` of cpr = C / 8); the cpr lanes of the row are neighbours, aligned to cpr
// (a power of two, at most 64, for kRowNormLayer), all active and all with the same RowNorm.
__device__ __forceinline__ u32x4_t row_norm_chunk(u32x4_t v, const RowNorm& n, uint32_t chunk, uint32_t cpr) {
  if (n.mode == kRowNormLayer) {
    const float c = (float)(cpr * 8u);
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) sum = __fadd_rn(sum, __fadd_rn(bf16_lo(v[e]), bf16_hi(v[e])));
    for (uint32_t off = cpr >> 1; off > 0; off >>= 1) sum = __fadd_rn(sum, __shfl_xor(sum, (int)off, kWave));
    const float mean = __fdiv_rn(sum, c);
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float d0 = __fsub_rn(bf16_lo(v[e]), mean), d1 = __fsub_rn(bf16_hi(v[e]), mean);
      sq = __fadd_rn(sq, __fadd_rn(__fmul_rn(d0, d0), __fmul_rn(d1, d1)));
    }
    for (uint32_t off = cpr >> 1; off > 0; off >>= 1) sq = __fadd_rn(sq, __shfl_xor(sq, (int)off, kWave));
    const float rstd = rsqrtf(__fadd_rn(__fdiv_rn(sq, c), n.eps));
    const u32x4_t g = *reinterpret_cast<const u32x4_t*>(n.gamma + chunk * 8u);
    u32x4_t b = {0u, 0u, 0u, 0u}, t;
    if (n.beta) b = *reinterpret_cast<const u32x4_t*>(n.beta + chunk * 8u);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float f0 = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(bf16_lo(v[e]), mean), rstd), bf16_lo(g[e])), bf16_lo(b[e]));
      const float f1 = __fadd_rn(__fmul_rn(__fmul_rn(__fsub_rn(bf16_hi(v[e]), mean), rstd), bf16_hi(g[e])), bf16_hi(b[e]));
      t[e] = pack_bf16x2(f0, f1);
    }
    return t;
  }
  if (n.mode == kRowNormAffine) {
    const float4 s0 = *reinterpret_cast<const float4*>(n.scale + chunk * 8u), s1 = *reinterpret_cast<const float4*>(n.scale + chunk * 8u + 4u);
    const float4 h0 = *reinterpret_cast<const float4*>(n.shift + chunk * 8u), h1 = *reinterpret_cast<const float4*>(n.shift + chunk * 8u + 4u);
    const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    const float sh[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
    u32x4_t t;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float f0 = __builtin_fmaf(bf16_lo(v[e]), sc[2 * e], sh[2 * e]), f1 = __builtin_fmaf(bf16_hi(v[e]), sc[2 * e + 1], sh[2 * e + 1]);
      if (n.act != F3D_ACT_NONE) {
        // the normalisation's output is rounded to bf16 before the activation, as two separate modules would
        f0 = xs_act(bf16_bits_to_float(float_to_bf16_bits(f0)), n.act);
        f1 = xs_act(bf16_bits_to_float(float_to_bf16_bits(f1)), n.act);
      }
      t[e] = pack_bf16x2(f0, f1);
    }
    return t;
  }
  return v;
}

// host side: whether the mode can be applied to rows of feat_dim channels by the kernels above
inline bool row_norm_supported(uint32_t mode, uint32_t feat_dim) {
  if (mode == kRowNormNone || mode == kRowNormAffine) return feat_dim % 8u == 0u;
  const uint32_t cpr = feat_dim / 8u;
  return mode == kRowNormLayer && feat_dim % 8u == 0u && cpr >= 1u && cpr <= 64u && (cpr & (cpr - 1u)) == 0u;
}

}  // namespace f3d
