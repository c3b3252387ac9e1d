// Dense layers for gfx950: bf16 GEMM with fused epilogues on MFMA, LayerNorm, the K=3 coordinate
// embedding and a per-channel affine + activation.
//
// These stand where the reference calls torch.nn.Linear / te.Linear / te.LayerNormMLP / norm
// callables (flash3dxfmr/layers/buck_swin.py:159,163; elem_wise.py:22-26; psh_ops.py:62;
// hourglass.py:65,148,150; flash3d.py:32; stage.py:67) and its demo op gemm_sm_bf16
// (src/psh/gemm.cuh:30-85).
//
// GEMM: y = act(x wT + bias) (+ residual), x [M,K] and w [N,K] both K-contiguous.  One 256-thread
// workgroup (2x2 waves) per 128x128 output tile, K in steps of 64 staged through padded LDS rows
// (conflict-free 128-bit fragment reads) with the next step prefetched into registers.  The product
// is formed transposed (A operand = w rows, B operand = x rows) so that a lane ends up with 4
// consecutive output columns of one row; the tile is rounded to bf16 (the rounding point of a
// Linear layer's output), laid out row-major in LDS and written back with 128-bit stores after the
// activation / residual.  Tiles that share x rows are neighbours in the XCD-remapped launch order.
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct alignas(16) U16x8 {
  uint16_t v[8];
};

constexpr int kGemmThreads = 256;
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDK = BK + 8;   // padded LDS row of the operand tiles (elements): 144 bytes
constexpr int LDC = BN + 8;   // padded LDS row of the bf16 output tile
constexpr int kGemmLds = (BM * LDK + BN * LDK) * 2;  // 36,864 bytes; the output tile (34,816) reuses it
constexpr int kNumXcdG = 8;

__device__ __forceinline__ float apply_act(float x, uint32_t act) {
  switch (act) {
    case F3D_ACT_GELU: return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
    case F3D_ACT_SILU: return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
    case F3D_ACT_RELU: return x > 0.f ? x : 0.f;
    default: return x;
  }
}

// B_TRANS: the second operand is given as b[K][N] (gemm_sm_bf16) instead of w[N][K]
template <bool B_TRANS>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, const uint16_t* __restrict__ w, uint32_t ldw,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual, uint32_t ldr,
    uint16_t* __restrict__ y, uint32_t ldy, uint32_t M, uint32_t N, uint32_t K, uint32_t act, uint32_t tiles_n,
    uint32_t n_tiles, uint32_t tiles_per_xcd) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds_gemm[];
  uint16_t* sX = lds_gemm;              // [BM][LDK]
  uint16_t* sW = lds_gemm + BM * LDK;   // [BN][LDK]
  uint16_t* sC = lds_gemm;              // [BM][LDC] after the K loop
  __shared__ float s_bias[BN];

  const uint32_t tile = (blockIdx.x % kNumXcdG) * tiles_per_xcd + blockIdx.x / kNumXcdG;
  if (tile >= n_tiles) return;
  const uint32_t tm = tile / tiles_n, tn = tile % tiles_n;
  const uint32_t m0 = tm * BM;
  const bool swiglu = act == F3D_ACT_SWIGLU;
  const uint32_t half_n = N / 2;
  // swiglu tiles pair 64 "value" columns with their 64 "gate" columns
  const uint32_t n0 = swiglu ? tn * (BN / 2) : tn * BN;
  auto wrow = [&](uint32_t r) -> uint32_t {  // weight row feeding tile column r
    if (!swiglu) return n0 + r;
    return r < BN / 2 ? n0 + r : half_n + n0 + (r - BN / 2);
  };
  auto wrow_ok = [&](uint32_t r) -> bool {
    if (!swiglu) return n0 + r < N;
    return n0 + (r % (BN / 2)) < half_n;
  };

  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t wm = wave >> 1, wn = wave & 1u;  // 2x2 waves, each 64 rows x 64 columns

  if (tid < BN) s_bias[tid] = (bias && wrow_ok(tid)) ? bf16_bits_to_float(bias[wrow(tid)]) : 0.f;

  f32x16_t acc[2][2];  // [n-subtile][m-subtile]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  // each thread moves 4 x-chunks and 4 w-chunks (16 bytes each) per K step
  u32x4_t rx[4], rw[4];
  auto fetch = [&](uint32_t k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t c = tid + i * kGemmThreads;
      const uint32_t row = c >> 3, kc = (c & 7u) * 8;
      const bool kin = k0 + kc < K;
      const u32x4_t z = {0u, 0u, 0u, 0u};
      rx[i] = (kin && m0 + row < M) ? *reinterpret_cast<const u32x4_t*>(x + (size_t)(m0 + row) * ldx + k0 + kc) : z;
      if (!B_TRANS) {
        rw[i] = (kin && wrow_ok(row)) ? *reinterpret_cast<const u32x4_t*>(w + (size_t)wrow(row) * ldw + k0 + kc) : z;
      } else {
        // b[K][N]: gather 8 k-values of column n0+row (only the demo op uses this path)
        u32x4_t t = z;
        if (n0 + row < N) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t ka = k0 + kc + 2 * e;
            const uint32_t lo = ka < K ? w[(size_t)ka * ldw + n0 + row] : 0u;
            const uint32_t hi = ka + 1 < K ? w[(size_t)(ka + 1) * ldw + n0 + row] : 0u;
            t[e] = lo | (hi << 16);
          }
        }
        rw[i] = t;
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t c = tid + i * kGemmThreads;
      const uint32_t row = c >> 3, kc = (c & 7u) * 8;
      *reinterpret_cast<u32x4_t*>(sX + row * LDK + kc) = rx[i];
      *reinterpret_cast<u32x4_t*>(sW + row * LDK + kc) = rw[i];
    }
  };

  fetch(0);
  for (uint32_t k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
    stage();
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8_t wf[2], xf[2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
        wf[a] = *reinterpret_cast<const bf16x8_t*>(sW + (wn * 64 + a * 32 + lq) * LDK + ks * 16 + half * 8);
#pragma unroll
      for (int b = 0; b < 2; ++b)
        xf[b] = *reinterpret_cast<const bf16x8_t*>(sX + (wm * 64 + b * 32 + lq) * LDK + ks * 16 + half * 8);
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[a], xf[b], acc[a][b], 0, 0, 0);
    }
  }
  __syncthreads();  // operand tiles are dead; reuse their space for the output tile

  // acc[a][b][g*4+r] = C[row = wm*64 + b*32 + lq][col = wn*64 + a*32 + g*8 + half*4 + r]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t col = wn * 64 + a * 32 + g * 8 + half * 4;
        const uint32_t row = wm * 64 + b * 32 + lq;
        uint2 pk;
        pk.x = pack_bf16x2(acc[a][b][g * 4 + 0] + s_bias[col + 0], acc[a][b][g * 4 + 1] + s_bias[col + 1]);
        pk.y = pack_bf16x2(acc[a][b][g * 4 + 2] + s_bias[col + 2], acc[a][b][g * 4 + 3] + s_bias[col + 3]);
        *reinterpret_cast<uint2*>(sC + row * LDC + col) = pk;
      }
  __syncthreads();

  if (!swiglu) {
    // 128 rows x 16 chunks; 16 neighbouring threads write one 256-byte output row segment
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t c = tid + i * kGemmThreads;
      const uint32_t row = c >> 4, cc = (c & 15u) * 8;
      if (m0 + row >= M || n0 + cc >= N) continue;
      u32x4_t t = *reinterpret_cast<const u32x4_t*>(sC + row * LDC + cc);
      if (act != F3D_ACT_NONE || residual) {
        u32x4_t r = {0u, 0u, 0u, 0u};
        if (residual) r = *reinterpret_cast<const u32x4_t*>(residual + (size_t)(m0 + row) * ldr + n0 + cc);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float f0 = bf16_lo(t[e]), f1 = bf16_hi(t[e]);
          if (act != F3D_ACT_NONE) {
            const uint32_t a2 = pack_bf16x2(apply_act(f0, act), apply_act(f1, act));  // activation output is bf16
            f0 = bf16_lo(a2); f1 = bf16_hi(a2);
          }
          if (residual) { f0 += bf16_lo(r[e]); f1 += bf16_hi(r[e]); }
          t[e] = pack_bf16x2(f0, f1);
        }
      }
      *reinterpret_cast<u32x4_t*>(y + (size_t)(m0 + row) * ldy + n0 + cc) = t;
    }
  } else {
    // out[:, n0 + j] = silu(value_j) * gate_j, 64 output columns per tile
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t c = tid + i * kGemmThreads;
      const uint32_t row = c >> 3, cc = (c & 7u) * 8;
      if (m0 + row >= M || n0 + cc >= half_n) continue;
      const u32x4_t a = *reinterpret_cast<const u32x4_t*>(sC + row * LDC + cc);
      const u32x4_t gt = *reinterpret_cast<const u32x4_t*>(sC + row * LDC + BN / 2 + cc);
      u32x4_t r = {0u, 0u, 0u, 0u}, t;
      if (residual) r = *reinterpret_cast<const u32x4_t*>(residual + (size_t)(m0 + row) * ldr + n0 + cc);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a0 = bf16_lo(a[e]), a1 = bf16_hi(a[e]);
        float f0 = apply_act(a0, F3D_ACT_SILU) * bf16_lo(gt[e]);
        float f1 = apply_act(a1, F3D_ACT_SILU) * bf16_hi(gt[e]);
        if (residual) {
          const uint32_t h2 = pack_bf16x2(f0, f1);
          f0 = bf16_lo(h2) + bf16_lo(r[e]);
          f1 = bf16_hi(h2) + bf16_hi(r[e]);
        }
        t[e] = pack_bf16x2(f0, f1);
      }
      *reinterpret_cast<u32x4_t*>(y + (size_t)(m0 + row) * ldy + n0 + cc) = t;
    }
  }
}

// ---- LayerNorm: LPR lanes per row (a wave covers 64 / LPR rows), the row kept in registers, fp32
//      two-pass statistics.  LPR * VPL 16-byte chunks cover a row. ----
template <int LPR, int VPL>
__global__ __launch_bounds__(256) void layernorm_kernel(const uint16_t* __restrict__ x,
                                                        const uint16_t* __restrict__ gamma,
                                                        const uint16_t* __restrict__ beta, uint16_t* __restrict__ y,
                                                        uint32_t M, uint32_t C, float eps) {
  constexpr int RPW = kWave / LPR;  // rows per wave
  const uint32_t lane = threadIdx.x % kWave, sub = lane % LPR;
  const uint32_t row = (blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave) * RPW + lane / LPR;
  const bool row_ok = row < M;
  const uint32_t nchunk = C / 8;
  u32x4_t v[VPL];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const uint32_t c = sub + i * LPR;
    v[i] = u32x4_t{0u, 0u, 0u, 0u};
    if (row_ok && c < nchunk) v[i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)row * C + c * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) sum += bf16_lo(v[i][e]) + bf16_hi(v[i][e]);
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, kWave);
  const float mean = sum / (float)C;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const uint32_t c = sub + i * LPR;
    if (c < nchunk) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d0 = bf16_lo(v[i][e]) - mean, d1 = bf16_hi(v[i][e]) - mean;
        sq += d0 * d0 + d1 * d1;
      }
    }
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, kWave);
  const float rstd = rsqrtf(sq / (float)C + eps);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const uint32_t c = sub + i * LPR;
    if (row_ok && c < nchunk) {
      const u32x4_t g = *reinterpret_cast<const u32x4_t*>(gamma + c * 8);
      u32x4_t b = {0u, 0u, 0u, 0u}, t;
      if (beta) b = *reinterpret_cast<const u32x4_t*>(beta + c * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float f0 = (bf16_lo(v[i][e]) - mean) * rstd * bf16_lo(g[e]) + bf16_lo(b[e]);
        const float f1 = (bf16_hi(v[i][e]) - mean) * rstd * bf16_hi(g[e]) + bf16_hi(b[e]);
        t[e] = pack_bf16x2(f0, f1);
      }
      *reinterpret_cast<u32x4_t*>(y + (size_t)row * C + c * 8) = t;
    }
  }
}

static void launch_layernorm(const uint16_t* x, const uint16_t* gamma, const uint16_t* beta, uint16_t* y, uint32_t m,
                             uint32_t c, float eps, hipStream_t s) {
  const uint32_t nchunk = c / 8;
#define F3D_LN(LPR, VPL)                                                                                       \
  hipLaunchKernelGGL((layernorm_kernel<LPR, VPL>), dim3(cdiv_u32(m, 4 * (kWave / LPR))), dim3(256), 0, s, x, gamma, \
                     beta, y, m, c, eps)
  if (nchunk <= 4) F3D_LN(4, 1);
  else if (nchunk <= 8) F3D_LN(8, 1);
  else if (nchunk <= 16) F3D_LN(16, 1);
  else if (nchunk <= 32) F3D_LN(32, 1);
  else if (nchunk <= 64) F3D_LN(64, 1);
  else if (nchunk <= 128) F3D_LN(64, 2);
  else if (nchunk <= 256) F3D_LN(64, 4);
  else F3D_LN(64, 8);
#undef F3D_LN
}

// ---- coordinate embedding: y[r, :] = bf16(coord[r, :]) wT + bias, w [C,3].  A thread owns one
//      8-channel chunk (its 24 weights and 8 biases stay in registers) and walks down the rows;
//      the C/8 threads of a row write one contiguous burst. ----
__global__ __launch_bounds__(256) void coord_embed_kernel(const uint16_t* __restrict__ coord,
                                                          const uint16_t* __restrict__ w,
                                                          const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
                                                          uint32_t M, uint32_t C, uint32_t rows_per_block) {
  const uint32_t cpr = C / 8;
  const uint32_t slots = blockDim.x / cpr;              // rows handled concurrently by the block
  const uint32_t ch = (threadIdx.x % cpr) * 8, slot = threadIdx.x / cpr;
  if (slot >= slots) return;
  float wx[8], wy[8], wz[8], bb[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint16_t* wr = w + (size_t)(ch + e) * 3;
    wx[e] = bf16_bits_to_float(wr[0]); wy[e] = bf16_bits_to_float(wr[1]); wz[e] = bf16_bits_to_float(wr[2]);
    bb[e] = bias ? bf16_bits_to_float(bias[ch + e]) : 0.f;
  }
  const uint32_t r_begin = blockIdx.x * rows_per_block;
  const uint32_t r_end = min(r_begin + rows_per_block, M);
  for (uint32_t row = r_begin + slot; row < r_end; row += slots) {
    float p[3];
#pragma unroll
    for (int d = 0; d < 3; ++d)  // fp16 -> bf16 cast of the layer input (psh_ops.py:67)
      p[d] = bf16_bits_to_float(float_to_bf16_bits(half_bits_to_float(coord[3 * (size_t)row + d])));
    u32x4_t t;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float f0 = __builtin_fmaf(p[2], wz[2 * e], __builtin_fmaf(p[1], wy[2 * e], p[0] * wx[2 * e])) + bb[2 * e];
      float f1 = __builtin_fmaf(p[2], wz[2 * e + 1], __builtin_fmaf(p[1], wy[2 * e + 1], p[0] * wx[2 * e + 1])) + bb[2 * e + 1];
      t[e] = pack_bf16x2(f0, f1);
    }
    *reinterpret_cast<u32x4_t*>(y + (size_t)row * C + ch) = t;
  }
}

// ---- y = act(x * scale[c] + shift[c]) --------------------------------------------------------------
__global__ __launch_bounds__(256) void affine_act_kernel(const uint16_t* __restrict__ x, const float* __restrict__ scale,
                                                         const float* __restrict__ shift, uint16_t* __restrict__ y,
                                                         uint32_t M, uint32_t C, uint32_t act) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t cpr = C / 8;
  const uint32_t row = (uint32_t)(gid / cpr), ch = (uint32_t)(gid % cpr) * 8;
  if (row >= M) return;
  const U16x8 t = *reinterpret_cast<const U16x8*>(x + (size_t)row * C + ch);
  U16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // normalisation output is rounded to bf16 before the activation, as two separate modules would
    float f = __builtin_fmaf(bf16_bits_to_float(t.v[e]), scale[ch + e], shift[ch + e]);
    if (act != F3D_ACT_NONE) f = apply_act(bf16_bits_to_float(float_to_bf16_bits(f)), act);
    o.v[e] = float_to_bf16_bits(f);
  }
  *reinterpret_cast<U16x8*>(y + (size_t)row * C + ch) = o;
}

int launch_xstat_linear(const uint16_t* x, uint32_t ldx, const uint16_t* gamma, const uint16_t* beta, float eps,
                        const uint16_t* w, const uint16_t* bias, const uint16_t* residual, uint32_t ldr, uint16_t* y,
                        uint32_t ldy, uint32_t M, uint32_t N, uint32_t K, uint32_t act, int device, hipStream_t s,
                        const uint16_t* coord = nullptr, const uint16_t* etab = nullptr);
// output-panel kernel for long inner dimensions and 128 / 256 outputs (ystat_linear.hip); F3D_ERR_UNSUPPORTED otherwise
int launch_ystat_linear(const uint16_t* x, uint32_t ldx, const uint16_t* w, const uint16_t* bias,
                        const uint16_t* residual, uint32_t ldr, uint16_t* y, uint32_t ldy, uint32_t M, uint32_t N,
                        uint32_t K, uint32_t act, int device, hipStream_t s);

static int launch_gemm(bool b_trans, const uint16_t* x, uint32_t ldx, const uint16_t* w, uint32_t ldw,
                       const uint16_t* bias, const uint16_t* residual, uint32_t ldr, uint16_t* y, uint32_t ldy,
                       uint32_t M, uint32_t N, uint32_t K, uint32_t act, hipStream_t s) {
  const uint32_t n_eff = act == F3D_ACT_SWIGLU ? N / 2 : N;
  const uint32_t tiles_m = cdiv_u32(M, BM);
  const uint32_t tiles_n = act == F3D_ACT_SWIGLU ? cdiv_u32(n_eff, BN / 2) : cdiv_u32(n_eff, BN);
  const uint64_t n_tiles64 = (uint64_t)tiles_m * tiles_n;
  if (n_tiles64 == 0) return F3D_OK;
  if (n_tiles64 > 0x7FFFFFF0ull) {
    set_error("GEMM too large for one launch (%llu tiles)", (unsigned long long)n_tiles64);
    return F3D_ERR_INVALID;
  }
  const uint32_t n_tiles = (uint32_t)n_tiles64;
  const uint32_t per_xcd = cdiv_u32(n_tiles, kNumXcdG);
  if (b_trans)
    hipLaunchKernelGGL(gemm_bf16_kernel<true>, dim3(per_xcd * kNumXcdG), dim3(kGemmThreads), kGemmLds, s, x, ldx, w, ldw,
                       bias, residual, ldr, y, ldy, M, N, K, act, tiles_n, n_tiles, per_xcd);
  else
    hipLaunchKernelGGL(gemm_bf16_kernel<false>, dim3(per_xcd * kNumXcdG), dim3(kGemmThreads), kGemmLds, s, x, ldx, w,
                       ldw, bias, residual, ldr, y, ldy, M, N, K, act, tiles_n, n_tiles, per_xcd);
  return F3D_OK;
}

}  // namespace f3d

extern "C" {

int f3d_linear_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* w, const f3d_bf16_t* bias,
                    const f3d_bf16_t* residual, uint32_t ldr, f3d_bf16_t* y, uint32_t ldy, uint32_t m, uint32_t n,
                    uint32_t k, uint32_t act, int device, void* stream) {
  using namespace f3d;
  StagedWeightsScope staged;
  F3D_CHECK_ARG(x && w && y, "null tensor pointer");
  F3D_CHECK_ARG(act <= F3D_ACT_RELU, "unknown activation id %u", act);
  const uint32_t n_out = act == F3D_ACT_SWIGLU ? n / 2 : n;
  F3D_CHECK_ARG(k % 8 == 0 && k > 0, "inner dimension K=%u must be a positive multiple of 8", k);
  F3D_CHECK_ARG(n_out % 8 == 0 && (act != F3D_ACT_SWIGLU || n % 16 == 0),
                "output width %u must be a multiple of 8", n_out);
  F3D_CHECK_ARG(ldx >= k && ldx % 8 == 0 && ldy >= n_out && ldy % 8 == 0 && (!residual || (ldr >= n_out && ldr % 8 == 0)),
                "row strides must be multiples of 8 and cover a row (ldx=%u ldy=%u ldr=%u)", ldx, ldy, ldr);
  F3D_CHECK_ARG((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)residual) & 15u) == 0,
                "x/w/y/residual must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  // small inner dimensions: row-panel kernel (x read once, w streamed); long inner dimensions with 128 / 256 outputs:
  // output-panel kernel (x streamed once, y in registers); otherwise the tiled GEMM
  int rc = launch_xstat_linear(x, ldx, nullptr, nullptr, 0.f, w, bias, residual, ldr, y, ldy, m, n, k, act, device, s);
  if (rc == F3D_ERR_UNSUPPORTED) rc = launch_ystat_linear(x, ldx, w, bias, residual, ldr, y, ldy, m, n, k, act, device, s);
  if (rc == F3D_ERR_UNSUPPORTED) rc = launch_gemm(false, x, ldx, w, k, bias, residual, ldr, y, ldy, m, n, k, act, s);
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_ln_linear_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                       const f3d_bf16_t* w, const f3d_bf16_t* bias, const f3d_bf16_t* residual, uint32_t ldr,
                       f3d_bf16_t* y, uint32_t ldy, uint32_t m, uint32_t n, uint32_t k, uint32_t act, int device,
                       void* stream) {
  using namespace f3d;
  StagedWeightsScope staged;
  F3D_CHECK_ARG(x && gamma && w && y, "null tensor pointer");
  F3D_CHECK_ARG(act <= F3D_ACT_RELU, "unknown activation id %u", act);
  const uint32_t n_out = act == F3D_ACT_SWIGLU ? n / 2 : n;
  F3D_CHECK_ARG(k == 32 || k == 64 || k == 128 || k == 256 || k == 512,
                "No kernel found for LayerNorm+Linear with inner dimension K=%u (supported: 32, 64, 128, 256, 512)", k);
  F3D_CHECK_ARG(n_out % 8 == 0 && (act != F3D_ACT_SWIGLU || n % 64 == 0), "output width %u must be a multiple of 8", n_out);
  F3D_CHECK_ARG(ldx >= k && ldx % 8 == 0 && ldy >= n_out && ldy % 8 == 0 && (!residual || (ldr >= n_out && ldr % 8 == 0)),
                "row strides must be aligned and cover a row (ldx=%u ldy=%u ldr=%u)", ldx, ldy, ldr);
  F3D_CHECK_ARG((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)residual | (uintptr_t)gamma | (uintptr_t)beta) & 15u) == 0,
                "x/w/y/residual/gamma/beta must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  int rc = launch_xstat_linear(x, ldx, gamma, beta, eps, w, bias, residual, ldr, y, ldy, m, n, k, act, device, s);
  if (rc == F3D_ERR_UNSUPPORTED) {
    // shape outside the fused kernel: normalise into the per-device workspace, then the tiled GEMM
    uint16_t* tmp = (uint16_t*)workspace(device, (size_t)m * k * sizeof(uint16_t), s);
    if (!tmp) return F3D_ERR_RUNTIME;
    F3D_CHECK_ARG(ldx == k, "LayerNorm+Linear on a strided input needs an output width that is a multiple of 64");
    launch_layernorm(x, gamma, beta, tmp, m, k, eps, s);
    rc = launch_gemm(false, tmp, k, w, k, bias, residual, ldr, y, ldy, m, n, k, act, s);
  }
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_embed_ln_linear_bf16(const f3d_half_t* coord, const f3d_bf16_t* embed_table, const f3d_bf16_t* gamma,
                             const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w, const f3d_bf16_t* bias, f3d_bf16_t* y,
                             uint32_t ldy, uint32_t m, uint32_t n, uint32_t k, int device, void* stream) {
  using namespace f3d;
  StagedWeightsScope staged;
  F3D_CHECK_ARG(coord && embed_table && gamma && w && y, "null tensor pointer");
  if (!(k == 32 || k == 64 || k == 128 || k == 256) || n % 32 != 0) {
    set_error("No embedding + LayerNorm + Linear kernel for width %u with %u outputs (widths 32, 64, 128, 256; outputs a "
              "multiple of 32)", k, n);
    return F3D_ERR_UNSUPPORTED;
  }
  F3D_CHECK_ARG(ldy >= n && ldy % 8 == 0, "row stride must be aligned and cover a row (ldy=%u)", ldy);
  F3D_CHECK_ARG((((uintptr_t)embed_table | (uintptr_t)w | (uintptr_t)y | (uintptr_t)gamma | (uintptr_t)beta) & 15u) == 0 &&
                    ((uintptr_t)coord & 1u) == 0,
                "embed_table/w/y/gamma/beta must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const int rc = launch_xstat_linear(nullptr, 0, gamma, beta, eps, w, bias, nullptr, 0, y, ldy, m, n, k, F3D_ACT_NONE, device,
                                     s, coord, embed_table);
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_gemm_sm_bf16(const f3d_bf16_t* a, const f3d_bf16_t* b, f3d_bf16_t* o, uint32_t m, uint32_t n, uint32_t k,
                     int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(a && b && o, "null tensor pointer");
  F3D_CHECK_ARG(k % 8 == 0 && n % 8 == 0 && k > 0, "gemm_sm_bf16 needs K and N to be multiples of 8 (K=%u N=%u)", k, n);
  F3D_CHECK_ARG((((uintptr_t)a | (uintptr_t)o) & 15u) == 0, "A/O must be 16-byte aligned");
  if (m == 0 || n == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  int rc = launch_gemm(true, a, k, b, n, nullptr, nullptr, 0, o, n, m, n, k, F3D_ACT_NONE, s);
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_layernorm_bf16(const f3d_bf16_t* x, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, f3d_bf16_t* y,
                       uint32_t m, uint32_t c, float eps, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(x && gamma && y, "null tensor pointer");
  F3D_CHECK_ARG(c % 8 == 0 && c >= 8 && c <= 4096, "LayerNorm width %u must be a multiple of 8 in [8, 4096]", c);
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  launch_layernorm(x, gamma, beta, y, m, c, eps, s);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_coord_embed_bf16(const f3d_half_t* coord, const f3d_bf16_t* w, const f3d_bf16_t* bias, f3d_bf16_t* y,
                         uint32_t m, uint32_t c, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(coord && w && y, "null tensor pointer");
  F3D_CHECK_ARG(c % 8 == 0 && c > 0 && c <= 2048, "embedding width %u must be a multiple of 8 in [8, 2048]", c);
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const uint32_t slots = 256 / (c / 8);
  uint32_t rows_per_block = slots * 16;                       // 16 rows per thread amortise the weight loads
  while (rows_per_block > slots && cdiv_u32(m, rows_per_block) < 1024) rows_per_block /= 2;
  hipLaunchKernelGGL(coord_embed_kernel, dim3(cdiv_u32(m, rows_per_block)), dim3(256), 0, s, coord, w, bias, y, m, c,
                     rows_per_block);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_affine_act_bf16(const f3d_bf16_t* x, const float* scale, const float* shift, f3d_bf16_t* y, uint32_t m,
                        uint32_t c, uint32_t act, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(x && scale && shift && y, "null tensor pointer");
  F3D_CHECK_ARG(c % 8 == 0 && c > 0, "channel count %u must be a positive multiple of 8", c);
  F3D_CHECK_ARG(act <= F3D_ACT_RELU && act != F3D_ACT_SWIGLU, "unsupported activation id %u", act);
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const size_t total = (size_t)m * (c / 8);
  hipLaunchKernelGGL(affine_act_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, x, scale, shift, y, m, c,
                     act);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
