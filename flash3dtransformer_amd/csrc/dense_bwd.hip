// Backward of the dense layers for gfx950: weight / bias gradient of a linear layer, LayerNorm backward and the
// backward of the gated activation.  The input gradient of a linear layer is itself a linear layer (dx = dy · w), so it
// runs on the forward kernels with the transposed weight.
//
// The reference takes these from torch.nn.Linear / TransformerEngine autograd (flash3dxfmr/layers/buck_swin.py:159-163,
// elem_wise.py:22-26, stage.py:94-99); nothing of it lives in the reference's own sources.
//
// Weight gradient  dw[n][k] = sum_m dy[m][n] x[m][k]  (fp32 out, bf16 in):
//   the reduction runs over the rows, which is the slow axis of both operands in memory, so both MFMA operands are
//   read TRANSPOSED from LDS (ds_read_b64_tr_b16: a lane receives four consecutive rows of one column).  A workgroup of
//   eight waves (4 x 2, two per SIMD) owns a 256 x 256 tile of dw and one slab of rows; a wave holds 64 x 128 of it in
//   128 accumulator registers and skips the 32 x 32 blocks that lie outside dw.  32-row stages stream HBM -> LDS
//   directly (global_load ... lds, no registers) through four stage buffers, so three stages are in flight behind the
//   one being multiplied; one barrier per stage.  Slabs are sized so that the launch is one round of the chip; every
//   slab writes its partial tile to the workspace and a second kernel sums the slabs in a fixed order (no atomics: the
//   result does not depend on scheduling).  The bias gradient rides along in the waves of the first k-tile as one more
//   product with a matrix of ones.
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

constexpr int kXcd = 8;
constexpr int kWgThreads = 512, kWgWaves = kWgThreads / kWave;
constexpr int kWgNT = 256, kWgKT = 256;      // tile of dw per workgroup
constexpr int kWgMT = 32;                    // rows per stage
constexpr int kWgNBuf = 4;                   // stage buffers: three stages in flight behind the one being multiplied
constexpr int kRowB = 512;                   // bytes per LDS row of either operand tile (256 bf16, no padding)
constexpr int kTileB = kWgMT * kRowB;        // one operand tile of a stage
constexpr int kWgBuf = 2 * kTileB;
constexpr int kWgLds = kWgNBuf * kWgBuf;
constexpr int kDmaPerTile = kTileB / 1024 / kWgWaves;   // direct loads (1 KB each) per wave, operand and stage
static_assert(kWgNT == 256 && kWgKT == 256 && kRowB == 512, "one direct load fills two LDS rows of 32 pieces");
static_assert(kDmaPerTile * kWgWaves * 1024 == kTileB && kWgLds <= 160 * 1024, "stage geometry");

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds + 16 l
__device__ __forceinline__ void wg_dma16(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

// two transposing reads -> one 8-value MFMA operand: slots 0..3 = rows r .. r+3, slots 4..7 = rows r+4 .. r+7 of the
// lane's column (the same row order for both operands, so the products pair up)
__device__ __forceinline__ bf16x8_t read_tr8(const char* p) {
  const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)p);
  const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(p + 4 * kRowB));
  return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// LDS layout of an operand tile: row r at r * 512 bytes, its 16-byte piece c stored at position c ^ 4 (r % 4).  The
// direct loads write positions linearly (a lane picks the global piece that belongs at its position).  A transposing
// read has 32 lanes touch 64 bytes of each of four consecutive rows; the swizzle sends the four rows to the four
// 64-byte quarters of the 256 bytes the 64 banks serve per clock (without it the rows, a multiple of 256 bytes apart,
// would all meet in the same banks).
__global__ __launch_bounds__(kWgThreads) void linear_wgrad_kernel(
    const uint16_t* __restrict__ dy, uint32_t lddy, const uint16_t* __restrict__ x, uint32_t ldx,
    float* __restrict__ part_w, float* __restrict__ part_b, uint32_t M, uint32_t N, uint32_t K, uint32_t n_tiles,
    uint32_t k_tiles, uint32_t slabs, uint32_t slab_rows, uint32_t items_per_xcd) {
  extern __shared__ __attribute__((aligned(16))) char lds_wg[];
  // workgroups of one XCD take consecutive items, so the tiles of one slab (which re-read the same rows of x and
  // dy) meet in one L2
  const uint32_t tiles = n_tiles * k_tiles, n_items = tiles * slabs;
  const uint32_t item = (blockIdx.x % kXcd) * items_per_xcd + blockIdx.x / kXcd;
  if (blockIdx.x / kXcd >= items_per_xcd || item >= n_items) return;
  const uint32_t slab = item / tiles, tile = item % tiles;
  const uint32_t n0 = (tile / k_tiles) * kWgNT, k0 = (tile % k_tiles) * kWgKT;
  const uint32_t m_begin = slab * slab_rows, m_end = min(M, m_begin + slab_rows);
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  // 4 x 2 waves; the two waves of a SIMD (wave, wave + 4) sit in different k halves
  const uint32_t nw = wave & 3u, kw = wave >> 2;
  const bool with_bias = part_b != nullptr && k0 == 0 && kw == 0;
  // 32 x 32 blocks of this wave's 64 x 128 that lie inside dw
  const uint32_t n_w = n0 + nw * 64u, k_w = k0 + kw * 128u;
  const uint32_t ni = n_w >= N ? 0u : min(2u, (N - n_w + 31u) / 32u), nj = k_w >= K ? 0u : min(4u, (K - k_w + 31u) / 32u);

  // ---- direct loads: instruction q of a tile fills rows 2q, 2q + 1; this wave issues q = kDmaPerTile wave + i.
  //      Pieces beyond the last column are clamped to the last valid piece (they only reach blocks of dw that are
  //      never stored), rows beyond the slab to its last row (and zeroed in LDS once they have landed). ----
  const uint32_t pieces_a = min(32u, (N - n0) / 8u), pieces_b = min(32u, (K - k0) / 8u);
  uint32_t d_row[kDmaPerTile], d_ca[kDmaPerTile], d_cb[kDmaPerTile];
#pragma unroll
  for (int i = 0; i < kDmaPerTile; ++i) {
    const uint32_t q = kDmaPerTile * wave + i;
    d_row[i] = 2u * q + lane / 32u;
    const uint32_t c = (lane & 31u) ^ ((d_row[i] & 3u) << 2);
    d_ca[i] = min(c, pieces_a - 1u) * 16u;
    d_cb[i] = min(c, pieces_b - 1u) * 16u;
  }
  auto issue = [&](uint32_t st) {
    const uint32_t m0 = m_begin + st * kWgMT, last = m_end - 1u - m0;   // m0 < m_end
    const char* ga = reinterpret_cast<const char*>(dy + (size_t)m0 * lddy + n0);
    const char* gb = reinterpret_cast<const char*>(x + (size_t)m0 * ldx + k0);
    char* buf = lds_wg + (st % kWgNBuf) * kWgBuf;
#pragma unroll
    for (int i = 0; i < kDmaPerTile; ++i) {
      const uint32_t r = min(d_row[i], last), q = kDmaPerTile * wave + i;
      wg_dma16(ga, r * lddy * 2u + d_ca[i], buf + q * 1024);
      wg_dma16(gb, r * ldx * 2u + d_cb[i], buf + kTileB + q * 1024);
    }
  };

  // ---- the lane's place in a transposing read: lane p of a 16-lane block points at row p / 4, columns 4 (p % 4)..;
  //      the swizzle value 4 (row % 4) = 4 (p / 4) is the same for every row the lane ever reads ----
  const uint32_t half = lane >> 5, p16 = lane & 15u, cgrp = (lane >> 4) & 1u;
  const uint32_t row_off = (8u * half + p16 / 4u) * kRowB, sw = (p16 / 4u) << 2, in_piece = 8u * (p16 & 1u);
  uint32_t a_off[2], b_off[4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
    a_off[i] = row_off + (((nw * 8u + 4u * i + 2u * cgrp + ((p16 & 3u) >> 1)) ^ sw) << 4) + in_piece;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    b_off[j] = kTileB + row_off + (((kw * 16u + 4u * j + 2u * cgrp + ((p16 & 3u) >> 1)) ^ sw) << 4) + in_piece;

  f32x16_t acc[2][4], accb[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) accb[i][e] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  }
  bf16x8_t ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;

  const uint32_t n_stage = m_end > m_begin ? (m_end - m_begin + kWgMT - 1) / kWgMT : 0u;
  static_assert(kWgMT == 32, "two k-steps per stage");
  // waits until this wave's loads of stage st have landed (at most the loads of the later stages, two of them at
  // that point, stay outstanding), zeroes the rows past the slab, and meets the other waves: after the barrier the
  // whole stage is in LDS and every wave has its operands of the stages before it in registers
  auto stage_ready = [&](uint32_t st) {
    const uint32_t later = min(n_stage - 1u - st, 2u);
    if (later == 2u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * kDmaPerTile) : "memory");
    else if (later == 1u) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDmaPerTile) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint32_t rows_left = m_end - (m_begin + st * kWgMT);
    if (rows_left < (uint32_t)kWgMT) {
      char* buf = lds_wg + (st % kWgNBuf) * kWgBuf;
#pragma unroll
      for (int i = 0; i < kDmaPerTile; ++i)
        if (d_row[i] >= rows_left) {
          const uint32_t pos = (kDmaPerTile * wave + i) * 1024u + lane * 16u;
          *reinterpret_cast<u32x4_t*>(buf + pos) = u32x4_t{0u, 0u, 0u, 0u};
          *reinterpret_cast<u32x4_t*>(buf + kTileB + pos) = u32x4_t{0u, 0u, 0u, 0u};
        }
    }
    wg_barrier_lds();
  };
  bf16x8_t fa[2][2], fb[2][4];
  auto frags = [&](uint32_t st, int ks, bf16x8_t (&a)[2], bf16x8_t (&b)[4]) {
    const char* buf = lds_wg + (st % kWgNBuf) * kWgBuf;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if ((uint32_t)i < ni) a[i] = read_tr8(buf + a_off[i] + ks * 16 * kRowB);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if ((uint32_t)j < nj) b[j] = read_tr8(buf + b_off[j] + ks * 16 * kRowB);
  };
  auto products = [&](const bf16x8_t (&a)[2], const bf16x8_t (&b)[4]) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if ((uint32_t)i < ni && (uint32_t)j < nj)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    if (with_bias) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if ((uint32_t)i < ni) accb[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], ones, accb[i], 0, 0, 0);
    }
  };
  // Three stages are requested ahead.  The hand-over to the next stage (wait, barrier, first operand reads) sits
  // between the two k-steps of a stage, so the products of the second k-step run over it.
#pragma unroll
  for (int st = 0; st < kWgNBuf - 1; ++st)
    if ((uint32_t)st < n_stage) issue(st);
  if (n_stage) {
    stage_ready(0);
    frags(0, 0, fa[0], fb[0]);
  }
  for (uint32_t st = 0; st < n_stage; ++st) {
    // the buffer of stage st - 1 is free: every wave read the last of it before the barrier that made stage st ready
    if (st + kWgNBuf - 1 < n_stage) issue(st + kWgNBuf - 1);
    frags(st, 1, fa[1], fb[1]);
    products(fa[0], fb[0]);
    if (st + 1 < n_stage) {
      stage_ready(st + 1);   // stages st + 2 and st + 3 are the ones still in flight
      frags(st + 1, 0, fa[0], fb[0]);
    }
    products(fa[1], fb[1]);
  }

  // ---- this slab's partial tile: accumulator slot e of a lane is row 8 (e / 4) + 4 half + e % 4, column lane % 32 ----
  float* pw = part_w + (size_t)slab * N * K;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint32_t n = n_w + 32u * i + 8u * (e / 4) + 4u * half + (e % 4);
      if (n >= N) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t k = k_w + 32u * j + (lane & 31u);
        if (k < K) pw[(size_t)n * K + k] = acc[i][j][e];
      }
      // every column of the product with the matrix of ones holds the row sum
      if (with_bias && (lane & 31u) == 0) part_b[(size_t)slab * N + n] = accb[i][e];
    }
  }
}

// out[i] = (accumulate ? out[i] : 0) + sum over p of part[p][i], for two arrays in one launch (the weight gradient and,
// in the workgroups past blocks_a, the bias gradient; len_b may be 0).  A workgroup owns 256 consecutive elements (64
// lanes x 4 floats, lengths are multiples of 4); its 16 partial groups each sum every 16th partial (independent 16-byte
// loads), then the first group adds the 16 group sums in ascending order: a fixed summation tree.
__global__ __launch_bounds__(1024) void sum_partials_kernel(const float* __restrict__ part_a, size_t len_a,
                                                            float* __restrict__ out_a, uint32_t blocks_a,
                                                            const float* __restrict__ part_b, size_t len_b,
                                                            float* __restrict__ out_b, uint32_t n_part,
                                                            uint32_t accumulate) {
  __shared__ float4 s_sum[16][64];
  const bool second = blockIdx.x >= blocks_a;
  const float* part = second ? part_b : part_a;
  float* out = second ? out_b : out_a;
  const size_t len = second ? len_b : len_a;
  const uint32_t tid = threadIdx.x, l = tid & 63u, g = tid >> 6;
  const size_t i = ((size_t)(blockIdx.x - (second ? blocks_a : 0u)) * 64u + l) * 4u;
  float4 s = {0.f, 0.f, 0.f, 0.f};
  if (i < len)
    for (uint32_t p = g; p < n_part; p += 16u) {
      const float4 v = *reinterpret_cast<const float4*>(part + (size_t)p * len + i);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  s_sum[g][l] = s;
  __syncthreads();
  if (g == 0 && i < len) {
    float4 t = {0.f, 0.f, 0.f, 0.f};
    if (accumulate) t = *reinterpret_cast<const float4*>(out + i);
    for (int r = 0; r < 16; ++r) {
      const float4 v = s_sum[r][l];
      t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
    }
    *reinterpret_cast<float4*>(out + i) = t;
  }
}

// ---- LayerNorm backward: LPR lanes per row, 8 channels per lane.
//   xhat = (x - mean) rstd, g = dh gamma, dx = rstd (g - mean(g) - xhat mean(g xhat)) (+ dres),
//   dgamma = sum_rows dh xhat, dbeta = sum_rows dh.  A thread walks rows with a grid stride and keeps its 8 + 8 column
//   sums in registers; the workgroup combines them through LDS and writes one partial per workgroup. ----
template <int LPR>
__global__ __launch_bounds__(256) void layernorm_bwd_kernel(const uint16_t* __restrict__ x, uint32_t ldx,
                                                            const uint16_t* dh, uint32_t lddh,
                                                            const uint16_t* __restrict__ gamma,
                                                            const uint16_t* dres, uint32_t lddr,
                                                            uint16_t* dx, uint32_t lddx,
                                                            float* __restrict__ part, uint32_t M, float eps) {
  constexpr int C = LPR * 8, RPB = 256 / LPR;
  __shared__ float s_col[256][17];
  const uint32_t tid = threadIdx.x, sub = tid % LPR, slot = tid / LPR;
  float g8[8], dg[8], db[8];
  {
    const u32x4_t g = *reinterpret_cast<const u32x4_t*>(gamma + sub * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) { g8[2 * e] = bf16_lo(g[e]); g8[2 * e + 1] = bf16_hi(g[e]); }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) dg[e] = db[e] = 0.f;
  // every lane of a row group runs the same number of iterations (the shuffles need all of them)
  for (uint32_t base = blockIdx.x * RPB; base < M; base += gridDim.x * RPB) {
    const uint32_t row = base + slot;
    const bool ok = row < M;
    u32x4_t vx = {0u, 0u, 0u, 0u}, vd = {0u, 0u, 0u, 0u}, vr = {0u, 0u, 0u, 0u};
    if (ok) {
      vx = *reinterpret_cast<const u32x4_t*>(x + (size_t)row * ldx + sub * 8);
      vd = *reinterpret_cast<const u32x4_t*>(dh + (size_t)row * lddh + sub * 8);
      if (dres) vr = *reinterpret_cast<const u32x4_t*>(dres + (size_t)row * lddr + sub * 8);
    }
    float xv[8], dv[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      xv[2 * e] = bf16_lo(vx[e]); xv[2 * e + 1] = bf16_hi(vx[e]);
      dv[2 * e] = bf16_lo(vd[e]); dv[2 * e + 1] = bf16_hi(vd[e]);
    }
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += xv[e];
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, kWave);
    const float mean = sum / (float)C;
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { xv[e] -= mean; sq += xv[e] * xv[e]; }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) sq += __shfl_xor(sq, off, kWave);
    const float rstd = rsqrtf(sq / (float)C + eps);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xv[e] *= rstd;                       // xhat
      const float g = dv[e] * g8[e];
      s1 += g; s2 += g * xv[e];
      dg[e] += dv[e] * xv[e]; db[e] += dv[e];   // rows past the end contribute zeros (dh = 0)
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) {
      s1 += __shfl_xor(s1, off, kWave);
      s2 += __shfl_xor(s2, off, kWave);
    }
    s1 /= (float)C; s2 /= (float)C;
    if (ok) {
      u32x4_t t;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float f0 = rstd * (dv[2 * e] * g8[2 * e] - s1 - xv[2 * e] * s2) + bf16_lo(vr[e]);
        float f1 = rstd * (dv[2 * e + 1] * g8[2 * e + 1] - s1 - xv[2 * e + 1] * s2) + bf16_hi(vr[e]);
        t[e] = pack_bf16x2(f0, f1);
      }
      *reinterpret_cast<u32x4_t*>(dx + (size_t)row * lddx + sub * 8) = t;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) { s_col[tid][e] = dg[e]; s_col[tid][8 + e] = db[e]; }
  __syncthreads();
  // thread (sub, e) for e < 16 sums the RPB row slots of its column
  for (uint32_t o = tid; o < LPR * 16u; o += 256u) {
    const uint32_t su = o / 16u, e = o % 16u;
    float s = 0.f;
    for (uint32_t r = 0; r < (uint32_t)RPB; ++r) s += s_col[r * LPR + su][e];
    // partial layout per workgroup: dgamma [C] then dbeta [C]
    part[(size_t)blockIdx.x * 2u * C + (e / 8u) * C + su * 8u + (e % 8u)] = s;
  }
}

// ---- gated activation backward: a = silu(z1) z2, dz1 = da z2 s (1 + z1 (1 - s)), dz2 = da silu(z1), s = sigmoid(z1);
//      z = [z1 | z2] per row.  dz may alias z and a may alias da (a thread reads its pieces before it writes them). ----
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* z, uint32_t ldz, const uint16_t* da,
                                                         uint32_t ldda, uint16_t* dz, uint32_t lddz, uint16_t* a,
                                                         uint32_t lda, uint32_t M, uint32_t H) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t cpr = H / 8;
  const uint32_t row = (uint32_t)(gid / cpr), ch = (uint32_t)(gid % cpr) * 8;
  if (row >= M) return;
  const u32x4_t v1 = *reinterpret_cast<const u32x4_t*>(z + (size_t)row * ldz + ch);
  const u32x4_t v2 = *reinterpret_cast<const u32x4_t*>(z + (size_t)row * ldz + H + ch);
  const u32x4_t vd = *reinterpret_cast<const u32x4_t*>(da + (size_t)row * ldda + ch);
  u32x4_t o1, o2, oa;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r1[2], r2[2], ra[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float z1 = h ? bf16_hi(v1[e]) : bf16_lo(v1[e]);
      const float z2 = h ? bf16_hi(v2[e]) : bf16_lo(v2[e]);
      const float d = h ? bf16_hi(vd[e]) : bf16_lo(vd[e]);
      const float s = 1.f / (1.f + __expf(-z1));
      const float sl = z1 * s;
      ra[h] = sl * z2;
      r1[h] = d * z2 * s * (1.f + z1 * (1.f - s));
      r2[h] = d * sl;
    }
    o1[e] = pack_bf16x2(r1[0], r1[1]);
    o2[e] = pack_bf16x2(r2[0], r2[1]);
    oa[e] = pack_bf16x2(ra[0], ra[1]);
  }
  *reinterpret_cast<u32x4_t*>(dz + (size_t)row * lddz + ch) = o1;
  *reinterpret_cast<u32x4_t*>(dz + (size_t)row * lddz + H + ch) = o2;
  if (a) *reinterpret_cast<u32x4_t*>(a + (size_t)row * lda + ch) = oa;
}

// dgamma / dbeta from the per-workgroup partial rows [dgamma | dbeta].  A workgroup owns 16 columns; its 64 row
// groups each sum every 64th partial row (independent loads, so many are in flight), then one thread per column adds
// the 64 group sums in ascending order: a fixed summation tree.
__global__ __launch_bounds__(1024) void ln_bwd_reduce_kernel(const float* __restrict__ part, uint32_t n_part, uint32_t C,
                                                             float* __restrict__ dgamma, float* __restrict__ dbeta,
                                                             uint32_t accumulate) {
  __shared__ float s_red[64][17];
  const uint32_t tid = threadIdx.x, col = blockIdx.x * 16u + (tid & 15u), rg = tid >> 4;
  float s = 0.f;
  if (col < 2u * C)
    for (uint32_t p = rg; p < n_part; p += 64u) s += part[(size_t)p * 2u * C + col];
  s_red[rg][tid & 15u] = s;
  __syncthreads();
  if (tid < 16u && col < 2u * C) {
    float* out = col < C ? dgamma + col : dbeta + (col - C);
    float t = accumulate ? *out : 0.f;
    for (uint32_t r = 0; r < 64u; ++r) t += s_red[r][tid];
    *out = t;
  }
}

int n_cu_of(int device, uint32_t* n_cu) {
  int v = 0;
  F3D_CHECK_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device));
  *n_cu = v > 0 ? (uint32_t)v : 256u;
  return F3D_OK;
}

}  // namespace
}  // namespace f3d

extern "C" {

int f3d_linear_wgrad_bf16(const f3d_bf16_t* dy, uint32_t lddy, const f3d_bf16_t* x, uint32_t ldx, float* dw, float* db,
                          uint32_t m, uint32_t n, uint32_t k, uint32_t accumulate, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(((dy && x) || m == 0) && dw, "null tensor pointer");
  F3D_CHECK_ARG(n > 0 && k > 0 && n % 8 == 0 && k % 8 == 0, "n=%u and k=%u must be positive multiples of 8", n, k);
  F3D_CHECK_ARG(lddy >= n && lddy % 8 == 0 && ldx >= k && ldx % 8 == 0,
                "row strides must be multiples of 8 and cover a row (lddy=%u ldx=%u)", lddy, ldx);
  F3D_CHECK_ARG((((uintptr_t)dy | (uintptr_t)x | (uintptr_t)dw | (uintptr_t)db) & 15u) == 0,
                "dy / x / dw / db must be 16-byte aligned");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  uint32_t n_cu = 0;
  if (int rc = n_cu_of(device, &n_cu)) return rc;
  const uint32_t n_tiles = cdiv_u32(n, kWgNT), k_tiles = cdiv_u32(k, kWgKT), tiles = n_tiles * k_tiles;
  // one round of the chip: as many row slabs as there are compute units per tile
  uint32_t slabs = tiles >= n_cu ? 1u : n_cu / tiles;
  const uint32_t stages = cdiv_u32(m, kWgMT);
  if (slabs > stages) slabs = stages ? stages : 1u;
  const uint32_t slab_rows = cdiv_u32(cdiv_u32(m, slabs), kWgMT) * kWgMT;
  if (m) slabs = cdiv_u32(m, slab_rows);
  const size_t nk = (size_t)n * k;
  const size_t part_w_bytes = (size_t)slabs * nk * 4, part_b_bytes = db ? (size_t)slabs * n * 4 : 0;
  char* ws = (char*)workspace(device, part_w_bytes + part_b_bytes, s);
  if (!ws) return F3D_ERR_RUNTIME;
  float* part_w = (float*)ws;
  float* part_b = db ? (float*)(ws + part_w_bytes) : nullptr;
  static bool attr_set[64] = {};
  if (device >= 0 && device < 64 && !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)linear_wgrad_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kWgLds));
    attr_set[device] = true;
  }
  const uint32_t n_items = tiles * slabs, items_per_xcd = cdiv_u32(n_items, kXcd);
  hipLaunchKernelGGL(linear_wgrad_kernel, dim3(items_per_xcd * kXcd), dim3(kWgThreads), kWgLds, s, dy, lddy, x, ldx,
                     part_w, part_b, m, n, k, n_tiles, k_tiles, slabs, slab_rows, items_per_xcd);
  const uint32_t blocks_w = (uint32_t)((nk + 255) / 256), blocks_b = db ? cdiv_u32(n, 256) : 0u;
  hipLaunchKernelGGL(sum_partials_kernel, dim3(blocks_w + blocks_b), dim3(1024), 0, s, part_w, nk, dw, blocks_w, part_b,
                     db ? (size_t)n : (size_t)0, db, slabs, accumulate);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_layernorm_bwd_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* dh, uint32_t lddh,
                           const f3d_bf16_t* gamma, const f3d_bf16_t* dres, uint32_t lddr, f3d_bf16_t* dx, uint32_t lddx,
                           float* dgamma, float* dbeta, uint32_t m, uint32_t c, float eps, uint32_t accumulate,
                           int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(((x && dh && dx) || m == 0) && gamma && dgamma && dbeta, "null tensor pointer");
  if (!(c == 32 || c == 64 || c == 128 || c == 256 || c == 512)) {
    set_error("No kernel found for LayerNorm backward at width %u (supported: 32, 64, 128, 256, 512)", c);
    return F3D_ERR_UNSUPPORTED;
  }
  F3D_CHECK_ARG(ldx >= c && ldx % 8 == 0 && lddh >= c && lddh % 8 == 0 && lddx >= c && lddx % 8 == 0 &&
                    (!dres || (lddr >= c && lddr % 8 == 0)),
                "row strides must be multiples of 8 and cover a row");
  F3D_CHECK_ARG((((uintptr_t)x | (uintptr_t)dh | (uintptr_t)gamma | (uintptr_t)dres | (uintptr_t)dx) & 15u) == 0,
                "x / dh / gamma / dres / dx must be 16-byte aligned");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  uint32_t n_cu = 0;
  if (int rc = n_cu_of(device, &n_cu)) return rc;
  const uint32_t rpb = 256u / (c / 8u);
  uint32_t wgs = cdiv_u32(m, rpb);
  if (wgs > n_cu * 8u) wgs = n_cu * 8u;
  if (wgs == 0) wgs = 1;
  float* part = (float*)workspace(device, (size_t)wgs * 2u * c * 4u, s);
  if (!part) return F3D_ERR_RUNTIME;
#define F3D_LNB(LPR)                                                                                                \
  hipLaunchKernelGGL((layernorm_bwd_kernel<LPR>), dim3(wgs), dim3(256), 0, s, x, ldx, dh, lddh, gamma, dres, lddr, \
                     dx, lddx, part, m, eps)
  switch (c) {
    case 32: F3D_LNB(4); break;
    case 64: F3D_LNB(8); break;
    case 128: F3D_LNB(16); break;
    case 256: F3D_LNB(32); break;
    default: F3D_LNB(64); break;
  }
#undef F3D_LNB
  hipLaunchKernelGGL(ln_bwd_reduce_kernel, dim3(cdiv_u32(2u * c, 16)), dim3(1024), 0, s, part, wgs, c, dgamma, dbeta,
                     accumulate);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_swiglu_bwd_bf16(const f3d_bf16_t* z, uint32_t ldz, const f3d_bf16_t* da, uint32_t ldda, f3d_bf16_t* dz,
                        uint32_t lddz, f3d_bf16_t* a, uint32_t lda, uint32_t m, uint32_t hidden, int device,
                        void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(z && da && dz, "null tensor pointer");
  F3D_CHECK_ARG(hidden > 0 && hidden % 8 == 0, "hidden=%u must be a positive multiple of 8", hidden);
  F3D_CHECK_ARG(ldz >= 2 * hidden && ldz % 8 == 0 && lddz >= 2 * hidden && lddz % 8 == 0 && ldda >= hidden &&
                    ldda % 8 == 0 && (!a || (lda >= hidden && lda % 8 == 0)),
                "row strides must be multiples of 8 and cover a row");
  F3D_CHECK_ARG((((uintptr_t)z | (uintptr_t)da | (uintptr_t)dz | (uintptr_t)a) & 15u) == 0,
                "z / da / dz / a must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const size_t threads = (size_t)m * (hidden / 8);
  F3D_CHECK_ARG((threads + 255) / 256 <= 0x7FFFFFFFull, "too many rows");
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, s, z, ldz, da, ldda, dz,
                     lddz, a, lda, m, hidden);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
