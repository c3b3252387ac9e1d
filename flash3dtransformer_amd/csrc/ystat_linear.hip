// Output-panel ("y-stationary") linear layer for gfx950: y = x wT + bias (+ residual) for LONG inner dimensions and
// narrow outputs (N = 128 or 256), the fc2 of the blocks' MLPs (flash3dxfmr/layers/elem_wise.py:22-26, where the
// reference runs te.LayerNormMLP's second GEMM).
//
// The row-panel kernel keeps x in registers, which stops at 512 inner features.  Here the OUTPUT is what stays in
// registers: a workgroup of eight waves owns 256 rows; waves w and w + 4 (the two waves of a SIMD) share a block of 64
// rows and split the output columns, so a wave holds 64 rows x N/2 columns of fp32 accumulators (128 registers at
// N = 256) and two waves per SIMD fit.  x and w stream through LDS 32 inner features at a time, four buffers deep,
// straight from HBM / L2 (global_load ... lds): x is read exactly once, in 32-byte pieces that land already in the
// matrix core's operand order (no transposition), and w comes from a fragment-major copy made per call by a small
// preparation kernel, so every LDS read of the main loop is linear.  The product is formed transposed (A operand =
// rows of w) so that a lane ends up with 4 consecutive output columns of one row for the epilogue.
//
// HBM bound at these shapes: bytes = M (K + N (+ N)) 2 against 2 M N K flops.
#include "xstat_common.h"

namespace f3d {

// One ring of four buffers (w and x of a chunk side by side), chunk c + 3 requested when chunk c starts.  (Separate
// requester waves for x and w, which lets the x ring be seven deep because the count of outstanding loads is per
// wave, measured 6 % slower: bytes in flight are not what limits this kernel.)
constexpr int kYsWaves = 8, kYsMT = 2, kYsBufs = 4, kYsChunkK = 32;

template <int N>
struct YsGeom {
  static constexpr int OT = N / 32;                       // output column tiles
  static constexpr int OTW = OT / 2;                      // tiles per wave
  static constexpr int W_BYTES = OT * 2 * 1024;           // w of a chunk: OT tiles x 2 k-steps x 64 lanes x 16 bytes
  static constexpr int X_BYTES = 4 * kYsMT * 2 * 1024;    // x of a chunk: 4 row blocks x 2 row tiles x 2 k-steps
  static constexpr int BUF = W_BYTES + X_BYTES;
  static constexpr int W_DMA = W_BYTES / 1024 / kYsWaves; // direct loads per wave and chunk
  static constexpr int X_DMA = 2;
  static constexpr size_t lds_bytes() { return (size_t)kYsBufs * BUF; }
};

__device__ __forceinline__ void ys_wait_vm(uint32_t n) {
  switch (n) {
#define F3D_W(V) case V: __builtin_amdgcn_s_waitcnt(0x0F70 | V); break;
    F3D_W(0) F3D_W(1) F3D_W(2) F3D_W(3) F3D_W(4) F3D_W(5) F3D_W(6) F3D_W(7) F3D_W(8) F3D_W(9) F3D_W(10) F3D_W(11)
    F3D_W(12) F3D_W(13) F3D_W(14) F3D_W(15)
#undef F3D_W
    // counts of 16 and more: the two high bits of the count sit in bits 15:14 of the immediate
#define F3D_W(V) case V: __builtin_amdgcn_s_waitcnt(0x0F70 | (V & 15) | ((V >> 4) << 14)); break;
    F3D_W(16) F3D_W(17) F3D_W(18) F3D_W(19) F3D_W(20) F3D_W(21) F3D_W(22) F3D_W(23) F3D_W(24) F3D_W(25) F3D_W(26)
    F3D_W(27) F3D_W(28) F3D_W(29) F3D_W(30) F3D_W(31)
#undef F3D_W
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}

// wp: w fragment-major per chunk of 32 inner features (ys_w_prep_kernel); bias [N], never null (zeros stand in)
template <int N>
__global__ __launch_bounds__(64 * kYsWaves) __attribute__((amdgpu_waves_per_eu(2, 2))) void ystat_linear_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, const uint16_t* __restrict__ wp, const uint16_t* __restrict__ bias,
    const uint16_t* __restrict__ residual, uint32_t ldr, uint16_t* __restrict__ y, uint32_t ldy, uint32_t M,
    uint32_t K) {
  using G = YsGeom<N>;
  constexpr int WAVES = kYsWaves, MT = kYsMT, NB = kYsBufs, OTW = G::OTW;
  constexpr int ROWS_WG = 64 * 4;
  extern __shared__ __attribute__((aligned(1024))) char lds_ys[];

  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t rb = wave & 3u, cg = wave >> 2;          // row block of 64 rows, half of the output columns
  const uint32_t wg_row0 = blockIdx.x * ROWS_WG;
  const uint32_t row0 = wg_row0 + rb * 64;

  // accumulators start from the bias: acc[o][mt][g*4+r] <-> output column (cg*OTW + o)*32 + g*8 + half*4 + r, row lq
  f32x16_t acc[OTW][MT];
#pragma unroll
  for (int o = 0; o < OTW; ++o)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint2 bb = *reinterpret_cast<const uint2*>(bias + (cg * OTW + o) * 32 + g * 8 + half * 4);
      const float b[4] = {bf16_lo(bb.x), bf16_hi(bb.x), bf16_lo(bb.y), bf16_hi(bb.y)};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[o][mt][g * 4 + r] = b[r];
    }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // nothing of this wave is in flight when the direct loads start

  // ---- streaming ----
  const uint32_t nchunk = K / kYsChunkK;
  constexpr uint32_t kPerChunk = G::W_DMA + G::X_DMA;     // direct loads of this wave per chunk
  // x: this wave fetches row tile mt = cg of its row block, both k-steps.  Lane (lq, half) takes the 16 bytes that
  // are its B-operand piece: row lq of the tile, inner features s*16 + half*8 .. +8.  Rows past M read row M - 1.
  const uint32_t x_row = min(row0 + cg * 32 + lq, M - 1) - wg_row0;
  const uint32_t x_lane = (x_row * ldx + half * 8u) * 2u;
  const char* x_wg = reinterpret_cast<const char*>(x + (size_t)wg_row0 * ldx);
  const uint32_t w_lane = wave * 1024u + lane * 16u;
  auto dma_chunk = [&](uint32_t c) __attribute__((always_inline)) {
    char* buf = lds_ys + (c % NB) * G::BUF;
#pragma unroll
    for (uint32_t i = 0; i < (uint32_t)G::W_DMA; ++i)
      xs_lds_dma16(reinterpret_cast<const char*>(wp) + (size_t)c * G::W_BYTES + i * (WAVES * 1024), w_lane,
                   buf + (wave + i * WAVES) * 1024);
#pragma unroll
    for (uint32_t s = 0; s < 2; ++s)
      xs_lds_dma16(x_wg + (size_t)c * (kYsChunkK * 2) + s * 32, x_lane,
                   buf + G::W_BYTES + (((rb * MT + cg) * 2 + s) * 1024));
  };
  dma_chunk(0);
  if (nchunk > 1) dma_chunk(1);
  if (nchunk > 2) dma_chunk(2);
  // chunk 0 must have landed; up to two younger chunks may stay in flight
  ys_wait_vm(nchunk > 2 ? 2 * kPerChunk : (nchunk > 1 ? kPerChunk : 0));
  wg_barrier_lds();

  for (uint32_t ci = 0; ci < nchunk; ++ci) {
    // chunk ci + 3 goes into the buffer of chunk ci - 1, which every wave has left
    if (ci + 3 < nchunk) dma_chunk(ci + 3);
    const char* buf = lds_ys + (ci % NB) * G::BUF;
    const char* sx = buf + G::W_BYTES + rb * (MT * 2 * 1024) + lane * 16;
    const char* sw = buf + (cg * OTW) * 2048 + lane * 16;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      bf16x8_t xb[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xb[mt] = *reinterpret_cast<const bf16x8_t*>(sx + (mt * 2 + s) * 1024);
#pragma unroll
      for (int o = 0; o < OTW; ++o) {
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(sw + (o * 2 + s) * 1024);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[o][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xb[mt], acc[o][mt], 0, 0, 0);
      }
    }
    // chunk ci + 1 must have landed: what may stay in flight are the chunks after it that have been requested
    const uint32_t requested = min(ci + 3, nchunk - 1);     // youngest chunk requested so far
    ys_wait_vm(requested > ci + 1 ? (requested - (ci + 1)) * kPerChunk : 0);
    wg_barrier_lds();   // not __syncthreads(): that would also wait for the chunks that are meant to stay in flight
  }


  // ---- output: bf16 (+ residual), through a wave-private LDS patch so that the stores are row-contiguous.  The
  //      residual pieces of the wave's whole panel are requested first: one memory latency for all of them ----
  static_assert((size_t)WAVES * 32 * kPatchRow * 2 <= G::lds_bytes(), "the output patches alias the chunk buffers");
  uint16_t* patch = reinterpret_cast<uint16_t*>(lds_ys) + wave * (32 * kPatchRow);
  uint16_t* y_wg = y + (size_t)wg_row0 * ldy;
  const uint16_t* res_wg = residual ? residual + (size_t)wg_row0 * ldr : nullptr;
  u32x4_t rres[MT][OTW][2];
  if (residual) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int o = 0; o < OTW; ++o)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
          const uint32_t row = min(row0 + mt * 32 + rr, M - 1);
          rres[mt][o][h2] = *reinterpret_cast<const u32x4_t*>(res_wg + ((row - wg_row0) * ldr + (cg * OTW + o) * 32 + ch));
        }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int o = 0; o < OTW; ++o) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 pk;   // a Linear's output is bf16
        pk.x = pack_bf16x2(acc[o][mt][g * 4 + 0], acc[o][mt][g * 4 + 1]);
        pk.y = pack_bf16x2(acc[o][mt][g * 4 + 2], acc[o][mt][g * 4 + 3]);
        *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const uint32_t row = row0 + mt * 32 + rr;
        u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
        if (residual) {
          const u32x4_t rv = rres[mt][o][h2];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rv[e]), bf16_hi(t[e]) + bf16_hi(rv[e]));
        }
        if (row < M) *reinterpret_cast<u32x4_t*>(y_wg + ((row - wg_row0) * ldy + (cg * OTW + o) * 32 + ch)) = t;
      }
    }
}

// w [N][K] row-major -> fragment-major per chunk of 32 inner features:
//   wp[(((c * N/32 + ot) * 2 + s) * 64 + half * 32 + lq) * 8 + e] = w[ot * 32 + lq][c * 32 + s * 16 + half * 8 + e]
// One thread per 16-byte piece; the first N / 8 threads also clear the stand-in for a missing bias.
__global__ __launch_bounds__(256) void ys_w_prep_kernel(const uint16_t* __restrict__ w, uint16_t* __restrict__ wp,
                                                        uint16_t* __restrict__ zero_bias, uint32_t N, uint32_t K) {
  const uint32_t piece = blockIdx.x * blockDim.x + threadIdx.x;
  if (piece < N / 8) *reinterpret_cast<uint4*>(zero_bias + piece * 8) = make_uint4(0u, 0u, 0u, 0u);
  if (piece >= N * (K / 8)) return;
  const uint32_t lq = piece % 32, half = (piece / 32) % 2, s = (piece / 64) % 2;
  const uint32_t ot = (piece / 128) % (N / 32), c = piece / (128 * (N / 32));
  *reinterpret_cast<uint4*>(wp + (size_t)piece * 8) =
      *reinterpret_cast<const uint4*>(w + (size_t)(ot * 32 + lq) * K + c * 32 + s * 16 + half * 8);
}

template <int N>
static int launch_ys(const uint16_t* x, uint32_t ldx, const uint16_t* wp, const uint16_t* bias, const uint16_t* residual,
                     uint32_t ldr, uint16_t* y, uint32_t ldy, uint32_t M, uint32_t K, int device, hipStream_t s) {
  constexpr size_t lds = YsGeom<N>::lds_bytes();
  static_assert(lds <= 160 * 1024, "chunk buffers exceed the LDS of a compute unit");
  static bool attr_set[64] = {};
  auto kern = ystat_linear_kernel<N>;
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  hipLaunchKernelGGL(kern, dim3(cdiv_u32(M, 256)), dim3(64 * kYsWaves), lds, s, x, ldx, wp, bias, residual, ldr, y, ldy,
                     M, K);
  return F3D_OK;
}

// Returns F3D_OK when launched, F3D_ERR_UNSUPPORTED when the shape is not covered (the caller then uses the tiled
// GEMM), another code on failure.  Covered: no activation, N = 128 or 256, K a multiple of 32 above what the row-panel
// kernel takes, enough rows to fill the chip, row offsets inside a workgroup's panel that fit 32 bits.
int launch_ystat_linear(const uint16_t* x, uint32_t ldx, const uint16_t* w, const uint16_t* bias,
                        const uint16_t* residual, uint32_t ldr, uint16_t* y, uint32_t ldy, uint32_t M, uint32_t N,
                        uint32_t K, uint32_t act, int device, hipStream_t s) {
  if (act != F3D_ACT_NONE || !(N == 128 || N == 256) || K <= 512 || K % 32 != 0 || M < 256u * 128u)
    return F3D_ERR_UNSUPPORTED;
  if ((uint64_t)N * K * 2 >= (1ull << 32) || (uint64_t)256 * ldx * 2 >= (1ull << 31)) return F3D_ERR_UNSUPPORTED;
  const size_t wp_bytes = (size_t)N * K * 2;
  bool ready = false;
  char* ws = (char*)weight_area(device, wp_bytes + (size_t)N * 2, &ready, s);
  if (!ws) return F3D_ERR_RUNTIME;
  uint16_t* wp = (uint16_t*)ws;
  uint16_t* zero_bias = (uint16_t*)(ws + wp_bytes);
  if (!ready) hipLaunchKernelGGL(ys_w_prep_kernel, dim3(cdiv_u32(N * (K / 8), 256)), dim3(256), 0, s, w, wp, zero_bias, N, K);
  if (!bias) bias = zero_bias;
  if (N == 256) return launch_ys<256>(x, ldx, wp, bias, residual, ldr, y, ldy, M, K, device, s);
  return launch_ys<128>(x, ldx, wp, bias, residual, ldr, y, ldy, M, K, device, s);
}

}  // namespace f3d
