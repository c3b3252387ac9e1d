// Middle of the gated MLP's backward in one kernel for gfx950.  For a = silu(z1) * z2 with [z1 | z2] = h w1^T + b1 and
// y = a w2^T + b2 it forms, 32 hidden features at a time,
//     z1, z2 = h w1[value rows]^T + b1, h w1[gate rows]^T + b1      (the fc1 output is recomputed, never stored)
//     da     = dy w2[:, those features]                              (never stored either)
//     a      = silu(z1) z2,  dz1 = da z2 s (1 + z1 (1 - s)),  dz2 = da z1 s,  s = sigmoid(z1)
// and writes a [M, H] and dz [M, 2 H], which the two weight gradients and the input gradient read.  The reference takes
// this step from TransformerEngine's LayerNormMLP autograd (flash3dxfmr/layers/elem_wise.py:22-26).
//
// A workgroup of eight waves owns 256 rows, 32 per wave.  A wave keeps its rows of h AND of dy in registers (matrix-core
// B-operand layout, 2 x K / 4 registers) for the whole kernel; per chunk the three weight blocks (32 value rows of w1, their
// 32 gate rows, 32 rows of w2^T: all [32][K]) stream L2 -> LDS directly (global_load ... lds) into one of two buffers,
// rows XOR-swizzled by 16-byte pieces so that the 128-bit operand reads of 16 rows fall into 16 different bank groups.
// The products are formed transposed (weight rows as the A operand), so a lane holds, for its row, 4 x 4 consecutive
// hidden features of each of the three tiles in the same accumulator slots: the gate arithmetic is lane-local.  The three
// result tiles go through a wave-private LDS patch so that the global stores are row-contiguous 16-byte pieces.
//
// Against fc1 recomputation + dy w2 + the one-pass gate backward as three kernels this saves writing and re-reading
// z (2 H per row) and da (H per row).
#include "xstat_common.h"

namespace f3d {
namespace {

constexpr int kGbWaves = 8;

template <int K>
struct GbGeom {
  static constexpr int ROWB = K * 2;                  // bytes per weight row
  static constexpr int CPR = K / 8;                   // 16-byte pieces per weight row (4, 8, 16 or 32)
  static constexpr int RPI = 1024 / ROWB;             // weight rows one direct load fills
  static constexpr int CHUNK = 96 * ROWB;             // value + gate + w2^T rows of 32 hidden features
  static constexpr int N_DMA = CHUNK / 1024;
  static constexpr int KP = K < 128 ? K : 128;        // columns per transposition pass of the prologue
  static constexpr int PROW = KP + 8;
  static constexpr int SLOT = CHUNK + 1024;           // a chunk buffer and, behind it, the chunk's 64 bias values as dwords
  static constexpr size_t loop_bytes() { return (size_t)2 * SLOT + (size_t)kGbWaves * 32 * kPatchRow * 2; }
  static constexpr size_t prologue_bytes() { return (size_t)kGbWaves * 32 * PROW * 2; }
  static constexpr size_t lds_bytes() { return loop_bytes() > prologue_bytes() ? loop_bytes() : prologue_bytes(); }
  static constexpr int MY_DMA_MAX = (N_DMA + kGbWaves - 1) / kGbWaves;
  // 16 consecutive rows read at one piece index must fall into 16 different 16-byte slots of the 256 bank bytes: rows
  // that share their offset modulo 256 get different swizzle values
  static constexpr int RP = CPR >= 16 ? 1 : 16 / CPR;     // rows sharing one swizzle value
  static constexpr int SWZ_MASK = (CPR < 16 ? CPR : 16) - 1;
  __host__ __device__ static constexpr uint32_t swz(uint32_t row) { return (row / RP) & SWZ_MASK; }
  static_assert(32 % RPI == 0 && 1024 % ROWB == 0, "a direct load fills whole rows of one weight block");
};

// 32 rows [row0, row0 + 32) of a row-major [M, K] tensor -> the wave's registers in B-operand layout: f[ks] of lane
// (lq, half) = columns 16 ks + 8 half .. + 7 of row row0 + lq (rows past M read row M - 1).  Coalesced 16-byte loads,
// turned through a wave-private patch.
template <int K>
__device__ __forceinline__ void load_rows_b(const uint16_t* __restrict__ src, uint32_t ld, uint32_t row0, uint32_t M,
                                            uint16_t* patch, uint32_t lane, bf16x8_t (&f)[K / 16]) {
  using G = GbGeom<K>;
  constexpr int KP = G::KP, PROW = G::PROW, PCPR = KP / 8, XLOADS = (32 * PCPR) / kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  u32x4_t v[K / KP][XLOADS];
#pragma unroll
  for (int kp = 0; kp < K / KP; ++kp)
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const uint32_t id = lane + i * kWave, rr = id / PCPR, kc = (id % PCPR) * 8;
      const uint32_t r = min(row0 + rr, M - 1);
      v[kp][i] = *reinterpret_cast<const u32x4_t*>(src + (size_t)r * ld + kp * KP + kc);
    }
#pragma unroll
  for (int kp = 0; kp < K / KP; ++kp) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const uint32_t id = lane + i * kWave, rr = id / PCPR, kc = (id % PCPR) * 8;
      *reinterpret_cast<u32x4_t*>(patch + rr * PROW + kc) = v[kp][i];
    }
#pragma unroll
    for (int ks = 0; ks < KP / 16; ++ks)
      f[kp * (KP / 16) + ks] = *reinterpret_cast<const bf16x8_t*>(patch + lq * PROW + ks * 16 + half * 8);
  }
}

// h [M, K] (LayerNorm output), dy [M, K], w1 [2 H, K] (value rows, then gate rows), b1 [2 H] or null, w2t [H, K] (w2
// transposed); a [M, H], dz [M, 2 H].  H a multiple of 32.
template <int K>
__global__ __launch_bounds__(64 * kGbWaves) __attribute__((amdgpu_waves_per_eu(2))) void mlp_gate_bwd_kernel(
    const uint16_t* __restrict__ h, uint32_t ldh, const uint16_t* __restrict__ dy, uint32_t lddy,
    const uint16_t* __restrict__ w1, const uint16_t* __restrict__ b1, const uint16_t* __restrict__ w2t,
    uint16_t* __restrict__ dz, uint32_t lddz, uint16_t* __restrict__ a, uint32_t lda, uint32_t M, uint32_t H) {
  using G = GbGeom<K>;
  constexpr int KS = K / 16, ROWB = G::ROWB, WAVES = kGbWaves, ROWS_WG = 32 * WAVES;
  extern __shared__ __attribute__((aligned(1024))) char lds_gb[];
  char* wbuf = lds_gb;                                                       // two chunk buffers (+ bias slots)
  uint16_t* patch = reinterpret_cast<uint16_t*>(lds_gb + 2 * G::SLOT);       // epilogue patches, one per wave

  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t wg_row0 = blockIdx.x * ROWS_WG, row0 = wg_row0 + wave * 32;
  const bool wg_full = wg_row0 + ROWS_WG <= M;   // every store of the workgroup is issued: the waits can count them
  patch += wave * (32 * kPatchRow);

  // ---- the wave's rows of h and dy -> registers ----
  bf16x8_t hf[KS], df[KS];
  {
    uint16_t* pp = reinterpret_cast<uint16_t*>(lds_gb) + wave * (32 * G::PROW);
    load_rows_b<K>(h, ldh, row0, M, pp, lane, hf);
    load_rows_b<K>(dy, lddy, row0, M, pp, lane, df);   // same patch: a wave's LDS operations complete in order
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();   // the transposition patches are dead; the space now holds weight chunks

  // ---- weight streaming: direct load q of a chunk fills LDS bytes [1024 q, 1024 q + 1024) = chunk rows
  //      [RPI q, RPI q + RPI); wave v issues q = v, v + WAVES, ... ----
  const uint32_t nchunk = H / 32;
  auto dma_chunk = [&](uint32_t c, uint32_t slot) {
#pragma unroll
    for (int i = 0; i < G::MY_DMA_MAX; ++i) {
      const uint32_t q = wave + i * WAVES;
      if (q >= (uint32_t)G::N_DMA) break;                       // wave-uniform
      const uint32_t lr = q * G::RPI + lane / G::CPR;           // row of the chunk: 0-31 value, 32-63 gate, 64-95 w2^T
      const uint32_t piece = (lane % G::CPR) ^ G::swz(lr);      // the piece that belongs at this lane's LDS position
      const uint32_t blk = __builtin_amdgcn_readfirstlane(q * G::RPI / 32u);
      const uint16_t* base = blk == 2 ? w2t : w1;
      const uint32_t grow = (blk == 1 ? H : 0u) + c * 32u + (lr & 31u);
      xs_lds_dma16(base, grow * (uint32_t)ROWB + piece * 16u, wbuf + slot * G::SLOT + q * 1024);
    }
    // the chunk's 32 value and 32 gate biases behind the weights, one dword each (the bf16 bits, zero-extended): no
    // load of the loop is one the compiler would wait for together with the stores in flight
    if (wave == 0 && b1) xs_lds_dma2(b1, ((lane < 32u ? 0u : H - 32u) + c * 32u + lane) * 2u, wbuf + slot * G::SLOT + G::CHUNK);
  };
  // A operand of tile block t (0 value, 1 gate, 2 w2^T), k-step ks: row lq of the block, 16-byte piece 2 ks + half
  const uint32_t a_row = lq * ROWB, a_swz = G::swz(lq);   // block offsets (32 rows) leave the swizzle value unchanged
  auto a_frag = [&](const char* buf, int t, int ks) -> bf16x8_t {
    return *reinterpret_cast<const bf16x8_t*>(buf + t * 32 * ROWB + a_row + (((uint32_t)(2 * ks) + half) ^ a_swz) * 16u);
  };

  dma_chunk(0, 0);
  for (uint32_t c = 0; c < nchunk; ++c) {
    const uint32_t slot = c & 1u;
    // chunk c has landed when at most the stores of the previous epilogue (6 per wave, issued after its requests, however
    // many of those the wave has) are outstanding; where some stores may be skipped (rows past M) everything is waited for
    if (wg_full && c > 0) xs_wait_vm(6); else __builtin_amdgcn_s_waitcnt(0x0F70);
    wg_barrier_lds();   // every wave's part of chunk c is in LDS; every wave is done reading chunk c - 1
    if (c + 1 < nchunk) dma_chunk(c + 1, slot ^ 1u);
    const char* buf = wbuf + slot * G::SLOT;
    // operands of k-step ks + 1 are requested before the products of k-step ks are issued
    f32x16_t da;
#pragma unroll
    for (int e = 0; e < 16; ++e) da[e] = 0.f;
    {
      bf16x8_t fr[2];
      fr[0] = a_frag(buf, 2, 0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) fr[(ks + 1) & 1] = a_frag(buf, 2, ks + 1);
        da = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ks & 1], df[ks], da, 0, 0, 0);
      }
    }
    // the fc1 accumulators start from the bias: slot 4 g + r of a lane is hidden feature 8 g + 4 half + r
    f32x16_t z1, z2;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x4_t bv = {0u, 0u, 0u, 0u}, bg = {0u, 0u, 0u, 0u};
      if (b1) {
        bv = *reinterpret_cast<const u32x4_t*>(buf + G::CHUNK + (g * 8 + half * 4) * 4);
        bg = *reinterpret_cast<const u32x4_t*>(buf + G::CHUNK + (32 + g * 8 + half * 4) * 4);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        z1[g * 4 + r] = __builtin_bit_cast(float, bv[r] << 16);
        z2[g * 4 + r] = __builtin_bit_cast(float, bg[r] << 16);
      }
    }
    {
      bf16x8_t fr[2][2];
      fr[0][0] = a_frag(buf, 0, 0);
      fr[0][1] = a_frag(buf, 1, 0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) {
          fr[(ks + 1) & 1][0] = a_frag(buf, 0, ks + 1);
          fr[(ks + 1) & 1][1] = a_frag(buf, 1, ks + 1);
        }
        z1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ks & 1][0], hf[ks], z1, 0, 0, 0);
        z2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[ks & 1][1], hf[ks], z2, 0, 0, 0);
      }
    }
    // ---- gate arithmetic, lane-local and in place: z1 <- a, z2 <- dz1, da <- dz2
    //      (u = z1 s = silu(z1); a = u z2; dz1 = da z2 (s + u (1 - s)); dz2 = da u) ----
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z1[e]));
      const float u = z1[e] * sg, q = z2[e], d = da[e];
      z1[e] = u * q;
      z2[e] = d * q * __builtin_fmaf(u, 1.0f - sg, sg);
      da[e] = d * u;
    }
    // ---- the three tiles -> patch -> row-contiguous stores ----
    auto flush = [&](const f32x16_t& v, uint16_t* out, uint32_t ld, uint32_t col) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 pk;
        pk.x = pack_bf16x2(v[g * 4 + 0], v[g * 4 + 1]);
        pk.y = pack_bf16x2(v[g * 4 + 2], v[g * 4 + 3]);
        *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
        if (row0 + rr < M) *reinterpret_cast<u32x4_t*>(out + (size_t)(row0 + rr) * ld + col + ch) = t;
      }
    };
    flush(z1, a, lda, c * 32);
    flush(z2, dz, lddz, c * 32);
    flush(da, dz, lddz, H + c * 32);
  }
}

template <int K>
int launch_gate_bwd(const uint16_t* h, uint32_t ldh, const uint16_t* dy, uint32_t lddy, const uint16_t* w1,
                    const uint16_t* b1, const uint16_t* w2t, uint16_t* dz, uint32_t lddz, uint16_t* a, uint32_t lda,
                    uint32_t M, uint32_t H, int device, hipStream_t s) {
  constexpr size_t lds = GbGeom<K>::lds_bytes();
  static_assert(lds <= 160 * 1024, "LDS budget");
  static bool attr_set[64] = {};
  auto kern = mlp_gate_bwd_kernel<K>;
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  hipLaunchKernelGGL(kern, dim3(cdiv_u32(M, 32 * kGbWaves)), dim3(64 * kGbWaves), lds, s, h, ldh, dy, lddy, w1, b1, w2t,
                     dz, lddz, a, lda, M, H);
  return F3D_OK;
}

}  // namespace
}  // namespace f3d

extern "C" int f3d_mlp_gate_bwd_bf16(const f3d_bf16_t* h, uint32_t ldh, const f3d_bf16_t* dy, uint32_t lddy,
                                     const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2t, f3d_bf16_t* dz,
                                     uint32_t lddz, f3d_bf16_t* a, uint32_t lda, uint32_t m, uint32_t c,
                                     uint32_t hidden, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(h && dy && w1 && w2t && dz && a, "null tensor pointer");
  if (!(c == 32 || c == 64 || c == 128 || c == 256) || hidden == 0 || hidden % 32 != 0 ||
      (uint64_t)hidden * c * 4 >= (1ull << 32)) {
    set_error("No kernel found for the fused gate backward at width %u, hidden %u (widths 32, 64, 128 and 256, hidden a "
              "multiple of 32)", c, hidden);
    return F3D_ERR_UNSUPPORTED;
  }
  F3D_CHECK_ARG(ldh >= c && ldh % 8 == 0 && lddy >= c && lddy % 8 == 0 && lddz >= 2 * hidden && lddz % 8 == 0 &&
                    lda >= hidden && lda % 8 == 0,
                "row strides must be multiples of 8 and cover a row");
  F3D_CHECK_ARG((((uintptr_t)h | (uintptr_t)dy | (uintptr_t)w1 | (uintptr_t)b1 | (uintptr_t)w2t | (uintptr_t)dz |
                  (uintptr_t)a) & 15u) == 0,
                "h / dy / w1 / b1 / w2t / dz / a must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  int rc;
  switch (c) {
    case 32: rc = launch_gate_bwd<32>(h, ldh, dy, lddy, w1, b1, w2t, dz, lddz, a, lda, m, hidden, device, s); break;
    case 64: rc = launch_gate_bwd<64>(h, ldh, dy, lddy, w1, b1, w2t, dz, lddz, a, lda, m, hidden, device, s); break;
    case 128: rc = launch_gate_bwd<128>(h, ldh, dy, lddy, w1, b1, w2t, dz, lddz, a, lda, m, hidden, device, s); break;
    default: rc = launch_gate_bwd<256>(h, ldh, dy, lddy, w1, b1, w2t, dz, lddz, a, lda, m, hidden, device, s); break;
  }
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}
