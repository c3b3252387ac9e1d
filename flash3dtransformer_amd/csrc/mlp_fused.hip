// Whole gated MLP of a transformer block in one kernel for gfx950:
//     y = (silu(LN(x) w1_valueT + b1_value) * (LN(x) w1_gateT + b1_gate)) w2T + b2 (+ residual)
// Stands where the reference runs te.LayerNormMLP(activation = "swiglu") followed by the residual add
// (flash3dxfmr/layers/elem_wise.py:22-26, stage.py:94-97).
//
// A workgroup of eight waves owns 256 rows, 32 per wave.  A wave keeps its rows of x in registers (matrix-core operand
// layout) for the whole kernel and walks the hidden features 32 at a time, in two halves of 16: the fc1 tile of a half
// has the 16 value features in its rows 0-15 and their 16 gate features in rows 16-31 (the product is formed
// transposed, rows of w1 as the A operand), which puts a value and its gate into the same lane (accumulator slots i
// and i + 8); the 8 gated products per lane, rounded to bf16, already ARE the B operand of the fc2 k-step of that
// half, which updates ALL output columns at once.  The hidden activations never leave the registers; the matching
// order of the hidden index inside a k-step is baked into the prepared copy of w2.
//
// Registers per wave at C = 256: x 64, the fc2 accumulators (32 rows x 256 outputs) 128, one fc1 tile 16, fragments in
// flight: under 256, so a SIMD holds TWO waves and one wave's matrix products run while the other forms its gate,
// issues its requests or waits.  Every weight fragment read from LDS feeds one product (1 KB per product: half of what
// the LDS of gfx950 delivers at the matrix core's full rate, measured 497 B/ns per CU with eight waves reading).
// The two waves of a SIMD drift apart by themselves (the one that loses the matrix core at the start of an interval
// stays behind by about a stage), which interleaves one's products with the other's gate arithmetic.  (Forcing them
// half an interval apart, as the row-panel linear kernel does, measured 12 % slower: the late waves then carry an fc1
// tile across the barrier and the loop no longer fits the registers.)
//
// Per chunk the weights stream L2 -> LDS directly (global_load ... lds), two buffers each: 64 rows of the
// LayerNorm-folded w1 (row-major, 16-byte pieces XOR-swizzled) and the chunk's slice of w2, which the preparation
// kernel stores fragment-major (the 64 lanes' 16-byte pieces of one fragment are consecutive), so its LDS reads are
// linear.  LayerNorm as in the row-panel linear kernel: the rows are normalised in registers (bf16((x - mean) * rstd)),
// w' = w * gamma, and the fc1 accumulators start from b' = b1 + w1 beta (fp32, fetched per chunk next to the weights).
//
// 6 * M * C * H flops (fc1 value + gate, fc2) against HBM traffic of x, residual and y only: the hidden activations
// (M x H bf16, 1 GB at 482 k rows x 1024) are never allocated.  Measured on MI355X against the LayerNorm+fc1+gate
// kernel followed by the fc2+residual kernel: 482,304 rows, C = 256, H = 1024: 0.75 ms against 0.94 ms; 250 k rows,
// C = 128, H = 512: 0.138 ms against 0.224 ms.  (A first form with 64 rows per wave and one wave per SIMD, whose
// register file the x rows (128) and the fc2 accumulators (256) fill, took 0.87 ms: with a single wave per SIMD
// nothing overlaps the issue of the roughly 1000 instructions that go with the 100 products of a chunk.)
//
// With the block's out-projection in front (PROJ kernels, f3d_proj_ln_mlp_swiglu_bf16; flash3dxfmr/layers/stage.py:92-102:
// proj, residual add, MLP, residual add): x1 = a wpT + bp + x is formed in the fc2 accumulators before the LayerNorm
// (the block input enters through products with an identity) and never reaches memory; the kernel then returns
// x1 + MLP(LayerNorm(x1)).  482,304 rows, C = 256: 0.78 ms against 0.155 + 0.70 ms for the projection kernel followed
// by this kernel without it.
#include <algorithm>

#include "xstat_common.h"

namespace f3d {

// f(std::integral_constant<uint32_t, 0>) ... f(std::integral_constant<uint32_t, N - 1>): a loop whose counter is a
// constant expression inside the body (statically indexed register arrays)
template <uint32_t N, uint32_t I = 0, class F>
__device__ __forceinline__ void mlp_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<uint32_t, I>{});
    mlp_static_for<N, I + 1>(f);
  }
}

constexpr int kMlpWaves = 8, kMlpBufs = 2;   // chunk c + 1 is requested when chunk c starts
constexpr int kMlpFragsAhead = 2;            // LDS fragment reads in flight ahead of their products

template <int K>
struct MlpGeom {
  using G = XsGeom<K>;
  static constexpr int OT = K / 32;                         // output column tiles of fc2
  static constexpr int CH1 = G::CHUNK_BYTES;                // w1 chunk: 64 rows
  static constexpr int CH2 = K * 32 * 2;                    // w2 chunk: K outputs x 32 hidden
  static constexpr int N_DMA2 = CH2 / 1024;
  static constexpr int NPC = K / kXsChunk;                  // 64-row chunks of the out-projection weight
  static constexpr size_t loop_bytes() { return (size_t)kMlpBufs * (CH1 + 1024 + CH2); }
  static constexpr size_t row_patch_bytes() { return (size_t)kMlpWaves * 32 * kPatchRow * 2; }
  // weight buffers and the b' slots of the w1 buffers; at least the prologue's transposition patches; with the
  // out-projection in front, the wave-private patches its result is re-laid through come after the weight buffers
  static constexpr size_t lds_bytes(bool proj = false) {
    const size_t loop = loop_bytes();
    const size_t patches = (size_t)kMlpWaves * 32 * (G::KP + 8) * 2;
    return proj ? loop + row_patch_bytes() : (loop > patches ? loop : patches);
  }
};

// The out-projection in front of the MLP (PROJ kernels): a [M][K] are the attention output rows, w [K][K] / b [K] the
// projection's weight and bias; the kernel's x is then the block input that the projection's result is added to.
// EMBED kernels: the block input is not read but formed: it is the coordinate embedding of the rows' points (coord fp16
// [M][3]; etab bf16 [K][8] = (wx, wy, wz, b, 0, 0, 0, 0) per channel), one product per 32 channels into the accumulators.
struct MlpProj {
  const uint16_t* a;
  uint32_t lda;
  const uint16_t* w;
  const uint16_t* b;
  const uint16_t* coord;
  const uint16_t* etab;
};

// the rows' (x, y, z, 1) as the B operand of the embedding product: lane (lq, half = 0) carries row lq's four values
__device__ __forceinline__ bf16x8_t embed_rows_operand(const uint16_t* coord, uint32_t row, uint32_t half) {
  u32x4_t cb = {0u, 0u, 0u, 0u};
  if (half == 0) {
    const uint16_t* cp = coord + (size_t)row * 3;
    cb[0] = pack_bf16x2(half_bits_to_float(cp[0]), half_bits_to_float(cp[1]));
    cb[1] = pack_bf16x2(half_bits_to_float(cp[2]), 1.0f);
  }
  return __builtin_bit_cast(bf16x8_t, cb);
}
// the (wx, wy, wz, b) of channels 32 tile + lq as the A operand
__device__ __forceinline__ bf16x8_t embed_channels_operand(const uint16_t* etab, uint32_t tile, uint32_t lq, uint32_t half) {
  u32x4_t ea = {0u, 0u, 0u, 0u};
  if (half == 0) ea = *reinterpret_cast<const u32x4_t*>(etab + (size_t)(tile * 32 + lq) * 8);
  return __builtin_bit_cast(bf16x8_t, ea);
}

// w1p: LayerNorm-folded fc1 weight [2 H][K] (value rows then gate rows), b32: b' = b1 + w1 beta as fp32 [2 H] (mlp_prep_kernel);
// w2p: fc2 weight, fragment-major per chunk (mlp_prep_kernel); bias2 [K] (zeros when the layer has none);
// H: hidden width, multiple of 32.
// PROJ: x1 = bf16(a wpT + bp + x) is formed first (the block's out-projection with its residual, held in registers
// only), and the kernel returns bf16(x1 + MLP(x1)): `residual` must be null, the fc2 accumulators start from x1 + b2.
template <int K, bool PROJ, bool EMBED = false>
__global__ __launch_bounds__(64 * kMlpWaves) __attribute__((amdgpu_waves_per_eu(2, 2))) void ln_mlp_swiglu_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, float eps, const uint16_t* __restrict__ w1p,
    const float* __restrict__ b32, const uint16_t* __restrict__ w2p, const uint16_t* __restrict__ bias2,
    const uint16_t* __restrict__ residual, uint32_t ldr, uint16_t* __restrict__ y, uint32_t ldy, uint32_t M,
    uint32_t H, uint32_t main_wgs, uint32_t tail_rows, MlpProj pj) {
  using G = XsGeom<K>;
  using MG = MlpGeom<K>;
  constexpr int KS = K / 16, ROWB = G::ROWB, WAVES = kMlpWaves, NB1 = kMlpBufs, NB2 = kMlpBufs, OT = MG::OT;
  constexpr int ROWS_WG = 32 * WAVES;
  static_assert(G::RP == 1 && G::SWZ_MASK == 15, "the half-tile addressing assumes K = 128 or 256");
  extern __shared__ __attribute__((aligned(1024))) char lds_mlp[];
  char* w1buf = lds_mlp;
  char* w2buf = lds_mlp + (size_t)NB1 * MG::CH1;
  char* s_side = w2buf + (size_t)NB2 * MG::CH2;   // per w1 slot: b' of the chunk's 64 fc1 features (fp32; 1 KB apart)

  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  // Workgroups [0, main_wgs) own 256 rows each; the workgroups after them share what is left in panels of tail_rows
  // rows (a multiple of 32, at most 256), of which only the first tail_rows / 32 waves have rows: the last, partly
  // filled turn of the chip then runs with fewer waves per SIMD and ends sooner.
  const bool in_tail = blockIdx.x >= main_wgs;
  const uint32_t wg_row0 = in_tail ? main_wgs * ROWS_WG + (blockIdx.x - main_wgs) * tail_rows : blockIdx.x * ROWS_WG;
  const uint32_t row0 = wg_row0 + wave * 32;
  const bool has_rows = (wave * 32 < (in_tail ? tail_rows : (uint32_t)ROWS_WG)) && row0 < M;

  // ---- weight streaming: per chunk 64 rows of w1 (N_DMA kilobytes), K x 32 of w2 (N_DMA2), the 64 values of b' (wave 0) ----
  const uint32_t nchunk = H / 32;
  static_assert(G::N_DMA % WAVES == 0 && MG::N_DMA2 % WAVES == 0, "direct loads split evenly over the waves");
  constexpr uint32_t kDma1 = G::N_DMA / WAVES, kDma2 = MG::N_DMA2 / WAVES;
  // One direct load moves 64 pieces = RPD w1 rows. The lane's byte offset inside such a group (its row of the group,
  // its piece of the row under the row's swizzle) is the same for every group the wave loads, because the groups of
  // one wave lie a multiple of 16 rows apart and the swizzle has period 16; everything else about an address is
  // uniform and goes into the scalar base. (Addresses recomputed per load in vector registers cost the issuing wave
  // about 60 cycles of dependent arithmetic each, with the matrix pipeline idle.)
  constexpr uint32_t RPD = 64 / G::CPR;
  static_assert((WAVES * RPD) % 16 == 0 && G::RP == 1 && 32 % RPD == 0, "one lane offset serves all groups of a wave");
  const uint32_t w1_lane_off = ((lane / G::CPR) * K + (((lane % G::CPR) ^ G::swz(wave * RPD + lane / G::CPR)) * 8u)) * 2u;
  const uint32_t tab_lane_off = (lane < 32 ? lane : H + lane - 32) * 4u;
  auto dma_chunk = [&](uint32_t c) __attribute__((always_inline)) {
    const char* b1 = w1buf + (c % NB1) * MG::CH1;
#pragma unroll
    for (uint32_t i = 0; i < kDma1; ++i) {
      const uint32_t qi = wave + i * WAVES, r0 = qi * RPD;                       // first chunk row of the group
      const uint32_t wrow0 = r0 < 32 ? c * 32u + r0 : H + c * 32u + (r0 - 32u);   // value rows, then gate rows
      xs_lds_dma16(reinterpret_cast<const char*>(w1p) + (size_t)wrow0 * (K * 2), w1_lane_off, b1 + qi * 1024);
    }
    const char* b2 = w2buf + (c % NB2) * MG::CH2;
#pragma unroll
    for (uint32_t i = 0; i < kDma2; ++i)
      xs_lds_dma16(reinterpret_cast<const char*>(w2p) + (size_t)c * MG::CH2 + (wave + i * WAVES) * 1024u, lane * 16u,
                   b2 + (wave + i * WAVES) * 1024);
    if (wave == 0) xs_lds_dma4(reinterpret_cast<const char*>(b32) + (size_t)c * 128, tab_lane_off, s_side + (c % NB1) * 1024);
  };
  // chunk c of the out-projection weight (rows 64 c .. 64 c + 63 of w, row-major) into w1 buffer c % NB1, laid out
  // like a w1 chunk
  auto dma_proj = [&](uint32_t c) __attribute__((always_inline)) {
    const char* b1 = w1buf + (c % NB1) * MG::CH1;
#pragma unroll
    for (uint32_t i = 0; i < kDma1; ++i) {
      const uint32_t qi = wave + i * WAVES;
      xs_lds_dma16(reinterpret_cast<const char*>(pj.w) + (size_t)(c * kXsChunk + qi * RPD) * (K * 2), w1_lane_off, b1 + qi * 1024);
    }
  };

  bf16x8_t xf[KS];
  f32x16_t acc2[OT];
  // acc2[ot][g*4+r] <-> output column ot*32 + g*8 + half*4 + r of row lq; they start from a bias
  auto acc2_from_bias = [&](const uint16_t* bias) __attribute__((always_inline)) {
#pragma unroll
    for (int ot = 0; ot < OT; ++ot)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint2 bb = *reinterpret_cast<const uint2*>(bias + ot * 32 + g * 8 + half * 4);
        acc2[ot][g * 4 + 0] = bf16_lo(bb.x); acc2[ot][g * 4 + 1] = bf16_hi(bb.x);
        acc2[ot][g * 4 + 2] = bf16_lo(bb.y); acc2[ot][g * 4 + 3] = bf16_hi(bb.y);
      }
  };
  if constexpr (PROJ) {
    // ---- out-projection first: the projection's first weight chunk is requested before anything else; the wave's 32
    //      rows of the attention output go straight into operand registers (16 bytes of a row per lane and k-step) ----
    dma_proj(0);
    {
      const uint32_t r = min(row0 + lq, M - 1);
      const uint16_t* ap = pj.a + (size_t)r * pj.lda + half * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) xf[ks] = *reinterpret_cast<const bf16x8_t*>(ap + ks * 16);
    }
    acc2_from_bias(pj.b);
    // a wpT: output tile 2 c + t (32 columns) from rows 32 t .. 32 t + 31 of chunk c; the MLP's first chunk is
    // requested under the projection's last one.  The block input is added ON THE MATRIX CORE: its 32 columns of a
    // tile, loaded straight into operand layout while the tile's products run, times a 32 x 32 identity (two
    // k-steps; exact: one bf16 value times one, summed in fp32) land in the same accumulators, so the residual needs
    // no re-laying and no vector arithmetic.
    const uint32_t poff = lq * ROWB + (((half ^ G::swz(lq)) & (uint32_t)(G::CPR - 1)) << 4);
    // identity fragments: k-step j of a tile holds its columns 16 j .. 16 j + 15; lane (lq, half) carries elements
    // 8 half .. 8 half + 7 of output column lq's row of the identity
    bf16x8_t idf[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) idf[j][e] = (lq == (uint32_t)(16 * j + e) + 8u * half) ? (__bf16)1.0f : (__bf16)0.0f;
    const uint16_t* xrow = EMBED ? nullptr : x + (size_t)min(row0 + lq, M - 1) * ldx + half * 8;      // rows past M read row M - 1
    // the block input's columns of chunk c's two tiles, requested one chunk ahead (chunk 0's before the first wait)
    bf16x8_t xt[2][2][2];
    auto load_xt = [&](uint32_t c) __attribute__((always_inline)) {
      if constexpr (!EMBED) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 2; ++j) xt[c & 1u][t][j] = *reinterpret_cast<const bf16x8_t*>(xrow + (2 * c + t) * 32 + j * 16);
      }
    };
    // EMBED: the block input is the embedding of the rows' coordinates: one product of a tile's channel parameters
    // with the rows' (x, y, z, 1) per tile instead of the two identity products (fp32, not rounded to bf16 in between)
    bf16x8_t cbe;
    if constexpr (EMBED) cbe = embed_rows_operand(pj.coord, min(row0 + lq, M - 1), half);
    load_xt(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    mlp_static_for<MG::NPC>([&](auto c_c) {
      constexpr uint32_t c = decltype(c_c)::value;
      if constexpr (c + 1 < (uint32_t)MG::NPC) dma_proj(c + 1);
      else dma_chunk(0);
      if (has_rows) {
        if constexpr (c + 1 < (uint32_t)MG::NPC) load_xt(c + 1);
        bf16x8_t eat[2];
        if constexpr (EMBED) {
#pragma unroll
          for (int t = 0; t < 2; ++t) eat[t] = embed_channels_operand(pj.etab, 2 * c + t, lq, half);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const char* sw = w1buf + (c % NB1) * MG::CH1 + t * 32 * ROWB;
          constexpr int kAhead = kMlpFragsAhead;
          bf16x8_t wf[KS];
#pragma unroll
          for (int ks = 0; ks < kAhead; ++ks) wf[ks] = *reinterpret_cast<const bf16x8_t*>(sw + (poff ^ (uint32_t)(ks * 32)));
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            if (ks + kAhead < KS) wf[ks + kAhead] = *reinterpret_cast<const bf16x8_t*>(sw + (poff ^ (uint32_t)((ks + kAhead) * 32)));
            acc2[2 * c + t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ks], xf[ks], acc2[2 * c + t], 0, 0, 0);
          }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          if constexpr (EMBED) {
            acc2[2 * c + t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(eat[t], cbe, acc2[2 * c + t], 0, 0, 0);
          } else {
#pragma unroll
            for (int j = 0; j < 2; ++j)
              acc2[2 * c + t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(idf[j], xt[c & 1u][t][j], acc2[2 * c + t], 0, 0, 0);
          }
        }
      }
      // the next chunk has landed; the block input's pieces requested above (4 loads, younger than the chunk's direct
      // loads) may stay in flight
      if (!EMBED && c + 1 < (uint32_t)MG::NPC && has_rows) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      wg_barrier_lds();
    });
    // x1 = bf16(projection + bias + x), 32 columns at a time: written to the wave's patch in the accumulator layout
    // and read back in operand layout (the k-steps 2 ot, 2 ot + 1 of the LayerNorm / fc1 panel), without a wait between
    // tiles (LDS serves a wave in order); the accumulators go on as x1 + b2, what the fc2 products add to
    if (has_rows) {
      uint16_t* pb = reinterpret_cast<uint16_t*>(lds_mlp + MG::loop_bytes()) + wave * (32 * kPatchRow);
#pragma unroll
      for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint2 bb = *reinterpret_cast<const uint2*>(bias2 + ot * 32 + g * 8 + half * 4);
          uint2 x1;
          x1.x = pack_bf16x2(acc2[ot][g * 4 + 0], acc2[ot][g * 4 + 1]);
          x1.y = pack_bf16x2(acc2[ot][g * 4 + 2], acc2[ot][g * 4 + 3]);
          *reinterpret_cast<uint2*>(pb + lq * kPatchRow + g * 8 + half * 4) = x1;
          acc2[ot][g * 4 + 0] = bf16_lo(x1.x) + bf16_lo(bb.x); acc2[ot][g * 4 + 1] = bf16_hi(x1.x) + bf16_hi(bb.x);
          acc2[ot][g * 4 + 2] = bf16_lo(x1.y) + bf16_lo(bb.y); acc2[ot][g * 4 + 3] = bf16_hi(x1.y) + bf16_hi(bb.y);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
          xf[2 * ot + j] = *reinterpret_cast<const bf16x8_t*>(pb + lq * kPatchRow + j * 16 + half * 8);
      }
    }
  } else {
    // ---- this wave's 32 rows of x -> registers (B-operand layout), through a wave-private transposition patch ----
    {
      constexpr int KP = G::KP, PROW = KP + 8, PCPR = KP / 8;
      static_assert((size_t)WAVES * 32 * PROW * 2 <= MG::lds_bytes(), "the transposition patches alias everything else");
      uint16_t* patch = reinterpret_cast<uint16_t*>(lds_mlp) + wave * (32 * PROW);
      constexpr int XLOADS = (32 * PCPR) / kWave;
      u32x4_t v[K / KP][XLOADS];
  #pragma unroll
      for (int kp = 0; kp < K / KP; ++kp)
  #pragma unroll
        for (int i = 0; i < XLOADS; ++i) {
          const uint32_t id = lane + i * kWave;
          const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
          const uint32_t r = min(row0 + rr, M - 1);
          v[kp][i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)r * ldx + kp * KP + kc);
        }
  #pragma unroll
      for (int kp = 0; kp < K / KP; ++kp) {
  #pragma unroll
        for (int i = 0; i < XLOADS; ++i) {
          const uint32_t id = lane + i * kWave;
          const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
          *reinterpret_cast<u32x4_t*>(patch + rr * PROW + kc) = v[kp][i];
        }
  #pragma unroll
        for (int ks = 0; ks < KP / 16; ++ks)
          xf[kp * (KP / 16) + ks] = *reinterpret_cast<const bf16x8_t*>(patch + lq * PROW + ks * 16 + half * 8);
      }
    }
  }
  // LayerNorm in place (statistics shifted by the row's first element; x <- bf16((x - mean) * rstd), one fragment at a
  // time and opaque, so that the floats of the first sweep are not held for the second)
  {
    const float x0 = __shfl((float)xf[0][0], lq, kWave);
    float s = 0.f, q = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = (float)xf[ks][e] - x0;
        s += d;
        q = __builtin_fmaf(d, d, q);
      }
    const float sm = pair_sum(s) * (1.0f / K);
    const float var = fmaxf(pair_sum(q) * (1.0f / K) - sm * sm, 0.f);
    const float rstd = rsqrtf(var + eps), shift = -(x0 + sm) * rstd;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4_t raw = __builtin_bit_cast(u32x4_t, xf[ks]);
      asm volatile("" : "+v"(raw));
      u32x4_t pk;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        pk[e] = pack_bf16x2(__builtin_fmaf(bf16_lo(raw[e]), rstd, shift), __builtin_fmaf(bf16_hi(raw[e]), rstd, shift));
      asm volatile("" : "+v"(pk));
      xf[ks] = __builtin_bit_cast(bf16x8_t, pk);
    }
  }
  if constexpr (!PROJ) {
    acc2_from_bias(bias2);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();   // the transposition patches are dead; the space now holds weight chunks
    dma_chunk(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  }

  // the lane's row of a half's fc1 tile inside the chunk buffer (half h adds 16 rows): value rows 0-15, gate rows 32-47
  const uint32_t trow = lq < 16 ? lq : lq + 16;
  const uint32_t frag_off = trow * ROWB + (((half ^ G::swz(trow)) & (uint32_t)(G::CPR - 1)) << 4);
  // fc1 of half h (0 / 1) of chunk c: acc1[i] <-> value feature (i/4)*8 + half*4 + i%4 of the half for i < 8, its gate
  // feature for i >= 8, row lq
  f32x16_t acc1;
  auto fc1 = [&](uint32_t c, int h) __attribute__((always_inline)) {
    const uint32_t slot = c % NB1;
    const char* sw = w1buf + slot * MG::CH1 + h * 16 * ROWB;
    constexpr int kAhead = kMlpFragsAhead;
    bf16x8_t wf[KS];
    auto read_frag = [&](int ks) __attribute__((always_inline)) {
      wf[ks] = *reinterpret_cast<const bf16x8_t*>(sw + (frag_off ^ (uint32_t)(ks * 32)));
    };
#pragma unroll
    for (int ks = 0; ks < kAhead; ++ks) read_frag(ks);
    {
      // the accumulators start from b' (fp32, 64 per chunk: the 32 value features, then the 32 gate features)
      const float* sb = reinterpret_cast<const float*>(s_side + slot * 1024) + h * 16 + half * 4;
      const float4 v0 = *reinterpret_cast<const float4*>(sb), v1 = *reinterpret_cast<const float4*>(sb + 8);
      const float4 g0 = *reinterpret_cast<const float4*>(sb + 32), g1 = *reinterpret_cast<const float4*>(sb + 40);
      acc1[0] = v0.x; acc1[1] = v0.y; acc1[2] = v0.z; acc1[3] = v0.w; acc1[4] = v1.x; acc1[5] = v1.y; acc1[6] = v1.z; acc1[7] = v1.w;
      acc1[8] = g0.x; acc1[9] = g0.y; acc1[10] = g0.z; acc1[11] = g0.w; acc1[12] = g1.x; acc1[13] = g1.y; acc1[14] = g1.z; acc1[15] = g1.w;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + kAhead < KS) read_frag(ks + kAhead);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ks], xf[ks], acc1, 0, 0, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 4 + kAhead, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (ks + kAhead < KS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // h = silu(value) * gate from the fp32 accumulators, rounded to bf16: the B operand of the half's fc2 k-step
  // (element e <-> hidden feature (e / 4) * 8 + half * 4 + e % 4 of the half)
  u32x4_t hb;
  auto gate = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);   // the reads of the next stage stay behind the gate: their registers are not free yet
#pragma unroll
    for (int p = 0; p < 4; ++p)
      hb[p] = pack_bf16x2(fast_silu(acc1[2 * p]) * acc1[2 * p + 8], fast_silu(acc1[2 * p + 1]) * acc1[2 * p + 9]);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto fc2 = [&](uint32_t c, int h) __attribute__((always_inline)) {
    const char* s2 = w2buf + (c % NB2) * MG::CH2 + lane * 16 + h * 1024;
    constexpr int kAhead2 = kMlpFragsAhead;
    bf16x8_t f[OT];
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) f[ot] = *reinterpret_cast<const bf16x8_t*>(s2 + ot * 2048);
#pragma unroll
    for (int ot = 0; ot < OT; ++ot)
      acc2[ot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[ot], __builtin_bit_cast(bf16x8_t, hb), acc2[ot], 0, 0, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead2, 0);
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (ot + kAhead2 < OT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  if (!has_rows) {
    // a wave without rows only carries its share of the weight requests and keeps the barriers in step
    for (uint32_t ci = 0; ci < nchunk; ++ci) {
      if (ci + 1 < nchunk) dma_chunk(ci + 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      wg_barrier_lds();
    }
    __syncthreads();
    return;
  }
  for (uint32_t ci = 0; ci < nchunk; ++ci) {
    // chunk ci + 1 goes into the buffers of chunk ci - 1, which every wave has left
    if (ci + 1 < nchunk) dma_chunk(ci + 1);
    fc1(ci, 0); gate(); fc2(ci, 0);
    fc1(ci, 1); gate(); fc2(ci, 1);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // chunk ci + 1 has landed
    wg_barrier_lds();
  }

  // ---- output: bf16(fc2) (+ residual), through a wave-private LDS patch so that the stores are row-contiguous ----
  uint16_t* y_wg = y + (size_t)wg_row0 * ldy;
  const uint16_t* res_wg = residual ? residual + (size_t)wg_row0 * ldr : nullptr;
  // the residual pieces of the wave's whole panel are requested at once (x is dead: its registers take them): one
  // memory latency for all of them instead of one per column tile
  u32x4_t rres[OT][2];
  if (residual) {
#pragma unroll
    for (int ot = 0; ot < OT; ++ot)
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const uint32_t row = min(row0 + rr, M - 1);            // rows past M read row M - 1
        rres[ot][h2] = *reinterpret_cast<const u32x4_t*>(res_wg + ((row - wg_row0) * ldr + ot * 32 + ch));
      }
  }
  __syncthreads();   // every wave is done with the weight buffers: their space takes the output patches
  static_assert((size_t)WAVES * 32 * kPatchRow * 2 <= (size_t)NB1 * MG::CH1, "the output patches alias the w1 buffers");
  uint16_t* patch = reinterpret_cast<uint16_t*>(lds_mlp) + wave * (32 * kPatchRow);
#pragma unroll
  for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 pk;
      pk.x = pack_bf16x2(acc2[ot][g * 4 + 0], acc2[ot][g * 4 + 1]);
      pk.y = pack_bf16x2(acc2[ot][g * 4 + 2], acc2[ot][g * 4 + 3]);
      *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
    }
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
      const uint32_t row = row0 + rr;
      const uint32_t lrow = wave * 32 + rr;
      u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
      if (residual) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rres[ot][h2][e]), bf16_hi(t[e]) + bf16_hi(rres[ot][h2][e]));
      }
      if (row < M) *reinterpret_cast<u32x4_t*>(y_wg + (lrow * ldy + ot * 32 + ch)) = t;
    }
  }
}


// Narrow layers (C = 32 / 64): all of w1', b' and w2 fit into LDS at once (7 / 13 KB per 32 hidden features), so
// a workgroup loads them once and then its waves walk 32-row tiles of x independently, with no barrier and no weight
// traffic per tile: the kernel moves x, the residual and y and nothing else. Same arithmetic as the streaming kernel
// above, stage by stage. What bounds it is the gate: per hidden feature and row one exp2 and one reciprocal
// (transcendental rate) and four ordinary operations, about 350 vector-ALU cycles per 16 hidden features of a tile
// against 128 / 224 cycles of matrix core. Measured on MI355X against the two-kernel path, launches of the weight
// preparation included: 1 M rows, C = 32, H = 128: 0.069 ms against 0.200 ms; 500 k rows, C = 64, H = 256: 0.091 ms
// against 0.198 ms; 3,000 rows: 0.017 ms against 0.024 / 0.026 ms.
constexpr int kMlpSmallWaves = 8;

template <int K>
__host__ __device__ constexpr size_t mlp_small_lds_bytes(uint32_t H, bool proj = false) {
  return (size_t)(H / 32) * (64 * K * 2 + K * 64 + 1024) + (size_t)kMlpSmallWaves * 32 * (K + 8) * 2 + (proj ? (size_t)K * K * 2 : 0);
}

// PROJ: as in the streaming kernel, x1 = bf16(a wpT + bp + x) is formed per tile in front of the LayerNorm (the
// projection weight sits in LDS with the others, the block input enters through products with an identity) and the
// kernel returns bf16(x1 + MLP(x1)); `residual` must be null.
template <int K, bool PROJ, bool EMBED = false>
__global__ __launch_bounds__(64 * kMlpSmallWaves) void ln_mlp_swiglu_small_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, float eps, const uint16_t* __restrict__ w1p,
    const float* __restrict__ b32, const uint16_t* __restrict__ w2p, const uint16_t* __restrict__ bias2,
    const uint16_t* __restrict__ residual, uint32_t ldr, uint16_t* __restrict__ y, uint32_t ldy, uint32_t M,
    uint32_t H, MlpProj pj) {
  using G = XsGeom<K>;
  constexpr int KS = K / 16, ROWB = G::ROWB, WAVES = kMlpSmallWaves, OT = K / 32;
  constexpr int CH1 = 64 * ROWB, CH2 = K * 64, N2 = CH2 / 1024, PROW = K + 8, PCPR = K / 8;
  static_assert(K == 32 || K == 64, "narrow layers only");
  static_assert(32 * kPatchRow <= 32 * PROW, "the output patch fits into the wave's transposition patch");
  extern __shared__ __attribute__((aligned(1024))) char lds_mlp[];
  const uint32_t nchunk = H / 32;
  char* w1buf = lds_mlp;
  char* w2buf = w1buf + (size_t)nchunk * CH1;
  char* s_side = w2buf + (size_t)nchunk * CH2;
  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  uint16_t* patch = reinterpret_cast<uint16_t*>(s_side + (size_t)nchunk * 1024) + wave * (32 * PROW);
  char* wpbuf = s_side + (size_t)nchunk * 1024 + (size_t)WAVES * 32 * PROW * 2;    // PROJ: the projection weight, laid out like a w1 chunk

  // ---- every weight of the layer -> LDS, the direct loads dealt out over the waves ----
  {
    if constexpr (PROJ) {
      constexpr uint32_t NP = (uint32_t)K * K * 2 / 1024;
      for (uint32_t j = wave; j < NP; j += WAVES) {
        const uint32_t r = (j * 64u + lane) / G::CPR, pc = lane % G::CPR;
        xs_lds_dma16(pj.w, (r * K + (pc ^ G::swz(r)) * 8u) * 2u, wpbuf + j * 1024);
      }
    }
    constexpr uint32_t per = G::N_DMA + N2 + 1;
    for (uint32_t pi = wave; pi < nchunk * per; pi += WAVES) {
      const uint32_t c = pi / per, j = pi % per;
      if (j < (uint32_t)G::N_DMA) {
        const uint32_t r = (j * 64u + lane) / G::CPR, pc = lane % G::CPR;      // chunk row, position of the lane's piece
        const uint32_t wrow = r < 32 ? c * 32u + r : H + c * 32u + (r - 32u);   // value rows, then gate rows
        xs_lds_dma16(w1p, (wrow * K + (pc ^ G::swz(r)) * 8u) * 2u, w1buf + c * CH1 + j * 1024);
      } else if (j < (uint32_t)G::N_DMA + N2) {
        const uint32_t q = j - G::N_DMA;
        xs_lds_dma16(w2p, c * CH2 + q * 1024u + lane * 16u, w2buf + c * CH2 + q * 1024);
      } else {
        xs_lds_dma4(b32, (lane < 32 ? c * 32u + lane : H + c * 32u + lane - 32u) * 4u, s_side + c * 1024);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  }

  const uint32_t trow = lq < 16 ? lq : lq + 16;
  const uint32_t frag_off = trow * ROWB + (((half ^ G::swz(trow)) & (uint32_t)(G::CPR - 1)) << 4);
  const uint32_t ntiles = (M + 31) / 32;
  // the rows of a tile as the lanes load them (row-contiguous 16-byte pieces); the next tile's are requested while the
  // current one is computed
  constexpr int XLOADS = (32 * PCPR) / kWave;
  u32x4_t xv[XLOADS];
  const uint16_t* const panel = PROJ ? pj.a : x;         // what the tile's operand rows are read from
  const uint32_t ld_panel = PROJ ? pj.lda : ldx;
  auto request_x = [&](uint32_t tile) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const uint32_t id = lane + i * kWave;
      const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
      const uint32_t r = min(tile * 32 + rr, M - 1);
      xv[i] = *reinterpret_cast<const u32x4_t*>(panel + (size_t)r * ld_panel + kc);
    }
  };
  // PROJ: identity fragments (k-step j of a 32-column tile holds its columns 16 j .. 16 j + 15) and the lane's offset
  // into a 32-row block of the projection weight
  bf16x8_t idf[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) idf[j][e] = (lq == (uint32_t)(16 * j + e) + 8u * half) ? (__bf16)1.0f : (__bf16)0.0f;
  const uint32_t poff = lq * ROWB + (((half ^ G::swz(lq)) & (uint32_t)(G::CPR - 1)) << 4);
  const uint32_t tile_step = gridDim.x * WAVES;
  if (blockIdx.x * WAVES + wave < ntiles) request_x(blockIdx.x * WAVES + wave);
  for (uint32_t tile = blockIdx.x * WAVES + wave; tile < ntiles; tile += tile_step) {
    const uint32_t row0 = tile * 32;
    // ---- the tile's rows of x -> registers (B-operand layout) through the wave's patch ----
    bf16x8_t xf[KS];
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const uint32_t id = lane + i * kWave;
      const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
      *reinterpret_cast<u32x4_t*>(patch + rr * PROW + kc) = xv[i];
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      xf[ks] = *reinterpret_cast<const bf16x8_t*>(patch + lq * PROW + ks * 16 + half * 8);
    if (tile + tile_step < ntiles) request_x(tile + tile_step);
    f32x16_t acc2[OT];
    if constexpr (PROJ) {
      // the block input's columns in operand layout, requested now; a wpT + bp; + x through the identity; x1 through
      // the wave's patch into operand layout; the accumulators go on as x1 + b2
      bf16x8_t xt[OT][2], eat[OT], cbe;
      if constexpr (EMBED) {
        cbe = embed_rows_operand(pj.coord, min(row0 + lq, M - 1), half);
#pragma unroll
        for (int ot = 0; ot < OT; ++ot) eat[ot] = embed_channels_operand(pj.etab, ot, lq, half);
      } else {
        const uint16_t* xrow = x + (size_t)min(row0 + lq, M - 1) * ldx + half * 8;
#pragma unroll
        for (int ot = 0; ot < OT; ++ot)
#pragma unroll
          for (int j = 0; j < 2; ++j) xt[ot][j] = *reinterpret_cast<const bf16x8_t*>(xrow + ot * 32 + j * 16);
      }
#pragma unroll
      for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint2 bb = *reinterpret_cast<const uint2*>(pj.b + ot * 32 + g * 8 + half * 4);
          acc2[ot][g * 4 + 0] = bf16_lo(bb.x); acc2[ot][g * 4 + 1] = bf16_hi(bb.x);
          acc2[ot][g * 4 + 2] = bf16_lo(bb.y); acc2[ot][g * 4 + 3] = bf16_hi(bb.y);
        }
        const char* sw = wpbuf + ot * 32 * ROWB;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t wf = *reinterpret_cast<const bf16x8_t*>(sw + (poff ^ (uint32_t)(ks * 32)));
          acc2[ot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[ks], acc2[ot], 0, 0, 0);
        }
      }
#pragma unroll
      for (int ot = 0; ot < OT; ++ot) {
        if constexpr (EMBED) {
          acc2[ot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(eat[ot], cbe, acc2[ot], 0, 0, 0);
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) acc2[ot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(idf[j], xt[ot][j], acc2[ot], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint2 bb = *reinterpret_cast<const uint2*>(bias2 + ot * 32 + g * 8 + half * 4);
          uint2 x1;
          x1.x = pack_bf16x2(acc2[ot][g * 4 + 0], acc2[ot][g * 4 + 1]);
          x1.y = pack_bf16x2(acc2[ot][g * 4 + 2], acc2[ot][g * 4 + 3]);
          *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = x1;
          acc2[ot][g * 4 + 0] = bf16_lo(x1.x) + bf16_lo(bb.x); acc2[ot][g * 4 + 1] = bf16_hi(x1.x) + bf16_hi(bb.x);
          acc2[ot][g * 4 + 2] = bf16_lo(x1.y) + bf16_lo(bb.y); acc2[ot][g * 4 + 3] = bf16_hi(x1.y) + bf16_hi(bb.y);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
          xf[2 * ot + j] = *reinterpret_cast<const bf16x8_t*>(patch + lq * kPatchRow + j * 16 + half * 8);
      }
    }
    // the residual rows of the tile, requested now, used at the end
    u32x4_t rres[OT][2];
    if (residual) {
#pragma unroll
      for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
          const uint32_t row = min(row0 + rr, M - 1);
          rres[ot][h2] = *reinterpret_cast<const u32x4_t*>(residual + ((size_t)row * ldr + ot * 32 + ch));
        }
    }
    // LayerNorm in place: x <- bf16((x - mean) * rstd), statistics shifted by the row's first element
    {
      const float x0 = __shfl((float)xf[0][0], lq, kWave);
      float sm = 0.f, sq = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = (float)xf[ks][e] - x0;
          sm += d;
          sq = __builtin_fmaf(d, d, sq);
        }
      const float mean = pair_sum(sm) * (1.0f / K);
      const float var = fmaxf(pair_sum(sq) * (1.0f / K) - mean * mean, 0.f);
      const float rstd = rsqrtf(var + eps), shift = -(x0 + mean) * rstd;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4_t raw = __builtin_bit_cast(u32x4_t, xf[ks]);
        u32x4_t pk;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          pk[e] = pack_bf16x2(__builtin_fmaf(bf16_lo(raw[e]), rstd, shift), __builtin_fmaf(bf16_hi(raw[e]), rstd, shift));
        xf[ks] = __builtin_bit_cast(bf16x8_t, pk);
      }
    }
    // fc2 accumulators start from the bias: acc2[ot][g*4+r] <-> output column ot*32 + g*8 + half*4 + r of row lq
    if constexpr (!PROJ) {
#pragma unroll
      for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint2 bb = *reinterpret_cast<const uint2*>(bias2 + ot * 32 + g * 8 + half * 4);
          acc2[ot][g * 4 + 0] = bf16_lo(bb.x); acc2[ot][g * 4 + 1] = bf16_hi(bb.x);
          acc2[ot][g * 4 + 2] = bf16_lo(bb.y); acc2[ot][g * 4 + 3] = bf16_hi(bb.y);
        }
    }
    for (uint32_t c = 0; c < nchunk; ++c) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // fc1 of the half: rows 0-15 value, 16-31 gate; the accumulators start from b' (fp32: the chunk's 32 value
        // features, then its 32 gate features)
        const char* sw = w1buf + c * CH1 + h * 16 * ROWB;
        const float* sb = reinterpret_cast<const float*>(s_side + c * 1024) + h * 16 + half * 4;
        const float4 v0 = *reinterpret_cast<const float4*>(sb), v1 = *reinterpret_cast<const float4*>(sb + 8);
        const float4 g0 = *reinterpret_cast<const float4*>(sb + 32), g1 = *reinterpret_cast<const float4*>(sb + 40);
        f32x16_t acc1 = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t wf = *reinterpret_cast<const bf16x8_t*>(sw + (frag_off ^ (uint32_t)(ks * 32)));
          acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[ks], acc1, 0, 0, 0);
        }
        u32x4_t hb;
#pragma unroll
        for (int p = 0; p < 4; ++p)
          hb[p] = pack_bf16x2(fast_silu(acc1[2 * p]) * acc1[2 * p + 8], fast_silu(acc1[2 * p + 1]) * acc1[2 * p + 9]);
        const char* s2 = w2buf + c * CH2 + lane * 16 + h * 1024;
#pragma unroll
        for (int ot = 0; ot < OT; ++ot) {
          const bf16x8_t f = *reinterpret_cast<const bf16x8_t*>(s2 + ot * 2048);
          acc2[ot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, __builtin_bit_cast(bf16x8_t, hb), acc2[ot], 0, 0, 0);
        }
      }
    }
    // ---- output: bf16(fc2) (+ residual) through the wave's patch, row-contiguous stores ----
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 pk;
        pk.x = pack_bf16x2(acc2[ot][g * 4 + 0], acc2[ot][g * 4 + 1]);
        pk.y = pack_bf16x2(acc2[ot][g * 4 + 2], acc2[ot][g * 4 + 3]);
        *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const uint32_t row = row0 + rr;
        u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
        if (residual) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rres[ot][h2][e]), bf16_hi(t[e]) + bf16_hi(rres[ot][h2][e]));
        }
        if (row < M) *reinterpret_cast<u32x4_t*>(y + ((size_t)row * ldy + ot * 32 + ch)) = t;
      }
    }
  }
}


// w2 [C][H] row-major -> fragment-major per chunk of 32 hidden features:
//   w2p[(((c * C/32 + ot) * 2 + s) * 64 + half * 32 + lq) * 8 + e] = w2[ot * 32 + lq][c * 32 + (2 s + e / 4) * 8 + half * 4 + e % 4]
// One thread per 16-byte piece.
// The LayerNorm fold of w1 (one wave per fc1 feature, blocks [0, fold_blocks)) rides in the same launch.
__global__ __launch_bounds__(256) void mlp_prep_kernel(const uint16_t* __restrict__ w1, const uint16_t* __restrict__ gamma,
                                                       const uint16_t* __restrict__ beta, const uint16_t* __restrict__ b1,
                                                       uint16_t* __restrict__ w1p, float* __restrict__ b32,
                                                       uint32_t fold_blocks, const uint16_t* __restrict__ w2,
                                                       uint16_t* __restrict__ w2p, uint16_t* __restrict__ zero_bias,
                                                       uint32_t C, uint32_t H) {
  if (blockIdx.x < fold_blocks) {
    const uint32_t n = blockIdx.x * 4 + threadIdx.x / kWave;
    if (n < 2 * H) ln_fold_row(w1, gamma, beta, b1, w1p, b32, C, n, threadIdx.x % kWave);
    return;
  }
  const uint32_t piece = (blockIdx.x - fold_blocks) * blockDim.x + threadIdx.x;
  if (piece < C / 8) *reinterpret_cast<uint4*>(zero_bias + piece * 8) = make_uint4(0u, 0u, 0u, 0u);   // stands in for a missing bias
  if (piece >= C * H / 8) return;
  const uint32_t lq = piece % 32, half = (piece / 32) % 2, s = (piece / 64) % 2;
  const uint32_t ot = (piece / 128) % (C / 32), c = piece / (128 * (C / 32));
  const uint16_t* src = w2 + (size_t)(ot * 32 + lq) * H + c * 32 + half * 4;
  const uint2 a = *reinterpret_cast<const uint2*>(src + (2 * s) * 8);
  const uint2 b = *reinterpret_cast<const uint2*>(src + (2 * s + 1) * 8);
  *reinterpret_cast<uint4*>(w2p + (size_t)piece * 8) = make_uint4(a.x, a.y, b.x, b.y);
}


template <int K, bool PROJ = false, bool EMBED = false>
static int launch_mlp(const uint16_t* x, uint32_t ldx, float eps, const uint16_t* w1p, const float* b32,
                           const uint16_t* w2p, const uint16_t* bias2, const uint16_t* residual, uint32_t ldr, uint16_t* y,
                           uint32_t ldy, uint32_t M, uint32_t H, int device, hipStream_t s, MlpProj pj = MlpProj{}) {
  constexpr size_t lds = MlpGeom<K>::lds_bytes(PROJ);
  static_assert(lds <= 160 * 1024, "chunk buffers exceed the LDS of a compute unit");
  static bool attr_set[64] = {};
  auto kern = ln_mlp_swiglu_kernel<K, PROJ, EMBED>;
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  // Whole turns of the chip run 256-row workgroups; what is left over is spread over all CUs in panels of fewer rows
  // (fewer waves with work per workgroup), so that the last turn is shorter than a full one.
  static int cus[64] = {};
  int n_cu = 256;
  if (device >= 0 && device < 64) {
    if (!cus[device]) F3D_CHECK_HIP(hipDeviceGetAttribute(&cus[device], hipDeviceAttributeMultiprocessorCount, device));
    n_cu = cus[device];
  }
  constexpr uint32_t kRows = 32 * kMlpWaves;
  const uint32_t panels = cdiv_u32(M, kRows);
  uint32_t main_wgs = panels, tail_rows = kRows, tail_wgs = 0;
  if (panels > (uint32_t)n_cu && panels % (uint32_t)n_cu != 0) {
    main_wgs = panels / (uint32_t)n_cu * (uint32_t)n_cu;
    const uint32_t left = M - main_wgs * kRows;
    tail_rows = cdiv_u32(cdiv_u32(left, (uint32_t)n_cu), 32u) * 32u;
    tail_wgs = cdiv_u32(left, tail_rows);
  }
  hipLaunchKernelGGL(kern, dim3(main_wgs + tail_wgs), dim3(64 * kMlpWaves), lds, s, x, ldx, eps, w1p, b32, w2p, bias2, residual,
                     ldr, y, ldy, M, H, main_wgs, tail_rows, pj);
  return F3D_OK;
}


template <int K, bool PROJ = false, bool EMBED = false>
static int launch_mlp_small(const uint16_t* x, uint32_t ldx, float eps, const uint16_t* w1p, const float* b32,
                            const uint16_t* w2p, const uint16_t* bias2, const uint16_t* residual, uint32_t ldr,
                            uint16_t* y, uint32_t ldy, uint32_t M, uint32_t H, int device, hipStream_t s,
                            MlpProj pj = MlpProj{}) {
  const size_t lds = mlp_small_lds_bytes<K>(H, PROJ);
  static int cus[64] = {};
  static size_t attr_lds[64] = {};
  int n_cu = 256;
  if (device >= 0 && device < 64) {
    if (!cus[device]) F3D_CHECK_HIP(hipDeviceGetAttribute(&cus[device], hipDeviceAttributeMultiprocessorCount, device));
    n_cu = cus[device];
  }
  auto kern = ln_mlp_swiglu_small_kernel<K, PROJ, EMBED>;
  if (device < 0 || device >= 64 || attr_lds[device] < lds) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_lds[device] = lds;
  }
  // as many resident workgroups as the LDS allows; each wave then walks its share of the 32-row tiles
  const uint32_t per_cu = (uint32_t)std::max<size_t>(1, std::min<size_t>(4, (160 * 1024) / lds));
  const uint32_t wgs = std::min<uint32_t>(cdiv_u32(cdiv_u32(M, 32), kMlpSmallWaves), (uint32_t)n_cu * per_cu);
  hipLaunchKernelGGL(kern, dim3(wgs), dim3(64 * kMlpSmallWaves), lds, s, x, ldx, eps, w1p, b32, w2p, bias2, residual, ldr,
                     y, ldy, M, H, pj);
  return F3D_OK;
}

}  // namespace f3d

extern "C" {

int f3d_ln_mlp_swiglu_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                           const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2,
                           const f3d_bf16_t* residual, uint32_t ldr, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                           uint32_t c, uint32_t hidden, int device, void* stream) {
  using namespace f3d;
  StagedWeightsScope staged;
  F3D_CHECK_ARG(x && gamma && w1 && w2 && y, "null tensor pointer");
  const bool narrow = c == 32 || c == 64;
  if (!(narrow || c == 128 || c == 256) || hidden == 0 || hidden % 32 != 0 || (uint64_t)hidden * c * 4 >= (1ull << 32) ||
      (c == 32 && mlp_small_lds_bytes<32>(hidden) > 160 * 1024) || (c == 64 && mlp_small_lds_bytes<64>(hidden) > 160 * 1024)) {
    set_error("No fused MLP kernel for width %u with hidden width %u (widths 128 and 256 with hidden a multiple of 32; "
              "widths 32 and 64 while all weights fit into LDS: hidden <= 640 / 288)", c, hidden);
    return F3D_ERR_UNSUPPORTED;
  }
  F3D_CHECK_ARG(ldx >= c && ldx % 8 == 0 && ldy >= c && ldy % 8 == 0 && (!residual || (ldr >= c && ldr % 8 == 0)),
                "row strides must be aligned and cover a row (ldx=%u ldy=%u ldr=%u)", ldx, ldy, ldr);
  F3D_CHECK_ARG((((uintptr_t)x | (uintptr_t)w1 | (uintptr_t)w2 | (uintptr_t)y | (uintptr_t)residual | (uintptr_t)gamma |
                  (uintptr_t)beta | (uintptr_t)b2) & 15u) == 0,
                "x/w1/w2/b2/y/residual/gamma/beta must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  // per call, in the per-device workspace: w1' (bf16 [2H][C]), b' (fp32 [2H]), w2 fragment-major (bf16 [C][H]), a zero
  // bias [C]
  const size_t w1_bytes = (size_t)2 * hidden * c * 2, b32_bytes = (((size_t)2 * hidden * 4) + 255) & ~(size_t)255;
  const size_t w2_bytes = (size_t)hidden * c * 2;
  bool ready = false;
  char* ws = (char*)weight_area(device, w1_bytes + b32_bytes + w2_bytes + (size_t)c * 2, &ready, s);
  if (!ws) return F3D_ERR_RUNTIME;
  uint16_t* w1p = (uint16_t*)ws;
  float* b32 = (float*)(ws + w1_bytes);
  uint16_t* w2p = (uint16_t*)(ws + w1_bytes + b32_bytes);
  uint16_t* zero_bias = (uint16_t*)(ws + w1_bytes + b32_bytes + w2_bytes);
  if (!b2) b2 = zero_bias;
  const uint32_t fold_blocks = cdiv_u32(2 * hidden, 4);
  if (!ready)
    hipLaunchKernelGGL(mlp_prep_kernel, dim3(fold_blocks + cdiv_u32(c * hidden / 8, 256)), dim3(256), 0, s, w1, gamma, beta, b1,
                       w1p, b32, fold_blocks, w2, w2p, zero_bias, c, hidden);
  int rc;
  if (c == 256) rc = launch_mlp<256>(x, ldx, eps, w1p, b32, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  else if (c == 32) rc = launch_mlp_small<32>(x, ldx, eps, w1p, b32, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  else if (c == 64) rc = launch_mlp_small<64>(x, ldx, eps, w1p, b32, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  else rc = launch_mlp<128>(x, ldx, eps, w1p, b32, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

// x != NULL: the block input is read; else coord / embed_table say how it is formed
static int proj_ln_mlp_impl(const f3d_bf16_t* a, uint32_t lda, const f3d_bf16_t* w_proj, const f3d_bf16_t* b_proj,
                            const f3d_bf16_t* x, uint32_t ldx, const f3d_half_t* coord, const f3d_bf16_t* embed_table,
                            const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w1,
                            const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2, f3d_bf16_t* y, uint32_t ldy,
                            uint32_t m, uint32_t c, uint32_t hidden, int device, void* stream) {
  using namespace f3d;
  StagedWeightsScope staged;
  const bool embed = x == nullptr;
  F3D_CHECK_ARG(a && w_proj && (x || (coord && embed_table)) && gamma && w1 && w2 && y, "null tensor pointer");
  const bool narrow = c == 32 || c == 64;
  if (!(narrow || c == 128 || c == 256) || hidden == 0 || hidden % 32 != 0 || (uint64_t)hidden * c * 4 >= (1ull << 32) ||
      (c == 32 && mlp_small_lds_bytes<32>(hidden, true) > 160 * 1024) ||
      (c == 64 && mlp_small_lds_bytes<64>(hidden, true) > 160 * 1024)) {
    set_error("No out-projection + MLP kernel for width %u with hidden width %u (widths 128 and 256 with hidden a multiple "
              "of 32; widths 32 and 64 while all weights fit into LDS)", c, hidden);
    return F3D_ERR_UNSUPPORTED;
  }
  F3D_CHECK_ARG(lda >= c && lda % 8 == 0 && (embed || (ldx >= c && ldx % 8 == 0)) && ldy >= c && ldy % 8 == 0,
                "row strides must be aligned and cover a row (lda=%u ldx=%u ldy=%u)", lda, ldx, ldy);
  F3D_CHECK_ARG((((uintptr_t)a | (uintptr_t)w_proj | (uintptr_t)b_proj | (uintptr_t)x | (uintptr_t)embed_table | (uintptr_t)w1 |
                  (uintptr_t)w2 | (uintptr_t)y | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)b2) & 15u) == 0 &&
                    ((uintptr_t)coord & 1u) == 0,
                "a/w_proj/b_proj/x/embed_table/w1/w2/b2/y/gamma/beta must be 16-byte aligned");
  if (m == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  // the MLP's prepared weights exactly as in f3d_ln_mlp_swiglu_bf16 (the same staged buffer serves both entry points)
  const size_t w1_bytes = (size_t)2 * hidden * c * 2, b32_bytes = (((size_t)2 * hidden * 4) + 255) & ~(size_t)255;
  const size_t w2_bytes = (size_t)hidden * c * 2;
  bool ready = false;
  char* ws = (char*)weight_area(device, w1_bytes + b32_bytes + w2_bytes + (size_t)c * 2, &ready, s);
  if (!ws) return F3D_ERR_RUNTIME;
  uint16_t* w1p = (uint16_t*)ws;
  float* b32 = (float*)(ws + w1_bytes);
  uint16_t* w2p = (uint16_t*)(ws + w1_bytes + b32_bytes);
  uint16_t* zero_bias = (uint16_t*)(ws + w1_bytes + b32_bytes + w2_bytes);
  if (!b2) b2 = zero_bias;
  const uint32_t fold_blocks = cdiv_u32(2 * hidden, 4);
  if (!ready)
    hipLaunchKernelGGL(mlp_prep_kernel, dim3(fold_blocks + cdiv_u32(c * hidden / 8, 256)), dim3(256), 0, s, w1, gamma, beta, b1,
                       w1p, b32, fold_blocks, w2, w2p, zero_bias, c, hidden);
  const MlpProj pj{a, lda, w_proj, b_proj ? b_proj : zero_bias, coord, embed_table};
  int rc;
#define F3D_PM(LAUNCH, KK)                                                                                                 \
  rc = embed ? LAUNCH<KK, true, true>(x, ldx, eps, w1p, b32, w2p, b2, nullptr, 0, y, ldy, m, hidden, device, s, pj)        \
             : LAUNCH<KK, true, false>(x, ldx, eps, w1p, b32, w2p, b2, nullptr, 0, y, ldy, m, hidden, device, s, pj)
  if (c == 256) F3D_PM(launch_mlp, 256);
  else if (c == 32) F3D_PM(launch_mlp_small, 32);
  else if (c == 64) F3D_PM(launch_mlp_small, 64);
  else F3D_PM(launch_mlp, 128);
#undef F3D_PM
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_proj_ln_mlp_swiglu_bf16(const f3d_bf16_t* a, uint32_t lda, const f3d_bf16_t* w_proj, const f3d_bf16_t* b_proj,
                                const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                                const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2,
                                f3d_bf16_t* y, uint32_t ldy, uint32_t m, uint32_t c, uint32_t hidden, int device,
                                void* stream) {
  if (!x) {
    f3d::set_error("null tensor pointer");
    return F3D_ERR_INVALID;
  }
  return proj_ln_mlp_impl(a, lda, w_proj, b_proj, x, ldx, nullptr, nullptr, gamma, beta, eps, w1, b1, w2, b2, y, ldy, m, c,
                          hidden, device, stream);
}

int f3d_embed_proj_ln_mlp_swiglu_bf16(const f3d_bf16_t* a, uint32_t lda, const f3d_bf16_t* w_proj, const f3d_bf16_t* b_proj,
                                      const f3d_half_t* coord, const f3d_bf16_t* embed_table, const f3d_bf16_t* gamma,
                                      const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w1, const f3d_bf16_t* b1,
                                      const f3d_bf16_t* w2, const f3d_bf16_t* b2, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                                      uint32_t c, uint32_t hidden, int device, void* stream) {
  if (!coord || !embed_table) {
    f3d::set_error("null tensor pointer");
    return F3D_ERR_INVALID;
  }
  return proj_ln_mlp_impl(a, lda, w_proj, b_proj, nullptr, 0, coord, embed_table, gamma, beta, eps, w1, b1, w2, b2, y, ldy, m,
                          c, hidden, device, stream);
}

}  // extern "C"
