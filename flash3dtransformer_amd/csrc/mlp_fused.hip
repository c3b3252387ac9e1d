// Whole gated MLP of a transformer block in one kernel for gfx950:
//     y = (silu(LN(x) w1_valueT + b1_value) * (LN(x) w1_gateT + b1_gate)) w2T + b2 (+ residual)
// Stands where the reference runs te.LayerNormMLP(activation = "swiglu") followed by the residual add
// (flash3dxfmr/layers/elem_wise.py:22-26, stage.py:94-97).
//
// A workgroup of four waves owns 64 * 4 rows.  Every wave keeps its 64 rows of x in registers (matrix-core operand
// layout) for the whole kernel and walks the hidden features 32 at a time: the fc1 products of the chunk (value and
// gate tiles), the gate in registers, and at once the fc2 update of ALL output columns from the 32 hidden values just
// made.  The hidden activations never leave the registers: the fc1 product is formed transposed (rows of w1 as the A
// operand), so a lane ends up with 16 hidden values of one row, which after rounding to bf16 already ARE a B operand
// of the fc2 product; the matching order of the hidden index inside a k-step is baked into the prepared copy of w2.
// The fc2 accumulators (64 rows x C outputs per wave, 256 registers at C = 256) are why a wave has the whole
// register file of its SIMD to itself (one wave per SIMD).
//
// Per chunk the weights stream HBM/L2 -> LDS directly (global_load ... lds), three buffers deep: 64 rows of the
// LayerNorm-folded w1 (row-major, 16-byte pieces XOR-swizzled) and the chunk's slice of w2, which the preparation
// kernel stores fragment-major (the 64 lanes' 16-byte pieces of one fragment are consecutive), so its LDS reads are
// linear.  LayerNorm as in the row-panel linear kernel: the rows are normalised in registers (bf16((x - mean) * rstd)),
// w' = w * gamma, and one extra k-step starts the fc1 accumulators from b' = b1 + w1 beta.
//
// Matrix-core bound: 6 * M * C * H flops (fc1 value + gate, fc2) against HBM traffic of x, residual and y only.
// The hidden activations (M x H bf16, 1 GB at 482 k rows x 1024) are never allocated.  Measured on MI355X at
// 482,304 rows, C = 256, H = 1024 against the LayerNorm+fc1+gate kernel followed by the fc2+residual kernel:
// 0.94 ms against 0.98 ms on the activations of a block with small random weights, 1.04 ms against 0.97 ms on
// unit-variance random tensors.  With one wave per SIMD the matrix core is busy about a third of the time.  A lone
// wave does reach 2.06 PFLOP/s on back-to-back products with two independent accumulators, and four waves per CU read
// LDS at 295 B/ns, so neither the product issue rate nor LDS bandwidth is the limit: the chunk loop has about 1000
// instructions for its 101 products, and with a single wave per SIMD nothing but the matrix core's own latency
// overlaps with their issue.  Two waves per SIMD need at most 256 registers per wave, which x (128) and the fc2
// accumulators (256) do not allow at C = 256.  So this kernel is a memory saving, not yet a speed-up, and the layers
// use it on request only.
#include "xstat_common.h"

namespace f3d {

// Buffers in LDS: chunk c + 1 is requested when chunk c starts.  fc1 reads w1 of chunk c in interval c (two buffers);
// fc2 of chunk c runs in interval c + 1, interleaved with the gate arithmetic of chunk c + 1 (three w2 buffers).
constexpr int kMlpWaves = 4, kMlpMT = 2, kMlpBufs1 = 2, kMlpBufs2 = 3;
// The x operands of the last kMlpXTail k-steps stay in LDS (wave-private, 16 bytes per lane, row tile and k-step) and
// are re-read every chunk: the registers they would occupy are what keeps the chunk loop free of spills.
constexpr int kMlpXTail = 2;

template <int K>
struct MlpGeom {
  using G = XsGeom<K>;
  static constexpr int OT = K / 32;                         // output column tiles of fc2
  static constexpr int CH1 = G::CHUNK_BYTES;                // w1 chunk: 64 rows
  static constexpr int CH2 = K * 32 * 2;                    // w2 chunk: K outputs x 32 hidden
  static constexpr int N_DMA2 = CH2 / 1024;
  // weight buffers, the table rows of the w1 slots, and the x operands kept in LDS
  static constexpr size_t lds_bytes() {
    return (size_t)kMlpBufs1 * (CH1 + 1024) + (size_t)kMlpBufs2 * CH2 +
           (size_t)kMlpWaves * kMlpMT * kMlpXTail * 1024;
  }
};

__device__ __forceinline__ void mlp_wait_vm(uint32_t n) {
  switch (n) {
#define F3D_W(N) case N: __builtin_amdgcn_s_waitcnt(0x0F70 | N); break;
    F3D_W(0) F3D_W(1) F3D_W(2) F3D_W(3) F3D_W(4) F3D_W(5) F3D_W(6) F3D_W(7) F3D_W(8) F3D_W(9) F3D_W(10) F3D_W(11)
    F3D_W(12) F3D_W(13) F3D_W(14) F3D_W(15)
#undef F3D_W
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}

// w1p: LayerNorm-folded fc1 weight [2 H][K] (value rows then gate rows), lnx: its table [2 H][8] (ln_fold_kernel);
// w2p: fc2 weight, fragment-major per chunk (mlp_w2_prep_kernel); bias2 [K] (zeros when the layer has none: loaded
// unconditionally, so that all its loads are in flight together); H: hidden width, multiple of 32.
template <int K>
__global__ __launch_bounds__(64 * kMlpWaves) __attribute__((amdgpu_waves_per_eu(1, 1))) void ln_mlp_swiglu_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, float eps, const uint16_t* __restrict__ w1p,
    const uint16_t* __restrict__ lnx, const uint16_t* __restrict__ w2p, const uint16_t* __restrict__ bias2,
    const uint16_t* __restrict__ residual, uint32_t ldr, uint16_t* __restrict__ y, uint32_t ldy, uint32_t M,
    uint32_t H) {
  using G = XsGeom<K>;
  using MG = MlpGeom<K>;
  constexpr int KS = K / 16, ROWB = G::ROWB, WAVES = kMlpWaves, MT = kMlpMT, NB1 = kMlpBufs1, NB2 = kMlpBufs2, OT = MG::OT;
  constexpr int ROWS_WG = 32 * MT * WAVES;
  extern __shared__ __attribute__((aligned(1024))) char lds_mlp[];
  char* w1buf = lds_mlp;
  char* w2buf = lds_mlp + (size_t)NB1 * MG::CH1;
  char* s_side = w2buf + (size_t)NB2 * MG::CH2;   // per w1 slot: the chunk's 64 rows of the bias table
  constexpr int XT = kMlpXTail, KSR = K / 16 - XT;                            // k-steps whose x operand is in registers
  bf16x8_t* s_xtail = reinterpret_cast<bf16x8_t*>(s_side + (size_t)NB1 * 1024);   // [wave][mt][j][lane]

  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t row0 = blockIdx.x * ROWS_WG + wave * (32 * MT);

  // ---- this wave's x rows -> registers (B-operand layout), transposed through a wave-private LDS patch ----
  bf16x8_t xf[MT][KS];
  {
    constexpr int KP = G::KP, PROW = KP + 8, PCPR = KP / 8;
    static_assert((size_t)WAVES * 32 * PROW * 2 <= (size_t)NB1 * MG::CH1 + (size_t)NB2 * MG::CH2, "the transposition patches alias the weight buffers");
    uint16_t* patch = reinterpret_cast<uint16_t*>(lds_mlp) + wave * (32 * PROW);
    constexpr int XLOADS = (32 * PCPR) / kWave;
    // every global load of the panel is requested before the first transposition pass (one memory latency in all)
    u32x4_t v[MT][K / KP][XLOADS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int kp = 0; kp < K / KP; ++kp)
#pragma unroll
        for (int i = 0; i < XLOADS; ++i) {
          const uint32_t id = lane + i * kWave;
          const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
          const uint32_t r = min(row0 + mt * 32 + rr, M - 1);
          v[mt][kp][i] = *reinterpret_cast<const u32x4_t*>(x + (size_t)r * ldx + kp * KP + kc);
        }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int kp = 0; kp < K / KP; ++kp) {
#pragma unroll
        for (int i = 0; i < XLOADS; ++i) {
          const uint32_t id = lane + i * kWave;
          const uint32_t rr = id / PCPR, kc = (id % PCPR) * 8;
          *reinterpret_cast<u32x4_t*>(patch + rr * PROW + kc) = v[mt][kp][i];
        }
#pragma unroll
        for (int ks = 0; ks < KP / 16; ++ks)
          xf[mt][kp * (KP / 16) + ks] = *reinterpret_cast<const bf16x8_t*>(patch + lq * PROW + ks * 16 + half * 8);
      }
  }
  // LayerNorm of this lane's rows in place: statistics (shifted by the row's first element against cancellation), then
  // x <- bf16((x - mean) * rstd), one fragment at a time (kept opaque so that the floats of the first sweep are not
  // held for the second)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const float x0 = __shfl((float)xf[mt][0][0], lq, kWave);
    float s = 0.f, q = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = (float)xf[mt][ks][e] - x0;
        s += d;
        q = __builtin_fmaf(d, d, q);
      }
    const float sm = pair_sum(s) * (1.0f / K);
    const float var = fmaxf(pair_sum(q) * (1.0f / K) - sm * sm, 0.f);
    const float rstd = rsqrtf(var + eps), shift = -(x0 + sm) * rstd;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4_t raw = __builtin_bit_cast(u32x4_t, xf[mt][ks]);
      asm volatile("" : "+v"(raw));
      u32x4_t pk;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        pk[e] = pack_bf16x2(__builtin_fmaf(bf16_lo(raw[e]), rstd, shift), __builtin_fmaf(bf16_hi(raw[e]), rstd, shift));
      asm volatile("" : "+v"(pk));
      xf[mt][ks] = __builtin_bit_cast(bf16x8_t, pk);
    }
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < XT; ++j) s_xtail[((wave * MT + mt) * XT + j) * 64 + lane] = xf[mt][KSR + j];

  // fc2 accumulators start from the bias: acc2[ot][mt][g*4+r] <-> output column ot*32 + g*8 + half*4 + r of row lq
  f32x16_t acc2[OT][MT];
#pragma unroll
  for (int ot = 0; ot < OT; ++ot)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint2 bb = *reinterpret_cast<const uint2*>(bias2 + ot * 32 + g * 8 + half * 4);
      const float b[4] = {bf16_lo(bb.x), bf16_hi(bb.x), bf16_lo(bb.y), bf16_hi(bb.y)};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc2[ot][mt][g * 4 + r] = b[r];
    }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // the x rows and the bias have arrived: nothing of this wave is in flight
  __syncthreads();                      // the transposition patches are dead; the space now holds w1 chunks

  // ---- weight streaming ----
  const uint32_t nchunk = H / 32;
  constexpr uint32_t kDma1 = G::N_DMA / WAVES, kDma2 = MG::N_DMA2 / WAVES;
  static_assert(G::N_DMA % WAVES == 0 && MG::N_DMA2 % WAVES == 0, "direct loads split evenly over the waves");
  const uint32_t my_dma = kDma1 + kDma2 + (wave == 0 ? 1u : 0u);
  // Per-lane parts of the direct-load addresses are kept to four registers; everything that depends on the chunk or
  // on the instruction's number goes into the (scalar) base pointer.
  //   w1: the i-th instruction of this wave covers the 16-byte pieces [64 qi, 64 qi + 64) of the chunk buffer,
  //       qi = wave + WAVES i, i.e. piece position my_p of chunk row my_r + i * RSTEP.  my_r < RSTEP and RSTEP is 8 or
  //       16, so the row's swizzle is swz(my_r) ^ (i * RSTEP & 15): two lane offsets cover every i.
  //   w2: linear;  table: row `lane` of the chunk (32 value rows, then 32 gate rows)
  constexpr uint32_t RSTEP = WAVES * 64 / G::CPR;
  static_assert((RSTEP == 8 || RSTEP == 16) && G::RP == 1 && G::SWZ_MASK == 15, "direct-load addressing assumes K = 128 or 256");
  const uint32_t my_r = (wave * 64u + lane) / G::CPR, my_p = lane % G::CPR;
  uint32_t w1_lane[2];
#pragma unroll
  for (uint32_t o = 0; o < 2; ++o) w1_lane[o] = my_r * (K * 2) + ((my_p ^ my_r ^ (o * 8u)) & (uint32_t)(G::CPR - 1)) * 16u;
  const uint32_t w2_lane = wave * 1024u + lane * 16u;
  const uint32_t tab_lane = (lane < 32 ? lane : H + lane - 32) * 16u;
  auto dma_chunk = [&](uint32_t c) __attribute__((always_inline)) {
    const uint32_t slot = c % NB1;
    const char* b1 = w1buf + slot * MG::CH1;
#pragma unroll
    for (uint32_t i = 0; i < kDma1; ++i) {
      const uint32_t rr = i * RSTEP;                                                  // row advance of instruction i
      const uint32_t wrow = rr < 32 ? c * 32u + rr : H + c * 32u + (rr - 32u);       // value rows, then gate rows
      xs_lds_dma16(reinterpret_cast<const char*>(w1p) + (size_t)wrow * (K * 2), w1_lane[(rr & 15u) ? 1 : 0],
                   b1 + (wave + i * WAVES) * 1024);
    }
    const char* b2 = w2buf + (c % NB2) * MG::CH2;
#pragma unroll
    for (uint32_t i = 0; i < kDma2; ++i)
      xs_lds_dma16(reinterpret_cast<const char*>(w2p) + (size_t)c * MG::CH2 + i * (WAVES * 1024), w2_lane,
                   b2 + (wave + i * WAVES) * 1024);
    if (wave == 0) xs_lds_dma16(reinterpret_cast<const char*>(lnx) + (size_t)c * 512, tab_lane, s_side + slot * 1024);
  };

  dma_chunk(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  const uint32_t frag_off = lq * ROWB + (((half ^ G::swz(lq)) & (uint32_t)(G::CPR - 1)) << 4);
  (void)my_dma;

  // fc1 of chunk c: value tile (nt 0) and gate tile (nt 1), transposed: acc1[nt][mt][g*4+r] <-> hidden feature
  // g*8 + half*4 + r of the chunk, row lq
  f32x16_t acc1[2][MT];
  auto fc1 = [&](uint32_t c) __attribute__((always_inline)) {
    const uint32_t slot = c % NB1;
    const char* sw = w1buf + slot * MG::CH1;
    constexpr int kAhead = 2;   // k-steps of LDS reads in flight ahead of their products
    bf16x8_t wf[KS][2];
    bf16x8_t xt[XT > 0 ? XT : 1][MT];   // x operands of the k-steps kept in LDS
    auto read_frag = [&](int ks) __attribute__((always_inline)) {
      const char* p = sw + (frag_off ^ (uint32_t)(ks * 32));
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) wf[ks][nt] = *reinterpret_cast<const bf16x8_t*>(p + nt * 32 * ROWB);
      if (ks >= KSR) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xt[ks - KSR][mt] = s_xtail[((wave * MT + mt) * XT + (ks - KSR)) * 64 + lane];
      }
    };
#pragma unroll
    for (int ks = 0; ks < kAhead; ++ks) read_frag(ks);
    {
      // bias k-step: the table rows (wsum_hi, wsum_hi, wsum_lo, b'_hi, b'_hi, b'_lo, 0, 0) against (0, 0, 0, 1, 0, 1, 0, 0)
      // start the accumulators from b' = b'_hi + b'_lo (exact: products with 1 in fp32)
      bf16x8_t tf[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) tf[nt] = *reinterpret_cast<const bf16x8_t*>(s_side + slot * 1024 + (nt * 32 + lq) * 16);
      bf16x8_t xe[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        u32x4_t d = {0u, half == 0 ? 0x3F800000u : 0u, half == 0 ? 0x3F800000u : 0u, 0u};
        asm volatile("" : "+v"(d));   // rebuilt per chunk: four registers are not worth holding
        xe[mt] = __builtin_bit_cast(bf16x8_t, d);
      }
      const f32x16_t zero = {};
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc1[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tf[nt], xe[mt], zero, 0, 0, 0);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + kAhead < KS) read_frag(ks + kAhead);
      bf16x8_t xb[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xb[mt] = ks < KSR ? xf[mt][ks] : xt[ks >= KSR ? ks - KSR : 0][mt];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc1[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ks][nt], xb[mt], acc1[nt][mt], 0, 0, 0);
    }
    // Pin the issue order (left alone, the scheduler sinks every LDS read to just before its first use, which
    // exposes the whole LDS latency twice per k-step): the table rows and kAhead k-steps of
    // fragments first, then the bias products, then per k-step its products followed by the reads of the
    // k-step kAhead later (w fragments, and the x operands that live in LDS)
    __builtin_amdgcn_sched_group_barrier(0x100, 2 + 2 * kAhead + (kAhead > KSR ? MT * (kAhead - KSR) : 0), 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * MT, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * MT, 0);
      // the operands of k-step ks + kAhead are requested now
      if (ks + kAhead < KS) {
        if (ks + kAhead >= KSR) __builtin_amdgcn_sched_group_barrier(0x100, 2 + MT, 0);
        else __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // Gate of the chunk in acc1: h = silu(value) * gate from the fp32 accumulators, rounded to bf16 (the hidden
  // activation's type).  hb[mt][s] is the B operand of fc2's k-step s for row tile mt: element e <-> hidden feature
  // (2 s + e / 4) * 8 + half * 4 + e % 4.  One piece is one register (two elements); a row tile has 8 pieces.
  u32x4_t hb[MT][2];
  auto gate_piece = [&](int mt, int q) __attribute__((always_inline)) {
    const int s = q / 4, p = q % 4;
    const int e0 = (2 * s + p / 2) * 4 + (p % 2) * 2;   // accumulator index g * 4 + r of element 2 p
    const float v0 = fast_silu(acc1[0][mt][e0]) * acc1[1][mt][e0];
    const float v1 = fast_silu(acc1[0][mt][e0 + 1]) * acc1[1][mt][e0 + 1];
    hb[mt][s][p] = pack_bf16x2(v0, v1);
  };
  // fc2 of chunk c, row tile mt, output tiles ot and ot + 1 (two independent accumulators alternate)
  auto fc2_pair = [&](uint32_t c, int mt, int ot) __attribute__((always_inline)) {
    const char* s2 = w2buf + (c % NB2) * MG::CH2 + lane * 16;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      bf16x8_t f[2];
#pragma unroll
      for (int o = 0; o < 2; ++o) f[o] = *reinterpret_cast<const bf16x8_t*>(s2 + ((ot + o) * 2 + s) * 1024);
#pragma unroll
      for (int o = 0; o < 2; ++o)
        acc2[ot + o][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[o], __builtin_bit_cast(bf16x8_t, hb[mt][s]),
                                                                   acc2[ot + o][mt], 0, 0, 0);
    }
  };
  static_assert(MT == 2 && OT % 2 == 0, "the interleave below is written for two row tiles");
  constexpr int kPairs = OT / 2;                      // fc2 steps per row tile
  constexpr int kPiecesPerPair = (8 + kPairs - 1) / kPairs;
  // the matrix core runs fc2 of (chunk cf, row tile mf) while the vector unit forms the gate of row tile mg of the
  // chunk in acc1; mf's operands in hb are complete, mg's are being written (mg != mf)
  auto fc2_with_gate = [&](uint32_t cf, int mf, int mg) __attribute__((always_inline)) {
#pragma unroll
    for (int pr = 0; pr < kPairs; ++pr) {
      fc2_pair(cf, mf, 2 * pr);
#pragma unroll
      for (int j = 0; j < kPiecesPerPair; ++j)
        if (pr * kPiecesPerPair + j < 8) gate_piece(mg, pr * kPiecesPerPair + j);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Interval ci:  fc1(ci);  fc2(ci - 1, tile 1) || gate(ci, tile 0);  fc2(ci, tile 0) || gate(ci, tile 1).
  // Chunk 0 has no pending fc2: its tile-0 gate runs alone.
  if (nchunk > 1) dma_chunk(1);
  fc1(0);
#pragma unroll
  for (int q = 0; q < 8; ++q) gate_piece(0, q);
  fc2_with_gate(0, 0, 1);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  for (uint32_t ci = 1; ci < nchunk; ++ci) {
    // chunk ci + 1 goes into the w1 buffer that chunk ci - 1 used and the w2 buffer that chunk ci - 2 used; every
    // wave has left both (the last read of w2 of chunk ci - 2 was in interval ci - 1)
    if (ci + 1 < nchunk) dma_chunk(ci + 1);
    fc1(ci);
    fc2_with_gate(ci - 1, 1, 0);
    fc2_with_gate(ci, 0, 1);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // chunk ci + 1 has landed
    __syncthreads();
  }
  // the residual pieces of the whole panel are requested now (x is dead: its registers take them), one memory latency
  // for all of them, hidden behind the last fc2 products
  uint16_t* y_wg = y + (size_t)(blockIdx.x * ROWS_WG) * ldy;
  const uint16_t* res_wg = residual ? residual + (size_t)(blockIdx.x * ROWS_WG) * ldr : nullptr;
  u32x4_t rres[MT][OT][2];
  if (residual) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
          const uint32_t row = min(row0 + mt * 32 + rr, M - 1);            // rows past M read row M - 1
          rres[mt][ot][h2] = *reinterpret_cast<const u32x4_t*>(res_wg + ((row - blockIdx.x * ROWS_WG) * ldr + ot * 32 + ch));
        }
  }
#pragma unroll
  for (int pr = 0; pr < kPairs; ++pr) fc2_pair(nchunk - 1, 1, 2 * pr);
  __syncthreads();   // every wave is done with the weight buffers: their space takes the output patches

  // ---- output: bf16(fc2) (+ residual), through a wave-private LDS patch so that the stores are row-contiguous ----
  static_assert((size_t)WAVES * 32 * kPatchRow * 2 <= (size_t)NB1 * MG::CH1 + (size_t)NB2 * MG::CH2, "the output patches alias the weight buffers");
  uint16_t* patch = reinterpret_cast<uint16_t*>(lds_mlp) + wave * (32 * kPatchRow);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 pk;
        pk.x = pack_bf16x2(acc2[ot][mt][g * 4 + 0], acc2[ot][mt][g * 4 + 1]);
        pk.y = pack_bf16x2(acc2[ot][mt][g * 4 + 2], acc2[ot][mt][g * 4 + 3]);
        *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
      }
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const uint32_t row = row0 + mt * 32 + rr;
        const uint32_t lrow = wave * (32 * MT) + mt * 32 + rr;
        u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
        if (residual) {
          const u32x4_t rv = rres[mt][ot][h2];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rv[e]), bf16_hi(t[e]) + bf16_hi(rv[e]));
        }
        if (row < M) *reinterpret_cast<u32x4_t*>(y_wg + (lrow * ldy + ot * 32 + ch)) = t;
      }
    }
}

// w2 [C][H] row-major -> fragment-major per chunk of 32 hidden features:
//   w2p[(((c * C/32 + ot) * 2 + s) * 64 + half * 32 + lq) * 8 + e] = w2[ot * 32 + lq][c * 32 + (2 s + e / 4) * 8 + half * 4 + e % 4]
// One thread per 16-byte piece.
__global__ __launch_bounds__(256) void mlp_w2_prep_kernel(const uint16_t* __restrict__ w2, uint16_t* __restrict__ w2p,
                                                          uint16_t* __restrict__ zero_bias, uint32_t C, uint32_t H) {
  const uint32_t piece = blockIdx.x * blockDim.x + threadIdx.x;
  if (piece < C / 8) *reinterpret_cast<uint4*>(zero_bias + piece * 8) = make_uint4(0u, 0u, 0u, 0u);   // stands in for a missing bias
  if (piece >= C * H / 8) return;
  const uint32_t lq = piece % 32, half = (piece / 32) % 2, s = (piece / 64) % 2;
  const uint32_t ot = (piece / 128) % (C / 32), c = piece / (128 * (C / 32));
  const uint16_t* src = w2 + (size_t)(ot * 32 + lq) * H + c * 32 + half * 4;
  const uint2 a = *reinterpret_cast<const uint2*>(src + (2 * s) * 8);
  const uint2 b = *reinterpret_cast<const uint2*>(src + (2 * s + 1) * 8);
  *reinterpret_cast<uint4*>(w2p + (size_t)piece * 8) = make_uint4(a.x, a.y, b.x, b.y);
}

template <int K>
static int launch_mlp(const uint16_t* x, uint32_t ldx, float eps, const uint16_t* w1p, const uint16_t* lnx,
                      const uint16_t* w2p, const uint16_t* bias2, const uint16_t* residual, uint32_t ldr, uint16_t* y,
                      uint32_t ldy, uint32_t M, uint32_t H, int device, hipStream_t s) {
  constexpr size_t lds = MlpGeom<K>::lds_bytes();
  static_assert(lds <= 160 * 1024, "chunk buffers exceed the LDS of a compute unit");
  static bool attr_set[64] = {};
  auto kern = ln_mlp_swiglu_kernel<K>;
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  hipLaunchKernelGGL(kern, dim3(cdiv_u32(M, 32 * kMlpMT * kMlpWaves)), dim3(64 * kMlpWaves), lds, s, x, ldx, eps, w1p,
                     lnx, w2p, bias2, residual, ldr, y, ldy, M, H);
  return F3D_OK;
}

}  // namespace f3d

extern "C" {

int f3d_ln_mlp_swiglu_bf16(const f3d_bf16_t* x, uint32_t ldx, const f3d_bf16_t* gamma, const f3d_bf16_t* beta, float eps,
                           const f3d_bf16_t* w1, const f3d_bf16_t* b1, const f3d_bf16_t* w2, const f3d_bf16_t* b2,
                           const f3d_bf16_t* residual, uint32_t ldr, f3d_bf16_t* y, uint32_t ldy, uint32_t m,
                           uint32_t c, uint32_t hidden, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(x && gamma && w1 && w2 && y, "null tensor pointer");
  if (!(c == 128 || c == 256) || hidden == 0 || hidden % 32 != 0 || (uint64_t)hidden * c * 4 >= (1ull << 32)) {
    set_error("No fused MLP kernel for width %u with hidden width %u (widths 128 and 256, hidden a multiple of 32)", c,
              hidden);
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
  // per call, in the per-device workspace: w1' (bf16 [2H][C]), its table (bf16 [2H][8]), w2 fragment-major (bf16 [C][H]),
  // a zero bias [C]
  const size_t w1_bytes = (size_t)2 * hidden * c * 2, tab_bytes = (size_t)2 * hidden * 16, w2_bytes = (size_t)hidden * c * 2;
  char* ws = (char*)workspace(device, w1_bytes + tab_bytes + w2_bytes + (size_t)c * 2);
  if (!ws) return F3D_ERR_RUNTIME;
  uint16_t* w1p = (uint16_t*)ws;
  uint16_t* table = (uint16_t*)(ws + w1_bytes);
  uint16_t* w2p = (uint16_t*)(ws + w1_bytes + tab_bytes);
  uint16_t* zero_bias = (uint16_t*)(ws + w1_bytes + tab_bytes + w2_bytes);
  if (!b2) b2 = zero_bias;
  launch_ln_fold(w1, gamma, beta, b1, w1p, table, nullptr, 2 * hidden, c, s);
  hipLaunchKernelGGL(mlp_w2_prep_kernel, dim3(cdiv_u32(c * hidden / 8, 256)), dim3(256), 0, s, w2, w2p, zero_bias, c, hidden);
  int rc;
  if (c == 256) rc = launch_mlp<256>(x, ldx, eps, w1p, table, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  else rc = launch_mlp<128>(x, ldx, eps, w1p, table, w2p, b2, residual, ldr, y, ldy, m, hidden, device, s);
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
