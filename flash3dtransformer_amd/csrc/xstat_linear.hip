// Row-panel ("x-stationary") linear layers for gfx950: y = act(LN?(x) wT + bias) (+ residual) for the
// small inner dimensions of the Flash3D blocks (K = channels, 32..512).
//
// Stands where the reference runs LayerNorm followed by torch.nn.Linear / te.Linear
// (flash3dxfmr/layers/stage.py:94-97, buck_swin.py:185,194, hourglass.py:99,181-183).
//
// Why not an output-tiled GEMM: with K this small a 128x128 tile re-reads 128 KB of operands per
// 8 MFLOP, which saturates L2 long before the matrix cores.  Here a workgroup owns a panel of
// 32 * MT * WAVES rows of x for ALL output columns: every wave keeps its 32 * MT rows, already in the
// MFMA B-operand layout, in registers for the whole kernel (x is read from HBM exactly once), while w
// streams through LDS in chunks of 64 output features.  Each 16-byte LDS fragment read feeds MT MFMAs;
// with MT = 1 the LDS read port is as busy as the matrix cores, so the large configuration uses MT = 2.
// The product is formed transposed (A = w rows, B = x rows) so a lane owns 4 consecutive output columns
// of one row for the epilogue (bias, GELU / SiLU / ReLU / swiglu, residual, bf16 store).
//
// w chunks travel HBM/L2 -> LDS directly (global_load ... lds, no staging registers), three buffers deep:
// chunk c+2 is requested when chunk c starts.  Rows are unpadded; the 16-byte piece p of chunk-row r sits
// at position p ^ swz(r), which spreads the 32 rows of one fragment read over all banks.
//
// LayerNorm is applied to the rows while they sit in registers: one sweep for the statistics, one that replaces
// x by bf16((x - mean) * rstd) (the reference's LayerNorm also hands bf16 to its Linear).  gamma and beta are folded
// into the weights by a small kernel:  LN(x) wT + b = xhat w'T + b',  w' = bf16(w * gamma),  b' = b + w beta (fp32).
// The main loop then is the plain one with bias b'.
#include "xstat_common.h"

namespace f3d {

// the 64-column epilogue patch (residual layers with K <= 256) or the 32-column one
template <int K, bool SWIGLU, int EPI>
constexpr bool xs_wide_flush() { return !SWIGLU && K <= 256 && EPI == 2; }

template <int K, int WAVES, int NBUF>
constexpr size_t xs_lds_bytes(bool wide) {
  using G = XsGeom<K>;
  const size_t front = (size_t)NBUF * G::CHUNK_BYTES;
  return front + (size_t)WAVES * 32 * (wide ? kPatchRow2 : kPatchRow) * 2 + (size_t)kXsBiasSlots * 256;
}

// EPI: 0 = bias only, 1 = runtime activation and / or residual, 2 = residual only (its pieces are prefetched).
// With LN the kernel expects w = w' and lnx = b' as fp32 [N], both prepared by ln_fold_kernel.
// NBUF: w chunk buffers in LDS (chunk c + NBUF - 1 is requested when chunk c starts).
// EMBED: the rows are not read but formed: row r is the coordinate embedding bf16(coord[r] . etab[c][0:3] + etab[c][3])
// of its point (coord fp16 [M][3]; etab bf16 [K][8] = (wx, wy, wz, b, 0, 0, 0, 0) per channel), one MFMA per 32 channels.
template <int K, int MT, int WAVES, int NBUF, bool LN, bool SWIGLU, int EPI, bool EMBED = false>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void xstat_linear_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, float eps, const uint16_t* __restrict__ w,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ lnx,
    const uint16_t* __restrict__ residual, uint32_t ldr, uint16_t* __restrict__ y, uint32_t ldy, uint32_t M,
    uint32_t N, uint32_t act, const uint16_t* __restrict__ coord, const uint16_t* __restrict__ etab) {
  using G = XsGeom<K>;
  constexpr int KS = K / 16;             // MFMA k-steps
  constexpr int ROWB = G::ROWB;
  constexpr int ROWS_WG = 32 * MT * WAVES;
  extern __shared__ __attribute__((aligned(1024))) char lds_xs[];
  constexpr size_t kFront = (size_t)NBUF * G::CHUNK_BYTES;
  constexpr uint32_t kAheadChunks = NBUF - 1;
  uint16_t* lds_patch = reinterpret_cast<uint16_t*>(lds_xs + kFront);
  // the bias of a chunk as fp32 (64 values), three slots: chunk c + 2 is parked while chunk c is being read
  constexpr bool WIDE = xs_wide_flush<K, SWIGLU, EPI>();   // a row tile's 64 columns in one flush
  constexpr int kPatchPitch = WIDE ? kPatchRow2 : kPatchRow;
  char* s_side = lds_xs + kFront + (size_t)WAVES * 32 * kPatchPitch * 2;
  auto s_bias = [&](uint32_t c) -> float* { return reinterpret_cast<float*>(s_side + (c % kXsBiasSlots) * 256); };

  const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t row0 = blockIdx.x * ROWS_WG + wave * (32 * MT);

  // ---- w chunk streaming ----
  const uint32_t n_out = SWIGLU ? N / 2 : N;
  // a swiglu chunk pairs 32 value rows with their 32 gate rows; a plain chunk is 64 consecutive rows
  constexpr uint32_t COLS = SWIGLU ? 32u : (uint32_t)kXsChunk;   // output columns per chunk
  // swiglu chunks are always full (the launcher checks); a plain last chunk may hold only its first 32
  // rows: the missing rows are read from the last valid one and their tile is not stored
  const uint32_t nchunk = (n_out + COLS - 1) / COLS;
  auto w_row = [&](uint32_t c, uint32_t r) -> uint32_t {  // weight row behind chunk-local row r
    if (!SWIGLU) return min(c * kXsChunk + r, N - 1);
    return r < 32 ? c * 32 + r : n_out + c * 32 + (r - 32);
  };
  // direct loads of chunk c into buffer slot: instruction q fills LDS bytes [1024 q, 1024 q + 1024) of the
  // buffer, i.e. chunk rows [q * 64 / CPR, ...); wave v issues instructions v, v + WAVES, ...
  constexpr uint32_t kMyDmaMax = (G::N_DMA + WAVES - 1) / WAVES;
  const bool bias_dma = LN || bias != nullptr;
  const uint32_t my_dma = G::N_DMA / WAVES + (wave < (uint32_t)(G::N_DMA % WAVES) ? 1u : 0u) + ((bias_dma && wave == 0) ? 1u : 0u);
  auto dma_chunk = [&](uint32_t c, uint32_t c_seq, uint32_t slot) {   // c: the chunk, c_seq: its place in this workgroup's order
    // the chunk's 64 bias values go to its bias slot: fp32 b' with LN, else the bf16 bits zero-extended to a dword
    if (wave == 0) {
      char* sb = reinterpret_cast<char*>(s_bias(c_seq));
      if (LN) xs_lds_dma4(lnx, w_row(c, lane) * 4u, sb);
      else if (bias) xs_lds_dma2(bias, w_row(c, lane) * 2u, sb);
    }
    const char* buf = lds_xs + slot * G::CHUNK_BYTES;
#pragma unroll
    for (uint32_t i = 0; i < kMyDmaMax; ++i) {
      const uint32_t qi = wave + i * WAVES;
      if (qi < (uint32_t)G::N_DMA) {
        const uint32_t r = (qi * 64u + lane) / G::CPR, p = lane % G::CPR;   // chunk row and position of this lane's piece
        const uint32_t piece = p ^ G::swz(r);
        xs_lds_dma16(w, (w_row(c, r) * K + piece * 8u) * 2u, buf + qi * 1024);
      }
    }
  };
  const bool wg_full = (blockIdx.x + 1) * ROWS_WG <= M;
  uint16_t* y_wg = y + (size_t)(blockIdx.x * ROWS_WG) * ldy;                  // wave-uniform bases
  const uint16_t* res_wg = residual ? residual + (size_t)(blockIdx.x * ROWS_WG) * ldr : nullptr;
  // Workgroups walk the output columns in rotated order: at any moment different workgroups write
  // different column ranges, which spreads the stores over the HBM channels (with a power-of-two row
  // pitch every workgroup would otherwise hit the same channels at the same time).
  const uint32_t c_start = (blockIdx.x * 5u) % nchunk;
  auto actual = [&](uint32_t i) -> uint32_t { const uint32_t t = i + c_start; return t >= nchunk ? t - nchunk : t; };

  if (!bias_dma && tid < 64 * kXsBiasSlots) reinterpret_cast<float*>(s_side)[tid] = 0.f;   // no bias: zeros, once
  // the first chunk(s) of w are requested before anything else, so that they travel while the rows are fetched
  dma_chunk(actual(0), 0, 0);
  if (kAheadChunks > 1 && nchunk > 1) dma_chunk(actual(1), 1, 1);

  // ---- this wave's x rows -> registers in the B-operand layout: fragment ks of row tile mt is 16 bytes of row lq
  //      at columns ks * 16 + half * 8, loaded straight into its register, all of them in flight at once (the four
  //      fragments that share a 128-byte line are requested back to back).  Rows past M read row M - 1. ----
  bf16x8_t xf[MT][KS];
  if constexpr (EMBED) {
    // The rows are the coordinate embedding of their points (flash3dxfmr/layers/psh_ops.py:67-68: Linear(3, K) of the
    // coordinates cast to bf16), formed here instead of being read: per row tile and 32 channels one product of the
    // channels' (wx, wy, wz, b) with the rows' (x, y, z, 1), rounded to bf16 as the embedding layer stores it and
    // re-laid from the accumulator layout into operand layout through the wave's (still unused) epilogue patch.
    static_assert(K % 32 == 0 && EPI == 0 && !SWIGLU, "embedding in front of a plain bias epilogue");
    uint16_t* ep = lds_patch + wave * (32 * kPatchPitch);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint32_t r = min(row0 + mt * 32 + lq, M - 1);
      u32x4_t cb = {0u, 0u, 0u, 0u};
      if (half == 0) {
        const uint16_t* cp = coord + (size_t)r * 3;
        cb[0] = pack_bf16x2(half_bits_to_float(cp[0]), half_bits_to_float(cp[1]));
        cb[1] = pack_bf16x2(half_bits_to_float(cp[2]), 1.0f);
      }
#pragma unroll
      for (int t = 0; t < K / 32; ++t) {
        u32x4_t ea = {0u, 0u, 0u, 0u};
        if (half == 0) ea = *reinterpret_cast<const u32x4_t*>(etab + (size_t)(t * 32 + lq) * 8);
        f32x16_t e;
#pragma unroll
        for (int i = 0; i < 16; ++i) e[i] = 0.f;
        e = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, ea), __builtin_bit_cast(bf16x8_t, cb), e, 0, 0, 0);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint2 pk;
          pk.x = pack_bf16x2(e[g * 4 + 0], e[g * 4 + 1]);
          pk.y = pack_bf16x2(e[g * 4 + 2], e[g * 4 + 3]);
          *reinterpret_cast<uint2*>(ep + lq * kPatchPitch + g * 8 + half * 4) = pk;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
          xf[mt][2 * t + j] = *reinterpret_cast<const bf16x8_t*>(ep + lq * kPatchPitch + j * 16 + half * 8);
      }
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint32_t r = min(row0 + mt * 32 + lq, M - 1);
      const uint16_t* xp = x + (size_t)r * ldx + half * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) xf[mt][ks] = *reinterpret_cast<const bf16x8_t*>(xp + ks * 16);
    }
  }
  // LayerNorm of this lane's rows in place: one sweep for the sums of d = x - x0 and d^2 (shifted by the row's first
  // element so that the variance does not cancel), one that writes bf16((x - mean) * rstd) back
  if (LN) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const float x0 = __shfl((float)xf[mt][0][0], lq, kWave);   // lane lq (half 0) holds element 0 of row lq
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
      // one fragment at a time (kept opaque: otherwise the compiler holds every row element as a float from the first
      // sweep to the second, 8 registers per fragment, and spills)
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
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the first chunk(s) have landed
  __syncthreads();

  // per-lane byte offset of its fragment inside a chunk buffer; k-step ks is reached by ^ (32 ks)
  const uint32_t frag_off = lq * ROWB + (((half ^ G::swz(lq)) & (uint32_t)(G::CPR - 1)) << 4);
  uint16_t* patch = lds_patch + wave * (32 * kPatchPitch);

  // accumulators: acc[nt][mt][g*4+r] <-> column nt*32 + g*8 + half*4 + r
  f32x16_t acc[2][MT];

  // stage 1: requests for chunk ci + NBUF - 1 (its buffer and its bias slot were last read in chunk ci - 1, which
  // every wave has left).  (Spread over the k-steps of stage 2 they break its issue pattern: measured 10 % slower.)
  auto stage_request = [&](uint32_t ci) {
    if (ci + kAheadChunks < nchunk) dma_chunk(actual(ci + kAheadChunks), ci + kAheadChunks, (ci + kAheadChunks) % NBUF);
  };
  // stage 2: the MFMAs of chunk ci; the accumulators start from the bias
  auto stage_mfma = [&](uint32_t ci) {
    const uint32_t slot = ci % NBUF;
    const char* sw = lds_xs + slot * G::CHUNK_BYTES;
    const float* sb = s_bias(ci);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4 b4 = *reinterpret_cast<const float4*>(sb + nt * 32 + g * 8 + half * 4);
        if (!LN) {   // bf16 bits in the low half of each dword
          b4.x = __uint_as_float(__float_as_uint(b4.x) << 16); b4.y = __uint_as_float(__float_as_uint(b4.y) << 16);
          b4.z = __uint_as_float(__float_as_uint(b4.z) << 16); b4.w = __uint_as_float(__float_as_uint(b4.w) << 16);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[nt][mt][g * 4 + 0] = b4.x; acc[nt][mt][g * 4 + 1] = b4.y;
          acc[nt][mt][g * 4 + 2] = b4.z; acc[nt][mt][g * 4 + 3] = b4.w;
        }
      }
    // w fragments are read kAhead k-steps before the MFMAs that consume them
    // (one k-step for the plain 256-feature large panels: the registers of the second one would spill)
    constexpr int kAhead = (KS < 2 || (K >= 256 && MT > 1 && !SWIGLU)) ? 1 : 2;
    bf16x8_t wf[KS][2];
    auto read_frag = [&](int ks) {
      const char* p = sw + (frag_off ^ (uint32_t)(ks * 32));
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) wf[ks][nt] = *reinterpret_cast<const bf16x8_t*>(p + nt * 32 * ROWB);
    };
#pragma unroll
    for (int ks = 0; ks < kAhead; ++ks) read_frag(ks);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + kAhead < KS) read_frag(ks + kAhead);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ks][nt], xf[mt][ks], acc[nt][mt], 0, 0, 0);
    }
    // pin the issue order: kAhead k-steps of LDS reads first, then one k-step of reads per k-step of MFMAs
    __builtin_amdgcn_sched_group_barrier(0x100, 8 + 2 * kAhead, 0);   // the 8 bias reads come first
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * MT, 0);
      if (ks + kAhead < KS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  };
  // stage 3: epilogue of chunk ci: the results go through a wave-private LDS patch so that the global stores are
  // row-contiguous.  Residual layers flush a row tile's 64 columns at once: 8 lanes read and write the 128 bytes (a
  // whole line) of one row; measured at 482,304 rows, 256 -> 256: 0.150 against 0.171 ms with 64-byte pieces.  The
  // bias-only epilogue keeps 32-column flushes (4 lanes per row): whole lines measured 3 % slower there (256 -> 768:
  // 0.276 against 0.268 ms, same GPU), although a store-only loop of the same geometry takes them faster (5.1 against
  // 3.7 TB/s): the layer is bound by the chain of stages of a wave, which the longer flush lengthens.
  constexpr int PW = WIDE ? 64 : 32;                          // output columns per flush
  constexpr int NF = (SWIGLU || WIDE) ? 1 : 2;                // flushes per row tile
  constexpr int PPITCH = WIDE ? kPatchRow2 : kPatchRow;       // patch pitch in elements
  constexpr int LPR = PW / 8, RPI = kWave / LPR, NI = 32 / RPI;   // lanes per row, rows per instruction, instructions
  // byte offsets of this lane's piece inside a block of RPI rows: kernel-lifetime constants, so that a store or a
  // residual load needs one vector register of address (the rest of the address is uniform)
  const uint32_t ch = (lane % LPR) * 8;      // this lane's 8 columns of a flush
  const uint32_t y_lane = ((lane / LPR) * ldy + ch) * 2u, r_lane = ((lane / LPR) * ldr + ch) * 2u;
  auto stage_epilogue = [&](uint32_t ci) {
    const uint32_t col0 = actual(ci) * COLS;   // first output column of the chunk
    // a plain last chunk may hold 32 columns only: the lanes of the missing ones read 32 columns further left (a valid
    // address, the value is not used) and store nothing
    auto col_ok = [&](int f) -> bool { return col0 + f * PW + ch < n_out; };
    // (a SIGNED offset: 64 bytes to the left of the flush's first column, which lies at least 32 columns into the row)
    auto r_off = [&](int f) -> ptrdiff_t { return col_ok(f) ? (ptrdiff_t)r_lane : (ptrdiff_t)r_lane - 64; };
    // uniform base of row block i of row tile mt (rows wave * 32 MT + mt * 32 + i * RPI ...), columns of flush f
    auto y_base = [&](int mt, int f, int i) -> char* {
      return reinterpret_cast<char*>(y_wg) + ((size_t)(wave * (32 * MT) + mt * 32 + i * RPI) * ldy + col0 + f * PW) * 2u;
    };
    auto r_base = [&](int mt, int f, int i) -> const char* {
      return reinterpret_cast<const char*>(res_wg) + ((size_t)(wave * (32 * MT) + mt * 32 + i * RPI) * ldr + col0 + f * PW) * 2u;
    };
    // Residual pieces of the whole chunk are requested up front (one memory latency for all of them, hidden
    // behind the packing below) instead of one by one where they are added.  Rows past M read row M - 1.
    u32x4_t rres[EPI == 2 ? MT : 1][NF][NI];
    if (EPI == 2) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
          for (int i = 0; i < NI; ++i) {
            if (wg_full) {
              rres[mt][f][i] = *reinterpret_cast<const u32x4_t*>(r_base(mt, f, i) + r_off(f));
            } else {
              const uint32_t rr = lane / LPR + i * RPI;
              const uint32_t lrow = min(row0 + mt * 32 + rr, M - 1) - blockIdx.x * ROWS_WG;
              const uint32_t col = col_ok(f) ? col0 + f * PW + ch : n_out - 8;
              rres[mt][f][i] = *reinterpret_cast<const u32x4_t*>(res_wg + (lrow * ldr + col));
            }
          }
    }
    auto flush_tile = [&](auto full_tag, int mt, int f) {
      // patch holds rows [mt*32, mt*32+32) x PW columns starting at output column col0 + f * PW
      constexpr bool kFull = decltype(full_tag)::value;
      const bool ok = col_ok(f);
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        // two row blocks at a time: their patch reads are in flight together, and no more registers are held than that
        if (i > 0 && i % 2 == 0) __builtin_amdgcn_sched_barrier(0);
        const uint32_t rr = lane / LPR + i * RPI;
        const uint32_t row = row0 + mt * 32 + rr;
        u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * PPITCH + ch);
        if (!kFull && row >= M) continue;
        if (EPI == 1) {
          if (!SWIGLU && act != F3D_ACT_NONE) {
#pragma unroll
            for (int e = 0; e < 4; ++e) t[e] = pack_bf16x2(xs_act(bf16_lo(t[e]), act), xs_act(bf16_hi(t[e]), act));
          }
          if (residual) {
            const u32x4_t rv = *reinterpret_cast<const u32x4_t*>(r_base(mt, f, i) + r_off(f));
#pragma unroll
            for (int e = 0; e < 4; ++e)
              t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rv[e]), bf16_hi(t[e]) + bf16_hi(rv[e]));
          }
        }
        if (EPI == 2) {
          const u32x4_t rv = rres[EPI == 2 ? mt : 0][f][i];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rv[e]), bf16_hi(t[e]) + bf16_hi(rv[e]));
        }
        if (ok) *reinterpret_cast<u32x4_t*>(y_base(mt, f, i) + y_lane) = t;
      }
    };
    auto epilogue = [&](auto full_tag) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (!SWIGLU) {
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              uint2 pk;   // Linear output is bf16
              pk.x = pack_bf16x2(acc[nt][mt][g * 4 + 0], acc[nt][mt][g * 4 + 1]);
              pk.y = pack_bf16x2(acc[nt][mt][g * 4 + 2], acc[nt][mt][g * 4 + 3]);
              *reinterpret_cast<uint2*>(patch + lq * PPITCH + (WIDE ? nt * 32 : 0) + g * 8 + half * 4) = pk;
            }
            if (!WIDE) flush_tile(full_tag, mt, nt);
          }
          if (WIDE) flush_tile(full_tag, mt, 0);
        } else {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            float hv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              // the gate is formed from the fp32 accumulators: one rounding (of the product) where the
              // reference rounds fc1 to bf16 first and the product again
              hv[r] = fast_silu(acc[0][mt][g * 4 + r]) * acc[1][mt][g * 4 + r];
            }
            uint2 pk;
            pk.x = pack_bf16x2(hv[0], hv[1]);
            pk.y = pack_bf16x2(hv[2], hv[3]);
            *reinterpret_cast<uint2*>(patch + lq * PPITCH + g * 8 + half * 4) = pk;
          }
          flush_tile(full_tag, mt, 0);
        }
      }
    };
    if (wg_full) epilogue(std::true_type{}); else epilogue(std::false_type{});
  };
  // Chunk ci + 1 must have landed when the interval ends.  Its requests were issued one interval ago; since then this
  // wave has issued the memory operations of one epilogue (stores, and the residual loads of EPI 2: kEpiOps of them
  // when every row of the workgroup is stored; none before the first epilogue) and the requests of chunk ci + 2
  // (my_dma).  Memory operations complete in order, so "at most that many outstanding" is the weakest wait that covers
  // chunk ci + 1, and it does not wait for the stores.  Allowing MORE than were issued would let the wait return before
  // the chunk has landed; where the epilogue's count is not fixed (partial workgroup, run-time residual) the stores
  // are therefore not allowed for: the wait is then early, never late.
  // (two flushes of 32 columns per row tile: a last chunk may issue half of them, so none are allowed for)
  const uint32_t kEpiOps = (EPI == 1 || !wg_full || NF > 1) ? 0u : (uint32_t)(MT * NI * (EPI == 2 ? 2 : 1));
  auto wait_next_chunk = [&](uint32_t ci) {
    if (kAheadChunks > 1 && ci + kAheadChunks < nchunk) xs_wait_vm(my_dma + (ci > 0 ? kEpiOps : 0u));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
  };

  // The two waves that share a SIMD (wave v and v + WAVES/2) run the stages of a barrier interval in
  // complementary order, so that one's epilogue (VALU, LDS, stores) overlaps the other's MFMAs:
  //   first half :  request(c)  mfma(c)      wait  epilogue(c)   | barrier
  //   second half:  epilogue(c-1)  request(c)  mfma(c)  wait      | barrier      (+ epilogue(last) at the end)
  // Both halves read chunk c's buffer and bias slot inside the same interval, so the rotations are unchanged.
  // The stores of a late epilogue are older than the requests that follow them, as the wait needs.
  const bool late_half = NBUF >= 3 && WAVES >= 8 && wave >= (uint32_t)(WAVES / 2);
  if (!late_half) {
    for (uint32_t ci = 0; ci < nchunk; ++ci) {
      stage_request(ci);
      stage_mfma(ci);
      wait_next_chunk(ci);
      stage_epilogue(ci);
      wg_barrier_lds();
    }
  } else {
    for (uint32_t ci = 0; ci < nchunk; ++ci) {
      if (ci > 0) stage_epilogue(ci - 1);
      stage_request(ci);
      stage_mfma(ci);
      wait_next_chunk(ci);
      wg_barrier_lds();
    }
    stage_epilogue(nchunk - 1);
  }
}

// w' = bf16(w * gamma) and b'[n] = bias[n] + sum_k w[n][k] * beta[k] as fp32.  One wave per output feature.
__global__ __launch_bounds__(256) void ln_fold_kernel(const uint16_t* __restrict__ w, const uint16_t* __restrict__ gamma,
                                                      const uint16_t* __restrict__ beta,
                                                      const uint16_t* __restrict__ bias, uint16_t* __restrict__ wp,
                                                      float* __restrict__ bias32, uint32_t N, uint32_t K) {
  const uint32_t n = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (n >= N) return;
  ln_fold_row(w, gamma, beta, bias, wp, bias32, K, n, lane);
}

void launch_ln_fold(const uint16_t* w, const uint16_t* gamma, const uint16_t* beta, const uint16_t* bias, uint16_t* wp,
                    float* bias32, uint32_t N, uint32_t K, hipStream_t s) {
  hipLaunchKernelGGL(ln_fold_kernel, dim3(cdiv_u32(N, 4)), dim3(256), 0, s, w, gamma, beta, bias, wp, bias32, N, K);
}

template <int K, int MT, int WAVES, int NBUF>
static int launch_k(bool ln, bool swiglu, hipStream_t s, const uint16_t* x, uint32_t ldx, float eps,
                    const uint16_t* w, const uint16_t* bias, const uint16_t* lnx,
                    const uint16_t* residual, uint32_t ldr, uint16_t* y, uint32_t ldy, uint32_t M, uint32_t N,
                    uint32_t act, int device, const uint16_t* coord = nullptr, const uint16_t* etab = nullptr) {
  const bool general = act != F3D_ACT_NONE || residual != nullptr;
  const bool res_only = act == F3D_ACT_NONE && residual != nullptr;
  const dim3 grid(cdiv_u32(M, 32 * MT * WAVES)), block(64 * WAVES);
#define F3D_XS(L, S, E, ...)                                                                                       \
  do {                                                                                                             \
    static bool attr_set[64] = {};                                                                                 \
    auto kern = xstat_linear_kernel<K, MT, WAVES, NBUF, L, S, E, ##__VA_ARGS__>;                                        \
    constexpr size_t lds = xs_lds_bytes<K, WAVES, NBUF>(xs_wide_flush<K, S, E>());                                 \
    if (device < 0 || device >= 64 || !attr_set[device]) {                                                         \
      F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
      if (device >= 0 && device < 64) attr_set[device] = true;                                                     \
    }                                                                                                              \
    hipLaunchKernelGGL(kern, grid, block, lds, s, x, ldx, eps, w, bias, lnx, residual, ldr, y, ldy, M, N,          \
                       act, coord, etab);                                                                          \
  } while (0)
  if constexpr (K <= 256) {
    if (coord) {       // the rows are the coordinate embedding, formed in the kernel (LayerNorm + bias epilogue only)
      if (!ln || swiglu || general) return F3D_ERR_UNSUPPORTED;
      F3D_XS(true, false, 0, true);
      return F3D_OK;
    }
  } else if (coord) {
    return F3D_ERR_UNSUPPORTED;
  }
  if (ln && swiglu) { if (res_only) F3D_XS(true, true, 2); else if (general) F3D_XS(true, true, 1); else F3D_XS(true, true, 0); }
  else if (ln) { if (res_only) F3D_XS(true, false, 2); else if (general) F3D_XS(true, false, 1); else F3D_XS(true, false, 0); }
  else if (swiglu) { if (res_only) F3D_XS(false, true, 2); else if (general) F3D_XS(false, true, 1); else F3D_XS(false, true, 0); }
  else { if (res_only) F3D_XS(false, false, 2); else if (general) F3D_XS(false, false, 1); else F3D_XS(false, false, 0); }
#undef F3D_XS
  return F3D_OK;
}

// Returns F3D_OK when launched, F3D_ERR_UNSUPPORTED when the shape is not covered (the caller then uses
// the tiled GEMM), another code on failure.
int launch_xstat_linear(const uint16_t* x, uint32_t ldx, const uint16_t* gamma, const uint16_t* beta, float eps,
                        const uint16_t* w, const uint16_t* bias, const uint16_t* residual, uint32_t ldr, uint16_t* y,
                        uint32_t ldy, uint32_t M, uint32_t N, uint32_t K, uint32_t act, int device, hipStream_t s,
                        const uint16_t* coord, const uint16_t* etab) {
  const bool ln = gamma != nullptr;
  const bool swiglu = act == F3D_ACT_SWIGLU;
  const uint32_t run_act = swiglu ? (uint32_t)F3D_ACT_NONE : act;
  if (M == 0) return F3D_OK;
  // whole 32-column tiles; a swiglu chunk pairs 32 value rows with 32 gate rows
  if (swiglu ? N % 64 != 0 : N % 32 != 0) return F3D_ERR_UNSUPPORTED;
  if (K != 32 && K != 64 && K != 128 && K != 256 && K != 512) return F3D_ERR_UNSUPPORTED;
  if ((uint64_t)N * K * 2 >= (1ull << 32)) return F3D_ERR_UNSUPPORTED;   // 32-bit byte offsets into w
  const uint16_t* lnx = nullptr;
  if (ln) {
    // w' (bf16 [N][K]) and b' (fp32 [N]): per call in the per-device workspace, or kept in the caller's staged buffer
    const size_t wp_bytes = ((size_t)N * K * 2 + 255) & ~(size_t)255;
    bool ready = false;
    char* ws = (char*)weight_area(device, wp_bytes + (size_t)N * 4, &ready, s);
    if (!ws) return F3D_ERR_RUNTIME;
    uint16_t* wp = (uint16_t*)ws;
    float* b32 = (float*)(ws + wp_bytes);
    if (!ready) launch_ln_fold(w, gamma, beta, bias, wp, b32, N, K, s);
    w = wp;
    lnx = (const uint16_t*)b32;   // the kernel reads b' from here
  }
  // Large panels (64 rows per wave, 8 waves, 3 chunk buffers: one workgroup per CU) when their workgroups fill
  // at least three quarters of the chip, otherwise 32 rows per wave in 4-wave workgroups with 2 buffers
  // (measured at 125 k rows: large panels 12 % faster; at 62 k rows: small panels 30 % faster).
  // (Two 4-wave workgroups of 64-row waves per CU measured 6 % slower than one 8-wave workgroup.)
  const bool big = M >= 512u * 192u;
#define F3D_XS_CASE(KK)                                                                                                  \
  case KK:                                                                                                               \
    return big ? launch_k<KK, 2, 8, 3>(ln, swiglu, s, x, ldx, eps, w, bias, lnx, residual, ldr, y, ldy, M, N,   \
                                       run_act, device, coord, etab)                                                     \
               : launch_k<KK, 1, 4, 2>(ln, swiglu, s, x, ldx, eps, w, bias, lnx, residual, ldr, y, ldy, M, N,   \
                                       run_act, device, coord, etab);
  switch (K) {
    F3D_XS_CASE(32)
    F3D_XS_CASE(64)
    F3D_XS_CASE(128)
    F3D_XS_CASE(256)
    case 512:
      // 512 inner features fill the register budget with 32 rows per wave; two 64 KB chunk buffers
      return launch_k<512, 1, 8, 2>(ln, swiglu, s, x, ldx, eps, w, bias, lnx, residual, ldr, y, ldy, M, N,
                                    run_act, device, coord, etab);
    default: return F3D_ERR_UNSUPPORTED;
  }
#undef F3D_XS_CASE
}

}  // namespace f3d
