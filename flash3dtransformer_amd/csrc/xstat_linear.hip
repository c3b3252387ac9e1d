// Row-panel ("x-stationary") linear layers for gfx950: y = act(LN?(x) wT + bias) (+ residual) for the
// small inner dimensions of the Flash3D blocks (K = channels, 32..512).
//
// Stands where the reference runs LayerNorm followed by torch.nn.Linear / te.Linear
// (flash3dxfmr/layers/stage.py:94-97, buck_swin.py:185,194, hourglass.py:99,181-183).
//
// Why not an output-tiled GEMM: with K this small a 128x128 tile re-reads 128 KB of operands per
// 8 MFLOP, which saturates L2 long before the matrix cores.  Here a workgroup owns a panel of
// 128 * MT rows of x for ALL output columns: every wave keeps its 32 * MT rows, already in the MFMA
// B-operand layout, in registers for the whole kernel (x is read from HBM exactly once, and because
// a lane pair holds a complete row the LayerNorm statistics are in-register sums plus one lane
// exchange), while w streams through LDS in chunks of 64 output features, double buffered, one
// barrier per chunk.  Each LDS fragment read feeds MT MFMAs.  The product is formed transposed
// (A = w rows, B = x rows) so a lane owns 4 consecutive output columns of one row for the epilogue
// (bias, GELU / SiLU / ReLU / swiglu, residual, bf16 store).
#include "f3d_device.h"
#include "f3d_internal.h"
#include <stdlib.h>
#include <type_traits>

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kXsThreads = 256;
constexpr int kXsChunk = 64;  // output features per w chunk (two 32-wide MFMA tiles)

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

// EPI: 0 = bias only, 1 = runtime activation and / or residual
template <int K, int MT, bool LN, bool SWIGLU, int EPI>
__global__ __launch_bounds__(kXsThreads) __attribute__((amdgpu_waves_per_eu((MT == 1 && K <= 256) ? 2 : 1, (MT == 1 && K <= 256) ? 2 : 1)))
void xstat_linear_kernel(
    const uint16_t* __restrict__ x, uint32_t ldx, const uint16_t* __restrict__ gamma,
    const uint16_t* __restrict__ beta, float eps, const uint16_t* __restrict__ w,
    const uint16_t* __restrict__ bias, const uint16_t* __restrict__ residual, uint32_t ldr,
    uint16_t* __restrict__ y, uint32_t ldy, uint32_t M, uint32_t N, uint32_t act) {
  constexpr int KS = K / 16;             // MFMA k-steps
  constexpr int WROW = K + 8;            // padded LDS row (elements)
  constexpr int CHUNK_ELEMS = kXsChunk * WROW;
  constexpr int CPR = K / 8;             // 16-byte chunks per row
  constexpr int NLOAD = (kXsChunk * CPR + kXsThreads - 1) / kXsThreads;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds_xs[];  // 2 x [64][WROW] w chunks
  __shared__ __attribute__((aligned(16))) float s_bias[2][kXsChunk];
  constexpr int kPatchRow = 40;  // 32 output columns + 8 pad (80-byte pitch keeps 16-byte alignment)
  __shared__ __attribute__((aligned(16))) uint16_t lds_patch[4 * 32 * kPatchRow];

  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t row0 = blockIdx.x * (128 * MT) + wave * (32 * MT);

  // ---- this wave's x rows -> registers in the B-operand layout.  Loaded row-contiguously
  //      (a row is one burst across CPR lanes) and transposed through a wave-private LDS patch ----
  bf16x8_t xf[MT][KS];
  {
    uint16_t* patch = lds_xs + wave * (32 * WROW);   // 4 x 32 x WROW elements fit in one w buffer pair
    constexpr int RPI = kWave / CPR > 0 ? kWave / CPR : 1;          // rows per load instruction
    constexpr int LPR = CPR < kWave ? CPR : kWave;                  // lanes per row
    constexpr int XLOADS = (32 * CPR) / kWave;                      // load instructions per m-tile
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int i = 0; i < XLOADS; ++i) {
        const uint32_t id = lane + i * kWave;
        const uint32_t rr = id / CPR, kc = (id % CPR) * 8;
        const uint32_t r = min(row0 + mt * 32 + rr, M - 1);
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + (size_t)r * ldx + kc);
        *reinterpret_cast<u32x4_t*>(patch + rr * WROW + kc) = v;
      }
      (void)RPI; (void)LPR;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        xf[mt][ks] = *reinterpret_cast<const bf16x8_t*>(patch + lq * WROW + ks * 16 + half * 8);
    }
  }
  if (LN) {
    // Statistics in one sweep over the packed registers (sums of d = x - x0 and d^2, shifted by the
    // row's first element so that the variance does not cancel), then a second sweep that normalises
    // in place.  The register fence between the sweeps keeps the compiler from holding all K values of
    // a row as fp32 across them, which would double the kernel's register footprint.
    float mean[MT], rstd[MT];
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
      mean[mt] = x0 + sm;
      rstd[mt] = rsqrtf(var + eps);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4_t raw = __builtin_bit_cast(u32x4_t, xf[mt][ks]);
        asm volatile("" : "+v"(raw));
        xf[mt][ks] = __builtin_bit_cast(bf16x8_t, raw);
      }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8_t g = *reinterpret_cast<const bf16x8_t*>(gamma + ks * 16 + half * 8);
      bf16x8_t b;
      if (beta) b = *reinterpret_cast<const bf16x8_t*>(beta + ks * 16 + half * 8);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float v = ((float)xf[mt][ks][e] - mean[mt]) * rstd[mt] * (float)g[e];
          if (beta) v += (float)b[e];
          xf[mt][ks][e] = (__bf16)v;  // the normalised activations are bf16, as a separate LayerNorm would emit
        }
    }
  }
  __syncthreads();  // the transpose patches are dead; the space now holds w chunks

  // ---- w chunk streaming ----
  const uint32_t n_out = SWIGLU ? N / 2 : N;
  // a swiglu chunk pairs 32 value rows with their 32 gate rows; a plain chunk is 64 consecutive rows
  constexpr uint32_t COLS = SWIGLU ? 32u : (uint32_t)kXsChunk;   // output columns per chunk
  const uint32_t nchunk = (n_out + COLS - 1) / COLS;
  auto w_row = [&](uint32_t c, uint32_t r) -> uint32_t {  // weight row behind chunk-local row r
    if (!SWIGLU) return c * kXsChunk + r;
    return r < 32 ? c * 32 + r : n_out + c * 32 + (r - 32);
  };
  // the launcher only takes shapes whose chunks are all full (N % 64 == 0), so no row guard is needed
  static_assert((kXsChunk * CPR) % kXsThreads == 0, "w chunk must split evenly over the workgroup");
  // two register sets: chunk c+2 is requested while chunk c is computed, so a w fetch has two chunk
  // computations to land before it is staged
  u32x4_t rwA[NLOAD], rwB[NLOAD];
  float rbA = 0.f, rbB = 0.f;
  auto fetch = [&](uint32_t c, u32x4_t (&rw)[NLOAD], float& rb) {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const uint32_t id = tid + i * kXsThreads;
      const uint32_t r = id / CPR, kc = (id % CPR) * 8;
      rw[i] = *reinterpret_cast<const u32x4_t*>(w + (size_t)w_row(c, r) * K + kc);
    }
    if (bias) rb = bf16_bits_to_float(bias[w_row(c, tid & (kXsChunk - 1))]);
  };
  auto stage = [&](uint32_t c, const u32x4_t (&rw)[NLOAD], float rb) {
    uint16_t* dst = lds_xs + (c & 1u) * CHUNK_ELEMS;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const uint32_t id = tid + i * kXsThreads;
      const uint32_t r = id / CPR, kc = (id % CPR) * 8;
      *reinterpret_cast<u32x4_t*>(dst + r * WROW + kc) = rw[i];
    }
    if (tid < kXsChunk) s_bias[c & 1u][tid] = rb;
  };

  const bool wg_full = (blockIdx.x + 1) * (128 * MT) <= M;
  // Workgroups walk the output columns in rotated order: at any moment different workgroups write
  // different column ranges, which spreads the stores over the HBM channels (with a power-of-two row
  // pitch every workgroup would otherwise hit the same channels at the same time).
  const uint32_t c_start = (blockIdx.x * 5u) % nchunk;
  auto actual = [&](uint32_t i) -> uint32_t { const uint32_t t = i + c_start; return t >= nchunk ? t - nchunk : t; };
  fetch(actual(0), rwA, rbA);
  if (nchunk > 1) fetch(actual(1), rwB, rbB);
  stage(0, rwA, rbA);
  if (nchunk > 2) fetch(actual(2), rwA, rbA);
  __syncthreads();
  // Order inside one step: MFMAs of chunk ci -> stage chunk ci+1 into the other LDS buffer -> request
  // chunk ci+3 into the register set just freed -> epilogue stores of chunk ci -> barrier.  The stores
  // are the youngest memory operations when the step ends, so nothing waits on them until a whole
  // chunk of MFMA work later.
  auto chunk_body = [&](auto parity, uint32_t ci) {
    constexpr bool odd = decltype(parity)::value;
    const uint32_t c = actual(ci);   // ci: position in this workgroup's order (selects LDS buffer / register set)
    const uint16_t* sw = lds_xs + (ci & 1u) * CHUNK_ELEMS;
    const float* sb = s_bias[ci & 1u];
    // accumulators start from the bias: acc[nt][mt][g*4+r] <-> column nt*32 + g*8 + half*4 + r
    f32x16_t acc[2][MT];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 b4 = *reinterpret_cast<const float4*>(sb + nt * 32 + g * 8 + half * 4);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[nt][mt][g * 4 + 0] = b4.x; acc[nt][mt][g * 4 + 1] = b4.y;
          acc[nt][mt][g * 4 + 2] = b4.z; acc[nt][mt][g * 4 + 3] = b4.w;
        }
      }
    // w fragments are read kAhead k-steps before the MFMAs that consume them
    constexpr int kAhead = KS < 4 ? KS : 4;
    bf16x8_t wf[KS][2];
    auto read_frag = [&](int ks) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
        wf[ks][nt] = *reinterpret_cast<const bf16x8_t*>(sw + (nt * 32 + lq) * WROW + ks * 16 + half * 8);
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
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * MT, 0);
      if (ks + kAhead < KS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    // next chunk into the other LDS buffer, then refill the freed register set two chunks ahead
    if (ci + 1 < nchunk) {
      if constexpr (odd) stage(ci + 1, rwA, rbA); else stage(ci + 1, rwB, rbB);
    }
    if (ci + 3 < nchunk) {
      if constexpr (odd) fetch(actual(ci + 3), rwA, rbA); else fetch(actual(ci + 3), rwB, rbB);
    }
    // ---- epilogue: the wave's 32 x 32 result tiles go through a wave-private LDS patch so that
    //      the global stores are row-contiguous 16-byte pieces (4 lanes = 64 bytes of one row) ----
    const uint32_t col0 = c * COLS;   // first output column of the chunk
    uint16_t* patch = lds_patch + wave * (32 * kPatchRow);
    auto flush_tile = [&](auto full_tag, int mt, uint32_t colbase) {
      // patch holds rows [mt*32, mt*32+32) x 32 columns starting at output column colbase
      constexpr bool kFull = decltype(full_tag)::value;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint32_t rr = (lane >> 2) + h2 * 16, ch = (lane & 3u) * 8;
        const uint32_t row = row0 + mt * 32 + rr;
        u32x4_t t = *reinterpret_cast<const u32x4_t*>(patch + rr * kPatchRow + ch);
        if (!kFull && row >= M) continue;
        if (EPI == 1) {
          if (!SWIGLU && act != F3D_ACT_NONE) {
#pragma unroll
            for (int e = 0; e < 4; ++e) t[e] = pack_bf16x2(xs_act(bf16_lo(t[e]), act), xs_act(bf16_hi(t[e]), act));
          }
          if (residual) {
            const u32x4_t rres = *reinterpret_cast<const u32x4_t*>(residual + (size_t)row * ldr + colbase + ch);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              t[e] = pack_bf16x2(bf16_lo(t[e]) + bf16_lo(rres[e]), bf16_hi(t[e]) + bf16_hi(rres[e]));
          }
        }
        *reinterpret_cast<u32x4_t*>(y + (size_t)row * ldy + colbase + ch) = t;
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
              *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
            }
            flush_tile(full_tag, mt, col0 + nt * 32);
          }
        } else {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            float hv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              // fc1 output is bf16 before the gated activation
              const uint32_t vg = pack_bf16x2(acc[0][mt][g * 4 + r], acc[1][mt][g * 4 + r]);
              hv[r] = fast_silu(bf16_lo(vg)) * bf16_hi(vg);
            }
            uint2 pk;
            pk.x = pack_bf16x2(hv[0], hv[1]);
            pk.y = pack_bf16x2(hv[2], hv[3]);
            *reinterpret_cast<uint2*>(patch + lq * kPatchRow + g * 8 + half * 4) = pk;
          }
          flush_tile(full_tag, mt, col0);
        }
      }
    };
    if (wg_full) epilogue(std::true_type{}); else epilogue(std::false_type{});
    __syncthreads();
  };
  for (uint32_t c = 0; c < nchunk; c += 2) {
    chunk_body(std::false_type{}, c);
    if (c + 1 < nchunk) chunk_body(std::true_type{}, c + 1);
  }
}

template <int K, int MT>
static void launch_k(bool ln_in, bool swiglu, dim3 grid, size_t lds, hipStream_t s, const uint16_t* x, uint32_t ldx,
                     const uint16_t* gamma, const uint16_t* beta, float eps, const uint16_t* w, const uint16_t* bias,
                     const uint16_t* residual, uint32_t ldr, uint16_t* y, uint32_t ldy, uint32_t M, uint32_t N,
                     uint32_t act) {
  const bool general = act != F3D_ACT_NONE || residual != nullptr;
#define F3D_XS(L, S)                                                                                                  \
  do {                                                                                                                \
    if (general)                                                                                                      \
      hipLaunchKernelGGL((xstat_linear_kernel<K, MT, L, S, 1>), grid, dim3(kXsThreads), lds, s, x, ldx, gamma, beta,   \
                         eps, w, bias, residual, ldr, y, ldy, M, N, act);                                             \
    else                                                                                                              \
      hipLaunchKernelGGL((xstat_linear_kernel<K, MT, L, S, 0>), grid, dim3(kXsThreads), lds, s, x, ldx, gamma, beta,   \
                         eps, w, bias, residual, ldr, y, ldy, M, N, act);                                             \
  } while (0)
  constexpr bool kLnOk = K <= 256;
  const bool ln = ln_in && kLnOk;
  if (ln && swiglu) F3D_XS(kLnOk, true);
  else if (ln) F3D_XS(kLnOk, false);
  else if (swiglu) F3D_XS(false, true);
  else F3D_XS(false, false);
#undef F3D_XS
}

// Returns false when the shape is not covered (the caller then uses the tiled GEMM).
bool launch_xstat_linear(const uint16_t* x, uint32_t ldx, const uint16_t* gamma, const uint16_t* beta, float eps,
                         const uint16_t* w, const uint16_t* bias, const uint16_t* residual, uint32_t ldr, uint16_t* y,
                         uint32_t ldy, uint32_t M, uint32_t N, uint32_t K, uint32_t act, hipStream_t s) {
  const bool ln = gamma != nullptr;
  const bool swiglu = act == F3D_ACT_SWIGLU;
  const uint32_t run_act = swiglu ? (uint32_t)F3D_ACT_NONE : act;
  if (M == 0) return true;
  if (N % 64 != 0) return false;     // chunks of 64 output features (32 value + 32 gate for swiglu) must be full
  if (ln && K == 512) return false;  // 128 row values per lane plus the fp32 statistics do not fit the register file
  // One 32-row tile per wave (MT = 1) leaves room for two workgroups per CU, which measured faster than
  // MT = 2 at every shape of the model; F3D_XS_MT=2 selects the larger panel for experiments.
  static const int mt_env = getenv("F3D_XS_MT") ? atoi(getenv("F3D_XS_MT")) : 1;
#define F3D_XS_CASE(KK, MTT)                                                                                        \
  case KK: {                                                                                                        \
    const size_t lds = (size_t)2 * kXsChunk * (KK + 8) * 2;                                                         \
    if (mt_env == 1 || MTT == 1)                                                                                    \
      launch_k<KK, 1>(ln, swiglu, dim3(cdiv_u32(M, 128)), lds, s, x, ldx, gamma, beta, eps, w, bias, residual,      \
                      ldr, y, ldy, M, N, run_act);                                                                  \
    else                                                                                                            \
      launch_k<KK, 2>(ln, swiglu, dim3(cdiv_u32(M, 256)), lds, s, x, ldx, gamma, beta, eps, w, bias, residual,      \
                      ldr, y, ldy, M, N, run_act);                                                                  \
    return true;                                                                                                    \
  }
  switch (K) {
    F3D_XS_CASE(32, 2)
    F3D_XS_CASE(64, 2)
    F3D_XS_CASE(128, 2)
    F3D_XS_CASE(256, 2)
    F3D_XS_CASE(512, 1)
    default: return false;
  }
#undef F3D_XS_CASE
}

}  // namespace f3d
