// Measurement aids of bench.py (built into bench_probe.so beside it; not part of libf3d_hip.so and of no use to a
// caller of the library).
//
// bench_probe_mfma_bf16: the rate at which the matrix cores of this GPU retire dense v_mfma_f32_32x32x16_bf16 products
// when nothing else runs (operands in registers, eight independent accumulators per wave, four waves per SIMD), and the
// shader clock they run at meanwhile.  With random operands the chip's power budget, not the issue rate, sets the
// clock; with a zero operand the multipliers do not toggle and the rate is the 2.5 PFLOP/s of the data sheet.  Every
// workgroup's first lane reads the shader-clock counter and the 100 MHz constant-rate counter at its start and end:
// their ratio is the clock the products ran at.
//
// bench_probe_issue: what the vector issue port of a SIMD takes per instruction of the attention forward's inner step
// (32 x 32 scores): 16 v_exp_f32, 8 v_cvt_pk_bf16_f32, four 32x32x16 and two 16x16x32 bf16 MFMAs, each kind alone and
// all of them together with the dependencies of the real step (exponentials of the previous score product, packed
// values feeding the P V^T and row-sum products), on register operands with no memory or LDS instruction, four
// waves per SIMD.  The mixed mode is the floor of the attention kernels at 32-wide heads in shader clocks per block.
//
// bench_probe_store_rows: what HBM takes when a [m][n] bf16 output is written the way the row-panel linear layers write
// it: workgroups of eight waves own 512 rows, walk the 64-column chunks in rotated order, and a wave stores its 64 rows
// of a chunk in row-contiguous pieces of 64 bytes (4 lanes per row, 16 rows per instruction) or 128 bytes (8 lanes per
// row, 8 rows per instruction), with or without a pause per chunk that stands for the products between two
// epilogues.  The write roof those layers sit under.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ sink, uint64_t* __restrict__ clocks,
                                                         uint32_t iters, uint32_t random_a, uint32_t random_b) {
  uint32_t h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h = h * 1664525u + 1013904223u;
      a[i][e] = (__bf16)(random_a ? ((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f : 0.f);
      h = h * 1664525u + 1013904223u;
      b[i][e] = (__bf16)(random_b ? ((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f : 0.f);
    }
  f32x16_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  const uint64_t c0 = clock64(), w0 = wall_clock64();
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j & 3], b[(j + 1) & 3], acc[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[j][i];
  const uint64_t c1 = clock64(), w1 = wall_clock64();
  if (s == 123.456f) sink[0] = s;   // keeps the products alive; never true for these operands
  if (clocks && threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

// MODE 0: 16 v_exp_f32 per iteration, 1: 8 v_cvt_pk_bf16_f32, 2: four 32x32x16 + two 16x16x32 products,
// 3: all of them, chained as in the attention step
template <int MODE>
__global__ __launch_bounds__(1024) void probe_issue_kernel(float* __restrict__ sink, uint64_t* __restrict__ clocks,
                                                           uint32_t iters) {
  uint32_t h = (blockIdx.x * 1024u + threadIdx.x) * 2654435761u;
  bf16x8_t kq[4], vv[2], ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      h = h * 1664525u + 1013904223u;
      kq[i][e] = (__bf16)(((int)((h >> 8) & 0xFFFFu) - 32768) / 262144.0f);     // |score| stays well under 1
    }
    h = h * 1664525u + 1013904223u;
    vv[0][e] = (__bf16)(((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f);
    h = h * 1664525u + 1013904223u;
    vv[1][e] = (__bf16)(((int)((h >> 8) & 0xFFFFu) - 32768) / 32768.0f);
    ones[e] = (__bf16)((threadIdx.x & 8u) ? 1.0f : 0.0f);
  }
  f32x16_t acc, sc;
  f32x4_t lacc = {0.f, 0.f, 0.f, 0.f};
  float x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc[i] = 0.f;
    sc[i] = (float)(threadIdx.x & 7u) * 0.01f;
    x[i] = (float)((threadIdx.x + i) & 15u) * 0.01f;
  }
  uint32_t pb[8] = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  f32x16_t sc2 = sc;
  auto block = [&](const f32x16_t& cur, f32x16_t& nxt) {
#pragma unroll
    for (int i = 0; i < 16; ++i) nxt[i] = 0.f;
    asm volatile("" : "+v"(kq[0]), "+v"(kq[2]));    // new K fragments every block as far as the compiler knows
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kq[0], kq[1], nxt, 0, 0, 0);
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kq[2], kq[3], nxt, 0, 0, 0);
    if constexpr (MODE == 3) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        pb[i] = __builtin_bit_cast(uint32_t, bf16x2_t{(__bf16)__builtin_amdgcn_exp2f(cur[2 * i]),
                                                      (__bf16)__builtin_amdgcn_exp2f(cur[2 * i + 1])});
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const probe_u32x4 praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
      const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vv[kk], pf, acc, 0, 0, 0);
      lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf, lacc, 0, 0, 0);
    }
  };
  const uint64_t c0 = clock64(), w0 = wall_clock64();
  for (uint32_t it = 0; it < iters; it += (MODE >= 2 ? 2u : 1u)) {
    if constexpr (MODE == 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) x[i] = __builtin_amdgcn_exp2f(-__builtin_fabsf(x[i]));   // source modifiers: one instruction; stays in (0, 1]
    } else if constexpr (MODE == 1) {
      // operands the compiler must take as new every trip, results it must take as used: eight bare conversions
      asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]));
      asm volatile("" : "+v"(x[8]), "+v"(x[9]), "+v"(x[10]), "+v"(x[11]), "+v"(x[12]), "+v"(x[13]), "+v"(x[14]), "+v"(x[15]));
#pragma unroll
      for (int i = 0; i < 8; ++i) pb[i] = __builtin_bit_cast(uint32_t, bf16x2_t{(__bf16)x[2 * i], (__bf16)x[2 * i + 1]});
      asm volatile("" ::"v"(pb[0]), "v"(pb[1]), "v"(pb[2]), "v"(pb[3]), "v"(pb[4]), "v"(pb[5]), "v"(pb[6]), "v"(pb[7]));
    } else {
      // two blocks per trip with the score registers swapped by name (no copies); the next block's scores start
      // before this block's exponentials, as in the kernels
      block(sc, sc2);
      block(sc2, sc);
    }
  }
  float s = lacc[0] + lacc[1] + lacc[2] + lacc[3];
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i] + sc[i] + sc2[i] + x[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += (float)pb[i];
  const uint64_t c1 = clock64(), w1 = wall_clock64();
  if (s == 123.456f) sink[0] = s;   // keeps the work alive; never true for these operands
  if (clocks && (threadIdx.x & 63u) == 0) {
    clocks[2 * (blockIdx.x * 16u + threadIdx.x / 64u)] = c1 - c0;
    clocks[2 * (blockIdx.x * 16u + threadIdx.x / 64u) + 1] = w1 - w0;
  }
}

template <int PIECE>
__global__ __launch_bounds__(512) void probe_store_rows_kernel(uint16_t* __restrict__ y, uint32_t ldy, uint32_t m, uint32_t n,
                                                              uint32_t pause) {
  const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const uint32_t nchunk = n / 64, c0 = (blockIdx.x * 5u) % nchunk;
  const uint32_t row_w = blockIdx.x * 512 + wave * 64;
  const probe_u32x4 v = {lane, wave, blockIdx.x, 7u};
  constexpr uint32_t LPR = PIECE / 16, RPI = 64 / LPR;   // lanes per row, rows per instruction
  for (uint32_t i = 0; i < nchunk; ++i) {
    const uint32_t c = (i + c0) % nchunk;
    for (uint32_t p = 0; p < pause; ++p) __builtin_amdgcn_s_sleep(1);
#pragma unroll
    for (uint32_t piece = 0; piece < 128 / PIECE; ++piece)
#pragma unroll
      for (uint32_t r0 = 0; r0 < 64; r0 += RPI) {
        const uint32_t row = row_w + r0 + lane / LPR, col = c * 64 + piece * (PIECE / 2) + (lane % LPR) * 8;
        if (row < m) *reinterpret_cast<probe_u32x4*>(y + ((size_t)row * ldy + col)) = v;
      }
  }
}

extern "C" {

// Writes all of y[m][n] (bf16, row stride ldy elements, n a multiple of 64) in pieces of piece_bytes (64 or 128) per
// row and instruction, `pause` s_sleep instructions per chunk.  Returns 0, -1 for bad arguments, or the HIP error code.
int bench_probe_store_rows(uint16_t* y, uint32_t ldy, uint32_t m, uint32_t n, uint32_t piece_bytes, uint32_t pause,
                           void* stream) {
  if (!y || m == 0 || n == 0 || n % 64 != 0 || ldy < n || ldy % 8 != 0 || (piece_bytes != 64 && piece_bytes != 128)) return -1;
  const dim3 grid((m + 511) / 512), block(512);
  if (piece_bytes == 64) hipLaunchKernelGGL(probe_store_rows_kernel<64>, grid, block, 0, (hipStream_t)stream, y, ldy, m, n, pause);
  else hipLaunchKernelGGL(probe_store_rows_kernel<128>, grid, block, 0, (hipStream_t)stream, y, ldy, m, n, pause);
  return (int)hipGetLastError();
}

// workgroups x 4 waves x iters x 8 products of 32,768 flops.  sink: one float of device memory (never written);
// clocks: 2 x workgroups uint64 of device memory (shader-clock ticks, 100 MHz ticks per workgroup) or NULL.
// Returns 0, or the HIP error code of the launch.
int bench_probe_mfma_bf16(uint32_t workgroups, uint32_t iters, uint32_t random_a, uint32_t random_b, float* sink,
                          uint64_t* clocks, void* stream) {
  if (!sink || workgroups == 0 || workgroups > 65536u || iters > (1u << 24)) return -1;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, sink, clocks, iters,
                     random_a, random_b);
  return (int)hipGetLastError();
}

// mode 0 .. 3 as described at the top; workgroups of 16 waves (four per SIMD when one workgroup sits on a CU).
// clocks: 2 x 16 x workgroups uint64 (shader-clock ticks, 100 MHz ticks per wave).  Returns 0, -1, or the HIP error code.
int bench_probe_issue(uint32_t mode, uint32_t workgroups, uint32_t iters, float* sink, uint64_t* clocks, void* stream) {
  if (!sink || !clocks || mode > 3u || workgroups == 0 || workgroups > 65536u || iters > (1u << 24)) return -1;
  const dim3 grid(workgroups), block(1024);
  hipStream_t s = (hipStream_t)stream;
  switch (mode) {
    case 0: hipLaunchKernelGGL(probe_issue_kernel<0>, grid, block, 0, s, sink, clocks, iters); break;
    case 1: hipLaunchKernelGGL(probe_issue_kernel<1>, grid, block, 0, s, sink, clocks, iters); break;
    case 2: hipLaunchKernelGGL(probe_issue_kernel<2>, grid, block, 0, s, sink, clocks, iters); break;
    default: hipLaunchKernelGGL(probe_issue_kernel<3>, grid, block, 0, s, sink, clocks, iters); break;
  }
  return (int)hipGetLastError();
}

}  // extern "C"
