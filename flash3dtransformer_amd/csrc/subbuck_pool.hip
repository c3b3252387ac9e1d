// Sub-bucket pooling for gfx950: the sub-bucket builder (ids, slots, inverse map, mean coordinates)
// and the per-row feature reduce.  Counterpart of local_subbuck_ker and reduce_feat_ker,
// src/psh/batch_psh_subbuck_reduce.cuh:104-298 and :300-359, launched by
// src/psh/batch_subbuck_pooling_dispatcher.cu:119-138.
//
// Builder design: one 1024-thread workgroup per tile of tile_pts = (1024 / S) * S consecutive points
// of one cloud.  The tile is rotated by a per-tile unit quaternion (stateless RNG), quantised inside
// its own bounding box, keyed by the 13-bit z-order cell, and sorted by (cell, position) with an LDS
// counting sort over the 8192 cells, as the reference does (shmem_cumsum_counter.cuh:25-167), made
// deterministic: the atomic claim only yields a point's place inside its cell's run in arbitration
// order; a second look at the run (almost always one or two points long) replaces it by the number of
// run members that come earlier in the input.  Consecutive runs of S sorted points form a
// sub-bucket.  Tile t owns output rows [t * tile_pts / S, ...) of its cloud, so no global counter
// is needed.  Every output is a pure function of (coords, seps, S, seed).
#include "f3d_device.h"
#include "f3d_internal.h"
#include "row_norm.h"

namespace f3d {

constexpr int kSubThreads = 1024;

// rotation by unit quaternion (w, x, y, z), every product and sum rounded separately: the nine coefficients ...
__device__ __forceinline__ void quat_matrix(const float q[4], float m[9]) {
  const float w = q[0], x = q[1], y = q[2], z = q[3];
  const float n1 = __fmul_rn(x, 2.0f), n2 = __fmul_rn(y, 2.0f), n3 = __fmul_rn(z, 2.0f);
  const float n4 = __fmul_rn(x, n1), n5 = __fmul_rn(y, n2), n6 = __fmul_rn(z, n3);
  const float n7 = __fmul_rn(x, n2), n8 = __fmul_rn(x, n3), n9 = __fmul_rn(y, n3);
  const float n10 = __fmul_rn(w, n1), n11 = __fmul_rn(w, n2), n12 = __fmul_rn(w, n3);
  m[0] = __fsub_rn(1.0f, __fadd_rn(n5, n6));
  m[1] = __fsub_rn(n7, n12);
  m[2] = __fadd_rn(n8, n11);
  m[3] = __fadd_rn(n7, n12);
  m[4] = __fsub_rn(1.0f, __fadd_rn(n4, n6));
  m[5] = __fsub_rn(n9, n10);
  m[6] = __fsub_rn(n8, n11);
  m[7] = __fadd_rn(n9, n10);
  m[8] = __fsub_rn(1.0f, __fadd_rn(n4, n5));
}

// ... and their application to a point
__device__ __forceinline__ void matrix_rotate(const float m[9], const float p[3], float out[3]) {
#pragma unroll
  for (int d = 0; d < 3; ++d)
    out[d] = __fadd_rn(__fadd_rn(__fmul_rn(m[3 * d], p[0]), __fmul_rn(m[3 * d + 1], p[1])), __fmul_rn(m[3 * d + 2], p[2]));
}

// Monotone 16-bit key of an fp16 bit pattern (a < b as numbers <=> key(a) < key(b) as unsigned) and its inverse
__device__ __forceinline__ uint32_t half_order_key(uint32_t h) { return (h & 0x8000u) ? (~h & 0xFFFFu) : (h | 0x8000u); }
__device__ __forceinline__ uint32_t half_from_key(uint32_t k) { return (k & 0x8000u) ? (k & 0x7FFFu) : (~k & 0xFFFFu); }

typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
// minimum of both 16-bit halves at once
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}

// Per-tile unit quaternion, one component per lane (lane % 4), so that the four draws, squares and divisions of the
// rotation cost a wave one pass instead of four; every lane ends up with all four components.
__device__ __forceinline__ void tile_quat_lanes(uint32_t seed, uint32_t cloud, uint32_t tile, uint32_t lane, float q[4]) {
  const float mine = __fadd_rn(0.1f, __fmul_rn(rng_u01(seed, cloud, tile, lane & 3u), 0.9f));
  float c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), i));
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __fadd_rn(acc, __fmul_rn(c[i], c[i]));
  const float unit = __fdiv_rn(mine, __fsqrt_rn(acc));
#pragma unroll
  for (int i = 0; i < 4; ++i) q[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, unit), i));
}

// acc[d] += x[d] of the lane s above, s = 1 .. S - 1 in this order (a sequential sum, as the members are summed one by
// one), for power-of-two groups of at most 16 lanes, which never straddle a row of 16 lanes.  Lane i reads lane i + s of
// its row through a row shift of the operand (DPP); a member past the tile's last point (tid + s >= m) is not added.
template <int SH>
__device__ __forceinline__ float row_up(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + SH, 0xF, 0xF, true));
}
template <int SH, int SMAX>
__device__ __forceinline__ void seq_sum_steps(const float (&x)[3], float (&acc)[3], uint32_t tid, uint32_t m) {
  if constexpr (SH < SMAX) {
    const bool take = tid + SH < m;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      const float v = row_up<SH>(x[d]);
      if (take) acc[d] = __fadd_rn(acc[d], v);
    }
    seq_sum_steps<SH + 1, SMAX>(x, acc, tid, m);
  }
}
__device__ __forceinline__ void seq_sum_row16(const float (&x)[3], float (&acc)[3], uint32_t S, uint32_t tid, uint32_t m) {
  switch (S) {
    case 2: seq_sum_steps<1, 2>(x, acc, tid, m); break;
    case 4: seq_sum_steps<1, 4>(x, acc, tid, m); break;
    case 8: seq_sum_steps<1, 8>(x, acc, tid, m); break;
    case 16: seq_sum_steps<1, 16>(x, acc, tid, m); break;
    default: break;   // S = 1: nothing to add
  }
}


__global__ __launch_bounds__(kSubThreads) void subbuck_build_kernel(
    const uint16_t* __restrict__ coord, const uint32_t* __restrict__ batch_sep,
    const uint32_t* __restrict__ reduced_batch_sep, uint32_t batch_size, uint32_t total_n, uint32_t subbuck_size,
    uint32_t tile_pts, uint32_t num_vox, uint32_t seed, uint32_t* __restrict__ subbuck_id,
    uint16_t* __restrict__ subbuck_off, uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced_coord,
    uint32_t reduced_n, uint32_t reduced_aligned_n) {
  // cell counters, then cell bases: two 16-bit fields per word (a tile has at most 1024 points), plus the end marker
  constexpr uint32_t kCells = 8192u, kCellWords = kCells / 2u, kWaves = kSubThreads / kWave;
  constexpr uint32_t kRunBytes = kWave * 6u, kArea = wave_run_area_bytes<kRunBytes>();
  __shared__ __attribute__((aligned(16))) uint32_t s_cell[kCellWords + 4];
  __shared__ __attribute__((aligned(16))) char s_rows[kWaves * kArea];   // the tile's 6-byte rows, a wave's 64 per area
  __shared__ uint16_t s_claim[kSubThreads];   // run position (arbitration order) -> point
  __shared__ uint16_t s_key[kSubThreads];     // rank (input order inside a run) -> point
  __shared__ uint32_t s_red[kWaves][3];       // per wave: packed keys of the minima and (complemented) maxima
  __shared__ uint32_t s_wsum[kWaves];
  __shared__ float s_mat[9];                  // the tile's rotation
  __shared__ float s_bb[9];                   // min, max, 1 / (max - min) per axis
  const uint32_t tid = threadIdx.x, cloud = blockIdx.y, tile = blockIdx.x;

  if (cloud == batch_size) {  // zero the alignment rows [reduced_n, reduced_aligned_n)
    const uint32_t r = reduced_n + tile * kSubThreads + tid;
    if (r < reduced_aligned_n) {
      uint16_t* q = reduced_coord + 3 * (size_t)r;
      q[0] = 0; q[1] = 0; q[2] = 0;
    }
    return;
  }

  const uint32_t start = cloud ? batch_sep[cloud - 1] : 0u;
  const uint32_t n = batch_sep[cloud] - start;
  const uint32_t rstart = cloud ? reduced_batch_sep[cloud - 1] : 0u;
  const uint32_t t0 = tile * tile_pts;
  if (t0 >= n) return;
  const uint32_t m = min(tile_pts, n - t0);
  const bool valid = tid < m;
  const size_t g = (size_t)start + t0 + tid;
  const uint32_t w = __builtin_amdgcn_readfirstlane(tid / kWave), l = tid % kWave;

  // The wave's 64 rows arrive as aligned 16-byte pieces in its LDS area (rows are 6 bytes apart: per-lane loads would
  // be 2-byte accesses).  64 rows are a multiple of 16 bytes, so every wave's run starts at the same offset of its area.
  const uint32_t wave0 = w * kWave;
  const uint32_t rows = wave0 < m ? min((uint32_t)kWave, m - wave0) : 0u;
  uint32_t shift = (uint32_t)((uintptr_t)(coord + 3 * ((size_t)start + t0)) & 15u);
  if (rows) shift = wave_fetch_run<kRunBytes>(coord + 3 * ((size_t)start + t0 + wave0), rows * 6u, coord + 3 * (size_t)total_n,
                                              s_rows + w * kArea, l);
  auto row_of = [&](uint32_t j) {              // point j of the tile
    return reinterpret_cast<const uint16_t*>(s_rows + (j / kWave) * kArea + shift + 6u * (j % kWave));
  };
  // thread t owns the counters of cells 8 t .. 8 t + 7 (four words) in the zero-fill and in the scan
  uint4* const my_cells = reinterpret_cast<uint4*>(s_cell) + tid;
  *my_cells = make_uint4(0u, 0u, 0u, 0u);
  if (w == 0) {
    // the tile's rotation, once per workgroup
    float q[4], mat[9];
    tile_quat_lanes(seed, cloud, tile, l, q);
    quat_matrix(q, mat);
    if (l < 9u) {
      float mine = mat[0];
#pragma unroll
      for (int i = 1; i < 9; ++i) mine = l == (uint32_t)i ? mat[i] : mine;
      s_mat[l] = mine;
    }
  }
  __syncthreads();
  float p[3] = {0.f, 0.f, 0.f};
  if (valid) {
    const uint16_t* h = row_of(tid);
#pragma unroll
    for (int d = 0; d < 3; ++d) p[d] = half_bits_to_float(h[d]);
  }
  float mat[9], r[3], rh[3];
#pragma unroll
  for (int i = 0; i < 9; ++i) mat[i] = s_mat[i];
  matrix_rotate(mat, p, r);
  // Bounding box of the rotated tile.  The rotated coordinates are fp16 values: as monotone 16-bit keys, two to a
  // register, with the maxima complemented, all six extremes are minima of three registers.
  uint32_t k[3];
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const uint32_t hb = float_to_half_bits(r[d]);
    rh[d] = half_bits_to_float((uint16_t)hb);
    k[d] = half_order_key(hb);
  }
  uint32_t red[3] = {k[0] | (k[1] << 16), k[2] | ((~k[0]) << 16), (~k[1] & 0xFFFFu) | ((~k[2]) << 16)};
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    red[i] = valid ? red[i] : 0xFFFFFFFFu;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) red[i] = pk_min_u16(red[i], __shfl_xor(red[i], off, kWave));
  }
  if (l == 0) {
#pragma unroll
    for (int i = 0; i < 3; ++i) s_red[w][i] = red[i];
  }
  __syncthreads();
  if (w == 0) {
    // the waves' extremes (16 lanes), then per axis the reciprocal of the extent, once per tile
    uint32_t fin[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      fin[i] = s_red[l & 15u][i];
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) fin[i] = pk_min_u16(fin[i], __shfl_xor(fin[i], off, kWave));
    }
    if (l < 3u) {
      const uint32_t kmin = l == 0u ? fin[0] & 0xFFFFu : l == 1u ? fin[0] >> 16 : fin[1] & 0xFFFFu;
      const uint32_t kmax = ~(l == 0u ? fin[1] >> 16 : l == 1u ? fin[2] : fin[2] >> 16) & 0xFFFFu;
      const float a = half_bits_to_float((uint16_t)half_from_key(kmin)), b = half_bits_to_float((uint16_t)half_from_key(kmax));
      s_bb[l] = a;
      s_bb[3u + l] = b;
      s_bb[6u + l] = __fdiv_rn(1.0f, __fsub_rn(b, a));
    }
  }
  __syncthreads();

  // ---- counting sort by cell ----
  uint32_t cell = 0, claim = 0;
  if (valid) {
    uint32_t v[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) v[d] = vox1(rh[d], make_vox_axis_inv(s_bb[d], s_bb[3 + d], s_bb[6 + d], num_vox));
    cell = zorder16(v[0], v[1], v[2]) >> 3;  // H_ZORDER_DIV with divisor 65536 / 8192
    const uint32_t sh = 16u * (cell & 1u);
    claim = (atomicAdd(&s_cell[cell >> 1], 1u << sh) >> sh) & 0xFFFFu;
  }
  __syncthreads();
  {
    // exclusive prefix over the 8192 counts: 8 per thread, then over the threads of a wave, then over the waves
    const uint4 c = *my_cells;
    const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
    uint32_t pre[8], run = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pre[2 * i] = run;
      run += cw[i] & 0xFFFFu;
      pre[2 * i + 1] = run;
      run += cw[i] >> 16;
    }
    uint32_t incl = run;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off, kWave);
      if (l >= (uint32_t)off) incl += up;
    }
    if (l == kWave - 1) s_wsum[w] = incl;
    __syncthreads();
    uint32_t base = incl - run;
    {
      const uint32_t part = l < w ? s_wsum[l] : 0u;        // sum over the waves before this one
      uint32_t tot = part;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) tot += __shfl_xor(tot, off, kWave);
      base += __builtin_amdgcn_readfirstlane(tot);
    }
    *my_cells = make_uint4((base + pre[0]) | ((base + pre[1]) << 16), (base + pre[2]) | ((base + pre[3]) << 16),
                           (base + pre[4]) | ((base + pre[5]) << 16), (base + pre[6]) | ((base + pre[7]) << 16));
    if (tid == kSubThreads - 1) s_cell[kCellWords] = m;   // "base" of the cell after the last one
  }
  __syncthreads();
  uint32_t run0 = 0, run1 = 0;
  if (valid) {
    run0 = (s_cell[cell >> 1] >> (16u * (cell & 1u))) & 0xFFFFu;
    run1 = (s_cell[(cell + 1u) >> 1] >> (16u * ((cell + 1u) & 1u))) & 0xFFFFu;
    s_claim[run0 + claim] = (uint16_t)tid;
  }
  __syncthreads();
  const uint32_t S = subbuck_size;
  const uint32_t rows_per_tile = tile_pts / S;
  const uint32_t row_base = rstart + tile * rows_per_tile;
  const bool pow2 = (S & (S - 1u)) == 0u;
  const uint32_t s_log = 31u - (uint32_t)__builtin_clz(S);
  if (valid) {
    // place inside the run = number of its members that come earlier in the input
    uint32_t before = 0;
    if (run1 - run0 > 1u)
      for (uint32_t j = run0; j < run1; ++j) before += (uint32_t)s_claim[j] < tid ? 1u : 0u;
    const uint32_t rank = run0 + before;
    s_key[rank] = (uint16_t)tid;
    // the point's own outputs, written by the point's thread: consecutive addresses
    const uint32_t sub = pow2 ? rank >> s_log : rank / S;
    subbuck_id[g] = tile * rows_per_tile + sub;
    subbuck_off[g] = (uint16_t)(rank - sub * S);
  }
  __syncthreads();

  // thread `tid` now stands for rank `tid`
  const uint32_t key = valid ? s_key[tid] : 0u;
  if (valid) unpool_ind[(size_t)row_base * S + tid] = (uint32_t)((size_t)start + t0 + key);
  // mean coordinate of every sub-bucket, members summed in rank order
  if (pow2 && S <= (uint32_t)kWave) {
    // a sub-bucket's ranks are neighbouring lanes of one wave: its first lane adds the others' coordinates one by one
    float x[3] = {0.f, 0.f, 0.f}, acc[3];
    if (valid) {
      const uint16_t* h = row_of(key);
#pragma unroll
      for (int d = 0; d < 3; ++d) x[d] = half_bits_to_float(h[d]);
    }
#pragma unroll
    for (int d = 0; d < 3; ++d) acc[d] = __fadd_rn(0.f, x[d]);
    if (S <= 16u) {
      // the group lies inside one row of 16 lanes: the neighbour s lanes up arrives through the data-parallel
      // primitive of the adder's operand (one instruction per member and coordinate, no LDS permute)
      seq_sum_row16(x, acc, S, tid, m);
    } else {
      for (uint32_t s = 1; s < S; ++s) {
        const bool take = tid + s < m;
#pragma unroll
        for (int d = 0; d < 3; ++d) {
          const float v = __shfl_down(x[d], s, kWave);
          if (take) acc[d] = __fadd_rn(acc[d], v);
        }
      }
    }
    if (valid && (tid & (S - 1u)) == 0u) {
      const uint32_t sub = tid >> s_log;
      const uint32_t cnt = min(S, m - tid);
      uint16_t* out = reduced_coord + 3 * (size_t)(row_base + sub);
      if (cnt == S) {
        // a full group: S is a power of two, so the division is an exact scaling (sums of fp16 values are far from
        // the subnormal range of fp32)
        const float inv_s = __builtin_bit_cast(float, (127u - s_log) << 23);
#pragma unroll
        for (int d = 0; d < 3; ++d) out[d] = float_to_half_bits(__fmul_rn(acc[d], inv_s));
      } else {
#pragma unroll
        for (int d = 0; d < 3; ++d) out[d] = float_to_half_bits(__fdiv_rn(acc[d], (float)cnt));
      }
    }
  } else {
    const uint32_t nrow = (m + S - 1) / S;
    if (tid < nrow) {
      const uint32_t cnt = min(S, m - tid * S);
      float acc[3] = {0.f, 0.f, 0.f};
      for (uint32_t s = 0; s < cnt; ++s) {
        const uint16_t* h = row_of(s_key[tid * S + s]);
#pragma unroll
        for (int d = 0; d < 3; ++d) acc[d] = __fadd_rn(acc[d], half_bits_to_float(h[d]));
      }
      uint16_t* out = reduced_coord + 3 * (size_t)(row_base + tid);
#pragma unroll
      for (int d = 0; d < 3; ++d) out[d] = float_to_half_bits(__fdiv_rn(acc[d], (float)cnt));
    }
  }
}

// ---- feature reduce ------------------------------------------------------------------------------
// One thread per (reduced row, 8-channel chunk): S gathered 16-byte loads, fp32 accumulate in slot
// order, one 16-byte store.  A row of C channels is covered by C/8 neighbouring lanes, so every
// gathered row is read as one contiguous burst.

struct alignas(16) Bf16x8 {
  uint16_t v[8];
};

template <int OP>
__device__ __forceinline__ float red_init() {
  return OP == F3D_O_MIN ? INFINITY : OP == F3D_O_MAX ? -INFINITY : 0.f;
}

template <int OP>
__device__ __forceinline__ float red_step(float acc, float v) {
  if (OP == F3D_O_MIN) return (v < acc) ? v : acc;
  if (OP == F3D_O_MAX) return (v > acc) ? v : acc;
  return __fadd_rn(acc, v);
}

// NORM: the reduced row (alignment rows included, as a norm layer applied to the whole tensor would) is normalised by
// the lanes that hold it before it is stored (row_norm.h).
template <int OP, bool NORM>
__global__ __launch_bounds__(256) void reduce_feat_vec8_kernel(
    const uint16_t* __restrict__ feat, const uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced,
    uint32_t total_n, uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t chunks_per_row, uint32_t S, RowNorm norm) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / chunks_per_row);
  const uint32_t chunk = (uint32_t)(gid - (size_t)row * chunks_per_row);
  if (row >= reduced_aligned_n) return;
  const uint32_t C = chunks_per_row * 8;
  Bf16x8 out;
  if (row >= reduced_n) {
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = 0;
  } else {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = red_init<OP>();
    uint32_t cnt = 0;
    const uint32_t* ind = unpool_ind + (size_t)row * S;
    for (uint32_t s = 0; s < S; ++s) {
      const uint32_t src = ind[s];
      if (src < total_n) {
        ++cnt;
        const Bf16x8 x = *reinterpret_cast<const Bf16x8*>(feat + (size_t)src * C + chunk * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = red_step<OP>(acc[i], bf16_bits_to_float(x.v[i]));
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float a = acc[i];
      if (OP == F3D_O_MEAN) a = __fdiv_rn(a, (float)cnt);
      if (cnt == 0) a = 0.f;
      out.v[i] = float_to_bf16_bits(a);
    }
  }
  if (NORM) {
    const u32x4_t v = row_norm_chunk(__builtin_bit_cast(u32x4_t, out), norm, chunk, chunks_per_row);
    *reinterpret_cast<u32x4_t*>(reduced + (size_t)row * C + chunk * 8) = v;
  } else {
    *reinterpret_cast<Bf16x8*>(reduced + (size_t)row * C + chunk * 8) = out;
  }
}

// any channel count: one thread per (row, channel)
template <int OP>
__global__ __launch_bounds__(256) void reduce_feat_scalar_kernel(
    const uint16_t* __restrict__ feat, const uint32_t* __restrict__ unpool_ind, uint16_t* __restrict__ reduced,
    uint32_t total_n, uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t C, uint32_t S) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = (uint32_t)(gid / C);
  const uint32_t c = (uint32_t)(gid - (size_t)row * C);
  if (row >= reduced_aligned_n) return;
  float a = 0.f;
  if (row < reduced_n) {
    a = red_init<OP>();
    uint32_t cnt = 0;
    for (uint32_t s = 0; s < S; ++s) {
      const uint32_t src = unpool_ind[(size_t)row * S + s];
      if (src < total_n) {
        ++cnt;
        a = red_step<OP>(a, bf16_bits_to_float(feat[(size_t)src * C + c]));
      }
    }
    if (OP == F3D_O_MEAN) a = __fdiv_rn(a, (float)cnt);
    if (cnt == 0) a = 0.f;
  }
  reduced[(size_t)row * C + c] = float_to_bf16_bits(a);
}

template <int OP>
static void launch_reduce(const uint16_t* feat, const uint32_t* unpool_ind, uint16_t* reduced, uint32_t total_n,
                          uint32_t reduced_n, uint32_t reduced_aligned_n, uint32_t C, uint32_t S, const RowNorm* norm,
                          hipStream_t s) {
  const bool vec = (C % 8 == 0) && (((uintptr_t)feat | (uintptr_t)reduced) % 16 == 0);
  if (vec) {
    const size_t total = (size_t)reduced_aligned_n * (C / 8);
    if (norm)
      hipLaunchKernelGGL((reduce_feat_vec8_kernel<OP, true>), dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, feat,
                         unpool_ind, reduced, total_n, reduced_n, reduced_aligned_n, C / 8, S, *norm);
    else
      hipLaunchKernelGGL((reduce_feat_vec8_kernel<OP, false>), dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, feat,
                         unpool_ind, reduced, total_n, reduced_n, reduced_aligned_n, C / 8, S, RowNorm{});
  } else {
    const size_t total = (size_t)reduced_aligned_n * C;
    hipLaunchKernelGGL(reduce_feat_scalar_kernel<OP>, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, feat,
                       unpool_ind, reduced, total_n, reduced_n, reduced_aligned_n, C, S);
  }
}

}  // namespace f3d

extern "C" {

int f3d_subbuck_build(const f3d_half_t* coord, const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n,
                      uint32_t instance_max_n, uint32_t subbuck_size, uint32_t num_vox, uint32_t* subbuck_id,
                      uint16_t* subbuck_off, const uint32_t* reduced_batch_sep, f3d_half_t* reduced_coord,
                      uint32_t reduced_aligned_n, uint32_t* unpool_ind, uint32_t reduced_n, int device,
                      void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(subbuck_size >= 1 && subbuck_size <= 1024, "subbuck_size=%u outside [1, 1024]", subbuck_size);
  F3D_CHECK_ARG(num_vox >= 2 && num_vox <= 0x10000u, "num_vox=%u does not fit the 16-bit voxel type", num_vox);
  F3D_CHECK_ARG(reduced_aligned_n >= reduced_n, "reduced buffer length(%u) is smaller than the reduced row count(%u)",
                reduced_aligned_n, reduced_n);
  F3D_CHECK_ARG(coord && batch_sep && subbuck_id && subbuck_off && reduced_batch_sep && reduced_coord && unpool_ind,
                "null tensor pointer");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  const uint32_t tile_pts = (1024u / subbuck_size) * subbuck_size;
  const uint32_t max_tiles = cdiv_u32(instance_max_n, tile_pts);
  const uint32_t pad_tiles = cdiv_u32(reduced_aligned_n - reduced_n, kSubThreads);
  const uint32_t gx = max_tiles > pad_tiles ? max_tiles : pad_tiles;
  if (gx == 0 || (batch_size == 0 && pad_tiles == 0)) return F3D_OK;
  SyncBracket sync(s);
  hipLaunchKernelGGL(subbuck_build_kernel, dim3(gx, batch_size + (pad_tiles ? 1 : 0)), dim3(kSubThreads), 0, s, coord,
                     batch_sep, reduced_batch_sep, batch_size, total_n, subbuck_size, tile_pts, num_vox | quantiser_bit(),
                     global_seed(),
                     subbuck_id, subbuck_off, unpool_ind, reduced_coord, reduced_n, reduced_aligned_n);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

static int reduce_feat_impl(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                            uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                            uint32_t reduced_aligned_n, const f3d::RowNorm* norm, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(red_op <= 3, "Unsupported reduction operation id-%u", red_op);
  F3D_CHECK_ARG(reduced_aligned_n >= reduced_n, "reduced buffer length(%u) is smaller than the reduced row count(%u)",
                reduced_aligned_n, reduced_n);
  F3D_CHECK_ARG(feat && unpool_ind && reduced_feat, "null tensor pointer");
  if (reduced_aligned_n == 0 || feat_dim == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  switch (red_op) {
    case F3D_O_MEAN: launch_reduce<F3D_O_MEAN>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, norm, s); break;
    case F3D_O_SUM: launch_reduce<F3D_O_SUM>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, norm, s); break;
    case F3D_O_MIN: launch_reduce<F3D_O_MIN>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, norm, s); break;
    default: launch_reduce<F3D_O_MAX>(feat, unpool_ind, reduced_feat, total_n, reduced_n, reduced_aligned_n, feat_dim, subbuck_size, norm, s); break;
  }
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_reduce_feat(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                    uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                    uint32_t reduced_aligned_n, int device, void* stream) {
  return reduce_feat_impl(feat, total_n, feat_dim, unpool_ind, reduced_n, subbuck_size, red_op, reduced_feat,
                          reduced_aligned_n, nullptr, device, stream);
}

int f3d_reduce_feat_norm(const f3d_bf16_t* feat, uint32_t total_n, uint32_t feat_dim, const uint32_t* unpool_ind,
                         uint32_t reduced_n, uint32_t subbuck_size, uint32_t red_op, f3d_bf16_t* reduced_feat,
                         uint32_t reduced_aligned_n, uint32_t norm_mode, const f3d_bf16_t* gamma, const f3d_bf16_t* beta,
                         const float* scale, const float* shift, float eps, uint32_t act, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(norm_mode == kRowNormLayer || norm_mode == kRowNormAffine, "unknown row normalisation %u", norm_mode);
  F3D_CHECK_ARG(norm_mode == kRowNormLayer ? gamma != nullptr : (scale != nullptr && shift != nullptr),
                "null normalisation parameter");
  F3D_CHECK_ARG(act <= F3D_ACT_RELU && act != F3D_ACT_SWIGLU && (norm_mode == kRowNormAffine || act == F3D_ACT_NONE),
                "unsupported activation id %u for normalisation %u", act, norm_mode);
  if (!row_norm_supported(norm_mode, feat_dim) ||
      (((uintptr_t)feat | (uintptr_t)reduced_feat | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)scale | (uintptr_t)shift) & 15u)) {
    set_error("No fused normalisation for %u channels (a multiple of 8; LayerNorm: 8 x a power of two up to 512; "
              "16-byte aligned tensors)", feat_dim);
    return F3D_ERR_UNSUPPORTED;
  }
  const RowNorm norm{norm_mode, gamma, beta, scale, shift, eps, act};
  return reduce_feat_impl(feat, total_n, feat_dim, unpool_ind, reduced_n, subbuck_size, red_op, reduced_feat,
                          reduced_aligned_n, &norm, device, stream);
}

int f3d_batch_subbuck_reduce(const f3d_half_t* scattered_coord, const f3d_bf16_t* scattered_feat,
                             const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n,
                             uint32_t instance_max_n, uint32_t feat_dim, uint32_t subbuck_size, uint32_t num_vox,
                             const f3d_half_t* bbox_min, const f3d_half_t* bbox_max, uint32_t* subbuck_id,
                             uint16_t* subbuck_off, const uint32_t* reduced_batch_sep, f3d_half_t* reduced_coord,
                             f3d_bf16_t* reduced_feat, uint32_t reduced_aligned_n, uint32_t* unpool_ind,
                             uint32_t reduced_n, uint32_t hash_type, uint32_t red_op, int device, void* stream) {
  // bbox_* and hash_type are part of the reference signature; its kernel quantises inside each
  // block's own box with the z-order hash regardless of them (dispatcher :108-109).
  (void)bbox_min; (void)bbox_max; (void)hash_type;
  F3D_CHECK_ARG(red_op <= 3, "Unsupported reduction operation id-%u", red_op);
  int rc = f3d_subbuck_build(scattered_coord, batch_sep, batch_size, total_n, instance_max_n, subbuck_size, num_vox,
                             subbuck_id, subbuck_off, reduced_batch_sep, reduced_coord, reduced_aligned_n, unpool_ind,
                             reduced_n, device, stream);
  if (rc != F3D_OK) return rc;
  return f3d_reduce_feat(scattered_feat, total_n, feat_dim, unpool_ind, reduced_n, subbuck_size, red_op, reduced_feat,
                         reduced_aligned_n, device, stream);
}

}  // extern "C"
