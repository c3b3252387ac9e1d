// Bucketed (scoped) multi-head attention backward for gfx950, streaming form: any scope size, head_dim 16 / 32 /
// 64 / 128, optional per-bucket valid lengths.
//
// Same mathematics as buck_swin_bwd.hip (the reference declares the op at src/f3d_frontend.cu:94-97 and ships no
// kernel source; its tests differentiate an SDPA oracle, tests/test_attn_bwd.py: B,L,H,D = 4,8192,4,{64,128} with one
// scope over all buckets, and its model runs buckets of 512 in scopes of 8, tests/test_psh_hourglass.py:56-57).
// With P = softmax(Q Kt / sqrt(D)) recomputed from the saved LSE:
//   Delta = rowsum(dO * O)   dV = Pt dO   dP = dO Vt   dS = P * (dP - Delta)   dQ = dS K / sqrt(D)   dK = dSt Q / sqrt(D)
//
// Three kernels, no atomics (every output row is written by exactly one wave):
//   delta : one lane pair per (row of a scope, head): Delta = rowsum(dO * O).
//   dkdv  : a workgroup of 4 waves owns 128 KEYS of one (batch, scope, head); a wave keeps its 32 keys' K and V rows
//           in registers as MFMA B operands and walks the scope's query tiles (32 queries: Q and dO rows through LDS,
//           direct HBM -> LDS loads, two buffers).  S = Q Kt and dP = dO Vt come out with a lane holding one key and
//           16 queries, so P and dS (bf16) already are the B operands of dVt += dOt P and dKt += Qt dS, whose A
//           operands (dOt, Qt) are read transposed from LDS (ds_read_b64_tr_b16).
//   dq    : a workgroup owns 128 QUERIES (Q, dO rows in registers, LSE and Delta one scalar per lane) and walks the
//           scope's key tiles (K and V rows through LDS); St = K Qt, dPt = V dOt, dQt += Kt dSt with Kt read transposed.
// LDS rows are unpadded with their 16-byte pieces XOR-swizzled, as in the resident kernels.
// Valid lengths (kv_len, may be null): keys at in-bucket position >= kv_len[bucket] have P = 0, and so have query rows
// there (the forward gave them O = 0, LSE = 0): their gradients are zero and they add nothing to dK / dV.
#include <type_traits>
#include <algorithm>
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

constexpr int kStreamWaves = 4;
constexpr int kStreamBlock = 32 * kStreamWaves;   // keys (dkdv) or queries (dq) per workgroup

template <int D>
struct SGeom {
  static constexpr int KSTEPS = D / 16;
  static constexpr int DT = D < 32 ? 1 : D / 32;   // 32-feature output tiles
  static constexpr int CPK = D / 8;                // 16-byte pieces per row
  static constexpr int ROWB = D * 2;               // bytes per row
  static constexpr int RPB = 1024 / ROWB;          // rows one direct-load instruction fills
  static constexpr int BLK = 32 / RPB;             // direct-load instructions per 32-row tile
  static constexpr int SWZ_DIV = 16 / CPK;         // rows sharing one swizzle value
  static constexpr int TILEB = 32 * ROWB;          // bytes of a 32-row tile
};

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds_addr + 16 l.
__device__ __forceinline__ void stream_dma16(const void* gbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

// 32 consecutive rows starting at `grow0` (bytes, uniform) of a tensor with row pitch ld_bytes -> a swizzled LDS
// tile; the BLK direct loads are shared by the workgroup's waves
template <int D>
__device__ __forceinline__ void stream_fill_tile(const char* grow0, uint32_t ld_bytes, uint32_t lds_tile, uint32_t wave,
                                                 uint32_t lane) {
  using G = SGeom<D>;
#pragma unroll
  for (int i = 0; i < (G::BLK + kStreamWaves - 1) / kStreamWaves; ++i) {
    const uint32_t blk = wave + i * kStreamWaves;       // uniform
    if (blk < (uint32_t)G::BLK) {
      const uint32_t r = lane / G::CPK, pos = lane % G::CPK;
      const uint32_t row = blk * G::RPB + r;
      const uint32_t ck = pos ^ ((row / G::SWZ_DIV) & (G::CPK - 1));
      const uint64_t g = (uint64_t)(uintptr_t)grow0 + (uint64_t)blk * G::RPB * ld_bytes;
      const uint64_t gu = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)g) |
                          ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(g >> 32)) << 32);
      stream_dma16(reinterpret_cast<const void*>((uintptr_t)gu), r * ld_bytes + ck * 16u,
                   __builtin_amdgcn_readfirstlane(lds_tile + blk * 1024u));
    }
  }
}

// the lane's byte offset of its 8-byte piece for the transposing reads of feature tile dt: row 4 half + l16 / 4 +
// 8 hi of a 32-row tile, features 32 dt + d_base + 4 (l16 % 4) .. + 3, the row's swizzle applied to the piece index
template <int D>
__device__ __forceinline__ uint32_t stream_tr_offset(uint32_t lane, uint32_t hi, uint32_t dt) {
  using G = SGeom<D>;
  const uint32_t half = lane >> 5, l16 = lane & 15u, d_base = 16u * ((lane >> 4) & 1u);
  const uint32_t row = 4u * half + l16 / 4u + 8u * hi;
  const uint32_t colb = (32u * dt + d_base + 4u * (l16 & 3u)) * 2u;         // byte column, a multiple of 8
  const uint32_t piece = (colb / 16u) ^ ((row / G::SWZ_DIV) & (G::CPK - 1));
  return row * G::ROWB + piece * 16u + (colb & 8u);
}

// A operand read transposed from a swizzled LDS tile of 32 rows: lane (m = feature of tile dt) gets, for k-step kk,
// slots 0..3 = rows 16 kk + 4 half + 0..3 and slots 4..7 = the same + 8 (the order in which an accumulator tile hands
// its rows to the next MFMA as a B operand).  Adding 16 rows leaves a row's swizzle value unchanged.
template <int D>
__device__ __forceinline__ void stream_load_tr(const char* tile, uint32_t tr_lo, uint32_t tr_hi, bool tr_lane,
                                               bf16x8_t (&f)[2]) {
  constexpr int ROWB = SGeom<D>::ROWB;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    i16x4_t lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
    if (tr_lane) {
      lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(tile + tr_lo + (kk * 16) * ROWB));
      hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(tile + tr_hi + (kk * 16) * ROWB));
    }
    f[kk] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  }
}

struct StreamItem {
  uint32_t batch, scope, head, blk;
};
// grid.y holds at most 65535 (batch, scope, head) items: a launch covers items [item0, item0 + gridDim.y)
__device__ __forceinline__ StreamItem stream_item(uint32_t num_scope, uint32_t num_head, uint32_t item0) {
  StreamItem it;
  const uint32_t item = item0 + blockIdx.y;
  it.blk = blockIdx.x;
  it.head = item % num_head;
  it.scope = (item / num_head) % num_scope;
  it.batch = item / (num_head * num_scope);
  return it;
}

// bucket ids and valid lengths of the scope -> LDS; returns false (uniformly) when an id lies outside the sequence:
// such a scope contributes nothing, as in the forward's backward-facing contract
__device__ __forceinline__ bool stream_scope_table(const uint32_t* scope_buckets, const int32_t* kv_len, uint32_t scope,
                                                   uint32_t scope_size, uint32_t bs, uint32_t n_bucket,
                                                   uint32_t* s_bucket, int32_t* s_len) {
  int bad = 0;
  for (uint32_t j = threadIdx.x; j < scope_size; j += blockDim.x) {
    const uint32_t b = scope_buckets[(size_t)scope * scope_size + j];
    s_bucket[j] = b;
    if (b >= n_bucket) bad = 1;
    s_len[j] = b >= n_bucket ? 0 : (kv_len ? min(max(kv_len[b], 0), (int32_t)bs) : (int32_t)bs);
  }
  return __syncthreads_or(bad) == 0;
}

// ---- Delta = rowsum(dO * O) over the rows the scopes cover ----------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const uint16_t* __restrict__ o, const uint16_t* __restrict__ d_o,
                                                        float* __restrict__ delta,
                                                        const uint32_t* __restrict__ scope_buckets, uint32_t num_scope,
                                                        uint32_t scope_size, uint32_t bs, uint32_t seq_len,
                                                        uint32_t num_head, uint32_t y0) {
  // thread -> (scope row, head); y0 + grid.y -> (batch, scope)
  const uint32_t scope = (y0 + blockIdx.y) % num_scope, batch = (y0 + blockIdx.y) / num_scope;
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t head = idx % num_head, loc = idx / num_head;
  if (loc >= scope_size * bs) return;
  const uint32_t b = scope_buckets[(size_t)scope * scope_size + loc / bs];
  if (b >= seq_len / bs) return;
  const size_t row = (size_t)batch * seq_len + (size_t)b * bs + loc % bs;
  const uint16_t* orow = o + (row * num_head + head) * D;
  const uint16_t* drow = d_o + (row * num_head + head) * D;
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < D / 8; ++c) {
    const u32x4_t a = *reinterpret_cast<const u32x4_t*>(orow + c * 8);
    const u32x4_t g = *reinterpret_cast<const u32x4_t*>(drow + c * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s = __builtin_fmaf(bf16_lo(a[e]), bf16_lo(g[e]), s);
      s = __builtin_fmaf(bf16_hi(a[e]), bf16_hi(g[e]), s);
    }
  }
  delta[row * num_head + head] = s;
}

template <int D>
constexpr size_t stream_lds_bytes(uint32_t scope_size) {
  return (size_t)4 * SGeom<D>::TILEB + (size_t)4 * 32 * 4 + (size_t)scope_size * 8;
}

// ---- dK, dV -------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(64 * kStreamWaves) void bwd_dkdv_stream_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    uint16_t* __restrict__ dk, uint16_t* __restrict__ dv, const uint32_t* __restrict__ scope_buckets,
    uint32_t num_scope, uint32_t scope_size, uint32_t bs, uint32_t seq_len, uint32_t num_head,
    const int32_t* __restrict__ kv_len, float scale, float scale_log2, uint32_t ldg, uint32_t item0) {
  using G = SGeom<D>;
  constexpr int KSTEPS = G::KSTEPS, ROWB = G::ROWB, DT = G::DT, TILEB = G::TILEB;
  extern __shared__ __attribute__((aligned(16))) char lds_s[];
  // two buffers of (Q tile, dO tile), then per buffer 32 LSE (exponent units) and 32 Delta, then the scope table
  float* s_lse2 = reinterpret_cast<float*>(lds_s + 4 * TILEB);
  float* s_delta = s_lse2 + 64;
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(s_delta + 64);
  int32_t* s_len = reinterpret_cast<int32_t*>(s_bucket + scope_size);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_s;

  const StreamItem it = stream_item(num_scope, num_head, item0);
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  if (!stream_scope_table(scope_buckets, kv_len, it.scope, scope_size, bs, n_bucket, s_bucket, s_len)) return;

  const uint32_t ldo = num_head * D;   // dO, dK, dV are dense [B, L, H, D]
  const size_t base_qkv = (size_t)it.batch * seq_len * ld + (size_t)it.head * D;
  const size_t base_o = (size_t)it.batch * seq_len * ldo + (size_t)it.head * D;
  const size_t base_l = (size_t)it.batch * seq_len * num_head + it.head;

  // this wave's 32 keys: scope-local rows [128 blk + 32 wave, + 32), lane -> key lq
  const uint32_t kloc0 = it.blk * kStreamBlock + wave * 32u;
  const uint32_t kj = kloc0 / bs, k_in_b0 = kloc0 - kj * bs;
  const uint32_t krow = s_bucket[kj] * bs + k_in_b0 + lq;            // row inside the sequence
  const bool key_ok = (int32_t)(k_in_b0 + lq) < s_len[kj];
  bf16x8_t kf[KSTEPS], vf[KSTEPS];
  {
    const uint16_t* kr = k + base_qkv + (size_t)krow * ld + half * 8;
    const uint16_t* vr = v + base_qkv + (size_t)krow * ld + half * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      kf[ks] = *reinterpret_cast<const bf16x8_t*>(kr + ks * 16);
      vf[ks] = *reinterpret_cast<const bf16x8_t*>(vr + ks * 16);
    }
  }

  const uint32_t n_tiles = scope_size * bs / 32u;
  // query tile t: rows [32 t, 32 t + 32) of the scope, all inside one bucket; Q and dO rows go to buffer t & 1
  auto tile_valid = [&](uint32_t t) -> int32_t {   // valid query rows of the tile (uniform)
    const uint32_t j = (t * 32u) / bs;
    return min(max(s_len[j] - (int32_t)(t * 32u - j * bs), 0), 32);
  };
  auto fill = [&](uint32_t t, uint32_t b) {   // tile t -> buffer b
    const uint32_t j = (t * 32u) / bs;
    const size_t grow = (size_t)__builtin_amdgcn_readfirstlane(s_bucket[j]) * bs + (t * 32u - j * bs);
    const uint32_t buf = lds0 + b * 2u * TILEB;
    stream_fill_tile<D>(reinterpret_cast<const char*>(q + base_qkv + grow * ld), ld * 2u, buf, wave, lane);
    stream_fill_tile<D>(reinterpret_cast<const char*>(d_o + base_o + grow * ldo), ldo * 2u, buf + TILEB, wave, lane);
    if (tid < 32) {
      s_lse2[b * 32 + tid] = lse[base_l + (grow + tid) * num_head] * 1.4426950408889634f;
      s_delta[b * 32 + tid] = delta[base_l + (grow + tid) * num_head];
    }
  };
  auto next_tile = [&](uint32_t t) {   // first tile at or after t with valid query rows
    while (t < n_tiles && tile_valid(t) == 0) ++t;
    return (uint32_t)__builtin_amdgcn_readfirstlane(t);
  };

  const uint32_t dir_off = lq * ROWB + ((half ^ ((lq / G::SWZ_DIV) & (G::CPK - 1))) * 16u);   // k-step ks: ^ (ks * 32)
  uint32_t tr_lo[DT], tr_hi[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    tr_lo[dt] = stream_tr_offset<D>(lane, 0, dt);
    tr_hi[dt] = stream_tr_offset<D>(lane, 1, dt);
  }
  const bool tr_lane = D >= 32 || 16u * ((lane >> 4) & 1u) < (uint32_t)D;

  f32x16_t acc_dk[DT], acc_dv[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc_dk[dt][i] = 0.f; acc_dv[dt][i] = 0.f; }

  uint32_t t = next_tile(0), b = 0;
  if (t < n_tiles) fill(t, b);
  while (t < n_tiles) {
    __builtin_amdgcn_s_waitcnt(0);   // this wave's loads of tile t have landed
    __syncthreads();                 // ... everybody's; and everybody has left the other buffer
    const uint32_t tn = next_tile(t + 1);
    if (tn < n_tiles) fill(tn, b ^ 1u);
    const char* sQ = lds_s + b * 2u * TILEB;
    const char* sD = sQ + TILEB;
    const float* lse2 = s_lse2 + b * 32;
    const float* dlt = s_delta + b * 32;
    const int32_t q_valid = tile_valid(t);

    f32x16_t s_acc, p_acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s_acc[i] = 0.f; p_acc[i] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bf16x8_t qa = *reinterpret_cast<const bf16x8_t*>(sQ + (dir_off ^ (ks * 32u)));
      const bf16x8_t da = *reinterpret_cast<const bf16x8_t*>(sD + (dir_off ^ (ks * 32u)));
      s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[ks], s_acc, 0, 0, 0);   // S[query][key]
      p_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vf[ks], p_acc, 0, 0, 0);   // dP[query][key]
    }
    // register i of a lane is query (i/4)*8 + 4 half + i%4 of the tile, for the lane's key
    uint32_t pb[8], sb[8];
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const float4 l4 = *reinterpret_cast<const float4*>(lse2 + g4 * 8 + half * 4);
      const float4 d4 = *reinterpret_cast<const float4*>(dlt + g4 * 8 + half * 4);
      const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dl[4] = {d4.x, d4.y, d4.z, d4.w};
      float p[4], ds[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool ok = key_ok && (int32_t)(g4 * 8 + half * 4 + r) < q_valid;
        p[r] = ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[g4 * 4 + r], scale_log2, -lv[r])) : 0.f;
        ds[r] = ok ? p[r] * (p_acc[g4 * 4 + r] - dl[r]) : 0.f;
      }
      pb[g4 * 2 + 0] = pack_bf16x2(p[0], p[1]);
      pb[g4 * 2 + 1] = pack_bf16x2(p[2], p[3]);
      sb[g4 * 2 + 0] = pack_bf16x2(ds[0], ds[1]);
      sb[g4 * 2 + 1] = pack_bf16x2(ds[2], ds[3]);
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x8_t dot[2], qtr[2];
      stream_load_tr<D>(sD, tr_lo[dt], tr_hi[dt], tr_lane, dot);
      stream_load_tr<D>(sQ, tr_lo[dt], tr_hi[dt], tr_lane, qtr);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
        const u32x4_t sraw = {sb[kk * 4 + 0], sb[kk * 4 + 1], sb[kk * 4 + 2], sb[kk * 4 + 3]};
        acc_dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dot[kk], __builtin_bit_cast(bf16x8_t, praw), acc_dv[dt], 0, 0, 0);
        acc_dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtr[kk], __builtin_bit_cast(bf16x8_t, sraw), acc_dk[dt], 0, 0, 0);
      }
    }
    t = tn;
    b ^= 1u;
  }

  // acc[dt][g4*4 + r] = d?t[feature 32 dt + g4*8 + 4 half + r][key lq]: 4 consecutive features of the lane's key per group
  // the gradients' rows are ldg elements apart (dense: ldg = ldo; thirds of one [B, L, 3 H D] tensor: ldg = 3 ldo)
  const size_t base_g = (size_t)it.batch * seq_len * ldg + (size_t)it.head * D;
  uint16_t* dkrow = dk + base_g + (size_t)krow * ldg;
  uint16_t* dvrow = dv + base_g + (size_t)krow * ldg;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const uint32_t d0 = dt * 32 + g4 * 8 + half * 4;
      if (d0 < (uint32_t)D) {
        uint2 a, b;
        a.x = pack_bf16x2(acc_dk[dt][g4 * 4 + 0] * scale, acc_dk[dt][g4 * 4 + 1] * scale);
        a.y = pack_bf16x2(acc_dk[dt][g4 * 4 + 2] * scale, acc_dk[dt][g4 * 4 + 3] * scale);
        b.x = pack_bf16x2(acc_dv[dt][g4 * 4 + 0], acc_dv[dt][g4 * 4 + 1]);
        b.y = pack_bf16x2(acc_dv[dt][g4 * 4 + 2], acc_dv[dt][g4 * 4 + 3]);
        *reinterpret_cast<uint2*>(dkrow + d0) = a;
        *reinterpret_cast<uint2*>(dvrow + d0) = b;
      }
    }
}

// ---- dQ -----------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(64 * kStreamWaves) void bwd_dq_stream_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    uint16_t* __restrict__ dq, const uint32_t* __restrict__ scope_buckets, uint32_t num_scope, uint32_t scope_size,
    uint32_t bs, uint32_t seq_len, uint32_t num_head, const int32_t* __restrict__ kv_len, float scale,
    float scale_log2, uint32_t ldg, uint32_t item0) {
  using G = SGeom<D>;
  constexpr int KSTEPS = G::KSTEPS, ROWB = G::ROWB, DT = G::DT, TILEB = G::TILEB;
  extern __shared__ __attribute__((aligned(16))) char lds_s[];
  // two buffers of (K tile, V tile); the float area of the dkdv layout stays unused; then the scope table
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(lds_s + 4 * TILEB + 4 * 32 * 4);
  int32_t* s_len = reinterpret_cast<int32_t*>(s_bucket + scope_size);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_s;

  const StreamItem it = stream_item(num_scope, num_head, item0);
  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  if (!stream_scope_table(scope_buckets, kv_len, it.scope, scope_size, bs, n_bucket, s_bucket, s_len)) return;

  const uint32_t ldo = num_head * D;
  const size_t base_qkv = (size_t)it.batch * seq_len * ld + (size_t)it.head * D;
  const size_t base_o = (size_t)it.batch * seq_len * ldo + (size_t)it.head * D;
  const size_t base_l = (size_t)it.batch * seq_len * num_head + it.head;

  // this wave's 32 queries
  const uint32_t qloc0 = it.blk * kStreamBlock + wave * 32u;
  const uint32_t qj = qloc0 / bs, q_in_b0 = qloc0 - qj * bs;
  const uint32_t qrow = s_bucket[qj] * bs + q_in_b0 + lq;
  const bool q_ok = (int32_t)(q_in_b0 + lq) < s_len[qj];
  bf16x8_t qf[KSTEPS], dof[KSTEPS];
  {
    const uint16_t* qr = q + base_qkv + (size_t)qrow * ld + half * 8;
    const uint16_t* dr = d_o + base_o + (size_t)qrow * ldo + half * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      qf[ks] = *reinterpret_cast<const bf16x8_t*>(qr + ks * 16);
      dof[ks] = *reinterpret_cast<const bf16x8_t*>(dr + ks * 16);
    }
  }
  const float lse2 = lse[base_l + (size_t)qrow * num_head] * 1.4426950408889634f;
  const float dlt = delta[base_l + (size_t)qrow * num_head];

  const uint32_t n_tiles = scope_size * bs / 32u;
  auto tile_valid = [&](uint32_t t) -> int32_t {   // valid keys of key tile t (uniform)
    const uint32_t j = (t * 32u) / bs;
    return min(max(s_len[j] - (int32_t)(t * 32u - j * bs), 0), 32);
  };
  auto fill = [&](uint32_t t, uint32_t b) {
    const uint32_t j = (t * 32u) / bs;
    const size_t grow = (size_t)__builtin_amdgcn_readfirstlane(s_bucket[j]) * bs + (t * 32u - j * bs);
    const uint32_t buf = lds0 + b * 2u * TILEB;
    stream_fill_tile<D>(reinterpret_cast<const char*>(k + base_qkv + grow * ld), ld * 2u, buf, wave, lane);
    stream_fill_tile<D>(reinterpret_cast<const char*>(v + base_qkv + grow * ld), ld * 2u, buf + TILEB, wave, lane);
  };
  auto next_tile = [&](uint32_t t) {
    while (t < n_tiles && tile_valid(t) == 0) ++t;
    return (uint32_t)__builtin_amdgcn_readfirstlane(t);
  };

  const uint32_t dir_off = lq * ROWB + ((half ^ ((lq / G::SWZ_DIV) & (G::CPK - 1))) * 16u);
  uint32_t tr_lo[DT], tr_hi[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    tr_lo[dt] = stream_tr_offset<D>(lane, 0, dt);
    tr_hi[dt] = stream_tr_offset<D>(lane, 1, dt);
  }
  const bool tr_lane = D >= 32 || 16u * ((lane >> 4) & 1u) < (uint32_t)D;

  f32x16_t acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

  uint32_t t = next_tile(0), b = 0;
  if (t < n_tiles) fill(t, b);
  while (t < n_tiles) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const uint32_t tn = next_tile(t + 1);
    if (tn < n_tiles) fill(tn, b ^ 1u);
    const char* sK = lds_s + b * 2u * TILEB;
    const char* sV = sK + TILEB;
    const int32_t k_valid = tile_valid(t);

    f32x16_t s_acc, p_acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s_acc[i] = 0.f; p_acc[i] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(sK + (dir_off ^ (ks * 32u)));
      const bf16x8_t va = *reinterpret_cast<const bf16x8_t*>(sV + (dir_off ^ (ks * 32u)));
      s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[ks], s_acc, 0, 0, 0);    // St[key][query]
      p_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, dof[ks], p_acc, 0, 0, 0);   // dPt[key][query]
    }
    // register i of a lane is key (i/4)*8 + 4 half + i%4 of the tile, for the lane's query
    uint32_t sb[8];
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      float pv[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const bool ok = q_ok && (int32_t)(((i + e) / 4) * 8 + half * 4 + (i + e) % 4) < k_valid;
        const float p = ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[i + e], scale_log2, -lse2)) : 0.f;
        pv[e] = ok ? p * (p_acc[i + e] - dlt) : 0.f;
      }
      sb[i / 2] = pack_bf16x2(pv[0], pv[1]);
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x8_t ktr[2];
      stream_load_tr<D>(sK, tr_lo[dt], tr_hi[dt], tr_lane, ktr);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const u32x4_t sraw = {sb[kk * 4 + 0], sb[kk * 4 + 1], sb[kk * 4 + 2], sb[kk * 4 + 3]};
        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktr[kk], __builtin_bit_cast(bf16x8_t, sraw), acc[dt], 0, 0, 0);
      }
    }
    t = tn;
    b ^= 1u;
  }
  const size_t base_g = (size_t)it.batch * seq_len * ldg + (size_t)it.head * D;
  uint16_t* dqrow = dq + base_g + (size_t)qrow * ldg;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const uint32_t d0 = dt * 32 + g4 * 8 + half * 4;
      if (d0 < (uint32_t)D) {
        uint2 a;
        a.x = pack_bf16x2(acc[dt][g4 * 4 + 0] * scale, acc[dt][g4 * 4 + 1] * scale);
        a.y = pack_bf16x2(acc[dt][g4 * 4 + 2] * scale, acc[dt][g4 * 4 + 3] * scale);
        *reinterpret_cast<uint2*>(dqrow + d0) = a;
      }
    }
}

template <int D>
static int launch_stream(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, const uint16_t* o,
                         const uint16_t* d_o, const float* lse, float* delta, uint16_t* dq, uint16_t* dk, uint16_t* dv,
                         const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                         uint32_t batch, uint32_t seq_len, uint32_t num_head, const int32_t* kv_len, uint32_t ldg,
                         int device, hipStream_t s) {
  const size_t lds = stream_lds_bytes<D>(scope_size);
  if (lds > 64 * 1024) {
    // the scope table is the only part that grows: 8 bytes per bucket of the scope
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)bwd_dkdv_stream_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)bwd_dq_stream_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  (void)device;
  const uint32_t scope_tokens = scope_size * bs;
  const uint32_t items = batch * num_scope * num_head;
  const float scale = 1.0f / sqrtf((float)D), scale_log2 = 1.4426950408889634f * scale;
  const uint32_t dthreads = 256, dgrid = cdiv_u32(scope_tokens * num_head, dthreads);
  constexpr uint32_t kMaxY = 65535u;      // grid.y limit: longer lists of items go out in several launches
  for (uint32_t y0 = 0; y0 < batch * num_scope; y0 += kMaxY)
    hipLaunchKernelGGL(bwd_delta_kernel<D>, dim3(dgrid, std::min(kMaxY, batch * num_scope - y0)), dim3(dthreads), 0, s, o, d_o,
                       delta, scope_buckets, num_scope, scope_size, bs, seq_len, num_head, y0);
  const dim3 block(64 * kStreamWaves);
  for (uint32_t item0 = 0; item0 < items; item0 += kMaxY) {
    const dim3 grid(scope_tokens / kStreamBlock, std::min(kMaxY, items - item0));
    hipLaunchKernelGGL(bwd_dkdv_stream_kernel<D>, grid, block, lds, s, q, k, v, ld, d_o, lse, delta, dk, dv, scope_buckets,
                       num_scope, scope_size, bs, seq_len, num_head, kv_len, scale, scale_log2, ldg, item0);
    hipLaunchKernelGGL(bwd_dq_stream_kernel<D>, grid, block, lds, s, q, k, v, ld, d_o, lse, delta, dq, scope_buckets,
                       num_scope, scope_size, bs, seq_len, num_head, kv_len, scale, scale_log2, ldg, item0);
  }
  return F3D_OK;
}

// Streaming backward for any scope size (buckets of a multiple of 128 rows), head_dim 16 / 32 / 64 / 128.
int launch_attn_bwd_stream(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, const uint16_t* o,
                           const uint16_t* d_o, const float* lse, float* delta, uint16_t* dq, uint16_t* dk, uint16_t* dv,
                           const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                           uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t head_dim, const int32_t* kv_len,
                           uint32_t ldg, int device, hipStream_t s) {
  if ((uint64_t)batch * num_scope * num_head > 0x7FFFFFF0ull) {
    set_error("attention problem too large for one launch (%llu items)", (unsigned long long)batch * num_scope * num_head);
    return F3D_ERR_INVALID;
  }
#define F3D_STREAM(DD)                                                                                                 \
  return launch_stream<DD>(q, k, v, ld, o, d_o, lse, delta, dq, dk, dv, scope_buckets, num_scope, scope_size, bs, batch, \
                           seq_len, num_head, kv_len, ldg, device, s)
  switch (head_dim) {
    case 16: F3D_STREAM(16);
    case 32: F3D_STREAM(32);
    case 64: F3D_STREAM(64);
    case 128: F3D_STREAM(128);
    default:
      set_error("No backward kernel found for head_dim=%u (supported: 16, 32, 64, 128)", head_dim);
      return F3D_ERR_UNSUPPORTED;
  }
#undef F3D_STREAM
}

}  // namespace f3d
