// Bucketed (scoped) multi-head attention backward for gfx950.
//
// Counterpart of pshattn.buck_swin_bwd (declared src/f3d_frontend.cu:94-97, called from
// flash3dxfmr/layers/buck_swin.py:69-95; the reference ships no kernel source for it, its tests
// differentiate an SDPA oracle, tests/test_attn_bwd.py).  Per batch row, scope and head, with
// P = softmax(Q Kt / sqrt(D)) recomputed from the saved LSE:
//   Delta = rowsum(dO * O)   dV = Pt dO   dP = dO Vt   dS = P * (dP - Delta)
//   dQ = dS K / sqrt(D)      dK = dSt Q / sqrt(D)
//
// Two kernels, one workgroup per (batch, scope, head), one wave per 32 tokens of the scope, the whole scope
// resident in LDS (scopes of 256 or 512 tokens, head_dim 16 or 32):
//   dkdv: a wave owns 32 KEYS (K, V rows as MFMA B operands in registers) and walks the query tiles;
//         S = Q Kt and dP = dO Vt come out with a lane holding one key and 16 queries, so P and dS (bf16) are
//         already the B operands of dVt += dOt P and dKt += Qt dS, whose A operands (dOt, Qt) are read
//         transposed from LDS (ds_read_b64_tr_b16).  Also writes Delta.
//   dq  : a wave owns 32 QUERIES (Q, dO rows in registers, LSE and Delta one scalar per lane) and walks the key
//         tiles; St = K Qt, dPt = V dOt, dQt += Kt dSt with Kt read transposed.
// LDS rows are unpadded with their 16-byte pieces XOR-swizzled (conflict-free 128-bit operand reads); the transposing
// reads address 8-byte pieces per lane and apply the same swizzle to their addresses.
// The score tile is computed twice (once per kernel), which keeps both kernels free of atomics: every output row
// is written by exactly one wave.  Rows that no scope covers are not written (the caller passes zeros).
#include <type_traits>
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

constexpr int kBwdMaxScope = 4;
constexpr int kBwdXcd = 8;

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds + 16 l.
__device__ __forceinline__ void bwd_dma16(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

template <int D>
struct BwdGeom {
  static constexpr int KSTEPS = D / 16;
  static constexpr int CPK = D / 8;              // 16-byte pieces per row
  static constexpr int ROWB = D * 2;             // bytes per row
  static constexpr int RPB = 1024 / ROWB;        // rows one direct-load instruction fills
  static constexpr int BLK_PER_WAVE = 32 / RPB;  // instructions per 32 rows
  static constexpr int SWZ_DIV = 16 / CPK;       // rows sharing one swizzle value
};

// rows [32 wave, 32 wave + 32) of the scope, from a [.., row, ld] tensor into a row-major LDS array
template <int D, bool SWZ>
__device__ __forceinline__ void bwd_fill_rows(const uint16_t* gbase, uint32_t ld, const uint32_t* s_bucket, uint32_t bs,
                                              uint32_t wave, uint32_t lane, char* buf) {
  using G = BwdGeom<D>;
#pragma unroll
  for (int i = 0; i < G::BLK_PER_WAVE; ++i) {
    const uint32_t blk = __builtin_amdgcn_readfirstlane(wave * G::BLK_PER_WAVE + i);
    const uint32_t row = blk * G::RPB + lane / G::CPK, pos = lane % G::CPK;
    const uint32_t j = (blk * G::RPB) / bs;   // uniform: a block never straddles buckets
    const uint32_t rowoff = ((s_bucket[j] * bs + (row - j * bs)) * ld) * 2u;
    const uint32_t ck = SWZ ? (pos ^ ((row / G::SWZ_DIV) & (G::CPK - 1))) : pos;
    bwd_dma16(gbase, rowoff + ck * 16u, buf + blk * 1024);
  }
}

// A operand read transposed from a swizzled LDS tile of 32 rows: lane (m = feature) gets, for k-step kk,
// slots 0..3 = rows 16 kk + 4 half + 0..3 and slots 4..7 = the same + 8 (the order in which an accumulator tile
// hands its rows to the next MFMA as a B operand).  tr_lo / tr_hi are the lane's byte offsets for the two row
// groups (their swizzle values differ); k-step kk adds 16 rows, which leaves the swizzle value unchanged.
template <int D>
__device__ __forceinline__ void bwd_load_tr(const char* tile, uint32_t tr_lo, uint32_t tr_hi, bool tr_lane,
                                            bf16x8_t (&f)[2]) {
  constexpr int ROWB = BwdGeom<D>::ROWB;
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

// the lane's byte offset of its 8-byte piece for the transposing reads: row 4 half + l16 / 4 + 8 hi of a 32-row
// tile, features d_base + 4 (l16 % 4) .. + 3, with the row's swizzle applied to the 16-byte piece index
template <int D>
__device__ __forceinline__ uint32_t bwd_tr_offset(uint32_t lane, uint32_t hi) {
  using G = BwdGeom<D>;
  const uint32_t half = lane >> 5, l16 = lane & 15u, d_base = 16u * ((lane >> 4) & 1u);
  const uint32_t row = 4u * half + l16 / 4u + 8u * hi;
  const uint32_t colb = (d_base + 4u * (l16 & 3u)) * 2u;                    // byte column, a multiple of 8
  const uint32_t piece = (colb / 16u) ^ ((row / G::SWZ_DIV) & (G::CPK - 1));
  return row * G::ROWB + piece * 16u + (colb & 8u);
}

struct BwdItem {
  uint32_t batch, scope, head;
};
__device__ __forceinline__ bool bwd_item(uint32_t n_items, uint32_t items_per_xcd, uint32_t num_scope,
                                         uint32_t num_head, BwdItem& it) {
  // workgroups of one XCD take consecutive items, so the heads of a scope (which share 128-byte lines) meet in one L2
  const uint32_t item = (blockIdx.x % kBwdXcd) * items_per_xcd + blockIdx.x / kBwdXcd;
  if (blockIdx.x / kBwdXcd >= items_per_xcd || item >= n_items) return false;
  it.batch = item / (num_head * num_scope);
  it.scope = (item / num_head) % num_scope;
  it.head = item % num_head;
  return true;
}

template <int D, int T>
constexpr size_t bwd_dkdv_lds_bytes() {
  return (size_t)2 * T * D * 2 + (size_t)2 * T * 4 + kBwdMaxScope * 4;
}
template <int D, int T>
constexpr size_t bwd_dq_lds_bytes() {
  return (size_t)2 * T * D * 2 + kBwdMaxScope * 4;
}

// ---- dK, dV (and Delta) -----------------------------------------------------------------------------
template <int D, int T>
__global__ __launch_bounds__(2 * T) void buck_swin_bwd_dkdv_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    const uint16_t* __restrict__ o, const uint16_t* __restrict__ d_o, const float* __restrict__ lse,
    float* __restrict__ delta, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv,
    const uint32_t* __restrict__ scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
    uint32_t seq_len, uint32_t num_head, float scale, float scale_log2, uint32_t n_items, uint32_t items_per_xcd,
    uint32_t ldg) {
  using G = BwdGeom<D>;
  constexpr int KSTEPS = G::KSTEPS, ROWB = G::ROWB, OPB = T * ROWB;
  extern __shared__ __attribute__((aligned(16))) char lds_bwd[];
  char* sQs = lds_bwd;              // Q
  char* sDs = lds_bwd + OPB;        // dO
  float* s_lse2 = reinterpret_cast<float*>(lds_bwd + 2 * OPB);   // LSE in the exponent's units (x log2 e)
  float* s_delta = s_lse2 + T;
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(s_delta + T);

  BwdItem it;
  if (!bwd_item(n_items, items_per_xcd, num_scope, num_head, it)) return;
  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  if (tid < scope_size) s_bucket[tid] = scope_buckets[(size_t)it.scope * scope_size + tid];
  __syncthreads();
  bool ok = true;
  for (uint32_t j = 0; j < scope_size; ++j) ok = ok && s_bucket[j] < n_bucket;
  if (!ok) return;   // a scope that names a bucket outside the sequence contributes nothing (uniform exit)

  const uint32_t ldo = num_head * D;   // o, dO, dK, dV are dense [B, L, H, D]
  const size_t base_qkv = (size_t)it.batch * seq_len * ld + (size_t)it.head * D;
  const size_t base_o = (size_t)it.batch * seq_len * ldo + (size_t)it.head * D;
  const size_t base_l = (size_t)it.batch * seq_len * num_head + it.head;

  bwd_fill_rows<D, true>(q + base_qkv, ld, s_bucket, bs, wave, lane, sQs);
  bwd_fill_rows<D, true>(d_o + base_o, ldo, s_bucket, bs, wave, lane, sDs);

  // this wave's 32 tokens: local rows [32 wave, 32 wave + 32), lane -> token lq
  const uint32_t loc = wave * 32 + lq;
  const uint32_t lj = loc / bs;
  const uint32_t grow = s_bucket[lj] * bs + (loc - lj * bs);    // row inside the sequence
  // Delta and LSE of the token (both halves of the lane pair compute half of the dot product)
  {
    constexpr int HALF_D = D / 2;
    const uint16_t* orow = o + base_o + (size_t)grow * ldo + half * HALF_D;
    const uint16_t* drow = d_o + base_o + (size_t)grow * ldo + half * HALF_D;
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < HALF_D / 8; ++c) {
      const u32x4_t a = *reinterpret_cast<const u32x4_t*>(orow + c * 8);
      const u32x4_t b = *reinterpret_cast<const u32x4_t*>(drow + c * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s = __builtin_fmaf(bf16_lo(a[e]), bf16_lo(b[e]), s);
        s = __builtin_fmaf(bf16_hi(a[e]), bf16_hi(b[e]), s);
      }
    }
    s += __shfl_xor(s, 32, kWave);
    if (half == 0) {
      s_delta[loc] = s;
      delta[base_l + (size_t)grow * num_head] = s;
      s_lse2[loc] = lse[base_l + (size_t)grow * num_head] * 1.4426950408889634f;
    }
  }
  // K and V rows of the wave's keys as B operands (lane = key lq, 8 features per k-step and half)
  bf16x8_t kf[KSTEPS], vf[KSTEPS];
  {
    const uint16_t* krow = k + base_qkv + (size_t)grow * ld + half * 8;
    const uint16_t* vrow = v + base_qkv + (size_t)grow * ld + half * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      kf[ks] = *reinterpret_cast<const bf16x8_t*>(krow + ks * 16);
      vf[ks] = *reinterpret_cast<const bf16x8_t*>(vrow + ks * 16);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);   // the direct loads of this wave have landed
  __syncthreads();

  const uint32_t dir_off = lq * ROWB + ((half ^ ((lq / G::SWZ_DIV) & (G::CPK - 1))) * 16u);   // k-step ks: ^ (ks * 32)
  const uint32_t tr_lo = bwd_tr_offset<D>(lane, 0), tr_hi = bwd_tr_offset<D>(lane, 1);
  const bool tr_lane = D >= 32 || 16u * ((lane >> 4) & 1u) < (uint32_t)D;

  f32x16_t acc_dk, acc_dv;
#pragma unroll
  for (int i = 0; i < 16; ++i) { acc_dk[i] = 0.f; acc_dv[i] = 0.f; }

  for (uint32_t qt = 0; qt < (uint32_t)(T / 32); ++qt) {
    const uint32_t tile = qt * 32u * ROWB;
    f32x16_t s_acc, p_acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s_acc[i] = 0.f; p_acc[i] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bf16x8_t qa = *reinterpret_cast<const bf16x8_t*>(sQs + tile + (dir_off ^ (ks * 32u)));
      const bf16x8_t da = *reinterpret_cast<const bf16x8_t*>(sDs + tile + (dir_off ^ (ks * 32u)));
      s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[ks], s_acc, 0, 0, 0);   // S[query][key]
      p_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vf[ks], p_acc, 0, 0, 0);   // dP[query][key]
    }
    bf16x8_t dot[2], qtr[2];
    bwd_load_tr<D>(sDs + tile, tr_lo, tr_hi, tr_lane, dot);
    bwd_load_tr<D>(sQs + tile, tr_lo, tr_hi, tr_lane, qtr);
    // register i of a lane is query (i/4)*8 + 4 half + i%4 of the tile
    uint32_t pb[8], sb[8];
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const float4 l4 = *reinterpret_cast<const float4*>(s_lse2 + qt * 32 + g4 * 8 + half * 4);
      const float4 d4 = *reinterpret_cast<const float4*>(s_delta + qt * 32 + g4 * 8 + half * 4);
      const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dl[4] = {d4.x, d4.y, d4.z, d4.w};
      float p[4], ds[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[g4 * 4 + r], scale_log2, -lv[r]));
        ds[r] = p[r] * (p_acc[g4 * 4 + r] - dl[r]);
      }
      pb[g4 * 2 + 0] = pack_bf16x2(p[0], p[1]);
      pb[g4 * 2 + 1] = pack_bf16x2(p[2], p[3]);
      sb[g4 * 2 + 0] = pack_bf16x2(ds[0], ds[1]);
      sb[g4 * 2 + 1] = pack_bf16x2(ds[2], ds[3]);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
      const u32x4_t sraw = {sb[kk * 4 + 0], sb[kk * 4 + 1], sb[kk * 4 + 2], sb[kk * 4 + 3]};
      acc_dv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dot[kk], __builtin_bit_cast(bf16x8_t, praw), acc_dv, 0, 0, 0);
      acc_dk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtr[kk], __builtin_bit_cast(bf16x8_t, sraw), acc_dk, 0, 0, 0);
    }
  }

  // acc[g4*4 + r] = d?t[feature g4*8 + 4 half + r][key lq]: 4 consecutive features of the lane's key per group
  // the gradients' rows are ldg elements apart (dense: ldg = ldo; thirds of one [B, L, 3 H D] tensor: ldg = 3 ldo)
  const size_t base_g = (size_t)it.batch * seq_len * ldg + (size_t)it.head * D;
  uint16_t* dkrow = dk + base_g + (size_t)grow * ldg;
  uint16_t* dvrow = dv + base_g + (size_t)grow * ldg;
#pragma unroll
  for (int g4 = 0; g4 < 4; ++g4) {
    const uint32_t d0 = g4 * 8 + half * 4;
    if (d0 < (uint32_t)D) {
      uint2 a, b;
      a.x = pack_bf16x2(acc_dk[g4 * 4 + 0] * scale, acc_dk[g4 * 4 + 1] * scale);
      a.y = pack_bf16x2(acc_dk[g4 * 4 + 2] * scale, acc_dk[g4 * 4 + 3] * scale);
      b.x = pack_bf16x2(acc_dv[g4 * 4 + 0], acc_dv[g4 * 4 + 1]);
      b.y = pack_bf16x2(acc_dv[g4 * 4 + 2], acc_dv[g4 * 4 + 3]);
      *reinterpret_cast<uint2*>(dkrow + d0) = a;
      *reinterpret_cast<uint2*>(dvrow + d0) = b;
    }
  }
}

// ---- dQ -----------------------------------------------------------------------------------------------
template <int D, int T>
__global__ __launch_bounds__(2 * T) void buck_swin_bwd_dq_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    const uint16_t* __restrict__ d_o, const float* __restrict__ lse, const float* __restrict__ delta,
    uint16_t* __restrict__ dq, const uint32_t* __restrict__ scope_buckets, uint32_t num_scope, uint32_t scope_size,
    uint32_t bs, uint32_t seq_len, uint32_t num_head, float scale, float scale_log2, uint32_t n_items,
    uint32_t items_per_xcd, uint32_t ldg) {
  using G = BwdGeom<D>;
  constexpr int KSTEPS = G::KSTEPS, ROWB = G::ROWB, OPB = T * ROWB;
  extern __shared__ __attribute__((aligned(16))) char lds_bwd[];
  char* sKs = lds_bwd;             // K
  char* sVs = lds_bwd + OPB;       // V
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(lds_bwd + 2 * OPB);

  BwdItem it;
  if (!bwd_item(n_items, items_per_xcd, num_scope, num_head, it)) return;
  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  if (tid < scope_size) s_bucket[tid] = scope_buckets[(size_t)it.scope * scope_size + tid];
  __syncthreads();
  bool ok = true;
  for (uint32_t j = 0; j < scope_size; ++j) ok = ok && s_bucket[j] < n_bucket;
  if (!ok) return;

  const uint32_t ldo = num_head * D;
  const size_t base_qkv = (size_t)it.batch * seq_len * ld + (size_t)it.head * D;
  const size_t base_o = (size_t)it.batch * seq_len * ldo + (size_t)it.head * D;
  const size_t base_l = (size_t)it.batch * seq_len * num_head + it.head;

  bwd_fill_rows<D, true>(k + base_qkv, ld, s_bucket, bs, wave, lane, sKs);
  bwd_fill_rows<D, true>(v + base_qkv, ld, s_bucket, bs, wave, lane, sVs);

  const uint32_t loc = wave * 32 + lq;
  const uint32_t lj = loc / bs;
  const uint32_t grow = s_bucket[lj] * bs + (loc - lj * bs);
  // Q and dO rows of the wave's queries as B operands; LSE and Delta of the lane's query
  bf16x8_t qf[KSTEPS], dof[KSTEPS];
  {
    const uint16_t* qrow = q + base_qkv + (size_t)grow * ld + half * 8;
    const uint16_t* drow = d_o + base_o + (size_t)grow * ldo + half * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      qf[ks] = *reinterpret_cast<const bf16x8_t*>(qrow + ks * 16);
      dof[ks] = *reinterpret_cast<const bf16x8_t*>(drow + ks * 16);
    }
  }
  const float lse2 = lse[base_l + (size_t)grow * num_head] * 1.4426950408889634f;
  const float dlt = delta[base_l + (size_t)grow * num_head];
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  const uint32_t dir_off = lq * ROWB + ((half ^ ((lq / G::SWZ_DIV) & (G::CPK - 1))) * 16u);
  const uint32_t tr_lo = bwd_tr_offset<D>(lane, 0), tr_hi = bwd_tr_offset<D>(lane, 1);
  const bool tr_lane = D >= 32 || 16u * ((lane >> 4) & 1u) < (uint32_t)D;

  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (uint32_t kt = 0; kt < (uint32_t)(T / 32); ++kt) {
    const uint32_t tile = kt * 32u * ROWB;
    f32x16_t s_acc, p_acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s_acc[i] = 0.f; p_acc[i] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(sKs + tile + (dir_off ^ (ks * 32u)));
      const bf16x8_t va = *reinterpret_cast<const bf16x8_t*>(sVs + tile + (dir_off ^ (ks * 32u)));
      s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[ks], s_acc, 0, 0, 0);    // St[key][query]
      p_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, dof[ks], p_acc, 0, 0, 0);   // dPt[key][query]
    }
    bf16x8_t ktr[2];
    bwd_load_tr<D>(sKs + tile, tr_lo, tr_hi, tr_lane, ktr);
    uint32_t sb[8];
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[i], scale_log2, -lse2));
      const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[i + 1], scale_log2, -lse2));
      sb[i / 2] = pack_bf16x2(p0 * (p_acc[i] - dlt), p1 * (p_acc[i + 1] - dlt));
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const u32x4_t sraw = {sb[kk * 4 + 0], sb[kk * 4 + 1], sb[kk * 4 + 2], sb[kk * 4 + 3]};
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktr[kk], __builtin_bit_cast(bf16x8_t, sraw), acc, 0, 0, 0);
    }
  }
  const size_t base_g = (size_t)it.batch * seq_len * ldg + (size_t)it.head * D;
  uint16_t* dqrow = dq + base_g + (size_t)grow * ldg;
#pragma unroll
  for (int g4 = 0; g4 < 4; ++g4) {
    const uint32_t d0 = g4 * 8 + half * 4;
    if (d0 < (uint32_t)D) {
      uint2 a;
      a.x = pack_bf16x2(acc[g4 * 4 + 0] * scale, acc[g4 * 4 + 1] * scale);
      a.y = pack_bf16x2(acc[g4 * 4 + 2] * scale, acc[g4 * 4 + 3] * scale);
      *reinterpret_cast<uint2*>(dqrow + d0) = a;
    }
  }
}

template <int D, int T>
static int launch_attn_bwd(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, const uint16_t* o,
                           const uint16_t* d_o, const float* lse, float* delta, uint16_t* dq, uint16_t* dk,
                           uint16_t* dv, const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                           uint32_t bs, uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t ldg, int device,
                           hipStream_t s) {
  static bool attr_set[64] = {};
  auto kern_a = buck_swin_bwd_dkdv_kernel<D, T>;
  auto kern_b = buck_swin_bwd_dq_kernel<D, T>;
  constexpr size_t lds_a = bwd_dkdv_lds_bytes<D, T>(), lds_b = bwd_dq_lds_bytes<D, T>();
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern_a, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_a));
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)kern_b, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_b));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  const uint32_t n_items = batch * num_scope * num_head;
  const uint32_t per_xcd = (n_items + kBwdXcd - 1) / kBwdXcd;
  const float scale = 1.0f / sqrtf((float)D), scale_log2 = 1.4426950408889634f * scale;
  hipLaunchKernelGGL(kern_a, dim3(per_xcd * kBwdXcd), dim3(2 * T), lds_a, s, q, k, v, ld, o, d_o, lse, delta, dk, dv,
                     scope_buckets, num_scope, scope_size, bs, seq_len, num_head, scale, scale_log2, n_items, per_xcd, ldg);
  hipLaunchKernelGGL(kern_b, dim3(per_xcd * kBwdXcd), dim3(2 * T), lds_b, s, q, k, v, ld, d_o, lse, delta, dq,
                     scope_buckets, num_scope, scope_size, bs, seq_len, num_head, scale, scale_log2, n_items, per_xcd, ldg);
  return F3D_OK;
}

}  // namespace f3d

extern "C" int f3d_buck_swin_bwd(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v,
                                 uint32_t qkv_row_stride, const f3d_bf16_t* o, const f3d_bf16_t* d_o,
                                 const float* lse, float* delta, f3d_bf16_t* dq, f3d_bf16_t* dk, f3d_bf16_t* dv,
                                 const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                                 uint32_t bucket_size, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                                 uint32_t head_dim, const int32_t* kv_len, int device, void* stream) {
  return f3d_buck_swin_bwd_strided(q, k, v, qkv_row_stride, o, d_o, lse, delta, dq, dk, dv, num_head * head_dim,
                                   scope_buckets, num_scope, scope_size, bucket_size, batch, seq_len, num_head, head_dim,
                                   kv_len, device, stream);
}

extern "C" int f3d_buck_swin_bwd_strided(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v,
                                         uint32_t qkv_row_stride, const f3d_bf16_t* o, const f3d_bf16_t* d_o,
                                         const float* lse, float* delta, f3d_bf16_t* dq, f3d_bf16_t* dk, f3d_bf16_t* dv,
                                         uint32_t grad_row_stride, const uint32_t* scope_buckets, uint32_t num_scope,
                                         uint32_t scope_size, uint32_t bucket_size, uint32_t batch, uint32_t seq_len,
                                         uint32_t num_head, uint32_t head_dim, const int32_t* kv_len, int device,
                                         void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(q && k && v && o && d_o && lse && delta && dq && dk && dv && scope_buckets, "null tensor pointer");
  F3D_CHECK_ARG(grad_row_stride >= num_head * head_dim && grad_row_stride % 8 == 0,
                "dq/dk/dv row stride %u must be a multiple of 8 and at least num_head*head_dim=%u", grad_row_stride,
                num_head * head_dim);
  F3D_CHECK_ARG(bucket_size >= 128 && bucket_size % 128 == 0, "bucket_size=%u must be a multiple of 128",
                bucket_size);
  F3D_CHECK_ARG(seq_len % bucket_size == 0, "sequence length %u is not a multiple of bucket_size=%u", seq_len,
                bucket_size);
  F3D_CHECK_ARG(qkv_row_stride >= num_head * head_dim && qkv_row_stride % 8 == 0,
                "q/k/v row stride %u must be a multiple of 8 and at least num_head*head_dim=%u", qkv_row_stride,
                num_head * head_dim);
  F3D_CHECK_ARG((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_o | (uintptr_t)dq |
                  (uintptr_t)dk | (uintptr_t)dv) & 15u) == 0,
                "q/k/v/o/dO/dQ/dK/dV must be 16-byte aligned");
  F3D_CHECK_ARG(scope_size >= 1, "scope_size must be at least 1");
  const uint32_t scope_tokens = scope_size * bucket_size;
  // the scope-resident kernels: small heads, a scope that fits LDS, no valid lengths, 32-bit row offsets
  const bool resident = (head_dim == 16 || head_dim == 32) && scope_size <= (uint32_t)kBwdMaxScope &&
                        (scope_tokens == 256 || scope_tokens == 512) && kv_len == nullptr &&
                        (uint64_t)seq_len * qkv_row_stride * 2 < (1ull << 32);
  if (!(head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128)) {
    set_error("No backward kernel found for head_dim=%u (supported: 16, 32, 64, 128)", head_dim);
    return F3D_ERR_UNSUPPORTED;
  }
  if (!resident && (uint64_t)scope_size * 8 > 32 * 1024) {
    set_error("attention backward: a scope of %u buckets exceeds the 4096 the scope table holds", scope_size);
    return F3D_ERR_UNSUPPORTED;
  }
  if (batch == 0 || num_scope == 0 || num_head == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  int rc;
#define F3D_BWD(DD, TT)                                                                                          \
  rc = launch_attn_bwd<DD, TT>(q, k, v, qkv_row_stride, o, d_o, lse, delta, dq, dk, dv, scope_buckets, num_scope, \
                               scope_size, bucket_size, batch, seq_len, num_head, grad_row_stride, device, s)
  if (!resident) {
    rc = launch_attn_bwd_stream(q, k, v, qkv_row_stride, o, d_o, lse, delta, dq, dk, dv, scope_buckets, num_scope,
                                scope_size, bucket_size, batch, seq_len, num_head, head_dim, kv_len, grad_row_stride,
                                device, s);
  } else if (head_dim == 16) {
    if (scope_tokens == 256) F3D_BWD(16, 256); else F3D_BWD(16, 512);
  } else {
    if (scope_tokens == 256) F3D_BWD(32, 256); else F3D_BWD(32, 512);
  }
#undef F3D_BWD
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}
