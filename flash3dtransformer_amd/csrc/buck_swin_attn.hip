// Bucketed (scoped) multi-head attention forward for gfx950.
//
// Counterpart of pshattn.buck_swin_fwd (declared src/f3d_frontend.cu:90-92, called from
// flash3dxfmr/layers/buck_swin.py:57; the reference ships no kernel source for it).  For every
// batch row, every scope (a row of scope_buckets) and every head: softmax(Q Kt / sqrt(D)) V over the
// rows of the scope's buckets, plus the natural-log LSE.
//
// Kernel shape: one 256-thread workgroup (4 waves) per (batch, scope, head, 128-query block); each
// wave owns 32 query rows.  K and V of the scope stream through LDS in tiles of KT keys (K row-major,
// V transposed), prefetched into registers one tile ahead.  Scores are computed TRANSPOSED,
// St = K Qt with v_mfma_f32_32x32x16_bf16, so that a lane holds 16 keys of ONE query: the softmax
// max / sum run inside the lane plus one exchange with lane^32, and the bf16 P values are already in
// the B-operand layout of the second MFMA, Ot += Vt Pt (keys are consumed in the permuted order the
// accumulator layout yields; V is staged in that same order).  Softmax runs in the exp2 domain with
// fp32 accumulation.  Workgroup ids are remapped so that the workgroups of one scope (which share
// K/V and the 512-byte token rows) land on the same XCD and its L2.
#include <type_traits>
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kAttnThreads = 256;
constexpr int kQBlock = 128;  // query rows per workgroup
constexpr int kNumXcd = 8;

// position of key (kk = key % 16) inside its group of 16 in the transposed V tile:
// storage order 0..3, 8..11, 4..7, 12..15
__device__ __forceinline__ uint32_t vperm16(uint32_t kk) { return (kk & 3u) | ((kk & 4u) << 1) | ((kk & 8u) >> 1); }

template <int D, int KT>
struct AttnCfg {
  static constexpr int DP = D < 32 ? 32 : D;           // rows of the transposed V tile seen by MFMA
  static constexpr int KSTEPS = D / 16;                 // k-steps of the QK product
  static constexpr int DT = DP / 32;                    // 32-row output tiles
  static constexpr int NSUB = KT / 32;                  // 32-key score subtiles per KV tile
  static constexpr int KROW = D + 8;                    // padded LDS row of K (elements)
  static constexpr int VROW = KT + 8;                   // padded LDS row of Vt (elements)
  static constexpr int CHUNKS = KT * D / 8;             // 16-byte chunks per K (or V) tile
  static constexpr int NCH = (CHUNKS + kAttnThreads - 1) / kAttnThreads;
  static constexpr int LDS_BYTES = (KT * KROW + D * VROW) * 2;   // plus 8 bytes per scope entry
};

template <int D, int KT>
__global__ __launch_bounds__(kAttnThreads) void buck_swin_fwd_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    uint16_t* __restrict__ o, float* __restrict__ lse, const uint32_t* __restrict__ scope_buckets,
    uint32_t num_scope, uint32_t scope_size, uint32_t bs, uint32_t seq_len, uint32_t num_head,
    const int32_t* __restrict__ kv_len, float scale_log2, uint32_t n_work, uint32_t work_per_xcd) {
  using C = AttnCfg<D, KT>;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds_attn[];
  uint16_t* sK = lds_attn;                  // [KT][KROW]
  uint16_t* sVt = lds_attn + KT * C::KROW;  // [D][VROW]
  // per scope entry: bucket id and number of valid keys (0 for an id outside the sequence), read once
  // from global memory so that the tile loop never waits on a scalar load
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(lds_attn + KT * C::KROW + D * C::VROW);
  int32_t* s_len = reinterpret_cast<int32_t*>(s_bucket + scope_size);

  // XCD-aware remap: hardware deals consecutive workgroup ids round-robin to the 8 XCDs
  const uint32_t work = (blockIdx.x % kNumXcd) * work_per_xcd + blockIdx.x / kNumXcd;
  if (work >= n_work) return;
  const uint32_t qblocks = scope_size * bs / kQBlock;
  uint32_t rem = work;
  const uint32_t qb = rem % qblocks; rem /= qblocks;
  const uint32_t head = rem % num_head; rem /= num_head;
  const uint32_t scope = rem % num_scope;
  const uint32_t batch = rem / num_scope;

  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t* my_scope = scope_buckets + (size_t)scope * scope_size;

  // ---- this wave's 32 query rows ----
  const uint32_t q_local = qb * kQBlock;                 // row offset inside the scope
  const uint32_t n_bucket = seq_len / bs;
  for (uint32_t j = tid; j < scope_size; j += kAttnThreads) {
    const uint32_t b = my_scope[j];
    s_bucket[j] = b;
    s_len[j] = b >= n_bucket ? 0 : (kv_len ? min(max(kv_len[b], 0), (int32_t)bs) : (int32_t)bs);
  }
  __syncthreads();
  const uint32_t q_bucket = s_bucket[q_local / bs];
  if (q_bucket >= n_bucket) return;  // a scope entry outside the sequence names no rows (uniform per workgroup)
  const uint32_t q_in_bucket = (q_local % bs) + wave * 32 + lq;
  const uint32_t q_row = q_bucket * bs + q_in_bucket;
  const size_t tok0 = (size_t)batch * seq_len;
  const int32_t q_valid_len = s_len[q_local / bs];

  bf16x8_t qf[C::KSTEPS];
  {
    const uint16_t* qp = q + (tok0 + q_row) * ld + head * D + half * 8;
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + ks * 16);
  }

  f32x16_t acc[C::DT];
#pragma unroll
  for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- KV tile iteration state ----
  const uint32_t tiles_per_bucket = bs / KT;
  uint32_t jb = 0, kt = 0;  // scope bucket index, tile inside the bucket
  auto bucket_len = [&](uint32_t j) -> int32_t { return s_len[j]; };
  auto settle = [&]() {  // advance (jb, kt) to the next tile that holds at least one valid key
    while (jb < scope_size) {
      if ((int32_t)(kt * KT) < bucket_len(jb)) return true;
      ++jb; kt = 0;
    }
    return false;
  };

  u32x4_t rk[C::NCH], rv[C::NCH];
  auto fetch = [&](uint32_t j, uint32_t t) {
    const size_t row0 = tok0 + (size_t)s_bucket[j] * bs + t * KT;
#pragma unroll
    for (int i = 0; i < C::NCH; ++i) {
      const uint32_t c = tid + i * kAttnThreads;
      if (C::CHUNKS % kAttnThreads == 0 || c < (uint32_t)C::CHUNKS) {
        const uint32_t key = c / (D / 8), dc = c % (D / 8);
        const size_t off = (row0 + key) * ld + head * D + dc * 8;
        rk[i] = *reinterpret_cast<const u32x4_t*>(k + off);
        rv[i] = *reinterpret_cast<const u32x4_t*>(v + off);
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < C::NCH; ++i) {
      const uint32_t c = tid + i * kAttnThreads;
      if (C::CHUNKS % kAttnThreads == 0 || c < (uint32_t)C::CHUNKS) {
        const uint32_t key = c / (D / 8), dc = c % (D / 8);
        *reinterpret_cast<u32x4_t*>(sK + key * C::KROW + dc * 8) = rk[i];
        const uint32_t pos = (key & ~15u) | vperm16(key & 15u);
        uint16_t* col = sVt + (dc * 8) * C::VROW + pos;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          col[(2 * e) * C::VROW] = (uint16_t)(rv[i][e] & 0xFFFFu);
          col[(2 * e + 1) * C::VROW] = (uint16_t)(rv[i][e] >> 16);
        }
      }
    }
  };

  bool have = settle();
  if (have) fetch(jb, kt);
  while (have) {
    const uint32_t cur_kt = kt;
    const int32_t cur_len = bucket_len(jb);
    __syncthreads();  // every wave is done reading the previous tile
    stage();
    __syncthreads();
    // prefetch the next tile while this one is consumed
    ++kt;
    if (kt == tiles_per_bucket) { ++jb; kt = 0; }
    have = settle();
    if (have) fetch(jb, kt);

    // ---- St = K Qt for the whole tile ----
    float s[C::NSUB * 16];
#pragma unroll
    for (int j = 0; j < C::NSUB; ++j) {
      f32x16_t sacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ++ks) {
        const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(sK + (j * 32 + lq) * C::KROW + ks * 16 + half * 8);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sacc, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) s[j * 16 + i] = sacc[i];
    }
    // ---- mask keys beyond the bucket's valid length (only a boundary tile pays for this) ----
    if ((int32_t)((cur_kt + 1) * KT) > cur_len) {
#pragma unroll
      for (int j = 0; j < C::NSUB; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int32_t key = cur_kt * KT + j * 32 + (i / 4) * 8 + half * 4 + (i % 4);
          if (key >= cur_len) s[j * 16 + i] = -INFINITY;
        }
    }
    // ---- online softmax (exp2 domain) ----
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < C::NSUB * 16; ++i) mx = fmaxf(mx, s[i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx * scale_log2);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);  // m_run = -inf -> 0
    m_run = m_new;
    float psum = 0.f;
    uint32_t pb[C::NSUB * 8];
#pragma unroll
    for (int i = 0; i < C::NSUB * 16; i += 2) {
      const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], scale_log2, -m_use));
      const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 1], scale_log2, -m_use));
      pb[i / 2] = pack_bf16x2(p0, p1);
      // row sum of the bf16-rounded probabilities (what the PV product sees): one dot2 per pair
      psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pb[i / 2]),
                                             __builtin_bit_cast(bf16x2_t, 0x3F803F80u), psum, false);
    }
    l_run = l_run * alpha + psum;
    // the running maximum settles after the first tiles: rescale the accumulators only when some
    // query of this wave actually moved (wave-uniform branch)
    if (__ballot(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] *= alpha;
    }
    // ---- Ot += Vt Pt ----
#pragma unroll
    for (int j = 0; j < C::NSUB; ++j)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        u32x4_t praw = {pb[j * 8 + kk * 4 + 0], pb[j * 8 + kk * 4 + 1], pb[j * 8 + kk * 4 + 2], pb[j * 8 + kk * 4 + 3]};
        const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
          bf16x8_t vf;
          if (D >= 32 || lq < (uint32_t)D) {
            vf = *reinterpret_cast<const bf16x8_t*>(sVt + (dt * 32 + lq) * C::VROW + j * 32 + kk * 16 + half * 8);
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) vf[e] = (__bf16)0.f;
          }
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[dt], 0, 0, 0);
        }
      }
  }

  // ---- epilogue: normalise, store O (bf16) and LSE ----
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const bool row_ok = (int32_t)q_in_bucket < q_valid_len && l_tot > 0.f;
  const float inv = row_ok ? 1.0f / l_tot : 0.f;
  uint16_t* op = o + ((tok0 + q_row) * num_head + head) * D;
#pragma unroll
  for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t d0 = dt * 32 + g * 8 + half * 4;
      if (D >= 32 || d0 < (uint32_t)D) {
        uint2 w;
        w.x = pack_bf16x2(acc[dt][g * 4 + 0] * inv, acc[dt][g * 4 + 1] * inv);
        w.y = pack_bf16x2(acc[dt][g * 4 + 2] * inv, acc[dt][g * 4 + 3] * inv);
        *reinterpret_cast<uint2*>(op + d0) = w;
      }
    }
  if (half == 0) {
    const float ln2 = 0.69314718055994530942f;
    lse[(tok0 + q_row) * num_head + head] = row_ok ? (m_run + __builtin_amdgcn_logf(l_tot)) * ln2 : 0.f;
  }
}

// ---- resident variant ---------------------------------------------------------------------------
// When a scope holds 256 or 512 tokens and head_dim <= 32 (the shape of every block of the Flash3D
// model: one 512-row bucket per scope, 32-wide heads) the K and V of a (scope, head) fit in LDS
// twice.  One persistent workgroup walks a list of (batch, scope, head) items: wave w owns the scope's
// query rows [32w, 32w+32) and runs them against all key tiles without any barrier, while the NEXT
// item's K / V stream from HBM straight into the other LDS buffer (global_load ... lds, no registers)
// and its Q into eight registers.  One barrier per item.
//
// LDS layout of one buffer: K [T][D] then V [T][D], both row-major exactly as the direct loads write
// them (a wave's 64 lanes fill 1 KB = 1024/(2D) consecutive rows).  K rows carry no padding: the
// 16-byte chunk c of row r is stored at position c ^ swz(r), swz(r) = (r / (128/D)) mod (D/8), which
// spreads the 32 rows of a ds_read_b128 over all banks.  V is read with ds_read_b64_tr_b16, which hands
// lane i of a 16-lane block column i%4 of the four 8-byte pieces addressed by lanes i/4 + {0,4,8,12}:
// with lane r pointing at key r/4, features 4(r%4).., a lane receives one feature of four consecutive
// keys, i.e. the MFMA A operand of V^T, with no transposed copy of V anywhere.
//
// Softmax without a running maximum (fast pass): Q is pre-multiplied by log2(e)/sqrt(D) (one bf16
// rounding), so the score MFMA emits exponents and the VALU only exponentiates: P = 2^S with the
// reference fixed at zero.  Softmax is shift-invariant and fp32 / bf16 share an 8-bit exponent, so this
// is exact as long as the numbers stay in range; a wave whose total row sum reaches 2^24 or stays under
// 2^-24 (scores that large also magnify the rounding of the pre-scaled Q) redoes its item with the general
// pass: unscaled Q, scale applied in fp32, running maximum.  Masked keys of a one-bucket scope are handled
// inside the fast pass (steps past the valid length are skipped, the boundary step gets -inf scores);
// scopes of several buckets of which some are partly valid take the general pass.
// f(std::integral_constant<uint32_t, 0>) ... f(std::integral_constant<uint32_t, N - 1>): a loop whose counter is a
// constant expression inside the body (immediate LDS offsets, statically indexed register arrays)
template <uint32_t N, uint32_t I = 0, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<uint32_t, I>{});
    static_for<N, I + 1>(f);
  }
}

constexpr int kResMaxScope = 4;  // buckets per scope: at most 512 tokens in buckets of at least 128
typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

// 16 bytes per lane from global memory straight into LDS: lane l of the wave lands at lds + 16 l.
// gbase and lds are wave-uniform, voff is the lane's byte offset from gbase.
__device__ __forceinline__ void lds_dma16(const void* gbase, uint32_t voff, const char* lds) {
  const uint32_t lds_addr =
      __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

template <int D, int T>
constexpr size_t resident_lds_bytes() {
  return 2 * (size_t)2 * T * D * 2 + 3 * kResMaxScope * 8;
}

template <int D, int T>
__global__ __launch_bounds__(2 * T) __attribute__((amdgpu_waves_per_eu(4, 4))) void buck_swin_fwd_resident_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    uint16_t* __restrict__ o, float* __restrict__ lse, const uint32_t* __restrict__ scope_buckets,
    uint32_t num_scope, uint32_t scope_size, uint32_t bs, uint32_t seq_len, uint32_t num_head,
    const int32_t* __restrict__ kv_len, float scale_log2, uint32_t n_items, uint32_t items_per_xcd,
    uint32_t n_slots) {
  constexpr int KT = 64;
  constexpr int KSTEPS = D / 16;
  constexpr int NSUB = KT / 32;
  constexpr int CPK = D / 8;               // 16-byte chunks per row
  constexpr int ROWB = D * 2;              // bytes per K / V row in LDS
  constexpr int RPB = 1024 / ROWB;         // rows one direct-load instruction fills
  constexpr int BLK_PER_WAVE = 32 / RPB;   // wave w fills the rows [32w, 32w+32) of K and of V
  constexpr int SWZ_DIV = 16 / CPK;        // rows sharing one swizzle value
  constexpr int OPB = T * ROWB;            // bytes of one operand (K or V)
  constexpr int BUF = 2 * OPB;             // bytes of one K + V buffer
  constexpr int N_TILES = T / KT;
  extern __shared__ __attribute__((aligned(16))) char lds_res[];
  uint32_t (*s_bucket)[kResMaxScope] = reinterpret_cast<uint32_t (*)[kResMaxScope]>(lds_res + 2 * BUF);
  int32_t (*s_len)[kResMaxScope] = reinterpret_cast<int32_t (*)[kResMaxScope]>(lds_res + 2 * BUF + 3 * kResMaxScope * 4);

  const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  const uint32_t xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  const uint32_t item_lo = xcd * items_per_xcd + slot;
  const uint32_t item_hi = min((xcd + 1) * items_per_xcd, n_items);
  if (item_lo >= item_hi) return;        // whole workgroup: no barrier has been passed yet
  const uint32_t my_items = (item_hi - item_lo + n_slots - 1) / n_slots;

  // item -> (batch, scope, head); the element offset of (first token of the batch, head) is uniform, the
  // per-thread part (row inside the sequence, chunk) fits 32 bits (checked by the host)
  auto item_scope = [&](uint32_t it) { return (it / num_head) % num_scope; };
  auto item_base = [&](uint32_t it) {
    return (size_t)(it / (num_head * num_scope)) * seq_len * ld + (size_t)(it % num_head) * D;
  };

  // bucket ids / valid lengths of one item's scope, handled by the first scope_size threads
  uint32_t tb = 0;
  int32_t tl = 0;
  auto load_table_ids = [&](uint32_t it) {
    if (tid < scope_size) tb = scope_buckets[(size_t)item_scope(it) * scope_size + tid];
  };
  auto load_table_len = [&]() {
    if (tid < scope_size) tl = tb >= n_bucket ? 0 : (kv_len ? min(max(kv_len[tb], 0), (int32_t)bs) : (int32_t)bs);
  };
  auto store_table = [&](uint32_t tslot) {
    if (tid < scope_size) {
      s_bucket[tslot][tid] = tb;
      s_len[tslot][tid] = tl;
    }
  };

  // direct HBM -> LDS loads of one item's K and V rows [32 wave, 32 wave + 32)
  auto issue_kv = [&](uint32_t it, uint32_t tslot, char* buf) {
    const size_t base = item_base(it);
#pragma unroll
    for (int i = 0; i < BLK_PER_WAVE; ++i) {
      const uint32_t blk = __builtin_amdgcn_readfirstlane(wave * BLK_PER_WAVE + i);
      const uint32_t row = blk * RPB + lane / CPK, pos = lane % CPK;
      const uint32_t j = (blk * RPB) / bs;               // uniform: a block never straddles buckets
      if (s_len[tslot][j] > 0) {
        const uint32_t rowoff = ((s_bucket[tslot][j] * bs + (row - j * bs)) * ld) * 2u;
        const uint32_t ck = pos ^ ((row / SWZ_DIV) & (CPK - 1));
        // Issued as inline assembly on purpose: the compiler then keeps no record of LDS writes in
        // flight and does not put a full vmcnt wait in front of the tile loop's LDS reads (they read the
        // OTHER buffer).  The wait that matters is the explicit one before the per-item barrier.
        lds_dma16(k + base, rowoff + ck * 16u, buf + blk * 1024);
        lds_dma16(v + base, rowoff + pos * 16u, buf + OPB + blk * 1024);
      }
    }
  };
  // this wave's 32 query rows sit at scope-local rows [32 wave, 32 wave + 32)
  const uint32_t q_local = wave * 32;
  const uint32_t qj = q_local / bs;
  const uint32_t q_in_bucket = (q_local - qj * bs) + lq;
  u32x4_t qraw[KSTEPS];
  auto issue_q = [&](uint32_t it, uint32_t tslot) {
    const uint32_t qb = s_bucket[tslot][qj];
    const uint32_t off = (((qb < n_bucket ? qb : 0u) * bs + q_in_bucket) * ld + half * 8) * 2u;
    const char* qp = reinterpret_cast<const char*>(q + item_base(it));
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qraw[ks] = *reinterpret_cast<const u32x4_t*>(qp + (off + ks * 32u));
  };

  // ---- prologue: tables of the first two items, K / V / Q of the first ----
  load_table_ids(item_lo);
  load_table_len();
  store_table(0);
  if (my_items > 1) {
    load_table_ids(item_lo + n_slots);
    load_table_len();
    store_table(1);
  }
  __syncthreads();
  issue_q(item_lo, 0);
  issue_kv(item_lo, 0, lds_res);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  // per-lane LDS byte offsets inside a buffer
  const uint32_t k_off = lq * ROWB + ((half ^ ((lq / SWZ_DIV) & (CPK - 1))) * 16u);   // k-step ks: ^ (ks * 32)
  const uint32_t l16 = lane & 15u, d_base = 16u * ((lane >> 4) & 1u);
  const uint32_t v_off = OPB + (4u * half + l16 / 4u) * ROWB + (d_base + 4u * (l16 & 3u)) * 2u;
  const bool v_lane = D >= 32 || d_base < (uint32_t)D;   // lanes whose V^T row exists

  for (uint32_t n = 0; n < my_items; ++n) {
    const uint32_t item = item_lo + n * n_slots;
    const uint32_t tcur = n % 3, tnext = (n + 1) % 3, tnext2 = (n + 2) % 3;
    const bool has_next = n + 1 < my_items;
    const char* sbuf = lds_res + (n & 1u) * BUF;
    const uint32_t q_bucket = s_bucket[tcur][qj];
    const bool q_exists = q_bucket < n_bucket;             // uniform per wave
    const uint32_t q_row = (q_exists ? q_bucket : 0u) * bs + q_in_bucket;
    const int32_t q_valid_len = s_len[tcur][qj];

    // Q of this item arrived during the previous one: scale and round once
    bf16x8_t qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      u32x4_t sc;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        sc[e] = pack_bf16x2(bf16_lo(qraw[ks][e]) * scale_log2, bf16_hi(qraw[ks][e]) * scale_log2);
      qf[ks] = __builtin_bit_cast(bf16x8_t, sc);
    }
    // put the next item's operands in flight
    if (has_next) {
      issue_q(item + n_slots, tnext);
      issue_kv(item + n_slots, tnext, lds_res + ((n + 1) & 1u) * BUF);
    }
    if (n + 2 < my_items) load_table_ids(item + 2 * n_slots);
    // valid key counts of the (at most four) buckets of this scope, as wave-uniform scalars
    static_assert(kResMaxScope == 4, "four bucket lengths are kept in scalars");
    const int32_t blen0 = __builtin_amdgcn_readfirstlane(s_len[tcur][0]);
    const int32_t blen1 = __builtin_amdgcn_readfirstlane(scope_size > 1 ? s_len[tcur][1] : 0);
    const int32_t blen2 = __builtin_amdgcn_readfirstlane(scope_size > 2 ? s_len[tcur][2] : 0);
    const int32_t blen3 = __builtin_amdgcn_readfirstlane(scope_size > 3 ? s_len[tcur][3] : 0);

    float m_ref = 0.f;        // reference subtracted from the scaled scores
    f32x16_t acc;
    float l_run = 0.f;
    constexpr uint32_t NSTEP = T / 32, QSTEP = NSTEP / 4;

    // V^T operand of a step: slots 0..3 of a lane are keys 16kk + 4 half + 0..3, slots 4..7 the same + 8
    auto load_v = [&](uint32_t st, bf16x8_t (&vf)[2]) {
      const char* vt = sbuf + st * 32u * ROWB + v_off;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        i16x4_t lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
        if (v_lane) {
          lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(vt + (kk * 16) * ROWB));
          hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(vt + (kk * 16 + 8) * ROWB));
        }
        vf[kk] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    // P = 2^S as bf16 pairs, row sum from the rounded values
    auto exp_pack = [&](const f32x16_t& sc, uint32_t (&pb)[8], float& psum) {
      psum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(sc[i]), __builtin_amdgcn_exp2f(sc[i + 1]));
        psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pb[i / 2]),
                                               __builtin_bit_cast(bf16x2_t, 0x3F803F80u), psum, false);
      }
    };
    auto pv = [&](const uint32_t (&pb)[8], const bf16x8_t (&vf)[2]) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kk], __builtin_bit_cast(bf16x8_t, praw), acc, 0, 0, 0);
      }
    };

    // ---- fast pass: reference fixed at zero; one bucket per scope may be partly valid ----
    // Fully unrolled over the steps of the scope (LDS offsets are immediates).  Step st issues the score MFMAs
    // of step st+1 from K fragments that were read a step earlier, requests the K fragments of step st+2 and
    // its own V fragments, exponentiates step st on the VALU while the matrix core runs, and ends with P V^T
    // of step st.  `n_valid` steps hold valid keys (a prefix of the scope); in the last of them only the first
    // `tail_keys` keys are valid and the others get a score of -inf (2^-inf = 0 exactly).  The row sum is
    // chained through the dot2 accumulator; whether it left the safe range is looked at once per item.
    auto load_k = [&](uint32_t st, bf16x8_t (&kf)[KSTEPS]) {
      const char* kt = sbuf + st * 32u * ROWB;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = *reinterpret_cast<const bf16x8_t*>(kt + (k_off ^ (ks * 32u)));
    };
    auto qk_from = [&](const bf16x8_t (&kf)[KSTEPS]) {
      f32x16_t sacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], sacc, 0, 0, 0);
      return sacc;
    };
    // The SIMD arbiter favours its oldest wave; left alone, that wave finishes its steps early and
    // idles at the barrier while the youngest runs the tail alone.  Each wave therefore lowers its own
    // priority as it advances (quarter by quarter), so a wave that is behind is served first.
    auto fast_pass = [&](uint32_t n_valid, int32_t tail_keys) {
      m_ref = 0.f;
      l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      bf16x8_t kf[2][KSTEPS];
      load_k(0, kf[0]);
      if (NSTEP > 1) load_k(1, kf[1]);
      f32x16_t sc[2];
      sc[0] = qk_from(kf[0]);
      __builtin_amdgcn_s_setprio(3);
      static_for<NSTEP>([&](auto st_c) {
        constexpr uint32_t st = decltype(st_c)::value;
        if (st < n_valid) {                 // uniform
          if (st == QSTEP) __builtin_amdgcn_s_setprio(2);
          if (st == 2 * QSTEP) __builtin_amdgcn_s_setprio(1);
          if (st == 3 * QSTEP) __builtin_amdgcn_s_setprio(0);
          f32x16_t& s_cur = sc[st & 1u];
          if constexpr (st + 1 < NSTEP) sc[(st + 1) & 1u] = qk_from(kf[(st + 1) & 1u]);
          if constexpr (st + 2 < NSTEP) load_k(st + 2, kf[st & 1u]);
          bf16x8_t vf[2];
          load_v(st, vf);
          if (st + 1 == n_valid && tail_keys < 32) {
            // (the empty asm keeps this a branch taken once per item instead of selects in every step)
            asm volatile("; boundary step: mask the keys past the valid length");
            // register i of a lane is key (i/4)*8 + 4 half + i%4 of the step
            const int32_t thr = tail_keys - (int32_t)half * 4;
#pragma unroll
            for (int i = 0; i < 16; ++i)
              if ((i / 4) * 8 + (i % 4) >= thr) s_cur[i] = -INFINITY;
          }
          uint32_t pb[8];
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(s_cur[i]), __builtin_amdgcn_exp2f(s_cur[i + 1]));
            l_run = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pb[i / 2]),
                                                    __builtin_bit_cast(bf16x2_t, 0x3F803F80u), l_run, false);
          }
          pv(pb, vf);
        }
      });
      __builtin_amdgcn_s_setprio(3);
    };

    // ---- general pass: masked keys, running-maximum softmax with the scale applied in fp32 ----
    // (one step at a time, no overlap; Q is read again because the fast pass only keeps the pre-scaled copy)
    auto general_pass = [&]() {
      bf16x8_t qr[KSTEPS];
      {
        const uint32_t off = ((q_row * ld) + half * 8) * 2u;
        const char* qp = reinterpret_cast<const char*>(q + item_base(item));
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) qr[ks] = *reinterpret_cast<const bf16x8_t*>(qp + (off + ks * 32u));
      }
      m_ref = -INFINITY;
      l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
      for (uint32_t st = 0; st < NSTEP; ++st) {
        // step st covers the 32 keys [32 st, 32 st + 32): position inside its bucket and that bucket's length
        const uint32_t jb = (st * 32u) / bs;
        const int32_t in_b = (int32_t)(st * 32u - jb * bs);
        const int32_t len = jb == 0 ? blen0 : jb == 1 ? blen1 : jb == 2 ? blen2 : blen3;
        if (in_b >= len) continue;          // no valid key in this step (uniform)
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
        const char* kt = sbuf + st * 32u * ROWB;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(kt + (k_off ^ (ks * 32u)));
          sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qr[ks], sc, 0, 0, 0);
        }
        bf16x8_t vf[2];
        load_v(st, vf);
        if (in_b + 32 > len) {
          // register i of a lane is key (i/4)*8 + 4 half + i%4 of the step
          const int32_t thr = len - in_b - (int32_t)half * 4;
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if ((i / 4) * 8 + (i % 4) >= thr) sc[i] = -INFINITY;
        }
        float mx = sc[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, sc[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        const float m_new = fmaxf(m_ref, mx * scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_ref - m_use);
        m_ref = m_new;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = __builtin_fmaf(sc[i], scale_log2, -m_use);
        uint32_t pb[8];
        float psum;
        exp_pack(sc, pb, psum);
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] *= alpha;
        pv(pb, vf);
      }
      if (m_ref == -INFINITY) m_ref = 0.f;
    };

    const bool any_valid = blen0 > 0 || blen1 > 0 || blen2 > 0 || blen3 > 0;
    const bool all_full = blen0 == (int32_t)bs && (scope_size < 2 || blen1 == (int32_t)bs) &&
                          (scope_size < 3 || blen2 == (int32_t)bs) && (scope_size < 4 || blen3 == (int32_t)bs);
    // queries at or beyond the valid length of their bucket produce zeros: a wave that owns only such rows has
    // nothing to compute (uniform per wave)
    const bool wave_has_rows = (int32_t)(q_local - qj * bs) < q_valid_len;
    if (q_exists && any_valid && wave_has_rows) {
      // the fast pass takes scopes whose keys are all valid, and one-bucket scopes with a valid prefix
      bool redo = !(all_full || scope_size == 1);
      if (!redo) {
        const uint32_t n_valid = all_full ? NSTEP : (uint32_t)(blen0 + 31) / 32u;
        const int32_t tail_keys = all_full ? 32 : blen0 - (int32_t)(n_valid - 1) * 32;
        fast_pass(n_valid, tail_keys);
        // redo with a moving reference if any row sum left the safe range (also catches inf / nan)
        const float l_chk = l_run + __shfl_xor(l_run, 32, kWave);
        redo = __ballot(!(l_chk > 0x1p-24f) || !(l_chk < 0x1p24f)) != 0;
      }
      if (redo) general_pass();
    } else {
      l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    }
    const float m_run = m_ref;
    if (n + 2 < my_items) load_table_len();
    // This wave's direct loads (issued a whole item ago) must have landed before the barrier below;
    // wait for them BEFORE the output stores are issued, so that the stores stay fire-and-forget
    // (vmcnt = 0, other counters untouched).
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (q_exists) {   // a scope entry outside the sequence names no rows
      const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
      const bool row_ok = (int32_t)q_in_bucket < q_valid_len && l_tot > 0.f;
      const float inv = row_ok ? 1.0f / l_tot : 0.f;
      // uniform 64-bit base of (batch element, head) + 32-bit lane offset
      const size_t obase = (size_t)(item / (num_head * num_scope)) * seq_len * num_head + item % num_head;
      char* op = reinterpret_cast<char*>(o + obase * D);
      const uint32_t orow_b = q_row * num_head * D * 2u;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t d0 = g * 8 + half * 4;
        if (D >= 32 || d0 < (uint32_t)D) {
          uint2 w;
          w.x = pack_bf16x2(acc[g * 4 + 0] * inv, acc[g * 4 + 1] * inv);
          w.y = pack_bf16x2(acc[g * 4 + 2] * inv, acc[g * 4 + 3] * inv);
          *reinterpret_cast<uint2*>(op + (orow_b + d0 * 2u)) = w;
        }
      }
      if (half == 0) {
        const float ln2 = 0.69314718055994530942f;
        *reinterpret_cast<float*>(reinterpret_cast<char*>(lse + obase) + q_row * num_head * 4u) =
            row_ok ? (m_run + __builtin_amdgcn_logf(l_tot)) * ln2 : 0.f;
      }
    }
    if (n + 2 < my_items) store_table(tnext2);
    __syncthreads();   // next buffer is complete; this buffer is free for the item after next
  }
}

template <int D, int T>
static int launch_attn_resident(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, uint16_t* o,
                                float* lse, const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size,
                                uint32_t bs, uint32_t batch, uint32_t seq_len, uint32_t num_head,
                                const int32_t* kv_len, int device, hipStream_t s) {
  const uint64_t n_items64 = (uint64_t)batch * num_scope * num_head;
  if (n_items64 == 0) return F3D_OK;
  if (n_items64 > 0x7FFFFFF0ull) {
    set_error("attention problem too large for one launch (%llu items)", (unsigned long long)n_items64);
    return F3D_ERR_INVALID;
  }
  const uint32_t n_items = (uint32_t)n_items64;
  int n_cu = 0;
  F3D_CHECK_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device));
  constexpr size_t lds = resident_lds_bytes<D, T>();
  const uint32_t wg_per_cu = (2 * T <= 512 && 2 * lds <= 160 * 1024) ? 2u : 1u;
  // workgroups: a multiple of the XCD count, no more than the chip holds at once, no more than items need
  const uint32_t items_per_xcd = cdiv_u32(n_items, kNumXcd);
  const uint32_t n_slots = std::max(1u, std::min((uint32_t)n_cu * wg_per_cu / kNumXcd, items_per_xcd));
  const float scale_log2 = 1.4426950408889634f / sqrtf((float)D);
  static bool attr_set[64] = {};   // raise the dynamic LDS limit once per instantiation and device
  if (device < 0 || device >= 64 || !attr_set[device]) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)buck_swin_fwd_resident_kernel<D, T>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (device >= 0 && device < 64) attr_set[device] = true;
  }
  hipLaunchKernelGGL((buck_swin_fwd_resident_kernel<D, T>), dim3(n_slots * kNumXcd), dim3(2 * T), lds, s, q, k, v, ld,
                     o, lse, scope_buckets, num_scope, scope_size, bs, seq_len, num_head, kv_len, scale_log2, n_items,
                     items_per_xcd, n_slots);
  return F3D_OK;
}

template <int D, int KT>
static int launch_attn(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, uint16_t* o, float* lse,
                       const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                       uint32_t batch, uint32_t seq_len, uint32_t num_head, const int32_t* kv_len, hipStream_t s) {
  using C = AttnCfg<D, KT>;
  const uint64_t n_work64 = (uint64_t)batch * num_scope * num_head * (scope_size * bs / kQBlock);
  if (n_work64 == 0) return F3D_OK;
  if (n_work64 > 0x7FFFFFF0ull) {
    set_error("attention problem too large for one launch (%llu workgroups)", (unsigned long long)n_work64);
    return F3D_ERR_INVALID;
  }
  const uint32_t n_work = (uint32_t)n_work64;
  const uint32_t per_xcd = cdiv_u32(n_work, kNumXcd);
  const float scale_log2 = 1.4426950408889634f / sqrtf((float)D);
  hipLaunchKernelGGL((buck_swin_fwd_kernel<D, KT>), dim3(per_xcd * kNumXcd), dim3(kAttnThreads),
                     C::LDS_BYTES + scope_size * 8, s, q, k,
                     v, ld, o, lse, scope_buckets, num_scope, scope_size, bs, seq_len, num_head, kv_len, scale_log2,
                     n_work, per_xcd);
  return F3D_OK;
}

}  // namespace f3d

extern "C" {

int f3d_buck_swin_fwd_strided(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v, uint32_t qkv_row_stride,
                              f3d_bf16_t* o, float* lse, const uint32_t* scope_buckets, uint32_t num_scope,
                              uint32_t scope_size, uint32_t bucket_size, uint32_t batch, uint32_t seq_len,
                              uint32_t num_head, uint32_t head_dim, const int32_t* kv_len, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(q && k && v && o && lse && scope_buckets, "null tensor pointer");
  F3D_CHECK_ARG(head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128,
                "No kernel found for head_dim=%u (supported: 16, 32, 64, 128)", head_dim);
  F3D_CHECK_ARG(bucket_size >= 128 && bucket_size % 128 == 0, "bucket_size=%u must be a multiple of 128",
                bucket_size);
  F3D_CHECK_ARG(scope_size >= 1 && scope_size <= 8192, "scope_size=%u outside [1, 8192]", scope_size);
  F3D_CHECK_ARG(seq_len % bucket_size == 0, "sequence length %u is not a multiple of bucket_size=%u", seq_len,
                bucket_size);
  F3D_CHECK_ARG(qkv_row_stride >= num_head * head_dim && qkv_row_stride % 8 == 0,
                "q/k/v row stride %u must be a multiple of 8 and at least num_head*head_dim=%u", qkv_row_stride,
                num_head * head_dim);
  F3D_CHECK_ARG((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15u) == 0,
                "q/k/v/o must be 16-byte aligned");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  int rc;
  // scopes of 256 or 512 tokens with narrow heads: K / V resident in LDS, persistent workgroups
  const uint32_t scope_tokens = scope_size * bucket_size;
  if (head_dim <= 32 && scope_size <= (uint32_t)kResMaxScope && (scope_tokens == 256 || scope_tokens == 512) &&
      (uint64_t)seq_len * qkv_row_stride * 2 < (1ull << 32)) {
#define F3D_RES(DD, TT)                                                                                         \
  rc = launch_attn_resident<DD, TT>(q, k, v, qkv_row_stride, o, lse, scope_buckets, num_scope, scope_size,      \
                                    bucket_size, batch, seq_len, num_head, kv_len, device, s)
    if (head_dim == 16) {
      if (scope_tokens == 256) F3D_RES(16, 256); else F3D_RES(16, 512);
    } else {
      if (scope_tokens == 256) F3D_RES(32, 256); else F3D_RES(32, 512);
    }
#undef F3D_RES
    if (rc != F3D_OK) return rc;
    F3D_CHECK_HIP(hipGetLastError());
    return F3D_OK;
  }
#define F3D_ATTN(DD, KK)                                                                                            \
  rc = launch_attn<DD, KK>(q, k, v, qkv_row_stride, o, lse, scope_buckets, num_scope, scope_size, bucket_size, batch, \
                           seq_len, num_head, kv_len, s)
  switch (head_dim) {
    case 16: F3D_ATTN(16, 128); break;
    case 32: F3D_ATTN(32, 64); break;
    case 64: F3D_ATTN(64, 64); break;
    default: F3D_ATTN(128, 64); break;
  }
#undef F3D_ATTN
  if (rc != F3D_OK) return rc;
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_buck_swin_fwd(const f3d_bf16_t* q, const f3d_bf16_t* k, const f3d_bf16_t* v, f3d_bf16_t* o, float* lse,
                      const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bucket_size,
                      uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t head_dim, const int32_t* kv_len,
                      int device, void* stream) {
  return f3d_buck_swin_fwd_strided(q, k, v, num_head * head_dim, o, lse, scope_buckets, num_scope, scope_size,
                                   bucket_size, batch, seq_len, num_head, head_dim, kv_len, device, stream);
}

}  // extern "C"
