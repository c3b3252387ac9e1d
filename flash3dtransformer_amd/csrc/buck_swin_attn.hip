// Bucketed (scoped) multi-head attention forward for gfx950.
//
// Counterpart of pshattn.buck_swin_fwd (declared src/f3d_frontend.cu:90-92, called from
// flash3dxfmr/layers/buck_swin.py:57; the reference ships no kernel source for it).  For every
// batch row, every scope (a row of scope_buckets) and every head: softmax(Q Kt / sqrt(D)) V over the
// rows of the scope's buckets, plus the natural-log LSE.
//
// Streaming kernel (any scope size, head_dim up to 128): one 256-thread workgroup (4 waves) per (batch, scope,
// head, 128-query block); each wave owns 32 query rows.  K and V of the scope stream through LDS in tiles of KT keys (K row-major;
// V row-major too for 32-wide heads, read with the transposing LDS load, and stored transposed for the other widths),
// prefetched into registers one tile ahead.  Scores are computed TRANSPOSED,
// St = K Qt with v_mfma_f32_32x32x16_bf16, so that a lane holds 16 keys of ONE query: the softmax
// max / sum run inside the lane plus one exchange with lane^32, and the bf16 P values are already in
// the B-operand layout of the second MFMA, Ot += Vt Pt (keys are consumed in the permuted order the
// accumulator layout yields; V is staged in that same order).  Softmax runs in the exp2 domain with
// fp32 accumulation: first with the reference fixed at zero and pre-scaled Q (no running maximum, no
// rescaling, row sums from the matrix core), and again with a running maximum for a workgroup whose row
// sums left the safe range.  Workgroup ids are remapped so that the workgroups of one scope (which share
// K/V and the 512-byte token rows) land on the same XCD and its L2.
#include <type_traits>
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

typedef short i16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(3))) i16x4_t lds_i16x4_t;

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
  // 32-wide heads keep V row-major [KT][D] (unpadded, as the global rows) and read it with the transposing LDS load;
  // the other widths stage a transposed copy [D][VROW]
  static constexpr bool V_ROW_MAJOR = D == 32;
  static constexpr int V_ELEMS = V_ROW_MAJOR ? KT * D : D * VROW;
  static constexpr int LDS_BYTES = (KT * KROW + V_ELEMS) * 2;   // plus 8 bytes per scope entry
};

template <int D, int KT>
__global__ __launch_bounds__(kAttnThreads) void buck_swin_fwd_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    uint16_t* __restrict__ o, float* __restrict__ lse, const uint32_t* __restrict__ scope_buckets,
    uint32_t num_scope, uint32_t scope_size, uint32_t bs, uint32_t seq_len, uint32_t num_head,
    const int32_t* __restrict__ kv_len, float scale_log2, uint32_t n_work, uint32_t work_per_xcd,
    uint32_t only_marked) {
  using C = AttnCfg<D, KT>;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds_attn[];
  uint16_t* sK = lds_attn;                  // [KT][KROW]
  uint16_t* sVt = lds_attn + KT * C::KROW;  // [D][VROW]
  // per scope entry: bucket id and number of valid keys (0 for an id outside the sequence), read once
  // from global memory so that the tile loop never waits on a scalar load
  uint32_t* s_bucket = reinterpret_cast<uint32_t*>(lds_attn + KT * C::KROW + C::V_ELEMS);
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
  // only_marked: this launch follows the bucket-streaming scope kernel, which leaves a NaN in the LSE of the rows whose
  // sums left the range of its fixed-reference softmax; only workgroups that own such a row go on (uniform decision)
  if (only_marked) {
    const float mark = lse[(tok0 + q_row) * num_head + head];
    if (!__syncthreads_or(mark != mark ? 1 : 0)) return;
  }

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
        if constexpr (C::V_ROW_MAJOR) {
          *reinterpret_cast<u32x4_t*>(sVt + key * D + dc * 8) = rv[i];
        } else {
          const uint32_t pos = (key & ~15u) | vperm16(key & 15u);
          uint16_t* col = sVt + (dc * 8) * C::VROW + pos;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            col[(2 * e) * C::VROW] = (uint16_t)(rv[i][e] & 0xFFFFu);
            col[(2 * e + 1) * C::VROW] = (uint16_t)(rv[i][e] >> 16);
          }
        }
      }
    }
  };
  // V^T operand of the 16 keys [key0, key0 + 16) of the staged tile (32-wide heads): the transposing load hands lane i
  // of a 16-lane block column i % 4 of the four 8-byte pieces addressed by lanes i / 4 + {0, 4, 8, 12}; with lane r
  // pointing at key r / 4, features 4 (r % 4) .., slots 0..3 of a lane are keys 4 half + 0..3, slots 4..7 the same + 8:
  // the key order of the packed P values
  const uint32_t v_tr_off = (4u * half + (lane & 15u) / 4u) * D + 16u * ((lane >> 4) & 1u) + 4u * (lane & 3u);   // elements
  auto v_frag_tr = [&](uint32_t key0) {
    const uint16_t* vt = sVt + key0 * D + v_tr_off;
    const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)vt);
    const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_t*)(vt + 8 * D));
    return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // ---- fast pass: softmax with the reference fixed at zero.  Q is pre-multiplied by log2(e) / sqrt(D) (one bf16
  //      rounding), so the score product emits exponents and the vector unit only exponentiates and packs; the row
  //      sums come from the matrix core (a 16x16x32 product of P with a 0 / 1 selector, see the scope-resident
  //      kernel below).  Exact as long as the numbers stay in range (softmax is shift-invariant, fp32 and bf16 share
  //      the exponent range); a workgroup with a row sum outside [2^-24, 2^24) (or not a number) redoes its scope
  //      with the running-maximum pass after it. ----
  bool redo = false, any_tile = false;
  {
    bf16x8_t qs[C::KSTEPS];
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ++ks) {
      const u32x4_t raw = __builtin_bit_cast(u32x4_t, qf[ks]);
      u32x4_t sc;
#pragma unroll
      for (int e = 0; e < 4; ++e) sc[e] = pack_bf16x2(bf16_lo(raw[e]) * scale_log2, bf16_hi(raw[e]) * scale_log2);
      qs[ks] = __builtin_bit_cast(bf16x8_t, sc);
    }
    bf16x8_t ones_sel;
    {
      const uint32_t m = lane & 15u, kb = lane >> 4;
      const __bf16 val = ((m < 8u) == ((kb & 1u) == 0u)) ? (__bf16)1.0f : (__bf16)0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ones_sel[e] = val;
    }
    f32x4_t lacc = {0.f, 0.f, 0.f, 0.f};
    bool have = settle();
    if (have) fetch(jb, kt);
    while (have) {
      any_tile = true;
      const uint32_t cur_kt = kt;
      const int32_t cur_len = bucket_len(jb);
      __syncthreads();  // every wave is done reading the previous tile
      stage();
      __syncthreads();
      ++kt;
      if (kt == tiles_per_bucket) { ++jb; kt = 0; }
      have = settle();
      if (have) fetch(jb, kt);
      const bool boundary = (int32_t)((cur_kt + 1) * KT) > cur_len;   // uniform
#pragma unroll
      for (int j = 0; j < C::NSUB; ++j) {
        f32x16_t sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < C::KSTEPS; ++ks) {
          const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(sK + (j * 32 + lq) * C::KROW + ks * 16 + half * 8);
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qs[ks], sacc, 0, 0, 0);
        }
        if (boundary) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int32_t key = cur_kt * KT + j * 32 + (i / 4) * 8 + half * 4 + (i % 4);
            if (key >= cur_len) sacc[i] = -INFINITY;
          }
        }
        uint32_t pb[8];
#pragma unroll
        for (int i = 0; i < 16; i += 2)
          pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(sacc[i]), __builtin_amdgcn_exp2f(sacc[i + 1]));
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
          const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
#pragma unroll
          for (int dt = 0; dt < C::DT; ++dt) {
            bf16x8_t vf;
            if constexpr (C::V_ROW_MAJOR) {
              vf = v_frag_tr(j * 32 + kk * 16);
            } else if (D >= 32 || lq < (uint32_t)D) {
              vf = *reinterpret_cast<const bf16x8_t*>(sVt + (dt * 32 + lq) * C::VROW + j * 32 + kk * 16 + half * 8);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e) vf[e] = (__bf16)0.f;
            }
            acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[dt], 0, 0, 0);
          }
          lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones_sel, pf, lacc, 0, 0, 0);
        }
      }
    }
    // lanes 0-31 of the selector product hold the row sums of queries 0-15 (lane % 16), lanes 32-63 those of 16-31
    const float l_fast = __shfl(lacc[0], (lq < 16u ? 0u : 32u) + (lq & 15u), kWave);
    redo = any_tile && __syncthreads_or((!(l_fast > 0x1p-24f) || !(l_fast < 0x1p24f)) ? 1 : 0) != 0;
    // the epilogue's formula: O = acc / l, LSE = (m + log2 l) ln 2 with m = 0; l_run is halved because the epilogue
    // adds the two half-waves' partial sums of the running-maximum pass
    m_run = any_tile ? 0.f : -INFINITY;
    l_run = 0.5f * l_fast;
  }
  if (redo) {
    // ---- general pass: running-maximum softmax with the scale applied in fp32, from the start of the scope ----
    jb = 0; kt = 0;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
    m_run = -INFINITY; l_run = 0.f;
    {
      // unscaled Q, read again: the fast pass kept only its pre-scaled copy
      const uint16_t* qp = q + (tok0 + q_row) * ld + head * D + half * 8;
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + ks * 16);
    }
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
            if constexpr (C::V_ROW_MAJOR) {
              vf = v_frag_tr(j * 32 + kk * 16);
            } else if (D >= 32 || lq < (uint32_t)D) {
              vf = *reinterpret_cast<const bf16x8_t*>(sVt + (dt * 32 + lq) * C::VROW + j * 32 + kk * 16 + half * 8);
            } else {
  #pragma unroll
              for (int e = 0; e < 8; ++e) vf[e] = (__bf16)0.f;
            }
            acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc[dt], 0, 0, 0);
          }
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

// the same with the LDS address given as a (wave-uniform) 32-bit number
__device__ __forceinline__ void lds_dma16_at(const void* gbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}

// ---- scope-resident kernel --------------------------------------------------------------------------
// When a scope holds 256 or 512 tokens and head_dim <= 32 (the shape of every block of the Flash3D model: one
// 512-row bucket per scope, 32-wide heads) the K and V of a (batch, scope, head) item fit in LDS twice.  One
// persistent workgroup of WAVES waves walks a list of items: the current item's K and V sit in one LDS buffer
// (2 T D bytes each) while the next item's stream HBM -> LDS directly (global_load ... lds, no registers) into the
// other and its Q into registers; one barrier per item.  A wave owns QB = T / (32 WAVES) blocks of 32 queries
// (one with the T / 32 waves the launcher picks: four waves per SIMD at under 128 registers, nothing spills, so no
// scratch reload ever waits behind the direct loads in flight) and walks the flattened sequence (step, block):
// every K / V fragment read from LDS feeds all of its blocks.
//
// LDS layout of one buffer: K [T][D] then V [T][D], both row-major exactly as the direct loads write them (a
// wave's 64 lanes fill 1 KB = 1024/(2D) consecutive rows).  K rows carry no padding: the 16-byte chunk c of row r
// is stored at position c ^ swz(r), swz(r) = (r / (128/D)) mod (D/8), which spreads the 32 rows of a ds_read_b128
// over all banks.  V is read with ds_read_b64_tr_b16, which hands lane i of a 16-lane block column i%4 of the four
// 8-byte pieces addressed by lanes i/4 + {0,4,8,12}: with lane r pointing at key r/4, features 4(r%4).., a lane
// receives one feature of four consecutive keys, i.e. the MFMA A operand of V^T, with no transposed copy of V
// anywhere.  Scores are computed transposed (S^T = K Q^T, a lane holds 16 keys of one query), so the packed P
// values already are the B operand of O^T += V^T P^T.
//
// Softmax without a running maximum (fast pass): Q is pre-multiplied by log2(e)/sqrt(D) (one bf16 rounding), so
// the score MFMA emits exponents and the VALU only exponentiates and packs: P = 2^S with the reference fixed at
// zero.  Softmax is shift-invariant and fp32 / bf16 share an 8-bit exponent, so this is exact as long as the
// numbers stay in range; a wave whose total row sum reaches 2^24 or stays under 2^-24 (scores that large also
// magnify the rounding of the pre-scaled Q) redoes its item with the general pass: unscaled Q, scale applied in
// fp32, running maximum.  Masked keys of a one-bucket scope are handled inside the fast pass (steps past the
// valid length are skipped, the boundary step gets -inf scores, 2^-inf = 0 exactly); scopes of several buckets of
// which some are partly valid take the general pass.
//
// What bounds the pass is the vector unit's issue port: per 32 x 32 scores a wave issues 16 v_exp_f32 (two slots
// each), 8 v_cvt_pk_bf16_f32 and six MFMAs (each holds the port for about nine clocks): 228 clocks measured for
// that mix alone against 160 clocks of matrix-core time.  Hence: the scores of the next (step, block) are issued before the
// exponentials of the current one, so that the matrix core works under them; the row sums come from the matrix
// core too (one 16x16x32 product of P with a 0 / 1 selector per 16 keys, a quarter of a score product, instead
// of eight dot instructions on the vector unit); the steps are fully unrolled (LDS offsets are immediates, no
// address arithmetic); the next item's loads are issued a few per step (all at once they hold every wave at the
// memory pipeline's door for a microsecond with the SIMDs idle).
template <int D, int T, int WAVES>
constexpr size_t scope_lds_bytes() {
  return (size_t)2 * 2 * T * D * 2;
}

// GEN: Q, K and V are not read but formed from the rows' coordinates (the first block of a model, whose input is the
// coordinate embedding: LayerNorm and the QKV projection of a rank-4 input fold into one 4-column matrix per output
// row plus a per-row scale).  `table` holds, per head and tile (0: Q in the exponent's units, 1: K, 2: V, 3: Q
// unscaled, for the general pass), 32 rows of 16 bf16, the A operand of one 32x32x16 product; `chol` the
// upper-triangular factor of the embedding's centred Gram matrix (10 numbers) and the LayerNorm epsilon.
struct ScopeGen {
  const uint16_t* coord;   // [batch * seq_len][3] fp16
  const uint16_t* table;   // [num_head][4][32][16] bf16
  const float* chol;       // L00 L01 L02 L03 L11 L12 L13 L22 L23 L33 eps
};

// STREAM: scopes of more than 512 tokens in buckets of exactly T rows.  An item is (batch, scope, head, query bucket); the
// scope's key buckets pass through the two LDS buffers one after the other (the next one streams in while the current one
// is consumed, exactly as the next item does otherwise) and the accumulators live across them.  Fixed-reference softmax
// only: a wave whose row sums leave its range writes NaN into its rows' LSE instead of a result, and the launcher runs
// the streaming kernel after this one for the workgroups that own such rows.
template <int D, int T, int WAVES, bool GEN = false, bool STREAM = false>
__global__ __launch_bounds__(64 * WAVES) void buck_swin_fwd_scope_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v, uint32_t ld,
    uint16_t* __restrict__ o, float* __restrict__ lse, const uint32_t* __restrict__ scope_buckets,
    uint32_t num_scope, uint32_t scope_size, uint32_t bs, uint32_t seq_len, uint32_t num_head,
    const int32_t* __restrict__ kv_len, float scale_log2, uint32_t n_items, uint32_t items_per_xcd,
    uint32_t n_slots, ScopeGen gen) {
  constexpr int QB = T / (32 * WAVES);     // 32-query blocks per wave
  static_assert(!GEN || (QB == 1 && D == 32), "rows formed in the kernel: one 32-row block per wave, 32-wide heads");
  static_assert(!(GEN && STREAM), "rows are formed in the kernel for resident scopes only");
  const uint32_t n_kb = STREAM ? scope_size : 1u;       // key buckets an item walks
  constexpr int KSTEPS = D / 16;
  constexpr int CPK = D / 8;               // 16-byte chunks per row
  constexpr int ROWB = D * 2;              // bytes per K / V row in LDS
  constexpr int RPB = 1024 / ROWB;         // rows one direct-load instruction fills
  constexpr int BPW = T / RPB / WAVES;     // direct-load instructions per wave and operand
  constexpr int SWZ_DIV = 16 / CPK;        // rows sharing one swizzle value
  constexpr int OPB = T * ROWB;            // bytes of one operand (K or V)
  constexpr int BUF = 2 * OPB;             // bytes of one K + V buffer
  constexpr uint32_t NSTEP = T / 32;
  static_assert(QB >= 1 && BPW >= 1 && (T / WAVES) % 32 == 0 && (T / WAVES) % RPB == 0, "a wave owns whole 32-query blocks and whole direct-load blocks");
  extern __shared__ __attribute__((aligned(16))) char lds_scope[];

  const uint32_t tid = threadIdx.x, lane = tid % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const uint32_t lq = lane & 31u, half = lane >> 5;
  const uint32_t n_bucket = seq_len / bs;
  const uint32_t xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
  const uint32_t item_lo = xcd * items_per_xcd + slot;
  const uint32_t item_hi = min((xcd + 1) * items_per_xcd, n_items);
  if (item_lo >= item_hi) return;        // whole workgroup: no barrier has been passed yet
  const uint32_t my_items = (item_hi - item_lo + n_slots - 1) / n_slots;

  // per-lane LDS byte offsets of the fragment reads
  const uint32_t k_off = lq * ROWB + ((half ^ ((lq / SWZ_DIV) & (CPK - 1))) * 16u);   // k-step ks: ^ (ks * 32)
  const uint32_t l16 = lane & 15u, d_base = 16u * ((lane >> 4) & 1u);
  const uint32_t v_off = OPB + (4u * half + l16 / 4u) * ROWB + (d_base + 4u * (l16 & 3u)) * 2u;
  const bool v_lane = D >= 32 || d_base < (uint32_t)D;   // lanes whose V^T row exists
  // per-lane byte offsets of the direct loads inside a block of RPB rows: lane l fills LDS bytes [16 l, 16 l + 16)
  // of the block, i.e. row l / CPK, chunk l % CPK; for K that chunk holds the row's chunk (l % CPK) ^ swizzle(row)
  const uint32_t dma_row = lane / CPK, dma_pos = lane % CPK;
  const uint32_t dma_k = (dma_row * ld + (dma_pos ^ ((dma_row / SWZ_DIV) & (CPK - 1))) * 8u) * 2u;
  const uint32_t dma_v = (dma_row * ld + dma_pos * 8u) * 2u;
  // Row-sum selector, the A operand of a 16x16x32 product whose B operand is a P fragment in the layout of the
  // 32x32x16 product (lane = query lane % 32, keys 8 (lane / 32) ..): as a 16x16x32 operand the fragment's lane is
  // (column lane % 16, k-block lane / 16), so even k-blocks hold queries 0-15 and odd ones queries 16-31.  Rows
  // 0-7 of the selector take the even k-blocks, rows 8-15 the odd ones: lanes 0-31 of the result hold the row sums
  // of queries 0-15 (lane % 16), lanes 32-63 those of queries 16-31, every register the same number.
  bf16x8_t ones_sel;
  {
    const uint32_t m = lane & 15u, kb = lane >> 4;
    const __bf16 val = ((m < 8u) == ((kb & 1u) == 0u)) ? (__bf16)1.0f : (__bf16)0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones_sel[e] = val;
  }
  const uint32_t l_src = (lq < 16u ? 0u : 32u) + (lq & 15u);

  // ---- item -> (head, scope, batch); the scope's bucket ids / valid key counts ----
  // An item index is head + num_head (scope + num_scope batch).  A workgroup's items are n_slots apart: its position
  // advances by a mixed-radix addition with carries, one division at the start and none per item (the scalar unit
  // is shared by all waves of a SIMD, and every wave does this bookkeeping).
  struct Pos {
    uint32_t qb, head, scope, batch;      // qb: the item's query bucket inside its scope (STREAM; 0 otherwise)
  };
  // STREAM: the query bucket is the fastest index, so that the items that share a scope's K and V run at the same time
  // on one XCD
  const uint32_t slots_h = n_slots / n_kb;
  const uint32_t d_qb = n_slots % n_kb, d_head = slots_h % num_head, d_scope = (slots_h / num_head) % num_scope,
                 d_batch = slots_h / (num_head * num_scope);
  auto advance = [&](Pos p) {
    uint32_t carry = 0;
    if constexpr (STREAM) {
      p.qb += d_qb;
      carry = p.qb >= n_kb ? 1u : 0u;
      p.qb -= carry ? n_kb : 0u;
    }
    p.head += d_head + carry;
    carry = p.head >= num_head ? 1u : 0u;
    p.head -= carry ? num_head : 0u;
    p.scope += d_scope + carry;
    carry = p.scope >= num_scope ? 1u : 0u;
    p.scope -= carry ? num_scope : 0u;
    p.batch += d_batch + carry;
    return p;
  };
  auto in_base = [&](const Pos& p) {      // element offset of (first token of the batch element, head), uniform
    return (size_t)p.batch * seq_len * ld + (size_t)p.head * D;
  };
  // Lane j < scope_size of every wave reads bucket j of an item's scope (two dependent loads, issued long before
  // their use); the consumer picks entries with v_readlane.
  auto load_ids = [&](const Pos& p) -> uint32_t {
    return lane < scope_size ? scope_buckets[(size_t)p.scope * scope_size + lane] : 0xFFFFFFFFu;
  };
  auto load_len = [&](uint32_t ids) -> int32_t {
    return ids >= n_bucket ? 0 : (kv_len ? min(max(kv_len[ids], 0), (int32_t)bs) : (int32_t)bs);
  };
  struct Scope {
    uint32_t ids;     // lane j: bucket id of scope entry j (0xFFFFFFFF beyond scope_size)
    int32_t len;      // lane j: its valid key count (0 for an id outside the sequence)
  };
  auto bucket_of = [&](const Scope& sc, uint32_t j) { return (uint32_t)__builtin_amdgcn_readlane(sc.ids, j); };
  auto len_of = [&](const Scope& sc, uint32_t j) { return (int32_t)__builtin_amdgcn_readlane(sc.len, j); };

  // K and V rows [wave T/WAVES, (wave + 1) T/WAVES) of an item go straight into an LDS buffer, 2 BPW direct loads of
  // 1 KB per wave: load i < BPW is K block i of the wave, load BPW + i its V block i.  kv_base() is the byte offset of
  // the wave's first row (valid when kv_wanted()).  Issued as inline assembly on purpose: the compiler then keeps no
  // record of LDS writes in flight and puts no full vmcnt wait in front of the fragment reads (they read the OTHER
  // buffer).  The wait that matters is the explicit one before the per-item barrier.
  // (STREAM: the key bucket kb of the sub-item, whose T rows the waves share)
  const uint32_t kv_row0 = wave * (T / WAVES), kv_j0 = STREAM ? 0u : kv_row0 / bs;     // a wave's rows never straddle buckets
  auto kv_wanted = [&](const Scope& sc, uint32_t kb) { return len_of(sc, STREAM ? kb : kv_j0) > 0; };
  auto kv_base = [&](const Pos& p, const Scope& sc, uint32_t kb) {
    const uint32_t j = STREAM ? kb : kv_j0;
    return in_base(p) * 2u + (size_t)(bucket_of(sc, j) * bs + (kv_row0 - kv_j0 * bs)) * ld * 2u;
  };
  // LDS addresses as plain 32-bit numbers (a generic pointer costs a null check per conversion)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_scope;
  auto issue_kv_one = [&](size_t goff, uint32_t i, uint32_t buf_addr) {
    const uint32_t blk = wave * BPW + (i < (uint32_t)BPW ? i : i - BPW);
    const size_t g = goff + (size_t)(i < (uint32_t)BPW ? i : i - BPW) * RPB * ld * 2u;
    if (i < (uint32_t)BPW) lds_dma16_at(reinterpret_cast<const char*>(k) + g, dma_k, buf_addr + blk * 1024);
    else lds_dma16_at(reinterpret_cast<const char*>(v) + g, dma_v, buf_addr + OPB + blk * 1024);
  };
  // row inside the sequence of query lq of block b (0 when the scope entry names no bucket of the sequence)
  auto q_row_of = [&](const Pos& p, const Scope& sc, uint32_t b) {
    const uint32_t q_local = (wave * QB + b) * 32u, qj = STREAM ? 0u : q_local / bs;
    const uint32_t id = bucket_of(sc, STREAM ? p.qb : qj);
    return (id < n_bucket ? id : 0u) * bs + (q_local - qj * bs) + lq;
  };
  u32x4_t qraw[QB][KSTEPS];
  auto issue_q_one = [&](const Pos& p, const Scope& sc, auto b_c) {
    constexpr uint32_t b = decltype(b_c)::value;
    const char* qp = reinterpret_cast<const char*>(q + in_base(p));
    const uint32_t off = (q_row_of(p, sc, b) * ld + half * 8u) * 2u;      // fits 32 bits (checked by the host)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qraw[b][ks] = *reinterpret_cast<const u32x4_t*>(qp + (off + ks * 32u));
  };

  // ---- prologue: the first item's scope, K / V / Q; the second item's bucket ids ----
  const uint32_t item_h = item_lo / n_kb;
  Pos p_cur = {item_lo % n_kb, item_h % num_head, (item_h / num_head) % num_scope, item_h / (num_head * num_scope)};
  Pos p_nxt = advance(p_cur);
  Scope cur, nxt;
  cur.ids = load_ids(p_cur);
  cur.len = load_len(cur.ids);
  nxt.ids = my_items > 1 ? load_ids(p_nxt) : 0xFFFFFFFFu;
  nxt.len = load_len(nxt.ids);
  // GEN: what an item's rows are formed from, requested one item ahead: the three coordinates of the lane's row
  // (row lq of the wave's 32, which are its queries and its share of the keys) and the A operands of the head's
  // Q / K / V tiles
  uint16_t g_c[3] = {0, 0, 0};
  u32x4_t g_a[3];
  auto gen_row = [&](const Pos& p, const Scope& sc) { return (size_t)p.batch * seq_len + q_row_of(p, sc, 0); };
  auto gen_tile_ptr = [&](const Pos& p, uint32_t tile) {
    return reinterpret_cast<const u32x4_t*>(gen.table + (((size_t)p.head * 4 + tile) * 32 + lq) * 16 + half * 8);
  };
  auto issue_gen = [&](const Pos& p, const Scope& sc) {
    const uint16_t* cp = gen.coord + gen_row(p, sc) * 3;
#pragma unroll
    for (int j = 0; j < 3; ++j) g_c[j] = cp[j];
#pragma unroll
    for (int tl = 0; tl < 3; ++tl) g_a[tl] = *gen_tile_ptr(p, tl);
  };
  float chol[11];
  if constexpr (GEN) {
#pragma unroll
    for (int i = 0; i < 11; ++i) chol[i] = gen.chol[i];
  }
  // the rows' B operand: c~ = (x, y, z, 1) / sqrt(var + eps) as bf16 high and low parts; lanes < 32 carry the high
  // parts twice (against the matrix's high and low parts), lanes >= 32 the low parts and two ones (the bias)
  auto gen_rows_operand = [&](const uint16_t (&c)[3]) {
    float cc[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) cc[j] = bf16_bits_to_float(float_to_bf16_bits(half_bits_to_float(c[j])));
    const float t0 = __builtin_fmaf(chol[0], cc[0], __builtin_fmaf(chol[1], cc[1], __builtin_fmaf(chol[2], cc[2], chol[3])));
    const float t1 = __builtin_fmaf(chol[4], cc[1], __builtin_fmaf(chol[5], cc[2], chol[6]));
    const float t2 = __builtin_fmaf(chol[7], cc[2], chol[8]);
    const float var = __builtin_fmaf(t0, t0, __builtin_fmaf(t1, t1, __builtin_fmaf(t2, t2, chol[9] * chol[9])));
    const float rstd = __builtin_amdgcn_rsqf(var + chol[10]);
    const float s[4] = {cc[0] * rstd, cc[1] * rstd, cc[2] * rstd, rstd};
    float hi[4], lo[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      hi[j] = bf16_bits_to_float(float_to_bf16_bits(s[j]));
      lo[j] = s[j] - hi[j];
    }
    u32x4_t b;
    if (half == 0) {
      b[0] = pack_bf16x2(hi[0], hi[1]);
      b[1] = pack_bf16x2(hi[2], hi[3]);
      b[2] = b[0];
      b[3] = b[1];
    } else {
      b[0] = pack_bf16x2(lo[0], lo[1]);
      b[1] = pack_bf16x2(lo[2], lo[3]);
      b[2] = 0x3F803F80u;     // (1, 1)
      b[3] = 0u;
    }
    return __builtin_bit_cast(bf16x8_t, b);
  };
  // one tile of the rows' projection, transposed: register i of lane (lq, half) is feature 8 half + i (i < 8) or
  // 16 + 8 half + i - 8 of row lq, the order of the score product's Q operand and of the 16-byte pieces of a K / V row
  auto gen_tile = [&](const u32x4_t& a, const bf16x8_t& rows) {
    f32x16_t z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), rows, z, 0, 0, 0);
  };
  auto pack_tile = [&](const f32x16_t& x, int ks) {
    u32x4_t w;
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(x[ks * 8 + 2 * e], x[ks * 8 + 2 * e + 1]);
    return w;
  };
  if constexpr (GEN) {
    issue_gen(p_cur, cur);
  } else {
    static_for<QB>([&](auto b_c) { issue_q_one(p_cur, cur, b_c); });
    if (kv_wanted(cur, 0)) {
      const size_t goff = kv_base(p_cur, cur, 0);
#pragma unroll
      for (uint32_t i = 0; i < 2u * BPW; ++i) issue_kv_one(goff, i, lds0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    __syncthreads();
  }

  // One turn of the loop is a sub-item: an item, or (STREAM) one key bucket of an item.  What lives across an item's
  // key buckets is declared out here.
  uint32_t n = 0, kb = 0;           // item counter, key bucket inside the item
  bf16x8_t qf[QB][KSTEPS];
  uint32_t q_row[QB];
  bool q_live[QB], q_exists[QB];
  int32_t q_len[QB];
  f32x16_t acc[QB];
  f32x4_t lacc[QB];
  float m_ref[QB], l_fin[QB];
  bool any_keys = false;            // STREAM: some key bucket of the item so far held a valid key
  const uint32_t n_sub = my_items * n_kb;
  for (uint32_t sub = 0; sub < n_sub; ++sub) {
    const bool first = !STREAM || kb == 0, last = !STREAM || kb + 1 == n_kb;
    const bool has_next = n + 1 < my_items;
    const char* const sbuf = lds_scope + (sub & 1u) * BUF;

    // Q of this item arrived during the previous one: scale into the exponent's units and round once
    if constexpr (GEN) {
      // form the item's Q (kept in registers), K and V (the wave's 32 rows of this item's LDS buffer: the buffer's
      // last readers, two items back, passed the previous barrier), then meet the other waves
      const bf16x8_t rows = gen_rows_operand(g_c);
      const f32x16_t tq = gen_tile(g_a[0], rows), tk = gen_tile(g_a[1], rows), tv = gen_tile(g_a[2], rows);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) qf[0][ks] = __builtin_bit_cast(bf16x8_t, pack_tile(tq, ks));
      char* const wb = const_cast<char*>(sbuf) + wave * 32u * ROWB;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        *reinterpret_cast<u32x4_t*>(wb + (k_off ^ (ks * 32u))) = pack_tile(tk, ks);
        *reinterpret_cast<u32x4_t*>(wb + OPB + lq * ROWB + (half + 2u * ks) * 16u) = pack_tile(tv, ks);
      }
      if (has_next) issue_gen(p_nxt, nxt);
      wg_barrier_lds();
    } else if (first) {
#pragma unroll
    for (int b = 0; b < QB; ++b)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        u32x4_t sc;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          sc[e] = pack_bf16x2(bf16_lo(qraw[b][ks][e]) * scale_log2, bf16_hi(qraw[b][ks][e]) * scale_log2);
        qf[b][ks] = __builtin_bit_cast(bf16x8_t, sc);
      }
    }
    // The next item's operands go in flight during the first half of this item's passes, a few vector-memory
    // instructions per step (issued all at once they would hold every wave of the workgroup at the memory pipeline's door for a
    // microsecond or two with the SIMDs idle): `vm_next` counts those already issued, 2 BPW direct loads of K / V
    // first, then the Q rows of the wave's QB blocks.
    constexpr uint32_t VM_OPS = GEN ? 0u : 2u * BPW + QB, VM_PER_STEP = (VM_OPS + NSTEP / 2 - 1) / (NSTEP / 2);   // all in the first half
    // (STREAM: the next sub-item is the item's next key bucket, or the first one of the next item together with its Q)
    const bool nx_same = STREAM && !last;
    const bool nxt_kv = nx_same ? kv_wanted(cur, kb + 1) : (has_next && kv_wanted(nxt, 0));
    const size_t nxt_goff = !nxt_kv ? 0 : (nx_same ? kv_base(p_cur, cur, kb + 1) : kv_base(p_nxt, nxt, 0));
    const uint32_t nxt_buf = lds0 + ((sub + 1) & 1u) * BUF;
    auto issue_vm = [&](auto i_c) {
      constexpr uint32_t i = decltype(i_c)::value;
      if constexpr (i < 2u * BPW) {
        if (nxt_kv) issue_kv_one(nxt_goff, i, nxt_buf);
      } else if constexpr (i < VM_OPS) {
        if (has_next && last) issue_q_one(p_nxt, nxt, std::integral_constant<uint32_t, i - 2u * BPW>{});
      }
    };
    uint32_t vm_next = 0;
    const Pos p_nxt2 = advance(p_nxt);
    Scope nxt2;
    nxt2.ids = n + 2 < my_items ? load_ids(p_nxt2) : 0xFFFFFFFFu;

    // per block: do its rows exist / are they valid (uniform), how many of them, which rows
    if (first) {
      any_keys = false;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        const uint32_t q_local = (wave * QB + b) * 32u, qj = STREAM ? p_cur.qb : q_local / bs;
        const int32_t in_b = (int32_t)(STREAM ? q_local : q_local - qj * bs);
        q_exists[b] = bucket_of(cur, qj) < n_bucket;
        q_len[b] = len_of(cur, qj) - in_b;               // valid rows of the block, counted from its first row
        q_live[b] = q_exists[b] && q_len[b] > 0;
        q_row[b] = q_row_of(p_cur, cur, b);
        m_ref[b] = 0.f;
        l_fin[b] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) lacc[b][i] = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;
      }
    }

    auto load_k = [&](uint32_t st, bf16x8_t (&kf)[KSTEPS]) {
      const char* kt = sbuf + st * 32u * ROWB;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = *reinterpret_cast<const bf16x8_t*>(kt + (k_off ^ (ks * 32u)));
    };
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
    auto scores = [&](const bf16x8_t (&kf)[KSTEPS], const bf16x8_t (&qq)[KSTEPS]) {
      f32x16_t sacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qq[ks], sacc, 0, 0, 0);
      return sacc;
    };
    // P V^T and the row sums of one (step, block)
    auto pv_rowsum = [&](const uint32_t (&pb)[8], const bf16x8_t (&vf)[2], f32x16_t& a, f32x4_t& la) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
        const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
        a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kk], pf, a, 0, 0, 0);
        la = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones_sel, pf, la, 0, 0, 0);
      }
    };

    // ---- fast pass: scopes whose keys are all valid, and one-bucket scopes with a valid prefix (steps past it are
    //      skipped, the boundary step gets -inf scores: 2^-inf = 0 exactly) ----
    // (STREAM: the sub-item's key bucket stands where a one-bucket scope stands otherwise)
    const int32_t len0 = len_of(cur, STREAM ? kb : 0u);
    const bool any_valid = STREAM ? len0 > 0 : __ballot(cur.len > 0) != 0;
    const bool all_full = STREAM ? len0 == (int32_t)bs : __ballot(lane < scope_size && cur.len != (int32_t)bs) == 0;
    bool any_live = false;
#pragma unroll
    for (int b = 0; b < QB; ++b) any_live = any_live || q_live[b];
    bool redo = false, failed = false;
    if (any_valid && any_live) {
      any_keys = true;
      redo = !(all_full || scope_size == 1 || STREAM);
      if (!redo) {
        const uint32_t n_full = all_full ? NSTEP : (uint32_t)len0 / 32u;        // steps whose 32 keys are all valid
        const int32_t tail_keys = all_full ? 0 : len0 - (int32_t)n_full * 32;   // valid keys of the step after them
        {
          // K fragments are requested a whole step before the score product that reads them (with one block per
          // wave that product belongs to the NEXT step, so they run two steps ahead), V fragments one step ahead
          constexpr uint32_t K_AHEAD = QB == 1 ? 2u : 1u;
          bf16x8_t kf[2][KSTEPS], vf[2][2];
          f32x16_t sc[2];
          load_k(0, kf[0]);
          if constexpr (K_AHEAD == 2 && NSTEP > 1) load_k(1, kf[1]);
          load_v(0, vf[0]);
          sc[0] = scores(kf[0], qf[0]);
          static_for<NSTEP>([&](auto st_c) {
            constexpr uint32_t st = decltype(st_c)::value;
            if (st < n_full) {               // uniform
              // The SIMD arbiter favours its oldest wave; left alone, that wave finishes early and idles at the
              // barrier while the other runs the tail alone.  Each wave lowers its own priority as it advances, so
              // the wave that is behind is served first.
              if constexpr (st % (NSTEP / 4) == 0) __builtin_amdgcn_s_setprio(3 - (int)(st / (NSTEP / 4)));
              static_for<VM_PER_STEP>([&](auto j_c) {
                issue_vm(std::integral_constant<uint32_t, st * VM_PER_STEP + decltype(j_c)::value>{});
              });
              vm_next = (st + 1) * VM_PER_STEP;
              if constexpr (K_AHEAD == 1 && st + 1 < NSTEP) load_k(st + 1, kf[(st + 1) & 1u]);
              if constexpr (st + 1 < NSTEP) load_v(st + 1, vf[(st + 1) & 1u]);
              static_for<QB>([&](auto b_c) {
                constexpr uint32_t b = decltype(b_c)::value;
                constexpr uint32_t u = st * QB + b;          // position in the flattened (step, block) sequence
                // the scores of the next (step, block) start now
                if constexpr (b + 1 < QB) sc[(u + 1) & 1u] = scores(kf[st & 1u], qf[b + 1]);
                else if constexpr (st + 1 < NSTEP) sc[(u + 1) & 1u] = scores(kf[(st + 1) & 1u], qf[0]);
                if constexpr (K_AHEAD == 2 && st + 2 < NSTEP) load_k(st + 2, kf[st & 1u]);
                const f32x16_t& s_cur = sc[u & 1u];
                uint32_t pb[8];
#pragma unroll
                for (int i = 0; i < 16; i += 2)
                  pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(s_cur[i]), __builtin_amdgcn_exp2f(s_cur[i + 1]));
                pv_rowsum(pb, vf[st & 1u], acc[b], lacc[b]);
              });
            }
          });
        }
        if (tail_keys > 0) {
          // the boundary step, once per item and out of the pipeline: keys at or past the valid length get a
          // score of -inf.  Register i of a lane is key (i/4)*8 + 4 half + i%4 of the step.
          bf16x8_t kf[KSTEPS], vf[2];
          load_k(n_full, kf);
          load_v(n_full, vf);
          const int32_t thr = tail_keys - (int32_t)half * 4;
          static_for<QB>([&](auto b_c) {
            constexpr uint32_t b = decltype(b_c)::value;
            f32x16_t sc = scores(kf, qf[b]);
            uint32_t pb[8];
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
              const float s0 = (i / 4) * 8 + (i % 4) >= thr ? -INFINITY : sc[i];
              const float s1 = ((i + 1) / 4) * 8 + ((i + 1) % 4) >= thr ? -INFINITY : sc[i + 1];
              pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(s0), __builtin_amdgcn_exp2f(s1));
            }
            pv_rowsum(pb, vf, acc[b], lacc[b]);
          });
        }
        // redo with a moving reference where a row sum left the safe range (also catches inf / nan)
        if constexpr (!STREAM) {
#pragma unroll
          for (int b = 0; b < QB; ++b) {
            l_fin[b] = __shfl(lacc[b][0], l_src, kWave);
            redo = redo || (q_live[b] && __ballot(!(l_fin[b] > 0x1p-24f) || !(l_fin[b] < 0x1p24f)) != 0);
          }
        }
      }
    }
    if constexpr (STREAM) {
      // the item's sums are complete after its last key bucket: out of range -> the rows are marked for the other kernel
      if (last && any_keys) {
#pragma unroll
        for (int b = 0; b < QB; ++b) {
          l_fin[b] = __shfl(lacc[b][0], l_src, kWave);
          failed = failed || (q_live[b] && __ballot(!(l_fin[b] > 0x1p-24f) || !(l_fin[b] < 0x1p24f)) != 0);
        }
      }
    }
    // ---- general pass: any mix of valid lengths, running-maximum softmax with the scale applied in fp32; one
    //      (block, step) at a time, nothing overlapped ----
    if (redo) {
#pragma unroll 1
      for (int b = 0; b < QB; ++b) {
        // unscaled Q, read again: the fast pass keeps only its pre-scaled copy
        bf16x8_t qr[KSTEPS];
        if constexpr (GEN) {
          // formed again from the row's coordinates with the head's unscaled tile
          const uint16_t* cp = gen.coord + gen_row(p_cur, cur) * 3;
          const uint16_t c3[3] = {cp[0], cp[1], cp[2]};
          const f32x16_t tq = gen_tile(*gen_tile_ptr(p_cur, 3), gen_rows_operand(c3));
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) qr[ks] = __builtin_bit_cast(bf16x8_t, pack_tile(tq, ks));
        } else {
          const char* qp = reinterpret_cast<const char*>(q + in_base(p_cur)) + (q_row_of(p_cur, cur, b) * ld + half * 8u) * 2u;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) qr[ks] = *reinterpret_cast<const bf16x8_t*>(qp + ks * 32u);
        }
        float m_run = -INFINITY, l_run = 0.f;
        f32x16_t a;
#pragma unroll
        for (int i = 0; i < 16; ++i) a[i] = 0.f;
#pragma unroll 1
        for (uint32_t st = 0; st < NSTEP; ++st) {
          // step st covers the 32 keys [32 st, 32 st + 32): position inside its bucket and that bucket's length
          const uint32_t jb = (st * 32u) / bs;
          const int32_t in_b = (int32_t)(st * 32u - jb * bs);
          const int32_t len = len_of(cur, jb);
          if (in_b >= len) continue;          // no valid key in this step (uniform)
          bf16x8_t kf[KSTEPS], vf[2];
          load_k(st, kf);
          load_v(st, vf);
          f32x16_t sc = scores(kf, qr);
          if (in_b + 32 > len) {
            const int32_t thr = len - in_b - (int32_t)half * 4;
#pragma unroll
            for (int i = 0; i < 16; ++i)
              if ((i / 4) * 8 + (i % 4) >= thr) sc[i] = -INFINITY;
          }
          float mx = sc[0];
#pragma unroll
          for (int i = 1; i < 16; ++i) mx = fmaxf(mx, sc[i]);
          mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
          const float m_new = fmaxf(m_run, mx * scale_log2);
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
          const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
          m_run = m_new;
          uint32_t pb[8];
          float psum = 0.f;
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            pb[i / 2] = pack_bf16x2(__builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], scale_log2, -m_use)),
                                    __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i + 1], scale_log2, -m_use)));
            psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pb[i / 2]),
                                                   __builtin_bit_cast(bf16x2_t, 0x3F803F80u), psum, false);
          }
          l_run = l_run * alpha + psum;
#pragma unroll
          for (int i = 0; i < 16; ++i) a[i] *= alpha;
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) {
            const u32x4_t praw = {pb[kk * 4 + 0], pb[kk * 4 + 1], pb[kk * 4 + 2], pb[kk * 4 + 3]};
            a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kk], __builtin_bit_cast(bf16x8_t, praw), a, 0, 0, 0);
          }
        }
        // hand the block's results to the epilogue through the variables the fast pass fills
        static_for<QB>([&](auto b_c) {
          constexpr uint32_t bb = decltype(b_c)::value;
          if (bb == (uint32_t)b) {
            acc[bb] = a;
            l_fin[bb] = l_run + __shfl_xor(l_run, 32, kWave);
            m_ref[bb] = (m_run == -INFINITY) ? 0.f : m_run;
          }
        });
      }
    }
    __builtin_amdgcn_s_setprio(3);
    // whatever of the next item's loads the passes above did not issue (short or skipped passes)
    static_for<VM_OPS>([&](auto i_c) {
      if (decltype(i_c)::value >= vm_next) issue_vm(i_c);
    });
    nxt2.len = load_len(nxt2.ids);
    // This wave's direct loads (issued during this item) must have landed before the barrier below; wait for them
    // BEFORE the output stores are issued, so that the stores stay fire-and-forget (vmcnt = 0, other counters
    // untouched).
    __builtin_amdgcn_s_waitcnt(0x0F70);

    // ---- epilogue: normalise, store O (bf16) and LSE ----
    const size_t obase = (size_t)p_cur.batch * seq_len * num_head + p_cur.head;
    char* const op = reinterpret_cast<char*>(o + obase * D);
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      if (!last) continue;                 // STREAM: more key buckets to come
      if (!q_exists[b]) continue;          // a scope entry outside the sequence names no rows
      if (STREAM && failed) {              // no result: the mark the streaming kernel looks for
        if (half == 0)
          *reinterpret_cast<float*>(reinterpret_cast<char*>(lse + obase) + q_row[b] * num_head * 4u) = __builtin_nanf("");
        continue;
      }
      const float l_tot = q_live[b] ? l_fin[b] : 0.f;
      const bool row_ok = (int32_t)lq < q_len[b] && l_tot > 0.f;
      const float inv = row_ok ? 1.0f / l_tot : 0.f;
      const uint32_t orow_b = q_row[b] * num_head * D * 2u;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t d0 = g * 8 + half * 4;
        if (D >= 32 || d0 < (uint32_t)D) {
          uint2 w;
          w.x = pack_bf16x2(acc[b][g * 4 + 0] * inv, acc[b][g * 4 + 1] * inv);
          w.y = pack_bf16x2(acc[b][g * 4 + 2] * inv, acc[b][g * 4 + 3] * inv);
          *reinterpret_cast<uint2*>(op + (orow_b + d0 * 2u)) = w;
        }
      }
      if (half == 0) {
        const float ln2 = 0.69314718055994530942f;
        *reinterpret_cast<float*>(reinterpret_cast<char*>(lse + obase) + q_row[b] * num_head * 4u) =
            row_ok ? (m_ref[b] + __builtin_amdgcn_logf(l_tot)) * ln2 : 0.f;
      }
    }
    if (last) {
      cur = nxt;
      nxt = nxt2;
      p_cur = p_nxt;
      p_nxt = p_nxt2;
      ++n;
      kb = 0;
    } else {
      ++kb;
    }
    // the next buffer is complete; this buffer is free for the item after next.  Not __syncthreads(): that would wait
    // for the output stores just issued.  (GEN: the barrier after an item's rows are formed does both jobs.)
    if constexpr (!GEN) wg_barrier_lds();
  }
}

template <int D, int T, int WAVES, bool GEN = false, bool STREAM = false>
static int launch_attn_scope(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, uint16_t* o, float* lse,
                             const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                             uint32_t batch, uint32_t seq_len, uint32_t num_head, const int32_t* kv_len, int device,
                             hipStream_t s, ScopeGen gen = ScopeGen{nullptr, nullptr, nullptr}) {
  const uint64_t n_items64 = (uint64_t)batch * num_scope * num_head * (STREAM ? scope_size : 1u);
  if (n_items64 == 0) return F3D_OK;
  if (n_items64 > 0x7FFFFFF0ull / (STREAM ? scope_size : 1u)) {
    set_error("attention problem too large for one launch (%llu items)", (unsigned long long)n_items64);
    return F3D_ERR_INVALID;
  }
  const uint32_t n_items = (uint32_t)n_items64;
  constexpr size_t lds = scope_lds_bytes<D, T, WAVES>();
  // once per instantiation and device: raise the dynamic LDS limit, ask how many workgroups a CU holds
  static int wg_per_cu[64] = {};
  int per_cu = (device >= 0 && device < 64) ? wg_per_cu[device] : 0;
  if (per_cu == 0) {
    F3D_CHECK_HIP(hipFuncSetAttribute((const void*)buck_swin_fwd_scope_kernel<D, T, WAVES, GEN, STREAM>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    F3D_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, buck_swin_fwd_scope_kernel<D, T, WAVES, GEN, STREAM>,
                                                               64 * WAVES, lds));
    if (per_cu < 1) per_cu = 1;
    if (device >= 0 && device < 64) wg_per_cu[device] = per_cu;
  }
  int n_cu = 0;
  F3D_CHECK_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device));
  // persistent workgroups: a multiple of the XCD count, no more than the chip holds at once, no more than items need
  const uint32_t items_per_xcd = cdiv_u32(n_items, kNumXcd);
  const uint32_t n_slots = std::max(1u, std::min((uint32_t)n_cu * (uint32_t)per_cu / kNumXcd, items_per_xcd));
  const float scale_log2 = 1.4426950408889634f / sqrtf((float)D);
  hipLaunchKernelGGL((buck_swin_fwd_scope_kernel<D, T, WAVES, GEN, STREAM>), dim3(n_slots * kNumXcd), dim3(64 * WAVES), lds, s, q, k,
                     v, ld, o, lse, scope_buckets, num_scope, scope_size, bs, seq_len, num_head, kv_len, scale_log2,
                     n_items, items_per_xcd, n_slots, gen);
  return F3D_OK;
}

// ---- LayerNorm + QKV projection of the coordinate embedding, folded --------------------------------------------
// The first block's input is x = E c, c = (x, y, z, 1), E = [w_embed | b_embed] (C x 4).  Over the channels,
// x - mean(x) = E' c with E' = E minus its column means, var(x) = |E' c|^2 / C = |L c|^2 with L the upper-triangular
// Cholesky factor of G = E'^T E' / C, and
//   qkv = W (gamma * (x - mean) * rstd + beta) + b = rstd * (M c) + b',   M = W diag(gamma) E'  (3C x 4),  b' = W beta + b.
// One wave per output row writes that row's 16 bf16 of the attention kernel's table: (M high parts, M low parts |
// M high parts, b' high, b' low, 0, 0), to be multiplied with (c~ high, c~ high | c~ low, 1, 1, 0, 0), c~ = rstd c;
// row position inside the head's 32-row tile = the row of the 32x32 accumulator layout that hands a lane the features
// 8 half .. 8 half + 7 and 16 + 8 half .. 16 + 8 half + 7.  One more wave writes the Cholesky factor and eps.
__global__ __launch_bounds__(64) void embed_qkv_fold_kernel(
    const uint16_t* __restrict__ ew, const uint16_t* __restrict__ eb, const uint16_t* __restrict__ gamma,
    const uint16_t* __restrict__ beta, float eps, const uint16_t* __restrict__ w, const uint16_t* __restrict__ b,
    uint32_t C, uint32_t num_head, float scale_log2, uint16_t* __restrict__ table, float* __restrict__ chol) {
  // one wave per output feature of the projection (block 3 C: the Cholesky factor); lanes stride over the channels
  const uint32_t row = blockIdx.x, lane = threadIdx.x;
  auto e_at = [&](uint32_t ch, uint32_t j) {
    return j < 3 ? bf16_bits_to_float(ew[ch * 3 + j]) : (eb ? bf16_bits_to_float(eb[ch]) : 0.f);
  };
  auto wave_sum = [&](double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
  };
  double mean[4] = {0, 0, 0, 0};
  for (uint32_t ch = lane; ch < C; ch += kWave)
    for (uint32_t j = 0; j < 4; ++j) mean[j] += e_at(ch, j);
  for (uint32_t j = 0; j < 4; ++j) mean[j] = wave_sum(mean[j]) / C;
  if (row < 3 * C) {
    double m[4] = {0, 0, 0, 0}, bp = 0;
    for (uint32_t ch = lane; ch < C; ch += kWave) {
      const double wv = bf16_bits_to_float(w[(size_t)row * C + ch]);
      const double wg = wv * (gamma ? bf16_bits_to_float(gamma[ch]) : 1.f);
      for (uint32_t j = 0; j < 4; ++j) m[j] += wg * (e_at(ch, j) - mean[j]);
      if (beta) bp += wv * bf16_bits_to_float(beta[ch]);
    }
    for (uint32_t j = 0; j < 4; ++j) m[j] = wave_sum(m[j]);
    bp = wave_sum(bp) + (b ? bf16_bits_to_float(b[row]) : 0.f);
    if (lane != 0) return;
    const uint32_t part = row / C, within = row % C, head = within / 32, d = within % 32;
    const uint32_t hf = (d % 16) / 8, i = d < 16 ? d % 8 : 8 + d % 8;
    const uint32_t r = (i % 4) + 8 * (i / 4) + 4 * hf;
    auto emit = [&](uint32_t tile, double sc) {
      uint16_t* out = table + (((size_t)head * 4 + tile) * 32 + r) * 16;
      for (uint32_t j = 0; j < 4; ++j) {
        const float f = (float)(m[j] * sc);
        const uint16_t hi = float_to_bf16_bits(f);
        out[j] = hi;
        out[4 + j] = float_to_bf16_bits(f - bf16_bits_to_float(hi));
        out[8 + j] = hi;
      }
      const float fb = (float)(bp * sc);
      const uint16_t bh = float_to_bf16_bits(fb);
      out[12] = bh;
      out[13] = float_to_bf16_bits(fb - bf16_bits_to_float(bh));
      out[14] = 0;
      out[15] = 0;
    };
    if (part == 0) {
      emit(0, (double)scale_log2);
      emit(3, 1.0);
    } else {
      emit(part, 1.0);
    }
    return;
  }
  double g[4][4];
  for (int a = 0; a < 4; ++a)
    for (int c = a; c < 4; ++c) {
      double s = 0;
      for (uint32_t ch = lane; ch < C; ch += kWave) s += ((double)e_at(ch, a) - mean[a]) * ((double)e_at(ch, c) - mean[c]);
      g[a][c] = wave_sum(s) / C;
    }
  if (lane != 0) return;
  double l[4][4];
  for (int a = 0; a < 4; ++a)
    for (int c = 0; c < 4; ++c) l[a][c] = 0;
  for (int a = 0; a < 4; ++a) {           // G = L^T L, row by row; a pivot that is not positive ends its row at zero
    double piv = g[a][a];
    for (int k2 = 0; k2 < a; ++k2) piv -= l[k2][a] * l[k2][a];
    if (!(piv > 0)) continue;
    l[a][a] = sqrt(piv);
    for (int c = a + 1; c < 4; ++c) {
      double s = g[a][c];
      for (int k2 = 0; k2 < a; ++k2) s -= l[k2][a] * l[k2][c];
      l[a][c] = s / l[a][a];
    }
  }
  int n = 0;
  for (int a = 0; a < 4; ++a)
    for (int c = a; c < 4; ++c) chol[n++] = (float)l[a][c];
  chol[10] = eps;
  for (n = 11; n < 16; ++n) chol[n] = 0.f;
}

template <int D, int KT>
static int launch_attn(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint32_t ld, uint16_t* o, float* lse,
                       const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bs,
                       uint32_t batch, uint32_t seq_len, uint32_t num_head, const int32_t* kv_len, hipStream_t s,
                       uint32_t only_marked = 0) {
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
                     n_work, per_xcd, only_marked);
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
  F3D_CHECK_ARG(scope_size >= 1 && scope_size <= 4096, "scope_size=%u outside [1, 4096]", scope_size);
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
  rc = launch_attn_scope<DD, TT, TT / 32>(q, k, v, qkv_row_stride, o, lse, scope_buckets, num_scope, scope_size, \
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
  // larger scopes in buckets of 256 / 512 rows with 16- or 32-wide heads (the reference model's scopes of 8 buckets of
  // 512): the scope-resident kernel with the key buckets streaming through its two LDS buffers, then the streaming
  // kernel for the rows it marked (sums outside the range of the fixed-reference softmax), which are rare
  if (head_dim <= 32 && (bucket_size == 256 || bucket_size == 512) && scope_tokens > 512 && scope_size <= 64 &&
      (uint64_t)seq_len * qkv_row_stride * 2 < (1ull << 32)) {
#define F3D_RES_STREAM(DD, TT, KK)                                                                                        \
  do {                                                                                                                    \
    rc = launch_attn_scope<DD, TT, TT / 32, false, true>(q, k, v, qkv_row_stride, o, lse, scope_buckets, num_scope,       \
                                                         scope_size, bucket_size, batch, seq_len, num_head, kv_len, device, \
                                                         s);                                                              \
    if (rc != F3D_OK) return rc;                                                                                          \
    F3D_CHECK_HIP(hipGetLastError());                                                                                     \
    rc = launch_attn<DD, KK>(q, k, v, qkv_row_stride, o, lse, scope_buckets, num_scope, scope_size, bucket_size, batch,   \
                             seq_len, num_head, kv_len, s, 1u);                                                           \
  } while (0)
    if (head_dim == 16) {
      if (bucket_size == 256) F3D_RES_STREAM(16, 256, 128); else F3D_RES_STREAM(16, 512, 128);
    } else {
      if (bucket_size == 256) F3D_RES_STREAM(32, 256, 64); else F3D_RES_STREAM(32, 512, 64);
    }
#undef F3D_RES_STREAM
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

int f3d_embed_qkv_fold_bf16(const f3d_bf16_t* embed_w, const f3d_bf16_t* embed_b, const f3d_bf16_t* gamma,
                            const f3d_bf16_t* beta, float eps, const f3d_bf16_t* w_qkv, const f3d_bf16_t* b_qkv, uint32_t c,
                            uint32_t num_head, uint32_t head_dim, f3d_bf16_t* table, float* chol, int device,
                            void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(embed_w && w_qkv && table && chol, "null tensor pointer");
  F3D_CHECK_ARG(c > 0 && num_head > 0 && c == num_head * head_dim, "channels %u != num_head %u * head_dim %u", c, num_head,
                head_dim);
  if (head_dim != 32) {
    set_error("rows are formed inside the attention kernel for head_dim 32 only (got %u)", head_dim);
    return F3D_ERR_UNSUPPORTED;
  }
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const float scale_log2 = 1.4426950408889634f / sqrtf((float)head_dim);
  hipLaunchKernelGGL(embed_qkv_fold_kernel, dim3(3 * c + 1), dim3(64), 0, s, embed_w, embed_b, gamma, beta, eps,
                     w_qkv, b_qkv, c, num_head, scale_log2, table, chol);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_embed_buck_swin_fwd(const f3d_half_t* coord, const f3d_bf16_t* table, const float* chol, f3d_bf16_t* o, float* lse,
                            const uint32_t* scope_buckets, uint32_t num_scope, uint32_t scope_size, uint32_t bucket_size,
                            uint32_t batch, uint32_t seq_len, uint32_t num_head, uint32_t head_dim, int device,
                            void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(coord && table && chol && o && lse && scope_buckets, "null tensor pointer");
  F3D_CHECK_ARG(bucket_size >= 128 && bucket_size % 128 == 0, "bucket_size=%u must be a multiple of 128", bucket_size);
  F3D_CHECK_ARG(seq_len % bucket_size == 0, "sequence length %u is not a multiple of bucket_size=%u", seq_len, bucket_size);
  F3D_CHECK_ARG((((uintptr_t)table | (uintptr_t)o) & 15u) == 0, "table / o must be 16-byte aligned");
  const uint32_t scope_tokens = scope_size * bucket_size;
  if (head_dim != 32 || scope_size < 1 || scope_size > (uint32_t)kResMaxScope || (scope_tokens != 256 && scope_tokens != 512) ||
      (uint64_t)seq_len * num_head * head_dim * 2 >= (1ull << 32)) {
    set_error("rows are formed inside the attention kernel for head_dim 32 and scopes of 256 or 512 tokens only "
              "(head_dim %u, %u tokens)", head_dim, scope_tokens);
    return F3D_ERR_UNSUPPORTED;
  }
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  SyncBracket sync(s);
  const ScopeGen gen = {coord, table, chol};
  int rc;
  if (scope_tokens == 256)
    rc = launch_attn_scope<32, 256, 8, true>(nullptr, nullptr, nullptr, num_head * head_dim, o, lse, scope_buckets, num_scope,
                                             scope_size, bucket_size, batch, seq_len, num_head, nullptr, device, s, gen);
  else
    rc = launch_attn_scope<32, 512, 16, true>(nullptr, nullptr, nullptr, num_head * head_dim, o, lse, scope_buckets, num_scope,
                                              scope_size, bucket_size, batch, seq_len, num_head, nullptr, device, s, gen);
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
