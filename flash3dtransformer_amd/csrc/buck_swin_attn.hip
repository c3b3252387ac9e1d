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
  static constexpr int LDS_BYTES = (KT * KROW + D * VROW) * 2;
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
  const uint32_t q_bucket = my_scope[q_local / bs];
  if (q_bucket >= n_bucket) return;  // a scope entry outside the sequence names no rows (uniform per workgroup)
  const uint32_t q_in_bucket = (q_local % bs) + wave * 32 + lq;
  const uint32_t q_row = q_bucket * bs + q_in_bucket;
  const size_t tok0 = (size_t)batch * seq_len;
  const int32_t q_valid_len = kv_len ? min(max(kv_len[q_bucket], 0), (int32_t)bs) : (int32_t)bs;

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
  auto bucket_len = [&](uint32_t j) -> int32_t {  // valid keys of scope bucket j; 0 for an out-of-range bucket id
    const uint32_t b = my_scope[j];
    if (b >= n_bucket) return 0;
    return kv_len ? min(max(kv_len[b], 0), (int32_t)bs) : (int32_t)bs;
  };
  auto settle = [&]() {  // advance (jb, kt) to the next tile that holds at least one valid key
    while (jb < scope_size) {
      if ((int32_t)(kt * KT) < bucket_len(jb)) return true;
      ++jb; kt = 0;
    }
    return false;
  };

  u32x4_t rk[C::NCH], rv[C::NCH];
  auto fetch = [&](uint32_t j, uint32_t t) {
    const size_t row0 = tok0 + (size_t)my_scope[j] * bs + t * KT;
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
      psum += p0 + p1;
      pb[i / 2] = pack_bf16x2(p0, p1);
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
  hipLaunchKernelGGL((buck_swin_fwd_kernel<D, KT>), dim3(per_xcd * kNumXcd), dim3(kAttnThreads), C::LDS_BYTES, s, q, k,
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
