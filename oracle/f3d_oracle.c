/*
 * CPU oracle for the Flash3D forward hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference algorithms, used as the checker in
 * tests/, in the smoke test and as the timed CPU baseline of the benchmark.  Nothing in the
 * product package links, loads or calls it.  Every function cites the reference source it
 * restates (paths relative to the reference tree).
 *
 * Pins (what keeps the oracle itself honest, see tests/test_oracle_*.py):
 *   vox/hash      : closed forms + known answers + bit-loop Morton brute force
 *   claim/scatter : scoreboard invariant + cumsum identity + multiset equality
 *   index/features: index is a bijection per cloud; gathering the input coordinates by it gives
 *                   the scattered coordinates of the scatter step, bit for bit
 *   reduce/unpool : numpy library routines on the same inputs
 *   sub-buckets   : structural invariants of tests/test_subbuck_reduce.py:486-631
 *
 * Where the reference is arbitration-ordered (atomic slot claims) the oracle fixes the order to
 * input order, which is one of the outcomes the reference can produce.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* scalar type helpers                                                                        */
/* ------------------------------------------------------------------------------------------ */

float f3d_or_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      man &= 0x3FFu;
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* float -> half, round to nearest even */
uint16_t f3d_or_float_to_half(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t abs = u & 0x7FFFFFFFu;
  if (abs >= 0x7F800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((abs > 0x7F800000u) ? 0x200u : 0u));
  }
  if (abs >= 0x477FF000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (abs < 0x38800000u) { /* subnormal half or zero */
    if (abs < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
    int e = (int)(abs >> 23);                     /* biased float exponent */
    uint32_t man = (abs & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    int shift = 126 - e;                          /* 14..24: bits dropped to reach 2^-24 units */
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
  uint32_t e = (abs >> 23) - 112u;
  uint32_t man = abs & 0x7FFFFFu;
  uint32_t q = (e << 10) | (man >> 13);
  uint32_t rem = man & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
  return (uint16_t)(sign | q);
}

float f3d_or_bf16_to_float(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* float -> bf16, round to nearest even; NaN stays NaN */
uint16_t f3d_or_float_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* ------------------------------------------------------------------------------------------ */
/* A1: voxel quantiser  — src/psh/hash_fns.cuh:23-33, clamp at src/common/arithmetic.cuh:26-28 */
/* ------------------------------------------------------------------------------------------ */

/* v = clamp(floor((c - min) * num_vox / (max - min)), 0, num_vox - 1).  Two roundings of the quotient:
 * mode 0 (default): the reference is built with nvcc --use_fast_math (CMakeLists.txt:49-52), which turns the fp32
 *   division into a multiplication by the reciprocal of the divisor; pinned with a correctly rounded
 *   reciprocal: q = fl(fl((c - min) * num_vox) * fl(1 / (max - min))), every step IEEE fp32;
 * mode 1: q = fl(fl((c - min) * num_vox) / fl(max - min)), the IEEE division the source text spells out
 *   (a build without fast-math).
 * clamp(x, lo, hi) = max(lo, min(x, hi)) with NaN-ignoring min (arithmetic.cuh:26-28), so a
 * degenerate axis (max == min: 0 * inf = 0 / 0 = NaN) lands on num_vox - 1. */
static int g_quantiser_mode = 0;

int f3d_or_set_quantiser(int mode) {
  if (mode != 0 && mode != 1) return -1;
  g_quantiser_mode = mode;
  return 0;
}

uint16_t f3d_or_vox1(float c, float mn, float mx, uint32_t num_vox) {
  volatile float den = mx - mn;
  volatile float inv = 1.0f / den;
  volatile float num = (c - mn) * (float)num_vox;
  volatile float q = g_quantiser_mode ? num / den : num * inv;
  float v = floorf(q);
  float hi = (float)(num_vox - 1u);
  float m = (v < hi) ? v : hi; /* NaN -> hi */
  float r = (m > 0.f) ? m : 0.f;
  return (uint16_t)r;
}

void f3d_or_vox_coord(const uint16_t *coord_h, uint32_t n, const uint16_t *bbox_min_h,
                      const uint16_t *bbox_max_h, uint32_t num_vox, uint16_t *vox_out) {
  float mn[3], mx[3];
  for (int d = 0; d < 3; ++d) {
    mn[d] = f3d_or_half_to_float(bbox_min_h[d]);
    mx[d] = f3d_or_half_to_float(bbox_max_h[d]);
  }
  for (uint32_t i = 0; i < n; ++i)
    for (int d = 0; d < 3; ++d)
      vox_out[3 * i + d] = f3d_or_vox1(f3d_or_half_to_float(coord_h[3 * i + d]), mn[d], mx[d], num_vox);
}

/* ------------------------------------------------------------------------------------------ */
/* A2: first-hash family — src/psh/hash_fns.cuh:48-68, 79-86, 113-135; enum :151-158           */
/* ------------------------------------------------------------------------------------------ */

/* 3-way bit spread, src/psh/hash_fns.cuh:79-86 (same mask ladder, it is the published
 * "Morton 3D magic bits" sequence for 21-bit inputs) */
uint64_t f3d_or_space_out_bit_3d(uint64_t x) {
  x = (x | x << 32) & 0x1f00000000ffffULL;
  x = (x | x << 16) & 0x1f0000ff0000ffULL;
  x = (x | x << 8) & 0x100f00f00f00f00fULL;
  x = (x | x << 4) & 0x10c30c30c30c30c3ULL;
  x = (x | x << 2) & 0x1249249249249249ULL;
  return x;
}

/* the u16 that every z-order hash starts from: low 16 bits of (morton48 >> 31) */
uint16_t f3d_or_zorder16(uint16_t vx, uint16_t vy, uint16_t vz) {
  uint64_t x = f3d_or_space_out_bit_3d(vx);
  uint64_t y = f3d_or_space_out_bit_3d(vy);
  uint64_t z = f3d_or_space_out_bit_3d(vz);
  return (uint16_t)((x | y << 1 | z << 2) >> 31);
}

/* hash_type: 1 ZORDER_DIV, 2 XORSUM_DIV, 3 ZORDER_MOD, 4 XORSUM_MOD.  divisor and num_bucket are
 * truncated to 16 bits exactly as the reference's HashT parameters are. */
uint16_t f3d_or_hash(uint16_t vx, uint16_t vy, uint16_t vz, uint32_t hash_type, uint32_t divisor,
                     uint32_t num_bucket) {
  uint16_t div16 = (uint16_t)divisor, nb16 = (uint16_t)num_bucket;
  switch (hash_type) {
    case 1: return (uint16_t)(f3d_or_zorder16(vx, vy, vz) / div16);
    case 2: return (uint16_t)((uint16_t)(vx ^ vy ^ vz) / div16);
    case 3: return (uint16_t)(f3d_or_zorder16(vx, vy, vz) % nb16);
    case 4: return (uint16_t)((uint16_t)(vx ^ vy ^ vz) % nb16);
    default: return 0xFFFFu;
  }
}

/* ------------------------------------------------------------------------------------------ */
/* A1+A2+A3: hash and slot claim — src/psh/batch_psh_bucket.cuh:100-152 with                    */
/* TwoStageCounter src/psh/two_stage_counter.cuh:65-131.  Claim order fixed to input order.     */
/* ------------------------------------------------------------------------------------------ */

/* bucket_counter [B, num_bucket] must be zero on entry (caller contract psh_main.py:54).
 * Returns 0, or -1 on a bad argument. */
int f3d_or_psh_claim(const uint16_t *coord_h, uint32_t total_n, const uint32_t *batch_sep,
                     uint32_t batch_size, const uint16_t *bbox_min_h, const uint16_t *bbox_max_h,
                     uint32_t num_vox, uint32_t divisor, uint32_t num_bucket, uint32_t hash_type,
                     uint16_t *bucket_id, uint32_t *bucket_counter, uint32_t *bucket_offset) {
  if (hash_type < 1 || hash_type > 4 || num_bucket == 0) return -1;
  float mn[3], mx[3];
  for (int d = 0; d < 3; ++d) {
    mn[d] = f3d_or_half_to_float(bbox_min_h[d]);
    mx[d] = f3d_or_half_to_float(bbox_max_h[d]);
  }
  uint32_t start = 0;
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b];
    if (end > total_n || end < start) return -1;
    uint32_t *cnt = bucket_counter + (size_t)b * num_bucket;
    for (uint32_t i = start; i < end; ++i) {
      uint16_t v[3];
      for (int d = 0; d < 3; ++d)
        v[d] = f3d_or_vox1(f3d_or_half_to_float(coord_h[3 * (size_t)i + d]), mn[d], mx[d], num_vox);
      uint16_t id = f3d_or_hash(v[0], v[1], v[2], hash_type, divisor, num_bucket);
      if (id >= num_bucket) return -2; /* "bucket divisor too small" guard, dispatcher :239-241 */
      bucket_id[i] = id;
      bucket_offset[i] = cnt[id]++;
    }
    start = end;
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* A4: overflow rebalance + recycle — src/psh/batch_psh_bucket.cuh:154-246 (probe rebalance),   */
/* :259-382 (recycle).  The reference moves a point whose slot is >= bucket_size (bucket != 0)   */
/* to the first probed neighbour bucket that still has room, racing on global counters with a   */
/* shared cuRAND state, and drops the losers into bucket 0; its result is not reproducible.      */
/* Deterministic restatement used by this build: overflow units, ordered by (bucket, slot), are  */
/* matched one to one, in order, with the free slots (ordered by (bucket, slot)) of the buckets   */
/* != 0 holding fewer than bucket_size points; units beyond the total free capacity are appended  */
/* to bucket 0 (the recycle bucket, which may exceed bucket_size exactly as in the reference).     */
/* Same invariants as the reference's: every point keeps exactly one (bucket, slot), slots are     */
/* dense per bucket, points of a bucket that neither overflows nor receives anything stay put.     */
/* In: first-hash ids / counts / stable slots.  Out (in place): final ids, counts, slots.          */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_psh_rebalance(uint16_t *bucket_id, uint32_t *bucket_counter, uint32_t *bucket_offset,
                         const uint32_t *batch_sep, uint32_t batch_size, uint32_t num_bucket,
                         uint32_t bucket_size) {
  uint32_t start = 0;
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b];
    uint32_t *cnt = bucket_counter + (size_t)b * num_bucket;
    /* point index of every (bucket, slot) */
    size_t *base = (size_t *)malloc(sizeof(size_t) * (num_bucket + 1));
    base[0] = 0;
    for (uint32_t k = 0; k < num_bucket; ++k) base[k + 1] = base[k] + cnt[k];
    uint32_t *who = (uint32_t *)malloc(sizeof(uint32_t) * (base[num_bucket] ? base[num_bucket] : 1));
    for (uint32_t i = start; i < end; ++i) who[base[bucket_id[i]] + bucket_offset[i]] = i;
    uint32_t *fin = (uint32_t *)malloc(sizeof(uint32_t) * num_bucket);
    for (uint32_t k = 0; k < num_bucket; ++k) fin[k] = (k != 0 && cnt[k] > bucket_size) ? bucket_size : cnt[k];
    uint32_t fb = 1; /* next bucket that may have room */
    for (uint32_t k = 1; k < num_bucket; ++k) {
      for (uint32_t slot = bucket_size; slot < cnt[k]; ++slot) {
        uint32_t p = who[base[k] + slot];
        /* a bucket that overflowed itself (cnt > bucket_size) never takes immigrants */
        while (fb < num_bucket && (cnt[fb] >= bucket_size || fin[fb] >= bucket_size)) ++fb;
        uint32_t dst = (fb < num_bucket) ? fb : 0u;
        bucket_id[p] = (uint16_t)dst;
        bucket_offset[p] = fin[dst]++;
      }
    }
    for (uint32_t k = 0; k < num_bucket; ++k) cnt[k] = fin[k];
    free(base); free(who); free(fin);
    start = end;
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* A5: cumsum + scatter + tail pad — src/psh/batch_psh_bucket.cuh:493-614                      */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_cumsum_scatter_pad(const uint16_t *coord_h, uint32_t total_n, const uint32_t *batch_sep,
                              uint32_t batch_size, uint32_t num_bucket, const uint16_t *bucket_id,
                              const uint32_t *bucket_counter, const uint32_t *bucket_offset,
                              uint32_t *cumsum_counter, uint16_t *scattered_h, uint32_t pad_to,
                              float pad_num) {
  if (pad_to < total_n) return -1;
  uint32_t start = 0;
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b];
    const uint32_t *cnt = bucket_counter + (size_t)b * num_bucket;
    uint32_t *cs = cumsum_counter + (size_t)b * num_bucket;
    uint32_t run = 0;
    for (uint32_t k = 0; k < num_bucket; ++k) { run += cnt[k]; cs[k] = run; } /* inclusive */
    for (uint32_t i = start; i < end; ++i) {
      uint32_t id = bucket_id[i];
      uint32_t base = id ? cs[id - 1] : 0u;
      size_t dst = (size_t)start + base + bucket_offset[i];
      if (dst >= pad_to) return -2;
      for (int d = 0; d < 3; ++d) scattered_h[3 * dst + d] = coord_h[3 * (size_t)i + d];
    }
    start = end;
  }
  uint16_t pad_h = f3d_or_float_to_half(pad_num);
  for (size_t r = total_n; r < pad_to; ++r)
    for (int d = 0; d < 3; ++d) scattered_h[3 * r + d] = pad_h;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Permutation index + feature scatter — src/psh/batch_psh_bucket.cuh:617-753 (the reference      */
/* writes scatter_idx_out2in[dst] = src, :725-736, and total_N + 3 into the pad rows, :670-679;    */
/* the feature move it announces is the same assignment on rows of row_bytes bytes).               */
/* cumsum_counter is the inclusive prefix that f3d_or_cumsum_scatter_pad leaves behind.            */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_scatter_feat_index(uint32_t total_n, const uint32_t *batch_sep, uint32_t batch_size,
                              uint32_t num_bucket, const uint16_t *bucket_id, const uint32_t *bucket_offset,
                              const uint32_t *cumsum_counter, const uint8_t *feat, uint32_t row_bytes,
                              uint32_t *idx_out2in, uint8_t *scattered_feat, uint32_t pad_to) {
  if (pad_to < total_n) return -1;
  uint32_t start = 0;
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b];
    const uint32_t *cs = cumsum_counter + (size_t)b * num_bucket;
    for (uint32_t i = start; i < end; ++i) {
      uint32_t id = bucket_id[i];
      uint32_t base = id ? cs[id - 1] : 0u;
      size_t dst = (size_t)start + base + bucket_offset[i];
      if (dst >= total_n) return -2;
      idx_out2in[dst] = i;
      if (feat) memcpy(scattered_feat + dst * row_bytes, feat + (size_t)i * row_bytes, row_bytes);
    }
    start = end;
  }
  for (size_t r = total_n; r < pad_to; ++r) {
    idx_out2in[r] = total_n + 3u;
    if (feat) memset(scattered_feat + r * row_bytes, 0, row_bytes);
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Scoreboard — src/psh/bucket_sanitizer_cpu.cpp:92-176: every (cloud, bucket, slot < count)    */
/* claimed exactly once, ids < num_bucket, slots < per-cloud max count.                         */
/* Returns 0 when clean, else a positive code: 1 id/slot overflow, 2 slot hit != once,          */
/* 3 residual (count minus claims) non-zero.  *bad_index receives the offending point/slot.      */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_scoreboard(const uint16_t *bucket_id, const uint32_t *bucket_counter,
                      const uint32_t *bucket_offset, const uint32_t *batch_sep, uint32_t batch_size,
                      uint32_t num_bucket, int64_t *bad_index) {
  uint32_t start = 0;
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b];
    const uint32_t *cnt = bucket_counter + (size_t)b * num_bucket;
    uint32_t maxcnt = 0;
    for (uint32_t k = 0; k < num_bucket; ++k) if (cnt[k] > maxcnt) maxcnt = cnt[k];
    uint8_t *table = (uint8_t *)calloc((size_t)num_bucket * (maxcnt ? maxcnt : 1), 1);
    int64_t *res = (int64_t *)malloc(sizeof(int64_t) * num_bucket);
    for (uint32_t k = 0; k < num_bucket; ++k) res[k] = cnt[k];
    int rc = 0;
    for (uint32_t i = start; i < end && !rc; ++i) {
      uint32_t id = bucket_id[i], off = bucket_offset[i];
      if (id >= num_bucket || off >= maxcnt) { rc = 1; *bad_index = i; break; }
      res[id] -= 1;
      if (table[(size_t)id * maxcnt + off] < 255) table[(size_t)id * maxcnt + off] += 1;
    }
    for (uint32_t k = 0; k < num_bucket && !rc; ++k) {
      for (uint32_t s = 0; s < cnt[k]; ++s)
        if (table[(size_t)k * maxcnt + s] != 1) { rc = 2; *bad_index = (int64_t)k * maxcnt + s; break; }
      if (!rc && res[k] != 0) { rc = 3; *bad_index = k; }
    }
    free(table);
    free(res);
    if (rc) return rc;
    start = end;
  }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Stateless RNG shared by the deterministic variants (not in the reference, which uses racing  */
/* cuRAND states src/common/rand.cuh:54-74): 32-bit integer finaliser chained over a key tuple. */
/* ------------------------------------------------------------------------------------------ */

static uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU;
  x ^= x >> 15; x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

uint32_t f3d_or_rng_u32(uint32_t seed, uint32_t a, uint32_t b, uint32_t c) {
  uint32_t h = mix32(seed + 0x9E3779B9u);
  h = mix32(h ^ (a + 0x85EBCA6Bu));
  h = mix32(h ^ (b + 0xC2B2AE35u));
  h = mix32(h ^ (c + 0x27D4EB2Fu));
  return h;
}

/* uniform in [0,1) with 24 bits */
float f3d_or_rng_u01(uint32_t seed, uint32_t a, uint32_t b, uint32_t c) {
  return (float)(f3d_or_rng_u32(seed, a, b, c) >> 8) * (1.0f / 16777216.0f);
}

/* ------------------------------------------------------------------------------------------ */
/* A6: sub-bucket builder — src/psh/batch_psh_subbuck_reduce.cuh:104-298 with                   */
/* CumsumCounter src/psh/shmem_cumsum_counter.cuh:25-167 and rand_quat/apply_quat_3d :54-102.   */
/*                                                                                            */
/* Deterministic restatement: each cloud is cut into tiles of tile_pts = (1024 / S) * S         */
/* consecutive points (1024 when S divides it, as in the reference).  Per tile: unit quaternion  */
/* with components U(0.1, 1) from the stateless RNG keyed (seed, cloud, tile, component);        */
/* rotate, round to fp16; tile bbox; quantise to num_vox cells; 13-bit z-order cell             */
/* (zorder16 / 8); order points by (cell, position in tile) — the reference's counting sort      */
/* with arbitration order fixed to input order; rank / S = local sub-bucket, rank % S = slot.    */
/* Tile t of a cloud owns output rows [t * tile_pts / S, ...), which replaces the reference's    */
/* racing atomicAdd on subbuck_cnt.  reduced_coord = fp32 mean (summed in rank order) of the     */
/* un-rotated member coordinates.  Rows [R, r_aligned) of reduced_coord are zero-filled.          */
/* ------------------------------------------------------------------------------------------ */

static void quat_rotate(const float q[4], const float p[3], float out[3]) {
  /* operation order of apply_quat_3d, batch_psh_subbuck_reduce.cuh:80-102, no contraction */
  volatile float w = q[0], x = q[1], y = q[2], z = q[3];
  volatile float n1 = x * 2.0f, n2 = y * 2.0f, n3 = z * 2.0f;
  volatile float n4 = x * n1, n5 = y * n2, n6 = z * n3;
  volatile float n7 = x * n2, n8 = x * n3, n9 = y * n3;
  volatile float n10 = w * n1, n11 = w * n2, n12 = w * n3;
  volatile float a0 = (1.0f - (n5 + n6)) * p[0], a1 = (n7 - n12) * p[1], a2 = (n8 + n11) * p[2];
  volatile float b0 = (n7 + n12) * p[0], b1 = (1.0f - (n4 + n6)) * p[1], b2 = (n9 - n10) * p[2];
  volatile float c0 = (n8 - n11) * p[0], c1 = (n9 + n10) * p[1], c2 = (1.0f - (n4 + n5)) * p[2];
  volatile float s0 = a0 + a1, s1 = b0 + b1, s2 = c0 + c1;
  out[0] = s0 + a2;
  out[1] = s1 + b2;
  out[2] = s2 + c2;
}

void f3d_or_tile_quat(uint32_t seed, uint32_t cloud, uint32_t tile, float q[4]) {
  volatile float acc = 0.f;
  for (uint32_t i = 0; i < 4; ++i) {
    volatile float u = f3d_or_rng_u01(seed, cloud, tile, i);
    volatile float s = u * 0.9f;
    q[i] = 0.1f + s;
    volatile float sq = q[i] * q[i];
    acc = acc + sq;
  }
  volatile float nrm = sqrtf(acc);
  for (int i = 0; i < 4; ++i) q[i] = q[i] / nrm;
}

static int cmp_u32(const void *a, const void *b) {
  uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
  return (x > y) - (x < y);
}

int f3d_or_subbuck_build(const uint16_t *coord_h, uint32_t total_n, const uint32_t *batch_sep,
                         const uint32_t *reduced_batch_sep, uint32_t batch_size, uint32_t subbuck_size,
                         uint32_t num_vox, uint32_t seed, uint32_t *subbuck_id, uint16_t *subbuck_off,
                         uint32_t *unpool_ind, uint16_t *reduced_coord_h, uint32_t r_aligned) {
  const uint32_t S = subbuck_size;
  if (S < 1 || S > 1024) return -1;
  const uint32_t tile_pts = (1024u / S) * S;
  const uint32_t rows_per_tile = tile_pts / S;
  uint32_t start = 0, rstart = 0;
  uint32_t keys[1024];
  uint16_t cell[1024];
  for (uint32_t b = 0; b < batch_size; ++b) {
    uint32_t end = batch_sep[b], rend = reduced_batch_sep[b];
    uint32_t n = end - start;
    if (rend - rstart != (n + S - 1) / S) return -2;
    uint32_t ntile = (n + tile_pts - 1) / tile_pts;
    for (uint32_t t = 0; t < ntile; ++t) {
      uint32_t t0 = start + t * tile_pts;
      uint32_t m = (n - t * tile_pts < tile_pts) ? n - t * tile_pts : tile_pts;
      float q[4];
      f3d_or_tile_quat(seed, b, t, q);
      uint16_t rot[1024][3];
      float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
      for (uint32_t j = 0; j < m; ++j) {
        float p[3], r[3];
        for (int d = 0; d < 3; ++d) p[d] = f3d_or_half_to_float(coord_h[3 * (size_t)(t0 + j) + d]);
        quat_rotate(q, p, r);
        for (int d = 0; d < 3; ++d) {
          rot[j][d] = f3d_or_float_to_half(r[d]);
          float rh = f3d_or_half_to_float(rot[j][d]);
          if (rh < mn[d]) mn[d] = rh;
          if (rh > mx[d]) mx[d] = rh;
        }
      }
      for (uint32_t j = 0; j < m; ++j) {
        uint16_t v[3];
        for (int d = 0; d < 3; ++d) v[d] = f3d_or_vox1(f3d_or_half_to_float(rot[j][d]), mn[d], mx[d], num_vox);
        cell[j] = (uint16_t)(f3d_or_zorder16(v[0], v[1], v[2]) / 8u);
        keys[j] = ((uint32_t)cell[j] << 10) | j;
      }
      qsort(keys, m, sizeof(uint32_t), cmp_u32);
      uint32_t row_base = rstart + t * rows_per_tile;
      for (uint32_t rank = 0; rank < m; ++rank) {
        uint32_t j = keys[rank] & 1023u;
        uint32_t g = t0 + j;
        uint32_t sub = rank / S, off = rank % S;
        subbuck_id[g] = t * rows_per_tile + sub;
        subbuck_off[g] = (uint16_t)off;
        unpool_ind[(size_t)(row_base + sub) * S + off] = g;
      }
      uint32_t nrow = (m + S - 1) / S;
      for (uint32_t sub = 0; sub < nrow; ++sub) {
        uint32_t cnt = (m - sub * S < S) ? m - sub * S : S;
        for (int d = 0; d < 3; ++d) {
          volatile float acc = 0.f;
          for (uint32_t s = 0; s < cnt; ++s) {
            uint32_t j = keys[sub * S + s] & 1023u;
            acc = acc + f3d_or_half_to_float(coord_h[3 * (size_t)(t0 + j) + d]);
          }
          volatile float mean = acc / (float)cnt;
          reduced_coord_h[3 * (size_t)(row_base + sub) + d] = f3d_or_float_to_half(mean);
        }
      }
    }
    start = end;
    rstart = rend;
  }
  (void)total_n;
  for (size_t r = rstart; r < r_aligned; ++r)
    for (int d = 0; d < 3; ++d) reduced_coord_h[3 * r + d] = 0;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* A7: feature reduce — src/psh/batch_psh_subbuck_reduce.cuh:300-359, op enum :47-52            */
/* fp32 accumulate in slot order, mean divides by the number of valid slots, empty row -> 0,    */
/* bf16 round-to-nearest-even.  Rows [reduced_n, r_aligned) are zero-filled.                      */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_reduce_feat(const uint16_t *feat_bf, uint32_t total_n, uint32_t feat_dim,
                       const uint32_t *unpool_ind, uint32_t reduced_n, uint32_t subbuck_size,
                       uint32_t red_op, uint16_t *reduced_bf, uint32_t r_aligned) {
  if (red_op > 3) return -1;
  for (uint32_t r = 0; r < reduced_n; ++r) {
    for (uint32_t c = 0; c < feat_dim; ++c) {
      float acc = (red_op == 2) ? INFINITY : (red_op == 3) ? -INFINITY : 0.f;
      uint32_t cnt = 0;
      for (uint32_t s = 0; s < subbuck_size; ++s) {
        uint32_t row = unpool_ind[(size_t)r * subbuck_size + s];
        if (row < total_n) {
          ++cnt;
          float v = f3d_or_bf16_to_float(feat_bf[(size_t)row * feat_dim + c]);
          if (red_op <= 1) acc = acc + v;
          else if (red_op == 2) acc = (v < acc) ? v : acc;
          else acc = (v > acc) ? v : acc;
        }
      }
      if (red_op == 0) acc = acc / (float)cnt;
      if (cnt == 0) acc = 0.f;
      reduced_bf[(size_t)r * feat_dim + c] = f3d_or_float_to_bf16(acc);
    }
  }
  for (size_t r = reduced_n; r < r_aligned; ++r)
    for (uint32_t c = 0; c < feat_dim; ++c) reduced_bf[r * feat_dim + c] = 0;
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* A8: additive unpool — src/psh/additive_unpool.cuh:43-86                                      */
/* up[r, c] = bf16(float(down[i, c]) + float(res[r, c])) for r = unpool_ind[i, s] < up_n.        */
/* Rows of `up` that no slot references are left untouched (caller decides their content).       */
/* ------------------------------------------------------------------------------------------ */

int f3d_or_additive_unpool(const uint16_t *res_bf, const uint16_t *down_bf, uint16_t *up_bf,
                           const uint32_t *unpool_ind, uint32_t up_n, uint32_t down_n,
                           uint32_t feat_dim, uint32_t subbuck_size) {
  for (uint32_t i = 0; i < down_n; ++i)
    for (uint32_t s = 0; s < subbuck_size; ++s) {
      uint32_t r = unpool_ind[(size_t)i * subbuck_size + s];
      if (r >= up_n) continue;
      for (uint32_t c = 0; c < feat_dim; ++c) {
        float sum = f3d_or_bf16_to_float(down_bf[(size_t)i * feat_dim + c]) +
                             f3d_or_bf16_to_float(res_bf[(size_t)r * feat_dim + c]);
        up_bf[(size_t)r * feat_dim + c] = f3d_or_float_to_bf16(sum);
      }
    }
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* backward of A8 and A7 — src/psh/additive_unpool.cuh:90-137,                                   */
/* src/psh/batch_psh_subbuck_reduce_bwd.cuh:39-126                                              */
/* ------------------------------------------------------------------------------------------ */
int f3d_or_additive_unpool_bwd(uint16_t *grad_res, uint16_t *grad_down, const uint16_t *grad_up,
                               const uint32_t *unpool_ind, uint32_t up_n, uint32_t down_n,
                               uint32_t feat_dim, uint32_t subbuck_size) {
  for (uint32_t i = 0; i < down_n; ++i)
    for (uint32_t c = 0; c < feat_dim; ++c) {
      float acc = 0.f;
      for (uint32_t s = 0; s < subbuck_size; ++s) {
        uint32_t r = unpool_ind[(size_t)i * subbuck_size + s];
        if (r >= up_n) continue;
        uint16_t g = grad_up[(size_t)r * feat_dim + c];
        grad_res[(size_t)r * feat_dim + c] = g;
        acc = acc + f3d_or_bf16_to_float(g);
      }
      grad_down[(size_t)i * feat_dim + c] = f3d_or_float_to_bf16(acc);
    }
  return 0;
}

/* The division of the mean is the correctly rounded fp32 quotient (the reference is built with fast math,
 * whose approximate quotient can differ in the last fp32 bit, i.e. at rare bf16 rounding ties). */
int f3d_or_reduce_feat_bwd(const uint16_t *grad_red, const uint16_t *input_bf, const uint32_t *unpool_ind,
                           uint16_t *grad_in, uint32_t total_n, uint32_t reduced_n, uint32_t feat_dim,
                           uint32_t subbuck_size, uint32_t red_op) {
  if (red_op > 3) return -1;
  for (uint32_t r = 0; r < reduced_n; ++r)
    for (uint32_t c = 0; c < feat_dim; ++c) {
      const uint32_t *ind = unpool_ind + (size_t)r * subbuck_size;
      uint16_t g = grad_red[(size_t)r * feat_dim + c];
      if (red_op <= 1) {
        uint32_t cnt = 0;
        for (uint32_t s = 0; s < subbuck_size; ++s) cnt += ind[s] < total_n;
        uint16_t out = g;
        if (red_op == 0) out = f3d_or_float_to_bf16(f3d_or_bf16_to_float(g) / (float)(cnt > 1 ? cnt : 1));
        for (uint32_t s = 0; s < subbuck_size; ++s)
          if (ind[s] < total_n) grad_in[(size_t)ind[s] * feat_dim + c] = out;
      } else {
        float best = (red_op == 3) ? -INFINITY : INFINITY;
        uint32_t win = 0;
        for (uint32_t s = 0; s < subbuck_size; ++s) {
          if (ind[s] >= total_n) continue;
          float v = f3d_or_bf16_to_float(input_bf[(size_t)ind[s] * feat_dim + c]);
          int better = (red_op == 3) ? (v > best) : (v < best);
          if (better) { best = v; win = s; }
        }
        for (uint32_t s = 0; s < subbuck_size; ++s)
          if (ind[s] < total_n) grad_in[(size_t)ind[s] * feat_dim + c] = (s == win) ? g : 0;
      }
    }
  return 0;
}
