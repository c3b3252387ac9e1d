// Device-side building blocks shared by the gfx950 kernels: 16-bit float conversions, the voxel
// quantiser and first-hash family, the stateless RNG, and wave64 helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace f3d {

constexpr int kWave = 64;

// Workgroup barrier that waits for this wave's LDS operations only.  __syncthreads() also waits for every outstanding
// global load and store of the wave (its release fence covers global memory), which serialises a loop whose stores
// and direct-to-LDS loads are meant to stay in flight across the barrier; what such a loop needs from global memory
// it waits for explicitly (s_waitcnt vmcnt).  The "memory" clobber keeps the compiler from moving accesses across.
__device__ __forceinline__ void wg_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- 16-bit float bit patterns <-> fp32 -------------------------------------------------------

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);  // v_cvt_f16_f32: round to nearest even
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));  // one 16-byte chunk = 8 bf16 / fp16 values

// two fp32 -> packed bf16 pair (low half = a), one instruction
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }

// ---- voxel quantiser (reference: src/psh/hash_fns.cuh:23-33) ----------------------------------
// floor(q), clamped to [0, num_vox - 1] with NaN -> num_vox - 1, where q is one of two roundings of
// (c - min) * num_vox / (max - min):
//   mode 0 (default): q = ((c - min) * num_vox) * inv with inv = 1 / (max - min) rounded once: what a build of
//           the reference with nvcc --use_fast_math (its CMakeLists.txt:49-52) evaluates, given an exact reciprocal;
//   mode 1: q = ((c - min) * num_vox) / (max - min), the IEEE division the source text spells out.
// All steps are separate IEEE fp32 operations: the translation units that use this are built with
// -ffp-contract=off.  Kernels receive the mode in bit 31 of their num_vox argument (num_vox <= 65536).
constexpr uint32_t kVoxDivideBit = 0x80000000u;

struct VoxAxis {
  float mn, inv, nv, hi, den;
  bool divide;
};

__device__ __forceinline__ VoxAxis make_vox_axis_f(float mn, float mx, uint32_t num_vox_mode) {
  const uint32_t num_vox = num_vox_mode & ~kVoxDivideBit;
  VoxAxis a;
  a.mn = mn;
  a.den = __fsub_rn(mx, mn);
  a.inv = __fdiv_rn(1.0f, a.den);
  a.nv = (float)num_vox;
  a.hi = (float)(num_vox - 1u);
  a.divide = (num_vox_mode & kVoxDivideBit) != 0;
  return a;
}

// the same with the reciprocal of the extent, fl(1 / fl(max - min)), computed by the caller
__device__ __forceinline__ VoxAxis make_vox_axis_inv(float mn, float mx, float inv, uint32_t num_vox_mode) {
  const uint32_t num_vox = num_vox_mode & ~kVoxDivideBit;
  VoxAxis a;
  a.mn = mn;
  a.den = __fsub_rn(mx, mn);
  a.inv = inv;
  a.nv = (float)num_vox;
  a.hi = (float)(num_vox - 1u);
  a.divide = (num_vox_mode & kVoxDivideBit) != 0;
  return a;
}

__device__ __forceinline__ VoxAxis make_vox_axis(uint16_t min_h, uint16_t max_h, uint32_t num_vox_mode) {
  return make_vox_axis_f(half_bits_to_float(min_h), half_bits_to_float(max_h), num_vox_mode);
}

__device__ __forceinline__ uint32_t vox1(float c, const VoxAxis& a) {
  const float t = __fmul_rn(__fsub_rn(c, a.mn), a.nv);
  const float q = a.divide ? __fdiv_rn(t, a.den) : __fmul_rn(t, a.inv);
  float v = floorf(q);
  float m = (v < a.hi) ? v : a.hi;  // NaN -> hi
  float r = (m > 0.f) ? m : 0.f;
  return (uint32_t)r;
}

// ---- first-hash family (reference: src/psh/hash_fns.cuh:48-135) --------------------------------

// spread the low 6 bits of x to bit positions 0,3,6,9,12,15
__device__ __forceinline__ uint32_t spread3_6(uint32_t x) {
  x = (x | (x << 8)) & 0x0000300Fu;
  x = (x | (x << 4)) & 0x000030C3u;
  x = (x | (x << 2)) & 0x00009249u;
  return x;
}

// low 16 bits of (morton48(x,y,z) >> 31): bits, from bit 0 up, y10 z10 x11 y11 z11 ... x15 y15
__device__ __forceinline__ uint32_t zorder16(uint32_t vx, uint32_t vy, uint32_t vz) {
  uint32_t xs = spread3_6((vx >> 11) & 0x1Fu);
  uint32_t ys = spread3_6((vy >> 10) & 0x3Fu);
  uint32_t zs = spread3_6((vz >> 10) & 0x1Fu);
  return (ys | (zs << 1) | (xs << 2)) & 0xFFFFu;
}

// Exact division of a 16-bit number by a 16-bit divisor with one multiply: q = mulhi(x, ceil(2^32 / d)) equals
// floor(x / d) for all x, d < 2^16 (the rounding error of the reciprocal times x stays below 1 / d).
struct Div16 {
  uint32_t d, magic;
};
__host__ __device__ __forceinline__ Div16 make_div16(uint32_t d) {
  Div16 r;
  r.d = d;
  r.magic = d > 1u ? (uint32_t)(0x100000000ull / d) + 1u : 0u;   // d = 1: quotient is x itself
  return r;
}
__device__ __forceinline__ uint32_t div16(uint32_t x, const Div16& v) {
  return v.d > 1u ? __umulhi(x, v.magic) : x;
}

// divisor16 / num_bucket16 are the 16-bit truncations the reference's HashT parameters apply
__device__ __forceinline__ uint32_t first_hash(uint32_t vx, uint32_t vy, uint32_t vz, uint32_t hash_type,
                                               uint32_t divisor16, uint32_t num_bucket16) {
  uint32_t h = (hash_type & 1u) ? zorder16(vx, vy, vz) : ((vx ^ vy ^ vz) & 0xFFFFu);
  return (hash_type <= 2u) ? h / divisor16 : h % num_bucket16;
}

// The same with the divisor prepared once (dv = make_div16(divisor16) for hash types 1 / 2, of num_bucket16 for
// 3 / 4) and the hash kind as compile-time constants, for the kernels that hash every point of a batch.
template <bool ZORDER, bool MOD>
__device__ __forceinline__ uint32_t first_hash_t(uint32_t vx, uint32_t vy, uint32_t vz, const Div16& dv) {
  const uint32_t h = ZORDER ? zorder16(vx, vy, vz) : ((vx ^ vy ^ vz) & 0xFFFFu);
  const uint32_t q = div16(h, dv);
  return MOD ? h - q * dv.d : q;
}

// ---- wave-cooperative access to runs of short records ---------------------------------------------------------
// A wave reads `bytes` consecutive bytes starting at the 2-byte aligned address `src` in aligned 16-byte pieces (lane
// l takes pieces l, l + 64, ...) and parks them in a wave-private LDS area; the run then starts at byte
// `returned shift` (0..14) of the area.  The first / last piece may reach up to 14 bytes before / past the run: they
// lie in the same 16-byte block as a byte of the run, hence in a page of the same allocation, but a piece that starts
// at or past `limit` (the end of the array) is not read.  MAXBYTES: largest run the caller passes.
template <uint32_t MAXBYTES>
constexpr uint32_t wave_run_area_bytes() {
  return ((MAXBYTES + 14u + 15u) / 16u) * 16u;
}
template <uint32_t MAXBYTES>
__device__ __forceinline__ uint32_t wave_fetch_run(const void* src, uint32_t bytes, const void* limit, char* area,
                                                   uint32_t lane) {
  const uintptr_t a = (uintptr_t)src, a0 = a & ~(uintptr_t)15, end = (uintptr_t)limit;
  const uint32_t shift = (uint32_t)(a - a0);
  const uint32_t pieces = (shift + bytes + 15u) / 16u;
  constexpr uint32_t MAXP = wave_run_area_bytes<MAXBYTES>() / 16u;
#pragma unroll
  for (uint32_t i = 0; i * kWave < MAXP; ++i) {
    const uint32_t p = lane + i * kWave;
    if (p < pieces && a0 + 16u * p < end)
      *reinterpret_cast<u32x4_t*>(area + 16u * p) = *reinterpret_cast<const u32x4_t*>(a0 + 16u * (uintptr_t)p);
  }
  return shift;
}

// ---- stateless RNG: 32-bit finaliser chained over (seed, a, b, c) -------------------------------

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU;
  x ^= x >> 15; x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

__device__ __forceinline__ uint32_t rng_u32(uint32_t seed, uint32_t a, uint32_t b, uint32_t c) {
  uint32_t h = mix32(seed + 0x9E3779B9u);
  h = mix32(h ^ (a + 0x85EBCA6Bu));
  h = mix32(h ^ (b + 0xC2B2AE35u));
  h = mix32(h ^ (c + 0x27D4EB2Fu));
  return h;
}

__device__ __forceinline__ float rng_u01(uint32_t seed, uint32_t a, uint32_t b, uint32_t c) {
  return (float)(rng_u32(seed, a, b, c) >> 8) * (1.0f / 16777216.0f);
}

// ---- wave64 helpers -----------------------------------------------------------------------------

__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// number of set bits of `mask` strictly below this lane
__device__ __forceinline__ uint32_t mask_rank(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Lanes of the wave whose `key` (low `nbits` bits significant) equals this lane's, restricted to
// lanes with `valid` set.  One ballot per key bit.
__device__ __forceinline__ uint64_t match_any(uint32_t key, uint32_t nbits, bool valid) {
  const uint64_t all = __ballot(valid);
  uint32_t lo = (uint32_t)all, hi = (uint32_t)(all >> 32);
  for (uint32_t k = 0; k < nbits; ++k) {
    const int32_t sbit = __builtin_amdgcn_sbfe((int32_t)key, k, 1u);   // all ones where this lane's bit is set
    const uint32_t sx = (uint32_t)sbit;
    const uint64_t b = __ballot(sbit < 0);
    lo &= ~((uint32_t)b ^ sx);                    // keep the lanes whose bit equals mine
    hi &= ~((uint32_t)(b >> 32) ^ sx);
  }
  return ((uint64_t)hi << 32) | lo;
}

}  // namespace f3d
