// PSH permutation index and row permutation of per-point features for gfx950.
// Completes batch_psh_cumsum_scatter_feat_index_postpad_ker (src/psh/batch_psh_bucket.cuh:617-753), which the
// reference leaves unfinished: it writes scatter_idx_out2in[dst] = src and the pad value total_N + 3 (:678) and
// stops before moving any feature.
//
// The destination row of input row g of cloud c is a closed form of what the bucketing op leaves behind:
//   dst = start_c + (cumsum_counter[c][b] - bucket_counter[c][b]) + bucket_offset[g],  b = bucket_id[g]
// (exclusive prefix of the final bucket counts plus the slot inside the bucket), so the index needs no state from
// inside the bucketing kernels.  One pass over the input rows writes the index and, if asked, moves the feature
// rows; a second entry point permutes further row-major tensors by the index in either direction.
// A row moves as one contiguous burst over neighbouring lanes (16 B per lane when the row size allows).
// HBM bound; algorithmic bytes per launch:
//   index + features : bucket_id 2 N + bucket_offset 4 N + index 4 pad_to + rows 2 * row_bytes * N (+ pad rows)
//   permute          : index 4 R + rows 2 * row_bytes * R
#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

// lanes that share one row: the smallest power of two that covers the row's units, at most one wave
static uint32_t lanes_for(uint32_t units) {
  uint32_t l = 1;
  while (l < units && l < kWave) l <<= 1;
  return l;
}

// rows [0, total_n): index and (optionally) feature row to the PSH position; rows [total_n, pad_to_n) of the
// outputs: index = total_n + 3, features zero.
template <typename V>
__global__ __launch_bounds__(256) void psh_index_scatter_kernel(
    const uint16_t* __restrict__ bucket_id, const uint32_t* __restrict__ bucket_offset,
    const uint32_t* __restrict__ bucket_counter, const uint32_t* __restrict__ cumsum_counter,
    const uint32_t* __restrict__ batch_sep, uint32_t batch_size, uint32_t total_n, uint32_t num_bucket,
    const V* __restrict__ feat, uint32_t units, uint32_t lanes_log2, uint32_t* __restrict__ idx_out2in,
    V* __restrict__ scattered_feat, uint32_t pad_to_n) {
  const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = gid >> lanes_log2, sub = gid & ((1u << lanes_log2) - 1u), lanes = 1u << lanes_log2;
  if (row >= pad_to_n) return;
  if (row >= total_n) {
    if (sub == 0) idx_out2in[row] = total_n + 3u;
    if (scattered_feat) {
      V zero = {};
      for (uint32_t u = sub; u < units; u += lanes) scattered_feat[(size_t)row * units + u] = zero;
    }
    return;
  }
  // The row's first unit, its bucket id and its slot are requested together: none of them depends on another, and
  // the destination needs the last two plus two table entries, which sit in the cache.
  V first = {};
  if (scattered_feat && sub < units) first = feat[(size_t)row * units + sub];
  const uint32_t b = bucket_id[row];
  const uint32_t slot = bucket_offset[row];
  // cloud of the row: first separator above it
  uint32_t lo = 0, hi = batch_size - 1;
  while (lo < hi) {
    const uint32_t mid = (lo + hi) >> 1;
    if (batch_sep[mid] > row) hi = mid; else lo = mid + 1;
  }
  const uint32_t start = lo ? batch_sep[lo - 1] : 0u;
  if (b >= num_bucket) return;   // not a bucket of this geometry: the buffers do not belong to these separators
  const size_t t = (size_t)lo * num_bucket + b;
  const uint32_t dst = start + (cumsum_counter[t] - bucket_counter[t]) + slot;
  if (dst >= total_n) return;    // same: a consistent set of buffers permutes rows inside [0, total_n)
  if (sub == 0) idx_out2in[dst] = row;
  if (scattered_feat) {
    if (sub < units) scattered_feat[(size_t)dst * units + sub] = first;
    for (uint32_t u = sub + lanes; u < units; u += lanes)
      scattered_feat[(size_t)dst * units + u] = feat[(size_t)row * units + u];
  }
}

// GATHER:  out[r] = idx[r] < n_other ? in[idx[r]] : 0      for r < n_idx   (out has n_idx rows, in has n_other)
// !GATHER: out[idx[r]] = in[r]  where idx[r] < n_other     for r < n_idx   (in has n_idx rows, out has n_other)
template <typename V, bool GATHER>
__global__ __launch_bounds__(256) void permute_rows_kernel(const uint32_t* __restrict__ idx, const V* __restrict__ in,
                                                           V* __restrict__ out, uint32_t n_idx, uint32_t n_other,
                                                           uint32_t units, uint32_t lanes_log2) {
  const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t row = gid >> lanes_log2, sub = gid & ((1u << lanes_log2) - 1u), lanes = 1u << lanes_log2;
  if (row >= n_idx) return;
  const uint32_t other = idx[row];
  const bool ok = other < n_other;
  if (GATHER) {
    V zero = {};
    for (uint32_t u = sub; u < units; u += lanes)
      out[(size_t)row * units + u] = ok ? in[(size_t)other * units + u] : zero;
  } else if (ok) {
    for (uint32_t u = sub; u < units; u += lanes) out[(size_t)other * units + u] = in[(size_t)row * units + u];
  }
}

struct RowShape {
  uint32_t unit_bytes, units, lanes_log2;
};

static RowShape row_shape(uint32_t row_bytes, const void* a, const void* b) {
  const uintptr_t bits = (uintptr_t)a | (uintptr_t)b | row_bytes;
  RowShape r;
  r.unit_bytes = (bits % 16 == 0) ? 16u : (bits % 8 == 0) ? 8u : (bits % 4 == 0) ? 4u : 2u;
  r.units = row_bytes / r.unit_bytes;
  const uint32_t lanes = lanes_for(r.units);
  r.lanes_log2 = 0;
  while ((1u << r.lanes_log2) < lanes) ++r.lanes_log2;
  return r;
}

}  // namespace f3d

extern "C" {

int f3d_psh_scatter_feat_index(const uint16_t* bucket_id, const uint32_t* bucket_offset,
                               const uint32_t* bucket_counter, const uint32_t* cumsum_counter,
                               const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n, uint32_t num_bucket,
                               const void* feat, uint32_t row_bytes, uint32_t* scatter_idx_out2in,
                               void* scattered_feat, uint32_t pad_to_n, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(bucket_id && bucket_offset && bucket_counter && cumsum_counter && batch_sep && scatter_idx_out2in,
                "null tensor pointer");
  F3D_CHECK_ARG((feat == nullptr) == (scattered_feat == nullptr), "feat and scattered_feat come together");
  F3D_CHECK_ARG(pad_to_n >= total_n, "Output buffer length(%u) is smaller than the input length(%u).", pad_to_n,
                total_n);
  F3D_CHECK_ARG(batch_size > 0 && num_bucket > 0, "empty batch");
  F3D_CHECK_ARG(!feat || (row_bytes > 0 && row_bytes % 2 == 0), "feature rows must be a positive even number of bytes");
  F3D_CHECK_ARG((uint64_t)pad_to_n * 64u < (1ull << 32), "too many rows for one launch");
  if (pad_to_n == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  RowShape rs = feat ? row_shape(row_bytes, feat, scattered_feat) : RowShape{16u, 0u, 0u};
  const uint32_t threads = 256, grid = cdiv_u32(pad_to_n << rs.lanes_log2, threads);
#define F3D_IDX(V)                                                                                                  \
  hipLaunchKernelGGL(psh_index_scatter_kernel<V>, dim3(grid), dim3(threads), 0, s, bucket_id, bucket_offset,       \
                     bucket_counter, cumsum_counter, batch_sep, batch_size, total_n, num_bucket, (const V*)feat,   \
                     rs.units, rs.lanes_log2, scatter_idx_out2in, (V*)scattered_feat, pad_to_n)
  switch (rs.unit_bytes) {
    case 16: F3D_IDX(uint4); break;
    case 8: F3D_IDX(uint2); break;
    case 4: F3D_IDX(uint32_t); break;
    default: F3D_IDX(uint16_t); break;
  }
#undef F3D_IDX
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

int f3d_permute_rows(const uint32_t* index, const void* in, void* out, uint32_t n_index, uint32_t n_other,
                     uint32_t row_bytes, uint32_t gather, int device, void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(index && in && out, "null tensor pointer");
  F3D_CHECK_ARG(row_bytes > 0 && row_bytes % 2 == 0, "rows must be a positive even number of bytes");
  F3D_CHECK_ARG((uint64_t)n_index * 64u < (1ull << 32), "too many rows for one launch");
  if (n_index == 0) return F3D_OK;
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  const RowShape rs = row_shape(row_bytes, in, out);
  const uint32_t threads = 256, grid = cdiv_u32(n_index << rs.lanes_log2, threads);
#define F3D_PERM(V)                                                                                                   \
  do {                                                                                                                \
    if (gather)                                                                                                       \
      hipLaunchKernelGGL((permute_rows_kernel<V, true>), dim3(grid), dim3(threads), 0, s, index, (const V*)in,       \
                         (V*)out, n_index, n_other, rs.units, rs.lanes_log2);                                         \
    else                                                                                                              \
      hipLaunchKernelGGL((permute_rows_kernel<V, false>), dim3(grid), dim3(threads), 0, s, index, (const V*)in,      \
                         (V*)out, n_index, n_other, rs.units, rs.lanes_log2);                                         \
  } while (0)
  switch (rs.unit_bytes) {
    case 16: F3D_PERM(uint4); break;
    case 8: F3D_PERM(uint2); break;
    case 4: F3D_PERM(uint32_t); break;
    default: F3D_PERM(uint16_t); break;
  }
#undef F3D_PERM
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
