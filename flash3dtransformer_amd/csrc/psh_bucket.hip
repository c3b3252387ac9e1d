// PSH bucketing for gfx950: voxel quantise -> first hash -> per-bucket slot claim -> cumsum ->
// scatter (+ tail padding).  Counterpart of the reference's three launches in
// src/psh/batch_psh_bucket_dispatcher.cu:287-320 (kernels in src/psh/batch_psh_bucket.cuh).
//
// Design (not a translation): the reference claims slots with shared->global atomics, so slot
// order depends on arbitration.  Here slots are a stable counting sort:
//   K1  hash_hist   one workgroup per tile of a cloud: quantise + hash, write bucket_id, LDS
//                   histogram of the tile -> tile_hist[cloud][tile][bucket]
//   K2a tile_scan   exclusive scan of tile_hist over the tiles of a cloud (in place -> tile base), totals
//   K2b bucket_plan per cloud: (optional) deterministic overflow rebalance plan, final bucket counts ->
//                   bucket_counter, inclusive scan over buckets -> cumsum_counter
//   K3  rank_scatter per tile: stable rank of every point among the tile's points of the same
//                   bucket (wave64 ballot matching + per-wave LDS counters), slot = tile base + rank,
//                   write bucket_offset and scatter the coordinate row; extra workgroups fill the pad rows
// No global atomics, no dependence on workgroup scheduling: bucket ids, counts AND slots are a pure
// function of the input.  HBM traffic per point: K1 6 B read + 2 B write, K3 8 B read + 10 B write.
#include <mutex>

#include "f3d_device.h"
#include "f3d_internal.h"

namespace f3d {

constexpr int kPshThreads = 256;

// Position inside a tile of the point handled by (wave w, round j, lane l): each wave owns a
// contiguous run of 64*ITEMS points and walks it 64 at a time, so (j, l) order is input order.
template <int ITEMS>
__device__ __forceinline__ uint32_t tile_pos(uint32_t w, uint32_t j, uint32_t l) {
  return w * (kWave * ITEMS) + j * kWave + l;
}

// The coordinate rows of a wave's 64 * ITEMS consecutive points are one run of 384 * ITEMS bytes: fetched in
// 16-byte pieces into a wave-private LDS area and picked up from there, a few vector-memory instructions per wave
// instead of three 2-byte loads per point (the memory pipeline is paced by instructions, not bytes, at that size).
template <int THREADS, int ITEMS, bool ZORDER, bool MOD>
__global__ __launch_bounds__(THREADS) void psh_hash_hist_kernel(
    const uint16_t* __restrict__ coord, uint16_t* __restrict__ bucket_id, const uint32_t* __restrict__ batch_sep,
    const uint16_t* __restrict__ bbox_min, const uint16_t* __restrict__ bbox_max, uint32_t num_vox, Div16 dv,
    uint32_t num_bucket, uint32_t total_n, uint32_t* __restrict__ tile_hist, uint32_t max_tiles) {
  extern __shared__ __attribute__((aligned(16))) uint32_t lds_hist[];
  constexpr uint32_t kRunBytes = 384u * ITEMS, kArea = wave_run_area_bytes<kRunBytes>();
  const uint32_t cloud = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
  const uint32_t start = cloud ? batch_sep[cloud - 1] : 0u;
  const uint32_t n = batch_sep[cloud] - start;
  const uint32_t tile0 = tile * (THREADS * ITEMS);
  if (tile0 >= n) return;  // uniform for the workgroup

  const uint32_t w = __builtin_amdgcn_readfirstlane(tid / kWave), l = tid % kWave;
  char* area = reinterpret_cast<char*>(lds_hist + num_bucket) + w * kArea;
  // this wave's rows [wave0, wave0 + rows) of the cloud
  const uint32_t wave0 = tile0 + w * (kWave * ITEMS);
  const uint32_t rows = wave0 < n ? min((uint32_t)(kWave * ITEMS), n - wave0) : 0u;
  uint32_t shift = 0;
  if (rows) shift = wave_fetch_run<kRunBytes>(coord + 3 * ((size_t)start + wave0), rows * 6u, coord + 3 * (size_t)total_n, area, l);

  for (uint32_t b = tid; b < num_bucket; b += THREADS) lds_hist[b] = 0u;
  VoxAxis ax[3];
#pragma unroll
  for (int d = 0; d < 3; ++d) ax[d] = make_vox_axis(bbox_min[d], bbox_max[d], num_vox);
  __syncthreads();

#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const uint32_t t = j * kWave + l;               // position inside the wave's run: (j, l) order is input order
    if (t < rows) {
      const uint16_t* p = reinterpret_cast<const uint16_t*>(area + shift + 6u * t);
      uint32_t v[3];
#pragma unroll
      for (int d = 0; d < 3; ++d) v[d] = vox1(half_bits_to_float(p[d]), ax[d]);
      const uint32_t id = first_hash_t<ZORDER, MOD>(v[0], v[1], v[2], dv);
      bucket_id[(size_t)start + wave0 + t] = (uint16_t)id;
      atomicAdd(&lds_hist[id], 1u);
    }
  }
  __syncthreads();
  uint32_t* out = tile_hist + ((size_t)cloud * max_tiles + tile) * num_bucket;
  for (uint32_t b = tid; b < num_bucket; b += THREADS) out[b] = lds_hist[b];
}

// ---- K2a: exclusive prefix of tile_hist over the tiles of a cloud -------------------------------
// grid (ceil(NB / 64), clouds) x 1024 threads.  Lane = bucket (64 neighbouring buckets per
// workgroup, so every access is a coalesced 256-byte row segment), wave = a contiguous range of tiles.
// Each wave first sums its range, the 16 partial sums are combined through LDS, then each wave
// rewrites its range with the running prefix.  All loads of a phase are independent of each other.
constexpr int kScanWaves = 16;

__global__ __launch_bounds__(kScanWaves * kWave) void psh_tile_scan_kernel(
    uint32_t* __restrict__ tile_hist, const uint32_t* __restrict__ bucket_counter_in, uint32_t* __restrict__ cnt_out,
    const uint32_t* __restrict__ batch_sep, uint32_t num_bucket, uint32_t tile_pts, uint32_t max_tiles) {
  __shared__ uint32_t part[kScanWaves][kWave];
  const uint32_t cloud = blockIdx.y, tid = threadIdx.x, w = tid / kWave, l = tid % kWave;
  const uint32_t b = blockIdx.x * kWave + l;
  const uint32_t start = cloud ? batch_sep[cloud - 1] : 0u;
  const uint32_t n = batch_sep[cloud] - start;
  const uint32_t ntile = (n + tile_pts - 1) / tile_pts;
  const uint32_t per = (ntile + kScanWaves - 1) / kScanWaves;
  const uint32_t t0 = min(w * per, ntile), t1 = min(t0 + per, ntile);
  const bool ok = b < num_bucket;
  uint32_t* h = tile_hist + (size_t)cloud * max_tiles * num_bucket + b;
  uint32_t sum = 0;
  if (ok)
    for (uint32_t t = t0; t < t1; ++t) sum += h[(size_t)t * num_bucket];
  part[w][l] = sum;
  __syncthreads();
  // slots continue from whatever the caller left in bucket_counter (zero by contract)
  uint32_t run = ok ? bucket_counter_in[(size_t)cloud * num_bucket + b] : 0u;
  for (uint32_t ww = 0; ww < w; ++ww) run += part[ww][l];
  if (ok) {
    for (uint32_t t = t0; t < t1; ++t) {
      const uint32_t c = h[(size_t)t * num_bucket];
      h[(size_t)t * num_bucket] = run;
      run += c;
    }
    if (w == kScanWaves - 1) cnt_out[(size_t)cloud * num_bucket + b] = run;
  }
}

// inclusive scan of lds_in[0..n) into lds_out[0..n) by the first wave (lane owns a contiguous chunk)
__device__ __forceinline__ uint32_t wave0_inclusive_scan(const uint32_t* lds_in, uint32_t* lds_out, uint32_t n,
                                                        uint32_t tid) {
  const uint32_t chunk = (n + kWave - 1) / kWave;
  const uint32_t b0 = tid * chunk;
  uint32_t sum = 0;
  for (uint32_t i = 0; i < chunk; ++i)
    if (b0 + i < n) sum += lds_in[b0 + i];
  uint32_t incl = sum;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off, kWave);
    if ((int)tid >= off) incl += up;
  }
  uint32_t run = incl - sum;
  for (uint32_t i = 0; i < chunk; ++i)
    if (b0 + i < n) {
      run += lds_in[b0 + i];
      lds_out[b0 + i] = run;
    }
  return __shfl(incl, kWave - 1, kWave);  // grand total
}

// ---- K2b: per-cloud bucket plan ---------------------------------------------------------------------
// One workgroup per cloud.  From the first-hash counts cnt[b]:
//   rebalance off: final counts = cnt.
//   rebalance on : points with slot >= bucket_size in a bucket other than 0 ("overflow units", ordered
//     by (bucket, slot)) are matched one to one, in order, with the free slots of the buckets other
//     than 0 that hold fewer than bucket_size points ("free units", ordered by (bucket, slot)); overflow
//     units beyond the total free capacity are appended to bucket 0, the recycle bucket.  For a z-order
//     hash this is the order-preserving (nearest in Morton order) transport of the excess.
// Outputs: bucket_counter = final counts, cumsum_counter = their inclusive scan, and for K3
// plan[cloud] = { cnt[NB], over_excl[NB], free_incl[NB], total_free }.
template <bool REBAL>
__global__ __launch_bounds__(kPshThreads) void psh_bucket_plan_kernel(
    const uint32_t* __restrict__ cnt_in, uint32_t* __restrict__ bucket_counter, uint32_t* __restrict__ cumsum_counter,
    uint32_t* __restrict__ plan, uint32_t num_bucket, uint32_t bucket_size) {
  extern __shared__ uint32_t lds_plan[];
  uint32_t* s_cnt = lds_plan;                 // first-hash counts
  uint32_t* s_a = lds_plan + num_bucket;      // overflow per bucket -> inclusive scan
  uint32_t* s_b = lds_plan + 2 * num_bucket;  // free per bucket -> inclusive scan
  uint32_t* s_fin = lds_plan + 3 * num_bucket;
  __shared__ uint32_t s_tot[2];
  const uint32_t cloud = blockIdx.x, tid = threadIdx.x;
  const uint32_t* cnt = cnt_in + (size_t)cloud * num_bucket;
  uint32_t* pl = plan + (size_t)cloud * (3 * num_bucket + 4);
  for (uint32_t b = tid; b < num_bucket; b += kPshThreads) {
    const uint32_t c = cnt[b];
    s_cnt[b] = c;
    if (REBAL) {
      s_a[b] = (b != 0 && c > bucket_size) ? c - bucket_size : 0u;
      s_b[b] = (b != 0 && c < bucket_size) ? bucket_size - c : 0u;
    }
  }
  __syncthreads();
  if (REBAL) {
    if (tid < kWave) {
      const uint32_t tot_over = wave0_inclusive_scan(s_a, s_a, num_bucket, tid);
      const uint32_t tot_free = wave0_inclusive_scan(s_b, s_b, num_bucket, tid);
      if (tid == 0) { s_tot[0] = tot_over; s_tot[1] = tot_free; }
    }
    __syncthreads();
    const uint32_t tot_over = s_tot[0], tot_free = s_tot[1];
    for (uint32_t b = tid; b < num_bucket; b += kPshThreads) {
      const uint32_t c = s_cnt[b];
      const uint32_t free_excl = b ? s_b[b - 1] : 0u, free_b = s_b[b] - free_excl;
      const uint32_t over_excl = b ? s_a[b - 1] : 0u;
      uint32_t fin;
      if (b == 0) {
        fin = c + (tot_over > tot_free ? tot_over - tot_free : 0u);
      } else {
        const uint32_t kept = c < bucket_size ? c : bucket_size;
        const uint32_t filled = tot_over > free_excl ? min(free_b, tot_over - free_excl) : 0u;
        fin = kept + filled;
      }
      s_fin[b] = fin;
      bucket_counter[(size_t)cloud * num_bucket + b] = fin;
      pl[b] = c;
      pl[num_bucket + b] = over_excl;
      pl[2 * num_bucket + b] = s_b[b];
    }
    if (tid == 0) pl[3 * num_bucket] = tot_free;
  } else {
    for (uint32_t b = tid; b < num_bucket; b += kPshThreads) {
      s_fin[b] = s_cnt[b];
      bucket_counter[(size_t)cloud * num_bucket + b] = s_cnt[b];
    }
  }
  __syncthreads();
  if (tid < kWave) wave0_inclusive_scan(s_fin, s_fin, num_bucket, tid);
  __syncthreads();
  for (uint32_t b = tid; b < num_bucket; b += kPshThreads) cumsum_counter[(size_t)cloud * num_bucket + b] = s_fin[b];
}

// Phases of one workgroup (one tile of THREADS * ITEMS points of one cloud):
//   1. every wave ranks its points inside their first-hash buckets (match + one LDS atomic per group),
//   2. the per-wave counts become exclusive prefixes over the waves,
//   3. every point gets its stable slot; rows that stay in their first-hash bucket are written (or
//      staged), rows in the overflow of a bucket are gathered densely over the lanes of the wave and
//      resolved there, so the search for their new bucket runs once per 64 of them rather than once
//      per 64 points,
//   4. STAGE (large tiles): the tile's rows are laid out in LDS in (bucket, slot) order and written run
//      by run, so that a bucket's rows of this tile reach memory as one contiguous piece instead of
//      isolated 6-byte writes.
// LDS layout in 32-bit words: head (per-wave counts [waves][NB]; STAGE reuses it for the staged rows,
// x|y as one word per row followed by z as 16 bits per row), then row_base, slot_base, s_cnt, s_over,
// s_free, [STAGE: linc, dst_base], then the tail (STAGE: staged bucket ids, 16 bits per row, which
// phase 3 borrows for the per-wave overflow lists; otherwise those lists, 64 entries of 16 bytes per wave).
template <int THREADS, int ITEMS, bool STAGE>
__host__ __device__ constexpr size_t psh_scatter_lds_bytes(uint32_t num_bucket) {
  const size_t waves = THREADS / kWave, tile = (size_t)THREADS * ITEMS;
  const size_t wave_words = waves * num_bucket, row_words = tile * 3 / 2;
  const size_t head = (STAGE && row_words > wave_words) ? row_words : wave_words;
  const size_t tables = (size_t)(STAGE ? 7 : 5) * num_bucket;
  const size_t tail = STAGE ? (tile / 2 > waves * 256 ? tile / 2 : waves * 256) : waves * 256;
  return (head + tables + tail) * sizeof(uint32_t);
}

// The large-tile configuration must fit eight waves per SIMD (at most 64 registers): its 1024-thread workgroups
// then run two to a CU.  With a few registers more a CU holds a single workgroup and the launch takes a third longer
// (measured: 173 against 127 us on 64 x 262,144 points).
template <int THREADS, int ITEMS, bool REBAL, bool STAGE>
__global__ __launch_bounds__(THREADS, (STAGE ? 8 : 1)) void psh_rank_scatter_kernel(
    const uint16_t* __restrict__ coord, uint16_t* __restrict__ bucket_id,
    uint32_t* __restrict__ bucket_offset, const uint32_t* __restrict__ batch_sep, uint32_t batch_size,
    const uint32_t* __restrict__ tile_base, const uint32_t* __restrict__ bucket_counter,
    const uint32_t* __restrict__ cumsum_counter, const uint32_t* __restrict__ plan, uint32_t num_bucket,
    uint32_t nbits, uint32_t max_tiles, uint32_t bucket_size, uint16_t* __restrict__ scatter_coord, uint32_t total_n,
    uint32_t pad_to_n, uint16_t pad_bits) {
  extern __shared__ uint32_t lds[];
  constexpr uint32_t kWaves = THREADS / kWave, kTile = THREADS * ITEMS;
  static_assert(!STAGE || kTile / 2 >= kWaves * 256, "the staged ids must cover the per-wave overflow lists");
  const uint32_t cloud = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;

  if (cloud == batch_size) {  // tail padding rows [total_n, pad_to_n)
    const uint32_t row0 = total_n + tile * kTile;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const uint32_t r = row0 + j * THREADS + tid;
      if (r < pad_to_n) {
        uint16_t* q = scatter_coord + 3 * (size_t)r;
        q[0] = pad_bits; q[1] = pad_bits; q[2] = pad_bits;
      }
    }
    return;
  }

  const uint32_t start = cloud ? batch_sep[cloud - 1] : 0u;
  const uint32_t n = batch_sep[cloud] - start;
  const uint32_t tile0 = tile * kTile;
  if (tile0 >= n) return;

  const uint32_t head_words = (STAGE && kTile * 3 / 2 > kWaves * num_bucket) ? kTile * 3 / 2 : kWaves * num_bucket;
  uint32_t* whist = lds;                               // [kWaves][NB] per-wave counts
  uint32_t* row_base = lds + head_words;               // [NB] first output row of the bucket (final layout)
  uint32_t* slot_base = row_base + num_bucket;         // [NB] tile base inside the first-hash bucket
  uint32_t* s_cnt = slot_base + num_bucket;            // REBAL: [NB] first-hash counts
  uint32_t* s_over = s_cnt + num_bucket;               // REBAL: [NB] exclusive scan of the overflow
  uint32_t* s_free = s_over + num_bucket;              // REBAL: [NB] inclusive scan of the free capacity
  uint32_t* linc = s_free + num_bucket;                // STAGE: [NB] inclusive scan of the tile's own bucket counts
  uint32_t* dst_base = linc + num_bucket;              // STAGE: [NB] output row of staged position 0 of the bucket
  uint32_t* tail = s_free + (STAGE ? 3 : 1) * num_bucket;
  uint32_t* s_xy = lds;                                // STAGE: [tile] x | y << 16, over the per-wave counts
  uint16_t* s_z = reinterpret_cast<uint16_t*>(lds + kTile);   // STAGE: [tile]
  uint16_t* s_id = reinterpret_cast<uint16_t*>(tail);  // STAGE: [tile] first-hash bucket, 0xFFFF = written directly
  const uint32_t w = tid / kWave, l = tid % kWave;
  uint4* ov_list = reinterpret_cast<uint4*>(tail) + w * kWave;   // this wave's gathered overflow rows: unit, source, x|y, z

  const uint32_t* tb = tile_base + ((size_t)cloud * max_tiles + tile) * num_bucket;
  const uint32_t* cs = cumsum_counter + (size_t)cloud * num_bucket;
  const uint32_t* fin = bucket_counter + (size_t)cloud * num_bucket;
  const uint32_t* pl = plan + (size_t)cloud * (3 * num_bucket + 4);
  for (uint32_t b = tid; b < num_bucket; b += THREADS) {
#pragma unroll
    for (uint32_t ww = 0; ww < kWaves; ++ww) whist[ww * num_bucket + b] = 0u;
    slot_base[b] = tb[b];
    row_base[b] = start + (cs[b] - fin[b]);  // exclusive cumsum of the final counts
    if (REBAL) {
      s_cnt[b] = pl[b];
      s_over[b] = pl[num_bucket + b];
      s_free[b] = pl[2 * num_bucket + b];
    }
  }
  const uint32_t tot_free = REBAL ? pl[3 * num_bucket] : 0u;

  // the tile's ids and rows, requested up front so that their latency hides behind the ranking
  uint32_t id[ITEMS], rank[ITEMS], pxy[ITEMS];
  uint16_t pz[ITEMS];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const uint32_t local = tile0 + tile_pos<ITEMS>(w, j, l);
    const bool in = local < n;
    const size_t g = (size_t)start + (in ? local : 0u);
    id[j] = in ? (uint32_t)bucket_id[g] : 0xFFFFFFFFu;
    const uint16_t* p = coord + 3 * g;
    pxy[j] = (uint32_t)p[0] | ((uint32_t)p[1] << 16);
    pz[j] = p[2];
  }
  __syncthreads();

  uint32_t* mine = whist + w * num_bucket;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const bool valid = id[j] != 0xFFFFFFFFu;
    const uint64_t peers = match_any(id[j], nbits, valid);
    const uint32_t r = mask_rank(peers);
    // the lowest peer claims the group's run of slots in the wave's counter and hands the old
    // value to the others
    uint32_t before = 0;
    if (valid && r == 0) before = atomicAdd(&mine[id[j]], (uint32_t)__popcll(peers));
    before = __shfl(before, __ffsll((unsigned long long)peers) - 1, kWave);
    rank[j] = before + r;
  }
  __syncthreads();
  // per-wave counts -> exclusive prefix over waves
  for (uint32_t b = tid; b < num_bucket; b += THREADS) {
    uint32_t run = 0;
#pragma unroll
    for (uint32_t ww = 0; ww < kWaves; ++ww) {
      const uint32_t c = whist[ww * num_bucket + b];
      whist[ww * num_bucket + b] = run;
      run += c;
    }
    if (STAGE) linc[b] = run;
  }
  __syncthreads();
  if (STAGE) {
    if (tid < kWave) wave0_inclusive_scan(linc, linc, num_bucket, tid);
    __syncthreads();
    // staged position p of bucket b goes to row row_base[b] + slot_base[b] + (p - first staged position of b)
    for (uint32_t b = tid; b < num_bucket; b += THREADS)
      dst_base[b] = row_base[b] + slot_base[b] - (b ? linc[b - 1] : 0u);
  }

  // Rows in the overflow of their bucket: the k-th overflow unit of the cloud takes the k-th free unit;
  // none left -> recycle bucket 0.  Lane i of the wave resolves the i-th gathered row.
  uint32_t ov_n = 0;   // wave-uniform
  auto resolve_overflow = [&]() {
    __builtin_amdgcn_wave_barrier();
    if (l < ov_n) {
      const uint4 e = ov_list[l];
      const uint32_t k = e.x;
      const size_t g = (size_t)start + tile0 + (w * (kWave * ITEMS) + e.y);
      uint32_t bucket, slot;
      if (k < tot_free) {
        uint32_t lo = 1, hi = num_bucket - 1;  // first bucket whose inclusive free count exceeds k
        while (lo < hi) {
          const uint32_t mid = (lo + hi) >> 1;
          if (s_free[mid] > k) hi = mid; else lo = mid + 1;
        }
        bucket = lo;
        slot = s_cnt[lo] + (k - s_free[lo - 1]);
      } else {
        bucket = 0;
        slot = s_cnt[0] + (k - tot_free);
      }
      bucket_id[g] = (uint16_t)bucket;
      bucket_offset[g] = slot;
      uint16_t* q = scatter_coord + 3 * ((size_t)row_base[bucket] + slot);
      q[0] = (uint16_t)e.z; q[1] = (uint16_t)(e.z >> 16); q[2] = (uint16_t)e.w;
    }
    __builtin_amdgcn_wave_barrier();
    ov_n = 0;
  };

#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const bool valid = id[j] != 0xFFFFFFFFu;
    const uint32_t bucket = valid ? id[j] : 0u;
    const uint32_t in_tile = mine[bucket] + rank[j];
    const uint32_t slot = slot_base[bucket] + in_tile;  // stable slot in the first-hash bucket
    const bool over = REBAL && valid && bucket != 0 && slot >= bucket_size;
    if (REBAL) {
      const uint64_t ovm = __ballot(over);
      if (ovm != 0) {
        const uint32_t n_ov = (uint32_t)__popcll(ovm);
        if (ov_n + n_ov > kWave) resolve_overflow();
        if (over)
          ov_list[ov_n + mask_rank(ovm)] = make_uint4(s_over[bucket] + (slot - bucket_size), j * kWave + l, pxy[j], pz[j]);
        ov_n += n_ov;
      }
    }
    if (STAGE) rank[j] = ((bucket ? linc[bucket - 1] : 0u) + in_tile) | (over ? 0x80000000u : 0u);  // staged position
    if (valid && !over) {
      const size_t g = (size_t)start + tile0 + tile_pos<ITEMS>(w, j, l);
      bucket_offset[g] = slot;
      if (!STAGE) {
        uint16_t* q = scatter_coord + 3 * ((size_t)row_base[bucket] + slot);
        q[0] = (uint16_t)pxy[j]; q[1] = (uint16_t)(pxy[j] >> 16); q[2] = pz[j];
      }
    }
  }
  if (REBAL) resolve_overflow();

  if (STAGE) {
    __syncthreads();   // the per-wave counts and overflow lists are consumed: their space takes the rows and ids
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (id[j] == 0xFFFFFFFFu) continue;
      const uint32_t pos = rank[j] & 0x7FFFFFFFu;
      s_id[pos] = (rank[j] >> 31) ? (uint16_t)0xFFFFu : (uint16_t)id[j];
      s_xy[pos] = pxy[j];
      s_z[pos] = pz[j];
    }
    __syncthreads();
    const uint32_t total = linc[num_bucket - 1];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const uint32_t pos = j * THREADS + tid;
      if (pos >= total) break;
      const uint32_t b = s_id[pos];
      if (b == 0xFFFFu) continue;
      uint16_t* q = scatter_coord + 3 * (size_t)(dst_base[b] + pos);
      const uint32_t xy = s_xy[pos];
      q[0] = (uint16_t)xy; q[1] = (uint16_t)(xy >> 16); q[2] = s_z[pos];
    }
  }
}

// min / max of every axis over all points; two-level: per-workgroup partials then one finishing wave.
__global__ __launch_bounds__(256) void bbox_partial_kernel(const uint16_t* __restrict__ coord, uint32_t total_n,
                                                          float* __restrict__ partial) {
  __shared__ float red[6][4];
  float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_n; i += (size_t)gridDim.x * blockDim.x) {
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      const float v = half_bits_to_float(coord[3 * i + d]);
      mn[d] = fminf(mn[d], v);
      mx[d] = fmaxf(mx[d], v);
    }
  }
#pragma unroll
  for (int d = 0; d < 3; ++d)
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mn[d] = fminf(mn[d], __shfl_xor(mn[d], off, kWave));
      mx[d] = fmaxf(mx[d], __shfl_xor(mx[d], off, kWave));
    }
  const uint32_t w = threadIdx.x / kWave;
  if (threadIdx.x % kWave == 0)
    for (int d = 0; d < 3; ++d) { red[d][w] = mn[d]; red[3 + d][w] = mx[d]; }
  __syncthreads();
  if (threadIdx.x < 6) {
    float a = red[threadIdx.x][0];
    for (int i = 1; i < 4; ++i) a = threadIdx.x < 3 ? fminf(a, red[threadIdx.x][i]) : fmaxf(a, red[threadIdx.x][i]);
    partial[blockIdx.x * 6 + threadIdx.x] = a;
  }
}

__global__ void bbox_final_kernel(const float* __restrict__ partial, uint32_t nblock, uint16_t* __restrict__ bbox_min,
                                  uint16_t* __restrict__ bbox_max) {
  const uint32_t d = threadIdx.x / kWave, l = threadIdx.x % kWave;  // 6 waves: one per output
  float a = d < 3 ? INFINITY : -INFINITY;
  for (uint32_t i = l; i < nblock; i += kWave) a = d < 3 ? fminf(a, partial[i * 6 + d]) : fmaxf(a, partial[i * 6 + d]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(a, off, kWave);
    a = d < 3 ? fminf(a, o) : fmaxf(a, o);
  }
  if (l == 0) {
    if (d < 3) bbox_min[d] = float_to_half_bits(a);
    else bbox_max[d - 3] = float_to_half_bits(a);
  }
}

static uint32_t pick_items(uint32_t instance_max_n, uint32_t batch_size) {
  // Larger tiles amortise the per-tile histogram traffic; smaller tiles give small inputs enough
  // workgroups to cover 256 CUs.
  const uint64_t pts = (uint64_t)instance_max_n * batch_size;
  if (pts >= (uint64_t)4 << 20) return 8;
  if (pts >= (uint64_t)1 << 20) return 4;
  if (pts >= (uint64_t)256 << 10) return 2;
  return 1;
}

template <int THREADS, int ITEMS, bool REBAL, bool STAGE>
static void launch_psh(const uint16_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter, uint32_t* bucket_offset,
                       const uint32_t* batch_sep, uint32_t batch_size, uint32_t total_n, uint32_t num_bucket,
                       uint32_t divisor16, uint32_t bucket_size, uint32_t num_vox, const uint16_t* bbox_min,
                       const uint16_t* bbox_max, uint32_t* cumsum_counter, uint16_t* scatter_coord, uint32_t pad_to_n,
                       uint16_t pad_bits, uint32_t hash_type, uint32_t* tile_hist, uint32_t* cnt_ws, uint32_t* plan_ws,
                       uint32_t max_tiles, uint32_t nbits, hipStream_t stream) {
  const uint32_t tile_pts = THREADS * ITEMS;
  if (max_tiles > 0 && batch_size > 0) {
    // hash types 1 / 2 divide the 16-bit hash by the divisor, 3 / 4 take it modulo the bucket count
    const bool zorder = (hash_type & 1u) != 0, mod = hash_type > 2u;
    const Div16 dv = make_div16(mod ? (num_bucket & 0xFFFFu) : divisor16);
    const size_t lds1 = num_bucket * sizeof(uint32_t) + (THREADS / kWave) * wave_run_area_bytes<384u * ITEMS>();
    auto k1 = zorder ? (mod ? psh_hash_hist_kernel<THREADS, ITEMS, true, true> : psh_hash_hist_kernel<THREADS, ITEMS, true, false>)
                     : (mod ? psh_hash_hist_kernel<THREADS, ITEMS, false, true> : psh_hash_hist_kernel<THREADS, ITEMS, false, false>);
    hipLaunchKernelGGL(k1, dim3(max_tiles, batch_size), dim3(THREADS), lds1, stream, coord, bucket_id, batch_sep,
                       bbox_min, bbox_max, num_vox | quantiser_bit(), dv, num_bucket, total_n, tile_hist, max_tiles);
    hipLaunchKernelGGL(psh_tile_scan_kernel, dim3(cdiv_u32(num_bucket, kWave), batch_size), dim3(kScanWaves * kWave), 0,
                       stream, tile_hist, bucket_counter, cnt_ws, batch_sep, num_bucket, tile_pts, max_tiles);
    hipLaunchKernelGGL(psh_bucket_plan_kernel<REBAL>, dim3(batch_size), dim3(kPshThreads),
                       4 * num_bucket * sizeof(uint32_t), stream, cnt_ws, bucket_counter, cumsum_counter, plan_ws,
                       num_bucket, bucket_size);
  }
  const uint32_t pad_tiles = cdiv_u32(pad_to_n - total_n, tile_pts);
  const uint32_t gx = max_tiles > pad_tiles ? max_tiles : pad_tiles;
  if (gx > 0) {
    const size_t lds = psh_scatter_lds_bytes<THREADS, ITEMS, STAGE>(num_bucket);
    auto kern = psh_rank_scatter_kernel<THREADS, ITEMS, REBAL, STAGE>;
    if (lds > 64 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, dim3(gx, batch_size + (pad_tiles ? 1 : 0)),
                       dim3(THREADS), lds, stream, coord, bucket_id,
                       bucket_offset, batch_sep, batch_size, tile_hist, bucket_counter, cumsum_counter, plan_ws,
                       num_bucket, nbits, max_tiles, bucket_size, scatter_coord, total_n, pad_to_n, pad_bits);
  }
}


// ---- scratch memory of the entry point that allocates nothing ---------------------------------------
// f3d_batch_psh_scatter_pad_hash_noalloc keeps the tile histograms, first-hash counts and the rebalance
// plan in this array instead of the grow-only workspace.  Every GPU the library runs on holds its own copy
// until the process ends.  The name `scratch` is a host-side stand-in for the symbol, not a device
// address: host code only ever uses the per-device address that hipGetSymbolAddress returned.
constexpr size_t kNoAllocScratchWords = F3D_PSH_NOALLOC_SCRATCH_BYTES / sizeof(uint32_t);
static __device__ __align__(256) uint32_t scratch[kNoAllocScratchWords];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static uint32_t* g_scratch_ptr[kMaxDevices] = {};

// Address of this device's copy of `scratch`; resolved once per device, with that device current.
// Returns nullptr (and sets the error) on failure.
uint32_t* psh_noalloc_scratch(int device) {
  if (device < 0 || device >= kMaxDevices) {
    set_error("device index %d outside [0, %d)", device, kMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[device]) return g_scratch_ptr[device];
  DeviceGuard guard(device);
  if (!guard.ok) {
    set_error("cannot select device %d", device);
    return nullptr;
  }
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || ptr == nullptr) {
    set_error("hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(e));
    return nullptr;
  }
  g_scratch_ptr[device] = static_cast<uint32_t*>(ptr);
  return g_scratch_ptr[device];
}

// Checks, kernel selection and the four launches shared by the two entry points.  `ws` = scratch memory of
// `ws_words` 32-bit words, or nullptr: then the library's grow-only workspace is used (and may be allocated).
static int psh_run(const f3d_half_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter,
                   uint32_t* bucket_offset, const uint32_t* batch_sep, uint32_t batch_size,
                   uint32_t total_n, uint32_t instance_max_n, uint32_t num_bucket,
                   uint32_t bucket_divisor, uint32_t bucket_size, uint32_t num_vox,
                   const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                   const int16_t* probe_offsets, uint32_t* cumsum_counter,
                   f3d_half_t* scatter_coord, uint32_t pad_to_n, float pad_num,
                   uint32_t hash_type, int device, void* stream, bool no_alloc) {
  // The probe table is part of the reference signature; the deterministic rebalance below does not
  // probe (see psh_bucket_plan_kernel) and never reads it.
  (void)probe_offsets;
  // argument checks of src/psh/batch_psh_bucket_dispatcher.cu:239-250
  F3D_CHECK_ARG(bucket_divisor != 0 && num_bucket != 0 && num_vox / bucket_divisor <= num_bucket,
                "bucket divisor too small");
  F3D_CHECK_ARG(pad_to_n >= total_n, "Output coord buffer length(%u) is smaller than the input length(%u).",
                pad_to_n, total_n);
  F3D_CHECK_ARG(hash_type >= 1 && hash_type <= 4,
                "Currently only four types of hash modes are supported. Requested hash_type=%u is unsupported.",
                hash_type);
  if (!(num_bucket == 32 || num_bucket == 64 || num_bucket == 128 || num_bucket == 256 || num_bucket == 512 ||
        num_bucket == 1024)) {
    set_error("No kernel found for num_bucket=%u hash_type=%u", num_bucket, hash_type);
    return F3D_ERR_UNSUPPORTED;
  }
  const uint32_t div16 = bucket_divisor & 0xFFFFu;
  F3D_CHECK_ARG(div16 != 0 && (hash_type > 2 || 0xFFFFu / div16 < num_bucket), "bucket divisor too small");
  F3D_CHECK_ARG(num_vox >= 2 && num_vox <= 0x10000u, "num_vox=%u does not fit the 16-bit voxel type", num_vox);
  F3D_CHECK_ARG(coord && bucket_id && bucket_counter && bucket_offset && batch_sep && bbox_min && bbox_max &&
                    cumsum_counter && scatter_coord,
                "null tensor pointer");
  if (pad_to_n == 0) return F3D_OK;

  hipStream_t s = (hipStream_t)stream;
  // Inputs large enough to fill the chip with 8192-point tiles use 1024-thread workgroups that stage
  // the scatter through LDS; smaller ones use 256-thread workgroups with tiles sized for parallelism.
  constexpr int kBigThreads = 1024, kBigItems = 8;
  const bool big = (uint64_t)cdiv_u32(instance_max_n, 8192u) * batch_size >= 512u;
  const uint32_t items = big ? (uint32_t)kBigItems : pick_items(instance_max_n, batch_size);
  const uint32_t tile_pts = (big ? (uint32_t)kBigThreads : (uint32_t)kPshThreads) * items;
  const uint32_t max_tiles = cdiv_u32(instance_max_n, tile_pts);
  const size_t hist_words = (size_t)batch_size * max_tiles * num_bucket;
  const size_t cnt_words = (size_t)batch_size * num_bucket;
  const size_t plan_words = (size_t)batch_size * (3 * num_bucket + 4);
  const size_t ws_words = hist_words + cnt_words + plan_words + 4;
  if (no_alloc && ws_words > kNoAllocScratchWords) {
      set_error("f3d_batch_psh_scatter_pad_hash_noalloc: this batch needs %zu bytes of scratch memory (%u clouds x %u "
              "tiles x %u buckets), the fixed scratch array holds %zu; use f3d_batch_psh_scatter_pad_hash",
              ws_words * sizeof(uint32_t), batch_size, max_tiles, num_bucket, kNoAllocScratchWords * sizeof(uint32_t));
    return F3D_ERR_UNSUPPORTED;
  }
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  uint32_t* tile_hist = no_alloc ? psh_noalloc_scratch(device) : (uint32_t*)workspace(device, ws_words * sizeof(uint32_t), s);
  if (!tile_hist) return F3D_ERR_RUNTIME;
  uint32_t* cnt_ws = tile_hist + hist_words;
  uint32_t* plan_ws = cnt_ws + cnt_words;
  const bool rebal = rebalance_mode() != 0 && bucket_size > 0;
  uint32_t nbits = 0;
  while ((1u << nbits) < num_bucket) ++nbits;
  _Float16 pad_h = (_Float16)pad_num;
  uint16_t pad_bits;
  __builtin_memcpy(&pad_bits, &pad_h, 2);

  SyncBracket sync(s);
#define F3D_PSH_ARGS                                                                                              \
  coord, bucket_id, bucket_counter, bucket_offset, batch_sep, batch_size, total_n, num_bucket, div16, bucket_size, \
      num_vox, bbox_min, bbox_max, cumsum_counter, scatter_coord, pad_to_n, pad_bits, hash_type, tile_hist, cnt_ws, \
      plan_ws, max_tiles, nbits, s
#define F3D_PSH_CASE(I)                                                                  \
  case I:                                                                                \
    if (rebal) launch_psh<kPshThreads, I, true, false>(F3D_PSH_ARGS);                    \
    else launch_psh<kPshThreads, I, false, false>(F3D_PSH_ARGS);                         \
    break;
  if (big) {
    if (rebal) launch_psh<kBigThreads, kBigItems, true, true>(F3D_PSH_ARGS);
    else launch_psh<kBigThreads, kBigItems, false, true>(F3D_PSH_ARGS);
  } else {
    switch (items) {
      F3D_PSH_CASE(1)
      F3D_PSH_CASE(2)
      F3D_PSH_CASE(4)
      F3D_PSH_CASE(8)
    }
  }
#undef F3D_PSH_CASE
#undef F3D_PSH_ARGS
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // namespace f3d

extern "C" {

int f3d_batch_psh_scatter_pad_hash(const f3d_half_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter,
                                   uint32_t* bucket_offset, const uint32_t* batch_sep, uint32_t batch_size,
                                   uint32_t total_n, uint32_t instance_max_n, uint32_t num_bucket,
                                   uint32_t bucket_divisor, uint32_t bucket_size, uint32_t num_vox,
                                   const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                                   const int16_t* probe_offsets, uint32_t* cumsum_counter,
                                   f3d_half_t* scatter_coord, uint32_t pad_to_n, float pad_num,
                                   uint32_t hash_type, int device, void* stream) {
  return f3d::psh_run(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, batch_size, total_n, instance_max_n,
                      num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max, probe_offsets,
                      cumsum_counter, scatter_coord, pad_to_n, pad_num, hash_type, device, stream, false);
}

int f3d_batch_psh_scatter_pad_hash_noalloc(const f3d_half_t* coord, uint16_t* bucket_id, uint32_t* bucket_counter,
                                           uint32_t* bucket_offset, const uint32_t* batch_sep, uint32_t batch_size,
                                           uint32_t total_n, uint32_t instance_max_n, uint32_t num_bucket,
                                           uint32_t bucket_divisor, uint32_t bucket_size, uint32_t num_vox,
                                           const f3d_half_t* bbox_min, const f3d_half_t* bbox_max,
                                           const int16_t* probe_offsets, uint32_t* cumsum_counter,
                                           f3d_half_t* scatter_coord, uint32_t pad_to_n, float pad_num,
                                           uint32_t hash_type, int device, void* stream) {
  return f3d::psh_run(coord, bucket_id, bucket_counter, bucket_offset, batch_sep, batch_size, total_n, instance_max_n,
                      num_bucket, bucket_divisor, bucket_size, num_vox, bbox_min, bbox_max, probe_offsets,
                      cumsum_counter, scatter_coord, pad_to_n, pad_num, hash_type, device, stream, true);
}

int f3d_coord_bbox(const f3d_half_t* coord, uint32_t total_n, f3d_half_t* bbox_min, f3d_half_t* bbox_max, int device,
                   void* stream) {
  using namespace f3d;
  F3D_CHECK_ARG(coord && bbox_min && bbox_max, "null tensor pointer");
  F3D_CHECK_ARG(total_n > 0, "bounding box of an empty point set");
  DeviceGuard guard(device);
  F3D_CHECK_ARG(guard.ok, "cannot select device %d", device);
  hipStream_t s = (hipStream_t)stream;
  uint32_t nblock = cdiv_u32(total_n, 256 * 8);
  if (nblock > 1024) nblock = 1024;
  // partials live after the PSH histogram area would; a private slice at the workspace start is
  // enough because the op is ordered on the same stream as its consumers
  float* partial = (float*)workspace(device, (size_t)1024 * 6 * sizeof(float), s);
  if (!partial) return F3D_ERR_RUNTIME;
  SyncBracket sync(s);
  hipLaunchKernelGGL(bbox_partial_kernel, dim3(nblock), dim3(256), 0, s, coord, total_n, partial);
  hipLaunchKernelGGL(bbox_final_kernel, dim3(1), dim3(6 * kWave), 0, s, partial, nblock, bbox_min, bbox_max);
  F3D_CHECK_HIP(hipGetLastError());
  return F3D_OK;
}

}  // extern "C"
