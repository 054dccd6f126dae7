// Latent-major pair list (CSR over latents) construction, plus small utility kernels
// (column sums, fills, casts).
#pragma once

#include "common.hpp"

namespace flexsae {

// ---------------------------------------------------------------------------------
// Pair list.  count (keeping each pair's rank in its group) -> exclusive scan -> fill -> sort
// each group ascending.
// ---------------------------------------------------------------------------------

__global__ void fill_u32_kernel(uint32_t *__restrict__ p, int64_t n, uint32_t value) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    p[i] = value;
}

// Start of a pair-list build: zero the per-latent counters and the long-latent counter.
__global__ void csr_init_kernel(uint32_t *__restrict__ counts, int64_t n, uint32_t *__restrict__ long_count) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    counts[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x == 0) *long_count = 0u;
}

// counts[f] += 1 for every pair, and rank[p] = the value the counter had before: a position
// inside the latent's group that is unique but depends on the order the atomics were served in
// (the groups are sorted afterwards).  Out-of-range indices are flagged and counted as latent 0.
__global__ void csr_count_kernel(const int64_t *__restrict__ indices, int64_t n_pairs, int64_t F,
                                 uint32_t *__restrict__ counts, uint32_t *__restrict__ rank,
                                 int *status_flag) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < n_pairs;
       p += stride) {
    int64_t f = indices[p];
    if (static_cast<uint64_t>(f) >= static_cast<uint64_t>(F)) {
      if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
      f = 0;
    }
    rank[p] = atomicAdd(counts + f, 1u);
  }
}

// Exclusive scan of the per-latent counts in two launches.  Every block owns kScanBlockElems
// consecutive latents: csr_scan_sums_kernel writes the block totals, csr_scan_apply_kernel
// adds up the totals of the blocks before it (a few hundred values at most), scans its own
// elements and writes begin[]; the last block writes begin[F].
constexpr int kScanThreads = 256;
constexpr int kScanPerThread = 8;
constexpr int kScanBlockElems = kScanThreads * kScanPerThread;

__device__ __forceinline__ uint32_t block_sum_u32(uint32_t v, uint32_t *smem /*[kScanThreads/64]*/) {
  // all threads receive the block total
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  const int wv = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) smem[wv] = v;
  __syncthreads();
  uint32_t t = 0;
  for (int w = 0; w < kScanThreads / kWave; ++w) t += smem[w];
  return t;
}

__global__ __launch_bounds__(kScanThreads) void csr_scan_sums_kernel(const uint32_t *__restrict__ counts,
                                                                     int64_t F,
                                                                     uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t smem[kScanThreads / kWave];
  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kScanBlockElems +
                     static_cast<int64_t>(threadIdx.x) * kScanPerThread;
  uint32_t tsum = 0;
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i) tsum += (i0 + i < F) ? counts[i0 + i] : 0u;
  const uint32_t tot = block_sum_u32(tsum, smem);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = tot;
}

__global__ __launch_bounds__(kScanThreads) void csr_scan_apply_kernel(uint32_t *__restrict__ begin,
                                                                      int64_t F,
                                                                      const uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t smem[kScanThreads / kWave];
  __shared__ uint32_t wave_tot[kScanThreads / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid >> 6;
  // offset of this block = sum of the totals of all earlier blocks
  uint32_t part = 0;
  for (uint32_t j = tid; j < blockIdx.x; j += kScanThreads) part += block_sums[j];
  const uint32_t block_off = block_sum_u32(part, smem);

  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kScanBlockElems +
                     static_cast<int64_t>(tid) * kScanPerThread;
  uint32_t x[kScanPerThread];
  uint32_t tsum = 0;
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i) {
    x[i] = (i0 + i < F) ? begin[i0 + i] : 0u;
    tsum += x[i];
  }
  uint32_t inc = tsum;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t y = __shfl_up(inc, off, kWave);
    if (lane >= off) inc += y;
  }
  if (lane == kWave - 1) wave_tot[wv] = inc;
  __syncthreads();
  uint32_t wave_off = 0;
  for (int w = 0; w < wv; ++w) wave_off += wave_tot[w];
  uint32_t run = block_off + wave_off + (inc - tsum);
#pragma unroll
  for (int i = 0; i < kScanPerThread; ++i) {
    if (i0 + i < F) begin[i0 + i] = run;
    run += x[i];
  }
  if (blockIdx.x == gridDim.x - 1 && tid == kScanThreads - 1) begin[F] = run;
}

// map[begin[f] + rank[p]] = p: every pair goes to its group without any further atomic.
__global__ void csr_fill_kernel(const int64_t *__restrict__ indices, int64_t n_pairs, int64_t F,
                                const uint32_t *__restrict__ begin, const uint32_t *__restrict__ rank,
                                uint32_t *__restrict__ map) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < n_pairs;
       p += stride) {
    int64_t f = indices[p];
    if (static_cast<uint64_t>(f) >= static_cast<uint64_t>(F)) f = 0;
    map[begin[f] + rank[p]] = static_cast<uint32_t>(p);
  }
}

// Sort every group ascending so that the list does not depend on the order in which the
// count kernel's atomics happened to be served.  One wavefront per latent: groups of up to
// 64 pairs are rank-sorted in registers (pair ids are distinct); longer ones are appended
// to long_list for csr_sort_long_kernel.
__global__ __launch_bounds__(256) void csr_sort_short_kernel(const uint32_t *__restrict__ begin,
                                                             uint32_t *__restrict__ map, int64_t F,
                                                             uint32_t *__restrict__ long_count,
                                                             uint32_t *__restrict__ long_list) {
  const int lane = lane_id();
  const int64_t f = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block();
  if (f >= F) return;
  const uint32_t s0 = begin[f];
  const uint32_t n = begin[f + 1] - s0;
  if (n <= 1) return;
  if (n > static_cast<uint32_t>(kWave)) {
    if (lane == 0) long_list[atomicAdd(long_count, 1u)] = static_cast<uint32_t>(f);
    return;
  }
  const bool have = static_cast<uint32_t>(lane) < n;
  const uint32_t x = have ? map[s0 + lane] : 0xffffffffu;
  uint32_t rank = 0;
  for (uint32_t j = 0; j < n; ++j) {
    const uint32_t y = static_cast<uint32_t>(bcast_i32(static_cast<int>(x), static_cast<int>(j)));
    rank += (y < x) ? 1u : 0u;
  }
  if (have) map[s0 + rank] = x;  // every lane read its element before any lane writes
}

// Bitonic network in which every comparator points the same way (first sub-step of each merge
// mirrors, the rest are plain strides), so a length that is not a power of two is handled by
// skipping comparators whose partner lies beyond the end.  Run by one whole block on a[0..n).
template <typename Ptr>
__device__ __forceinline__ void block_bitonic_sort(Ptr a, uint32_t n) {
  uint32_t np2 = 1;
  while (np2 < n) np2 <<= 1;
  for (uint32_t k = 2; k <= np2; k <<= 1) {
    // mirrored sub-step: inside each block of k, position i pairs with (k-1-i)
    for (uint32_t t = threadIdx.x; t < np2 / 2; t += blockDim.x) {
      const uint32_t blk = t / (k / 2), i = t % (k / 2);
      const uint32_t lo = blk * k + i, hi = blk * k + (k - 1 - i);
      if (hi < n) {
        const uint32_t x = a[lo], y = a[hi];
        if (x > y) {
          a[lo] = y;
          a[hi] = x;
        }
      }
    }
    __syncthreads();
    for (uint32_t j = k / 4; j > 0; j >>= 1) {
      for (uint32_t t = threadIdx.x; t < np2 / 2; t += blockDim.x) {
        const uint32_t lo = (t / j) * (2 * j) + (t % j), hi = lo + j;
        if (hi < n) {
          const uint32_t x = a[lo], y = a[hi];
          if (x > y) {
            a[lo] = y;
            a[hi] = x;
          }
        }
      }
      __syncthreads();
    }
  }
}

// Long groups (more than 64 pairs): one block per group, striding over the list.  Groups of up
// to kSortLdsElems pairs are sorted in LDS, longer ones in place in global memory.  With `slot`
// given, the positions of the group's pairs are written there as well.
// A latent that is in a large share of the rows (thousands of pairs) is not compared at all: a
// pair id is row * K + step, so counting the group's pairs per row and scanning the counts places
// every pair (a counting sort over the rows, O(pairs + rows) instead of the network's
// O(pairs log^2 pairs)); pairs of the same row, if a row holds the latent more than once, are
// ranked among themselves afterwards.  Taken when the rows fit the LDS counters and the network
// would cost several times more.
constexpr uint32_t kSortLdsElems = 8192;
constexpr uint32_t kSortRowsMax = 8192;  // rows (B) the counting sort has LDS counters for
// buf + rowcnt + wave_tot come to 65 600 bytes of LDS per block: more than the 64 KiB of earlier gfx9
// parts, within the 160 KiB a workgroup may use on gfx950 (the only target of this library)
static_assert((kSortLdsElems + kSortRowsMax + 1024 / kWave) * 4 <= 160 * 1024, "LDS of csr_sort_long_kernel");
__global__ __launch_bounds__(1024) void csr_sort_long_kernel(const uint32_t *__restrict__ begin,
                                                            uint32_t *__restrict__ map,
                                                            const uint32_t *__restrict__ long_count,
                                                            const uint32_t *__restrict__ long_list,
                                                            uint32_t *__restrict__ slot, uint32_t n_rows,
                                                            uint32_t K) {
  __shared__ uint32_t buf[kSortLdsElems];  // the group (network), or its pairs grouped by row (counting sort)
  __shared__ uint32_t rowcnt[kSortRowsMax];
  __shared__ uint32_t wave_tot[1024 / kWave];
  const uint32_t n_long = *long_count;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid >> 6;
  for (uint32_t w = blockIdx.x; w < n_long; w += gridDim.x) {
    const uint32_t f = long_list[w];
    const uint32_t base = begin[f];
    uint32_t *a = map + base;
    const uint32_t n = begin[f + 1] - base;
    if (n <= kSortLdsElems) {
      uint32_t lg = 1;
      while ((1u << lg) < n) ++lg;
      // network: about n/2 * lg*(lg+1)/2 comparators; counting: a few passes over n pairs and n_rows counters
      const bool by_rows = n_rows <= kSortRowsMax && K > 0 &&
                           static_cast<uint64_t>(n) * lg * (lg + 1) > 4ull * (static_cast<uint64_t>(n) + n_rows);
      if (by_rows) {  // uniform over the block
        for (uint32_t r = tid; r < n_rows; r += blockDim.x) rowcnt[r] = 0u;
        __syncthreads();
        for (uint32_t i = tid; i < n; i += blockDim.x) atomicAdd(&rowcnt[a[i] / K], 1u);
        __syncthreads();
        // exclusive scan of rowcnt[0..n_rows): every thread owns eight consecutive counters
        {
          constexpr uint32_t PER = kSortRowsMax / 1024;
          uint32_t x[PER], tsum = 0;
#pragma unroll
          for (uint32_t i = 0; i < PER; ++i) {
            const uint32_t r = static_cast<uint32_t>(tid) * PER + i;
            x[i] = r < n_rows ? rowcnt[r] : 0u;
            tsum += x[i];
          }
          uint32_t inc = tsum;
#pragma unroll
          for (int off = 1; off < kWave; off <<= 1) {
            const uint32_t y = __shfl_up(inc, off, kWave);
            if (lane >= off) inc += y;
          }
          if (lane == kWave - 1) wave_tot[wv] = inc;
          __syncthreads();
          uint32_t run = inc - tsum;
          for (int q = 0; q < wv; ++q) run += wave_tot[q];
#pragma unroll
          for (uint32_t i = 0; i < PER; ++i) {
            const uint32_t r = static_cast<uint32_t>(tid) * PER + i;
            if (r < n_rows) rowcnt[r] = run;
            run += x[i];
          }
          __syncthreads();
        }
        // placement by row; the atomics leave rowcnt[r] at the end of row r's pairs
        for (uint32_t i = tid; i < n; i += blockDim.x) {
          const uint32_t id = a[i];
          buf[atomicAdd(&rowcnt[id / K], 1u)] = id;
        }
        __syncthreads();
        // pairs of one row are in the order of the atomics: rank them among themselves on the way out
        for (uint32_t i = tid; i < n; i += blockDim.x) {
          const uint32_t id = buf[i], r = id / K;
          const uint32_t s0 = r ? rowcnt[r - 1] : 0u, s1 = rowcnt[r];
          uint32_t rank = 0;
          for (uint32_t j = s0; j < s1; ++j) rank += (buf[j] < id) ? 1u : 0u;
          a[s0 + rank] = id;
          if (slot) slot[id] = base + s0 + rank;
        }
        __syncthreads();
        continue;
      }
      for (uint32_t i = tid; i < n; i += blockDim.x) buf[i] = a[i];
      __syncthreads();
      block_bitonic_sort(buf, n);
      for (uint32_t i = tid; i < n; i += blockDim.x) {
        a[i] = buf[i];
        if (slot) slot[buf[i]] = base + i;
      }
      __syncthreads();
    } else {
      block_bitonic_sort(a, n);  // ends with a barrier
      if (slot)
        for (uint32_t i = tid; i < n; i += blockDim.x) slot[a[i]] = base + i;
    }
  }
}

// ---------------------------------------------------------------------------------
// Bucketed construction (the default): the latents are cut into buckets of 2^shift consecutive
// ids, sized so that a bucket holds a few thousand pairs.  csr_bucket_count_kernel counts, for
// every chunk of consecutive pairs, how many fall into each bucket (LDS atomics only); an
// exclusive scan of that table (bucket-major) gives every (bucket, chunk) its place;
// csr_bucket_scatter_kernel moves (latent within bucket, pair id) there; csr_bucket_sort_kernel
// then finishes one bucket per block inside the LDS: per-latent counts -> begin[], placement,
// and a rank sort of every group, so that map[] comes out ascending inside each latent and
// slot[] (its inverse) is written on the way.  No atomics reach memory except one per latent
// with more than 64 pairs (appended to long_list; csr_sort_long_kernel sorts those groups).
// ---------------------------------------------------------------------------------
constexpr int kBucketThreads = 256;
constexpr int kBucketMaxBuckets = 8192;  // LDS counters of the count / scatter kernels
constexpr int kSortThreads = 1024;
constexpr int kSortMaxLatents = 4096;    // latents per bucket (2^shift) at most
constexpr int kSortCap = 8192;           // pairs of a bucket that are sorted inside the LDS

__global__ __launch_bounds__(kBucketThreads) void csr_bucket_count_kernel(
    const int64_t *__restrict__ indices, int64_t n_pairs, int64_t F, int shift, uint32_t n_buckets,
    int64_t chunk, uint32_t n_chunks, uint32_t *__restrict__ table, uint32_t *__restrict__ long_count,
    int *status_flag) {
  __shared__ uint32_t hist[kBucketMaxBuckets];
  for (uint32_t q = threadIdx.x; q < n_buckets; q += kBucketThreads) hist[q] = 0u;
  if (blockIdx.x == 0 && threadIdx.x == 0) *long_count = 0u;
  __syncthreads();
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * chunk;
  const int64_t p1 = (p0 + chunk) < n_pairs ? (p0 + chunk) : n_pairs;
  for (int64_t p = p0 + threadIdx.x; p < p1; p += kBucketThreads) {
    int64_t f = indices[p];
    if (static_cast<uint64_t>(f) >= static_cast<uint64_t>(F)) {
      if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
      f = 0;
    }
    atomicAdd(&hist[f >> shift], 1u);
  }
  __syncthreads();
  for (uint32_t q = threadIdx.x; q < n_buckets; q += kBucketThreads)
    table[static_cast<size_t>(q) * n_chunks + blockIdx.x] = hist[q];
}

// tmp[place] = (latent within its bucket) << 32 | pair id; inside one (bucket, chunk) cell the
// order is that of the LDS atomics, which the sort kernel removes.
__global__ __launch_bounds__(kBucketThreads) void csr_bucket_scatter_kernel(
    const int64_t *__restrict__ indices, int64_t n_pairs, int64_t F, int shift, uint32_t n_buckets,
    int64_t chunk, uint32_t n_chunks, const uint32_t *__restrict__ table, uint64_t *__restrict__ tmp) {
  __shared__ uint32_t cursor[kBucketMaxBuckets];
  for (uint32_t q = threadIdx.x; q < n_buckets; q += kBucketThreads)
    cursor[q] = table[static_cast<size_t>(q) * n_chunks + blockIdx.x];
  __syncthreads();
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * chunk;
  const int64_t p1 = (p0 + chunk) < n_pairs ? (p0 + chunk) : n_pairs;
  const int64_t mask = (static_cast<int64_t>(1) << shift) - 1;
  for (int64_t p = p0 + threadIdx.x; p < p1; p += kBucketThreads) {
    int64_t f = indices[p];
    if (static_cast<uint64_t>(f) >= static_cast<uint64_t>(F)) f = 0;
    const uint32_t place = atomicAdd(&cursor[f >> shift], 1u);
    tmp[place] = (static_cast<uint64_t>(f & mask) << 32) | static_cast<uint64_t>(static_cast<uint32_t>(p));
  }
}

// Exclusive scan of a[0..n) in LDS by a whole block of kSortThreads threads (n <= 8 per thread);
// every thread owns 8 consecutive entries.  Ends with a barrier.
__device__ __forceinline__ void block_exclusive_scan_lds(uint32_t *a, uint32_t n, uint32_t *wave_tot) {
  constexpr int PER = kSortMaxLatents / kSortThreads;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid >> 6;
  uint32_t x[PER];
  uint32_t tsum = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const uint32_t k = static_cast<uint32_t>(tid) * PER + i;
    x[i] = (k < n) ? a[k] : 0u;
    tsum += x[i];
  }
  uint32_t inc = tsum;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t y = __shfl_up(inc, off, kWave);
    if (lane >= off) inc += y;
  }
  if (lane == kWave - 1) wave_tot[wv] = inc;
  __syncthreads();
  uint32_t run = inc - tsum;
  for (int w = 0; w < wv; ++w) run += wave_tot[w];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const uint32_t k = static_cast<uint32_t>(tid) * PER + i;
    if (k < n) a[k] = run;
    run += x[i];
  }
  __syncthreads();
}

// One block per bucket.  `map` and `slot` are written here and, in the large-bucket path, map
// is read back by other wavefronts of the same block after a barrier.  cnt[] holds, in turn, the
// per-latent counts, the first position of every latent (after the scan) and the end of every
// latent's group (after the placement, whose atomics advance it).
__global__ __launch_bounds__(kSortThreads) void csr_bucket_sort_kernel(
    const uint64_t *__restrict__ tmp, const uint32_t *__restrict__ table, uint32_t n_chunks, int shift,
    int64_t F, uint32_t *begin, uint32_t *map, uint32_t *slot, uint32_t *long_count, uint32_t *long_list) {
  __shared__ uint32_t cnt[kSortMaxLatents + 1];
  __shared__ uint32_t ids[kSortCap];  // pair ids grouped by latent
  __shared__ uint32_t wave_tot[kSortThreads / kWave];
  __shared__ uint32_t any_long;
  const int tid = threadIdx.x;
  const uint32_t q = blockIdx.x;
  const uint32_t lpb = 1u << shift;
  const int64_t f0 = static_cast<int64_t>(q) << shift;
  const uint32_t nlat = (F - f0) < static_cast<int64_t>(lpb) ? static_cast<uint32_t>(F - f0) : lpb;
  const uint32_t base = table[static_cast<size_t>(q) * n_chunks];
  const uint32_t end = table[static_cast<size_t>(q + 1) * n_chunks];  // the scan's total after the last bucket
  const uint32_t n = end - base;
  const bool in_lds = n <= static_cast<uint32_t>(kSortCap);
  for (uint32_t k = tid; k <= lpb; k += kSortThreads) cnt[k] = 0u;
  if (tid == 0) any_long = 0u;
  __syncthreads();
  for (uint64_t i = tid; i < n; i += kSortThreads) atomicAdd(&cnt[static_cast<uint32_t>(tmp[base + i] >> 32)], 1u);
  __syncthreads();
  block_exclusive_scan_lds(cnt, lpb, wave_tot);
  if (tid == 0) cnt[lpb] = n;
  __syncthreads();
  for (uint32_t k = tid; k < nlat; k += kSortThreads) {
    begin[f0 + k] = base + cnt[k];
    if (cnt[k + 1] - cnt[k] > static_cast<uint32_t>(kWave)) {
      long_list[atomicAdd(long_count, 1u)] = static_cast<uint32_t>(f0 + k);
      any_long = 1u;
    }
  }
  if (q == gridDim.x - 1 && tid == 0) begin[F] = end;
  __syncthreads();
  // placement: inside a group the order is that of the atomics
  for (uint64_t i = tid; i < n; i += kSortThreads) {
    const uint64_t kv = tmp[base + i];
    const uint32_t place = atomicAdd(&cnt[static_cast<uint32_t>(kv >> 32)], 1u);
    if (in_lds)
      ids[place] = static_cast<uint32_t>(kv);
    else
      map[base + place] = static_cast<uint32_t>(kv);
  }
  __syncthreads();  // also makes the block's own writes to map visible to all its wavefronts
  // from here: the group of latent k is [k ? cnt[k-1] : 0, cnt[k])

  if (in_lds) {
    // every pair finds its rank inside its group by counting the smaller ids
    for (uint64_t i = tid; i < n; i += kSortThreads) {
      const uint64_t kv = tmp[base + i];
      const uint32_t key = static_cast<uint32_t>(kv >> 32), id = static_cast<uint32_t>(kv);
      const uint32_t s0 = key ? cnt[key - 1] : 0u, len = cnt[key] - s0;
      if (len > static_cast<uint32_t>(kWave)) continue;
      uint32_t rank = 0;
      for (uint32_t j = 0; j < len; ++j) rank += (ids[s0 + j] < id) ? 1u : 0u;
      map[base + s0 + rank] = id;
      if (slot) slot[id] = base + s0 + rank;
    }
    if (any_long) {
      // groups of more than 64 pairs go out as they are: csr_sort_long_kernel orders them and
      // writes their slots.  The latent of position j is found by bisection over the group ends.
      for (uint32_t j = tid; j < n; j += kSortThreads) {  // n <= kSortCap here
        uint32_t lo = 0, hi = lpb - 1;  // smallest k with cnt[k] > j
        while (lo < hi) {
          const uint32_t mid = (lo + hi) >> 1;
          if (cnt[mid] > j)
            hi = mid;
          else
            lo = mid + 1;
        }
        const uint32_t s0 = lo ? cnt[lo - 1] : 0u;
        if (cnt[lo] - s0 > static_cast<uint32_t>(kWave)) map[base + j] = ids[j];
      }
    }
    return;
  }

  // A bucket too large for the LDS (hot latents): the groups were placed in map; one wavefront
  // per latent rank-sorts its group there.
  const int lane = tid & (kWave - 1);
  for (uint32_t k = tid >> 6; k < nlat; k += kSortThreads / kWave) {
    const uint32_t s0 = k ? cnt[k - 1] : 0u, len = cnt[k] - s0;
    if (len == 0 || len > static_cast<uint32_t>(kWave)) continue;
    const bool have = static_cast<uint32_t>(lane) < len;
    const uint32_t x = have ? map[base + s0 + lane] : 0xffffffffu;
    uint32_t rank = 0;
    for (uint32_t j = 0; j < len; ++j) {
      const uint32_t y = static_cast<uint32_t>(bcast_i32(static_cast<int>(x), static_cast<int>(j)));
      rank += (y < x) ? 1u : 0u;
    }
    if (have) {
      map[base + s0 + rank] = x;  // every lane read its element before any lane writes
      if (slot) slot[x] = base + s0 + rank;
    }
  }
}

__global__ void copy_u32_kernel(uint32_t *__restrict__ dst, const uint32_t *__restrict__ src, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = src[i];
}

// slot[map[s]] = s: position of every pair in the latent-major list.
__global__ void csr_inverse_kernel(const uint32_t *__restrict__ map, int64_t n_pairs,
                                   uint32_t *__restrict__ slot) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t s = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; s < n_pairs; s += stride)
    slot[map[s]] = static_cast<uint32_t>(s);
}

// Column sums of a row-major [rows, ld] fp32 matrix over `cols` columns, in two stages with a
// fixed summation order (deterministic): stage 1 sums kColsumRows rows per block into
// partial[chunk, cols]; stage 2 adds the chunks in order and writes
// out[c] = scale * sum  with  scale = coef * (grad_out ? grad_out[0] : 1).
constexpr int kColsumRows = 64;

// stage 1 for column c and row chunk `chunk`
__device__ __forceinline__ void colsum_partial_one(const float *__restrict__ x, int64_t rows, int64_t ld, int cols,
                                                   float *__restrict__ partial, int c, int64_t chunk) {
  if (c >= cols) return;
  const int64_t r0 = chunk * kColsumRows;
  if (r0 >= rows) return;
  const int64_t r1 = (r0 + kColsumRows) < rows ? (r0 + kColsumRows) : rows;
  float s = 0.f;
  int64_t r = r0;
  for (; r + 8 <= r1; r += 8) {  // eight independent loads in flight
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = x[(r + u) * ld + c];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; r < r1; ++r) s += x[r * ld + c];
  partial[chunk * cols + c] = s;
}

__global__ __launch_bounds__(256) void colsum_partial_kernel(const float *__restrict__ x, int64_t rows,
                                                             int64_t ld, int cols,
                                                             float *__restrict__ partial) {
  colsum_partial_one(x, rows, ld, cols, partial, static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x),
                     static_cast<int64_t>(blockIdx.y));
}

__global__ __launch_bounds__(256) void colsum_final_kernel(const float *__restrict__ partial,
                                                           int n_chunks, int cols,
                                                           const float *__restrict__ grad_out, float coef,
                                                           float *__restrict__ out) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  float s = 0.f;
  int k = 0;
  for (; k + 8 <= n_chunks; k += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = partial[static_cast<int64_t>(k + u) * cols + c];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; k < n_chunks; ++k) s += partial[static_cast<int64_t>(k) * cols + c];
  out[c] = s * coef * (grad_out ? grad_out[0] : 1.f);
}

__global__ void fill_f32_kernel(float *__restrict__ p, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t n4 = n >> 2;
  float4 *p4 = reinterpret_cast<float4 *>(p);
  const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride)
    p4[i] = z;
  for (int64_t i = (n4 << 2) + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride)
    p[i] = 0.f;
}

// dst = GT(src * scale[0]) (scale null: a plain cast)
template <typename GT>
__global__ void cast_from_f32_kernel(void *__restrict__ dst, const float *__restrict__ src,
                                     int64_t n, const float *__restrict__ scale = nullptr) {
  const float g = scale ? scale[0] : 1.0f;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t n4 = n >> 2;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride) {
    float x[4];
    load_vec<float, 4>(src, i * 4, x);
#pragma unroll
    for (int k = 0; k < 4; ++k) x[k] *= g;
    store_vec<GT, 4>(dst, i * 4, x);
  }
  for (int64_t i = (n4 << 2) + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    float x[1] = {src[i] * g};
    store_vec<GT, 1>(dst, i, x);
  }
}

}  // namespace flexsae
