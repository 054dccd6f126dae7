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
// to kSortLdsElems pairs are sorted in LDS, longer ones in place in global memory.
constexpr uint32_t kSortLdsElems = 8192;
__global__ __launch_bounds__(256) void csr_sort_long_kernel(const uint32_t *__restrict__ begin,
                                                            uint32_t *__restrict__ map,
                                                            const uint32_t *__restrict__ long_count,
                                                            const uint32_t *__restrict__ long_list) {
  __shared__ uint32_t buf[kSortLdsElems];
  const uint32_t n_long = *long_count;
  for (uint32_t w = blockIdx.x; w < n_long; w += gridDim.x) {
    const uint32_t f = long_list[w];
    uint32_t *a = map + begin[f];
    const uint32_t n = begin[f + 1] - begin[f];
    if (n <= kSortLdsElems) {
      for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) buf[i] = a[i];
      __syncthreads();
      block_bitonic_sort(buf, n);
      for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) a[i] = buf[i];
      __syncthreads();
    } else {
      block_bitonic_sort(a, n);
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

__global__ __launch_bounds__(256) void colsum_partial_kernel(const float *__restrict__ x, int64_t rows,
                                                             int64_t ld, int cols,
                                                             float *__restrict__ partial) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * kColsumRows;
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
  partial[static_cast<int64_t>(blockIdx.y) * cols + c] = s;
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

template <typename GT>
__global__ void cast_from_f32_kernel(void *__restrict__ dst, const float *__restrict__ src,
                                     int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t n4 = n >> 2;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride) {
    float x[4];
    load_vec<float, 4>(src, i * 4, x);
    store_vec<GT, 4>(dst, i * 4, x);
  }
  for (int64_t i = (n4 << 2) + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    float x[1] = {src[i]};
    store_vec<GT, 1>(dst, i, x);
  }
}

}  // namespace flexsae
