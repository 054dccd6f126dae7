// Forward kernels: fused embedding-bag + bias - target + squared error, for the TopK loss
// (one squared error at the end of the row) and the HierarchicalTopK loss (one after
// every prefix), without ever materialising the [B,K,D] reconstruction.
#pragma once

#include "common.hpp"

namespace flexsae {

// Work decomposition: one wavefront per (row b, D-tile) item.  A tile is 64*VEC
// consecutive columns, lane l owning columns [l*VEC, (l+1)*VEC) of the tile, so one
// gathered row piece is a single vector load per lane and 64*VEC*sizeof(W) contiguous
// bytes per wavefront.  The row's indices/vals are fetched 64 at a time with one
// coalesced load (lane j holds step k0+j) and handed out with v_readlane, which puts
// the row number in a scalar register: the gather address is scalar-base + lane offset.
// U independent gathers are issued before the first one is consumed.
//
// Per item the wavefront writes resid[b, tile] = r_{b,K-1} - target_b (fp32) and one
// fp32 partial sum of squares into partial[item]; loss_finalize_kernel adds the
// partials in a fixed order, so the loss is bit-reproducible from run to run.
template <typename WT, int VEC, bool HIER, int U>
__global__ __launch_bounds__(256) void sae_fwd_kernel(
    const int64_t *__restrict__ indices, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const void *__restrict__ bias, int bias_dtype,
    const void *__restrict__ target, int target_dtype, float *__restrict__ resid,
    float *__restrict__ partial, int *status_flag, int64_t n_items, int ntiles, int K, int64_t F,
    int D) {
  const int lane = lane_id();
  const int64_t item = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block();
  if (item >= n_items) return;  // uniform per wavefront
  const int64_t b = item / ntiles;
  const int tile = static_cast<int>(item - b * ntiles);
  const int d0 = tile * (kWave * VEC) + lane * VEC;
  const bool active = d0 < D;  // D % VEC == 0 is checked on the host
  const int dsafe = active ? d0 : 0;

  float r[VEC], t[VEC], acc[VEC];
  load_vec_dyn<WT, VEC>(bias, bias_dtype, dsafe, r);
  load_vec_dyn<WT, VEC>(target, target_dtype, b * D + dsafe, t);
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = 0.f;

  const int64_t pair0 = b * K;
  for (int k0 = 0; k0 < K; k0 += kWave) {
    const int kk = k0 + lane;
    int64_t my_idx = 0;
    float my_val = 0.f;
    if (kk < K) {
      my_idx = indices[pair0 + kk];
      my_val = load_scalar(vals, vals_dtype, pair0 + kk);
    }
    if (static_cast<uint64_t>(my_idx) >= static_cast<uint64_t>(F)) {
      if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
      my_idx = 0;
      my_val = 0.f;
    }
    const int my_row = static_cast<int>(my_idx);
    const int n = (K - k0) < kWave ? (K - k0) : kWave;  // uniform

    auto consume = [&](const float(&w)[VEC], float v) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        r[i] = fmaf(w[i], v, r[i]);
        if constexpr (HIER) {
          const float diff = r[i] - t[i];
          acc[i] = fmaf(diff, diff, acc[i]);
        }
      }
    };

    int j = 0;
    for (; j + U <= n; j += U) {
      float w[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t row = bcast_i32(my_row, j + u);
        load_vec<WT, VEC>(weight, row * D + dsafe, w[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) consume(w[u], bcast_f32(my_val, j + u));
    }
    for (; j < n; ++j) {
      float w[VEC];
      const int64_t row = bcast_i32(my_row, j);
      load_vec<WT, VEC>(weight, row * D + dsafe, w);
      consume(w, bcast_f32(my_val, j));
    }
  }

  float lsum = 0.f;
  float e[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    e[i] = r[i] - t[i];
    if constexpr (HIER) {
      lsum += acc[i];
    } else {
      lsum = fmaf(e[i], e[i], lsum);
    }
  }
  if (active) {
    store_vec<float, VEC>(resid, b * D + d0, e);
  } else {
    lsum = 0.f;
  }
  lsum = wave_sum_lane63(lsum);
  if (lane == kWave - 1) partial[item] = lsum;
}

// loss[0] = inv_count * sum(partial[0..n)), one block, fixed summation order, double
// accumulation (n is B * ntiles, up to a few million).
// (the body, for a block of 1024 threads; `red` is 1024 doubles of LDS)
__device__ __forceinline__ void loss_finalize_block(const float *__restrict__ partial, int64_t n, double inv_count,
                                                    float *__restrict__ loss, double *red) {
  double s = 0.0;
  int64_t i = threadIdx.x;
  for (; i + 7 * 1024 < n; i += 8 * 1024) {  // eight independent loads in flight
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = partial[i + u * 1024];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += static_cast<double>(x[u]);
  }
  for (; i < n; i += 1024) s += static_cast<double>(partial[i]);
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if (static_cast<int>(threadIdx.x) < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) loss[0] = static_cast<float>(red[0] * inv_count);
}

__global__ __launch_bounds__(1024) void loss_finalize_kernel(const float *__restrict__ partial,
                                                             int64_t n, double inv_count,
                                                             float *__restrict__ loss) {
  __shared__ double red[1024];
  loss_finalize_block(partial, n, inv_count, loss, red);
}

}  // namespace flexsae
