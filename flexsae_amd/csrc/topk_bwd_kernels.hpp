// TopK backward: latent-major segment reduction producing dW (written once, no atomics) and
// dvals, from the pair list and the forward residual.
#pragma once

#include "common.hpp"
#include "segment_kernels.hpp"

namespace flexsae {

// For the slots [s_begin, s_end) of latent f (W row tile in w[]), over the lane's VEC columns:
//   acc      += vals[p] * scale * resid[b_p]          (dW contribution)
//   dvals[p] += scale * <resid[b_p], W[f]>            (one wave reduction per slot, then an atomic)
// resid rows are read through the caches (the [B,D] matrix is small next to W).
template <int VEC, int U>
__device__ __forceinline__ void topk_accumulate_slots(
    const uint32_t *__restrict__ map, const void *__restrict__ vals, int vals_dtype,
    const float *__restrict__ resid, float scale, float *__restrict__ dvals, const float (&w)[VEC],
    uint32_t s_begin, uint32_t s_end, int K, int D, int dsafe, float (&acc)[VEC]) {
  const int lane = lane_id();
  for (uint32_t s = s_begin; s < s_end; s += kWave) {
    const uint32_t slot = s + lane;
    uint32_t p = 0;
    float v = 0.f;
    if (slot < s_end) {
      p = map[slot];
      v = load_scalar(vals, vals_dtype, p) * scale;
    }
    const int my_b = static_cast<int>(p / static_cast<uint32_t>(K));
    const int n = (s_end - s) < static_cast<uint32_t>(kWave) ? static_cast<int>(s_end - s) : kWave;
    float my_dot = 0.f;

    auto step = [&](int j, const float(&g)[VEC]) {
      const float vj = bcast_f32(v, j);
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        acc[i] = fmaf(vj, g[i], acc[i]);
        dot = fmaf(g[i], w[i], dot);
      }
      dot = wave_sum_bcast(dot);
      if (lane == j) my_dot = dot;
    };

    // U gathers in flight; a group reaching past the end re-reads the last row (a cache hit)
    for (int j = 0; j < n; j += U) {
      float g[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int jj = (j + u) < n ? (j + u) : (n - 1);
        const int64_t brow = bcast_i32(my_b, jj);
        load_vec<float, VEC>(resid, brow * D + dsafe, g[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u < n) step(j + u, g[u]);  // uniform
    }
    if (slot < s_end) unsafeAtomicAdd(dvals + p, my_dot * scale);
  }
}

// TopK backward of one slice.  scale = grad_out * 2/(B*D).
// Blocks [0, n_long_blocks): long latents, one wavefront per (64-pair chunk, tile): adds its
// dvals, leaves its dW contribution in partial[chunk, slice column] (fp32) for
// seg_reduce_long_finalize_kernel (next launch).  They come first so hot latents start at once.
// Remaining blocks: one wavefront per (tile of the slice, latent f), tile-major, so that at any
// moment the waves in flight share one B x tile slice of resid (L2-sized).  tile = 64*VEC
// columns, lane l owning VEC consecutive columns.  dW[f, tile] is written exactly once, in the
// gradient's final dtype; latents without pairs get zeros; latents with more than kSegChunk
// pairs are skipped here.
template <typename WT, typename GT, int VEC, int U>
__global__ __launch_bounds__(256) void topk_bwd_kernel(
    const uint32_t *__restrict__ begin, const uint32_t *__restrict__ map,
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const float *__restrict__ resid,
    const float *__restrict__ grad_out, float coef, void *__restrict__ dW,
    float *__restrict__ dvals, float *__restrict__ partial, int64_t n_items, unsigned n_long_blocks,
    int tps, int col0, int slice_w, int64_t F, int K, int D) {
  const int lane = lane_id();
  const float scale = coef * grad_out[0];
  if (blockIdx.x >= n_long_blocks) {
    const int64_t item =
        static_cast<int64_t>(blockIdx.x - n_long_blocks) * (blockDim.x >> 6) + wave_in_block();
    if (item >= n_items) return;  // uniform per wavefront
    const int t = static_cast<int>(item / F);
    const int64_t f = item - static_cast<int64_t>(t) * F;
    const uint32_t s_begin = begin[f];
    const uint32_t s_end = begin[f + 1];
    if (s_end - s_begin > static_cast<uint32_t>(kSegChunk)) return;
    const int d0 = col0 + t * (kWave * VEC) + lane * VEC;
    const bool active = d0 < D;
    const int dsafe = active ? d0 : 0;
    float w[VEC], acc[VEC];
    load_vec<WT, VEC>(weight, f * D + dsafe, w);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      acc[i] = 0.f;
      if (!active) w[i] = 0.f;
    }
    topk_accumulate_slots<VEC, U>(map, vals, vals_dtype, resid, scale, dvals, w, s_begin, s_end, K, D,
                                  dsafe, acc);
    if (active) store_vec<GT, VEC>(dW, f * D + d0, acc);
    return;
  }
  const uint32_t n_long = *long_count;
  if (n_long == 0) return;
  const uint32_t n_chunks = chunk_begin[n_long];
  const int64_t total = static_cast<int64_t>(n_chunks) * tps;
  const int64_t n_waves = static_cast<int64_t>(n_long_blocks) * (blockDim.x >> 6);
  for (int64_t wk = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block(); wk < total;
       wk += n_waves) {
    // tile-major over the work list as well
    const int t = static_cast<int>(wk / n_chunks);
    const uint32_t chunk = static_cast<uint32_t>(wk - static_cast<int64_t>(t) * n_chunks);
    const LongChunk c = seg_decode_chunk(begin, long_list, chunk_begin, n_long, chunk);
    const int pc = t * (kWave * VEC) + lane * VEC;
    const int d0 = col0 + pc;
    const bool active = d0 < D;
    const int dsafe = active ? d0 : 0;
    float w[VEC], acc[VEC];
    load_vec<WT, VEC>(weight, c.f * D + dsafe, w);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      acc[i] = 0.f;
      if (!active) w[i] = 0.f;
    }
    topk_accumulate_slots<VEC, U>(map, vals, vals_dtype, resid, scale, dvals, w, c.s0, c.s1, K, D, dsafe,
                                  acc);
    store_vec<float, VEC>(partial, static_cast<int64_t>(chunk) * slice_w + pc, acc);
  }
}

}  // namespace flexsae
