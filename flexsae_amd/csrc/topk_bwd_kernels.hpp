// TopK backward: latent-major segment reduction producing dW (written once, no atomics) and
// dvals, from the pair list and the forward residual.
#pragma once

#include "common.hpp"
#include "segment_kernels.hpp"

#ifndef FLEXSAE_TOPK_ONE_GROUP
#define FLEXSAE_TOPK_ONE_GROUP 1
#endif
// rows of a group of eight that share one uniform "are there rows left" test
#ifndef FLEXSAE_TOPK_ROWS_PER_TEST
#define FLEXSAE_TOPK_ROWS_PER_TEST 2
#endif
#ifndef FLEXSAE_TOPK_NT
#define FLEXSAE_TOPK_NT true
#endif

namespace flexsae {

// For the slots [s_begin, s_end) of latent f (W row tile in w[]), over the lane's VEC columns:
//   acc      += vals[p] * scale * resid[b_p]          (dW contribution)
//   dv_tile[slot] = scale * <resid[b_p], W[f]>        (this tile's share of dvals[p]; the lane that
//                                                      owns the slot stores it, so stores coalesce;
//                                                      topk_dvals_finalize_kernel adds the tiles up)
// resid rows (element type RT) are read through the caches: the waves in flight share one
// B x tile slice of the [B,D] matrix, which has to stay in the 4 MB L2 of every XCD.
template <typename RT, int VEC>
__device__ __forceinline__ void topk_accumulate_slots(
    const vec_t<uint32_t, 2> *__restrict__ slot_bv,
    const void *__restrict__ resid, float scale, float *__restrict__ dv_tile, const float (&w)[VEC],
    uint32_t s_begin, uint32_t s_end, int D, int dsafe, float (&acc)[VEC]) {
  using S = typename Traits<RT>::store_t;
  const int lane = lane_id();
  // row address = scalar base of the row + the lane's fixed byte offset
  const uint32_t lane_off = static_cast<uint32_t>(dsafe) * sizeof(S);
  const size_t row_bytes = static_cast<size_t>(D) * sizeof(S);
  for (uint32_t s = s_begin; s < s_end; s += kWave) {
    const uint32_t slot = s + lane;
    int my_b = 0;
    float v = 0.f;
    if (slot < s_end) {  // the pair's (batch row, val) record; the val of an out-of-range index is zero there
      const vec_t<uint32_t, 2> bv = slot_bv[slot];
      my_b = static_cast<int>(bv[0]);
      v = __uint_as_float(bv[1]) * scale;
    }
    const int n = (s_end - s) < static_cast<uint32_t>(kWave) ? static_cast<int>(s_end - s) : kWave;
    float my_dot = 0.f;
    // eight gathers in flight; a group reaching past the end re-reads the last row (a cache hit);
    // the eight dot products of a group share one transposed wave reduction
    for (int j = 0; j < n; j += 8) {
      raw_vec_t<RT, VEC> buf[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int jj = (j + u) < n ? (j + u) : (n - 1);
        const char *row = static_cast<const char *>(resid) +
                          static_cast<size_t>(static_cast<uint32_t>(bcast_i32(my_b, jj))) * row_bytes;
        buf[u] = *reinterpret_cast<const raw_vec_t<RT, VEC> *>(row + lane_off);
      }
      float dots[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        dots[u] = 0.f;
        if (j + u < n) {  // uniform
          float x[VEC];
          unpack_raw<RT, VEC>(buf[u], x);
          const float vj = bcast_f32(v, j + u);
          float dot = 0.f;
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            acc[i] = fmaf(vj, x[i], acc[i]);
            dot = fmaf(x[i], w[i], dot);
          }
          dots[u] = dot;
        }
      }
      const float tot = wave_sum8_transposed(dots);  // lane L: total of slot s + j + (L & 7)
      if ((lane >> 3) == (j >> 3)) my_dot = tot;
    }
    if (slot < s_end) dv_tile[slot] = my_dot * scale;
  }
}

// One short latent (1 to kSegChunk pairs) for one tile: the pair records of the latent are one
// contiguous load, the residual rows are gathered through a buffer descriptor (no vector ALU work
// for addresses) eight at a time (with the next eight already requested when registers allow),
// and each group of eight shares one transposed wave reduction for the dvals dot products.  Inside a
// group, rows are requested and consumed two at a time under one uniform test, so a latent with
// nine pairs costs ten rows, not sixteen (a test per row costs more than it saves; the odd slot
// past the end re-reads the last row, a cache hit, with a val of zero).  With bf16 weights and a
// bf16 residual copy the products run on packed pairs (dot2) without unpacking.
template <typename WT, typename GT, typename RT, int VEC>
__device__ __forceinline__ void topk_short_latent(
    const vec_t<uint32_t, 2> *__restrict__ slot_bv, const void *__restrict__ weight, int vals_dtype,
    const GatherSource &rows_src, uint32_t row_stride, float scale, void *__restrict__ dW,
    float *__restrict__ dv_tile, int64_t f, uint32_t b0, int n, int d0, int D) {
  using S = typename Traits<RT>::store_t;
  const int lane = lane_id();
  const bool active = d0 < D;
  const uint32_t lane_off = static_cast<uint32_t>(active ? d0 : 0) * sizeof(S);
  constexpr bool kDot2 = Traits<WT>::dtype == FLEXSAE_BF16 && Traits<RT>::dtype == FLEXSAE_BF16 && VEC % 2 == 0;
  const bool late_scale = kDot2 && vals_dtype == FLEXSAE_BF16;  // vals enter the dot2 as they are

  const raw_vec_t<WT, VEC> wraw = load_raw<WT, VEC, FLEXSAE_TOPK_NT>(weight, f * D + (active ? d0 : 0));
  // lanes past the end hold row 0 and a val of zero
  const vec_t<uint32_t, 2> bv = lane < n ? __builtin_nontemporal_load(slot_bv + b0 + lane) : vec_t<uint32_t, 2>{0u, 0u};
  const int my_b = static_cast<int>(bv[0]);
  const uint32_t vbits = bv[1];

  // two groups of eight rows in flight, or one when a group alone takes 32 registers: the
  // kernel gains more from another wavefront per SIMD than from the deeper prefetch
  constexpr bool kTwoGroups = sizeof(raw_vec_t<RT, VEC>) * 8 <= 64 || !FLEXSAE_TOPK_ONE_GROUP;
  raw_vec_t<RT, VEC> buf_a[8], buf_b[kTwoGroups ? 8 : 1];
  auto issue = [&](raw_vec_t<RT, VEC>(&buf)[8], int j) {
#pragma unroll
    for (int h = 0; h < 8; h += FLEXSAE_TOPK_ROWS_PER_TEST) {
      if (h == 0 || j + h < n) {  // uniform: the second half of a group only when it has rows
#pragma unroll
        for (int u = h; u < h + FLEXSAE_TOPK_ROWS_PER_TEST; ++u) {
          const int jj = (j + u) < n ? (j + u) : (n - 1);
          buf[u] = gather_raw<RT, VEC>(rows_src, lane_off, static_cast<uint32_t>(bcast_i32(my_b, jj)) * row_stride);
        }
      }
    }
  };
  issue(buf_a, 0);
  if constexpr (kTwoGroups) {
    if (n > 8) issue(buf_b, 8);
  }

  float w[VEC], acc[VEC];
  unpack_raw<WT, VEC>(wraw, w);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    acc[i] = 0.f;
    if (!active) w[i] = 0.f;
  }
  uint32_t ww[(VEC + 1) / 2] = {};  // the W piece as packed pairs (dot2 path)
  if constexpr (kDot2) {
    __builtin_memcpy(ww, &wraw, sizeof(raw_vec_t<WT, VEC>));
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i)
      if (!active) ww[i] = 0u;
  }
  const float v = __uint_as_float(vbits) * (late_scale ? 1.f : scale);
  float my_dot = 0.f;
  auto consume = [&](const raw_vec_t<RT, VEC>(&rows)[8], int j) {  // slots j .. j+7 of the latent
    float dots[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) dots[u] = 0.f;
#pragma unroll
    for (int h = 0; h < 8; h += FLEXSAE_TOPK_ROWS_PER_TEST) {
      if (h != 0 && j + h >= n) continue;  // uniform
#pragma unroll
      for (int u = h; u < h + FLEXSAE_TOPK_ROWS_PER_TEST; ++u) {
        float dot = 0.f;
        if constexpr (kDot2) {
          uint32_t xw[VEC / 2];
          __builtin_memcpy(xw, &rows[u], sizeof(xw));
#pragma unroll
          for (int i = 0; i < VEC / 2; ++i) dot = dot2_bf16(xw[i], ww[i], dot);
          if (late_scale) {  // uniform
            // a bf16 val widened to fp32 keeps its 16 bits in the upper half
            const uint32_t v_hi = static_cast<uint32_t>(bcast_i32(static_cast<int>(vbits), j + u));
            const uint32_t v_lo = v_hi >> 16;
#pragma unroll
            for (int i = 0; i < VEC / 2; ++i) {
              acc[2 * i] = dot2_bf16(xw[i], v_lo, acc[2 * i]);
              acc[2 * i + 1] = dot2_bf16(xw[i], v_hi, acc[2 * i + 1]);
            }
          } else {
            float x[VEC];
            unpack_raw<RT, VEC>(rows[u], x);
            const float vj = bcast_f32(v, j + u);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = fmaf(vj, x[i], acc[i]);
          }
        } else {
          float x[VEC];
          unpack_raw<RT, VEC>(rows[u], x);
          const float vj = bcast_f32(v, j + u);
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            acc[i] = fmaf(vj, x[i], acc[i]);
            dot = fmaf(x[i], w[i], dot);
          }
        }
        dots[u] = dot;
      }
    }
    const float tot = wave_sum8_transposed(dots);  // lane L: total of slot j + (L & 7)
    if ((lane >> 3) == (j >> 3)) my_dot = tot;
  };
  if constexpr (kTwoGroups) {
    for (int j = 0; j < n; j += 16) {
      consume(buf_a, j);
      if (j + 16 < n) issue(buf_a, j + 16);
      if (j + 8 < n) {
        consume(buf_b, j + 8);
        if (j + 24 < n) issue(buf_b, j + 24);
      }
    }
  } else {
    for (int j = 0; j < n; j += 8) {
      consume(buf_a, j);
      if (j + 8 < n) issue(buf_a, j + 8);
    }
  }
  if (late_scale) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] *= scale;
  }
  if (active) store_vec<GT, VEC, FLEXSAE_TOPK_NT>(dW, f * D + d0, acc);
  if (lane < n) dv_tile[b0 + lane] = my_dot * scale;
}

// TopK backward of one slice.  scale = grad_out * 2/(B*D).
// Blocks [0, n_long_blocks): long latents, one wavefront per (64-pair chunk, tile): stores its
// dvals shares, leaves its dW contribution in partial[chunk, slice column] (fp32) for
// seg_reduce_long_finalize_kernel (next launch).  They come first so hot latents start at once.
// Remaining blocks: one wavefront per (tile of the slice = blockIdx.y, latent f); blocks are
// handed out x first, i.e. tile-major, so that at any moment the waves in flight share one
// B x tile slice of resid (L2-sized); see topk_short_latent.  tile = 64*VEC columns, lane l owning VEC consecutive columns.
// dW[f, tile] is written exactly once, in the gradient's final dtype; latents without pairs
// get zeros.
template <typename WT, typename GT, typename RT, int VEC>
__global__ __launch_bounds__(256) void topk_bwd_kernel(
    const uint32_t *__restrict__ begin, const uint32_t *__restrict__ map,
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const vec_t<uint32_t, 2> *__restrict__ slot_bv,
    const void *__restrict__ weight, const void *__restrict__ vals, int vals_dtype,
    const void *__restrict__ resid, const float *__restrict__ grad_out, float coef,
    void *__restrict__ dW, float *__restrict__ dv_part, int64_t n_pairs, float *__restrict__ partial,
    unsigned n_long_blocks, int tps, int col0, int slice_w, int64_t F, int K, int D,
    uint32_t resid_bytes) {
  const int lane = lane_id();
  const float scale = coef * grad_out[0];
  if (blockIdx.x >= n_long_blocks) {
    // blockIdx.y = tile of the slice, blockIdx.x - n_long_blocks = group of latents
    const int64_t f = static_cast<int64_t>(blockIdx.x - n_long_blocks) * (blockDim.x >> 6) + wave_in_block();
    if (f >= F) return;  // uniform per wavefront
    const int t = static_cast<int>(blockIdx.y);
    const uint32_t b0 = begin[f];
    const uint32_t n = begin[f + 1] - b0;
    if (n > static_cast<uint32_t>(kSegChunk)) return;  // chunk role
    const int d0 = col0 + t * (kWave * VEC) + lane * VEC;
    if (n == 0) {  // unused latent: zeros
      const float zero[VEC] = {};
      if (d0 < D) store_vec<GT, VEC, FLEXSAE_TOPK_NT>(dW, f * D + d0, zero);
      return;
    }
    const GatherSource rows_src = make_gather_source(resid, resid_bytes);
    topk_short_latent<WT, GT, RT, VEC>(
        slot_bv, weight, vals_dtype, rows_src, static_cast<uint32_t>(D) * sizeof(typename Traits<RT>::store_t), scale,
        dW, dv_part + (col0 / (kWave * VEC) + t) * n_pairs, f, b0, static_cast<int>(n), d0, D);
    return;
  }
  const uint32_t n_long = *long_count;
  if (n_long == 0) return;
  const uint32_t n_chunks = chunk_begin[n_long];
  const int64_t total = static_cast<int64_t>(n_chunks) * tps;
  const int64_t n_waves = static_cast<int64_t>(n_long_blocks) * gridDim.y * (blockDim.x >> 6);
  for (int64_t wk = (static_cast<int64_t>(blockIdx.y) * n_long_blocks + blockIdx.x) * (blockDim.x >> 6) +
                    wave_in_block();
       wk < total; wk += n_waves) {
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
    topk_accumulate_slots<RT, VEC>(slot_bv, resid, scale, dv_part + (col0 / (kWave * VEC) + t) * n_pairs, w, c.s0,
                                   c.s1, D, dsafe, acc);
    store_vec<float, VEC>(partial, static_cast<int64_t>(chunk) * slice_w + pc, acc);
  }
}

// dvals[map[slot]] = sum over the column tiles of dv_part[tile, slot], in tile order
// (every pair sits in exactly one slot, so dvals is written once and needs no zero-fill).
__global__ void topk_dvals_finalize_kernel(const uint32_t *__restrict__ map,
                                           const float *__restrict__ dv_part, int n_tiles,
                                           int64_t n_pairs, float *__restrict__ dvals) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t s = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; s < n_pairs; s += stride) {
    float acc = 0.f;
    for (int t = 0; t < n_tiles; ++t) acc += dv_part[t * n_pairs + s];
    dvals[map[s]] = acc;
  }
}

// Preparation of a TopK backward, one launch:
//   slot_bv[s] = (batch row, val as fp32 bits) of the pair in slot s of the latent-major list: what
//     the backward reads per pair, contiguous per latent instead of scattered over vals; a pair
//     whose index lies outside [0, F) gets a val of zero, as in the forward (the pair list files it
//     under latent 0), so that it adds nothing to dW (`indices` may be null: every val is kept);
//   resid16[i] = bf16(resid[i]) for i < n_resid (n_resid = 0: no copy wanted).
__global__ void topk_prepare_kernel(const uint32_t *__restrict__ map, const int64_t *__restrict__ indices,
                                    int64_t F, const void *__restrict__ vals,
                                    int vals_dtype, int64_t n_pairs, int K,
                                    vec_t<uint32_t, 2> *__restrict__ slot_bv, const float *__restrict__ resid,
                                    int64_t n_resid, void *__restrict__ resid16) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (int64_t s = tid; s < n_pairs; s += stride) {
    const uint32_t p = map[s];
    vec_t<uint32_t, 2> r;
    r[0] = p / static_cast<uint32_t>(K);
    float v = load_scalar(vals, vals_dtype, p);
    if (indices && static_cast<uint64_t>(indices[p]) >= static_cast<uint64_t>(F)) v = 0.f;
    r[1] = __float_as_uint(v);
    slot_bv[s] = r;
  }
  const int64_t n4 = n_resid >> 2;
  for (int64_t i = tid; i < n4; i += stride) {
    float x[4];
    load_vec<float, 4>(resid, i * 4, x);
    store_vec<bf16_t, 4>(resid16, i * 4, x);
  }
  for (int64_t i = (n4 << 2) + tid; i < n_resid; i += stride) {
    float x[1] = {resid[i]};
    store_vec<bf16_t, 1>(resid16, i, x);
  }
}

}  // namespace flexsae
