// HierarchicalTopK backward: reverse sweep over K per (row, D-tile).
#pragma once

#include "common.hpp"
#include "csr_kernels.hpp"
#include "fwd_kernels.hpp"

namespace flexsae {

// One wavefront per (row b, D-tile) item; a tile is 64*C columns and lane l owns the
// columns l, l+64, ..., l+64*(C-1) of the tile.  With this interleaved ownership every
// atomic instruction of the scatter covers 64 consecutive fp32 of one dW row (two full
// 128-byte lines), which is the densest request the L2 atomic units can be given.
//
// State per lane and owned column: e = r_{b,k} - t_b (starts from the saved forward
// residual) and S = sum_{k' >= k} scale * e_{k'}.  Walking k = K-1 .. 0:
//   S    += scale * e                        (scale = grad_out * 2/(B*K*D))
//   dW[idx_k]  += vals_k * S                 (fp32 atomics)
//   dvals_k     = <W[idx_k], S>              (wave reduction; added across tiles by atomics)
//   e    -= vals_k * W[idx_k]                (step back to r_{b,k-1} - t_b)
// and finally dbias += S.
template <typename WT, int C, int U>
__global__ __launch_bounds__(256) void hier_bwd_kernel(
    const int64_t *__restrict__ indices, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const float *__restrict__ resid,
    const float *__restrict__ grad_out, float coef, float *__restrict__ dW,
    float *__restrict__ dvals, float *__restrict__ dbias, int *status_flag, int64_t n_items,
    int ntiles, int K, int64_t F, int D) {
  using S_t = typename Traits<WT>::store_t;
  const S_t *__restrict__ W = static_cast<const S_t *>(weight);
  const int lane = lane_id();
  const int64_t item = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block();
  if (item >= n_items) return;  // uniform per wavefront
  const int64_t b = item / ntiles;
  const int tile = static_cast<int>(item - b * ntiles);
  const int dbase = tile * (kWave * C) + lane;
  const float scale = coef * grad_out[0];

  bool act[C];
  int dcol[C];
  float e[C], S[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int d = dbase + c * kWave;
    act[c] = d < D;
    dcol[c] = act[c] ? d : 0;
    e[c] = act[c] ? resid[b * D + d] : 0.f;
    S[c] = 0.f;
  }

  const int64_t pair0 = b * K;
  for (int k0 = ((K - 1) / kWave) * kWave; k0 >= 0; k0 -= kWave) {
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
    float my_dval = 0.f;

    auto step = [&](int j, int64_t rowoff, const float(&w)[C]) {
      const float v = bcast_f32(my_val, j);
      float dot = 0.f;
#pragma unroll
      for (int c = 0; c < C; ++c) {
        S[c] = fmaf(scale, e[c], S[c]);
        if (act[c]) unsafeAtomicAdd(dW + rowoff + dcol[c], S[c] * v);
        dot = fmaf(w[c], S[c], dot);
        e[c] = fmaf(-w[c], v, e[c]);
      }
      dot = wave_sum_bcast(dot);
      if (lane == j) my_dval = dot;
    };

    int j = n - 1;
    for (; j - (U - 1) >= 0; j -= U) {
      float w[U][C];
      int64_t rowoff[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        rowoff[u] = static_cast<int64_t>(bcast_i32(my_row, j - u)) * D;
#pragma unroll
        for (int c = 0; c < C; ++c) w[u][c] = act[c] ? Traits<WT>::up(W[rowoff[u] + dcol[c]]) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) step(j - u, rowoff[u], w[u]);
    }
    for (; j >= 0; --j) {
      float w[C];
      const int64_t rowoff = static_cast<int64_t>(bcast_i32(my_row, j)) * D;
#pragma unroll
      for (int c = 0; c < C; ++c) w[c] = act[c] ? Traits<WT>::up(W[rowoff + dcol[c]]) : 0.f;
      step(j, rowoff, w);
    }
    if (kk < K) unsafeAtomicAdd(dvals + pair0 + kk, my_dval);
  }
#pragma unroll
  for (int c = 0; c < C; ++c)
    if (act[c]) unsafeAtomicAdd(dbias + dcol[c], S[c]);
}

}  // namespace flexsae

namespace flexsae {

// Sweep kernel of the two-phase backward.  Same reverse walk as hier_bwd_kernel, but the
// per-pair contribution vals_k * S is STORED instead of being added to dW with atomics (the
// L2 atomic units retire about one fp32 per clock and channel, far below what the walk can
// produce).  The contribution of pair p goes to row slot[p] of P, slot[] being the pair's
// position in the latent-major pair list, so that all rows of one latent are adjacent and a
// segment reduction (segment_kernels.hpp) can stream them.  Only the columns
// [col0, col0 + tps*64*VEC) of the problem (one "slice") are handled per launch, so P needs
// B*K*slice_width elements.  Every tile leaves its share of the dvals dot products in dv_part;
// hier_dvals_finalize_kernel adds the shares in tile order (deterministic).
//
// One wavefront per (tile of the slice, row b), tile-major: the wavefronts in flight at any
// moment gather from the same 64*VEC-column slice of W, which is small enough to stay in the
// on-chip caches while it is being reused by every row.  Lane l owns VEC consecutive columns,
// so the gathered weight piece and the stored contribution are one vector access per lane.
template <typename WT, typename PT, int VEC, int U>
__global__ __launch_bounds__(256) void hier_sweep_kernel(
    const int64_t *__restrict__ indices, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const float *__restrict__ resid,
    const float *__restrict__ grad_out, float coef, const uint32_t *__restrict__ slot,
    void *__restrict__ P, float *__restrict__ dv_part, float *__restrict__ s_final, int s_final_ld,
    int *status_flag, int64_t n_items, int64_t B, int col0, int slice_w, int K, int64_t F,
    int D) {
  const int lane = lane_id();
  const int64_t item = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block();
  if (item >= n_items) return;  // uniform per wavefront
  const int t = static_cast<int>(item / B);
  const int64_t b = item - static_cast<int64_t>(t) * B;
  const int pc = t * (kWave * VEC) + lane * VEC;  // column inside the slice
  const int d0 = col0 + pc;
  const bool active = d0 < D;
  const int dsafe = active ? d0 : 0;
  const float scale = coef * grad_out[0];

  float e[VEC], S[VEC];
  load_vec<float, VEC>(resid, b * D + dsafe, e);
#pragma unroll
  for (int i = 0; i < VEC; ++i) S[i] = 0.f;

  constexpr int UB = U / 8;  // blocks of eight steps whose gathers are in flight together
  static_assert(U % 8 == 0, "the prefetch depth counts blocks of eight steps");
  const int64_t pair0 = b * K;
  for (int k0 = ((K - 1) / kWave) * kWave; k0 >= 0; k0 -= kWave) {
    const int kk = k0 + lane;
    int64_t my_idx = 0;
    float my_val = 0.f;
    int my_slot = 0;
    if (kk < K) {
      my_idx = indices[pair0 + kk];
      my_val = load_scalar(vals, vals_dtype, pair0 + kk);
      my_slot = static_cast<int>(slot[pair0 + kk]);
    }
    if (static_cast<uint64_t>(my_idx) >= static_cast<uint64_t>(F)) {
      if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
      my_idx = 0;
      my_val = 0.f;
    }
    const int my_row = static_cast<int>(my_idx);
    const int n = (K - k0) < kWave ? (K - k0) : kWave;  // uniform
    float my_dval = 0.f;

    // Steps run from n-1 down to 0 in aligned blocks of eight; the eight dot products of a block
    // share one transposed wave reduction, whose result for step j lands in lane j.  Lanes beyond
    // column D gather zeros, so their dot products vanish, and what they store lands in the
    // padding columns of P, which nobody reads.
    for (int m = ((n + 7) >> 3) - 1; m >= 0; m -= UB) {
      raw_vec_t<WT, VEC> w[UB][8];
#pragma unroll
      for (int ub = 0; ub < UB; ++ub) {
        if (m - ub >= 0) {  // uniform
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int j = (m - ub) * 8 + q;
            const int jj = j < n ? j : (n - 1);  // past the end: re-read the last row
            w[ub][q] = gather_row_piece<WT, VEC>(weight, static_cast<uint32_t>(bcast_i32(my_row, jj)), D, d0);
          }
        }
      }
#pragma unroll
      for (int ub = 0; ub < UB; ++ub) {
        if (m - ub >= 0) {  // uniform
          float dots[8];
#pragma unroll
          for (int q = 7; q >= 0; --q) {
            const int j = (m - ub) * 8 + q;
            dots[q] = 0.f;
            if (j < n) {  // uniform
              const float v = bcast_f32(my_val, j);
              const uint32_t prow = static_cast<uint32_t>(bcast_i32(my_slot, j));
              float wj[VEC], contrib[VEC];
              unpack_raw<WT, VEC>(w[ub][q], wj);
              float dot = 0.f;
#pragma unroll
              for (int i = 0; i < VEC; ++i) {
                S[i] = fmaf(scale, e[i], S[i]);
                contrib[i] = S[i] * v;
                dot = fmaf(wj[i], S[i], dot);
                e[i] = fmaf(-wj[i], v, e[i]);
              }
              // no streaming hint: the slice is read back at once by the segment reduction
              scatter_row_piece<PT, VEC, false>(P, prow, slice_w, pc, contrib);
              dots[q] = dot;
            }
          }
          const float tot = wave_sum8_transposed(dots);  // lane L: total of step 8*(m-ub) + (L & 7)
          if ((lane >> 3) == (m - ub)) my_dval = tot;
        }
      }
    }
    // this tile's share of dvals; hier_dvals_finalize_kernel adds the tiles up in order
    if (kk < K) dv_part[(static_cast<int64_t>(col0 / (kWave * VEC)) + t) * (B * K) + pair0 + kk] = my_dval;
  }
  // the row's total S_{b,0} (its share of dbias) goes to s_final[b, column]; a column sum over
  // b follows (thousands of atomics per dbias element would serialise instead)
  if (!active) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) S[i] = 0.f;
  }
  store_vec<float, VEC>(s_final, b * s_final_ld + col0 + pc, S);
}

// dvals[p] = sum over the column tiles of dv_part[tile, p], in tile order (deterministic).
__global__ void hier_dvals_finalize_kernel(const float *__restrict__ dv_part, int n_tiles, int64_t n_pairs,
                                           float *__restrict__ dvals) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < n_pairs; p += stride) {
    float acc = 0.f;
    for (int t = 0; t < n_tiles; ++t) acc += dv_part[t * n_pairs + p];
    dvals[p] = acc;
  }
}

// What follows the slices of a hierarchical step, in one launch of 1024-thread blocks (the three
// parts are independent; each computes what its own kernel computes, bit for bit):
//   block 0                 the loss from the per-(tile, row) partials (loss_finalize_kernel), when
//                           loss_partial is given;
//   the next n_colsum_blocks stage 1 of the column sums of s_final (colsum_partial_kernel): a block
//                           takes 256 columns of four consecutive row chunks;
//   the rest                dvals from its per-tile shares (hier_dvals_finalize_kernel).
__global__ __launch_bounds__(1024) void hier_epilogue_kernel(
    const float *__restrict__ loss_partial, int64_t n_loss_partials, double inv_count, float *__restrict__ loss,
    const float *__restrict__ s_final, int64_t rows, int64_t ld, int cols, float *__restrict__ colsum_part,
    unsigned n_colsum_blocks, const float *__restrict__ dv_part, int n_tiles, int64_t n_pairs,
    float *__restrict__ dvals) {
  __shared__ double red[1024];
  if (blockIdx.x == 0) {
    if (loss_partial) loss_finalize_block(loss_partial, n_loss_partials, inv_count, loss, red);
    return;
  }
  const unsigned blk = blockIdx.x - 1;
  if (blk < n_colsum_blocks) {
    const unsigned col_blocks = static_cast<unsigned>((cols + 255) / 256);
    const unsigned bx = blk % col_blocks, by = blk / col_blocks;
    colsum_partial_one(s_final, rows, ld, cols, colsum_part, static_cast<int>(bx * 256 + (threadIdx.x & 255)),
                       static_cast<int64_t>(by) * 4 + (threadIdx.x >> 8));
    return;
  }
  const int64_t n_blocks = static_cast<int64_t>(gridDim.x) - 1 - n_colsum_blocks;
  const int64_t stride = n_blocks * 1024;
  for (int64_t p = static_cast<int64_t>(blk - n_colsum_blocks) * 1024 + threadIdx.x; p < n_pairs; p += stride) {
    float acc = 0.f;
    for (int t = 0; t < n_tiles; ++t) acc += dv_part[t * n_pairs + p];
    dvals[p] = acc;
  }
}

}  // namespace flexsae
