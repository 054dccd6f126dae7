// Latent-major segment reduction: out[f, slice] = sum of the rows [begin[f], begin[f+1]) of
// P[., slice] (rows of one latent are adjacent), with fp32 accumulation and one write per
// output element.  Short groups (<= 64 rows) are reduced by one wavefront; long ones are cut
// into chunks of 64 rows whose fp32 partial sums are combined in chunk order, so a hot latent is
// spread over many wavefronts and the summation order stays fixed (deterministic).
#pragma once

#include "common.hpp"

#ifndef FLEXSAE_REDUCE_NT
#define FLEXSAE_REDUCE_NT true
#endif

namespace flexsae {

constexpr int kSegChunk = 64;  // rows per chunk; groups longer than this count as "long"
constexpr int kSegClasses = kSegChunk + 1;  // row counts 0..kSegChunk of the list ordered by row count (below)
constexpr int kSegBigRows = 9;  // latents with at least this many rows get a group of lanes to themselves there

// acc += sum of rows [r0, r0+n) of X (row stride `ld` elements) over the lane's VEC columns at pc.
// Rows are fetched up to U at a time; n is uniform over the wavefront, so the tests around the
// loads are scalar branches and a short group issues exactly its own loads, all in flight at once.
template <typename PT, int VEC, int U, bool NT = false>
__device__ __forceinline__ void accumulate_rows(const void *__restrict__ X, int64_t r0, int n,
                                                int64_t ld, int pc, float (&acc)[VEC]) {
  for (int j = 0; j < n; j += U) {
    raw_vec_t<PT, VEC> raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j + u < n) raw[u] = load_raw<PT, VEC, NT>(X, (r0 + j + u) * ld + pc);  // uniform
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j + u < n) {  // uniform
        float x[VEC];
        unpack_raw<PT, VEC>(raw[u], x);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += x[i];
      }
    }
  }
}

// The same sum in the order of the reduction by pieces (below), so that both reductions give the
// same bits for long latents: four running sums, row j goes to sum j % 4, combined as
// (s0 + s1) + (s2 + s3).
template <typename PT, int VEC, int U, bool NT = false>
__device__ __forceinline__ void accumulate_rows_by4(const void *__restrict__ X, int64_t r0, int n,
                                                    int64_t ld, int pc, float (&acc)[VEC]) {
  static_assert(U % 4 == 0, "rows are dealt to four sums");
  float part[4][VEC];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int i = 0; i < VEC; ++i) part[g][i] = 0.f;
  for (int j = 0; j < n; j += U) {
    raw_vec_t<PT, VEC> raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j + u < n) raw[u] = load_raw<PT, VEC, NT>(X, (r0 + j + u) * ld + pc);  // uniform
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j + u < n) {  // uniform
        float x[VEC];
        unpack_raw<PT, VEC>(raw[u], x);
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[u & 3][i] += x[i];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = (part[0][i] + part[1][i]) + (part[2][i] + part[3][i]);
}

// Decode work item `chunk` of the long-latent work list: which latent, which rows.
struct LongChunk {
  uint32_t long_slot;
  int64_t f;
  uint32_t s0, s1;  // rows [s0, s1) of the pair list
};
__device__ __forceinline__ LongChunk seg_decode_chunk(const uint32_t *__restrict__ begin,
                                                      const uint32_t *__restrict__ long_list,
                                                      const uint32_t *__restrict__ chunk_begin,
                                                      uint32_t n_long, uint32_t chunk) {
  uint32_t lo = 0, hi = n_long;  // largest i with chunk_begin[i] <= chunk
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (chunk_begin[mid] <= chunk) lo = mid; else hi = mid;
  }
  LongChunk c;
  c.long_slot = lo;
  c.f = long_list[lo];
  c.s0 = begin[c.f] + (chunk - chunk_begin[lo]) * kSegChunk;
  const uint32_t s_lim = begin[c.f + 1];
  c.s1 = (s_lim - c.s0) < static_cast<uint32_t>(kSegChunk) ? s_lim : c.s0 + kSegChunk;
  return c;
}

// Segment reduction of one slice.
// Blocks [0, n_long_blocks): long latents.  Every (64-row chunk, tile) is reduced by one
// wavefront into partial[chunk, slice column] (fp32); the wavefronts stride over the work list,
// whose length is only known on the device.  seg_reduce_long_finalize_kernel (next launch)
// combines the partials in chunk order.  These blocks come first so that hot latents start
// at once and overlap with the bulk of the work.
// Remaining blocks: one wavefront per (latent, tile of 64*VEC columns of the slice); latents
// without rows get zeros; latents with more than kSegChunk rows are skipped.
template <typename PT, typename GT, int VEC, int U>
__global__ __launch_bounds__(256) void seg_reduce_kernel(
    const uint32_t *__restrict__ begin, const uint32_t *__restrict__ long_count,
    const uint32_t *__restrict__ long_list, const uint32_t *__restrict__ chunk_begin,
    const void *__restrict__ P, float *__restrict__ partial, void *__restrict__ out,
    const float *__restrict__ scale, int64_t F, unsigned n_long_blocks, int tps, int col0,
    int slice_w, int D) {
  const int lane = lane_id();
  if (blockIdx.x >= n_long_blocks) {
    // one wavefront per (latent, tile), tiles of a latent adjacent: the launch reads P front to back
    const int64_t item = static_cast<int64_t>(blockIdx.x - n_long_blocks) * (blockDim.x >> 6) + wave_in_block();
    const int64_t f = item / tps;
    if (f >= F) return;  // uniform per wavefront
    const int t = static_cast<int>(item - f * tps);
    const uint32_t s0 = begin[f];
    const uint32_t n = begin[f + 1] - s0;
    if (n > static_cast<uint32_t>(kSegChunk)) return;
    const int pc = t * (kWave * VEC) + lane * VEC;
    const int d0 = col0 + pc;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    accumulate_rows<PT, VEC, U, FLEXSAE_REDUCE_NT>(P, s0, static_cast<int>(n), slice_w, pc, acc);
    if (scale) {  // the rows were produced for a unit upstream gradient
      const float g = scale[0];
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] *= g;
    }
    if (d0 < D) store_vec<GT, VEC, FLEXSAE_REDUCE_NT>(out, f * D + d0, acc);
    return;
  }
  const uint32_t n_long = *long_count;
  if (n_long == 0) return;
  const int64_t total = static_cast<int64_t>(chunk_begin[n_long]) * tps;
  const int64_t n_waves = static_cast<int64_t>(n_long_blocks) * (blockDim.x >> 6);
  for (int64_t w = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block(); w < total;
       w += n_waves) {
    const uint32_t chunk = static_cast<uint32_t>(w / tps);
    const int t = static_cast<int>(w - static_cast<int64_t>(chunk) * tps);
    const LongChunk c = seg_decode_chunk(begin, long_list, chunk_begin, n_long, chunk);
    const int pc = t * (kWave * VEC) + lane * VEC;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    accumulate_rows_by4<PT, VEC, 8, FLEXSAE_REDUCE_NT>(P, c.s0, static_cast<int>(c.s1 - c.s0), slice_w, pc, acc);
    store_vec<float, VEC>(partial, static_cast<int64_t>(chunk) * slice_w + pc, acc);
  }
}

// Same reduction with a finer work item: sixteen lanes (a quarter of a wavefront), 16 bytes each,
// serve one (latent, 256-byte piece of the slice's rows of P) -- 128 columns of bf16 contributions,
// 64 of fp32 -- so that a slice may be any whole number of such pieces wide.  A narrow slice is what
// keeps the contributions of one slice in the memory-side cache between the launch that writes them
// and this one.  The four latents (or pieces) of a wavefront have different row counts: the loop
// runs to the longest, loads beyond a group's own count are masked off.  Work order: pieces of a
// latent adjacent, latents ascending, so the launch still reads P front to back.  G > 1: a group
// serves G latents taken from the list ordered by row count (cls_list / cls_begin, see
// seg_class_scatter_kernel; chosen by the caller where most latents have no or few rows), and
// latents without rows are not written here.
constexpr int kPieceLanes = 16;
constexpr int kPieceBytes = kPieceLanes * 16;

template <typename PT, typename GT, int U, int G>
__global__ __launch_bounds__(256) void seg_reduce_piece_kernel(
    const uint32_t *__restrict__ begin, const uint32_t *__restrict__ long_count,
    const uint32_t *__restrict__ long_list, const uint32_t *__restrict__ chunk_begin,
    const void *__restrict__ P, float *__restrict__ partial, void *__restrict__ out,
    const float *__restrict__ scale, int64_t F, unsigned n_long_blocks, int pps, int pps_shift, int col0,
    int slice_w, int D, int update, const uint32_t *__restrict__ cls_list,
    const uint32_t *__restrict__ cls_begin) {
  using S = typename Traits<PT>::store_t;
  constexpr int EV = 16 / static_cast<int>(sizeof(S));  // columns per lane
  constexpr int kGroupsPerBlock = 256 / kPieceLanes;
  const int sub = static_cast<int>(threadIdx.x) & (kPieceLanes - 1);
  const int group = static_cast<int>(threadIdx.x) / kPieceLanes;
  const S *__restrict__ Pp = static_cast<const S *>(P);

  // acc += rows r0, r0+step, ... (n of them) of P at the lane's columns; n differs between the
  // groups of a wavefront
  auto accumulate = [&](int64_t r0, int n, int step, int pc, float (&acc)[EV]) {
    const S *row = Pp + r0 * slice_w + pc;
    const int64_t stride = static_cast<int64_t>(step) * slice_w;
    for (int j = 0; __any(j < n); j += U) {
      raw_vec_t<PT, EV> raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        raw[u] = raw_vec_t<PT, EV>{};
        if (j + u < n)
          raw[u] = __builtin_nontemporal_load(reinterpret_cast<const raw_vec_t<PT, EV> *>(row + (j + u) * stride));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float x[EV];
        unpack_raw<PT, EV>(raw[u], x);
#pragma unroll
        for (int i = 0; i < EV; ++i) acc[i] += x[i];  // masked-off loads left zeros
      }
    }
  };

  // A latent's finished sum goes to out[f, d0..]; in update mode it is subtracted from what is there
  // (out is then the weight matrix, the sum arrives scaled by the step size, and latents without
  // rows are left alone).
  auto emit = [&](int64_t f, int d0, float (&acc)[EV]) {
    if (d0 >= D) return;
    if (update) {
      float w[EV];
      load_vec<GT, EV>(out, f * D + d0, w);
#pragma unroll
      for (int i = 0; i < EV; ++i) acc[i] = w[i] - acc[i];
    }
    store_vec<GT, EV, FLEXSAE_REDUCE_NT>(out, f * D + d0, acc);
  };

  if (blockIdx.x >= n_long_blocks) {
    // (latent block, piece) of this group of lanes; a latent block is G consecutive latents.  The
    // block's first item is split with one wave-uniform division; the sixteen groups then only
    // divide a number below pps + 16 (a 64-bit division per lane would cost more instructions than
    // the rest of a short item)
    const int64_t item0 = static_cast<int64_t>(blockIdx.x - n_long_blocks) * kGroupsPerBlock;
    int64_t fb;
    int t;
    if (pps_shift >= 0) {  // pps is a power of two (the usual slice widths): shifts only
      const int64_t item = item0 + group;
      fb = item >> pps_shift;
      t = static_cast<int>(item & ((1 << pps_shift) - 1));
    } else {
      const int64_t f_first = item0 / pps;
      const uint32_t rem = static_cast<uint32_t>(item0 - f_first * pps) + static_cast<uint32_t>(group);
      const uint32_t q = rem / static_cast<uint32_t>(pps);
      fb = f_first + q;
      t = static_cast<int>(rem - q * static_cast<uint32_t>(pps));
    }
    const int pc = t * (kPieceLanes * EV) + sub * EV;
    const int d0 = col0 + pc;
    const float g = scale ? scale[0] : 1.0f;  // the rows were produced for a unit upstream gradient
    float acc[EV];
#pragma unroll
    for (int i = 0; i < EV; ++i) acc[i] = 0.f;
    if constexpr (G == 1) {
      const int64_t f = fb;
      uint32_t s0 = 0, n = 0;
      if (f < F) {
        s0 = begin[f];
        n = begin[f + 1] - s0;
      }
      const bool mine = f < F && n <= static_cast<uint32_t>(kSegChunk);  // longer ones: chunked below
      accumulate(s0, mine ? static_cast<int>(n) : 0, 1, pc, acc);
      if (scale) {
#pragma unroll
        for (int i = 0; i < EV; ++i) acc[i] *= g;
      }
      if (mine && !(update && n == 0)) emit(f, d0, acc);
    } else {
      // Few rows per latent and most latents without any: the latents come from the list that
      // seg_class_scatter_kernel wrote, ordered by row count (those without rows first: they are
      // zeroed by seg_zero_rows_kernel and skipped here; those with more than kSegChunk rows are not
      // in it).  A group serves G consecutive entries, i.e. G latents of (nearly always) the same row
      // count, so the four groups of a wavefront finish together; their rows are fetched U at a time
      // regardless of where one latent ends and the next begins, and a latent's sum is stored when
      // its last row has been added.  The order of the additions of a latent is the same as with G = 1.
      // Work items: first the latents with kSegBigRows rows or more, one per group and the heaviest
      // first (a group that had four of them would still be running long after the rest of the launch),
      // then the others, G per group.
      const uint32_t lo = cls_begin[1], mid = cls_begin[kSegBigRows], hi = cls_begin[kSegChunk + 1];
      const int64_t n_big = static_cast<int64_t>(hi - mid);
      int64_t first;  // first entry of this group
      int count;      // entries it serves
      if (fb < n_big) {
        first = static_cast<int64_t>(hi) - 1 - fb;
        count = 1;
      } else {
        first = static_cast<int64_t>(lo) + (fb - n_big) * G;
        const int64_t left = static_cast<int64_t>(mid) - first;
        count = left < G ? (left > 0 ? static_cast<int>(left) : 0) : G;
      }
      uint32_t fv = 0, b0v = 0, b1v = 0;  // lane j < count of the group: entry j, its latent and rows
      if (sub < count) {
        fv = cls_list[first + sub];
        b0v = begin[fv];
        b1v = begin[fv + 1];
      }
      uint32_t c[G + 1], off[G], fid[G];  // row i of the group's list, c[j] <= i < c[j+1], is row i + off[j] of P
      c[0] = 0;
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const uint32_t b0 = static_cast<uint32_t>(__shfl(static_cast<int>(b0v), j, kPieceLanes));
        const uint32_t b1 = static_cast<uint32_t>(__shfl(static_cast<int>(b1v), j, kPieceLanes));
        fid[j] = static_cast<uint32_t>(__shfl(static_cast<int>(fv), j, kPieceLanes));
        c[j + 1] = c[j] + (b1 - b0);  // nothing for entries beyond the list
        off[j] = b0 - c[j];
      }
      const uint32_t total = c[G];
      for (uint32_t i0 = 0; __any(i0 < total); i0 += U) {
        raw_vec_t<PT, EV> raw[U];
        uint32_t whose[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t i = i0 + u;
          raw[u] = raw_vec_t<PT, EV>{};
          whose[u] = fid[0];
          uint32_t o = off[0];
#pragma unroll
          for (int j = 1; j < G; ++j)
            if (i >= c[j]) {
              whose[u] = fid[j];
              o = off[j];
            }
          if (i < total)
            raw[u] = __builtin_nontemporal_load(reinterpret_cast<const raw_vec_t<PT, EV> *>(
                Pp + static_cast<int64_t>(i + o) * slice_w + pc));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t i = i0 + u;
          float x[EV];
          unpack_raw<PT, EV>(raw[u], x);
#pragma unroll
          for (int k = 0; k < EV; ++k) acc[k] += x[k];  // masked-off loads left zeros
          bool last = false;  // the last row of its latent
#pragma unroll
          for (int j = 1; j <= G; ++j) last |= i + 1 == c[j];
          if (i < total && last) {
            if (scale) {
#pragma unroll
              for (int k = 0; k < EV; ++k) acc[k] *= g;
            }
            emit(static_cast<int64_t>(whose[u]), d0, acc);
#pragma unroll
            for (int k = 0; k < EV; ++k) acc[k] = 0.f;
          }
        }
      }
    }
    return;
  }
  // Long latents: one wavefront per (64-row chunk, piece); its four groups take every fourth row
  // (sixteen rows in flight per wavefront) and their sums are added across the groups in a fixed
  // order.  A hot latent's chunks are spread over many wavefronts.
  const uint32_t n_long = *long_count;
  if (n_long == 0) return;
  constexpr int kGroups = kWave / kPieceLanes;
  const int64_t total = static_cast<int64_t>(chunk_begin[n_long]) * pps;
  const int64_t n_waves = static_cast<int64_t>(n_long_blocks) * (blockDim.x >> 6);
  const int g = (static_cast<int>(threadIdx.x) & (kWave - 1)) / kPieceLanes;
  for (int64_t w = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block(); w < total; w += n_waves) {
    const uint32_t chunk = static_cast<uint32_t>(w / pps);
    const int t = static_cast<int>(w - static_cast<int64_t>(chunk) * pps);
    const LongChunk c = seg_decode_chunk(begin, long_list, chunk_begin, n_long, chunk);
    const int rows = static_cast<int>(c.s1 - c.s0);
    const int pc = t * (kPieceLanes * EV) + sub * EV;
    float acc[EV];
#pragma unroll
    for (int i = 0; i < EV; ++i) acc[i] = 0.f;
    accumulate(static_cast<int64_t>(c.s0) + g, (rows - g + kGroups - 1) / kGroups, kGroups, pc, acc);
#pragma unroll
    for (int i = 0; i < EV; ++i) acc[i] = add_across_rows(acc[i]);
    if (g == 0) store_vec<float, EV>(partial, static_cast<int64_t>(chunk) * slice_w + pc, acc);
  }
}

// Long latents of the piece reduction, second step: out[f, slice] = sum of the latent's chunk
// partials in a fixed order.  One wavefront per (long latent, 64-column piece of the fp32
// partials); its four groups take every fourth chunk and are added up as above.  `block` of
// `n_blocks` blocks of 256 threads share the work (a launch of its own, or the leading blocks of
// the next slice's training-step launch).
template <typename GT>
__device__ __forceinline__ void seg_piece_finalize_body(
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const float *__restrict__ partial,
    void *__restrict__ out, const float *__restrict__ scale, int pieces, int col0, int slice_w, int D,
    int update, unsigned block, unsigned n_blocks) {
  constexpr int EV = 4, U = 4, kGroups = kWave / kPieceLanes;
  const int lane = lane_id();
  const int sub = lane & (kPieceLanes - 1), g = lane / kPieceLanes;
  const uint32_t n_long = *long_count;
  const int64_t total = static_cast<int64_t>(n_long) * pieces;
  const int64_t n_waves = static_cast<int64_t>(n_blocks) * (blockDim.x >> 6);
  for (int64_t w = static_cast<int64_t>(block) * (blockDim.x >> 6) + wave_in_block(); w < total; w += n_waves) {
    const uint32_t i = static_cast<uint32_t>(w / pieces);
    const int t = static_cast<int>(w - static_cast<int64_t>(i) * pieces);
    const int pc = t * (kPieceLanes * EV) + sub * EV;
    const int d0 = col0 + pc;
    const uint32_t c0 = chunk_begin[i], c1 = chunk_begin[i + 1];
    const int n = (static_cast<int>(c1 - c0) - g + kGroups - 1) / kGroups;
    const float *row = partial + (static_cast<int64_t>(c0) + g) * slice_w + pc;
    const int64_t stride = static_cast<int64_t>(kGroups) * slice_w;
    float acc[EV] = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; __any(j < n); j += U) {
      vec_t<float, EV> raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        raw[u] = vec_t<float, EV>{};
        if (j + u < n) raw[u] = *reinterpret_cast<const vec_t<float, EV> *>(row + (j + u) * stride);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int k = 0; k < EV; ++k) acc[k] += raw[u][k];
    }
#pragma unroll
    for (int k = 0; k < EV; ++k) acc[k] = add_across_rows(acc[k]);
    if (scale) {
      const float gs = scale[0];
#pragma unroll
      for (int k = 0; k < EV; ++k) acc[k] *= gs;
    }
    if (g == 0 && d0 < D) {
      const int64_t o = static_cast<int64_t>(long_list[i]) * D + d0;
      if (update) {  // out is the weight matrix: subtract the (scaled) sum from it
        float w[EV];
        load_vec<GT, EV>(out, o, w);
#pragma unroll
        for (int k = 0; k < EV; ++k) acc[k] = w[k] - acc[k];
      }
      store_vec<GT, EV>(out, o, acc);
    }
  }
}

template <typename GT>
__global__ __launch_bounds__(256) void seg_reduce_piece_finalize_kernel(
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const float *__restrict__ partial,
    void *__restrict__ out, const float *__restrict__ scale, int pieces, int col0, int slice_w, int D,
    int update) {
  seg_piece_finalize_body<GT>(long_count, long_list, chunk_begin, partial, out, scale, pieces, col0, slice_w, D, update,
                              blockIdx.x, gridDim.x);
}

// Long latents, second step of the reduction by tiles: out[f, slice] = sum of the latent's chunk
// partials, in chunk order.
template <typename GT, int VEC, int U>
__device__ __forceinline__ void seg_long_finalize_body(
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const float *__restrict__ partial,
    void *__restrict__ out, const float *__restrict__ scale, int tps, int col0, int slice_w, int D,
    unsigned block, unsigned n_blocks) {
  const int lane = lane_id();
  const uint32_t n_long = *long_count;
  const int64_t total = static_cast<int64_t>(n_long) * tps;
  const int64_t n_waves = static_cast<int64_t>(n_blocks) * (blockDim.x >> 6);
  for (int64_t w = static_cast<int64_t>(block) * (blockDim.x >> 6) + wave_in_block(); w < total;
       w += n_waves) {
    const uint32_t i = static_cast<uint32_t>(w / tps);
    const int t = static_cast<int>(w - static_cast<int64_t>(i) * tps);
    const int pc = t * (kWave * VEC) + lane * VEC;
    const int d0 = col0 + pc;
    const uint32_t c0 = chunk_begin[i], c1 = chunk_begin[i + 1];
    float acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = 0.f;
    accumulate_rows_by4<float, VEC, U>(partial, c0, static_cast<int>(c1 - c0), slice_w, pc, acc);
    if (scale) {
      const float g = scale[0];
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[k] *= g;
    }
    if (d0 < D) store_vec<GT, VEC>(out, static_cast<int64_t>(long_list[i]) * D + d0, acc);
  }
}

template <typename GT, int VEC, int U>
__global__ __launch_bounds__(256) void seg_reduce_long_finalize_kernel(
    const uint32_t *__restrict__ long_count, const uint32_t *__restrict__ long_list,
    const uint32_t *__restrict__ chunk_begin, const float *__restrict__ partial,
    void *__restrict__ out, const float *__restrict__ scale, int tps, int col0, int slice_w, int D) {
  seg_long_finalize_body<GT, VEC, U>(long_count, long_list, chunk_begin, partial, out, scale, tps, col0, slice_w, D,
                                     blockIdx.x, gridDim.x);
}

// The second step of a slice's hot latents as a parcel that another launch can carry: the
// training-step kernel of the next slice runs it in its leading blocks (it touches neither the
// contributions nor the partial sums, and the reduction that overwrites the partial sums comes after
// it in the stream), which saves a launch per slice.
struct HotFinalize {
  const uint32_t *long_count;
  const uint32_t *long_list;
  const uint32_t *chunk_begin;
  const float *partial;
  void *out;
  const float *scale;
  int mode;   // 0: nothing, 1: pieces of 64 columns, 2: tiles of 256 columns, 3: tiles of 128 columns
  int units;  // pieces or tiles per slice
  int col0, slice_w, D, update;
  unsigned n_blocks;  // blocks of 256 threads that share it
};

template <typename GT>
__device__ __forceinline__ void hot_finalize_run(const HotFinalize &h, unsigned block) {
  if (h.mode == 1)
    seg_piece_finalize_body<GT>(h.long_count, h.long_list, h.chunk_begin, h.partial, h.out, h.scale, h.units, h.col0,
                                h.slice_w, h.D, h.update, block, h.n_blocks);
  else if (h.mode == 2)
    seg_long_finalize_body<GT, 4, 8>(h.long_count, h.long_list, h.chunk_begin, h.partial, h.out, h.scale, h.units,
                                     h.col0, h.slice_w, h.D, block, h.n_blocks);
  else if (h.mode == 3)
    seg_long_finalize_body<GT, 2, 8>(h.long_count, h.long_list, h.chunk_begin, h.partial, h.out, h.scale, h.units,
                                     h.col0, h.slice_w, h.D, block, h.n_blocks);
}

template <typename GT>
__global__ __launch_bounds__(256) void hot_finalize_kernel(HotFinalize h) {
  hot_finalize_run<GT>(h, blockIdx.x);
}

// long_list[0..*long_count) = latents with more than kSegChunk pairs (any order);
// *long_count must be zero on entry.
__global__ void seg_find_long_kernel(const uint32_t *__restrict__ begin, int64_t F,
                                     uint32_t *__restrict__ long_count,
                                     uint32_t *__restrict__ long_list) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t f = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; f < F; f += stride)
    if (begin[f + 1] - begin[f] > static_cast<uint32_t>(kSegChunk))
      long_list[atomicAdd(long_count, 1u)] = static_cast<uint32_t>(f);
}

// chunk_begin[i] = number of chunks of the long latents before long_list[i]
// (chunk_begin[n_long] = total); single block.  Also clears zero_me[0..n_zero) when given (n_zero <= 1024).
__global__ __launch_bounds__(1024) void seg_chunk_table_kernel(const uint32_t *__restrict__ begin,
                                                               const uint32_t *__restrict__ long_count,
                                                               const uint32_t *__restrict__ long_list,
                                                               uint32_t *__restrict__ chunk_begin,
                                                               uint32_t *__restrict__ zero_me, int n_zero) {
  __shared__ uint32_t wave_tot[1024 / kWave];
  __shared__ uint32_t carry_s;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid >> 6;
  // counters of the kernels that follow in the stream (the class histogram and cursors below)
  if (zero_me && tid < n_zero) zero_me[tid] = 0u;
  const uint32_t n_long = *long_count;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (uint32_t base = 0; base < n_long; base += 1024) {
    const uint32_t i = base + tid;
    uint32_t c = 0;
    if (i < n_long) {
      const uint32_t f = long_list[i];
      c = (begin[f + 1] - begin[f] + kSegChunk - 1) / kSegChunk;
    }
    uint32_t inc = c;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t y = __shfl_up(inc, off, kWave);
      if (lane >= off) inc += y;
    }
    if (lane == kWave - 1) wave_tot[wv] = inc;
    __syncthreads();
    uint32_t wave_off = 0;
    for (int w = 0; w < wv; ++w) wave_off += wave_tot[w];
    const uint32_t excl = carry_s + wave_off + inc - c;
    if (i < n_long) chunk_begin[i] = excl;
    __syncthreads();
    if (tid == 1023) carry_s = excl + c;
    __syncthreads();
  }
  if (tid == 0) chunk_begin[n_long] = carry_s;
}

// ---- latents ordered by row count ----------------------------------------------------------
// Where most latents have no pair at all and the rest one or a few (B*K <= 2F, skewed indices), the
// reduction by pieces works from a list of the latents ordered by their number of rows:
//   cls_list[cls_begin[n] .. cls_begin[n+1]) = the latents with exactly n rows, 0 <= n <= kSegChunk
// (any order inside a class; latents with more rows are not listed: they go through the chunked
// path).  Class 0 is zeroed in one pass over whole rows of the output (seg_zero_rows_kernel); the
// groups of lanes of the reduction take four consecutive entries of the classes 1..kSegChunk, which
// nearly always have the same row count, so no load slot is wasted on unequal groups.
// Two launches: a histogram over the classes, then the placement (a counting sort whose cursors
// are advanced once per block and class).  hist, cursor: kSegClasses counters each, zero on entry.
constexpr int kClassPerThread = 8;  // latents per thread of the placement kernel

__global__ __launch_bounds__(256) void seg_class_hist_kernel(const uint32_t *__restrict__ begin, int64_t F,
                                                             uint32_t *__restrict__ hist) {
  __shared__ uint32_t h[kSegClasses];
  for (int t = threadIdx.x; t < kSegClasses; t += 256) h[t] = 0u;
  __syncthreads();
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t f0 = static_cast<int64_t>(blockIdx.x) * blockDim.x; f0 < F; f0 += stride) {  // uniform per block
    const int64_t f = f0 + threadIdx.x;
    uint32_t n = kSegClasses;  // not counted
    if (f < F) n = begin[f + 1] - begin[f];
    // the empty class is the common one: counted per wavefront, not per lane
    const unsigned long long empties = __ballot(n == 0u);
    if (lane_id() == 0 && empties) atomicAdd(&h[0], static_cast<uint32_t>(__popcll(empties)));
    if (n != 0u && n < static_cast<uint32_t>(kSegClasses)) atomicAdd(&h[n], 1u);
  }
  __syncthreads();
  for (int t = threadIdx.x; t < kSegClasses; t += 256)
    if (h[t]) atomicAdd(&hist[t], h[t]);
}

__global__ __launch_bounds__(256) void seg_class_scatter_kernel(const uint32_t *__restrict__ begin, int64_t F,
                                                                const uint32_t *__restrict__ hist,
                                                                uint32_t *__restrict__ cursor,
                                                                uint32_t *__restrict__ cls_begin,
                                                                uint32_t *__restrict__ cls_list) {
  __shared__ uint32_t base[kSegClasses + 1];  // first entry of every class
  __shared__ uint32_t cnt[kSegClasses];       // this block's latents per class, then where they start in the class
  const int tid = threadIdx.x;
  if (tid <= kSegClasses) {
    uint32_t s = 0;
    for (int k = 0; k < tid; ++k) s += hist[k];
    base[tid] = s;
    if (blockIdx.x == 0) cls_begin[tid] = s;
  }
  if (tid < kSegClasses) cnt[tid] = 0u;
  __syncthreads();
  const int64_t f_block = static_cast<int64_t>(blockIdx.x) * (256 * kClassPerThread);
  uint32_t cls[kClassPerThread], rank[kClassPerThread];
#pragma unroll
  for (int i = 0; i < kClassPerThread; ++i) {
    const int64_t f = f_block + i * 256 + tid;
    cls[i] = kSegClasses;  // not listed
    rank[i] = 0u;
    if (f < F) {
      const uint32_t n = begin[f + 1] - begin[f];
      if (n < static_cast<uint32_t>(kSegClasses)) cls[i] = n;
    }
    if (cls[i] < static_cast<uint32_t>(kSegClasses)) rank[i] = atomicAdd(&cnt[cls[i]], 1u);
  }
  __syncthreads();
  if (tid < kSegClasses) {
    const uint32_t c = cnt[tid];
    cnt[tid] = c ? atomicAdd(&cursor[tid], c) : 0u;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kClassPerThread; ++i)
    if (cls[i] < static_cast<uint32_t>(kSegClasses))
      cls_list[base[cls[i]] + cnt[cls[i]] + rank[i]] = static_cast<uint32_t>(f_block + i * 256 + tid);
}

// out[f, 0..D) = 0 for the latents without rows (class 0 of the list): one wavefront per row, EV
// columns per lane like the reduction by pieces (D is a multiple of EV and rows are 16-byte aligned
// wherever that reduction runs).
template <typename PT, typename GT>
__global__ __launch_bounds__(256) void seg_zero_rows_kernel(const uint32_t *__restrict__ cls_begin,
                                                            const uint32_t *__restrict__ cls_list,
                                                            void *__restrict__ out, int D) {
  constexpr int EV = 16 / static_cast<int>(sizeof(typename Traits<PT>::store_t));
  const uint32_t n = cls_begin[1];
  const int lane = lane_id();
  float zero[EV];
#pragma unroll
  for (int i = 0; i < EV; ++i) zero[i] = 0.f;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * (blockDim.x >> 6);
  for (int64_t w = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + wave_in_block(); w < n; w += n_waves) {
    const int64_t row = static_cast<int64_t>(cls_list[w]) * D;
    for (int d = lane * EV; d < D; d += kWave * EV) store_vec<GT, EV, FLEXSAE_REDUCE_NT>(out, row + d, zero);
  }
}

}  // namespace flexsae
