// HierarchicalTopK training step with privatised accumulators for hot latents.
//
// A latent that many batch rows select (skewed indices: a few latents in most rows) receives one
// contribution per selecting row; staged like the others, each of them is written to memory and
// read back.  Here the kHotMax most frequent latents of the batch get accumulators in the LDS
// instead: a block walks kHotRowsPerBlock rows of one 128-column tile, adds the contributions of
// marked pairs into its accumulators, and writes one partial sum per (block, hot latent) at the
// end -- kHotRowsPerBlock times fewer bytes through the memory fabric for those pairs.
//
// The accumulators are 32-bit integers (fixed point with one exponent per block), added with LDS
// atomics: integer addition is associative, so the sums do not depend on the order in which the
// block's wavefronts arrive, and the result stays bit-reproducible.  The exponent comes from a
// rigorous bound: for row b and every column, |S_j| = c |sum_{k>=j} e_k| <= c sqrt(K sum_k e_k^2)
// (Cauchy-Schwarz; sum_k e_k^2 is the row's loss partial, known after the forward walk), so a
// contribution v_j S_j is below X_b = max_j |v_j| * c * sqrt(K * max over the wavefront's columns of
// sum_k e_k^2) < 2^E_b.  A hot latent occurs at most once per row (latents with a repeated row are
// not marked, see hot_mark_kernel), so an accumulator takes at most kHotRowsPerBlock additions of
// magnitude below 2^E, E the block's exponent: scaled by 2^(22 - E) they are below 2^22 each and
// their sum stays below 2^29.  E = the largest E_b of the block's first rows (one per wavefront)
// plus `headroom`; a later row with E_b > E is walked without its hot pairs, remembered, and
// walked again after the first pass, when the block raises its exponent to the largest one asked
// for (the accumulators are shifted down accordingly).  Which rows are deferred depends only on
// the data, so the result is deterministic either way.
#pragma once

#include "common.hpp"
#include "hier_train_kernel.hpp"
#include "segment_kernels.hpp"

namespace flexsae {

constexpr int kHotMax = 288;            // accumulator rows in the LDS: 288 * 128 columns * 4 bytes = 144 KiB
constexpr int kHotCols = 128;           // columns per tile (two per lane)
constexpr int kHotThreads = 1024;       // one block per compute unit: its LDS holds the accumulators
constexpr int kHotWaves = kHotThreads / kWave;
constexpr int kHotRowsPerBlock = 128;   // fixed: the grouping of the sums must not depend on the slice width
constexpr int kHotRowsPerWave = kHotRowsPerBlock / kHotWaves;
constexpr int kHotRowsLog2 = 7;
static_assert((1 << kHotRowsLog2) == kHotRowsPerBlock, "log2 of the rows per block");
constexpr uint32_t kHotSlotBit = 0x80000000u;  // marks a pair of a hot latent in hslot[]; the low bits are its accumulator row
constexpr uint32_t kHotNone = 0xffffffffu;
constexpr int kHotExpMin = -96;         // exponents are clamped to [kHotExpMin, 127]: 2^(22 - E) stays a normal float

// Control words of the hot-latent tables (one uint32 each).
enum { kHotNHot = 0, kHotNCand = 1, kHotLong2Count = 2, kHotThreshold = 3, kHotDeferred = 4, kHotCtrlWords = 64 };

__device__ __forceinline__ float wave_max_bcast(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));       // lanes whose source does not exist receive 0: the values are >= 0
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  v = fmaxf(v, dpp_move<0x142, 0xa>(v));
  v = fmaxf(v, dpp_move<0x143, 0xc>(v));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ---- which latents are hot -----------------------------------------------------------------
// Candidates: the latents with the most pairs, at most kHotMax of them, taken from the list of
// latents with more than kSegChunk pairs: all with a pair count above T, T the (kHotMax+1)-th
// largest count (found by a radix select over four 8-bit digits), so the choice does not depend on
// the order of that list.  Single block.  cand_list[c] = latent, long_cand[i] = candidate number of
// long_list[i] or kHotNone; clears the counters that the kernels after it advance.
__global__ __launch_bounds__(1024) void hot_select_kernel(const uint32_t *__restrict__ begin,
                                                          const uint32_t *__restrict__ long_count,
                                                          const uint32_t *__restrict__ long_list,
                                                          uint32_t *__restrict__ ctrl,
                                                          uint32_t *__restrict__ cand_list,
                                                          uint32_t *__restrict__ long_cand, uint32_t max_hot) {
  constexpr uint32_t kCached = 8192;  // pair counts kept in the LDS (each costs two dependent loads from memory)
  __shared__ uint32_t hist[256];
  __shared__ uint32_t cnt_lds[kCached];
  __shared__ uint32_t sel_prefix, sel_k, sel_prefix_next, sel_k_next, n_cand_s;
  __shared__ uint32_t wave_tot[4];
  const int tid = threadIdx.x;
  const uint32_t n_long = *long_count;
  for (uint32_t i = tid; i < n_long && i < kCached; i += 1024) {
    const uint32_t f = long_list[i];
    cnt_lds[i] = begin[f + 1] - begin[f];
  }
  __syncthreads();
  auto count_of = [&](uint32_t i) {
    if (i < kCached) return cnt_lds[i];
    const uint32_t f = long_list[i];
    return begin[f + 1] - begin[f];
  };
  uint32_t T = kSegChunk;  // every long latent is a candidate when there are at most max_hot of them
  if (n_long > max_hot) {
    if (tid == 0) {
      sel_prefix = 0;
      sel_k = max_hot + 1;  // the (max_hot+1)-th largest count
    }
    for (int pass = 3; pass >= 0; --pass) {
      if (tid < 256) hist[tid] = 0;
      __syncthreads();
      const uint32_t prefix = sel_prefix;
      const int hi_shift = 8 * (pass + 1);
      for (uint32_t i = tid; i < n_long; i += 1024) {
        const uint32_t c = count_of(i);
        if (pass == 3 || (c >> hi_shift) == (prefix >> hi_shift)) atomicAdd(&hist[(c >> (8 * pass)) & 255u], 1u);
      }
      __syncthreads();
      {
        // the digit d with (entries above d) < k <= (entries above d) + hist[d]: a suffix sum over the
        // 256 bins (shuffles inside each of the four wavefronts that hold them, then their totals);
        // exactly one thread finds itself selected (k is at most the number of entries counted)
        const int lane = tid & (kWave - 1), wv = tid >> 6;
        const uint32_t h = tid < 256 ? hist[tid] : 0u;
        uint32_t sfx = h;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
          const uint32_t y = __shfl_down(sfx, off, kWave);
          if (lane + off < kWave) sfx += y;
        }
        if (lane == 0 && wv < 4) wave_tot[wv] = sfx;
        __syncthreads();
        if (tid < 256) {
          uint32_t above = sfx - h;
          for (int w = wv + 1; w < 4; ++w) above += wave_tot[w];
          const uint32_t k = sel_k;
          if (above < k && k <= above + h) {
            sel_k_next = k - above;
            sel_prefix_next = prefix | (static_cast<uint32_t>(tid) << (8 * pass));
          }
        }
      }
      __syncthreads();
      if (tid == 0) {
        sel_k = sel_k_next;
        sel_prefix = sel_prefix_next;
      }
      __syncthreads();
    }
    T = sel_prefix;
  }
  if (tid == 0) {
    n_cand_s = 0;
    ctrl[kHotNHot] = 0;
    ctrl[kHotLong2Count] = 0;
    ctrl[kHotThreshold] = T;
    ctrl[kHotDeferred] = 0;
  }
  __syncthreads();
  for (uint32_t i = tid; i < n_long; i += 1024) {
    const uint32_t c = count_of(i);
    uint32_t cand = kHotNone;
    if (max_hot > 0 && c > T) {
      cand = atomicAdd(&n_cand_s, 1u);  // at most max_hot by the choice of T
      cand_list[cand] = long_list[i];
    }
    long_cand[i] = cand;
  }
  __syncthreads();
  if (tid == 0) ctrl[kHotNCand] = n_cand_s;
}

// One block per candidate: a candidate none of whose rows holds it twice becomes a hot latent (an
// accumulator then takes at most one addition per row, which the bound on its sums counts on); it
// gets an accumulator row h and its pairs are marked in hslot[].  cand_state[c] = h or kHotNone.
// hslot must hold a copy of slot[] on entry.
__global__ __launch_bounds__(1024) void hot_mark_kernel(const uint32_t *__restrict__ begin,
                                                       const uint32_t *__restrict__ map,
                                                       uint32_t *__restrict__ ctrl,
                                                       const uint32_t *__restrict__ cand_list,
                                                       uint32_t *__restrict__ cand_state,
                                                       uint32_t *__restrict__ hot_list,
                                                       uint32_t *__restrict__ hslot, uint32_t K) {
  __shared__ uint32_t h_s;
  const uint32_t c = blockIdx.x;
  if (c >= ctrl[kHotNCand]) return;  // uniform per block
  const uint32_t f = cand_list[c];
  const uint32_t s0 = begin[f], s1 = begin[f + 1];
  int dup = 0;
  for (uint32_t i = s0 + threadIdx.x; i + 1 < s1; i += blockDim.x)  // the pair ids of a latent ascend
    dup |= (map[i] / K == map[i + 1] / K) ? 1 : 0;
  dup = __syncthreads_or(dup);
  if (threadIdx.x == 0) {
    const uint32_t h = dup ? kHotNone : atomicAdd(&ctrl[kHotNHot], 1u);
    if (!dup) hot_list[h] = f;
    cand_state[c] = h;
    h_s = h;
  }
  __syncthreads();
  const uint32_t h = h_s;
  if (h == kHotNone) return;
  for (uint32_t i = s0 + threadIdx.x; i < s1; i += blockDim.x) hslot[map[i]] = kHotSlotBit | h;
}

// long2_list = the latents with more than kSegChunk pairs that did not become hot (any order):
// what the chunked part of the segment reduction still serves.
__global__ void hot_cold_long_kernel(const uint32_t *__restrict__ long_count,
                                     const uint32_t *__restrict__ long_list,
                                     const uint32_t *__restrict__ long_cand,
                                     const uint32_t *__restrict__ cand_state, uint32_t *__restrict__ ctrl,
                                     uint32_t *__restrict__ long2_list) {
  const uint32_t n_long = *long_count;
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n_long; i += stride) {
    const uint32_t c = long_cand[i];
    const bool hot = c != kHotNone && cand_state[c] != kHotNone;
    if (!hot) long2_list[atomicAdd(&ctrl[kHotLong2Count], 1u)] = long_list[i];
  }
}

// out[0] = latents with more than kSegChunk pairs, out[1] = their pairs in chunks of kSegChunk,
// out[2] = latents without a pair.  One block (the pair list's segment starts are read once:
// 4 bytes per latent); `out` may be pinned host memory.
__global__ __launch_bounds__(1024) void pair_stats_kernel(const uint32_t *__restrict__ begin, int64_t F,
                                                          const uint32_t *__restrict__ long_count,
                                                          const uint32_t *__restrict__ chunk_begin,
                                                          uint32_t *__restrict__ out) {
  __shared__ uint32_t wave_tot[1024 / kWave];
  uint32_t mine = 0;  // per lane, so that the loads of several rounds are in flight together
#pragma unroll 8
  for (int64_t f = threadIdx.x; f < F; f += 1024) mine += begin[f + 1] == begin[f] ? 1u : 0u;
  uint32_t empty = mine;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) empty += static_cast<uint32_t>(__shfl_xor(static_cast<int>(empty), off, kWave));
  if (lane_id() == 0) wave_tot[threadIdx.x >> 6] = empty;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
    for (int w = 0; w < 1024 / kWave; ++w) total += wave_tot[w];
    const uint32_t n_long = *long_count;
    out[0] = n_long;
    out[1] = chunk_begin[n_long];
    out[2] = total;
  }
}

// ---- second step of the hot latents ---------------------------------------------------------
// out[f, tile] = sum over the row blocks of the block partials of hot latent f, in block order
// (four running sums, combined as (s0 + s1) + (s2 + s3)).  The partials keep the accumulators'
// layout: [tile][row block][accumulator row][2][64], element (i, l) being column 2 l + i of the tile.
struct HotBlockFinalize {
  const uint32_t *ctrl;       // null: nothing to do
  const uint32_t *hot_list;
  const float *partial;
  void *out;
  const float *scale;
  int n_tiles, n_row_blocks, col0, D, update;
};

template <typename GT>
__device__ __forceinline__ void hot_block_finalize_run(const HotBlockFinalize &h, unsigned block, unsigned n_blocks) {
  if (!h.ctrl) return;
  const int lane = lane_id();
  const uint32_t n_hot = h.ctrl[kHotNHot];
  const int64_t total = static_cast<int64_t>(n_hot) * h.n_tiles;
  const int64_t n_waves = static_cast<int64_t>(n_blocks) * (blockDim.x >> 6);
  for (int64_t w = static_cast<int64_t>(block) * (blockDim.x >> 6) + wave_in_block(); w < total; w += n_waves) {
    const uint32_t hh = static_cast<uint32_t>(w / h.n_tiles);
    const int t = static_cast<int>(w - static_cast<int64_t>(hh) * h.n_tiles);
    const float *p = h.partial + (static_cast<int64_t>(t) * h.n_row_blocks * kHotMax + hh) * kHotCols + lane;
    const int64_t stride = static_cast<int64_t>(kHotMax) * kHotCols;
    float part[4][2];
#pragma unroll
    for (int g = 0; g < 4; ++g) part[g][0] = part[g][1] = 0.f;
    for (int rb = 0; rb < h.n_row_blocks; rb += 4) {
      float x[4][2];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        x[u][0] = x[u][1] = 0.f;
        if (rb + u < h.n_row_blocks) {  // uniform
          x[u][0] = p[(rb + u) * stride];
          x[u][1] = p[(rb + u) * stride + kWave];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        part[u][0] += x[u][0];
        part[u][1] += x[u][1];
      }
    }
    float acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) acc[i] = (part[0][i] + part[1][i]) + (part[2][i] + part[3][i]);
    if (h.scale) {
      const float g = h.scale[0];
      acc[0] *= g;
      acc[1] *= g;
    }
    const int d0 = h.col0 + t * kHotCols + 2 * lane;
    if (d0 < h.D) {
      const int64_t o = static_cast<int64_t>(h.hot_list[hh]) * h.D + d0;
      if (h.update) {  // out is the weight matrix: subtract the (scaled) sum from it
        float wv[2];
        load_vec<GT, 2>(h.out, o, wv);
        acc[0] = wv[0] - acc[0];
        acc[1] = wv[1] - acc[1];
      }
      store_vec<GT, 2>(h.out, o, acc);
    }
  }
}

template <typename GT>
__global__ __launch_bounds__(256) void hot_block_finalize_kernel(HotBlockFinalize h) {
  hot_block_finalize_run<GT>(h, blockIdx.x, gridDim.x);
}

// ---- the training-step kernel with hot-latent accumulators ---------------------------------
// One block of kHotThreads per (row block of kHotRowsPerBlock rows, 128-column tile of the slice):
// blockIdx = row block * n_tiles + tile, so that with the usual round-robin placement the blocks
// of one tile share an L2.  Wavefront w walks rows row block * 128 + i * 16 + w, i = 0..7, each
// exactly like hier_train_kernel (all K gathers at once, forward walk, reverse walk), except that
// a pair whose hslot has the hot bit adds its contribution to the block's accumulator row instead
// of storing it.  The leading work of every block is its share of the previous slice's second
// steps (fin, hfin); the last is the flush of its accumulators to
// hot_partial[tile][row block][accumulator row][2][64].
// OFF32: the weight matrix is smaller than 4 GiB, the slice of contributions smaller than 2 GiB
// and D a whole number of tiles.  Rows and contribution rows are then addressed through one
// descriptor each plus a 32-bit byte offset that the lanes compute for all steps of a row at once
// (lane k: step k), so a step's gather and store need one lane read each and no scalar address
// arithmetic; for a hot pair the same word carries the hot bit and the byte offset of its
// accumulator row.  This kernel is bound by the instructions it issues, not by its bytes.
template <typename WT, typename PT, int KMAX, bool FULL, bool OFF32>
__global__ __launch_bounds__(kHotThreads) void hier_train_hot_kernel(
    const int64_t *__restrict__ indices, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const void *__restrict__ bias, int bias_dtype,
    const void *__restrict__ target, int target_dtype, float coef,
    const uint32_t *__restrict__ hslot, void *__restrict__ P, float *__restrict__ dv_part,
    float *__restrict__ colsum_part, float *__restrict__ loss_partial,
    int *status_flag, int64_t B, int n_tiles, int n_row_blocks, int col0, int slice_w, int K, int64_t F, int D,
    uint32_t *__restrict__ ctrl, float *__restrict__ hot_partial, int headroom, HotFinalize fin,
    HotBlockFinalize hfin) {
  constexpr int VEC = 2;
  using Piece = RowPiece<WT, VEC>;
  using raw_t = typename Piece::raw_t;
  using S_t = typename Traits<WT>::store_t;
  static_assert(sizeof(raw_t) == 4 && KMAX <= kWave && KMAX % 8 == 0, "16-bit weights, at most 64 steps");
  __shared__ int acc_lds[kHotMax * kHotCols];
  __shared__ int exp_lds[kHotWaves];
  __shared__ float colsum_lds[kHotWaves][kHotCols];  // each wavefront's sum of S over its rows (for dbias)
  __shared__ int ask_lds;   // the largest exponent a deferred row asked for
  __shared__ int bad_lds;   // a row's bound was not finite
  const int lane = lane_id();
  const int wv = wave_in_block();

  // this block's share of the previous slice's second steps
  hot_finalize_run<WT>(fin, blockIdx.x);
  hot_block_finalize_run<WT>(hfin, blockIdx.x, gridDim.x);

  const int t = static_cast<int>(blockIdx.x % static_cast<unsigned>(n_tiles));
  const int rb = static_cast<int>(blockIdx.x / static_cast<unsigned>(n_tiles));
  const int n_hot = static_cast<int>(ctrl[kHotNHot] < static_cast<uint32_t>(kHotMax) ? ctrl[kHotNHot] : kHotMax);
  for (int i = threadIdx.x; i < n_hot * kHotCols; i += kHotThreads) acc_lds[i] = 0;
  for (int i = threadIdx.x; i < kHotWaves * kHotCols; i += kHotThreads) (&colsum_lds[0][0])[i] = 0.f;
  if (threadIdx.x == 0) {
    ask_lds = kHotExpMin - 1;
    bad_lds = 0;
  }
  __syncthreads();

  const int pc = t * kHotCols + lane * VEC;  // column inside the slice
  const int d0 = col0 + pc;
  const bool active = d0 < D;
  const int dsafe = active ? d0 : 0;
  auto k_bound = [&]() {
    int kb = K;
    asm volatile("" : "+s"(kb));
    return kb;
  };
  const uint32_t w_row_bytes = static_cast<uint32_t>(D) * sizeof(S_t);
  const uint32_t w_lane_bytes = static_cast<uint32_t>(d0) * sizeof(S_t);  // beyond the row if !active
  const uint32_t p_row_bytes = static_cast<uint32_t>(slice_w) * sizeof(typename Traits<PT>::store_t);
  const uint32_t p_lane_bytes = static_cast<uint32_t>(pc) * sizeof(typename Traits<PT>::store_t);
  const __amdgpu_buffer_rsrc_t w_all = matrix_descriptor(weight, static_cast<uint64_t>(F) * w_row_bytes);
  const __amdgpu_buffer_rsrc_t p_all = matrix_descriptor(P, static_cast<uint64_t>(B) * K * p_row_bytes);
  int *const my_acc = acc_lds + lane;  // element (i, lane) of accumulator row h is my_acc[h * 128 + i * 64]

  int exp_block = kHotExpMin;   // the block's exponent E (uniform over the block once set)
  float qscale = 0.f;           // 2^(22 - E)
  uint32_t deferred = 0;        // rows of this wavefront left for the second pass
  int ask = kHotExpMin - 1;

#pragma unroll 1
  for (int pass = 0; pass < 2; ++pass) {
    uint32_t todo = pass == 0 ? (1u << kHotRowsPerWave) - 1u : deferred;
    bool calibrate = pass == 0;
#pragma unroll 1
    while (todo != 0) {  // uniform
      const int i = __builtin_ctz(todo);
      todo &= todo - 1;
      const int64_t b = static_cast<int64_t>(rb) * kHotRowsPerBlock + i * kHotWaves + wv;
      const bool valid = b < B;  // uniform
      const int64_t pair0 = b * K;

      int my_row = 0, my_slot = 0;
      float my_val = 0.f, my_dval = 0.f;
      float e[VEC], acc[VEC];
      raw_t raw[KMAX];
      int exp_row = kHotExpMin;
      if (valid) {
        // everything the row needs before its gathers, requested at once and waited for once: a load
        // issued after the stores of the row before it returns after them, so every separate wait here
        // would cost a trip to memory of its own
        const int64_t mine = pair0 + (lane < K ? lane : 0);
        int64_t idx = indices[mine];
        const uint32_t val_bits = load_scalar_bits(vals, vals_dtype, mine);
        my_slot = static_cast<int>(hslot[mine]);
        const PairBits bias_bits = load_pair_bits(bias, bias_dtype, dsafe);
        const PairBits target_bits = load_pair_bits(target, target_dtype, b * D + dsafe);
        my_val = scalar_from_bits(val_bits, vals_dtype);
        if (lane >= K) {
          idx = 0;
          my_val = 0.f;
          my_slot = 0;
        }
        if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(F)) {
          if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
          idx = 0;
          my_val = 0.f;
        }
        my_row = static_cast<int>(idx);
        if constexpr (OFF32) {
          // byte offsets instead of row numbers: of the weight row, and of the contribution row or
          // (hot bit kept) of the accumulator row
          my_row = static_cast<int>(static_cast<uint32_t>(my_row) * w_row_bytes);
          const uint32_t sl = static_cast<uint32_t>(my_slot);
          my_slot = static_cast<int>((sl & kHotSlotBit) ? (kHotSlotBit | ((sl & ~kHotSlotBit) * (kHotCols * 4u)))
                                                        : sl * p_row_bytes);
        }
        float tt[VEC];
        pair_from_bits(bias_bits, bias_dtype, e);
        pair_from_bits(target_bits, target_dtype, tt);
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          e[c] -= tt[c];
          acc[c] = 0.f;
        }
        {
          const int kb = k_bound();
#pragma unroll
          for (int k = 0; k < KMAX; ++k) {
            if (FULL || k < kb) {  // uniform
              const uint32_t row = static_cast<uint32_t>(bcast_i32(my_row, k));
              const auto dw = OFF32 ? descriptor_load_at<sizeof(raw_t)>(w_all, w_lane_bytes, row)
                                    : descriptor_load<sizeof(raw_t)>(row_descriptor(weight, row, w_row_bytes), w_lane_bytes);
              __builtin_memcpy(&raw[k], &dw, sizeof(raw_t));
            }
          }
          // all gathers are in flight before the walk waits for the first of them: left to itself
          // the scheduler starts the walk's first step between the first two gathers
          __builtin_amdgcn_sched_barrier(0);
        }
        // forward walk
        const int kb_fwd = k_bound();
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          if (FULL || k < kb_fwd) {  // uniform
            const float v = bcast_f32(my_val, k);
            float w[VEC];
            Piece::unpack(raw[k], w);
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
              e[c] = fmaf(w[c], v, e[c]);
              acc[c] = fmaf(e[c], e[c], acc[c]);
            }
          }
        }
        float lsum = 0.f;
#pragma unroll
        for (int c = 0; c < VEC; ++c) lsum += active ? acc[c] : 0.f;
        lsum = wave_sum_lane63(lsum);
        if (lane == kWave - 1) loss_partial[(static_cast<int64_t>(col0 / kHotCols) + t) * B + b] = lsum;
        // the row's bound on its contributions: max |v| * c * sqrt(K * max over the columns of sum_k e_k^2)
        const float acc_max = wave_max_bcast(fmaxf(acc[0], acc[1]));
        const float v_max = wave_max_bcast(fabsf(my_val));
        const float bound = v_max * coef * __builtin_sqrtf(static_cast<float>(K) * acc_max);
        if (!(bound <= 3.0e38f)) {  // infinity or NaN in the inputs: the block's partial sums are made NaN
          if (lane == 0) bad_lds = 1;
        } else if (bound > 0.f) {
          int ex;
          (void)__builtin_frexpf(bound, &ex);  // bound < 2^ex
          exp_row = ex < kHotExpMin ? kHotExpMin : ex;
        }
      }
      if (calibrate) {  // the first row of every wavefront of the block sets the block's exponent
        calibrate = false;
        if (lane == 0) exp_lds[wv] = exp_row;
        __syncthreads();
        int ex = kHotExpMin;
#pragma unroll
        for (int w2 = 0; w2 < kHotWaves; ++w2) ex = exp_lds[w2] > ex ? exp_lds[w2] : ex;
        ex += headroom;
        exp_block = ex < kHotExpMin ? kHotExpMin : (ex > 127 ? 127 : ex);
        exp_block = __builtin_amdgcn_readfirstlane(exp_block);
        qscale = __builtin_ldexpf(1.0f, 22 - exp_block);
      }
      const bool hot_ok = exp_row <= exp_block;  // uniform
      if (pass == 0 && !hot_ok) {
        deferred |= 1u << i;
        ask = exp_row > ask ? exp_row : ask;
      }
      if (!valid) continue;

      // reverse walk, eight steps per dvals reduction
      float S[VEC];
#pragma unroll
      for (int c = 0; c < VEC; ++c) S[c] = 0.f;
      const int kb_rev = k_bound();
#pragma unroll
      for (int k8 = KMAX - 8; k8 >= 0; k8 -= 8) {
        if (FULL || k8 < kb_rev) {  // uniform
          float dots[8];
#pragma unroll
          for (int u = 7; u >= 0; --u) {
            const int k = k8 + u;
            dots[u] = 0.f;
            if (FULL || k < kb_rev) {  // uniform
              const float v = bcast_f32(my_val, k);
              const uint32_t prow = static_cast<uint32_t>(bcast_i32(my_slot, k));
              // (laundered in place, its last use: keeps the unpacked values of the forward walk from
              // being kept alive across the two walks, at no copy)
              Piece::launder(raw[k]);
              float w[VEC], contrib[VEC];
              Piece::unpack(raw[k], w);
              float dot = 0.f;
#pragma unroll
              for (int c = 0; c < VEC; ++c) {
                S[c] = fmaf(coef, e[c], S[c]);
                contrib[c] = S[c] * v;
                dot = fmaf(w[c], S[c], dot);
                e[c] = fmaf(-w[c], v, e[c]);
              }
              const bool is_hot = (prow & kHotSlotBit) != 0;  // uniform: a pair of a hot latent
              if (is_hot && hot_ok) {
                int *a = OFF32 ? reinterpret_cast<int *>(reinterpret_cast<char *>(my_acc) + (prow & ~kHotSlotBit))
                               : my_acc + (prow & ~kHotSlotBit) * kHotCols;
#pragma unroll
                for (int c = 0; c < VEC; ++c) {
                  // round(contrib * 2^(22 - E)) as an integer: |.| <= 2^22, so adding 1.5 * 2^23 leaves it in
                  // the low mantissa bits (round to nearest even), one instruction instead of three
                  const int q = __float_as_int(fmaf(contrib[c], qscale, 12582912.0f)) - 0x4B400000;
                  __hip_atomic_fetch_add(a + c * kWave, q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
              } else if (!is_hot) {
                vec_t<uint32_t, VEC * sizeof(typename Traits<PT>::store_t) / 4> packed;
                if constexpr (Traits<PT>::dtype == FLEXSAE_BF16) {
                  packed[0] = f32x2_to_bf16x2_bits(contrib[0], contrib[1]);
                } else {
                  static_assert(Traits<PT>::dtype == FLEXSAE_F32, "contributions are staged as bf16 or fp32");
#pragma unroll
                  for (int c = 0; c < VEC; ++c) packed[c] = __float_as_uint(contrib[c]);
                }
                if constexpr (OFF32) descriptor_store_at<sizeof(packed), false>(p_all, p_lane_bytes, prow, packed);
                else descriptor_store<sizeof(packed), false>(row_descriptor(P, prow, p_row_bytes), p_lane_bytes, packed);
              }
              dots[u] = dot;  // zero where the lane is beyond column D: its w is zero
            }
          }
          const float tot = wave_sum8_transposed(dots);  // lane L: total of step k8 + (L & 7)
          if ((lane >> 3) == (k8 >> 3)) my_dval = tot;
        }
      }
      // this tile's share of dvals; the epilogue adds the tiles up in order.  (A uniform base plus a
      // lane number formed here: kept across the walks, the lane's 64-bit address is spilled, and
      // its reload waits for every store of the row.)
      {
        uint32_t z = 0;
        asm volatile("" : "+s"(z));  // a zero the optimiser cannot see through
        const uint32_t ln = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
        float *const dv_row = dv_part + (static_cast<int64_t>(col0 / kHotCols) + t) * (B * K) + pair0;
        if (ln < static_cast<uint32_t>(K)) dv_row[ln] = my_dval;
      }
      // the row's final S (the gradient of its reconstruction) is only needed summed over the rows,
      // for dbias: summed here per wavefront in row order, the wavefronts' sums added in order at
      // the end of the block, the blocks' sums in order by colsum_final_kernel -- a fixed order that
      // does not depend on the slice width (a deferred row is walked twice with the same S: counted
      // in the first pass).  The plain step sums the same values in another fixed order (runs of 64
      // rows), so dbias may differ from its in the last bits.
      if (pass == 0) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) colsum_lds[wv][lane * VEC + c] += S[c];
      }
    }
    if (pass == 0) {
      // rows left for the second pass anywhere in the block: raise the block's exponent to the
      // largest one they ask for and shift the accumulators down by the difference
      if (ask >= kHotExpMin && lane == 0) {
        atomicMax(&ask_lds, ask);
        atomicAdd(&ctrl[kHotDeferred], static_cast<uint32_t>(__builtin_popcount(deferred)));  // a statistic
      }
      __syncthreads();
      const int want = ask_lds;  // uniform over the block
      if (want > exp_block) {
        const int shift = want - exp_block;
        for (int j = threadIdx.x; j < n_hot * kHotCols; j += kHotThreads) {
          const int a = acc_lds[j];
          acc_lds[j] = shift >= 31 ? 0 : ((a >> (shift - 1)) + 1) >> 1;  // rounded to nearest (arithmetic shifts)
        }
        exp_block = want;
        qscale = __builtin_ldexpf(1.0f, 22 - exp_block);
        __syncthreads();
      }
    }
  }
  __syncthreads();
  // flush: the block's partial sums of the hot latents, as floats
  {
    const float unscale = bad_lds ? __builtin_nanf("") : __builtin_ldexpf(1.0f, exp_block - 22);
    float *dst = hot_partial + (static_cast<int64_t>(t) * n_row_blocks + rb) * (static_cast<int64_t>(kHotMax) * kHotCols);
    for (int j = threadIdx.x; j < n_hot * kHotCols; j += kHotThreads) dst[j] = static_cast<float>(acc_lds[j]) * unscale;
  }
  // stage 1 of dbias for this block's rows and columns: the wavefronts' sums in order
  if (threadIdx.x < kHotCols) {
    const int d = col0 + t * kHotCols + static_cast<int>(threadIdx.x);
    if (d < D) {
      float sum = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < kHotWaves; ++w2) sum += colsum_lds[w2][threadIdx.x];
      colsum_part[static_cast<int64_t>(rb) * D + d] = sum;
    }
  }
}

}  // namespace flexsae
