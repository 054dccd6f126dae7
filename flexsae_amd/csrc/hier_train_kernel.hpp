// HierarchicalTopK, forward and reverse walk in one kernel ("training step" kernel).
#pragma once

#include "common.hpp"
#include "segment_kernels.hpp"

namespace flexsae {

// A gathered piece of a weight row (VEC consecutive columns of one lane) kept in raw form.
template <typename WT, int VEC>
struct RowPiece;
template <>
struct RowPiece<float, 2> {
  using raw_t = vec_t<float, 2>;
  static __device__ __forceinline__ void unpack(const raw_t &r, float (&w)[2]) {
    w[0] = r[0];
    w[1] = r[1];
  }
  // hides the value from common-subexpression elimination (see the kernel)
  static __device__ __forceinline__ void launder(raw_t &r) { asm volatile("" : "+v"(r)); }
};
template <>
struct RowPiece<float, 1> {
  using raw_t = float;
  static __device__ __forceinline__ void unpack(const raw_t &r, float (&w)[1]) { w[0] = r; }
  static __device__ __forceinline__ void launder(raw_t &r) { asm volatile("" : "+v"(r)); }
};
template <>
struct RowPiece<bf16_t, 2> {
  using raw_t = uint32_t;
  static __device__ __forceinline__ void unpack(const raw_t &r, float (&w)[2]) {
    w[0] = __uint_as_float(r << 16);
    w[1] = __uint_as_float(r & 0xffff0000u);
  }
  static __device__ __forceinline__ void launder(raw_t &r) { asm volatile("" : "+v"(r)); }
};
template <>
struct RowPiece<f16_t, 2> {
  using raw_t = uint32_t;
  static __device__ __forceinline__ void unpack(const raw_t &r, float (&w)[2]) {
    w[0] = f16_bits_to_f32(static_cast<uint16_t>(r & 0xffffu));
    w[1] = f16_bits_to_f32(static_cast<uint16_t>(r >> 16));
  }
  static __device__ __forceinline__ void launder(raw_t &r) { asm volatile("" : "+v"(r)); }
};

// One wavefront per (tile of the slice, row b), tile-major; a tile is 64*VEC columns and lane l owns
// columns VEC*l .. VEC*l+VEC-1 (VEC = 2: 128-column tiles, 256 bytes of a 16-bit row per gather;
// VEC = 1, for fp32 weights with more than 64 steps: 64-column tiles, again 256 bytes and one
// register per row).  The wavefront issues the gathers of all K row pieces at once (the memory
// pipeline keeps up to 63 of them in flight per wavefront, so a few wavefronts per SIMD cover the
// latency), keeps the pieces in registers -- one register per row for 16-bit weights -- and walks
// them twice:
//   forward  k = 0..K-1 : e += v_k w_k ; loss += e^2             (e starts as bias - target)
//   reverse  k = K-1..0 : S += c e ; P[slot_k] = v_k S ; dvals_k = <w_k, S> ; e -= v_k w_k
// i.e. sae_fwd_kernel and hier_sweep_kernel sharing one gather.  The gradient quantities are
// those of a unit upstream gradient (c = 2/(B*K*D)); the caller scales them afterwards.
// KMAX bounds K at compile time so that the row pieces can live in registers; steps k >= K
// are skipped by uniform branches, or not tested at all when FULL says K == KMAX.  Every block
// of eight steps reduces its eight dvals dot products with one transposed wave reduction.
// Row gathers and contribution stores go through per-row buffer descriptors: their address
// arithmetic runs on the scalar unit, lanes beyond column D read zeros (so their dot products
// vanish), and what such lanes store lands in the padding columns of P, which nobody reads.
// LDSROWS (FULL variants only): the first LDSROWS row pieces are loaded straight into the LDS
// (buffer load with the LDS as destination, one dword per lane) instead of registers, which buys
// one more wavefront per SIMD: 120 instead of 152 registers at 128 steps (four wavefronts, 8 KB of
// LDS each), 216 instead of 276 at 256 steps (two wavefronts, 16 KB each).  Both walks read them
// back with plain LDS loads.  bias - target is fetched before the gathers are issued: the memory
// counter retires in order, so anything issued after them can only be waited for together with
// all of them, and the forward walk could not start while rows are still arriving.
// fin: the second step of the previous slice's hot latents (see HotFinalize), run by the leading blocks
// of the launch into a gradient of the weight's own dtype.
// STREAM: the contributions are stored with the non-temporal hint.  That is the faster choice
// when all of P is written before any of it is read back (it is far larger than the caches);
// when P is one slice that the reduction reads right after this launch, plain stores leave part
// of it in the memory-side cache and the pair of launches is faster.
template <typename WT, typename PT, int KMAX, bool FULL, bool STREAM, int VEC, int LDSROWS = 0>
__global__ __launch_bounds__(256) void hier_train_kernel(
    const int64_t *__restrict__ indices, const void *__restrict__ weight,
    const void *__restrict__ vals, int vals_dtype, const void *__restrict__ bias, int bias_dtype,
    const void *__restrict__ target, int target_dtype, float coef,
    const uint32_t *__restrict__ slot, void *__restrict__ P, float *__restrict__ dv_part,
    float *__restrict__ s_final, int s_final_ld, float *__restrict__ loss_partial,
    int *status_flag, int64_t n_items, int64_t B, int col0, int slice_w, int K, int64_t F, int D, HotFinalize fin) {
  using Piece = RowPiece<WT, VEC>;
  using raw_t = typename Piece::raw_t;
  using S_t = typename Traits<WT>::store_t;
  constexpr int KC = (KMAX + kWave - 1) / kWave;  // 64-step chunks held per lane
  static_assert(KMAX % 8 == 0, "KMAX must be a multiple of 8");
  static_assert(LDSROWS == 0 || (sizeof(raw_t) == 4 && LDSROWS <= KMAX && FULL), "LDS rows hold one dword per lane");
  // the first LDSROWS row pieces live in the LDS (loaded straight into it), the rest in registers
  __shared__ uint32_t lds_rows[LDSROWS > 0 ? (256 / kWave) * LDSROWS * kWave : 1];
  uint32_t *const my_lds = lds_rows + wave_in_block() * (LDSROWS * kWave);
  const int lane = lane_id();
  // the leading blocks finish the hot latents of the previous slice (fin.n_blocks of them; none at the first slice)
  if (blockIdx.x < fin.n_blocks) {
    hot_finalize_run<WT>(fin, blockIdx.x);
    return;
  }
  const int64_t item = static_cast<int64_t>(blockIdx.x - fin.n_blocks) * (blockDim.x >> 6) + wave_in_block();
  if (item >= n_items) return;  // uniform per wavefront
  const int t = static_cast<int>(item / B);
  const int64_t b = item - static_cast<int64_t>(t) * B;
  const int pc = t * (kWave * VEC) + lane * VEC;  // column inside the slice
  const int d0 = col0 + pc;
  const bool active = d0 < D;
  const int dsafe = active ? d0 : 0;
  const int64_t pair0 = b * K;
  // Each phase tests k < K against its own copy of K: sharing the 128 comparison results
  // between the phases costs more (scalar registers spilled into vector lanes) than redoing them.
  auto k_bound = [&]() {
    int kb = K;
    asm volatile("" : "+s"(kb));
    return kb;
  };

  // Everything the row needs before its gathers is requested at once and waited for once: the
  // conversions branch on run-time dtypes, and a wait inside each of them made this a chain of
  // five or six trips to memory, one after the other, before the first gather was issued.
  int my_row[KC], my_slot[KC];
  float my_val[KC], my_dval[KC];
  int64_t idx_bits[KC];
  uint32_t val_bits[KC];
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const int kk = c * kWave + lane;
    const int64_t mine = pair0 + (kk < K ? kk : 0);
    idx_bits[c] = indices[mine];
    val_bits[c] = load_scalar_bits(vals, vals_dtype, mine);
    my_slot[c] = static_cast<int>(slot[mine]);
  }
  // bias - target before the gathers: the memory counter retires in order, so a load issued after
  // the gathers could only be waited for together with all of them
  float e[VEC], tt[VEC], acc[VEC];
  if constexpr (VEC == 2) {
    const PairBits bias_bits = load_pair_bits(bias, bias_dtype, dsafe);
    const PairBits target_bits = load_pair_bits(target, target_dtype, b * D + dsafe);
    pair_from_bits(bias_bits, bias_dtype, e);
    pair_from_bits(target_bits, target_dtype, tt);
  } else {
    static_assert(VEC == 1, "one or two columns per lane");
    const uint32_t bias_bits = load_scalar_bits(bias, bias_dtype, dsafe);
    const uint32_t target_bits = load_scalar_bits(target, target_dtype, b * D + dsafe);
    e[0] = scalar_from_bits(bias_bits, bias_dtype);
    tt[0] = scalar_from_bits(target_bits, target_dtype);
  }
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const int kk = c * kWave + lane;
    int64_t idx = idx_bits[c];
    my_val[c] = scalar_from_bits(val_bits[c], vals_dtype);
    my_dval[c] = 0.f;
    if (kk >= K) {
      idx = 0;
      my_val[c] = 0.f;
      my_slot[c] = 0;
    }
    if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(F)) {
      if (status_flag) atomicOr(status_flag, FLEXSAE_FLAG_INDEX_RANGE);
      idx = 0;
      my_val[c] = 0.f;
    }
    my_row[c] = static_cast<int>(idx);
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    e[i] -= tt[i];
    acc[i] = 0.f;
  }

  // all gathers at once
  raw_t raw[KMAX];
  const uint32_t w_row_bytes = static_cast<uint32_t>(D) * sizeof(S_t);
  const uint32_t w_lane_bytes = static_cast<uint32_t>(d0) * sizeof(S_t);  // beyond the row if !active
  {
    const int kb = k_bound();
    if constexpr (LDSROWS > 0) {
      // The loads into the LDS first, in a loop of their own, then a scheduling barrier: the wait
      // below counts on every one of them having been issued before the first register gather,
      // and nothing else orders the two kinds of load (they carry no dependence on each other).
#pragma unroll
      for (int k = 0; k < LDSROWS; ++k) {
        const uint32_t row = static_cast<uint32_t>(bcast_i32(my_row[k / kWave], k % kWave));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            row_descriptor(weight, row, w_row_bytes),
            (__attribute__((address_space(3))) void *)(my_lds + k * kWave),
            4, w_lane_bytes, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int k = LDSROWS; k < KMAX; ++k) {
      if (FULL || k < kb) {  // uniform
        const uint32_t row = static_cast<uint32_t>(bcast_i32(my_row[k / kWave], k % kWave));
        const auto dw = descriptor_load<sizeof(raw_t)>(row_descriptor(weight, row, w_row_bytes), w_lane_bytes);
        __builtin_memcpy(&raw[k], &dw, sizeof(raw_t));
      }
    }
    if constexpr (LDSROWS > 0) __builtin_amdgcn_sched_barrier(0);  // no gather sinks below the wait either
  }


  if constexpr (LDSROWS > 0) {
    // The compiler does not order LDS reads after the loads that fill the LDS.  The memory counter
    // retires in order (and holds at most 63), so once no more than (loads issued - LDSROWS) are
    // outstanding the first LDSROWS have landed; the memory clobber keeps the reads below.
    static_assert(FULL, "the wait below counts on all KMAX loads having been issued");
    constexpr int kLeft = KMAX - LDSROWS < 63 ? KMAX - LDSROWS : 63;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLeft) : "memory");
  }

  // forward walk
  const int kb_fwd = k_bound();
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    if (FULL || k < kb_fwd) {  // uniform
      const float v = bcast_f32(my_val[k / kWave], k % kWave);
      float w[VEC];
      if constexpr (LDSROWS > 0) {
        if (k < LDSROWS) {
          raw_t rk;
          const uint32_t x = my_lds[k * kWave + lane];
          __builtin_memcpy(&rk, &x, sizeof(raw_t));
          Piece::unpack(rk, w);
        } else {
          Piece::unpack(raw[k], w);
        }
      } else {
        Piece::unpack(raw[k], w);
      }
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        e[i] = fmaf(w[i], v, e[i]);
        acc[i] = fmaf(e[i], e[i], acc[i]);
      }
    }
  }
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < VEC; ++i) lsum += active ? acc[i] : 0.f;
  lsum = wave_sum_lane63(lsum);
  // one partial per (global tile, row); the finalize kernel adds them in a fixed order
  if (lane == kWave - 1) loss_partial[(static_cast<int64_t>(col0 / (kWave * VEC)) + t) * B + b] = lsum;

  // reverse walk, eight steps per dvals reduction
  float S[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) S[i] = 0.f;
  const int kb_rev = k_bound();
  const uint32_t p_row_bytes = static_cast<uint32_t>(slice_w) * sizeof(typename Traits<PT>::store_t);
  const uint32_t p_lane_bytes = static_cast<uint32_t>(pc) * sizeof(typename Traits<PT>::store_t);
#pragma unroll
  for (int k8 = KMAX - 8; k8 >= 0; k8 -= 8) {
    if (FULL || k8 < kb_rev) {  // uniform
      float dots[8];
      raw_t from_lds[8];  // the block's LDS rows, fetched together ahead of their use
      if constexpr (LDSROWS > 0) {
        if (k8 < LDSROWS) {
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const uint32_t x = my_lds[(k8 + u) * kWave + lane];
            __builtin_memcpy(&from_lds[u], &x, sizeof(raw_t));
          }
        }
      }
#pragma unroll
      for (int u = 7; u >= 0; --u) {
        const int k = k8 + u;
        dots[u] = 0.f;
        if (FULL || k < kb_rev) {  // uniform
          const float v = bcast_f32(my_val[k / kWave], k % kWave);
          const uint32_t prow = static_cast<uint32_t>(bcast_i32(my_slot[k / kWave], k % kWave));
          // Without this the compiler reuses the unpacked values of the forward walk, which
          // doubles the registers held across the two walks; re-unpacking costs one op per value.
          raw_t rk;
          if constexpr (LDSROWS > 0) {
            if (k < LDSROWS) {
              rk = from_lds[u];
            } else {
              rk = raw[k];
            }
          } else {
            rk = raw[k];
          }
          Piece::launder(rk);
          float w[VEC], contrib[VEC];
          Piece::unpack(rk, w);
          float dot = 0.f;
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            S[i] = fmaf(coef, e[i], S[i]);
            contrib[i] = S[i] * v;
            dot = fmaf(w[i], S[i], dot);
            e[i] = fmaf(-w[i], v, e[i]);
          }
          vec_t<uint32_t, VEC * sizeof(typename Traits<PT>::store_t) / 4> packed;
          if constexpr (Traits<PT>::dtype == FLEXSAE_BF16) {
            static_assert(VEC == 2, "bf16 contributions are stored as pairs");
            packed[0] = f32x2_to_bf16x2_bits(contrib[0], contrib[VEC - 1]);
          } else {
            static_assert(Traits<PT>::dtype == FLEXSAE_F32, "contributions are staged as bf16 or fp32");
#pragma unroll
            for (int i = 0; i < VEC; ++i) packed[i] = __float_as_uint(contrib[i]);
          }
          descriptor_store<sizeof(packed), STREAM>(row_descriptor(P, prow, p_row_bytes), p_lane_bytes, packed);
          dots[u] = dot;  // zero where the lane is beyond column D: its w is zero
        }
      }
      const float tot = wave_sum8_transposed(dots);  // lane L: total of step k8 + (L & 7)
      if ((lane >> 3) == ((k8 % kWave) >> 3)) my_dval[k8 / kWave] = tot;
    }
  }
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const int kk = c * kWave + lane;
    // this tile's share of dvals; hier_dvals_finalize_kernel adds the tiles up in order
    if (kk < K) dv_part[(static_cast<int64_t>(col0 / (kWave * VEC)) + t) * (B * K) + pair0 + kk] = my_dval[c];
  }
  if (!active) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) S[i] = 0.f;
  }
  store_vec<float, VEC>(s_final, b * s_final_ld + col0 + pc, S);
}

// dst[i] = src[i] * scale[0] (dtype in, same dtype out; dst may be src); used to apply the
// upstream gradient to the unit-gradient results of the training-step kernel.  In place with a
// scale of exactly one, the usual loss.backward(), the kernel returns at once.
template <typename T>
__global__ void scale_kernel(void *dst, const void *src, int64_t n,
                             const float *__restrict__ scale) {
  const float g = scale[0];
  if (dst == src && g == 1.0f) return;  // in place by one: nothing to do
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t n4 = n >> 2;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride) {
    float x[4];
    load_vec<T, 4>(src, i * 4, x);
#pragma unroll
    for (int k = 0; k < 4; ++k) x[k] *= g;
    store_vec<T, 4>(dst, i * 4, x);
  }
  for (int64_t i = (n4 << 2) + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    float x[1];
    load_vec<T, 1>(src, i, x);
    x[0] *= g;
    store_vec<T, 1>(dst, i, x);
  }
}

}  // namespace flexsae
