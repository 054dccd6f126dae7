// Device-side helpers shared by all kernels: dtype conversion, vector loads/stores,
// wavefront (64-lane) reductions.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flexsae_amd.h"

namespace flexsae {

constexpr int kWave = 64;

// Storage tags for the 16-bit element types (the bits are handled by hand so the
// code does not depend on any header's bf16/fp16 class).
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// round-to-nearest-even through the hardware converter (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  const __bf16 h = static_cast<__bf16>(f);
  uint16_t u;
  __builtin_memcpy(&u, &h, 2);
  return u;
}

// two floats -> two bf16 packed in one dword (element 0 in the low half), one instruction
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 x = {lo, hi};
  const bf16x2 y = __builtin_convertvector(x, bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &y, 4);
  return u;
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  _Float16 x;
  __builtin_memcpy(&x, &h, 2);
  return static_cast<float>(x);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 x = static_cast<_Float16>(f);
  uint16_t h;
  __builtin_memcpy(&h, &x, 2);
  return h;
}

template <typename T>
struct Traits;
template <>
struct Traits<float> {
  using store_t = float;
  static constexpr int dtype = FLEXSAE_F32;
  __device__ static __forceinline__ float up(float v) { return v; }
  __device__ static __forceinline__ float down(float v) { return v; }
};
template <>
struct Traits<bf16_t> {
  using store_t = uint16_t;
  static constexpr int dtype = FLEXSAE_BF16;
  __device__ static __forceinline__ float up(uint16_t v) { return bf16_bits_to_f32(v); }
  __device__ static __forceinline__ uint16_t down(float v) { return f32_to_bf16_bits(v); }
};
template <>
struct Traits<f16_t> {
  using store_t = uint16_t;
  static constexpr int dtype = FLEXSAE_F16;
  __device__ static __forceinline__ float up(uint16_t v) { return f16_bits_to_f32(v); }
  __device__ static __forceinline__ uint16_t down(float v) { return f32_to_f16_bits(v); }
};

template <typename S, int N>
using vec_t = S __attribute__((ext_vector_type(N)));

// o[0..VEC) = float(base[off .. off+VEC)); (base+off) must be aligned to VEC elements.
template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const void *base, int64_t off, float (&o)[VEC]) {
  using S = typename Traits<T>::store_t;
  const S *p = static_cast<const S *>(base) + off;
  if constexpr (VEC == 1) {
    o[0] = Traits<T>::up(*p);
  } else {
    const vec_t<S, VEC> v = *reinterpret_cast<const vec_t<S, VEC> *>(p);
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = Traits<T>::up(v[i]);
  }
}

// NT: non-temporal (streaming) store, for data that is written once and not read again soon,
// so that it does not push reusable lines out of the L2.
template <typename T, int VEC, bool NT = false>
__device__ __forceinline__ void store_vec(void *base, int64_t off, const float (&x)[VEC]) {
  using S = typename Traits<T>::store_t;
  S *p = static_cast<S *>(base) + off;
  auto put = [](auto *dst, auto v) {
    if constexpr (NT) __builtin_nontemporal_store(v, dst); else *dst = v;
  };
  if constexpr (Traits<T>::dtype == FLEXSAE_BF16 && VEC == 2) {
    put(reinterpret_cast<uint32_t *>(p), f32x2_to_bf16x2_bits(x[0], x[1]));
  } else if constexpr (Traits<T>::dtype == FLEXSAE_BF16 && VEC > 2) {
    vec_t<uint32_t, VEC / 2> v;
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) v[i] = f32x2_to_bf16x2_bits(x[2 * i], x[2 * i + 1]);
    put(reinterpret_cast<vec_t<uint32_t, VEC / 2> *>(p), v);
  } else if constexpr (VEC == 1) {
    put(p, Traits<T>::down(x[0]));
  } else {
    vec_t<S, VEC> v;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = Traits<T>::down(x[i]);
    put(reinterpret_cast<vec_t<S, VEC> *>(p), v);
  }
}

// One element of a tensor whose dtype is only known at run time (vals, bias, target:
// small tensors next to the gathered weight rows).
__device__ __forceinline__ float load_scalar(const void *base, int dtype, int64_t i) {
  if (dtype == FLEXSAE_F32) return static_cast<const float *>(base)[i];
  const uint16_t h = static_cast<const uint16_t *>(base)[i];
  return dtype == FLEXSAE_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

// The same in two halves, for code that wants several such loads in flight before it waits for
// any of them: the bits as loaded (16-bit types in the low half), and their conversion.
__device__ __forceinline__ uint32_t load_scalar_bits(const void *base, int dtype, int64_t i) {
  if (dtype == FLEXSAE_F32) return static_cast<const uint32_t *>(base)[i];
  return static_cast<const uint16_t *>(base)[i];
}
__device__ __forceinline__ float scalar_from_bits(uint32_t bits, int dtype) {
  if (dtype == FLEXSAE_F32) return __uint_as_float(bits);
  const uint16_t h = static_cast<uint16_t>(bits);
  return dtype == FLEXSAE_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}
// two consecutive elements starting at an even element offset (the tensor's base 8-byte aligned)
struct PairBits {
  uint32_t lo, hi;
};
__device__ __forceinline__ PairBits load_pair_bits(const void *base, int dtype, int64_t off) {
  PairBits r;
  if (dtype == FLEXSAE_F32) {
    const uint2 v = *reinterpret_cast<const uint2 *>(static_cast<const uint32_t *>(base) + off);
    r.lo = v.x;
    r.hi = v.y;
  } else {
    r.lo = *reinterpret_cast<const uint32_t *>(static_cast<const uint16_t *>(base) + off);
    r.hi = 0u;
  }
  return r;
}
__device__ __forceinline__ void pair_from_bits(const PairBits &r, int dtype, float (&o)[2]) {
  if (dtype == FLEXSAE_F32) {
    o[0] = __uint_as_float(r.lo);
    o[1] = __uint_as_float(r.hi);
  } else if (dtype == FLEXSAE_BF16) {
    o[0] = __uint_as_float(r.lo << 16);
    o[1] = __uint_as_float(r.lo & 0xffff0000u);
  } else {
    o[0] = f16_bits_to_f32(static_cast<uint16_t>(r.lo));
    o[1] = f16_bits_to_f32(static_cast<uint16_t>(r.lo >> 16));
  }
}

// VEC consecutive elements of a run-time-typed tensor; takes the vector path when the
// dtype equals the compile-time type T (the common case: all tensors share a dtype).
template <typename T, int VEC>
__device__ __forceinline__ void load_vec_dyn(const void *base, int dtype, int64_t off,
                                             float (&o)[VEC]) {
  if (dtype == Traits<T>::dtype) {
    load_vec<T, VEC>(base, off, o);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = load_scalar(base, dtype, off + i);
  }
}

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_move(float v) {
  // lanes whose row is masked out, or whose source lane does not exist, receive 0
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}

__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }

// Sum over the 64 lanes of the wavefront using DPP moves only (no LDS traffic).
// The total is valid in lane 63; use wave_sum_bcast() to have it in every lane.
__device__ __forceinline__ float wave_sum_lane63(float v) {
  v += dpp_move<0xB1>(v);         // quad_perm [1,0,3,2]: lane ^ 1
  v += dpp_move<0x4E>(v);         // quad_perm [2,3,0,1]: lane ^ 2
  v += dpp_move<0x141>(v);        // row_half_mirror: the other quad of each 8
  v += dpp_move<0x140>(v);        // row_mirror: the other half of each 16-lane row
  v += dpp_move<0x142, 0xa>(v);   // row_bcast15 into rows 1 and 3
  v += dpp_move<0x143, 0xc>(v);   // row_bcast31 into rows 2 and 3
  return v;
}

__device__ __forceinline__ float wave_sum_bcast(float v) {
  v = wave_sum_lane63(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// z(lane) + z(lane^16) + z(lane^32) + z(lane^48) in every lane, with the lane-swap instructions
// of gfx950 (vector ALU only; a shuffle through the LDS crossbar would cost a round trip each).
__device__ __forceinline__ float add_across_rows(float z) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  // swaps the odd 16-lane rows of the first operand with the even rows of the second
  const u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(z), __float_as_uint(z), false, false);
  z = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  // swaps the upper 32 lanes of the first operand with the lower 32 of the second
  const u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(z), __float_as_uint(z), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over the 64 lanes of eight values per lane at once: returns, in lane L, the wave-wide
// total of d[L & 7].  Three exchange stages inside each group of 8 lanes halve the number of
// live values while doubling the lanes summed (partner L^7, then L^2, then L^1: together they
// generate the whole group), then three stages add the eight groups (L^8 by a row rotation,
// L^16 and L^32 by lane swaps).  About 3.5 VALU operations per value instead of 12.
__device__ __forceinline__ float wave_sum8_transposed(const float (&d)[8]) {
  const int lane = lane_id();
  const bool b2 = (lane & 4) != 0, b1 = (lane & 2) != 0, b0 = (lane & 1) != 0;
  float r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float keep = b2 ? d[i + 4] : d[i];
    const float give = b2 ? d[i] : d[i + 4];
    r[i] = keep + dpp_move<0x141>(give);  // row_half_mirror: lane ^ 7
  }
  float q[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = b1 ? r[i + 2] : r[i];
    const float give = b1 ? r[i] : r[i + 2];
    q[i] = keep + dpp_move<0x4E>(give);  // quad_perm [2,3,0,1]: lane ^ 2
  }
  const float keep = b0 ? q[1] : q[0];
  const float give = b0 ? q[0] : q[1];
  float z = keep + dpp_move<0xB1>(give);  // quad_perm [1,0,3,2]: lane ^ 1
  z += dpp_move<0x128>(z);                // row_ror:8 within the 16-lane row: lane ^ 8
  z = add_across_rows(z);
  return z;
}

// VEC consecutive elements as stored (no conversion): lets a kernel keep many loads in flight
// in few registers and convert at the point of use.
template <typename T, int VEC>
using raw_vec_t = vec_t<typename Traits<T>::store_t, VEC>;

template <typename T, int VEC, bool NT = false>
__device__ __forceinline__ raw_vec_t<T, VEC> load_raw(const void *base, int64_t off) {
  using S = typename Traits<T>::store_t;
  const raw_vec_t<T, VEC> *p = reinterpret_cast<const raw_vec_t<T, VEC> *>(static_cast<const S *>(base) + off);
  if constexpr (NT) return __builtin_nontemporal_load(p);  // read once: do not keep it in the L2
  else return *p;
}

template <typename T, int VEC>
__device__ __forceinline__ void unpack_raw(const raw_vec_t<T, VEC> &v, float (&o)[VEC]) {
#pragma unroll
  for (int i = 0; i < VEC; ++i) o[i] = Traits<T>::up(v[i]);
}


// Row gathers through a buffer descriptor: the lane's byte offset travels in a vector register,
// the (uniform) row offset in a scalar one, so a gather costs no vector ALU work for addressing;
// reads beyond `bytes` return zeros.  The matrix must be smaller than 4 GiB.
struct GatherSource {
  __amdgpu_buffer_rsrc_t rsrc;
};
__device__ __forceinline__ GatherSource make_gather_source(const void *base, uint32_t bytes) {
  GatherSource g;
  g.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
  return g;
}
template <typename T, int VEC>
__device__ __forceinline__ raw_vec_t<T, VEC> gather_raw(const GatherSource &g, uint32_t lane_bytes,
                                                        uint32_t row_bytes_offset) {
  constexpr int kBytes = VEC * static_cast<int>(sizeof(typename Traits<T>::store_t));
  raw_vec_t<T, VEC> out;
  if constexpr (kBytes == 2) {
    const uint16_t v = __builtin_amdgcn_raw_buffer_load_b16(g.rsrc, lane_bytes, row_bytes_offset, 0);
    __builtin_memcpy(&out, &v, 2);
  } else if constexpr (kBytes == 4) {
    const uint32_t v = __builtin_amdgcn_raw_buffer_load_b32(g.rsrc, lane_bytes, row_bytes_offset, 0);
    __builtin_memcpy(&out, &v, 4);
  } else if constexpr (kBytes == 8) {
    const vec_t<uint32_t, 2> v = __builtin_amdgcn_raw_buffer_load_b64(g.rsrc, lane_bytes, row_bytes_offset, 0);
    __builtin_memcpy(&out, &v, 8);
  } else {
    static_assert(kBytes == 16, "gathers are 2 to 16 bytes per lane");
    const vec_t<uint32_t, 4> v = __builtin_amdgcn_raw_buffer_load_b128(g.rsrc, lane_bytes, row_bytes_offset, 0);
    __builtin_memcpy(&out, &v, 16);
  }
  return out;
}

// One row of a row-major matrix as a buffer descriptor: row_bytes bytes at base + row*row_bytes
// (row must be wave-uniform, so the address arithmetic runs on the scalar unit; any matrix
// size).  A lane offset at or beyond row_bytes reads zeros, and a store there is dropped.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_descriptor(const void *base, uint32_t row,
                                                                 uint32_t row_bytes) {
  const char *p = static_cast<const char *>(base) + static_cast<uint64_t>(row) * row_bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(p), 0, static_cast<int>(row_bytes), 0x00020000);
}
// N bytes (4, 8 or 16) per lane through a descriptor, as dwords
template <int N>
__device__ __forceinline__ vec_t<uint32_t, N / 4> descriptor_load(__amdgpu_buffer_rsrc_t r, uint32_t lane_bytes) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 bytes per lane");
  if constexpr (N == 4) {
    vec_t<uint32_t, 1> v;
    v[0] = __builtin_amdgcn_raw_buffer_load_b32(r, lane_bytes, 0, 0);
    return v;
  } else if constexpr (N == 8) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, lane_bytes, 0, 0);
  } else {
    return __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, 0, 0);
  }
}
// NT: non-temporal (streaming) store
template <int N, bool NT = false>
__device__ __forceinline__ void descriptor_store(__amdgpu_buffer_rsrc_t r, uint32_t lane_bytes,
                                                 const vec_t<uint32_t, N / 4> &v) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 bytes per lane");
  constexpr int kAux = NT ? 2 : 0;  // cache-policy bits of the instruction: bit 1 = nt
  if constexpr (N == 4) __builtin_amdgcn_raw_buffer_store_b32(v[0], r, lane_bytes, 0, kAux);
  else if constexpr (N == 8) __builtin_amdgcn_raw_buffer_store_b64(v, r, lane_bytes, 0, kAux);
  else __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_bytes, 0, kAux);
}

// The same through a descriptor of a whole matrix of fewer than 4 GiB, the (wave-uniform) byte
// offset of the row in a scalar register that the instruction adds by itself: where the row
// offsets of all steps are computed at once by the lanes (one multiplication per lane) and read
// back lane by lane, a gather or a store costs no address arithmetic at all.  No lane may lie
// beyond its row: nothing is clipped at the row's end here.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t matrix_descriptor(const void *base, uint64_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0,
                                           static_cast<int>(static_cast<uint32_t>(bytes)), 0x00020000);
}
template <int N>
__device__ __forceinline__ vec_t<uint32_t, N / 4> descriptor_load_at(__amdgpu_buffer_rsrc_t r, uint32_t lane_bytes,
                                                                     uint32_t row_bytes_offset) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 bytes per lane");
  if constexpr (N == 4) {
    vec_t<uint32_t, 1> v;
    v[0] = __builtin_amdgcn_raw_buffer_load_b32(r, lane_bytes, row_bytes_offset, 0);
    return v;
  } else if constexpr (N == 8) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, lane_bytes, row_bytes_offset, 0);
  } else {
    return __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, row_bytes_offset, 0);
  }
}
template <int N, bool NT = false>
__device__ __forceinline__ void descriptor_store_at(__amdgpu_buffer_rsrc_t r, uint32_t lane_bytes,
                                                    uint32_t row_bytes_offset, const vec_t<uint32_t, N / 4> &v) {
  static_assert(N == 4 || N == 8 || N == 16, "4, 8 or 16 bytes per lane");
  constexpr int kAux = NT ? 2 : 0;
  if constexpr (N == 4) __builtin_amdgcn_raw_buffer_store_b32(v[0], r, lane_bytes, row_bytes_offset, kAux);
  else if constexpr (N == 8) __builtin_amdgcn_raw_buffer_store_b64(v, r, lane_bytes, row_bytes_offset, kAux);
  else __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_bytes, row_bytes_offset, kAux);
}

// VEC consecutive elements of row `row` (wave-uniform) of a row-major matrix, starting at column
// d0, as stored.  Lanes with d0 beyond the row get zeros.  Pieces of at least four bytes go
// through a row descriptor (address arithmetic on the scalar unit).
template <typename T, int VEC>
__device__ __forceinline__ raw_vec_t<T, VEC> gather_row_piece(const void *base, uint32_t row, int D, int d0) {
  using S = typename Traits<T>::store_t;
  constexpr int kBytes = VEC * static_cast<int>(sizeof(S));
  raw_vec_t<T, VEC> out;
  if constexpr (kBytes >= 4) {
    const auto dw = descriptor_load<kBytes>(row_descriptor(base, row, static_cast<uint32_t>(D) * sizeof(S)),
                                            static_cast<uint32_t>(d0) * sizeof(S));
    __builtin_memcpy(&out, &dw, kBytes);
  } else {
    out = load_raw<T, VEC>(base, static_cast<int64_t>(row) * D + (d0 < D ? d0 : 0));
    if (d0 >= D) out = raw_vec_t<T, VEC>{};
  }
  return out;
}

// x[0..VEC) rounded to T and stored at row `row` (wave-uniform), column `col`, of a row-major
// matrix with `ld` columns; col + VEC <= ld must hold for every lane.  NT: streaming store.
template <typename T, int VEC, bool NT>
__device__ __forceinline__ void scatter_row_piece(void *base, uint32_t row, int ld, int col, const float (&x)[VEC]) {
  using S = typename Traits<T>::store_t;
  constexpr int kBytes = VEC * static_cast<int>(sizeof(S));
  if constexpr (kBytes >= 4) {
    vec_t<uint32_t, kBytes / 4> packed;
    if constexpr (Traits<T>::dtype == FLEXSAE_BF16) {
#pragma unroll
      for (int i = 0; i < VEC / 2; ++i) packed[i] = f32x2_to_bf16x2_bits(x[2 * i], x[2 * i + 1]);
    } else if constexpr (Traits<T>::dtype == FLEXSAE_F32) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) packed[i] = __float_as_uint(x[i]);
    } else {
#pragma unroll
      for (int i = 0; i < VEC / 2; ++i)
        packed[i] = static_cast<uint32_t>(f32_to_f16_bits(x[2 * i])) |
                    (static_cast<uint32_t>(f32_to_f16_bits(x[2 * i + 1])) << 16);
    }
    descriptor_store<kBytes, NT>(row_descriptor(base, row, static_cast<uint32_t>(ld) * sizeof(S)),
                                   static_cast<uint32_t>(col) * sizeof(S), packed);
  } else {
    store_vec<T, VEC, NT>(base, static_cast<int64_t>(row) * ld + col, x);
  }
}

// acc + a.lo*b.lo + a.hi*b.hi on two packed bf16 pairs (one instruction on gfx950)
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  bf16x2 x, y;
  __builtin_memcpy(&x, &a, 4);
  __builtin_memcpy(&y, &b, 4);
  return __builtin_amdgcn_fdot2_f32_bf16(x, y, acc, false);
}

// Wave index inside the block as a scalar (uniform) value, so that everything
// derived from it is addressed through scalar registers.
__device__ __forceinline__ int wave_in_block() {
  return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
}

__device__ __forceinline__ int bcast_i32(int v, int src_lane) {
  return __builtin_amdgcn_readlane(v, src_lane);
}
__device__ __forceinline__ float bcast_f32(float v, int src_lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

}  // namespace flexsae
