// C-ABI entry points (include/flexsae_amd.h): argument validation, kernel selection and
// launches.  No allocation, no synchronisation, no global state.
#include <hip/hip_runtime.h>

#include "common.hpp"
#include "fwd_kernels.hpp"
#include "hier_bwd_kernels.hpp"
#include "topk_bwd_kernels.hpp"

using namespace flexsae;

namespace {

constexpr int kBlock = 256;              // threads per block of the wave-per-item kernels
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr size_t kAlign = 256;

inline bool valid_dtype(int d) { return d == FLEXSAE_F32 || d == FLEXSAE_BF16 || d == FLEXSAE_F16; }
inline size_t dtype_size(int d) { return d == FLEXSAE_F32 ? 4 : 2; }
inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

int check_shape(const flexsae_shape *s) {
  if (!s) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (s->B <= 0 || s->K <= 0 || s->F <= 0 || s->D <= 0) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(s->weight_dtype) || !valid_dtype(s->vals_dtype) || !valid_dtype(s->bias_dtype) ||
      !valid_dtype(s->target_dtype))
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (s->F >= (1LL << 31) || s->D >= (1LL << 31) || s->K >= (1LL << 31)) return FLEXSAE_ERR_UNSUPPORTED;
  if (s->B > ((1LL << 32) - 1) / s->K) return FLEXSAE_ERR_UNSUPPORTED;  // B*K < 2^32
  return FLEXSAE_OK;
}

int launch_status() { return hipGetLastError() == hipSuccess ? FLEXSAE_OK : FLEXSAE_ERR_LAUNCH; }

// Largest vector width (elements per lane) the row layout allows: every row start and
// every lane offset must be aligned to the vector, and wider than 16 bytes gains nothing.
int pick_vec(int64_t D, size_t elem_size, const void *base, int max_vec) {
  for (int v = max_vec; v > 1; v >>= 1) {
    if (static_cast<size_t>(v) * elem_size > 16) continue;
    if (D % v == 0 && aligned(base, v * elem_size)) return v;
  }
  return 1;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline unsigned grid_for(int64_t n_threads, int block, int64_t cap) {
  int64_t g = ceil_div(n_threads, block);
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return static_cast<unsigned>(g);
}

struct FwdPlan {
  int vec;
  int ntiles;
  int64_t n_items;
};

FwdPlan plan_fwd(const flexsae_shape *s, const void *weight, const void *target, const void *bias,
                 const float *resid) {
  const size_t es = dtype_size(s->weight_dtype);
  int vec = pick_vec(s->D, es, weight, es == 4 ? 4 : 8);
  // resid is stored with fp32 vectors of the same width, target/bias are read with the
  // weight's vector type when they share its dtype
  if (s->target_dtype == s->weight_dtype && !aligned(target, vec * es)) vec = 1;
  if (s->bias_dtype == s->weight_dtype && !aligned(bias, vec * es)) vec = 1;
  if (!aligned(resid, vec * 4)) vec = 1;
  // a tile of 64*vec columns that is mostly padding wastes lanes: narrow it for small D
  while (vec > 1 && s->D < static_cast<int64_t>(kWave) * vec && s->D % (vec / 2) == 0) vec >>= 1;
  FwdPlan p;
  p.vec = vec;
  p.ntiles = static_cast<int>(ceil_div(s->D, static_cast<int64_t>(kWave) * vec));
  p.n_items = s->B * p.ntiles;
  return p;
}

template <typename WT, int VEC, bool HIER>
void launch_fwd_t(const flexsae_shape *s, const FwdPlan &p, const int64_t *indices,
                  const void *weight, const void *vals, const void *bias, const void *target,
                  float *resid, float *partial, int *status_flag, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>(ceil_div(p.n_items, kWavesPerBlock));
  hipLaunchKernelGGL((sae_fwd_kernel<WT, VEC, HIER, 8>), dim3(grid), dim3(kBlock), 0, st, indices,
                     weight, vals, s->vals_dtype, bias, s->bias_dtype, target, s->target_dtype,
                     resid, partial, status_flag, p.n_items, p.ntiles, static_cast<int>(s->K),
                     s->F, static_cast<int>(s->D));
}

template <typename WT, bool HIER>
void launch_fwd_v(const flexsae_shape *s, const FwdPlan &p, const int64_t *indices,
                  const void *weight, const void *vals, const void *bias, const void *target,
                  float *resid, float *partial, int *status_flag, hipStream_t st) {
  switch (p.vec) {
    case 8:
      if constexpr (sizeof(typename Traits<WT>::store_t) == 2) {
        launch_fwd_t<WT, 8, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                  status_flag, st);
        break;
      }
      [[fallthrough]];
    case 4:
      launch_fwd_t<WT, 4, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                status_flag, st);
      break;
    case 2:
      launch_fwd_t<WT, 2, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                status_flag, st);
      break;
    default:
      launch_fwd_t<WT, 1, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                status_flag, st);
  }
}

template <bool HIER>
int forward(const flexsae_shape *s, const int64_t *indices, const void *weight, const void *vals,
            const void *bias, const void *target, float *loss, float *resid, void *workspace,
            size_t workspace_bytes, int *status_flag, void *stream) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!indices || !weight || !vals || !bias || !target || !loss || !resid)
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(indices, 8) || !aligned(weight, dtype_size(s->weight_dtype)) ||
      !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(bias, dtype_size(s->bias_dtype)) ||
      !aligned(target, dtype_size(s->target_dtype)) || !aligned(loss, 4) || !aligned(resid, 16))
    return FLEXSAE_ERR_ALIGNMENT;
  if (!workspace || workspace_bytes < flexsae_fwd_workspace_bytes(s) || !aligned(workspace, kAlign))
    return FLEXSAE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const FwdPlan p = plan_fwd(s, weight, target, bias, resid);
  float *partial = static_cast<float *>(workspace);
  switch (s->weight_dtype) {
    case FLEXSAE_F32:
      launch_fwd_v<float, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                status_flag, st);
      break;
    case FLEXSAE_BF16:
      launch_fwd_v<bf16_t, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                 status_flag, st);
      break;
    default:
      launch_fwd_v<f16_t, HIER>(s, p, indices, weight, vals, bias, target, resid, partial,
                                status_flag, st);
  }
  rc = launch_status();
  if (rc != FLEXSAE_OK) return rc;
  const double count = static_cast<double>(s->B) * static_cast<double>(s->D) *
                       (HIER ? static_cast<double>(s->K) : 1.0);
  hipLaunchKernelGGL(loss_finalize_kernel, dim3(1), dim3(1024), 0, st, partial, p.n_items,
                     1.0 / count, loss);
  return launch_status();
}

template <typename WT>
void launch_hier_bwd_t(const flexsae_shape *s, const int64_t *indices, const void *weight,
                       const void *vals, const float *resid, const float *grad_out, float coef,
                       float *dW, float *dvals, float *dbias, int *status_flag, hipStream_t st) {
  const int K = static_cast<int>(s->K), D = static_cast<int>(s->D);
  // widest tile that the row length fills without padding (C columns per lane)
  const int C = (D % 256 == 0) ? 4 : (D % 128 == 0) ? 2 : 1;
  const int ntiles = static_cast<int>(ceil_div(D, static_cast<int64_t>(kWave) * C));
  const int64_t n_items = s->B * ntiles;
  const unsigned grid = static_cast<unsigned>(ceil_div(n_items, kWavesPerBlock));
#define FLEXSAE_LAUNCH_HB(CC)                                                                    \
  hipLaunchKernelGGL((hier_bwd_kernel<WT, CC, 4>), dim3(grid), dim3(kBlock), 0, st, indices,     \
                     weight, vals, s->vals_dtype, resid, grad_out, coef, dW, dvals, dbias,       \
                     status_flag, n_items, ntiles, K, s->F, D)
  if (C == 4) {
    FLEXSAE_LAUNCH_HB(4);
  } else if (C == 2) {
    FLEXSAE_LAUNCH_HB(2);
  } else {
    FLEXSAE_LAUNCH_HB(1);
  }
#undef FLEXSAE_LAUNCH_HB
}

void zero_f32(float *p, int64_t n, hipStream_t st) {
  hipLaunchKernelGGL(fill_f32_kernel, dim3(grid_for(ceil_div(n, 4), 256, 1 << 16)), dim3(256), 0, st,
                     p, n);
}

template <typename WT, typename GT>
void launch_topk_bwd_t(const flexsae_shape *s, const uint32_t *begin, const uint32_t *map,
                       const void *weight, const void *vals, const float *resid,
                       const float *grad_out, float coef, void *dW, float *dvals, int vec,
                       hipStream_t st) {
  const int K = static_cast<int>(s->K), D = static_cast<int>(s->D);
  const int ntiles = static_cast<int>(ceil_div(D, static_cast<int64_t>(kWave) * vec));
  const int64_t n_items = s->F * ntiles;
  const unsigned grid = static_cast<unsigned>(ceil_div(n_items, kWavesPerBlock));
#define FLEXSAE_LAUNCH_TB(VV)                                                                     \
  hipLaunchKernelGGL((topk_bwd_kernel<WT, GT, VV, 4, true>), dim3(grid), dim3(kBlock), 0, st,     \
                     begin, map, weight, vals, s->vals_dtype, resid, grad_out, coef, dW, dvals,   \
                     n_items, ntiles, s->F, K, D)
  if (vec == 4) {
    FLEXSAE_LAUNCH_TB(4);
  } else if (vec == 2) {
    FLEXSAE_LAUNCH_TB(2);
  } else {
    FLEXSAE_LAUNCH_TB(1);
  }
#undef FLEXSAE_LAUNCH_TB
}

template <typename WT>
void launch_topk_bwd_g(const flexsae_shape *s, const uint32_t *begin, const uint32_t *map,
                       const void *weight, const void *vals, const float *resid,
                       const float *grad_out, float coef, void *dW, int dW_dtype, float *dvals,
                       int vec, hipStream_t st) {
  switch (dW_dtype) {
    case FLEXSAE_F32:
      launch_topk_bwd_t<WT, float>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dvals,
                                   vec, st);
      break;
    case FLEXSAE_BF16:
      launch_topk_bwd_t<WT, bf16_t>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dvals,
                                    vec, st);
      break;
    default:
      launch_topk_bwd_t<WT, f16_t>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dvals,
                                   vec, st);
  }
}

}  // namespace

extern "C" {

int flexsae_abi_version(void) { return FLEXSAE_ABI_VERSION; }

const char *flexsae_status_string(int status) {
  switch (status) {
    case FLEXSAE_OK:
      return "ok";
    case FLEXSAE_ERR_INVALID_ARGUMENT:
      return "invalid argument (null pointer, non-positive size or unknown dtype)";
    case FLEXSAE_ERR_UNSUPPORTED:
      return "unsupported size (need F, D, K < 2^31 and B*K < 2^32)";
    case FLEXSAE_ERR_WORKSPACE:
      return "workspace missing, too small or not 256-byte aligned";
    case FLEXSAE_ERR_LAUNCH:
      return "HIP kernel launch failed";
    case FLEXSAE_ERR_ALIGNMENT:
      return "tensor pointer not aligned to its element size";
    default:
      return "unknown status";
  }
}

size_t flexsae_fwd_workspace_bytes(const flexsae_shape *s) {
  if (check_shape(s) != FLEXSAE_OK) return 0;
  // one fp32 partial per (row, tile); the narrowest tile is 64 columns
  return round_up(static_cast<size_t>(s->B) * static_cast<size_t>(ceil_div(s->D, kWave)) * 4, kAlign);
}

int flexsae_hier_fwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const void *bias, const void *target, float *loss,
                     float *resid, void *workspace, size_t workspace_bytes, int *status_flag,
                     void *stream) {
  return forward<true>(shape, indices, weight, vals, bias, target, loss, resid, workspace,
                       workspace_bytes, status_flag, stream);
}

int flexsae_topk_fwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const void *bias, const void *target, float *loss,
                     float *resid, void *workspace, size_t workspace_bytes, int *status_flag,
                     void *stream) {
  return forward<false>(shape, indices, weight, vals, bias, target, loss, resid, workspace,
                        workspace_bytes, status_flag, stream);
}

int flexsae_hier_bwd(const flexsae_shape *s, const int64_t *indices, const void *weight,
                     const void *vals, const float *resid, const float *grad_out, float *dW_acc,
                     float *dvals, float *dbias, int flags, int *status_flag, void *stream) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!indices || !weight || !vals || !resid || !grad_out || !dW_acc || !dvals || !dbias)
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(indices, 8) || !aligned(weight, dtype_size(s->weight_dtype)) ||
      !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(resid, 4) || !aligned(grad_out, 4) ||
      !aligned(dW_acc, 16) || !aligned(dvals, 16) || !aligned(dbias, 16))
    return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!(flags & FLEXSAE_BWD_OUTPUTS_PREZEROED)) {
    zero_f32(dW_acc, s->F * s->D, st);
    zero_f32(dvals, s->B * s->K, st);
    zero_f32(dbias, s->D, st);
  }
  const float coef = static_cast<float>(
      2.0 / (static_cast<double>(s->B) * static_cast<double>(s->K) * static_cast<double>(s->D)));
  switch (s->weight_dtype) {
    case FLEXSAE_F32:
      launch_hier_bwd_t<float>(s, indices, weight, vals, resid, grad_out, coef, dW_acc, dvals,
                               dbias, status_flag, st);
      break;
    case FLEXSAE_BF16:
      launch_hier_bwd_t<bf16_t>(s, indices, weight, vals, resid, grad_out, coef, dW_acc, dvals,
                                dbias, status_flag, st);
      break;
    default:
      launch_hier_bwd_t<f16_t>(s, indices, weight, vals, resid, grad_out, coef, dW_acc, dvals,
                               dbias, status_flag, st);
  }
  return launch_status();
}

size_t flexsae_csr_workspace_bytes(int64_t B, int64_t K, int64_t F) {
  if (B <= 0 || K <= 0 || F <= 0) return 0;
  // cursor[F] | long_count (padded) | long_list[B*K/65 + 1]
  return round_up(static_cast<size_t>(F) * 4, kAlign) + kAlign +
         round_up((static_cast<size_t>(B) * static_cast<size_t>(K) / 65 + 1) * 4, kAlign);
}

int flexsae_csr_build(const int64_t *indices, int64_t B, int64_t K, int64_t F, uint32_t *begin,
                      uint32_t *map, void *workspace, size_t workspace_bytes, int *status_flag,
                      void *stream) {
  if (!indices || !begin || !map || B <= 0 || K <= 0 || F <= 0) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (F >= (1LL << 31) || B > ((1LL << 32) - 1) / K) return FLEXSAE_ERR_UNSUPPORTED;
  if (!aligned(indices, 8) || !aligned(begin, 4) || !aligned(map, 4)) return FLEXSAE_ERR_ALIGNMENT;
  if (!workspace || workspace_bytes < flexsae_csr_workspace_bytes(B, K, F) ||
      !aligned(workspace, kAlign))
    return FLEXSAE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t n_pairs = B * K;
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  uint32_t *cursor = reinterpret_cast<uint32_t *>(ws);
  uint32_t *long_count = reinterpret_cast<uint32_t *>(ws + round_up(static_cast<size_t>(F) * 4, kAlign));
  uint32_t *long_list = reinterpret_cast<uint32_t *>(reinterpret_cast<uint8_t *>(long_count) + kAlign);

  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(F + 1, 256, 4096)), dim3(256), 0, st, begin,
                     F + 1, 0u);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, long_count, static_cast<int64_t>(1), 0u);
  hipLaunchKernelGGL(csr_count_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st,
                     indices, n_pairs, F, begin, status_flag);
  hipLaunchKernelGGL(csr_scan_kernel, dim3(1), dim3(kScanThreads), 0, st, begin, cursor, F);
  hipLaunchKernelGGL(csr_fill_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, indices,
                     n_pairs, F, cursor, map);
  hipLaunchKernelGGL(csr_sort_short_kernel, dim3(static_cast<unsigned>(ceil_div(F, kWavesPerBlock))),
                     dim3(kBlock), 0, st, begin, map, F, long_count, long_list);
  hipLaunchKernelGGL(csr_sort_long_kernel, dim3(512), dim3(256), 0, st, begin, map, long_count,
                     long_list);
  return launch_status();
}

int flexsae_topk_bwd(const flexsae_shape *s, const uint32_t *begin, const uint32_t *map,
                     const void *weight, const void *vals, const float *resid,
                     const float *grad_out, void *dW, int dW_dtype, float *dvals, float *dbias,
                     int flags, void *stream) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!begin || !map || !weight || !vals || !resid || !grad_out || !dW || !dvals || !dbias ||
      !valid_dtype(dW_dtype))
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(begin, 4) || !aligned(map, 4) || !aligned(weight, dtype_size(s->weight_dtype)) ||
      !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(resid, 4) || !aligned(grad_out, 4) ||
      !aligned(dW, dtype_size(dW_dtype)) || !aligned(dvals, 16) || !aligned(dbias, 16))
    return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!(flags & FLEXSAE_BWD_OUTPUTS_PREZEROED)) {
    zero_f32(dvals, s->B * s->K, st);
    zero_f32(dbias, s->D, st);
  }
  const float coef =
      static_cast<float>(2.0 / (static_cast<double>(s->B) * static_cast<double>(s->D)));
  // vector width: resid rows are read as fp32 vectors, weight/dW rows in their own types
  int vec = 4;
  while (vec > 1 && (s->D % vec != 0 || !aligned(resid, vec * 4) ||
                     !aligned(weight, vec * dtype_size(s->weight_dtype)) ||
                     !aligned(dW, vec * dtype_size(dW_dtype))))
    vec >>= 1;
  while (vec > 1 && s->D < static_cast<int64_t>(kWave) * vec && s->D % (vec / 2) == 0) vec >>= 1;
  switch (s->weight_dtype) {
    case FLEXSAE_F32:
      launch_topk_bwd_g<float>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                               dvals, vec, st);
      break;
    case FLEXSAE_BF16:
      launch_topk_bwd_g<bf16_t>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                                dvals, vec, st);
      break;
    default:
      launch_topk_bwd_g<f16_t>(s, begin, map, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                               dvals, vec, st);
  }
  rc = launch_status();
  if (rc != FLEXSAE_OK) return rc;
  const int rows_per_block = 64;
  hipLaunchKernelGGL(colsum_kernel,
                     dim3(static_cast<unsigned>(ceil_div(s->D, 256)),
                          static_cast<unsigned>(ceil_div(s->B, rows_per_block))),
                     dim3(256), 0, st, resid, grad_out, coef, dbias, s->B, static_cast<int>(s->D),
                     rows_per_block);
  return launch_status();
}

int flexsae_cast_from_f32(void *dst, int dst_dtype, const float *src, int64_t n, void *stream) {
  if (!dst || !src || n < 0 || !valid_dtype(dst_dtype)) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (n == 0) return FLEXSAE_OK;
  if (!aligned(src, 16) || !aligned(dst, 4 * dtype_size(dst_dtype))) return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(grid_for(ceil_div(n, 4), 256, 1 << 16));
  switch (dst_dtype) {
    case FLEXSAE_F32:
      hipLaunchKernelGGL(cast_from_f32_kernel<float>, grid, dim3(256), 0, st, dst, src, n);
      break;
    case FLEXSAE_BF16:
      hipLaunchKernelGGL(cast_from_f32_kernel<bf16_t>, grid, dim3(256), 0, st, dst, src, n);
      break;
    default:
      hipLaunchKernelGGL(cast_from_f32_kernel<f16_t>, grid, dim3(256), 0, st, dst, src, n);
  }
  return launch_status();
}

}  // extern "C"
