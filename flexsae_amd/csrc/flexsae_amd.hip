// C-ABI entry points (include/flexsae_amd.h): argument validation, kernel selection and
// launches.  No allocation, no synchronisation, no global state.
#include <hip/hip_runtime.h>
#include <stdlib.h>

#include <mutex>

#include "common.hpp"
#include "fwd_kernels.hpp"
#include "csr_kernels.hpp"
#include "hier_bwd_kernels.hpp"
#include "hier_train_kernel.hpp"
#include "hier_hot_kernel.hpp"
#include "segment_kernels.hpp"
#include "topk_bwd_kernels.hpp"

using namespace flexsae;

// Device memory of flexsae_hier_fwd_static, the one entry point that takes no workspace: the
// forward kernels' per-(row, tile) loss partials live here.  Every GPU the library runs on holds
// its own copy of the array until the process ends.  Host code never uses the array's name as an
// address: the per-device address comes from hipGetSymbolAddress (static_scratch_for_current_device).
constexpr size_t kStaticScratchBytes = FLEXSAE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// gathers in flight per wavefront before the first one is consumed
#ifndef FLEXSAE_SWEEP_U
#define FLEXSAE_SWEEP_U 16
#endif
#ifndef FLEXSAE_REDUCE_U
#define FLEXSAE_REDUCE_U 4
#endif
#ifndef FLEXSAE_PIECE_U
#define FLEXSAE_PIECE_U 4
#endif
#ifndef FLEXSAE_FWD_U
#define FLEXSAE_FWD_U 8
#endif
#ifndef FLEXSAE_TOPK_VEC8
#define FLEXSAE_TOPK_VEC8 1
#endif
#ifndef FLEXSAE_TOPK_RESID16
#define FLEXSAE_TOPK_RESID16 1
#endif

namespace {

constexpr int kBlock = 256;              // threads per block of the wave-per-item kernels
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr size_t kAlign = 256;
constexpr int kBwdSgdUpdate = 1 << 20;  // internal flag of the slice loop: dW is the weight matrix, updated in place
constexpr int kBwdHot = 1 << 21;        // internal flag of the slice loop: hot latents are accumulated in the LDS
constexpr unsigned kLongBlocks = 1024;    // leading blocks of a reduction launch that serve hot latents

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
  // D < 2^29: a row of any matrix here (at most 4 bytes per element) fits a buffer descriptor
  if (s->F >= (1LL << 31) || s->D >= (1LL << 29) || s->K >= (1LL << 31)) return FLEXSAE_ERR_UNSUPPORTED;
  if (s->B > ((1LL << 32) - 1) / s->K) return FLEXSAE_ERR_UNSUPPORTED;  // B*K < 2^32
  return FLEXSAE_OK;
}

int launch_status() { return hipGetLastError() == hipSuccess ? FLEXSAE_OK : FLEXSAE_ERR_LAUNCH; }

// Address of `scratch` on the current device, looked up once per device and kept.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch_for_current_device(void **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FLEXSAE_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return FLEXSAE_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return FLEXSAE_OK;
}

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
  int vec = pick_vec(s->D, es, weight, 4);  // 256-column tiles measured faster than 512
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
  hipLaunchKernelGGL((sae_fwd_kernel<WT, VEC, HIER, FLEXSAE_FWD_U>), dim3(grid), dim3(kBlock), 0, st, indices,
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

// How a pair list is built for a given problem size.  The bucketed construction serves every
// size whose bucket count fits the LDS counters of its kernels; beyond that (more than
// kBucketMaxBuckets * kSortMaxLatents latents) the list is built with one memory atomic per pair.
struct CsrPlan {
  bool bucketed;
  int shift;           // a bucket is 2^shift consecutive latents
  uint32_t n_buckets;
  int64_t chunk;       // consecutive pairs counted by one block
  uint32_t n_chunks;
  size_t table_len;    // n_buckets * n_chunks (+1 entry for the total)
};

CsrPlan plan_csr(int64_t n_pairs, int64_t F) {
  CsrPlan p;
  // latents per bucket: about 2048 pairs per bucket on average, a power of two
  int shift = 0;
  while (shift < 12 && (static_cast<int64_t>(2) << shift) * n_pairs <= 2048 * F) ++shift;
  static_assert((1 << 12) == kSortMaxLatents, "shift limit follows the LDS counters of the sort kernel");
  while (shift < 12 && ceil_div(F, static_cast<int64_t>(1) << shift) > kBucketMaxBuckets) ++shift;
  p.shift = shift;
  const int64_t n_buckets = ceil_div(F, static_cast<int64_t>(1) << shift);
  p.bucketed = n_buckets <= kBucketMaxBuckets;
  p.n_buckets = static_cast<uint32_t>(p.bucketed ? n_buckets : 0);
  p.chunk = 2048;
  while (p.bucketed && ceil_div(n_pairs, p.chunk) * n_buckets > (static_cast<int64_t>(1) << 22)) p.chunk *= 2;
  p.n_chunks = static_cast<uint32_t>(ceil_div(n_pairs, p.chunk));
  p.table_len = p.bucketed ? static_cast<size_t>(n_buckets) * p.n_chunks : 0;
  return p;
}

// Scratch of the pair-list construction, carved out of one workspace:
//   bucketed: tmp[B*K] u64 | table[table_len + 1] | scan block sums | long_count (one aligned
//             slot) | long_list[B*K/65 + 1]
//   atomic:   rank[B*K] u32 | scan block sums[ceil(F/kScanBlockElems)] | long_count | long_list
struct CsrScratch {
  CsrPlan plan;
  uint64_t *tmp;
  uint32_t *table;
  uint32_t *rank;
  uint32_t *block_sums;
  uint32_t *long_count;
  uint32_t *long_list;
};

size_t csr_scan_sums_bytes(int64_t n) {
  return round_up(static_cast<size_t>(ceil_div(n, kScanBlockElems)) * 4, kAlign);
}

size_t csr_scratch_bytes(int64_t n_pairs, int64_t F, CsrScratch *sc, uint8_t *ws) {
  const CsrPlan pl = plan_csr(n_pairs, F);
  size_t off = 0;
  if (sc) {
    sc->plan = pl;
    sc->tmp = nullptr;
    sc->table = nullptr;
    sc->rank = nullptr;
  }
  if (pl.bucketed) {
    if (sc) sc->tmp = reinterpret_cast<uint64_t *>(ws + off);
    off += round_up(static_cast<size_t>(n_pairs) * 8, kAlign);
    if (sc) sc->table = reinterpret_cast<uint32_t *>(ws + off);
    off += round_up((pl.table_len + 1) * 4, kAlign);
    if (sc) sc->block_sums = reinterpret_cast<uint32_t *>(ws + off);
    off += csr_scan_sums_bytes(static_cast<int64_t>(pl.table_len));
  } else {
    if (sc) sc->rank = reinterpret_cast<uint32_t *>(ws + off);
    off += round_up(static_cast<size_t>(n_pairs) * 4, kAlign);
    if (sc) sc->block_sums = reinterpret_cast<uint32_t *>(ws + off);
    off += csr_scan_sums_bytes(F);
  }
  if (sc) sc->long_count = reinterpret_cast<uint32_t *>(ws + off);
  off += kAlign;
  if (sc) sc->long_list = reinterpret_cast<uint32_t *>(ws + off);
  off += round_up((static_cast<size_t>(n_pairs) / 65 + 1) * 4, kAlign);
  return off;
}

CsrScratch carve_csr_scratch(void *workspace, int64_t F, int64_t n_pairs) {
  CsrScratch sc;
  csr_scratch_bytes(n_pairs, F, &sc, static_cast<uint8_t *>(workspace));
  return sc;
}

// begin[F+1], map[B*K] and, when `slot` is given, its inverse slot[B*K]; leaves the list of
// latents with more than 64 pairs in sc.long_list / sc.long_count.
void csr_build_launch(const int64_t *indices, int64_t B, int64_t K, int64_t F, uint32_t *begin,
                      uint32_t *map, uint32_t *slot, const CsrScratch &sc, int *status_flag, hipStream_t st) {
  const int64_t n_pairs = B * K;
  const CsrPlan &pl = sc.plan;
  if (pl.bucketed) {
    hipLaunchKernelGGL(csr_bucket_count_kernel, dim3(pl.n_chunks), dim3(kBucketThreads), 0, st, indices, n_pairs,
                       F, pl.shift, pl.n_buckets, pl.chunk, pl.n_chunks, sc.table, sc.long_count, status_flag);
    const int64_t len = static_cast<int64_t>(pl.table_len);
    const unsigned scan_blocks = static_cast<unsigned>(ceil_div(len, kScanBlockElems));
    hipLaunchKernelGGL(csr_scan_sums_kernel, dim3(scan_blocks), dim3(kScanThreads), 0, st, sc.table, len,
                       sc.block_sums);
    hipLaunchKernelGGL(csr_scan_apply_kernel, dim3(scan_blocks), dim3(kScanThreads), 0, st, sc.table, len,
                       sc.block_sums);
    hipLaunchKernelGGL(csr_bucket_scatter_kernel, dim3(pl.n_chunks), dim3(kBucketThreads), 0, st, indices,
                       n_pairs, F, pl.shift, pl.n_buckets, pl.chunk, pl.n_chunks, sc.table, sc.tmp);
    hipLaunchKernelGGL(csr_bucket_sort_kernel, dim3(pl.n_buckets), dim3(kSortThreads), 0, st, sc.tmp, sc.table,
                       pl.n_chunks, pl.shift, F, begin, map, slot, sc.long_count, sc.long_list);
    hipLaunchKernelGGL(csr_sort_long_kernel, dim3(1024), dim3(1024), 0, st, begin, map, sc.long_count,
                       sc.long_list, slot, static_cast<uint32_t>(B < (1LL << 31) ? B : 0xffffffffLL),
                       static_cast<uint32_t>(K));
    return;
  }
  hipLaunchKernelGGL(csr_init_kernel, dim3(grid_for(F + 1, 256, 4096)), dim3(256), 0, st, begin, F + 1,
                     sc.long_count);
  hipLaunchKernelGGL(csr_count_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st,
                     indices, n_pairs, F, begin, sc.rank, status_flag);
  const unsigned scan_blocks = static_cast<unsigned>(ceil_div(F, kScanBlockElems));
  hipLaunchKernelGGL(csr_scan_sums_kernel, dim3(scan_blocks), dim3(kScanThreads), 0, st, begin, F,
                     sc.block_sums);
  hipLaunchKernelGGL(csr_scan_apply_kernel, dim3(scan_blocks), dim3(kScanThreads), 0, st, begin, F,
                     sc.block_sums);
  hipLaunchKernelGGL(csr_fill_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, indices,
                     n_pairs, F, begin, sc.rank, map);
  hipLaunchKernelGGL(csr_sort_short_kernel,
                     dim3(static_cast<unsigned>(ceil_div(F, kWavesPerBlock))), dim3(kBlock), 0, st,
                     begin, map, F, sc.long_count, sc.long_list);
  hipLaunchKernelGGL(csr_sort_long_kernel, dim3(1024), dim3(1024), 0, st, begin, map, sc.long_count,
                     sc.long_list, static_cast<uint32_t *>(nullptr), static_cast<uint32_t>(B < (1LL << 31) ? B : 0xffffffffLL),
                     static_cast<uint32_t>(K));
  if (slot)
    hipLaunchKernelGGL(csr_inverse_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, map, n_pairs,
                       slot);
}

// Columns per tile of the training-step kernel: one register per gathered row piece, so 16-bit
// weights take two columns per lane (128-column tiles) and fp32 weights one once K exceeds 64.
inline int64_t train_tile_cols(const flexsae_shape *s) {
  return (s->weight_dtype == FLEXSAE_F32 && s->K > 64) ? 64 : 128;
}

// ---- two-phase hierarchical backward: workspace plan -----------------------------------

constexpr int kClsStride = 80;  // slots per counter array of the class list
static_assert(kSegClasses + 1 <= kClsStride, "a counter array holds one slot per class and the total");

// Most latents without a pair, the rest with few: the reduction by pieces then works from the list
// of latents ordered by row count and the rows of latents without pairs are zeroed in one pass.
// Whether that pays depends on how many latents really are without a pair: with two pairs per latent
// on average it does for skewed indices (two thirds of the latents empty: the step a sixth faster) and
// does not for uniform ones (an eighth of them empty: the step 8 % slower).  Only the caller can know,
// from an earlier step: FLEXSAE_BWD_DENSE_LATENTS says "most latents have pairs".
inline bool sparse_latents(const flexsae_shape *s, int flags = 0) {
  return !(flags & FLEXSAE_BWD_DENSE_LATENTS) && s->B * s->K <= 2 * s->F;
}

struct HierBwdPlan {
  int vec;                 // columns per lane
  int tile;                // 64 * vec columns per wavefront
  size_t p_size;           // bytes per element of the contribution matrix P
  int64_t d_pad;           // D rounded up to a whole number of tiles
  size_t n_pairs;          // B * K
  size_t n_rows;           // B
  size_t n_partial_rows;   // upper bound on the number of 64-pair chunks of long latents
  size_t off_begin, off_map, off_slot, off_csr, off_chunk, off_cls, off_cls_list, off_sfinal, off_colsum, off_loss, off_dvpart, off_partial;  // per-slice buffers follow
  size_t n_loss_partials;  // training-step kernel: one per (tile of 64 or 128 columns, row)
  size_t fixed_bytes;      // everything that does not depend on the slice width
  // hot-latent tables (only with `hot`): slots with the hot pairs marked, control words, the hot
  // latents, the candidates and what became of them, the long latents that stayed cold and their
  // chunk table
  bool hot;
  size_t off_hslot, off_hot_ctrl, off_hot_list, off_cand_list, off_cand_state, off_long_cand, off_long2, off_chunk2;
  size_t n_row_blocks;     // blocks of kHotRowsPerBlock rows
};

// Hot-latent accumulators: 16-bit weights of at most 64 steps (one register per row piece, four
// wavefronts per SIMD next to 144 KiB of accumulators) whose slices the piece reduction serves.
inline bool hot_supported(const flexsae_shape *s) {
  return s->D % 4 == 0 && s->K <= 64 && s->weight_dtype != FLEXSAE_F32 &&
         s->D % (s->weight_dtype == FLEXSAE_BF16 ? 8 : 4) == 0 && s->B * s->K < (1LL << 31);
}

HierBwdPlan plan_hier_bwd(const flexsae_shape *s, bool hot = false) {
  HierBwdPlan p;
  p.vec = (s->D % 4 == 0) ? 4 : (s->D % 2 == 0) ? 2 : 1;
  p.tile = kWave * p.vec;
  p.p_size = (s->weight_dtype == FLEXSAE_BF16) ? 2 : 4;  // bf16 weights: bf16 contributions
  p.d_pad = ceil_div(s->D, p.tile) * p.tile;
  p.n_pairs = static_cast<size_t>(s->B) * static_cast<size_t>(s->K);
  p.n_rows = static_cast<size_t>(s->B);
  p.n_partial_rows = p.n_pairs / kSegChunk + p.n_pairs / 65 + 2;
  size_t off = 0;
  p.off_begin = off;
  off += round_up(static_cast<size_t>(s->F + 1) * 4, kAlign);
  p.off_map = off;
  off += round_up(p.n_pairs * 4, kAlign);
  p.off_slot = off;
  off += round_up(p.n_pairs * 4, kAlign);
  p.off_csr = off;
  off += flexsae_csr_workspace_bytes(s->B, s->K, s->F);
  p.off_chunk = off;
  off += round_up((p.n_pairs / 65 + 2) * 4, kAlign);
  // latents ordered by row count (sparse shapes, see seg_class_scatter_kernel): three counter
  // arrays of kClsStride slots (histogram, cursors, first entry of every class) and the list
  p.off_cls = off;
  off += round_up(3 * static_cast<size_t>(kClsStride) * 4, kAlign);
  p.off_cls_list = off;
  off += round_up(static_cast<size_t>(s->F) * 4, kAlign);
  p.off_sfinal = off;  // S_{b,0} of every row, [B, d_pad] fp32: dbias is its column sum
  off += round_up(p.n_rows * static_cast<size_t>(p.d_pad) * 4, kAlign);
  p.off_colsum = off;  // partial column sums, [ceil(B/64), D] fp32
  off += round_up(static_cast<size_t>(ceil_div(s->B, kColsumRows)) * static_cast<size_t>(s->D) * 4, kAlign);
  p.off_loss = off;
  p.n_loss_partials = p.n_rows * static_cast<size_t>(p.d_pad / 64 + 1);
  off += round_up(p.n_loss_partials * 4, kAlign);
  // per-tile shares of dvals, [number of tiles, B*K] fp32, added up in tile order afterwards
  // (tiles are 64 or 128 columns in the training-step kernel, 64*vec in the sweep kernel)
  p.off_dvpart = off;
  const int64_t tt = train_tile_cols(s);
  off += round_up(static_cast<size_t>(p.d_pad / (p.tile < tt ? p.tile : tt)) * p.n_pairs * 4, kAlign);
  p.hot = hot;
  p.n_row_blocks = static_cast<size_t>(ceil_div(s->B, kHotRowsPerBlock));
  if (hot) {
    const size_t n_long_max = p.n_pairs / 65 + 2;
    p.off_hslot = off;
    off += round_up(p.n_pairs * 4, kAlign);
    p.off_hot_ctrl = off;
    off += round_up(kHotCtrlWords * 4, kAlign);
    p.off_hot_list = off;
    off += round_up(kHotMax * 4, kAlign);
    p.off_cand_list = off;
    off += round_up(kHotMax * 4, kAlign);
    p.off_cand_state = off;
    off += round_up(kHotMax * 4, kAlign);
    p.off_long_cand = off;
    off += round_up(n_long_max * 4, kAlign);
    p.off_long2 = off;
    off += round_up(n_long_max * 4, kAlign);
    p.off_chunk2 = off;
    off += round_up(n_long_max * 4, kAlign);
  }
  p.off_partial = off;
  p.fixed_bytes = off;
  return p;
}

// Slice granule (columns) of the training step.  The training-step kernel works on tiles of
// train_tile_cols(); when dW rows can be written 16 bytes per lane, the reduction works on
// 256-byte pieces of P (seg_reduce_piece_kernel) and a slice may be any number of training tiles
// wide; otherwise slices are whole reduction tiles (64 * vec columns).
inline int64_t piece_cols(const HierBwdPlan &p) { return kPieceBytes / static_cast<int64_t>(p.p_size); }

inline bool piece_reduce_ok(const flexsae_shape *s, const HierBwdPlan &p, const void *dW, int dW_dtype) {
  const int64_t ev = 16 / static_cast<int64_t>(p.p_size);  // columns per lane of the piece reduction
  return s->D % ev == 0 && train_tile_cols(s) % piece_cols(p) == 0 &&
         (dW == nullptr || aligned(dW, static_cast<size_t>(ev) * dtype_size(dW_dtype)));
}

// Columns the slice loop works on: D rounded up to whole reduction tiles, or to whole training tiles
// when the piece reduction lets slices end there.
inline int64_t hier_cols_used(const flexsae_shape *s, const HierBwdPlan &p, bool train, bool piece) {
  if (!(train && piece)) return p.d_pad;
  const int64_t tt = train_tile_cols(s);
  return ceil_div(s->D, tt) * tt;
}

// Forward-only inputs of the training-step variant of the slice loop (null = plain backward).
struct TrainArgs {
  const void *bias;
  const void *target;
  float *loss;              // finished by the epilogue from the per-(tile, row) partials
  int64_t n_loss_partials;
  double inv_count;         // 1 / (B*K*D)
};

// largest K the training-step kernel holds in registers
inline bool train_supported(const flexsae_shape *s) { return s->D % 4 == 0 && s->K <= 256; }

// Row pieces the training-step kernel keeps in the LDS instead of registers (one dword per lane
// and row: 16-bit weights with two columns per lane, fp32 with one), chosen so that one more
// wavefront fits each SIMD: 256 steps 216 instead of 276 registers (two wavefronts instead of one,
// 16 KB of LDS each), 128 steps 120 instead of 152 (four instead of three, 8 KB each), 64 steps 72
// instead of 88.
#ifndef FLEXSAE_LDS_256
#define FLEXSAE_LDS_256 64
#endif
#ifndef FLEXSAE_LDS_128
#define FLEXSAE_LDS_128 32
#endif
#ifndef FLEXSAE_LDS_64
#define FLEXSAE_LDS_64 16
#endif
template <typename WT, int KMAX, int VEC>
constexpr int train_lds_rows() {
  if (VEC * sizeof(typename Traits<WT>::store_t) != 4) return 0;
  return KMAX == 256 ? FLEXSAE_LDS_256 : KMAX == 128 ? FLEXSAE_LDS_128 : KMAX == 64 ? FLEXSAE_LDS_64 : 0;
}

template <typename WT, typename PT, int KMAX, int VEC = 2>
void launch_train_kernel(const flexsae_shape *s, const TrainArgs &ta, const int64_t *indices,
                         const void *weight, const void *vals, float coef, const uint32_t *slot, void *P,
                         float *dvals, float *s_final, int d_pad, float *loss_partial, int *status_flag,
                         int64_t cols, int col0, int slice_w, hipStream_t st, const HotFinalize &fin) {
  constexpr int LDSROWS = train_lds_rows<WT, KMAX, VEC>();
  const int64_t n_items = s->B * (cols / (kWave * VEC));
  // K == KMAX (the usual powers of two) runs the variant without per-step bound tests, part of its
  // row pieces in the LDS
  const bool stream = slice_w >= d_pad;  // all of P in one launch: streaming stores
  const auto kernel = s->K == KMAX
                          ? (stream ? hier_train_kernel<WT, PT, KMAX, true, true, VEC, LDSROWS>
                                    : hier_train_kernel<WT, PT, KMAX, true, false, VEC, LDSROWS>)
                          : (stream ? hier_train_kernel<WT, PT, KMAX, false, true, VEC, 0>
                                    : hier_train_kernel<WT, PT, KMAX, false, false, VEC, 0>);
  hipLaunchKernelGGL(kernel, dim3(fin.n_blocks + static_cast<unsigned>(ceil_div(n_items, kWavesPerBlock))), dim3(kBlock),
                     0, st, indices, weight, vals, s->vals_dtype, ta.bias, s->bias_dtype, ta.target, s->target_dtype,
                     coef, slot, P, dvals, s_final, d_pad, loss_partial, status_flag, n_items, s->B, col0,
                     slice_w, static_cast<int>(s->K), s->F, static_cast<int>(s->D), fin);
}

template <typename WT, typename PT>
void launch_train_kernel_k(const flexsae_shape *s, const TrainArgs &ta, const int64_t *indices,
                           const void *weight, const void *vals, float coef, const uint32_t *slot, void *P,
                           float *dvals, float *s_final, int d_pad, float *loss_partial,
                           int *status_flag, int64_t cols, int col0, int slice_w, hipStream_t st,
                           const HotFinalize &fin) {
#define FLEXSAE_TRAIN(KM)                                                                              \
  launch_train_kernel<WT, PT, KM>(s, ta, indices, weight, vals, coef, slot, P, dvals, s_final, d_pad,  \
                                  loss_partial, status_flag, cols, col0, slice_w, st, fin)
  // (the fp32 16-step instantiation allocates registers badly; 32 covers it)
  if (s->K <= 16 && sizeof(typename Traits<WT>::store_t) == 2) {
    FLEXSAE_TRAIN(16);
  } else if (s->K <= 32) {
    FLEXSAE_TRAIN(32);
  } else if (s->K <= 64) {
    FLEXSAE_TRAIN(64);
  } else if constexpr (sizeof(typename Traits<WT>::store_t) == 2) {
    if (s->K <= 128) {
      FLEXSAE_TRAIN(128);
    } else {  // 129..256 steps: two wavefronts per SIMD with 64 rows in the LDS (K = 256), else one
      FLEXSAE_TRAIN(256);
    }
  } else if (s->K <= 128) {  // fp32 rows of 65..128 steps: one column per lane
    launch_train_kernel<WT, PT, 128, 1>(s, ta, indices, weight, vals, coef, slot, P, dvals, s_final, d_pad,
                                        loss_partial, status_flag, cols, col0, slice_w, st, fin);
  } else {
    launch_train_kernel<WT, PT, 256, 1>(s, ta, indices, weight, vals, coef, slot, P, dvals, s_final, d_pad,
                                        loss_partial, status_flag, cols, col0, slice_w, st, fin);
  }
#undef FLEXSAE_TRAIN
}

// The training-step kernel with hot-latent accumulators (16-bit weights, K <= 64): one block per
// (row block, 128-column tile); every block first takes its share of the previous slice's second steps.
template <typename WT, typename PT>
void launch_train_hot_kernel(const flexsae_shape *s, const TrainArgs &ta, const int64_t *indices,
                             const void *weight, const void *vals, float coef, const uint32_t *hslot, void *P,
                             float *dvals, float *colsum_part, float *loss_partial, int *status_flag,
                             int64_t cols, int col0, int slice_w, hipStream_t st, HotFinalize fin,
                             const HotBlockFinalize &hfin, uint32_t *ctrl, float *hot_partial,
                             int n_row_blocks, int headroom) {
  if constexpr (sizeof(typename Traits<WT>::store_t) == 2) {
    const int n_tiles = static_cast<int>(cols / kHotCols);
    const unsigned grid = static_cast<unsigned>(n_tiles) * static_cast<unsigned>(n_row_blocks);
    if (fin.mode != 0) fin.n_blocks = grid;  // every block takes a share
    // 32-bit byte offsets from one descriptor per matrix where the matrices allow it
    const bool off32 = s->D % kHotCols == 0 &&
                       static_cast<uint64_t>(s->F) * s->D * sizeof(typename Traits<WT>::store_t) < (uint64_t{1} << 32) &&
                       static_cast<uint64_t>(s->B) * s->K * slice_w * sizeof(typename Traits<PT>::store_t) < (uint64_t{1} << 31);
#define FLEXSAE_TRAIN_HOT(KM)                                                                                   \
  do {                                                                                                          \
    const auto kernel = s->K == KM ? (off32 ? hier_train_hot_kernel<WT, PT, KM, true, true>                     \
                                            : hier_train_hot_kernel<WT, PT, KM, true, false>)                   \
                                   : (off32 ? hier_train_hot_kernel<WT, PT, KM, false, true>                    \
                                            : hier_train_hot_kernel<WT, PT, KM, false, false>);                 \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kHotThreads), 0, st, indices, weight, vals, s->vals_dtype, ta.bias, \
                       s->bias_dtype, ta.target, s->target_dtype, coef, hslot, P, dvals, colsum_part,           \
                       loss_partial, status_flag, s->B, n_tiles, n_row_blocks, col0, slice_w,                   \
                       static_cast<int>(s->K), s->F, static_cast<int>(s->D), ctrl, hot_partial, headroom, fin, hfin); \
  } while (0)
    if (s->K <= 16) {
      FLEXSAE_TRAIN_HOT(16);
    } else if (s->K <= 32) {
      FLEXSAE_TRAIN_HOT(32);
    } else {
      FLEXSAE_TRAIN_HOT(64);
    }
#undef FLEXSAE_TRAIN_HOT
  }
}

// per-slice buffers after the fixed part: chunk partials[n_partial_rows, w] | P[B*K, w]
size_t hier_partial_bytes(const HierBwdPlan &p, int64_t slice_w) {
  return round_up(p.n_partial_rows * static_cast<size_t>(slice_w) * 4, kAlign);
}

size_t hier_p_bytes(const HierBwdPlan &p, int64_t slice_w) {
  return round_up(p.n_pairs * static_cast<size_t>(slice_w) * p.p_size, kAlign);
}

// one buffer of block partials of the hot latents: [tiles of the slice][row blocks][kHotMax][128] fp32
size_t hier_hot_partial_bytes(const HierBwdPlan &p, int64_t slice_w) {
  return round_up(static_cast<size_t>(ceil_div(slice_w, kHotCols)) * p.n_row_blocks * kHotMax * kHotCols * 4, kAlign);
}

// ... | chunk partials | P | (hot: two buffers of block partials, used by alternate slices)
size_t hier_bwd_bytes(const HierBwdPlan &p, int64_t slice_w) {
  return p.fixed_bytes + hier_partial_bytes(p, slice_w) + hier_p_bytes(p, slice_w) +
         (p.hot ? 2 * hier_hot_partial_bytes(p, slice_w) : 0);
}

// Segment reduction of one slice plus the finalize step of its hot latents.  fp32 contributions
// are read 16 bytes per lane (256-column tiles), or, when `narrow`, 8 bytes per lane (128-column
// tiles, twice the wavefronts): faster once a latent has about four rows or more, slower for
// shorter groups.
template <typename PT, typename GT, int VEC>
void launch_seg_reduce(bool narrow, const uint32_t *begin, const CsrScratch &sc, const uint32_t *chunk_begin,
                       const void *P, float *partial, void *dW, const float *dw_scale, int64_t F, int tps,
                       int col0, int sw, int D, hipStream_t st, int piece_cols = 0, int64_t cols = 0, int64_t n_pairs = 0,
                       int update = 0, const uint32_t *cls_begin = nullptr, const uint32_t *cls_list = nullptr,
                       HotFinalize *defer = nullptr) {
  // the second step of the hot latents: launched here, or handed back through `defer` for the next
  // training-step launch to carry
  auto finalize = [&](int mode, int units) {
    HotFinalize h = {sc.long_count, sc.long_list, chunk_begin, partial, dW, dw_scale, mode, units, col0, sw, D, update, 256u};
    if (defer) {
      h.n_blocks = 64u;  // riding along with a long launch: few blocks, so that they cost little where there is nothing to do
      *defer = h;
    }
    else
      hipLaunchKernelGGL((hot_finalize_kernel<GT>), dim3(h.n_blocks), dim3(kBlock), 0, st, h);
  };
  if (piece_cols > 0) {  // 256-byte pieces, sixteen lanes each
    const int pps = static_cast<int>(cols / piece_cols);
    int pps_shift = -1;  // log2(pps) when pps is a power of two
    for (int sh = 0; sh < 16; ++sh)
      if (pps == (1 << sh)) pps_shift = sh;
    // latents per group of lanes: four, taken from the list ordered by row count, where most latents
    // have no or few rows (with four rows per latent on average the bookkeeping already costs more
    // than the shorter launch saves); the list holds at most min(F, pairs) latents with rows
#define FLEXSAE_PIECE_REDUCE(G, N_ITEMS, CLS_LIST, CLS_BEGIN)                                                      \
  hipLaunchKernelGGL((seg_reduce_piece_kernel<PT, GT, FLEXSAE_PIECE_U, G>),                                        \
                     dim3(kLongBlocks +                                                                            \
                          static_cast<unsigned>(ceil_div((N_ITEMS) * pps, kBlock / kPieceLanes))),             \
                     dim3(kBlock), 0, st, begin, sc.long_count, sc.long_list, chunk_begin, P, partial, dW, dw_scale, \
                     F, kLongBlocks, pps, pps_shift, col0, sw, D, update, CLS_LIST, CLS_BEGIN)
    if (cls_list) {
      // work items of the list: one per latent with kSegBigRows rows or more, one per four others
      const int64_t n_listed_max = F < n_pairs ? F : n_pairs;
      const int64_t n_items_max = n_pairs / kSegBigRows + ceil_div(n_listed_max, 4) + 1;
      FLEXSAE_PIECE_REDUCE(4, n_items_max, cls_list, cls_begin);
    } else {
      FLEXSAE_PIECE_REDUCE(1, F, static_cast<const uint32_t *>(nullptr), static_cast<const uint32_t *>(nullptr));
    }
#undef FLEXSAE_PIECE_REDUCE
    // the chunk partials of hot latents are combined per 64-column piece
    finalize(1, static_cast<int>(cols / kWave));
    return;
  }
  constexpr bool kCanNarrow = sizeof(typename Traits<PT>::store_t) == 4 && VEC == 4;
  if (kCanNarrow && narrow) {
    constexpr int RV = kCanNarrow ? 2 : VEC;
    const int rtps = tps * (VEC / RV);
    const unsigned n_short_blocks = static_cast<unsigned>(ceil_div(F * rtps, kWavesPerBlock));
    hipLaunchKernelGGL((seg_reduce_kernel<PT, GT, RV, FLEXSAE_REDUCE_U>), dim3(kLongBlocks + n_short_blocks),
                       dim3(kBlock), 0, st, begin, sc.long_count, sc.long_list, chunk_begin, P, partial, dW, dw_scale,
                       F, kLongBlocks, rtps, col0, sw, D);
    static_assert(RV == 2 || !kCanNarrow, "the narrow reduction works on tiles of 128 columns");
    finalize(3, rtps);
    return;
  }
  const unsigned n_short_blocks = static_cast<unsigned>(ceil_div(F * tps, kWavesPerBlock));
  hipLaunchKernelGGL((seg_reduce_kernel<PT, GT, VEC, FLEXSAE_REDUCE_U>), dim3(kLongBlocks + n_short_blocks),
                     dim3(kBlock), 0, st, begin, sc.long_count, sc.long_list, chunk_begin, P, partial, dW, dw_scale, F,
                     kLongBlocks, tps, col0, sw, D);
  if constexpr (VEC == 4) {
    finalize(2, tps);
  } else {
    hipLaunchKernelGGL((seg_reduce_long_finalize_kernel<GT, VEC, 8>), dim3(256), dim3(kBlock), 0, st, sc.long_count,
                       sc.long_list, chunk_begin, partial, dW, dw_scale, tps, col0, sw, D);
  }
}

template <typename WT, typename PT, typename GT, int VEC>
void launch_hier_slices(const flexsae_shape *s, const HierBwdPlan &pl, int64_t slice_w,
                        const int64_t *indices, const void *weight, const void *vals,
                        const float *resid, const float *grad_out, float coef, void *dW,
                        float *dvals, float *dbias, uint8_t *ws, int flags, int *status_flag,
                        hipStream_t st, const TrainArgs *train = nullptr, int piece = 0) {
  const bool do_sweep = !(flags & FLEXSAE_BWD_REDUCE_ONLY);
  const bool do_reduce = !(flags & FLEXSAE_BWD_SWEEP_ONLY);
  // in-place weight update: `grad_out` is the step size and dW the weight matrix (piece reduction only)
  const int update = (flags & kBwdSgdUpdate) ? 1 : 0;
  const float *dw_scale = (flags & (FLEXSAE_BWD_SCALE_BY_GRAD_OUT | kBwdSgdUpdate)) ? grad_out : nullptr;
  const uint32_t *begin = reinterpret_cast<const uint32_t *>(ws + pl.off_begin);
  const uint32_t *slot = reinterpret_cast<const uint32_t *>(ws + pl.off_slot);
  const CsrScratch sc = carve_csr_scratch(ws + pl.off_csr, s->F, s->B * s->K);
  uint32_t *chunk_begin = reinterpret_cast<uint32_t *>(ws + pl.off_chunk);
  float *s_final = reinterpret_cast<float *>(ws + pl.off_sfinal);
  float *dv_part = reinterpret_cast<float *>(ws + pl.off_dvpart);
  float *colsum_part = reinterpret_cast<float *>(ws + pl.off_colsum);
  const int n_chunks = static_cast<int>(ceil_div(s->B, kColsumRows));
  const int d_pad = static_cast<int>(pl.d_pad);
  const int K = static_cast<int>(s->K), D = static_cast<int>(s->D);
  const int sw = static_cast<int>(slice_w);
  const bool narrow_reduce = s->B * s->K >= 4 * s->F;
  float *partial = reinterpret_cast<float *>(ws + pl.off_partial);
  void *P = ws + pl.off_partial + hier_partial_bytes(pl, slice_w);
  // Hot latents (training step only): their pairs are marked in hslot and accumulated by the
  // training-step kernel; the chunked part of the reduction then serves the long latents that stayed
  // cold, from a list and a chunk table of their own.
  const bool hot = (flags & kBwdHot) != 0 && pl.hot && train != nullptr;
  uint32_t *hot_ctrl = hot ? reinterpret_cast<uint32_t *>(ws + pl.off_hot_ctrl) : nullptr;
  const uint32_t *hot_list = hot ? reinterpret_cast<const uint32_t *>(ws + pl.off_hot_list) : nullptr;
  float *hot_partial[2] = {nullptr, nullptr};
  CsrScratch sc_cold = sc;  // the long latents the reduction serves
  if (hot) {
    uint8_t *base = static_cast<uint8_t *>(P) + hier_p_bytes(pl, slice_w);
    hot_partial[0] = reinterpret_cast<float *>(base);
    hot_partial[1] = reinterpret_cast<float *>(base + hier_hot_partial_bytes(pl, slice_w));
    sc_cold.long_count = hot_ctrl + kHotLong2Count;
    sc_cold.long_list = reinterpret_cast<uint32_t *>(ws + pl.off_long2);
    chunk_begin = reinterpret_cast<uint32_t *>(ws + pl.off_chunk2);
  }
  const int hot_headroom = (flags & FLEXSAE_BWD_HOT_NO_HEADROOM) ? -6 : 2;
  // columns that are worked on: whole reduction tiles, or, with the piece reduction, whole training
  // tiles (tiles that lie entirely beyond column D are left out, and so are their shares below)
  const int64_t d_used = hier_cols_used(s, pl, train != nullptr, piece != 0);
  // The sweep kernel's tile (64 * sweep_vec columns per wavefront): narrower than the reduction's
  // when a slice would otherwise hold too few wavefronts to cover the memory latency (small B).
  // (not below the tile width the per-tile dvals shares of the workspace are laid out for)
  int sweep_vec = VEC;
  const int min_sweep_vec = static_cast<int>((pl.tile < train_tile_cols(s) ? pl.tile : train_tile_cols(s)) / kWave);
  while (sweep_vec > 1 && sweep_vec > min_sweep_vec && s->B * (slice_w / (kWave * sweep_vec)) < 6144) sweep_vec >>= 1;
  // Sparse shapes reduce every slice by pieces from the list of latents ordered by row count; the
  // rows of latents without pairs are zeroed here, whole rows in one pass (the in-place update leaves
  // them alone).
  const bool sparse = piece != 0 && sparse_latents(s, flags);
  const uint32_t *cls_begin = reinterpret_cast<const uint32_t *>(ws + pl.off_cls) + 2 * kClsStride;
  const uint32_t *cls_list = reinterpret_cast<const uint32_t *>(ws + pl.off_cls_list);
  if (sparse && do_reduce && !update)
    hipLaunchKernelGGL((seg_zero_rows_kernel<PT, GT>), dim3(2048), dim3(kBlock), 0, st, cls_begin, cls_list, dW, D);
  // In the training step the second step of a slice's hot latents travels with the next slice's
  // training-step launch (a gradient of the weight's own dtype only: that is what that kernel writes);
  // the last slice's gets a launch of its own.
  HotFinalize pending = {};
  HotBlockFinalize pending_hot = {};
  const bool fold = std::is_same<GT, WT>::value && train != nullptr && do_sweep && do_reduce;
  int slice_no = 0;
  for (int64_t col0 = 0; col0 < s->D; col0 += slice_w, ++slice_no) {
    const int64_t cols = (d_used - col0) < slice_w ? (d_used - col0) : slice_w;
    const int tps = static_cast<int>(cols / pl.tile);
    if (train && do_sweep && hot) {
      launch_train_hot_kernel<WT, PT>(s, *train, indices, weight, vals, coef,
                                      reinterpret_cast<const uint32_t *>(ws + pl.off_hslot), P, dv_part, colsum_part,
                                      reinterpret_cast<float *>(ws + pl.off_loss), status_flag, cols,
                                      static_cast<int>(col0), sw, st, pending, pending_hot, hot_ctrl,
                                      hot_partial[slice_no & 1], static_cast<int>(pl.n_row_blocks), hot_headroom);
      pending = HotFinalize{};
      pending_hot = HotBlockFinalize{};
    } else if (train && do_sweep) {
      launch_train_kernel_k<WT, PT>(s, *train, indices, weight, vals, coef, slot, P, dv_part, s_final, d_pad,
                                    reinterpret_cast<float *>(ws + pl.off_loss), status_flag, cols,
                                    static_cast<int>(col0), sw, st, pending);
      pending = HotFinalize{};
    } else if (do_sweep) {
#define FLEXSAE_SWEEP(SV)                                                                                      \
  hipLaunchKernelGGL((hier_sweep_kernel<WT, PT, SV, FLEXSAE_SWEEP_U>),                                         \
                     dim3(static_cast<unsigned>(ceil_div(s->B * (cols / (kWave * SV)), kWavesPerBlock))),      \
                     dim3(kBlock), 0, st, indices, weight, vals, s->vals_dtype, resid, grad_out, coef, slot, P, \
                     dv_part, s_final, d_pad, status_flag, s->B * (cols / (kWave * SV)), s->B,                 \
                     static_cast<int>(col0), sw, K, s->F, D)
      if (sweep_vec == VEC) {
        FLEXSAE_SWEEP(VEC);
      } else if (sweep_vec == (VEC >= 2 ? VEC / 2 : 1)) {
        FLEXSAE_SWEEP((VEC >= 2 ? VEC / 2 : 1));
      } else {
        FLEXSAE_SWEEP(1);
      }
#undef FLEXSAE_SWEEP
    }
    if (!do_reduce) continue;
    // Pieces where the slice is not made of whole reduction tiles, where most latents are empty
    // (four latents per group of lanes), for the in-place update, and where a slice of
    // contributions is about the size of the memory-side cache (measured 1 % faster there); else one
    // wavefront per (latent, reduction tile), which wastes no load slots on the unequal row counts
    // of the four latents a wavefront would otherwise share (4 % faster on slices read from HBM).
    const bool cache_sized = static_cast<size_t>(s->B * s->K) * static_cast<size_t>(sw) * pl.p_size <= (size_t{384} << 20);
    const bool by_pieces =
        piece != 0 && (update || cols % pl.tile != 0 || sparse_latents(s, flags) || cache_sized);
    launch_seg_reduce<PT, GT, VEC>(narrow_reduce, begin, sc_cold, chunk_begin, P, partial, dW, dw_scale, s->F, tps,
                                   static_cast<int>(col0), sw, D, st, by_pieces ? piece : 0, cols, s->B * s->K, update,
                                   sparse ? cls_begin : nullptr, sparse ? cls_list : nullptr, fold ? &pending : nullptr);
    if (hot) {
      // the block partials of the slice's hot latents are added up by the next training-step launch
      // (they live in the buffer that launch does not write), or here
      const HotBlockFinalize h = {hot_ctrl, hot_list, hot_partial[slice_no & 1], dW, dw_scale,
                                  static_cast<int>(cols / kHotCols), static_cast<int>(pl.n_row_blocks),
                                  static_cast<int>(col0), D, update};
      if (fold)
        pending_hot = h;
      else
        hipLaunchKernelGGL((hot_block_finalize_kernel<GT>), dim3(256), dim3(kBlock), 0, st, h);
    }
  }
  if (pending.n_blocks != 0) {
    pending.n_blocks = 256u;
    hipLaunchKernelGGL((hot_finalize_kernel<GT>), dim3(pending.n_blocks), dim3(kBlock), 0, st, pending);
  }
  if (pending_hot.ctrl != nullptr)
    hipLaunchKernelGGL((hot_block_finalize_kernel<GT>), dim3(256), dim3(kBlock), 0, st, pending_hot);
  if (!do_sweep) return;
  if (!do_reduce && !train) return;  // measurement aid of the plain backward: sweep kernels only
  if (flags & FLEXSAE_BWD_SKIP_EPILOGUE) return;
  // one launch: dvals = its per-tile shares added in tile order; stage 1 of dbias = column sums of
  // s_final over the rows, in a fixed order; the loss of the training step from its partials
  {
    // (the hot-latent training step has formed stage 1 of the column sums on chip)
    const unsigned n_colsum_blocks = hot ? 0u : static_cast<unsigned>(ceil_div(D, 256) * ceil_div(n_chunks, 4));
    const unsigned n_dvals_blocks = grid_for(s->B * s->K, 1024, 2048);
    hipLaunchKernelGGL(hier_epilogue_kernel, dim3(1 + n_colsum_blocks + n_dvals_blocks), dim3(1024), 0, st,
                       train ? reinterpret_cast<const float *>(ws + pl.off_loss) : static_cast<const float *>(nullptr),
                       train ? train->n_loss_partials : 0, train ? train->inv_count : 0.0,
                       train ? train->loss : static_cast<float *>(nullptr), s_final, s->B,
                       static_cast<int64_t>(d_pad), D, colsum_part, n_colsum_blocks, dv_part,
                       static_cast<int>(d_used / (train ? train_tile_cols(s) : kWave * sweep_vec)), s->B * s->K, dvals);
  }
  // (one partial per block of kHotRowsPerBlock rows from the hot-latent step, else per chunk of kColsumRows)
  hipLaunchKernelGGL(colsum_final_kernel, dim3(static_cast<unsigned>(ceil_div(D, 256))), dim3(256), 0, st,
                     colsum_part, hot ? static_cast<int>(pl.n_row_blocks) : n_chunks, D,
                     static_cast<const float *>(nullptr), 1.0f, dbias);
}

template <typename WT, typename PT, int VEC>
void launch_hier_slices_g(const flexsae_shape *s, const HierBwdPlan &pl, int64_t slice_w,
                          const int64_t *indices, const void *weight, const void *vals,
                          const float *resid, const float *grad_out, float coef, void *dW,
                          int dW_dtype, float *dvals, float *dbias, uint8_t *ws, int flags,
                          int *status_flag, hipStream_t st, const TrainArgs *train, int piece) {
  switch (dW_dtype) {
    case FLEXSAE_F32:
      launch_hier_slices<WT, PT, float, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                             coef, dW, dvals, dbias, ws, flags, status_flag, st, train, piece);
      break;
    case FLEXSAE_BF16:
      launch_hier_slices<WT, PT, bf16_t, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                              coef, dW, dvals, dbias, ws, flags, status_flag, st, train, piece);
      break;
    default:
      launch_hier_slices<WT, PT, f16_t, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                             coef, dW, dvals, dbias, ws, flags, status_flag, st, train, piece);
  }
}

template <int VEC>
void launch_hier_slices_w(const flexsae_shape *s, const HierBwdPlan &pl, int64_t slice_w,
                          const int64_t *indices, const void *weight, const void *vals,
                          const float *resid, const float *grad_out, float coef, void *dW,
                          int dW_dtype, float *dvals, float *dbias, uint8_t *ws, int flags,
                          int *status_flag, hipStream_t st, const TrainArgs *train = nullptr, int piece = 0) {
  switch (s->weight_dtype) {
    case FLEXSAE_F32:
      launch_hier_slices_g<float, float, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                              coef, dW, dW_dtype, dvals, dbias, ws, flags, status_flag, st, train, piece);
      break;
    case FLEXSAE_BF16:
      launch_hier_slices_g<bf16_t, bf16_t, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                                coef, dW, dW_dtype, dvals, dbias, ws, flags, status_flag, st, train, piece);
      break;
    default:
      launch_hier_slices_g<f16_t, float, VEC>(s, pl, slice_w, indices, weight, vals, resid, grad_out,
                                              coef, dW, dW_dtype, dvals, dbias, ws, flags, status_flag, st, train, piece);
  }
}

// What follows the pair list in a hierarchical workspace: the chunk table of the hot latents and, for
// sparse shapes, the list of latents ordered by row count.
void finish_pair_list(const flexsae_shape *s, const HierBwdPlan &pl, uint8_t *ws, const uint32_t *begin,
                      const CsrScratch &sc, hipStream_t st, int flags = 0) {
  uint32_t *cls = reinterpret_cast<uint32_t *>(ws + pl.off_cls);
  const bool sparse = sparse_latents(s, flags);
  hipLaunchKernelGGL(seg_chunk_table_kernel, dim3(1), dim3(1024), 0, st, begin, sc.long_count, sc.long_list,
                     reinterpret_cast<uint32_t *>(ws + pl.off_chunk), sparse ? cls : static_cast<uint32_t *>(nullptr),
                     2 * kClsStride);
  if (!sparse) return;
  // few blocks: every block ends with one memory atomic per class it met, all on the same counters
  hipLaunchKernelGGL(seg_class_hist_kernel, dim3(grid_for(s->F, 256, 128)), dim3(256), 0, st, begin, s->F, cls);
  hipLaunchKernelGGL(seg_class_scatter_kernel, dim3(static_cast<unsigned>(ceil_div(s->F, 256 * kClassPerThread))),
                     dim3(256), 0, st, begin, s->F, cls, cls + kClsStride, cls + 2 * kClsStride,
                     reinterpret_cast<uint32_t *>(ws + pl.off_cls_list));
}

// Hot-latent tables of a workspace whose pair list is complete: the slots with the hot pairs marked,
// the hot latents, the long latents that stayed cold and their chunk table.
void build_hot_tables(const flexsae_shape *s, const HierBwdPlan &pl, uint8_t *ws, const CsrScratch &sc, hipStream_t st) {
  const uint32_t *begin = reinterpret_cast<const uint32_t *>(ws + pl.off_begin);
  const uint32_t *map = reinterpret_cast<const uint32_t *>(ws + pl.off_map);
  uint32_t *hslot = reinterpret_cast<uint32_t *>(ws + pl.off_hslot);
  uint32_t *ctrl = reinterpret_cast<uint32_t *>(ws + pl.off_hot_ctrl);
  uint32_t *hot_list = reinterpret_cast<uint32_t *>(ws + pl.off_hot_list);
  uint32_t *cand_list = reinterpret_cast<uint32_t *>(ws + pl.off_cand_list);
  uint32_t *cand_state = reinterpret_cast<uint32_t *>(ws + pl.off_cand_state);
  uint32_t *long_cand = reinterpret_cast<uint32_t *>(ws + pl.off_long_cand);
  uint32_t *long2 = reinterpret_cast<uint32_t *>(ws + pl.off_long2);
  const int64_t n_pairs = s->B * s->K;
  hipLaunchKernelGGL(copy_u32_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, hslot,
                     reinterpret_cast<const uint32_t *>(ws + pl.off_slot), n_pairs);
  hipLaunchKernelGGL(hot_select_kernel, dim3(1), dim3(1024), 0, st, begin, sc.long_count, sc.long_list, ctrl,
                     cand_list, long_cand, static_cast<uint32_t>(kHotMax));
  hipLaunchKernelGGL(hot_mark_kernel, dim3(kHotMax), dim3(1024), 0, st, begin, map, ctrl, cand_list, cand_state,
                     hot_list, hslot, static_cast<uint32_t>(s->K));
  hipLaunchKernelGGL(hot_cold_long_kernel, dim3(64), dim3(256), 0, st, sc.long_count, sc.long_list, long_cand,
                     cand_state, ctrl, long2);
  hipLaunchKernelGGL(seg_chunk_table_kernel, dim3(1), dim3(1024), 0, st, begin, ctrl + kHotLong2Count, long2,
                     reinterpret_cast<uint32_t *>(ws + pl.off_chunk2), static_cast<uint32_t *>(nullptr), 0);
}

// ---- TopK backward: workspace plan and slice loop ---------------------------------------

struct TopkBwdPlan {
  int vec, tile;
  int64_t d_pad;
  size_t n_pairs, n_partial_rows;
  size_t off_colsum, off_long_count, off_long_list, off_chunk, off_resid16, off_dvpart, off_slotbv, off_partial, fixed_bytes;
  bool resid16;  // gather a bf16 copy of the residual (bf16 weights): half the cache footprint
};

TopkBwdPlan plan_topk_bwd(const flexsae_shape *s, int flags = 0) {
  TopkBwdPlan p;
  // The reference hands its backward the residual gradient in the weight dtype
  // (topk_kernels.py:52,221); for bf16 weights the gathers here read a bf16 copy as well, unless
  // the caller asks for the fp32 residual (no copy, but narrower tiles and so more per-tile dvals
  // shares: flexsae_topk_bwd_workspace_bytes returns the larger of the two layouts).
  p.resid16 = FLEXSAE_TOPK_RESID16 && s->weight_dtype == FLEXSAE_BF16 && !(flags & FLEXSAE_TOPK_BWD_FP32_RESIDUAL);
  p.vec = (s->D % 4 == 0) ? 4 : (s->D % 2 == 0) ? 2 : 1;
  // all-bf16: 16 bytes per lane (512-column tiles) halve the per-tile overheads
  if (FLEXSAE_TOPK_VEC8 && p.resid16 && s->D % 8 == 0) p.vec = 8;
  p.tile = kWave * p.vec;
  p.d_pad = ceil_div(s->D, p.tile) * p.tile;
  p.n_pairs = static_cast<size_t>(s->B) * static_cast<size_t>(s->K);
  p.n_partial_rows = p.n_pairs / kSegChunk + p.n_pairs / 65 + 2;
  size_t off = 0;
  p.off_colsum = off;
  off += round_up(static_cast<size_t>(ceil_div(s->B, kColsumRows)) * static_cast<size_t>(s->D) * 4, kAlign);
  p.off_long_count = off;
  off += kAlign;
  p.off_long_list = off;
  off += round_up((p.n_pairs / 65 + 1) * 4, kAlign);
  p.off_chunk = off;
  off += round_up((p.n_pairs / 65 + 2) * 4, kAlign);
  p.off_resid16 = off;
  if (p.resid16) off += round_up(static_cast<size_t>(s->B) * static_cast<size_t>(s->D) * 2, kAlign);
  p.off_dvpart = off;  // per-tile shares of dvals: [d_pad / tile, B*K] fp32
  off += round_up(static_cast<size_t>(p.d_pad / p.tile) * p.n_pairs * 4, kAlign);
  p.off_slotbv = off;  // (batch row, val) of every pair in pair-list order
  off += round_up(p.n_pairs * 8, kAlign);
  p.off_partial = off;
  p.fixed_bytes = off;
  return p;
}

size_t topk_bwd_bytes(const TopkBwdPlan &p, int64_t slice_w) {
  return p.fixed_bytes + round_up(p.n_partial_rows * static_cast<size_t>(slice_w) * 4, kAlign);
}

template <typename WT, typename GT, typename RT, int VEC>
void launch_topk_slices(const flexsae_shape *s, const TopkBwdPlan &pl, int64_t slice_w,
                        const uint32_t *begin, const uint32_t *map, const void *weight,
                        const void *vals, const void *resid, const float *grad_out, float coef,
                        void *dW, float *dvals, uint8_t *ws, hipStream_t st) {
  const uint32_t *long_count = reinterpret_cast<const uint32_t *>(ws + pl.off_long_count);
  const uint32_t *long_list = reinterpret_cast<const uint32_t *>(ws + pl.off_long_list);
  const uint32_t *chunk_begin = reinterpret_cast<const uint32_t *>(ws + pl.off_chunk);
  float *partial = reinterpret_cast<float *>(ws + pl.off_partial);
  float *dv_part = reinterpret_cast<float *>(ws + pl.off_dvpart);
  const int64_t n_pairs = static_cast<int64_t>(pl.n_pairs);
  const int K = static_cast<int>(s->K), D = static_cast<int>(s->D), sw = static_cast<int>(slice_w);
  for (int64_t col0 = 0; col0 < s->D; col0 += slice_w) {
    const int64_t cols = (pl.d_pad - col0) < slice_w ? (pl.d_pad - col0) : slice_w;
    const int tps = static_cast<int>(cols / pl.tile);
    const int64_t n_short_blocks = ceil_div(s->F, static_cast<int64_t>(kWavesPerBlock));
    const size_t resid_bytes =
        static_cast<size_t>(s->B) * static_cast<size_t>(s->D) * sizeof(typename Traits<RT>::store_t);
    hipLaunchKernelGGL((topk_bwd_kernel<WT, GT, RT, VEC>),
                       dim3(kLongBlocks + static_cast<unsigned>(n_short_blocks), static_cast<unsigned>(tps)),
                       dim3(kBlock), 0, st, begin, map, long_count, long_list, chunk_begin,
                       reinterpret_cast<const vec_t<uint32_t, 2> *>(ws + pl.off_slotbv), weight, vals,
                       s->vals_dtype, resid, grad_out, coef, dW, dv_part, n_pairs, partial, kLongBlocks, tps,
                       static_cast<int>(col0), sw, s->F, K, D, static_cast<uint32_t>(resid_bytes));
    hipLaunchKernelGGL((seg_reduce_long_finalize_kernel<GT, VEC, 8>), dim3(256), dim3(kBlock), 0, st,
                       long_count, long_list, chunk_begin, partial, dW, static_cast<const float *>(nullptr), tps,
                       static_cast<int>(col0), sw, D);
  }
}

template <typename WT, typename RT, int VEC>
void launch_topk_slices_g(const flexsae_shape *s, const TopkBwdPlan &pl, int64_t slice_w,
                          const uint32_t *begin, const uint32_t *map, const void *weight,
                          const void *vals, const void *resid, const float *grad_out, float coef,
                          void *dW, int dW_dtype, float *dvals, uint8_t *ws, hipStream_t st) {
  switch (dW_dtype) {
    case FLEXSAE_F32:
      launch_topk_slices<WT, float, RT, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                             coef, dW, dvals, ws, st);
      break;
    case FLEXSAE_BF16:
      launch_topk_slices<WT, bf16_t, RT, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                              coef, dW, dvals, ws, st);
      break;
    default:
      launch_topk_slices<WT, f16_t, RT, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                             coef, dW, dvals, ws, st);
  }
}

// `resid` is the fp32 residual, or its bf16 copy when the plan says so (bf16 weights only)
template <int VEC>
void launch_topk_slices_w(const flexsae_shape *s, const TopkBwdPlan &pl, int64_t slice_w,
                          const uint32_t *begin, const uint32_t *map, const void *weight,
                          const void *vals, const void *resid, const float *grad_out, float coef,
                          void *dW, int dW_dtype, float *dvals, uint8_t *ws, hipStream_t st) {
  switch (s->weight_dtype) {
    case FLEXSAE_F32:
      launch_topk_slices_g<float, float, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                              coef, dW, dW_dtype, dvals, ws, st);
      break;
    case FLEXSAE_BF16:
      if (pl.resid16)
        launch_topk_slices_g<bf16_t, bf16_t, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                                  coef, dW, dW_dtype, dvals, ws, st);
      else
        launch_topk_slices_g<bf16_t, float, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                                 coef, dW, dW_dtype, dvals, ws, st);
      break;
    default:
      launch_topk_slices_g<f16_t, float, VEC>(s, pl, slice_w, begin, map, weight, vals, resid, grad_out,
                                              coef, dW, dW_dtype, dvals, ws, st);
  }
}

}  // namespace

extern "C" {

int flexsae_abi_version(void) { return FLEXSAE_ABI_VERSION; }

#ifndef FLEXSAE_BUILD_ID
#define FLEXSAE_BUILD_ID "unknown"
#endif
const char *flexsae_build_id(void) { return FLEXSAE_BUILD_ID; }

const char *flexsae_status_string(int status) {
  switch (status) {
    case FLEXSAE_OK:
      return "ok";
    case FLEXSAE_ERR_INVALID_ARGUMENT:
      return "invalid argument (null pointer, non-positive size or unknown dtype)";
    case FLEXSAE_ERR_UNSUPPORTED:
      return "unsupported size (need F, K < 2^31, D < 2^29 and B*K < 2^32)";
    case FLEXSAE_ERR_WORKSPACE:
      return "workspace missing, too small or not 256-byte aligned";
    case FLEXSAE_ERR_LAUNCH:
      return "HIP kernel launch failed";
    case FLEXSAE_ERR_ALIGNMENT:
      return "tensor pointer not aligned to its element size";
    case FLEXSAE_ERR_SCRATCH_LIMIT:
      return "problem too large for the static scratch of this entry point (use the variant that takes a workspace)";
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

int flexsae_hier_fwd_static(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                            const void *vals, const void *bias, const void *target, float *loss,
                            float *resid, int *status_flag, void *stream) {
  const int rc = check_shape(shape);
  if (rc != FLEXSAE_OK) return rc;
  if (flexsae_fwd_workspace_bytes(shape) > kStaticScratchBytes) return FLEXSAE_ERR_SCRATCH_LIMIT;
  void *ptr = nullptr;
  const int src = static_scratch_for_current_device(&ptr);
  if (src != FLEXSAE_OK) return src;
  // every partial the finalize kernel reads is written by the forward kernel of the same call:
  // nothing in the array has to start at zero
  return forward<true>(shape, indices, weight, vals, bias, target, loss, resid, ptr, kStaticScratchBytes,
                       status_flag, stream);
}

int flexsae_topk_fwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const void *bias, const void *target, float *loss,
                     float *resid, void *workspace, size_t workspace_bytes, int *status_flag,
                     void *stream) {
  return forward<false>(shape, indices, weight, vals, bias, target, loss, resid, workspace,
                        workspace_bytes, status_flag, stream);
}

int flexsae_hier_bwd_atomic(const flexsae_shape *s, const int64_t *indices, const void *weight,
                            const void *vals, const float *resid, const float *grad_out,
                            float *dW_acc, float *dvals, float *dbias, int flags, int *status_flag,
                            void *stream) {
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

size_t flexsae_hier_bwd_workspace_bytes(const flexsae_shape *s, int64_t slice_cols) {
  if (check_shape(s) != FLEXSAE_OK) return 0;
  const HierBwdPlan pl = plan_hier_bwd(s);
  int64_t sw = slice_cols <= 0 ? pl.tile : ceil_div(slice_cols, pl.tile) * pl.tile;
  if (sw > pl.d_pad) sw = pl.d_pad;
  return hier_bwd_bytes(pl, sw);
}

size_t flexsae_hier_fwd_bwd_workspace_bytes_flags(const flexsae_shape *s, int64_t slice_cols, int flags) {
  if (check_shape(s) != FLEXSAE_OK || !train_supported(s)) return 0;
  const bool hot = (flags & FLEXSAE_BWD_HOT_LATENTS) && hot_supported(s);
  const HierBwdPlan pl = plan_hier_bwd(s, hot);
  const int64_t granule = piece_reduce_ok(s, pl, nullptr, s->weight_dtype) ? train_tile_cols(s) : pl.tile;
  int64_t sw = slice_cols <= 0 ? granule : ceil_div(slice_cols, granule) * granule;
  if (sw > pl.d_pad) sw = pl.d_pad;
  return hier_bwd_bytes(pl, sw);
}

size_t flexsae_hier_fwd_bwd_workspace_bytes(const flexsae_shape *s, int64_t slice_cols) {
  return flexsae_hier_fwd_bwd_workspace_bytes_flags(s, slice_cols, 0);
}

int flexsae_hier_hot_latents_supported(const flexsae_shape *s) {
  return check_shape(s) == FLEXSAE_OK && train_supported(s) && hot_supported(s) ? 1 : 0;
}

int flexsae_hier_pair_stats(const flexsae_shape *s, const void *workspace, uint32_t *stats, void *stream) {
  const int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!workspace || !stats) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(workspace, kAlign) || !aligned(stats, 4)) return FLEXSAE_ERR_ALIGNMENT;
  const HierBwdPlan pl = plan_hier_bwd(s);  // the part of the layout every hierarchical workspace shares
  uint8_t *ws = static_cast<uint8_t *>(const_cast<void *>(workspace));
  const CsrScratch sc = carve_csr_scratch(ws + pl.off_csr, s->F, s->B * s->K);
  hipLaunchKernelGGL(pair_stats_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const uint32_t *>(ws + pl.off_begin), s->F, sc.long_count,
                     reinterpret_cast<const uint32_t *>(ws + pl.off_chunk), stats);
  return launch_status();
}

int flexsae_hier_hot_stats(const flexsae_shape *s, const void *workspace, uint32_t *stats, void *stream) {
  const int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!workspace || !stats) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!train_supported(s) || !hot_supported(s)) return FLEXSAE_ERR_UNSUPPORTED;
  if (!aligned(workspace, kAlign) || !aligned(stats, 4)) return FLEXSAE_ERR_ALIGNMENT;
  const HierBwdPlan pl = plan_hier_bwd(s, true);
  const uint32_t *ctrl = reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(workspace) + pl.off_hot_ctrl);
  static_assert(kHotNHot == 0 && kHotNCand == 1 && kHotLong2Count == 2 && kHotThreshold == 3 && kHotDeferred == 4,
                "flexsae_hier_hot_stats hands out the first five control words");
  hipLaunchKernelGGL(copy_u32_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), stats, ctrl,
                     static_cast<int64_t>(5));
  return launch_status();
}

int flexsae_hier_bwd(const flexsae_shape *s, const int64_t *indices, const void *weight,
                     const void *vals, const float *resid, const float *grad_out, void *dW,
                     int dW_dtype, float *dvals, float *dbias, void *workspace,
                     size_t workspace_bytes, int flags, int *status_flag, void *stream) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!grad_out || !dW || !valid_dtype(dW_dtype)) return FLEXSAE_ERR_INVALID_ARGUMENT;
  const HierBwdPlan pl = plan_hier_bwd(s);
  if (!workspace || !aligned(workspace, kAlign) || workspace_bytes < hier_bwd_bytes(pl, pl.tile))
    return FLEXSAE_ERR_WORKSPACE;
  // widest slice (whole tiles) the workspace can hold
  int64_t slice_w = pl.tile;
  while (slice_w + pl.tile <= pl.d_pad && hier_bwd_bytes(pl, slice_w + pl.tile) <= workspace_bytes)
    slice_w += pl.tile;
  // REDUCE_ONLY on a kept pair list: with a single-slice workspace this is the deferred reduction
  // of staged contributions, which only reads the workspace and writes dW; on a sliced workspace
  // it is the reduction phase of every slice (profiling), which still needs the other arguments
  const bool reduce_only = (flags & FLEXSAE_BWD_REDUCE_ONLY) && (flags & FLEXSAE_BWD_REUSE_PAIR_LIST) &&
                           slice_w >= pl.d_pad;
  if (!reduce_only && (!indices || !weight || !vals || !resid || !dvals || !dbias))
    return (flags & FLEXSAE_BWD_SCALE_BY_GRAD_OUT) ? FLEXSAE_ERR_WORKSPACE : FLEXSAE_ERR_INVALID_ARGUMENT;
  if ((flags & FLEXSAE_BWD_SCALE_BY_GRAD_OUT) && !reduce_only)
    return slice_w < pl.d_pad ? FLEXSAE_ERR_WORKSPACE : FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(grad_out, 4) || !aligned(dW, pl.vec * dtype_size(dW_dtype))) return FLEXSAE_ERR_ALIGNMENT;
  if (!reduce_only &&
      (!aligned(indices, 8) || !aligned(weight, pl.vec * dtype_size(s->weight_dtype)) ||
       !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(resid, pl.vec * 4) || !aligned(dvals, 16) ||
       !aligned(dbias, 16)))
    return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  uint32_t *begin = reinterpret_cast<uint32_t *>(ws + pl.off_begin);
  uint32_t *map = reinterpret_cast<uint32_t *>(ws + pl.off_map);
  const CsrScratch sc = carve_csr_scratch(ws + pl.off_csr, s->F, s->B * s->K);
  if (!(flags & FLEXSAE_BWD_REUSE_PAIR_LIST)) {
    csr_build_launch(indices, s->B, s->K, s->F, begin, map, reinterpret_cast<uint32_t *>(ws + pl.off_slot), sc,
                     status_flag, st);
    finish_pair_list(s, pl, ws, begin, sc, st, flags);
  }
  const float coef = static_cast<float>(
      2.0 / (static_cast<double>(s->B) * static_cast<double>(s->K) * static_cast<double>(s->D)));
  if (pl.vec == 4) {
    launch_hier_slices_w<4>(s, pl, slice_w, indices, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                            dvals, dbias, ws, flags, status_flag, st);
  } else if (pl.vec == 2) {
    launch_hier_slices_w<2>(s, pl, slice_w, indices, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                            dvals, dbias, ws, flags, status_flag, st);
  } else {
    launch_hier_slices_w<1>(s, pl, slice_w, indices, weight, vals, resid, grad_out, coef, dW, dW_dtype,
                            dvals, dbias, ws, flags, status_flag, st);
  }
  return launch_status();
}

int flexsae_hier_pair_list_layout(const flexsae_shape *s, size_t *begin_offset, size_t *map_offset) {
  const int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!begin_offset || !map_offset) return FLEXSAE_ERR_INVALID_ARGUMENT;
  const HierBwdPlan pl = plan_hier_bwd(s);
  *begin_offset = pl.off_begin;
  *map_offset = pl.off_map;
  return FLEXSAE_OK;
}

int flexsae_hier_import_pair_list(const flexsae_shape *s, const uint32_t *begin, const uint32_t *map,
                                  void *workspace, size_t workspace_bytes, void *stream) {
  const int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!begin || !map) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!aligned(begin, 4) || !aligned(map, 4)) return FLEXSAE_ERR_ALIGNMENT;
  const HierBwdPlan pl = plan_hier_bwd(s);
  if (!workspace || !aligned(workspace, kAlign) || workspace_bytes < hier_bwd_bytes(pl, pl.tile))
    return FLEXSAE_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  uint32_t *ws_begin = reinterpret_cast<uint32_t *>(ws + pl.off_begin);
  uint32_t *ws_map = reinterpret_cast<uint32_t *>(ws + pl.off_map);
  const CsrScratch sc = carve_csr_scratch(ws + pl.off_csr, s->F, s->B * s->K);
  const int64_t n_pairs = s->B * s->K;
  if (ws_begin != begin)
    hipLaunchKernelGGL(copy_u32_kernel, dim3(grid_for(s->F + 1, 256, 4096)), dim3(256), 0, st, ws_begin, begin,
                       s->F + 1);
  if (ws_map != map)
    hipLaunchKernelGGL(copy_u32_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, ws_map, map, n_pairs);
  hipLaunchKernelGGL(csr_inverse_kernel, dim3(grid_for(n_pairs, 256, 8192)), dim3(256), 0, st, ws_map, n_pairs,
                     reinterpret_cast<uint32_t *>(ws + pl.off_slot));
  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, sc.long_count, static_cast<int64_t>(1), 0u);
  hipLaunchKernelGGL(seg_find_long_kernel, dim3(grid_for(s->F, 256, 2048)), dim3(256), 0, st, ws_begin, s->F,
                     sc.long_count, sc.long_list);
  finish_pair_list(s, pl, ws, ws_begin, sc, st);
  return launch_status();
}

int flexsae_hier_fwd_bwd_supported(const flexsae_shape *s) {
  return check_shape(s) == FLEXSAE_OK && train_supported(s) ? 1 : 0;
}

}  // extern "C"

namespace {

// flexsae_hier_fwd_bwd, or with `sgd_step` (a device scalar) flexsae_hier_sgd_step: dW is then the
// weight matrix itself and every touched row has step * (its unit-gradient row) subtracted.
int hier_fwd_bwd_impl(const flexsae_shape *s, const int64_t *indices, const void *weight,
                      const void *vals, const void *bias, const void *target, float *loss,
                      void *dW, int dW_dtype, float *dvals, float *dbias, void *workspace,
                      size_t workspace_bytes, int flags, int *status_flag, void *stream,
                      const float *sgd_step) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (sgd_step) {
    if (flags & (FLEXSAE_BWD_NO_DW | FLEXSAE_BWD_SWEEP_ONLY | FLEXSAE_BWD_REDUCE_ONLY | FLEXSAE_BWD_SKIP_EPILOGUE))
      return FLEXSAE_ERR_INVALID_ARGUMENT;
    if (!aligned(sgd_step, 4)) return FLEXSAE_ERR_ALIGNMENT;
  }
  const bool no_dw = (flags & FLEXSAE_BWD_NO_DW) != 0;
  const bool defer_reduce = (flags & FLEXSAE_BWD_SWEEP_ONLY) != 0 && !no_dw;
  if (!indices || !weight || !vals || !bias || !target || !loss || !dvals || !dbias ||
      (!defer_reduce && !no_dw && (!dW || !valid_dtype(dW_dtype))))
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (!train_supported(s)) return FLEXSAE_ERR_UNSUPPORTED;
  // hot-latent accumulators: a hint, taken where the shape allows them, the reductions run in this
  // call and every pointer is aligned for the piece reduction (the workspace layout depends on it)
  const bool hot = (flags & FLEXSAE_BWD_HOT_LATENTS) && hot_supported(s) && !defer_reduce &&
                   piece_reduce_ok(s, plan_hier_bwd(s), (defer_reduce || no_dw) ? nullptr : dW, dW_dtype);
  const HierBwdPlan pl = plan_hier_bwd(s, hot);  // D % 4 == 0 here, so tiles are 256 columns
  if (!aligned(indices, 8) || !aligned(weight, 4 * dtype_size(s->weight_dtype)) ||
      !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(bias, 2 * dtype_size(s->bias_dtype)) ||
      !aligned(target, 2 * dtype_size(s->target_dtype)) || !aligned(loss, 4) ||
      (!defer_reduce && !no_dw && !aligned(dW, 4 * dtype_size(dW_dtype))) || !aligned(dvals, 16) ||
      !aligned(dbias, 16))
    return FLEXSAE_ERR_ALIGNMENT;
  // slices are whole training tiles when the reduction can work on 256-byte pieces, else whole
  // reduction tiles
  const bool piece = piece_reduce_ok(s, pl, (defer_reduce || no_dw) ? nullptr : dW, dW_dtype);
  if (sgd_step && !piece) return FLEXSAE_ERR_UNSUPPORTED;  // only the piece reduction updates in place
  const int64_t granule = piece ? train_tile_cols(s) : pl.tile;
  if (!workspace || !aligned(workspace, kAlign) || workspace_bytes < hier_bwd_bytes(pl, granule))
    return FLEXSAE_ERR_WORKSPACE;
  int64_t slice_w = granule;
  while (slice_w + granule <= pl.d_pad && hier_bwd_bytes(pl, slice_w + granule) <= workspace_bytes)
    slice_w += granule;
  if (defer_reduce && slice_w < pl.d_pad) return FLEXSAE_ERR_WORKSPACE;  // contributions must all fit
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  uint32_t *begin = reinterpret_cast<uint32_t *>(ws + pl.off_begin);
  uint32_t *map = reinterpret_cast<uint32_t *>(ws + pl.off_map);
  const CsrScratch sc = carve_csr_scratch(ws + pl.off_csr, s->F, s->B * s->K);
  if (!(flags & FLEXSAE_BWD_REUSE_PAIR_LIST)) {
    csr_build_launch(indices, s->B, s->K, s->F, begin, map, reinterpret_cast<uint32_t *>(ws + pl.off_slot), sc,
                     status_flag, st);
    finish_pair_list(s, pl, ws, begin, sc, st, flags);
  }
  if (hot && !((flags & FLEXSAE_BWD_REUSE_PAIR_LIST) && (flags & FLEXSAE_BWD_REUSE_HOT_TABLES)))
    build_hot_tables(s, pl, ws, sc, st);
  const double count = static_cast<double>(s->B) * static_cast<double>(s->K) * static_cast<double>(s->D);
  const float coef = static_cast<float>(2.0 / count);
  const TrainArgs ta = {bias, target, loss, s->B * (hier_cols_used(s, pl, true, piece) / train_tile_cols(s)),
                        1.0 / count};
  // without dW the reductions are left out like in the deferred case (dW_dtype only selects a template then)
  launch_hier_slices_w<4>(s, pl, slice_w, indices, weight, vals, nullptr, sgd_step, coef, dW,
                          no_dw ? s->weight_dtype : dW_dtype, dvals, dbias, ws,
                          (flags & (FLEXSAE_BWD_SWEEP_ONLY | FLEXSAE_BWD_REDUCE_ONLY | FLEXSAE_BWD_SKIP_EPILOGUE |
                                    FLEXSAE_BWD_HOT_NO_HEADROOM | FLEXSAE_BWD_DENSE_LATENTS)) |
                              (no_dw ? FLEXSAE_BWD_SWEEP_ONLY : 0) | (sgd_step ? kBwdSgdUpdate : 0) | (hot ? kBwdHot : 0),
                          status_flag, st, &ta, piece ? static_cast<int>(piece_cols(pl)) : 0);
  return launch_status();
}

}  // namespace

extern "C" {

int flexsae_hier_fwd_bwd(const flexsae_shape *s, const int64_t *indices, const void *weight,
                         const void *vals, const void *bias, const void *target, float *loss,
                         void *dW, int dW_dtype, float *dvals, float *dbias, void *workspace,
                         size_t workspace_bytes, int flags, int *status_flag, void *stream) {
  return hier_fwd_bwd_impl(s, indices, weight, vals, bias, target, loss, dW, dW_dtype, dvals, dbias, workspace,
                           workspace_bytes, flags & ~(kBwdSgdUpdate | kBwdHot), status_flag, stream, nullptr);
}

int flexsae_hier_sgd_step(const flexsae_shape *s, const int64_t *indices, void *weight, const void *vals,
                          const void *bias, const void *target, const float *step, float *loss,
                          float *dvals, float *dbias, void *workspace, size_t workspace_bytes, int flags,
                          int *status_flag, void *stream) {
  if (!step || !s) return FLEXSAE_ERR_INVALID_ARGUMENT;
  return hier_fwd_bwd_impl(s, indices, weight, vals, bias, target, loss, weight, s->weight_dtype, dvals, dbias,
                           workspace, workspace_bytes,
                           flags & (FLEXSAE_BWD_REUSE_PAIR_LIST | FLEXSAE_BWD_HOT_LATENTS | FLEXSAE_BWD_REUSE_HOT_TABLES |
                                    FLEXSAE_BWD_HOT_NO_HEADROOM | FLEXSAE_BWD_DENSE_LATENTS),
                           status_flag, stream, step);
}

int flexsae_scale(void *dst, const void *src, int dtype, int64_t n, const float *scale, void *stream) {
  if (!dst || !src || !scale || n < 0 || !valid_dtype(dtype)) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (n == 0) return FLEXSAE_OK;
  if (!aligned(src, 4 * dtype_size(dtype)) || !aligned(dst, 4 * dtype_size(dtype)) || !aligned(scale, 4))
    return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(grid_for(ceil_div(n, 4), 256, 4096));  // few blocks: in place by one they all return at once
  switch (dtype) {
    case FLEXSAE_F32:
      hipLaunchKernelGGL(scale_kernel<float>, grid, dim3(256), 0, st, dst, src, n, scale);
      break;
    case FLEXSAE_BF16:
      hipLaunchKernelGGL(scale_kernel<bf16_t>, grid, dim3(256), 0, st, dst, src, n, scale);
      break;
    default:
      hipLaunchKernelGGL(scale_kernel<f16_t>, grid, dim3(256), 0, st, dst, src, n, scale);
  }
  return launch_status();
}

size_t flexsae_csr_workspace_bytes(int64_t B, int64_t K, int64_t F) {
  if (B <= 0 || K <= 0 || F <= 0) return 0;
  if (B > ((1LL << 32) - 1) / K) return 0;
  return csr_scratch_bytes(B * K, F, nullptr, nullptr);
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
  const CsrScratch sc = carve_csr_scratch(workspace, F, B * K);
  csr_build_launch(indices, B, K, F, begin, map, nullptr, sc, status_flag, static_cast<hipStream_t>(stream));
  return launch_status();
}

size_t flexsae_topk_bwd_workspace_bytes(const flexsae_shape *s, int64_t slice_cols) {
  if (check_shape(s) != FLEXSAE_OK) return 0;
  // The query takes no flags, so it covers both layouts of the call: the bf16-residual one (wide
  // tiles plus the bf16 copy of the residual) and the FLEXSAE_TOPK_BWD_FP32_RESIDUAL one (narrower
  // tiles: twice the per-tile dvals shares, which outweighs the copy once K exceeds 256).
  size_t need = 0;
  for (const int flags : {0, static_cast<int>(FLEXSAE_TOPK_BWD_FP32_RESIDUAL)}) {
    const TopkBwdPlan pl = plan_topk_bwd(s, flags);
    int64_t sw = slice_cols <= 0 ? pl.tile : ceil_div(slice_cols, pl.tile) * pl.tile;
    if (sw > pl.d_pad) sw = pl.d_pad;
    const size_t bytes = topk_bwd_bytes(pl, sw);
    if (bytes > need) need = bytes;
  }
  return need;
}

int flexsae_topk_bwd(const flexsae_shape *s, const uint32_t *begin, const uint32_t *map,
                     const int64_t *indices, const void *weight, const void *vals, const float *resid,
                     const float *grad_out, void *dW, int dW_dtype, float *dvals, float *dbias,
                     void *workspace, size_t workspace_bytes, int flags, void *stream) {
  int rc = check_shape(s);
  if (rc != FLEXSAE_OK) return rc;
  if (!begin || !map || !weight || !vals || !resid || !grad_out || !dW || !dvals || !dbias ||
      !valid_dtype(dW_dtype))
    return FLEXSAE_ERR_INVALID_ARGUMENT;
  // the residual rows are gathered through a 32-bit buffer descriptor
  if (static_cast<size_t>(s->B) * static_cast<size_t>(s->D) * 4 > 0xffffffffull) return FLEXSAE_ERR_UNSUPPORTED;
  const TopkBwdPlan pl = plan_topk_bwd(s, flags);
  if (!aligned(begin, 4) || !aligned(map, 4) || (indices && !aligned(indices, 8)) ||
      !aligned(weight, pl.vec * dtype_size(s->weight_dtype)) ||
      !aligned(vals, dtype_size(s->vals_dtype)) || !aligned(resid, pl.resid16 ? 16 : pl.vec * 4) ||
      !aligned(grad_out, 4) || !aligned(dW, pl.vec * dtype_size(dW_dtype)) || !aligned(dvals, 16) ||
      !aligned(dbias, 4))
    return FLEXSAE_ERR_ALIGNMENT;
  if (!workspace || !aligned(workspace, kAlign) || workspace_bytes < topk_bwd_bytes(pl, pl.tile))
    return FLEXSAE_ERR_WORKSPACE;
  int64_t slice_w = pl.tile;
  while (slice_w + pl.tile <= pl.d_pad && topk_bwd_bytes(pl, slice_w + pl.tile) <= workspace_bytes)
    slice_w += pl.tile;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t *ws = static_cast<uint8_t *>(workspace);
  // (every output element is written exactly once: nothing needs a zero-fill, whatever `flags` says)
  // latents with more than 64 pairs and their chunk table
  uint32_t *long_count = reinterpret_cast<uint32_t *>(ws + pl.off_long_count);
  uint32_t *long_list = reinterpret_cast<uint32_t *>(ws + pl.off_long_list);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, long_count, static_cast<int64_t>(1), 0u);
  hipLaunchKernelGGL(seg_find_long_kernel, dim3(grid_for(s->F, 256, 2048)), dim3(256), 0, st, begin, s->F,
                     long_count, long_list);
  hipLaunchKernelGGL(seg_chunk_table_kernel, dim3(1), dim3(1024), 0, st, begin, long_count, long_list,
                     reinterpret_cast<uint32_t *>(ws + pl.off_chunk), static_cast<uint32_t *>(nullptr), 0);
  const float coef =
      static_cast<float>(2.0 / (static_cast<double>(s->B) * static_cast<double>(s->D)));
  // per-pair records and, for bf16 weights, the bf16 copy of the residual: one launch
  const void *gather_src = pl.resid16 ? static_cast<const void *>(ws + pl.off_resid16) : resid;
  {
    const int64_t n_resid = pl.resid16 ? s->B * s->D : 0;
    const int64_t work = s->B * s->K > ceil_div(n_resid, 4) ? s->B * s->K : ceil_div(n_resid, 4);
    hipLaunchKernelGGL(topk_prepare_kernel, dim3(grid_for(work, 256, 1 << 16)), dim3(256), 0, st, map, indices,
                       s->F, vals, s->vals_dtype, s->B * s->K, static_cast<int>(s->K),
                       reinterpret_cast<vec_t<uint32_t, 2> *>(ws + pl.off_slotbv), resid, n_resid,
                       pl.resid16 ? static_cast<void *>(ws + pl.off_resid16) : nullptr);
  }
  if (pl.vec == 8) {
    launch_topk_slices_g<bf16_t, bf16_t, 8>(s, pl, slice_w, begin, map, weight, vals, gather_src, grad_out, coef,
                                            dW, dW_dtype, dvals, ws, st);
  } else if (pl.vec == 4) {
    launch_topk_slices_w<4>(s, pl, slice_w, begin, map, weight, vals, gather_src, grad_out, coef, dW,
                            dW_dtype, dvals, ws, st);
  } else if (pl.vec == 2) {
    launch_topk_slices_w<2>(s, pl, slice_w, begin, map, weight, vals, gather_src, grad_out, coef, dW,
                            dW_dtype, dvals, ws, st);
  } else {
    launch_topk_slices_w<1>(s, pl, slice_w, begin, map, weight, vals, gather_src, grad_out, coef, dW,
                            dW_dtype, dvals, ws, st);
  }
  hipLaunchKernelGGL(topk_dvals_finalize_kernel, dim3(grid_for(s->B * s->K, 256, 8192)), dim3(256), 0, st, map,
                     reinterpret_cast<const float *>(ws + pl.off_dvpart), static_cast<int>(pl.d_pad / pl.tile),
                     s->B * s->K, dvals);
  rc = launch_status();
  if (rc != FLEXSAE_OK) return rc;
  // dbias = coef * grad_out * column sums of resid, in a fixed order
  float *colsum_part = reinterpret_cast<float *>(ws + pl.off_colsum);
  const int n_chunks = static_cast<int>(ceil_div(s->B, kColsumRows));
  const int D = static_cast<int>(s->D);
  hipLaunchKernelGGL(colsum_partial_kernel,
                     dim3(static_cast<unsigned>(ceil_div(D, 256)), static_cast<unsigned>(n_chunks)), dim3(256),
                     0, st, resid, s->B, s->D, D, colsum_part);
  hipLaunchKernelGGL(colsum_final_kernel, dim3(static_cast<unsigned>(ceil_div(D, 256))), dim3(256), 0, st,
                     colsum_part, n_chunks, D, grad_out, coef, dbias);
  return launch_status();
}

int flexsae_scale_from_f32(void *dst, int dst_dtype, const float *src, int64_t n, const float *scale,
                           void *stream) {
  if (!dst || !src || n < 0 || !valid_dtype(dst_dtype)) return FLEXSAE_ERR_INVALID_ARGUMENT;
  if (n == 0) return FLEXSAE_OK;
  if (!aligned(src, 16) || !aligned(dst, 4 * dtype_size(dst_dtype)) || !aligned(scale, 4)) return FLEXSAE_ERR_ALIGNMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(grid_for(ceil_div(n, 4), 256, 1 << 16));
  switch (dst_dtype) {
    case FLEXSAE_F32:
      hipLaunchKernelGGL(cast_from_f32_kernel<float>, grid, dim3(256), 0, st, dst, src, n, scale);
      break;
    case FLEXSAE_BF16:
      hipLaunchKernelGGL(cast_from_f32_kernel<bf16_t>, grid, dim3(256), 0, st, dst, src, n, scale);
      break;
    default:
      hipLaunchKernelGGL(cast_from_f32_kernel<f16_t>, grid, dim3(256), 0, st, dst, src, n, scale);
  }
  return launch_status();
}

int flexsae_cast_from_f32(void *dst, int dst_dtype, const float *src, int64_t n, void *stream) {
  return flexsae_scale_from_f32(dst, dst_dtype, src, n, nullptr, stream);
}

}  // extern "C"
