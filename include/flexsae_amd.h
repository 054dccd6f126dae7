/*
 * flexsae_amd -- C ABI of the MI355X (gfx950) implementation of the fused SAE
 * decoder-loss path: TopK and HierarchicalTopK loss, forward and backward.
 *
 * Every entry point takes raw device pointers and sizes, launches its kernels on
 * the given HIP stream and returns immediately (no allocation, no
 * synchronisation, no host<->device copy, no global state -- except the static
 * scratch array of flexsae_hier_fwd_static).  Return value:
 * FLEXSAE_OK or a negative flexsae_status; nothing throws or aborts.
 *
 * Conventions shared by all entry points
 *   - Tensors are contiguous row-major: indices[B,K] int64, weight[F,D],
 *     vals[B,K], bias[D], target[B,D]; weight/vals/bias/target each carry their
 *     own flexsae_dtype (fp32, bf16 or fp16) and are upcast to fp32 on load; all
 *     arithmetic and accumulation is fp32.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - `status_flag` (may be NULL) is a device int that kernels OR bits into:
 *     FLEXSAE_FLAG_INDEX_RANGE when an index lies outside [0,F).  Such an index
 *     is treated as latent 0 with value 0 so that no kernel ever reads or writes
 *     outside the tensors; the caller decides when to look at the flag.
 *   - `grad_out` is a DEVICE pointer to the upstream fp32 scalar gradient; it is
 *     folded into the kernels' scale factor, so there is no separate pass that
 *     multiplies the gradients afterwards.
 *   - Workspaces must be 256-byte aligned; their contents need not be
 *     initialised and are garbage afterwards.
 *
 * "replaces" comments name the reference function (file:line under the reference
 * checkout, torch-ext/flex_sae/) whose work the entry point takes over.
 */
#ifndef FLEXSAE_AMD_H
#define FLEXSAE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLEXSAE_ABI_VERSION 3

typedef enum {
  FLEXSAE_OK = 0,
  FLEXSAE_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive size, bad enum      */
  FLEXSAE_ERR_UNSUPPORTED = -2,      /* size beyond what the kernels index (see below) */
  FLEXSAE_ERR_WORKSPACE = -3,        /* workspace missing, too small or misaligned     */
  FLEXSAE_ERR_LAUNCH = -4,           /* the HIP runtime refused a launch               */
  FLEXSAE_ERR_ALIGNMENT = -5,        /* a tensor pointer is not aligned to its element */
  FLEXSAE_ERR_SCRATCH_LIMIT = -6     /* problem beyond the static scratch of *_static  */
} flexsae_status;

typedef enum { FLEXSAE_F32 = 0, FLEXSAE_BF16 = 1, FLEXSAE_F16 = 2 } flexsae_dtype;

enum { FLEXSAE_FLAG_INDEX_RANGE = 1 };

/* flags for the backward entry points */
enum {
  FLEXSAE_BWD_OUTPUTS_PREZEROED = 1, /* caller already zero-filled the accumulators            */
  /* the hierarchical entry points that take a workspace: */
  FLEXSAE_BWD_REUSE_PAIR_LIST = 2,   /* the workspace still holds the pair list of a previous   */
                                     /* call with the same indices and shape: do not rebuild it */
  /* flexsae_hier_bwd (and, for measurements, flexsae_hier_fwd_bwd): */
  FLEXSAE_BWD_SWEEP_ONLY = 4,        /* run only the sweep kernels (contributions stay in the   */
                                     /* workspace; meaningful when one slice covers all of D)   */
  FLEXSAE_BWD_REDUCE_ONLY = 8,       /* run only the segment reductions on the contributions    */
                                     /* already in the workspace; with REUSE_PAIR_LIST and a    */
                                     /* single-slice workspace only grad_out, dW and workspace  */
                                     /* are read (the rest may be NULL): the deferred reduction */
  FLEXSAE_BWD_SCALE_BY_GRAD_OUT = 16,/* deferred reduction only: the contributions were made    */
                                     /* for a unit upstream gradient; multiply dW by grad_out[0]*/
  FLEXSAE_BWD_NO_DW = 32,            /* flexsae_hier_fwd_bwd only: dW is not wanted (may be     */
                                     /* NULL); the segment reductions are left out, whatever    */
                                     /* the width of the workspace, and nothing is deferred     */
  FLEXSAE_TOPK_BWD_FP32_RESIDUAL = 256, /* flexsae_topk_bwd with bf16 weights: gather the fp32  */
                                     /* residual instead of a bf16 copy of it (slower, and dvals */
                                     /* then carry fp32 rounding only instead of bf16's)         */
  FLEXSAE_BWD_HOT_LATENTS = 128,     /* flexsae_hier_fwd_bwd / flexsae_hier_sgd_step: give the  */
                                     /* most frequent latents of the batch accumulators in the  */
                                     /* LDS (see flexsae_hier_hot_latents_supported); a hint,   */
                                     /* ignored where the shape or the call does not allow it.  */
                                     /* The workspace must come from                            */
                                     /* flexsae_hier_fwd_bwd_workspace_bytes_flags(.., flags)   */
  FLEXSAE_BWD_REUSE_HOT_TABLES = 1024, /* with REUSE_PAIR_LIST and HOT_LATENTS: the workspace   */
                                     /* also still holds the hot-latent tables of a previous    */
                                     /* call with HOT_LATENTS on the same indices and shape     */
  FLEXSAE_BWD_DENSE_LATENTS = 2048,  /* a hint for shapes with at most two pairs per latent on   */
                                     /* average (B*K <= 2F), which by default reduce from a list */
                                     /* of the latents ordered by pair count and zero the rows  */
                                     /* of latents without pairs in one pass: most latents DO   */
                                     /* have pairs (uniform indices), so do not.  Same results, */
                                     /* bit for bit; 8 % faster where an eighth of the latents  */
                                     /* is empty, a sixth slower where two thirds are           */
                                     /* (flexsae_hier_pair_stats counts them).  A pair list     */
                                     /* built under this flag has no such list: REUSE_PAIR_LIST */
                                     /* on it needs the flag again                              */
  FLEXSAE_BWD_HOT_NO_HEADROOM = 512, /* NOT PART OF THE STABLE ABI (a test aid): the block      */
                                     /* exponent of the hot-latent accumulators is set 8 bits   */
                                     /* lower than usual, so that most rows take the deferred   */
                                     /* second pass; results stay valid                         */
  FLEXSAE_BWD_SKIP_EPILOGUE = 64     /* NOT PART OF THE STABLE ABI (a measurement aid of this   */
                                     /* library's own benchmark, with no counterpart in the     */
                                     /* reference; may change or go without an ABI bump).       */
                                     /* flexsae_hier_fwd_bwd: leave out the kernels that finish */
                                     /* loss, dvals and dbias (those outputs are then not       */
                                     /* written), so that a call with NO_DW or SWEEP_ONLY runs  */
                                     /* the training-step kernel alone                          */
};

/* Problem description.  Limits: 1 <= B,K,F,D; F < 2^31; D < 2^29; B*K < 2^32. */
typedef struct {
  int64_t B, K, F, D;
  int32_t weight_dtype, vals_dtype, bias_dtype, target_dtype; /* flexsae_dtype */
} flexsae_shape;

int flexsae_abi_version(void);
/* Identifier of the sources and compiler flags the library was built from (a 16-digit hash set by
 * the build script; "unknown" for other builds): lets a stored measurement name the build it is of. */
const char *flexsae_build_id(void);
const char *flexsae_status_string(int status);

/* Bytes of workspace the two forward entry points need for `shape`. */
size_t flexsae_fwd_workspace_bytes(const flexsae_shape *shape);

/*
 * HierarchicalTopK forward.
 * replaces: _hierarchical_sae_forward + hierarchical_sae_forward_kernel and the
 *           host-side loss_per_batch.sum()/(B*K*D)  (hierarchical_kernels.py:12-89, 190-227)
 * out: loss[1] fp32 (mean over B*K*D of (r_{b,k,d}-t_{b,d})^2, summed in a fixed order);
 *      resid[B,D] fp32 = r_{b,K-1} - target_b, the only state the backward needs
 *      (the reference saves final_recon and re-reads target instead).
 */
int flexsae_hier_fwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const void *bias, const void *target, float *loss,
                     float *resid, void *workspace, size_t workspace_bytes, int *status_flag,
                     void *stream);

/*
 * HierarchicalTopK forward for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): flexsae_hier_fwd without the workspace argument.
 * No counterpart in the reference (its launcher allocates with torch, hierarchical_kernels.py:200-201).
 * The per-(row, tile) loss partials go to a static device array of FLEXSAE_STATIC_SCRATCH_BYTES
 * that every GPU the library runs on holds until the process ends; the call allocates nothing
 * (no hipMalloc/hipFree, no allocating library routine).  Limit: B * ceil(D/64) * 4 bytes must fit
 * the array (FLEXSAE_ERR_SCRATCH_LIMIT beyond; e.g. B=16384, D=8192 needs 8 MiB).  The first call
 * on a device looks the array's address up (make it before a graph capture starts).  All calls on
 * one GPU share the array: calls that overlap in time on one GPU (different streams) race; calls
 * on one stream are safe.  Outputs are bit-identical to flexsae_hier_fwd's.
 */
#define FLEXSAE_STATIC_SCRATCH_BYTES (16u << 20)
int flexsae_hier_fwd_static(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                            const void *vals, const void *bias, const void *target, float *loss,
                            float *resid, int *status_flag, void *stream);

/*
 * TopK forward, fully fused (gather, scale, sum over K, + bias, - target, mean square).
 * replaces: embedding_bag_forward + embedding_bag_forward_kernel and the eager tail
 *           of triton_topk_sae_loss  (topk_kernels.py:15-68, 213-223)
 * out: loss[1] fp32 (mean over B*D); resid[B,D] fp32 = r_b - target_b.
 */
int flexsae_topk_fwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const void *bias, const void *target, float *loss,
                     float *resid, void *workspace, size_t workspace_bytes, int *status_flag,
                     void *stream);

/*
 * Bytes of workspace flexsae_hier_bwd needs to process `slice_cols` columns of D per pass
 * (rounded up to whole 64*vec-column tiles, capped at D; slice_cols <= 0 asks for the minimum).
 * The workspace holds the latent-major pair list, the per-tile shares of dvals (about
 * D/128 x B*K fp32), and per slice column one contribution per (b,k) pair (bf16 for bf16 weights,
 * else fp32): about B*K*slice_cols*sizeof elements.
 */
size_t flexsae_hier_bwd_workspace_bytes(const flexsae_shape *shape, int64_t slice_cols);

/*
 * HierarchicalTopK backward, two phases per slice of D columns:
 *   sweep   : reverse walk over K per row; stores the per-pair contribution vals_k * S_k of the
 *             slice into the workspace, and the tile's shares of dvals and dbias;
 *   reduce  : latent-major segment reduction of those contributions (sorted pair list, fp32
 *             accumulation, fixed order) writing dW once in `dW_dtype` -- no atomics on dW, the
 *             result is deterministic, hot latents are split into 64-pair chunks.
 * The number of passes is ceil(D / slice width); the slice width is the widest one the given
 * workspace can hold (see flexsae_hier_bwd_workspace_bytes), so memory is the caller's choice.
 * replaces: _hierarchical_sae_backward + hierarchical_sae_backward_kernel, the three
 *           mul_(grad) passes of HierarchicalSAELossFunction.backward and the autograd engine's
 *           cast of the fp32 gradient  (hierarchical_kernels.py:92-187, 230-270, 294-299)
 * in : resid from flexsae_hier_fwd; grad_out device scalar.
 * out: dW[F,D] in dW_dtype, dvals[B,K] fp32, dbias[D] fp32: every element written once, all
 *      sums in a fixed order (bit-reproducible); FLEXSAE_BWD_OUTPUTS_PREZEROED is accepted and
 *      has nothing left to skip.
 */
int flexsae_hier_bwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                     const void *vals, const float *resid, const float *grad_out, void *dW,
                     int dW_dtype, float *dvals, float *dbias, void *workspace,
                     size_t workspace_bytes, int flags, int *status_flag, void *stream);

/*
 * HierarchicalTopK training step: forward AND backward in one pass over the gathered rows.
 * The sweep kernel of flexsae_hier_bwd is replaced by a kernel that gathers each row piece
 * once, keeps the K pieces of a (row, 128-column tile) in registers, walks them forward (loss)
 * and then backward (contributions, dvals), so the weight rows are gathered once per step
 * instead of twice.  The gradients returned are those of a UNIT upstream gradient; multiply by
 * the real one afterwards (flexsae_scale for dW; dvals/dbias are small).  Same workspace, same
 * slicing and the same segment reduction as flexsae_hier_bwd (use
 * flexsae_hier_bwd_workspace_bytes).
 * Supported when D % 4 == 0 and K <= 256 (the row pieces of a tile are kept on chip: in registers
 * and, for K = 64, 128 or 256, a quarter of them in the LDS):
 * flexsae_hier_fwd_bwd_supported() tells; otherwise FLEXSAE_ERR_UNSUPPORTED (use
 * flexsae_hier_fwd + flexsae_hier_bwd).
 * replaces: the forward and backward kernels and launchers together
 *           (hierarchical_kernels.py:12-187, 190-270), for the loss.backward() pattern of
 *           the reference's training loop (reference example.py:76-77).
 * out: loss[1]; dW[F,D] in dW_dtype; dvals[B,K] fp32; dbias[D] fp32 -- for grad_out = 1.
 * Deferred reduction: with FLEXSAE_BWD_SWEEP_ONLY in `flags` (and a workspace wide enough for a
 * single slice, else FLEXSAE_ERR_WORKSPACE) the segment reduction is left out and dW is not
 * touched (may be NULL); a later flexsae_hier_bwd on the same workspace with
 * FLEXSAE_BWD_REUSE_PAIR_LIST | FLEXSAE_BWD_REDUCE_ONLY | FLEXSAE_BWD_SCALE_BY_GRAD_OUT finishes dW
 * with the upstream gradient folded in, so no separate scaling pass over dW is needed.  The
 * price is that the workspace (B*K*D contributions) must stay alive in between.
 * With FLEXSAE_BWD_NO_DW (a decoder whose weight needs no gradient) the reductions are left out
 * for any workspace width: loss, dvals and dbias as usual, dW untouched (may be NULL).
 * Slicing: the workspace decides the slice width.  flexsae_hier_fwd_bwd_workspace_bytes gives the
 * bytes for slices of `slice_cols` columns, rounded up to whole training tiles (128 columns for
 * 16-bit weights, 64 or 128 for fp32) when D is a multiple of the reduction's 16-byte lane width
 * (8 columns of bf16 contributions, 4 of fp32) -- the reduction then works on 256-byte pieces --
 * and to whole 256-column tiles otherwise; slice_cols <= 0 asks for the minimum; 0 is returned for
 * unsupported shapes.  A slice is reduced right after it has been written, while part of it may
 * still be in the memory-side cache (256-column slices measured fastest at B*K = 2^19).  A workspace from
 * flexsae_hier_bwd_workspace_bytes is accepted as well.  The query assumes a dW aligned for that
 * 16-byte lane width (4 elements of fp32 or fp16 contributions' gradient, 8 of bf16); a dW aligned
 * less than that switches the piece reduction off, slices are then whole 256-column tiles, and a
 * workspace of the minimum width from this query is answered with FLEXSAE_ERR_WORKSPACE: ask
 * flexsae_hier_bwd_workspace_bytes instead.
 */
int flexsae_hier_fwd_bwd_supported(const flexsae_shape *shape);
size_t flexsae_hier_fwd_bwd_workspace_bytes(const flexsae_shape *shape, int64_t slice_cols);
/*
 * Hot-latent accumulators (FLEXSAE_BWD_HOT_LATENTS): where indices are skewed, a few latents are
 * selected by most batch rows, and the reference's backward piles its atomic adds up on their rows
 * of dW (hierarchical_kernels.py:155-161).  With the flag, the (up to 288) latents with the most
 * pairs -- more than 64 and no batch row holding the latent twice -- are summed in LDS accumulators
 * by blocks of 128 batch rows instead of being staged pair by pair, in 32-bit fixed point with one
 * exponent per block (integer sums do not depend on the order of the additions: results stay
 * bit-reproducible, and identical for every slice width).  Supported for 16-bit weights with
 * K <= 64 and D a multiple of 8 (bf16) or 4 (fp16); `_supported` says whether the flag would be
 * honoured for `shape`, `_workspace_bytes_flags` is the workspace query for a call with `flags`
 * (the accumulators' block partials take (slice columns / 128) x ceil(B / 128) x 147456 bytes, twice).
 * Slices are best chosen so that (slice columns / 128) x ceil(B / 128) is a multiple of the number
 * of compute units (one block each).
 */
int flexsae_hier_hot_latents_supported(const flexsae_shape *shape);
size_t flexsae_hier_fwd_bwd_workspace_bytes_flags(const flexsae_shape *shape, int64_t slice_cols, int flags);
/*
 * What the last call with FLEXSAE_BWD_HOT_LATENTS on `workspace` did (a diagnostic with no counterpart
 * in the reference): stats[0..5) (device memory) = hot latents, candidates (latents above the pair-count
 * threshold), long latents left to the chunked reduction, the threshold, and the number of
 * (row, tile) walks that were deferred to the second pass, summed over the slices.
 */
int flexsae_hier_hot_stats(const flexsae_shape *shape, const void *workspace, uint32_t *stats, void *stream);
/*
 * How skewed the indices of the last call on `workspace` were (any hierarchical backward / training
 * step workspace whose pair list is complete; no counterpart in the reference): stats[0] = latents
 * with more than 64 pairs, stats[1] = their 64-pair chunks, i.e. between 64 stats[1] - 63 stats[0] and
 * 64 stats[1] of the B*K pairs belong to such latents, stats[2] = latents without any pair.  `stats`
 * (three words) may be device memory or pinned host memory (the kernel then writes across the bus and
 * the caller polls an event: no synchronisation); a caller can use it to decide whether the next step
 * is worth FLEXSAE_BWD_HOT_LATENTS (many pairs on frequent latents) and FLEXSAE_BWD_DENSE_LATENTS (few
 * latents without pairs).
 */
int flexsae_hier_pair_stats(const flexsae_shape *shape, const void *workspace, uint32_t *stats, void *stream);
int flexsae_hier_fwd_bwd(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                         const void *vals, const void *bias, const void *target, float *loss,
                         void *dW, int dW_dtype, float *dvals, float *dbias, void *workspace,
                         size_t workspace_bytes, int flags, int *status_flag, void *stream);

/*
 * HierarchicalTopK training step with the plain-SGD weight update fused in: the same pass as
 * flexsae_hier_fwd_bwd, but the segment reduction, instead of writing a dense dW[F,D], subtracts
 * step[0] * (unit-gradient row) from every weight row that the batch touches, in place, in the
 * weight's own dtype (fp32 arithmetic, one rounding).  Rows of latents without pairs are neither
 * read nor written, so the dense zero-fill, the dense dW and the optimizer's passes over dW and W
 * are all gone.  `step` is a device fp32 scalar: learning rate times the upstream gradient of the
 * loss.  loss, dvals and dbias are returned as by flexsae_hier_fwd_bwd (unit upstream gradient;
 * dvals is what the encoder's backward needs, dbias the bias's update) and are computed from the
 * weights as they were on entry: within a slice of columns every read of the weights precedes the
 * reduction that updates that slice, and other slices touch other columns.
 * Supported where flexsae_hier_fwd_bwd is and the reduction can work 16 bytes per lane on the
 * staged contributions: D a multiple of 8 for bf16 weights (bf16 contributions, weight rows 16-byte
 * aligned), of 4 for fp32 and fp16 weights (fp32 contributions; weight rows aligned to 4 elements:
 * 16 bytes for fp32, 8 for fp16); otherwise FLEXSAE_ERR_UNSUPPORTED.  Workspace as for
 * flexsae_hier_fwd_bwd (for FLEXSAE_BWD_HOT_LATENTS from the _flags query); the flags accepted are
 * FLEXSAE_BWD_REUSE_PAIR_LIST, FLEXSAE_BWD_HOT_LATENTS (the accumulators' sums update the weight rows
 * of the hot latents the same way), FLEXSAE_BWD_REUSE_HOT_TABLES and FLEXSAE_BWD_DENSE_LATENTS; others
 * are ignored.
 * replaces: the dense dW of the backward (hierarchical_kernels.py:241-243, 294-297) together with
 *           the optimizer pass that consumes it in a training loop written like reference
 *           example.py:76-77 with torch.optim.SGD (no momentum, no weight decay: for those the
 *           untouched rows change too, and the dense gradient is the right interface).
 */
int flexsae_hier_sgd_step(const flexsae_shape *shape, const int64_t *indices, void *weight,
                          const void *vals, const void *bias, const void *target, const float *step,
                          float *loss, float *dvals, float *dbias, void *workspace, size_t workspace_bytes,
                          int flags, int *status_flag, void *stream);

/*
 * dst[n] = src[n] * scale[0]  (same dtype in and out; `scale` is a device fp32 scalar).  dst may
 * be src (in place); then a scale of exactly 1 costs one empty launch.
 * replaces: the dW.mul_(grad) pass of HierarchicalSAELossFunction.backward
 *           (hierarchical_kernels.py:294-297), needed only after flexsae_hier_fwd_bwd.
 */
int flexsae_scale(void *dst, const void *src, int dtype, int64_t n, const float *scale, void *stream);

/*
 * HierarchicalTopK backward, single-pass fallback that needs no workspace: the same reverse
 * sweep, scattering into an fp32 accumulator with atomics (as the reference kernel does).
 * Slower (every contribution is a read-modify-write of dW in memory) and not bit-reproducible.
 * replaces: same reference code as flexsae_hier_bwd.
 * out: dW_acc[F,D] fp32, dvals[B,K] fp32, dbias[D] fp32, all zero-filled here unless
 *      FLEXSAE_BWD_OUTPUTS_PREZEROED is set in `flags`.
 */
int flexsae_hier_bwd_atomic(const flexsae_shape *shape, const int64_t *indices, const void *weight,
                            const void *vals, const float *resid, const float *grad_out,
                            float *dW_acc, float *dvals, float *dbias, int flags, int *status_flag,
                            void *stream);

/* Bytes of workspace flexsae_csr_build needs. */
size_t flexsae_csr_workspace_bytes(int64_t B, int64_t K, int64_t F);

/*
 * Latent-major pair list for the TopK backward: begin[F+1] (exclusive prefix of
 * the per-latent pair counts, begin[F] = B*K) and map[B*K] holding pair ids
 * p = b*K + t grouped by latent, ascending inside a group (a stable counting
 * sort, so the result is deterministic).  Built as a bucketed counting sort whose atomics stay
 * in the LDS; with more than 8192*4096 latents, with one memory atomic per pair.
 * replaces: count_per_embedding_kernel, count.cumsum(0), map_embeddings_and_outputs_kernel
 *           (topk_kernels.py:71-94, 149-163; there the order inside a group is racy)
 */
int flexsae_csr_build(const int64_t *indices, int64_t B, int64_t K, int64_t F, uint32_t *begin,
                      uint32_t *map, void *workspace, size_t workspace_bytes, int *status_flag,
                      void *stream);

/*
 * Sharing one pair list between the two losses when both are evaluated on the same `indices`
 * (the reference rebuilds its map in every embedding_bag_backward call, topk_kernels.py:149-163).
 * flexsae_hier_pair_list_layout: byte offsets, inside a workspace of flexsae_hier_bwd /
 *   flexsae_hier_fwd_bwd, of the begin[F+1] and map[B*K] arrays those calls build; after such a
 *   call, workspace + offset can be handed to flexsae_topk_bwd as they are.
 * flexsae_hier_import_pair_list: the other direction; copies begin/map (from flexsae_csr_build
 *   or from another workspace) into `workspace` and derives the rest (slots, hot-latent tables),
 *   after which flexsae_hier_bwd / flexsae_hier_fwd_bwd can run with FLEXSAE_BWD_REUSE_PAIR_LIST.
 */
int flexsae_hier_pair_list_layout(const flexsae_shape *shape, size_t *begin_offset, size_t *map_offset);
int flexsae_hier_import_pair_list(const flexsae_shape *shape, const uint32_t *begin, const uint32_t *map,
                                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * TopK backward: latent-major segment reduction (no atomics on dW).
 * replaces: aggregate_gradient_for_embedding_kernel and its launch, plus the autograd of
 *           the eager loss tail that produces `gradient` and the bias gradient
 *           (topk_kernels.py:97-137, 165-184, 220-223)
 * in : begin/map from flexsae_csr_build; resid from flexsae_topk_fwd; grad_out device scalar;
 *      indices[B,K] (may be NULL): when given, a pair whose index lies outside [0, F) counts with a
 *      value of zero, as it did in the forward (the pair list files it under latent 0), so dW, dvals
 *      and dbias are the gradients of the loss the forward returned; NULL skips that test.
 * out: dW[F,D] written once in `dW_dtype` (every row, zeros for unused latents);
 *      dvals[B,K] fp32, every element written once (per-tile shares added in tile order);
 *      dbias[D] fp32 (column sums in a fixed order).  All three are bit-reproducible;
 *      nothing needs a zero-fill (FLEXSAE_BWD_OUTPUTS_PREZEROED is accepted and ignored).
 * With bf16 weights the residual rows are gathered from a bf16 copy made in the workspace: the
 * reference's backward likewise receives the residual gradient in the weight dtype
 * (topk_kernels.py:52 makes the bag output weight-typed, so autograd casts its gradient).  That
 * rounding shows in dvals (about 4e-3 normwise instead of 1e-6); FLEXSAE_TOPK_BWD_FP32_RESIDUAL in
 * `flags` gathers the fp32 residual instead (twice the cache footprint, slower).
 * Limit: B*D*4 bytes < 4 GiB (FLEXSAE_ERR_UNSUPPORTED beyond), the gathers use 32-bit offsets.
 */
int flexsae_topk_bwd(const flexsae_shape *shape, const uint32_t *begin, const uint32_t *map,
                     const int64_t *indices, const void *weight, const void *vals, const float *resid,
                     const float *grad_out, void *dW, int dW_dtype, float *dvals, float *dbias,
                     void *workspace, size_t workspace_bytes, int flags, void *stream);

/*
 * Bytes of workspace flexsae_topk_bwd needs to process `slice_cols` columns of D per pass
 * (rounded to whole tiles, capped at D; <= 0 asks for the minimum).  The slice width only
 * sizes the fp32 partial sums of latents with more than 64 pairs (hot latents are cut into
 * 64-pair chunks that are reduced by separate wavefronts and then combined in a fixed order);
 * the fixed part holds the per-pair records, the per-tile dvals shares (one fp32 per pair and
 * tile) and, for bf16 weights, the bf16 residual copy.  The result covers both layouts of the
 * call, with and without FLEXSAE_TOPK_BWD_FP32_RESIDUAL (the larger of the two).
 */
size_t flexsae_topk_bwd_workspace_bytes(const flexsae_shape *shape, int64_t slice_cols);

/*
 * dst[n] (dtype) = src[n] (fp32), round-to-nearest-even.  Used to hand the fp32
 * scatter accumulator of the hierarchical backward over in the weight's dtype.
 * replaces: the autograd engine's implicit cast of the fp32 gradients returned at
 *           hierarchical_kernels.py:299.
 */
int flexsae_cast_from_f32(void *dst, int dst_dtype, const float *src, int64_t n, void *stream);

/*
 * dst[n] (dtype) = src[n] (fp32) * scale[0], one rounding (`scale` a device fp32 scalar; NULL = 1).
 * For gradients of fp16 weights: the unit-gradient dW of flexsae_hier_fwd_bwd is of magnitude
 * 2/(B*K*D), below fp16's range, so it is kept in fp32 and meets the upstream gradient (a loss
 * scale, typically) before the only rounding.
 * replaces: dW.mul_(grad) in fp32 followed by the engine's cast to the leaf dtype
 *           (hierarchical_kernels.py:294-299).
 */
int flexsae_scale_from_f32(void *dst, int dst_dtype, const float *src, int64_t n, const float *scale,
                           void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLEXSAE_AMD_H */
