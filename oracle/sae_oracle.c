/*
 * CPU oracle for the SAE decoder-loss path (TopK and HierarchicalTopK).
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may call this file;
 * it exists so that tests, the smoke check and the benchmark's CPU-baseline leg
 * can compare the HIP kernels with an independent statement of the algorithm.
 *
 * What it restates (reference file:line, relative to the reference checkout):
 *   - hierarchical loss definition      torch-ext/flex_sae/hierarchical_kernels.py:312-323
 *   - top-k loss definition             torch-ext/flex_sae/topk_kernels.py:226-237
 *   - gradient scale 2/(B*K*D)          torch-ext/flex_sae/hierarchical_kernels.py:135
 *   - loss scale 1/(B*K*D)              torch-ext/flex_sae/hierarchical_kernels.py:226
 *   - top-k divisor B*D                 torch-ext/flex_sae/topk_kernels.py:220-223
 *   - which inputs receive gradients    torch-ext/flex_sae/hierarchical_kernels.py:294-299,
 *                                       torch-ext/flex_sae/topk_kernels.py:210
 *   - latent-major pair list (CSR)      torch-ext/flex_sae/topk_kernels.py:140-163
 *
 * Inputs arrive as float32 (the caller upcasts bf16/fp16 exactly, as the
 * reference kernels do on load: hierarchical_kernels.py:49-64, topk_kernels.py:38);
 * every accumulation here is in double, so the oracle is the "true" value of the
 * closed form for those float inputs, not a bit-level model of any kernel.
 *
 * The gradients are obtained from the definition, not from the kernels' reverse
 * sweep trick: the forward prefix sums r_k are formed explicitly, g_k = c*(r_k-t),
 * S_j = sum_{k>=j} g_k, dvals_j = <w_j,S_j>, dW[idx_j] += v_j*S_j, dbias = S_0.
 *
 * Pinning (see tests/test_oracle.py): exact rational known-answer vectors in
 * tests/golden/, brute-force numpy loops, central finite differences, torch
 * autograd in float64 on an independent restatement, and algebraic invariants
 * (K=1 equivalence, mean-of-prefix-TopK identity, vals=0 closed form,
 * permutation invariance, duplicate merging, scatter mass conservation).
 *
 * Parallelism: OpenMP over slices of D.  A slice owns its columns of dW and
 * dbias, so there are no write conflicts and results do not depend on the
 * thread count except for the final (fixed-order) sums over slices.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define SLICE 16 /* columns handled together; keeps the per-row scratch small */

int sae_oracle_version(void) { return 1; }

int sae_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/*
 * mode 0: TopK          L = 1/(B*D)   * sum_{b,d}   (r_{b,K-1,d} - t_{b,d})^2
 * mode 1: Hierarchical  L = 1/(B*K*D) * sum_{b,k,d} (r_{b,k,d}   - t_{b,d})^2
 * with r_{b,k} = bias + sum_{j<=k} vals[b,j] * W[idx[b,j]].
 *
 * Outputs (any may be NULL): loss[1]; dW[F*D], dvals[B*K], dbias[D] already
 * multiplied by grad_out.  dW32 is an alternative float destination for dW when
 * an F*D array of doubles would be too large (accumulation is still in double,
 * slice by slice).  Returns 0, or -1 on a bad argument / out-of-range index,
 * -2 when scratch memory cannot be allocated.
 */
int sae_oracle_loss_grads(int mode, const int64_t *idx, const float *W, const float *vals,
                          const float *bias, const float *target, int64_t B, int64_t K, int64_t F,
                          int64_t D, double grad_out, double *loss, double *dW, float *dW32,
                          double *dvals, double *dbias) {
  if (B <= 0 || K <= 0 || F <= 0 || D <= 0 || (mode != 0 && mode != 1)) return -1;
  for (int64_t p = 0; p < B * K; ++p)
    if (idx[p] < 0 || idx[p] >= F) return -1;

  const int64_t nslice = (D + SLICE - 1) / SLICE;
  const int want_dw = (dW != NULL) || (dW32 != NULL);
  const double c = (mode == 1 ? 2.0 / ((double)B * (double)K * (double)D)
                              : 2.0 / ((double)B * (double)D)) * grad_out;
  double *loss_part = (double *)calloc((size_t)nslice, sizeof(double));
  double *dv_part = NULL; /* [nslice][B*K] would be large; accumulate per thread instead */
  int nthreads = sae_oracle_max_threads();
  if (dvals) dv_part = (double *)calloc((size_t)nthreads * (size_t)(B * K), sizeof(double));
  if (!loss_part || (dvals && !dv_part)) {
    free(loss_part);
    free(dv_part);
    return -2;
  }
  int failed = 0;

#pragma omp parallel
  {
#ifdef _OPENMP
    const int tid = omp_get_thread_num();
#else
    const int tid = 0;
#endif
    double *g = (double *)malloc((size_t)K * SLICE * sizeof(double));
    double *acc = want_dw ? (double *)malloc((size_t)F * SLICE * sizeof(double)) : NULL;
    if (!g || (want_dw && !acc)) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp barrier
    if (!failed) {
      double *dv = dv_part ? dv_part + (size_t)tid * (size_t)(B * K) : NULL;
#pragma omp for schedule(dynamic, 1)
      for (int64_t s = 0; s < nslice; ++s) {
        const int64_t d0 = s * SLICE;
        const int w = (int)((D - d0) < SLICE ? (D - d0) : SLICE);
        if (acc) memset(acc, 0, (size_t)F * SLICE * sizeof(double));
        double lsum = 0.0;
        double db[SLICE];
        for (int i = 0; i < w; ++i) db[i] = 0.0;
        for (int64_t b = 0; b < B; ++b) {
          const int64_t *ib = idx + b * K;
          const float *vb = vals + b * K;
          const float *tb = target + b * D + d0;
          double r[SLICE];
          for (int i = 0; i < w; ++i) r[i] = (double)bias[d0 + i];
          /* forward: explicit prefix reconstructions and per-step residual gradients */
          for (int64_t k = 0; k < K; ++k) {
            const float *wr = W + ib[k] * D + d0;
            const double v = (double)vb[k];
            double *gk = g + k * SLICE;
            for (int i = 0; i < w; ++i) {
              r[i] += v * (double)wr[i];
              const double diff = r[i] - (double)tb[i];
              if (mode == 1) {
                lsum += diff * diff;
                gk[i] = c * diff;
              } else if (k == K - 1) {
                lsum += diff * diff;
                gk[i] = c * diff;
              } else {
                gk[i] = 0.0;
              }
            }
          }
          /* backward: suffix sums of g */
          double S[SLICE];
          for (int i = 0; i < w; ++i) S[i] = 0.0;
          for (int64_t j = K - 1; j >= 0; --j) {
            const float *wr = W + ib[j] * D + d0;
            const double v = (double)vb[j];
            const double *gj = g + j * SLICE;
            double dot = 0.0;
            for (int i = 0; i < w; ++i) {
              S[i] += gj[i];
              dot += (double)wr[i] * S[i];
            }
            if (dv) dv[b * K + j] += dot;
            if (acc) {
              double *a = acc + ib[j] * SLICE;
              for (int i = 0; i < w; ++i) a[i] += v * S[i];
            }
          }
          for (int i = 0; i < w; ++i) db[i] += S[i];
        }
        loss_part[s] = lsum;
        if (dbias)
          for (int i = 0; i < w; ++i) dbias[d0 + i] = db[i];
        if (dW)
          for (int64_t f = 0; f < F; ++f)
            for (int i = 0; i < w; ++i) dW[f * D + d0 + i] = acc[f * SLICE + i];
        if (dW32)
          for (int64_t f = 0; f < F; ++f)
            for (int i = 0; i < w; ++i) dW32[f * D + d0 + i] = (float)acc[f * SLICE + i];
      }
    }
    free(g);
    free(acc);
  }

  if (!failed) {
    if (loss) {
      double tot = 0.0;
      for (int64_t s = 0; s < nslice; ++s) tot += loss_part[s];
      const double div = (mode == 1) ? (double)B * (double)K * (double)D : (double)B * (double)D;
      loss[0] = tot / div;
    }
    if (dvals) {
      for (int64_t p = 0; p < B * K; ++p) {
        double t = 0.0;
        for (int th = 0; th < nthreads; ++th) t += dv_part[(size_t)th * (size_t)(B * K) + p];
        dvals[p] = t;
      }
    }
  }
  free(loss_part);
  free(dv_part);
  return failed ? -2 : 0;
}

/*
 * Latent-major pair list: begin[F+1] (exclusive prefix of the per-latent pair
 * counts) and map[B*K], the pair ids p = b*K + t grouped by latent, ascending p
 * inside a group (i.e. a stable counting sort of the pairs by latent).  The
 * reference builds the same structure (topk_kernels.py:149-163) but leaves the
 * order inside a group to the race between its atomics.
 */
int sae_oracle_csr(const int64_t *idx, int64_t B, int64_t K, int64_t F, uint32_t *begin,
                   uint32_t *map) {
  if (B <= 0 || K <= 0 || F <= 0 || B * K > 0xffffffffLL) return -1;
  const int64_t n = B * K;
  memset(begin, 0, (size_t)(F + 1) * sizeof(uint32_t));
  for (int64_t p = 0; p < n; ++p) {
    if (idx[p] < 0 || idx[p] >= F) return -1;
    begin[idx[p] + 1]++;
  }
  for (int64_t f = 0; f < F; ++f) begin[f + 1] += begin[f];
  uint32_t *cur = (uint32_t *)malloc((size_t)F * sizeof(uint32_t));
  if (!cur) return -2;
  memcpy(cur, begin, (size_t)F * sizeof(uint32_t));
  for (int64_t p = 0; p < n; ++p) map[cur[idx[p]]++] = (uint32_t)p;
  free(cur);
  return 0;
}
