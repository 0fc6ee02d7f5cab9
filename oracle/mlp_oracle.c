/*
 * CPU oracle for the data-parallel MLP training step.  TEST INFRASTRUCTURE ONLY:
 * nothing that ships (the HIP library, the host driver) links or calls this file.
 *
 * It restates, in the plainest possible C, the arithmetic of the reference's hot path:
 *   forward GEMM   Y  = X * W^T            reference call site mlp_omp.cc:474-488
 *   weight grad    dW = dZ[r]^T * A[r]     reference call site mlp_omp.cc:529-531,565-580
 *   input grad     dA = dZ * W             reference call site mlp_omp.cc:655-671
 *   reduce + SGD   W  = fma(-lr, sum_r G_r, W)   mlp_omp.cc:136-145 (adds), 240-250 (last add + fmadd)
 * plus the semantics the benchmark configs add on top (bias, ReLU, ReLU mask, db = column sum),
 * whose meaning is fixed by c2_bench/mlp_caffe2.py:208-217 (FC + Relu) and :251-267 (W += -lr*dW).
 *
 * GEMMs accumulate in double and round once to float, so the oracle is strictly more
 * accurate than any fp32 implementation it checks.  The reduce follows the reference's
 * arithmetic exactly (fp32 left fold over replicas, one fused multiply-add with -lr rounded
 * to float), so a correct device kernel that folds in replica order matches it bit for bit.
 *
 * Pinning (what fixes these functions besides their own formulas) lives in tests/test_oracle.py:
 * numpy float64 matmul (library routine), identity / one-hot special cases, a finite-difference
 * gradient check of the whole step, and the reference's closed-form all-reduce test
 * (mlp_omp.cc:325-373).
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define IDX(i, ld, j) ((size_t)(i) * (size_t)(ld) + (size_t)(j))

/* Y[M x N] = X[M x K] * W[N x K]^T (+ b[N]) ; optional ReLU.  (mlp_omp.cc:474-488) */
void oracle_fc_forward(int M, int N, int K, const float* X, int ldx, const float* W, int ldw,
                       const float* b, int relu, float* Y, int ldy) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; ++i) {
    const float* x = X + IDX(i, ldx, 0);
    for (int j = 0; j < N; ++j) {
      const float* w = W + IDX(j, ldw, 0);
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)x[k] * (double)w[k];
      if (b) acc += (double)b[j];
      float y = (float)acc;
      if (relu && !(y > 0.0f)) y = 0.0f;
      Y[IDX(i, ldy, j)] = y;
    }
  }
}

/* dW[M x N] = dZ[K x M]^T * A[K x N] over the K batch rows of ONE replica; db[M] = column sums
 * of dZ (db may be NULL).  The reference splits the batch over sockets the same way
 * (k_begin/k_end, mlp_omp.cc:529-531) and writes one dW per socket (mlp_omp.cc:579). */
void oracle_fc_wgrad(int M, int N, int K, const float* dZ, int lddz, const float* A, int lda,
                     float* dW, int lddw, float* db) {
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
#pragma omp for schedule(static)
    for (int i = 0; i < M; ++i) {
      for (int j = 0; j < N; ++j) acc[j] = 0.0;
      double colsum = 0.0;
      for (int k = 0; k < K; ++k) {
        double g = (double)dZ[IDX(k, lddz, i)];
        const float* a = A + IDX(k, lda, 0);
        colsum += g;
        for (int j = 0; j < N; ++j) acc[j] += g * (double)a[j];
      }
      for (int j = 0; j < N; ++j) dW[IDX(i, lddw, j)] = (float)acc[j];
      if (db) db[i] = (float)colsum;
    }
    free(acc);
  }
}

/* dA[M x N] = dZ[M x K] * W[K x N]; when mask_src != NULL the result is multiplied by
 * [mask_src > 0] (the ReLU derivative taken at the forward activation).  (mlp_omp.cc:655-671) */
void oracle_fc_dgrad(int M, int N, int K, const float* dZ, int lddz, const float* W, int ldw,
                     const float* mask_src, int ldm, float* dA, int ldda) {
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
#pragma omp for schedule(static)
    for (int i = 0; i < M; ++i) {
      for (int j = 0; j < N; ++j) acc[j] = 0.0;
      for (int k = 0; k < K; ++k) {
        double g = (double)dZ[IDX(i, lddz, k)];
        const float* w = W + IDX(k, ldw, 0);
        for (int j = 0; j < N; ++j) acc[j] += g * (double)w[j];
      }
      for (int j = 0; j < N; ++j) {
        float v = (float)acc[j];
        if (mask_src && !(mask_src[IDX(i, ldm, j)] > 0.0f)) v = 0.0f;
        dA[IDX(i, ldda, j)] = v;
      }
    }
    free(acc);
  }
}

/* Loss front-end of the Caffe2 harness (mlp_caffe2.py:221-239): per replica
 *   dist_i = 0.5 * sum_j (label[i][j] - pred[i][j])^2      (SquaredL2Distance, one value per row)
 *   loss_r = (1/B) * sum_{i in replica r} dist_i           (AveragedLoss over the replica's B rows)
 * and the total loss is the sum of the R replica losses (net.Sum, :236-238).  The gradient that
 * enters the backward pass is d(total)/d(pred) = (pred - label) / B.  Rows [r*B, (r+1)*B) belong
 * to replica r.  Accumulation in double; dY rounded to float once. */
void oracle_l2_loss(int R, int B, int N, const float* pred, int ldp, const float* label, int ldl, float* dY, int lddy,
                    double* loss_per_replica) {
  const double inv_b = 1.0 / (double)B;
  for (int r = 0; r < R; ++r) {
    double acc = 0.0;
    for (int i = r * B; i < (r + 1) * B; ++i) {
      double dist = 0.0;
      for (int j = 0; j < N; ++j) {
        const double d = (double)pred[IDX(i, ldp, j)] - (double)label[IDX(i, ldl, j)];
        dist += 0.5 * d * d;
        if (dY) dY[IDX(i, lddy, j)] = (float)(d * inv_b);
      }
      acc += dist;
    }
    loss_per_replica[r] = acc * inv_b;
  }
}

/* W[i] = fma(-lr, G_0[i] + G_1[i] + ... + G_{R-1}[i], W[i]) with fp32 adds in replica order and a
 * single-rounding fma, G_r = G + r*stride.  Arithmetic of mlp_omp.cc:140-143 (zmm add) and
 * :242-249 (add, then _mm512_fmadd_ps with -alpha rounded to float); R == 1 is :218-221. */
void oracle_reduce_sgd(float* W, const float* G, size_t n, size_t stride, int R, float lr) {
  const float neg_lr = -lr;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float s = G[i];
    for (int r = 1; r < R; ++r) s = s + G[(size_t)r * stride + i];
    W[i] = fmaf(neg_lr, s, W[i]);
  }
}

/*
 * One full training step on flat, densely packed arrays (ld == ncols everywhere).
 *   nf[0..L]        layer widths
 *   X   [R*B x nf[0]],  dY [R*B x nf[L]]
 *   W   concatenation over l of ( W_l[nf[l+1] x nf[l]] , b_l[nf[l+1]] )   -- updated in place
 *   acts   concatenation over l=0..L of A_l [R*B x nf[l]]   (A_0 = X is copied in)
 *   dWall  R copies, each laid out like W: per-replica gradients (before the reduce)
 *   dX  [R*B x nf[0]]
 * relu_last != 0 applies ReLU after the last layer as well (mlp_caffe2.py:215-217 does);
 * the benchmark configs use ReLU between layers only.
 * given_acts != 0 skips the forward pass and takes `acts` as input: the backward pass is then
 * evaluated on exactly those activations.  Tests use it to compare a device backward pass on the
 * device's own activations, because the ReLU mask [A > 0] is discontinuous: an activation that
 * rounds to +1e-9 on one side and to 0 on the other legitimately flips a whole gradient entry.
 * Returns 0, or -1 on allocation failure.
 */
int oracle_mlp_step(int L, const int* nf, int B, int R, int relu_last, int given_acts, float lr,
                    const float* X, const float* dY, float* W, float* acts, float* dWall, float* dX) {
  const int MB = R * B;
  size_t P = 0, maxw = 0;
  for (int l = 0; l < L; ++l) P += (size_t)nf[l + 1] * nf[l] + nf[l + 1];
  for (int l = 0; l <= L; ++l)
    if ((size_t)nf[l] > maxw) maxw = nf[l];

  size_t* woff = (size_t*)malloc(sizeof(size_t) * (L + 1));
  size_t* aoff = (size_t*)malloc(sizeof(size_t) * (L + 2));
  float* dz_cur = (float*)malloc(sizeof(float) * MB * maxw);
  float* dz_nxt = (float*)malloc(sizeof(float) * MB * maxw);
  if (!woff || !aoff || !dz_cur || !dz_nxt) return -1;
  woff[0] = 0;
  for (int l = 0; l < L; ++l) woff[l + 1] = woff[l] + (size_t)nf[l + 1] * nf[l] + nf[l + 1];
  aoff[0] = 0;
  for (int l = 0; l <= L; ++l) aoff[l + 1] = aoff[l] + (size_t)MB * nf[l];

  if (!given_acts) memcpy(acts, X, sizeof(float) * MB * nf[0]);
  for (int l = 0; l < L && !given_acts; ++l) {
    const float* Wl = W + woff[l];
    const float* bl = Wl + (size_t)nf[l + 1] * nf[l];
    int relu = (l < L - 1) || relu_last;
    oracle_fc_forward(MB, nf[l + 1], nf[l], acts + aoff[l], nf[l], Wl, nf[l], bl, relu,
                      acts + aoff[l + 1], nf[l + 1]);
  }

  /* dZ of the last layer: the upstream gradient, masked if the last layer has a ReLU */
  for (size_t i = 0; i < (size_t)MB * nf[L]; ++i) {
    float g = dY[i];
    if (relu_last && !(acts[aoff[L] + i] > 0.0f)) g = 0.0f;
    dz_cur[i] = g;
  }

  for (int l = L - 1; l >= 0; --l) {
    const float* Wl = W + woff[l];
    for (int r = 0; r < R; ++r) {
      float* dWl = dWall + (size_t)r * P + woff[l];
      float* dbl = dWl + (size_t)nf[l + 1] * nf[l];
      oracle_fc_wgrad(nf[l + 1], nf[l], B, dz_cur + (size_t)r * B * nf[l + 1], nf[l + 1],
                      acts + aoff[l] + (size_t)r * B * nf[l], nf[l], dWl, nf[l], dbl);
    }
    float* out = (l == 0) ? dX : dz_nxt;
    oracle_fc_dgrad(MB, nf[l], nf[l + 1], dz_cur, nf[l + 1], Wl, nf[l],
                    (l > 0) ? acts + aoff[l] : NULL, nf[l], out, nf[l]);
    if (l > 0) {
      float* t = dz_cur;
      dz_cur = dz_nxt;
      dz_nxt = t;
    }
  }

  oracle_reduce_sgd(W, dWall, P, P, R, lr);

  free(woff);
  free(aoff);
  free(dz_cur);
  free(dz_nxt);
  return 0;
}
