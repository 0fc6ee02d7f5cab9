/*
 * CPU baseline: an OpenMP SPMD restatement of the reference's mlp_omp main loop, timed by the
 * cpu_baseline leg of bench.py.  TEST / MEASUREMENT INFRASTRUCTURE ONLY -- the product never
 * links it.  The reference itself cannot be built here (it needs Intel MKL and TBB headers), so
 * this file restates its structure:
 *
 *   threads          R "sockets" x T threads, thread id = socket * T + thread-in-socket
 *                    (Partition.cc:8-23)
 *   forward          per thread one sequential SGEMM on its block of the output, blocks from the
 *                    2-D partition with aspect ratio 4 (mlp_omp.cc:441-510)
 *   weight gradient  batch (k) split over sockets, 2-D partition of (n_out, n_in) inside a socket
 *                    with aspect ratio 1/2 and 16-aligned rows, one dW per socket
 *                    (mlp_omp.cc:513-600)
 *   input gradient   2-D partition with aspect ratio 1/2, result written in place over the
 *                    activation (mlp_omp.cc:619-691)
 *   update           ring reduce-scatter + all-gather with the SGD update fused into the first
 *                    all-gather step, flag handshakes between neighbouring sockets
 *                    (mlp_omp.cc:56-295).  Two schedules, as in the reference:
 *                    - all threads run the update of a layer after its input gradient
 *                      (OVERLAP_ALL_REDUCE undefined, mlp_omp.cc:724-734);
 *                    - overlapped (OVERLAP_ALL_REDUCE, mlp_omp.cc:519-524,601-615,692-723): the last
 *                      Tc threads of every socket are communication threads.  While the others
 *                      compute the weight gradient of layer l they run the all-gather (with the
 *                      SGD update) of layer l+1, while the others compute the input gradient of
 *                      layer l they run the reduce-scatter of layer l, and after layer 0 its
 *                      all-gather.  Tc comes from the reference's table by threads per socket
 *                      (mlp_bench_common.h:40-48: none below 5 threads, so the 4-thread sockets of
 *                      a 16-core host run the first schedule, like the reference would).
 * and adds what the benchmark configurations add to the reference: bias, ReLU between layers,
 * the ReLU mask in the backward pass, db = column sums, an explicit upstream gradient dY.
 *
 * SGEMM comes from a cblas_sgemm the caller passes in (OpenBLAS shipped with scipy, threads = 1,
 * called sequentially inside each thread exactly like the reference calls MKL), or from the
 * built-in kernel below when none is given.
 *
 * Pinned by tests/test_cpu_port.py: final weights and dX against the float64-accumulating oracle,
 * and the ring all-reduce against the reference's closed-form check (mlp_omp.cc:325-373).
 */
#include <math.h>
#include <omp.h>
#include <stdatomic.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define PADF 16 /* pad columns of every matrix, = one 64-byte line of floats (mlp_bench_common.h:9-10) */
#define LINE 16

typedef void (*cblas_sgemm_fn)(int order, int transa, int transb, int m, int n, int k, float alpha, const float* a,
                               int lda, const float* b, int ldb, float beta, float* c, int ldc);
enum { ROW_MAJOR = 101, NO_TRANS = 111, TRANS = 112 };

/* ---- work partition (Partition.cc:25-222), restated in C ------------------------------------ */

static int ceil_div(int a, int b) { return (a + b - 1) / b; }
static int imin(int a, int b) { return a < b ? a : b; }
static size_t zmin(size_t a, size_t b) { return a < b ? a : b; }

static void block_shape(int m, int n, int rows, int cols, int m_align, int* bm, int* bn) {
  *bm = m_align ? ceil_div(ceil_div(m, 16), rows) * 16 : ceil_div(m, rows);
  *bn = ceil_div(ceil_div(n, 16), cols) * 16;
}

void port_partition_2d_intra(int m, int n, double ar, int m_align, int T, int t, int out[4]) {
  int mb = 1, nb = T, bm, bn;
  block_shape(m, n, mb, nb, m_align, &bm, &bn);
  double best = fabs((double)bm / bn - ar);
  for (int rows = 2; rows <= T; ++rows) {
    if (T % rows) continue;
    int cols = T / rows, per = ceil_div(m, rows), cbm, cbn;
    if (m_align) {
      if (ar < 1 && bm == 16 && per < 16) continue;
      if (per <= 8) continue;
    }
    if (ceil_div(n, cols) <= 8) continue;
    block_shape(m, n, rows, cols, m_align, &cbm, &cbn);
    double d = fabs((double)cbm / cbn - ar);
    if (d < best) {
      best = d; mb = rows; nb = cols; bm = cbm; bn = cbn;
    } else {
      break;
    }
  }
  (void)mb;
  int mt = t / nb, nt = t % nb;
  out[0] = imin(mt * bm, m);
  out[1] = imin(out[0] + bm, m);
  out[2] = imin(nt * bn, n);
  out[3] = imin(out[2] + bn, n);
}

void port_partition_2d(int m, int n, double ar, int m_align, int ns, int sid, int T, int t, int out[4]) {
  int per = ceil_div(m, ns);
  port_partition_2d_intra(per, n, ar, m_align, T, t, out);
  int base = imin(sid * per, m);
  out[0] = imin(base + out[0], m);
  out[1] = imin(base + out[1], m);
}

/* ring neighbourhood (mlp_bench_common.cc:13-14,170-190) */
static const int RINGS[2][8] = {{0, 1, 2, 4, 7, 6, 5, 3}, {0, 3, 5, 6, 7, 4, 2, 1}};

void port_ring_info(int ns, int sid, int task, int out[3]) {
  int which = task % 2;
  if (ns < 8) {
    int up = (sid + 1) % ns, down = (sid + ns - 1) % ns;
    out[0] = sid;
    out[1] = which ? up : down;
    out[2] = which ? down : up;
    return;
  }
  int pos = 0;
  while (RINGS[which][pos] != sid) ++pos;
  out[0] = pos;
  out[1] = RINGS[which][(pos + ns - 1) % ns];
  out[2] = RINGS[which][(pos + 1) % ns];
}

/* ---- built-in SGEMM (used when no BLAS is supplied) ------------------------------------------ */
/* C[m x n] = op(A) * op(B), row major, alpha = 1, beta = 0.  Plain k-blocked loops that the
 * compiler vectorises along n; adequate as a fallback, far from a tuned BLAS. */
void port_builtin_sgemm(int order, int ta, int tb, int m, int n, int k, float alpha, const float* a, int lda,
                        const float* b, int ldb, float beta, float* c, int ldc) {
  (void)order; (void)alpha; (void)beta;
  enum { KB = 256 };
  float* bt = NULL;
  if (tb == TRANS) { /* B given as [n x k]: transpose once into [k x n] */
    bt = (float*)malloc(sizeof(float) * (size_t)k * n);
    for (int j = 0; j < n; ++j)
      for (int p = 0; p < k; ++p) bt[(size_t)p * n + j] = b[(size_t)j * ldb + p];
    b = bt;
    ldb = n;
  }
  for (int i = 0; i < m; ++i) memset(c + (size_t)i * ldc, 0, sizeof(float) * n);
  for (int k0 = 0; k0 < k; k0 += KB) {
    int k1 = imin(k0 + KB, k);
    for (int i = 0; i < m; ++i) {
      float* ci = c + (size_t)i * ldc;
      for (int p = k0; p < k1; ++p) {
        float av = (ta == TRANS) ? a[(size_t)p * lda + i] : a[(size_t)i * lda + p];
        const float* bp = b + (size_t)p * ldb;
#pragma omp simd
        for (int j = 0; j < n; ++j) ci[j] += av * bp[j];
      }
    }
  }
  free(bt);
}

/* ---- ring all-reduce with fused SGD (mlp_omp.cc:56-295) -------------------------------------- */

typedef struct {
  int ns, T;
  _Atomic int* done; /* [ns*T*16] flags, 16 phases per thread (mlp_omp.cc:50,117-123) */
} ring_ctx;

static void handshake(ring_ctx* rc, int tid, int prev_tid, int* phase) {
  atomic_store_explicit(&rc->done[tid * 16 + *phase], 1, memory_order_release);
  _Atomic int* wait = &rc->done[prev_tid * 16 + *phase];
  while (!atomic_load_explicit(wait, memory_order_acquire)) {
#if defined(__x86_64__)
    __builtin_ia32_pause();
#endif
  }
  atomic_store_explicit(wait, 0, memory_order_relaxed);
  *phase = (*phase + 1) % 16;
}

typedef struct { size_t begin, end; } span_t;

static span_t thread_span(size_t chunk, size_t per_chunk, size_t per_thread, int t, size_t total) {
  size_t cb = zmin(chunk * per_chunk, total), ce = zmin(cb + per_chunk, total);
  span_t s;
  s.begin = zmin(cb + (size_t)t * per_thread, ce);
  s.end = zmin(s.begin + per_thread, ce);
  return s;
}

/* Threads of a socket set aside for the all-reduce when it overlaps the GEMMs, by threads per
 * socket (mlp_bench_common.h:40-48). */
int port_comm_threads(int T) {
  if (T < 5) return 0;
  if (T < 10) return 1;
  if (T < 20) return 2;
  return 4;
}

typedef struct {
  int idx, prev, next;
  size_t per_chunk, per_thread;
} ring_plan;

static ring_plan plan_ring(const ring_ctx* rc, size_t weight_size, int sid, int t) {
  const int ns = rc->ns, T = rc->T;
  int ring[3];
  port_ring_info(ns, sid, t, ring);
  ring_plan p;
  p.idx = ring[0];
  p.prev = ring[1];
  p.next = ring[2];
  /* Deviation from the reference, on purpose.  With fewer than 8 sockets the reference keeps
   * idx_in_ring = sid also for the reversed ring of odd tasks (mlp_bench_common.cc:183-189), but
   * the chunk schedule below needs a position that grows along `next`; the reference's rule only
   * closes the ring for 2 sockets, and its own start-up check would fail for 3..7 sockets with
   * two or more threads per socket.  Count the position along the ring direction instead. */
  if (ns < 8 && (t % 2)) p.idx = (ns - sid) % ns;
  p.per_chunk = (weight_size + (size_t)ns * LINE - 1) / ns / LINE * LINE;
  p.per_thread = (p.per_chunk + (size_t)T * LINE - 1) / T / LINE * LINE;
  return p;
}

/* grads, push, weights: ns stacked replicas of `weight_size` floats each; rc->T threads of every
 * socket take part, t is this thread's index among them. */

/* reduce-scatter (mlp_omp.cc:56-169); the last addition is left to the all-gather's first step */
static void ring_reduce_scatter(ring_ctx* rc, float* grads, float* push, size_t weight_size, int sid, int t, int* phase) {
  const int ns = rc->ns, T = rc->T, tid = sid * T + t;
  const ring_plan p = plan_ring(rc, weight_size, sid, t);
  float* g = grads + (size_t)sid * weight_size;
  float* pb = push + (size_t)sid * weight_size;
  float* pb_next = push + (size_t)p.next * weight_size;
  for (int step = 0; step < ns - 1; ++step) {
    int chunk = (p.idx - step + ns) % ns;
    span_t s = thread_span((size_t)chunk, p.per_chunk, p.per_thread, t, weight_size);
    memcpy(pb_next + s.begin, g + s.begin, sizeof(float) * (s.end - s.begin));
    handshake(rc, tid, p.prev * T + t, phase);
    int rd = (chunk - 1 + ns) % ns;
    s = thread_span((size_t)rd, p.per_chunk, p.per_thread, t, weight_size);
    if (step < ns - 2) {
#pragma omp simd
      for (size_t i = s.begin; i < s.end; ++i) g[i] = g[i] + pb[i];
    }
  }
}

/* all-gather with the update fused into its first step (mlp_omp.cc:171-295) */
static void ring_allgather(ring_ctx* rc, float* weights, float* grads, float* push, size_t weight_size, float alpha,
                           int sid, int t, int* phase) {
  const int ns = rc->ns, T = rc->T, tid = sid * T + t;
  const ring_plan p = plan_ring(rc, weight_size, sid, t);
  float* g = grads + (size_t)sid * weight_size;
  float* pb = push + (size_t)sid * weight_size;
  float* w = weights + (size_t)sid * weight_size;
  float* w_next = weights + (size_t)p.next * weight_size;
  const float neg_alpha = -alpha;
  if (ns == 1) {
    span_t s = thread_span(0, p.per_chunk, p.per_thread, t, weight_size);
#pragma omp simd
    for (size_t i = s.begin; i < s.end; ++i) w[i] = fmaf(neg_alpha, g[i], w[i]);
  }
  for (int step = 0; step < ns - 1; ++step) {
    int chunk = (p.idx + 1 - step + ns) % ns;
    span_t s = thread_span((size_t)chunk, p.per_chunk, p.per_thread, t, weight_size);
    if (step == 0) {
#pragma omp simd
      for (size_t i = s.begin; i < s.end; ++i) {
        float v = fmaf(neg_alpha, g[i] + pb[i], w[i]);
        w[i] = v;
        w_next[i] = v;
      }
    } else {
      memcpy(w_next + s.begin, w + s.begin, sizeof(float) * (s.end - s.begin));
    }
    handshake(rc, tid, p.prev * T + t, phase);
  }
}

static void ring_update(ring_ctx* rc, float* weights, float* grads, float* push, size_t weight_size, float alpha,
                        int sid, int t, int* phase) {
  ring_reduce_scatter(rc, grads, push, weight_size, sid, t, phase);
  ring_allgather(rc, weights, grads, push, weight_size, alpha, sid, t, phase);
}

/* The reference's start-up check of the all-reduce (mlp_omp.cc:325-373) on an arbitrary shape:
 * G_r[i][j] = r + i + j, W[i][j] = i*j, alpha = 1.  Returns the number of wrong elements over
 * all replicas (0 = pass); threads = ns * T. */
int port_check_all_reduce(int rows, int cols, int ns, int T) {
  const int ld = cols + PADF;
  const size_t wsz = (size_t)rows * ld;
  float* w = (float*)calloc(wsz * ns, sizeof(float));
  float* g = (float*)calloc(wsz * ns, sizeof(float));
  float* pb = (float*)calloc(wsz * ns, sizeof(float));
  ring_ctx rc = {ns, T, (_Atomic int*)calloc((size_t)ns * T * 16, sizeof(_Atomic int))};
  for (int s = 0; s < ns; ++s)
    for (int i = 0; i < rows; ++i)
      for (int j = 0; j < cols; ++j) {
        g[s * wsz + (size_t)i * ld + j] = (float)(s + i + j);
        w[s * wsz + (size_t)i * ld + j] = (float)i * (float)j;
      }
  int ran = 0;
#pragma omp parallel num_threads(ns* T)
  {
    if (omp_get_num_threads() == ns * T) {
      int tid = omp_get_thread_num(), phase = 0;
      ring_update(&rc, w, g, pb, wsz, 1.0f, tid / T, tid % T, &phase);
#pragma omp atomic
      ran += 1;
    }
  }
  int bad = (ran == ns * T) ? 0 : -1;
  for (int s = 0; s < ns && bad >= 0; ++s)
    for (int i = 0; i < rows; ++i)
      for (int j = 0; j < cols; ++j) {
        float expected = (float)i * (float)j - (float)((i + j) * ns + (ns - 1) * ns / 2);
        if (fabsf(w[s * wsz + (size_t)i * ld + j] - expected) > 1e-5f) ++bad;
      }
  free(w); free(g); free(pb); free((void*)rc.done);
  return bad;
}

/* ---- the training loop ------------------------------------------------------------------------ */

typedef struct {
  int rows, cols, ld;
  float* d;
} mat_t;

static mat_t mat_alloc(int rows, int cols) {
  mat_t m = {rows, cols, cols + PADF, NULL};
  if (posix_memalign((void**)&m.d, 4096, sizeof(float) * ((size_t)rows + PADF) * (size_t)m.ld)) m.d = NULL;
  if (m.d) memset(m.d, 0, sizeof(float) * ((size_t)rows + PADF) * (size_t)m.ld);
  return m;
}

/*
 * Runs `warmup + iters` training steps and times the last `iters`.
 *   nf[0..L], B rows per replica, R replicas ("sockets"), T threads per replica
 *   X [R*B x nf[0]], dY [R*B x nf[L]], W_in = concatenation over l of (W_l [nf[l+1] x nf[l]], b_l) -- dense
 *   restore != 0: every step starts from W_in again (what the GPU benchmark does)
 *   sgemm: cblas_sgemm-compatible function or NULL for the built-in kernel
 * Outputs (may be NULL): W_out (same layout as W_in, after the last step), dX_out [R*B x nf[0]],
 *   times_ms[5] = average per step of {fwd, wgt_grad, bwd, wgt_update, whole step}.
 * Returns 0, -1 on allocation failure, -2 if OpenMP did not provide R*T threads.
 */
static int mlp_run(int L, const int* nf, int B, int R, int T, int Tc, float lr, int relu_last, const float* X,
                   const float* dY, const float* W_in, int warmup, int iters, int restore, cblas_sgemm_fn sgemm,
                   float* W_out, float* dX_out, double* times_ms) {
  if (!sgemm) sgemm = port_builtin_sgemm;
  if (Tc < 0 || Tc >= T) return -3;
  const int Tg = T - Tc; /* threads of a socket that compute the backward GEMMs */
  const int MB = R * B, nthreads = R * T;
  mat_t* act = (mat_t*)calloc((size_t)L + 2, sizeof(mat_t));
  mat_t *wt = (mat_t*)calloc((size_t)L, sizeof(mat_t)), *gr = (mat_t*)calloc((size_t)L, sizeof(mat_t)),
        *pb = (mat_t*)calloc((size_t)L, sizeof(mat_t));
  int* brows = (int*)calloc((size_t)L, sizeof(int)); /* rows per replica incl. the rows that hold the bias */
  int ok = 1;
  for (int l = 0; l <= L; ++l) ok &= (act[l] = mat_alloc(MB, nf[l])).d != NULL;
  ok &= (act[L + 1] = mat_alloc(MB, nf[0])).d != NULL; /* spare buffer for the layer-0 input gradient (mlp_omp.cc:408) */
  for (int l = 0; l < L; ++l) {
    /* weights, gradients and push buffers hold R stacked replicas (mlp_omp.cc:395-403); the bias
     * of a replica is appended below its weight rows so that one ring pass updates both */
    const int ld = nf[l] + PADF;
    brows[l] = nf[l + 1] + ceil_div(nf[l + 1], ld);
    ok &= (wt[l] = mat_alloc(R * brows[l], nf[l])).d != NULL;
    ok &= (gr[l] = mat_alloc(R * brows[l], nf[l])).d != NULL;
    ok &= (pb[l] = mat_alloc(R * brows[l], nf[l])).d != NULL;
  }
  /* the ring is run by all T threads of a socket, or by its Tc communication threads */
  ring_ctx rc = {R, Tc > 0 ? Tc : T, (_Atomic int*)calloc((size_t)nthreads * 16, sizeof(_Atomic int))};
  if (!ok || !rc.done) return -1;

  for (int i = 0; i < MB; ++i) memcpy(act[0].d + (size_t)i * act[0].ld, X + (size_t)i * nf[0], sizeof(float) * nf[0]);

  double t_phase[4] = {0, 0, 0, 0}, t_total = 0;
  int ran = 0;

#pragma omp parallel num_threads(nthreads)
  {
    if (omp_get_num_threads() == nthreads) {
      const int tid = omp_get_thread_num(), sid = tid / T, t = tid % T;
      int phase = 0, blk[4];
      double my_phase[4] = {0, 0, 0, 0}, t_begin = 0;
#pragma omp atomic
      ran += 1;

      for (int it = 0; it < warmup + iters; ++it) {
        if (it == 0 || restore) { /* (re)load the initial weights into this socket's replica */
          size_t off = 0;
          for (int l = 0; l < L; ++l) {
            float* w = wt[l].d + (size_t)sid * brows[l] * wt[l].ld;
            for (int i = t; i < nf[l + 1]; i += T)
              memcpy(w + (size_t)i * wt[l].ld, W_in + off + (size_t)i * nf[l], sizeof(float) * nf[l]);
            if (t == 0) memcpy(w + (size_t)nf[l + 1] * wt[l].ld, W_in + off + (size_t)nf[l + 1] * nf[l], sizeof(float) * nf[l + 1]);
            off += (size_t)nf[l + 1] * nf[l] + nf[l + 1];
          }
#pragma omp barrier
        }
        if (it == warmup) {
#pragma omp barrier
          t_begin = omp_get_wtime();
          for (int i = 0; i < 4; ++i) my_phase[i] = 0;
        }

        /* forward (mlp_omp.cc:441-510) */
        for (int l = 0; l < L; ++l) {
          double t0 = omp_get_wtime();
          const int n = nf[l + 1], k = nf[l];
          port_partition_2d(MB, n, 4.0, 0, R, sid, T, t, blk);
          const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
          const float* w = wt[l].d + (size_t)sid * brows[l] * wt[l].ld;
          if (bm > 0 && bn > 0) {
            float* c = act[l + 1].d + (size_t)blk[0] * act[l + 1].ld + blk[2];
            sgemm(ROW_MAJOR, NO_TRANS, TRANS, bm, bn, k, 1.0f, act[l].d + (size_t)blk[0] * act[l].ld, act[l].ld,
                  w + (size_t)blk[2] * wt[l].ld, wt[l].ld, 0.0f, c, act[l + 1].ld);
            const float* bias = w + (size_t)n * wt[l].ld + blk[2];
            const int relu = (l < L - 1) || relu_last;
            for (int i = 0; i < bm; ++i) {
              float* ci = c + (size_t)i * act[l + 1].ld;
#pragma omp simd
              for (int j = 0; j < bn; ++j) {
                float v = ci[j] + bias[j];
                ci[j] = (relu && !(v > 0.0f)) ? 0.0f : v;
              }
            }
          }
          my_phase[0] += omp_get_wtime() - t0;
#pragma omp barrier
        }

        /* the upstream gradient takes the place of the output (the reference reuses the output
         * buffer as dY, mlp_omp.cc:565,655) */
        {
          int r0 = (int)((long long)MB * tid / nthreads), r1 = (int)((long long)MB * (tid + 1) / nthreads);
          for (int i = r0; i < r1; ++i) {
            float* o = act[L].d + (size_t)i * act[L].ld;
            const float* g = dY + (size_t)i * nf[L];
            for (int j = 0; j < nf[L]; ++j) o[j] = (relu_last && !(o[j] > 0.0f)) ? 0.0f : g[j];
          }
#pragma omp barrier
        }

        /* backward (mlp_omp.cc:513-736) */
        for (int l = L - 1; l >= 0; --l) {
          double t0 = omp_get_wtime();
          if (t < Tg) {
            /* weight gradient: k split over sockets, (m, n) split over the socket's GEMM threads */
            const int m = nf[l + 1], n = nf[l], k = MB;
            const int kps = ceil_div(k, R), k0 = imin(sid * kps, k), k1 = imin(k0 + kps, k);
            port_partition_2d_intra(m, n, 0.5, 1, Tg, t, blk);
            const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
            float* g = gr[l].d + (size_t)sid * brows[l] * gr[l].ld;
            if (bm > 0 && bn > 0)
              sgemm(ROW_MAJOR, TRANS, NO_TRANS, bm, bn, k1 - k0, 1.0f, act[l + 1].d + (size_t)k0 * act[l + 1].ld + blk[0],
                    act[l + 1].ld, act[l].d + (size_t)k0 * act[l].ld + blk[2], act[l].ld, 0.0f,
                    g + (size_t)blk[0] * gr[l].ld + blk[2], gr[l].ld);
            if (bm > 0 && blk[2] == 0) { /* bias gradient of these rows: column sums of this socket's dZ slice */
              float* db = g + (size_t)m * gr[l].ld + blk[0];
              for (int j = 0; j < bm; ++j) db[j] = 0.0f;
              for (int p = k0; p < k1; ++p) {
                const float* z = act[l + 1].d + (size_t)p * act[l + 1].ld + blk[0];
#pragma omp simd
                for (int j = 0; j < bm; ++j) db[j] += z[j];
              }
            }
            my_phase[1] += omp_get_wtime() - t0;
          } else if (l < L - 1) {
            /* communication thread: all-gather + SGD of the layer above (mlp_omp.cc:601-615); its last
             * reader, the input gradient of that layer, ended at the barrier before */
            ring_allgather(&rc, wt[l + 1].d, gr[l + 1].d, pb[l + 1].d, (size_t)brows[l + 1] * wt[l + 1].ld, lr, sid, t - Tg,
                           &phase);
            my_phase[3] += omp_get_wtime() - t0;
          }
#pragma omp barrier
          t0 = omp_get_wtime();
          if (t < Tg) {
            /* input gradient, in place over the activation; masked by the ReLU derivative */
            const int n = nf[l], k = nf[l + 1];
            port_partition_2d(MB, n, 0.5, 0, R, sid, Tg, t, blk);
            const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
            mat_t* C = &act[l == 0 ? L + 1 : l];
            const float* w = wt[l].d + (size_t)sid * brows[l] * wt[l].ld;
            if (bm > 0 && bn > 0) {
              if (l > 0) {
                /* the mask must be taken before the GEMM overwrites the activation */
                float* tmp = (float*)malloc(sizeof(float) * (size_t)bm * bn);
                sgemm(ROW_MAJOR, NO_TRANS, NO_TRANS, bm, bn, k, 1.0f, act[l + 1].d + (size_t)blk[0] * act[l + 1].ld,
                      act[l + 1].ld, w + blk[2], wt[l].ld, 0.0f, tmp, bn);
                for (int i = 0; i < bm; ++i) {
                  float* ci = C->d + (size_t)(blk[0] + i) * C->ld + blk[2];
                  const float* ti = tmp + (size_t)i * bn;
#pragma omp simd
                  for (int j = 0; j < bn; ++j) ci[j] = (ci[j] > 0.0f) ? ti[j] : 0.0f;
                }
                free(tmp);
              } else {
                sgemm(ROW_MAJOR, NO_TRANS, NO_TRANS, bm, bn, k, 1.0f, act[l + 1].d + (size_t)blk[0] * act[l + 1].ld,
                      act[l + 1].ld, w + blk[2], wt[l].ld, 0.0f, C->d + (size_t)blk[0] * C->ld + blk[2], C->ld);
              }
            }
            my_phase[2] += omp_get_wtime() - t0;
          } else {
            /* communication thread: reduce-scatter of this layer's gradients (mlp_omp.cc:692-705) */
            ring_reduce_scatter(&rc, gr[l].d, pb[l].d, (size_t)brows[l] * wt[l].ld, sid, t - Tg, &phase);
            my_phase[3] += omp_get_wtime() - t0;
          }
#pragma omp barrier
          t0 = omp_get_wtime();
          if (Tc == 0) {
            ring_update(&rc, wt[l].d, gr[l].d, pb[l].d, (size_t)brows[l] * wt[l].ld, lr, sid, t, &phase);
            my_phase[3] += omp_get_wtime() - t0;
          } else if (l == 0 && t >= Tg) { /* the all-gather nothing is left to overlap with (mlp_omp.cc:709-723) */
            ring_allgather(&rc, wt[0].d, gr[0].d, pb[0].d, (size_t)brows[0] * wt[0].ld, lr, sid, t - Tg, &phase);
            my_phase[3] += omp_get_wtime() - t0;
          }
        }
        /* the forward pass of the next step reads the activations the backward pass overwrote:
         * restore the input rows this thread owns is not needed (act[0] is never written), but
         * all updates must have landed before the next forward pass */
#pragma omp barrier
      }
      double dt = omp_get_wtime() - t_begin;
#pragma omp critical
      {
        for (int i = 0; i < 4; ++i)
          if (my_phase[i] > t_phase[i]) t_phase[i] = my_phase[i]; /* max over threads, like report_timing */
        if (dt > t_total) t_total = dt;
      }
    }
  }

  int rc_code = (ran == nthreads) ? 0 : -2;
  if (rc_code == 0) {
    if (W_out) {
      size_t off = 0;
      for (int l = 0; l < L; ++l) {
        for (int i = 0; i < nf[l + 1]; ++i)
          memcpy(W_out + off + (size_t)i * nf[l], wt[l].d + (size_t)i * wt[l].ld, sizeof(float) * nf[l]);
        memcpy(W_out + off + (size_t)nf[l + 1] * nf[l], wt[l].d + (size_t)nf[l + 1] * wt[l].ld, sizeof(float) * nf[l + 1]);
        off += (size_t)nf[l + 1] * nf[l] + nf[l + 1];
      }
    }
    if (dX_out)
      for (int i = 0; i < MB; ++i)
        memcpy(dX_out + (size_t)i * nf[0], act[L + 1].d + (size_t)i * act[L + 1].ld, sizeof(float) * nf[0]);
    if (times_ms) {
      for (int i = 0; i < 4; ++i) times_ms[i] = t_phase[i] / iters * 1e3;
      times_ms[4] = t_total / iters * 1e3;
    }
  }
  for (int l = 0; l <= L + 1; ++l) free(act[l].d);
  for (int l = 0; l < L; ++l) { free(wt[l].d); free(gr[l].d); free(pb[l].d); }
  free(act); free(wt); free(gr); free(pb); free(brows); free((void*)rc.done);
  return rc_code;
}

int port_mlp_run(int L, const int* nf, int B, int R, int T, float lr, int relu_last, const float* X, const float* dY,
                 const float* W_in, int warmup, int iters, int restore, cblas_sgemm_fn sgemm, float* W_out,
                 float* dX_out, double* times_ms) {
  return mlp_run(L, nf, B, R, T, 0, lr, relu_last, X, dY, W_in, warmup, iters, restore, sgemm, W_out, dX_out, times_ms);
}

/* The overlapped schedule with Tc communication threads per socket (Tc < 0: the reference's table).
 * Returns -3 when Tc leaves no GEMM thread. */
int port_mlp_run_overlap(int L, const int* nf, int B, int R, int T, int Tc, float lr, int relu_last, const float* X,
                         const float* dY, const float* W_in, int warmup, int iters, int restore, cblas_sgemm_fn sgemm,
                         float* W_out, float* dX_out, double* times_ms) {
  if (Tc < 0) Tc = port_comm_threads(T);
  return mlp_run(L, nf, B, R, T, Tc, lr, relu_last, X, dY, W_in, warmup, iters, restore, sgemm, W_out, dX_out, times_ms);
}
