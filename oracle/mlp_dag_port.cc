/*
 * CPU baseline, second scheduler: a restatement of the reference's mlp_tbb -- the training step as
 * a dependency-counted task graph executed by one arena of worker threads per "socket" -- timed by
 * the cpu_baseline leg next to the OpenMP restatement (mlp_omp_port.c).  TEST / MEASUREMENT
 * INFRASTRUCTURE ONLY -- the product never links it.  The reference needs TBB (<= 2020) and MKL
 * headers, neither of which this image has, so the graph machinery is restated on std::thread:
 *
 *   arenas     one pool of T threads per socket (tbb::task_arena per socket, mlp_tbb.cc:1229-1232);
 *              a node runs in the arena of the socket it belongs to
 *   nodes      continue_node semantics (mlp_tbb.cc:478): a node starts once every predecessor has
 *              finished; an edge into another socket's graph just enqueues into that arena (the
 *              reference needs an async_node per such edge, mlp_tbb.cc:463-476)
 *   forward    per layer and socket T block tasks (the tbb::parallel_for of mlp_tbb.cc:815-913,
 *              blocks from get_2dpartition with aspect ratio 4) and a join; layer l+1 of a socket
 *              depends only on layer l of the same socket (mlp_tbb.cc:1289-1311)
 *   backward   per layer and socket: weight-gradient block tasks, join, input-gradient block
 *              tasks, join (the two parallel_for of FullyConnectedBackward, mlp_tbb.cc:957-1196),
 *              chained per socket from the last layer down (mlp_tbb.cc:1314-1330); both use
 *              T - T_comm tasks, T_comm from the table at mlp_bench_common.h:40-48
 *   all-reduce per layer a sub-graph of ReduceScatter(step, socket, task) and AllGather(step,
 *              socket, task) nodes (mlp_tbb.cc:142-456,486-655): step s of a socket depends on
 *              step s-1 of the previous socket in the ring; the SGD update is fused into the first
 *              all-gather step.  It starts when every socket has finished the layer's backward
 *              node and runs concurrently with the backward nodes of the layers below
 *              (mlp_tbb.cc:1344-1357).
 *
 * Deliberate differences from the reference, all needed for correct results:
 *   - with fewer than 5 threads per socket the reference's table gives zero all-reduce tasks (no
 *     update at all); here at least one task per socket runs, on the same threads as the GEMMs;
 *   - for two sockets the reference makes the first all-gather step depend only on the same
 *     socket's reduce-scatter step (mlp_tbb.cc:601-605) although it reads what the other socket
 *     pushed; here it depends on both;
 *   - the position in the reversed ring of odd tasks counts along the ring direction (the
 *     reference's rule, mlp_bench_common.cc:183-189, only closes the ring for two sockets);
 *   - bias, ReLU, the ReLU mask, db and an explicit dY are added as in mlp_omp_port.c.
 *
 * Pinned by tests/test_cpu_port.py: final weights and dX against the float64-accumulating oracle
 * and bit-for-bit against the OpenMP restatement (same block shapes, same ring arithmetic).
 */
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

extern "C" {
typedef void (*cblas_sgemm_fn)(int order, int transa, int transb, int m, int n, int k, float alpha, const float* a,
                               int lda, const float* b, int ldb, float beta, float* c, int ldc);
void port_partition_2d_intra(int m, int n, double ar, int m_align, int T, int t, int out[4]);
void port_partition_2d(int m, int n, double ar, int m_align, int ns, int sid, int T, int t, int out[4]);
void port_ring_info(int ns, int sid, int task, int out[3]);
void port_builtin_sgemm(int order, int ta, int tb, int m, int n, int k, float alpha, const float* a, int lda,
                        const float* b, int ldb, float beta, float* c, int ldc);
}

namespace {

enum { ROW_MAJOR = 101, NO_TRANS = 111, TRANS = 112 };
enum Phase { P_FWD = 0, P_WGT = 1, P_BWD = 2, P_UPD = 3, P_NONE = 4 };
constexpr int PADF = 16, LINE = 16;

/* threads per socket reserved for the all-reduce (mlp_bench_common.h:40-48) */
int comm_threads(int T) {
  if (T >= 20) return 4;
  if (T >= 10) return 2;
  if (T >= 5) return 1;
  return 0;
}

double now() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

struct Mat {
  int rows = 0, cols = 0, ld = 0;
  float* d = nullptr;
  bool alloc(int r, int c) {
    rows = r; cols = c; ld = c + PADF;
    const size_t bytes = sizeof(float) * ((size_t)r + PADF) * (size_t)ld;
    if (posix_memalign((void**)&d, 4096, bytes)) d = nullptr;
    if (d) memset(d, 0, bytes);
    return d != nullptr;
  }
  ~Mat() { free(d); }
};

/* ---- the task graph ---------------------------------------------------------------------------- */

struct Node {
  std::function<void()> fn;  // empty = join node
  int arena = 0, ndeps = 0, phase = P_NONE;
  std::vector<int> succ;
};

class Graph {
 public:
  Graph(int arenas, int threads_per_arena) : pools_(arenas), per_thread_(arenas * threads_per_arena) {
    for (auto& t : per_thread_) std::fill(t.phase_s, t.phase_s + 4, 0.0);
    for (int a = 0; a < arenas; ++a) {
      pools_[a].reset(new Pool);
      for (int t = 0; t < threads_per_arena; ++t)
        pools_[a]->threads.emplace_back([this, a, t, threads_per_arena] { work(a, a * threads_per_arena + t); });
    }
  }
  ~Graph() {
    for (auto& p : pools_) {
      { std::lock_guard<std::mutex> g(p->m); p->stop = true; }
      p->cv.notify_all();
    }
    for (auto& p : pools_)
      for (auto& t : p->threads) t.join();
  }
  int add(int arena, int phase, std::function<void()> fn) {
    nodes_.emplace_back();
    nodes_.back().fn = std::move(fn);
    nodes_.back().arena = arena;
    nodes_.back().phase = phase;
    return (int)nodes_.size() - 1;
  }
  void edge(int from, int to) {
    nodes_[from].succ.push_back(to);
    nodes_[to].ndeps++;
  }
  /* one pass over the graph: the analogue of dag_root.try_put + wait_for_all (mlp_tbb.cc:1361-1365) */
  void run(int root, int exit_node) {
    if (pending_.size() != nodes_.size()) pending_ = std::vector<std::atomic<int>>(nodes_.size());
    for (size_t i = 0; i < nodes_.size(); ++i) pending_[i].store(nodes_[i].ndeps, std::memory_order_relaxed);
    exit_ = exit_node;
    done_.store(false, std::memory_order_release);
    push(root);
    std::unique_lock<std::mutex> g(done_m_);
    done_cv_.wait(g, [this] { return done_.load(std::memory_order_acquire); });
  }
  void reset_times() {
    for (auto& t : per_thread_) std::fill(t.phase_s, t.phase_s + 4, 0.0);
  }
  /* per phase the maximum over threads of the time spent in it, like report_timing takes it */
  void max_times(double out[4]) const {
    for (int p = 0; p < 4; ++p) {
      out[p] = 0;
      for (auto& t : per_thread_) out[p] = std::max(out[p], t.phase_s[p]);
    }
  }
  size_t size() const { return nodes_.size(); }

 private:
  struct Pool {
    std::mutex m;
    std::condition_variable cv;
    std::deque<int> q;
    bool stop = false;
    std::vector<std::thread> threads;
  };
  struct alignas(64) ThreadTimes { double phase_s[4]; };

  void push(int id) {
    Pool& p = *pools_[nodes_[id].arena];
    { std::lock_guard<std::mutex> g(p.m); p.q.push_back(id); }
    p.cv.notify_one();
  }
  void finish(int id) {
    for (int s : nodes_[id].succ)
      if (pending_[s].fetch_sub(1, std::memory_order_acq_rel) == 1) {
        if (!nodes_[s].fn && s != exit_) finish(s);  // joins complete on the spot
        else push(s);
      }
    if (id == exit_) {
      { std::lock_guard<std::mutex> g(done_m_); done_.store(true, std::memory_order_release); }
      done_cv_.notify_all();
    }
  }
  void work(int arena, int thread_index) {
    Pool& p = *pools_[arena];
    for (;;) {
      int id;
      {
        std::unique_lock<std::mutex> g(p.m);
        p.cv.wait(g, [&p] { return p.stop || !p.q.empty(); });
        if (p.q.empty()) return;
        id = p.q.front();
        p.q.pop_front();
      }
      Node& n = nodes_[id];
      if (n.fn) {
        const double t0 = now();
        n.fn();
        if (n.phase < P_NONE) per_thread_[thread_index].phase_s[n.phase] += now() - t0;
      }
      finish(id);
    }
  }

  std::vector<Node> nodes_;
  std::vector<std::atomic<int>> pending_;
  std::vector<std::unique_ptr<Pool>> pools_;
  std::vector<ThreadTimes> per_thread_;
  std::mutex done_m_;
  std::condition_variable done_cv_;
  std::atomic<bool> done_{false};
  int exit_ = -1;
};

struct Span { size_t begin, end; };
Span task_span(size_t chunk, size_t per_chunk, size_t per_task, int task, size_t total) {
  const size_t cb = std::min(chunk * per_chunk, total), ce = std::min(cb + per_chunk, total);
  Span s;
  s.begin = std::min(cb + (size_t)task * per_task, ce);
  s.end = std::min(s.begin + per_task, ce);
  return s;
}

}  // namespace

/*
 * Same contract as port_mlp_run (mlp_omp_port.c): runs warmup + iters steps, times the last iters.
 * times_ms[5] = {fwd, wgt_grad, bwd, wgt_update (max over threads of the time inside such tasks),
 * whole step}.  Returns 0, -1 on allocation failure.
 */
extern "C" int port_mlp_dag_run(int L, const int* nf, int B, int R, int T, float lr, int relu_last, const float* X,
                                const float* dY, const float* W_in, int warmup, int iters, int restore,
                                cblas_sgemm_fn sgemm, float* W_out, float* dX_out, double* times_ms) {
  if (!sgemm) sgemm = port_builtin_sgemm;
  const int MB = R * B;
  const int Tcomm = std::max(1, comm_threads(T));
  const int Tg = std::max(1, T - comm_threads(T));
  std::vector<Mat> act(L + 2), wt(L), gr(L), pb(L);
  std::vector<int> brows(L);
  bool ok = true;
  for (int l = 0; l <= L; ++l) ok = ok && act[l].alloc(MB, nf[l]);
  ok = ok && act[L + 1].alloc(MB, nf[0]);  // spare buffer for the layer-0 input gradient (mlp_tbb.cc:1252-1254)
  for (int l = 0; l < L; ++l) {
    // R stacked replicas (mlp_tbb.cc:1240-1249); a replica's bias sits in extra rows below its weights
    const int ld = nf[l] + PADF;
    brows[l] = nf[l + 1] + (nf[l + 1] + ld - 1) / ld;
    ok = ok && wt[l].alloc(R * brows[l], nf[l]) && gr[l].alloc(R * brows[l], nf[l]) && pb[l].alloc(R * brows[l], nf[l]);
  }
  if (!ok) return -1;
  for (int i = 0; i < MB; ++i) memcpy(act[0].d + (size_t)i * act[0].ld, X + (size_t)i * nf[0], sizeof(float) * nf[0]);

  auto load_weights = [&](int sid, int t, int nt) {
    size_t off = 0;
    for (int l = 0; l < L; ++l) {
      float* w = wt[l].d + (size_t)sid * brows[l] * wt[l].ld;
      for (int i = t; i < nf[l + 1]; i += nt)
        memcpy(w + (size_t)i * wt[l].ld, W_in + off + (size_t)i * nf[l], sizeof(float) * nf[l]);
      if (t == 0)
        memcpy(w + (size_t)nf[l + 1] * wt[l].ld, W_in + off + (size_t)nf[l + 1] * nf[l], sizeof(float) * nf[l + 1]);
      off += (size_t)nf[l + 1] * nf[l] + nf[l + 1];
    }
  };

  Graph g(R, T);
  const int root = g.add(0, P_NONE, nullptr), exit_node = g.add(0, P_NONE, nullptr);

  // (re)load of the initial weights, inside the step like the GPU benchmark's restore
  std::vector<int> chain(R);  // last node of each socket's chain so far
  for (int s = 0; s < R; ++s) {
    if (restore) {
      const int join = g.add(s, P_NONE, nullptr);
      for (int t = 0; t < T; ++t) {
        const int n = g.add(s, P_NONE, [&, s, t] { load_weights(s, t, T); });
        g.edge(root, n);
        g.edge(n, join);
      }
      chain[s] = join;
    } else {
      chain[s] = root;
    }
  }

  // forward
  for (int l = 0; l < L; ++l)
    for (int s = 0; s < R; ++s) {
      const int join = g.add(s, P_NONE, nullptr);
      for (int t = 0; t < T; ++t) {
        const int n = g.add(s, P_FWD, [&, l, s, t] {
          int blk[4];
          const int nn = nf[l + 1], k = nf[l];
          port_partition_2d(MB, nn, 4.0, 0, R, s, T, t, blk);
          const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
          if (bm <= 0 || bn <= 0) return;
          const float* w = wt[l].d + (size_t)s * brows[l] * wt[l].ld;
          float* c = act[l + 1].d + (size_t)blk[0] * act[l + 1].ld + blk[2];
          sgemm(ROW_MAJOR, NO_TRANS, TRANS, bm, bn, k, 1.0f, act[l].d + (size_t)blk[0] * act[l].ld, act[l].ld,
                w + (size_t)blk[2] * wt[l].ld, wt[l].ld, 0.0f, c, act[l + 1].ld);
          const float* bias = w + (size_t)nn * wt[l].ld + blk[2];
          const bool relu = (l < L - 1) || relu_last;
          for (int i = 0; i < bm; ++i) {
            float* ci = c + (size_t)i * act[l + 1].ld;
            for (int j = 0; j < bn; ++j) {
              const float v = ci[j] + bias[j];
              ci[j] = (relu && !(v > 0.0f)) ? 0.0f : v;
            }
          }
        });
        g.edge(chain[s], n);
        g.edge(n, join);
      }
      chain[s] = join;
    }

  // the upstream gradient takes the place of the output (the reference reuses the output buffer as
  // dY, mlp_tbb.cc:1319-1322); each socket copies its own rows
  for (int s = 0; s < R; ++s) {
    const int join = g.add(s, P_NONE, nullptr);
    for (int t = 0; t < T; ++t) {
      const int n = g.add(s, P_NONE, [&, s, t] {
        const int r0 = s * B + (int)((long long)B * t / T), r1 = s * B + (int)((long long)B * (t + 1) / T);
        for (int i = r0; i < r1; ++i) {
          float* o = act[L].d + (size_t)i * act[L].ld;
          const float* gy = dY + (size_t)i * nf[L];
          for (int j = 0; j < nf[L]; ++j) o[j] = (relu_last && !(o[j] > 0.0f)) ? 0.0f : gy[j];
        }
      });
      g.edge(chain[s], n);
      g.edge(n, join);
    }
    chain[s] = join;
  }

  // backward, and per layer the all-reduce sub-graph
  const float neg_alpha = -lr;
  for (int l = L - 1; l >= 0; --l) {
    for (int s = 0; s < R; ++s) {
      const int join_w = g.add(s, P_NONE, nullptr);
      for (int t = 0; t < Tg; ++t) {
        const int n = g.add(s, P_WGT, [&, l, s, t] {
          // weight gradient: batch (k) split over sockets, (m, n) split inside the socket
          int blk[4];
          const int m = nf[l + 1], nn = nf[l], k = MB;
          const int kps = (k + R - 1) / R, k0 = std::min(s * kps, k), k1 = std::min(k0 + kps, k);
          port_partition_2d_intra(m, nn, 0.5, 1, Tg, t, blk);
          const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
          float* gs = gr[l].d + (size_t)s * brows[l] * gr[l].ld;
          if (bm > 0 && bn > 0)
            sgemm(ROW_MAJOR, TRANS, NO_TRANS, bm, bn, k1 - k0, 1.0f, act[l + 1].d + (size_t)k0 * act[l + 1].ld + blk[0],
                  act[l + 1].ld, act[l].d + (size_t)k0 * act[l].ld + blk[2], act[l].ld, 0.0f,
                  gs + (size_t)blk[0] * gr[l].ld + blk[2], gr[l].ld);
          if (bm > 0 && blk[2] == 0) {  // bias gradient of these rows: column sums of the socket's dZ slice
            float* db = gs + (size_t)m * gr[l].ld + blk[0];
            for (int j = 0; j < bm; ++j) db[j] = 0.0f;
            for (int p = k0; p < k1; ++p) {
              const float* z = act[l + 1].d + (size_t)p * act[l + 1].ld + blk[0];
              for (int j = 0; j < bm; ++j) db[j] += z[j];
            }
          }
        });
        g.edge(chain[s], n);
        g.edge(n, join_w);
      }
      const int join_b = g.add(s, P_NONE, nullptr);
      for (int t = 0; t < Tg; ++t) {
        const int n = g.add(s, P_BWD, [&, l, s, t] {
          // input gradient, in place over the activation, masked by the ReLU derivative
          int blk[4];
          const int nn = nf[l], k = nf[l + 1];
          port_partition_2d(MB, nn, 0.5, 0, R, s, Tg, t, blk);
          const int bm = blk[1] - blk[0], bn = blk[3] - blk[2];
          if (bm <= 0 || bn <= 0) return;
          Mat& C = act[l == 0 ? L + 1 : l];
          const float* w = wt[l].d + (size_t)s * brows[l] * wt[l].ld;
          if (l > 0) {
            std::vector<float> tmp((size_t)bm * bn);
            sgemm(ROW_MAJOR, NO_TRANS, NO_TRANS, bm, bn, k, 1.0f, act[l + 1].d + (size_t)blk[0] * act[l + 1].ld,
                  act[l + 1].ld, w + blk[2], wt[l].ld, 0.0f, tmp.data(), bn);
            for (int i = 0; i < bm; ++i) {
              float* ci = C.d + (size_t)(blk[0] + i) * C.ld + blk[2];
              const float* ti = tmp.data() + (size_t)i * bn;
              for (int j = 0; j < bn; ++j) ci[j] = (ci[j] > 0.0f) ? ti[j] : 0.0f;
            }
          } else {
            sgemm(ROW_MAJOR, NO_TRANS, NO_TRANS, bm, bn, k, 1.0f, act[l + 1].d + (size_t)blk[0] * act[l + 1].ld,
                  act[l + 1].ld, w + blk[2], wt[l].ld, 0.0f, C.d + (size_t)blk[0] * C.ld + blk[2], C.ld);
          }
        });
        g.edge(join_w, n);
        g.edge(n, join_b);
      }
      chain[s] = join_b;
    }

    // all-reduce of layer l: starts when every socket has finished the layer's backward node
    const int ar_root = g.add(0, P_NONE, nullptr);
    for (int s = 0; s < R; ++s) g.edge(chain[s], ar_root);
    const size_t weight_size = (size_t)brows[l] * wt[l].ld;
    const size_t per_chunk = (weight_size + (size_t)R * LINE - 1) / R / LINE * LINE;
    const size_t per_task = (per_chunk + (size_t)Tcomm * LINE - 1) / Tcomm / LINE * LINE;
    auto ring = [&](int s, int task, int* idx, int* prev, int* next) {
      int info[3];
      port_ring_info(R, s, task, info);
      *idx = (R < 8 && (task % 2)) ? (R - s) % R : info[0];
      *prev = info[1];
      *next = info[2];
    };
    // rs[step][s][task], ag[step][s][task]
    std::vector<int> rs((size_t)std::max(R - 1, 0) * R * Tcomm), ag((size_t)std::max(R - 1, 1) * R * Tcomm);
    auto at = [&](std::vector<int>& v, int step, int s, int task) -> int& { return v[((size_t)step * R + s) * Tcomm + task]; };
    for (int step = 0; step < R - 1; ++step)
      for (int s = 0; s < R; ++s)
        for (int task = 0; task < Tcomm; ++task) {
          int idx, prev, next;
          ring(s, task, &idx, &prev, &next);
          const int n = g.add(s, P_UPD, [&, l, step, s, task, idx, next, weight_size, per_chunk, per_task] {
            // accumulate what the previous socket pushed in its step-1, then push the chunk onward
            // (mlp_tbb.cc:205-236)
            float* gsock = gr[l].d + (size_t)s * weight_size;
            const float* mine = pb[l].d + (size_t)s * weight_size;
            float* to = pb[l].d + (size_t)next * weight_size;
            const int chunk = (idx - step + R) % R;
            const Span sp = task_span((size_t)chunk, per_chunk, per_task, task, weight_size);
            if (step > 0)
              for (size_t i = sp.begin; i < sp.end; ++i) gsock[i] = gsock[i] + mine[i];
            memcpy(to + sp.begin, gsock + sp.begin, sizeof(float) * (sp.end - sp.begin));
          });
          at(rs, step, s, task) = n;
          if (step == 0) g.edge(ar_root, n);
          else g.edge(at(rs, step - 1, prev, task), n);
        }
    for (int step = 0; step < std::max(R - 1, 1); ++step)
      for (int s = 0; s < R; ++s)
        for (int task = 0; task < Tcomm; ++task) {
          int idx, prev, next;
          ring(s, task, &idx, &prev, &next);
          const int n = g.add(s, P_UPD, [&, l, step, s, task, idx, next, weight_size, per_chunk, per_task] {
            // first step: last add and the SGD update, written to this socket and the next; later
            // steps forward the chunk received in the step before (mlp_tbb.cc:345-420)
            float* w = wt[l].d + (size_t)s * weight_size;
            float* w_next = wt[l].d + (size_t)next * weight_size;
            const float* gsock = gr[l].d + (size_t)s * weight_size;
            const float* mine = pb[l].d + (size_t)s * weight_size;
            if (R == 1) {
              const Span sp = task_span(0, per_chunk, per_task, task, weight_size);
              for (size_t i = sp.begin; i < sp.end; ++i) w[i] = fmaf(neg_alpha, gsock[i], w[i]);
              return;
            }
            const int chunk = (idx + 1 - step + R) % R;
            const Span sp = task_span((size_t)chunk, per_chunk, per_task, task, weight_size);
            if (step == 0) {
              for (size_t i = sp.begin; i < sp.end; ++i) {
                const float v = fmaf(neg_alpha, gsock[i] + mine[i], w[i]);
                w[i] = v;
                w_next[i] = v;
              }
            } else {
              memcpy(w_next + sp.begin, w + sp.begin, sizeof(float) * (sp.end - sp.begin));
            }
          });
          at(ag, step, s, task) = n;
          if (R == 1) {
            g.edge(ar_root, n);
          } else if (step == 0) {
            g.edge(at(rs, R - 2, s, task), n);
            g.edge(at(rs, R - 2, prev, task), n);
          } else {
            g.edge(at(ag, step - 1, prev, task), n);
            g.edge(at(ag, step - 1, s, task), n);
          }
          if (step == std::max(R - 1, 1) - 1) g.edge(n, exit_node);
        }
  }
  for (int s = 0; s < R; ++s) g.edge(chain[s], exit_node);

  if (!restore)
    for (int s = 0; s < R; ++s) load_weights(s, 0, 1);
  double t_begin = 0;
  for (int it = 0; it < warmup + iters; ++it) {
    if (it == warmup) {
      g.reset_times();
      t_begin = now();
    }
    g.run(root, exit_node);
  }
  const double t_total = now() - t_begin;

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
    double ph[4];
    g.max_times(ph);
    for (int i = 0; i < 4; ++i) times_ms[i] = ph[i] / std::max(iters, 1) * 1e3;
    times_ms[4] = t_total / std::max(iters, 1) * 1e3;
  }
  return 0;
}

/* number of graph nodes of one step, for tests of the graph shape */
extern "C" int port_mlp_dag_comm_tasks(int T) { return std::max(1, comm_threads(T)); }
