#include "Partition.h"

#include <algorithm>
#include <cassert>
#include <cmath>

#include <omp.h>

int nsockets = 1;

namespace {

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// extent of one thread block when `count` items are cut into `parts`; optionally rounded so that
// every block starts on a multiple of 16 (one 64-byte line of floats)
inline int block_extent(int count, int parts, bool align16) {
  return align16 ? ceil_div(ceil_div(count, 16), parts) * 16 : ceil_div(count, parts);
}

struct Span {
  int begin, end;
};

inline Span clamp_block(int index, int extent, int limit) {
  int b = std::min(index * extent, limit);
  return {b, std::min(b + extent, limit)};
}

}  // namespace

int get_num_threads_per_socket() {
  int total = omp_in_parallel() ? omp_get_num_threads() : omp_get_max_threads();
  assert(total % nsockets == 0);
  return total / nsockets;
}

int get_socket_num() { return omp_get_thread_num() / get_num_threads_per_socket(); }

int get_thread_num_in_socket() { return omp_get_thread_num() % get_num_threads_per_socket(); }

int get_work_per_socket(int work) { return ceil_div(work, nsockets); }

// ---- 1-D ----------------------------------------------------------------------------------

std::pair<int, int> get_partition(int work, int socket_id, int nthreads_per_socket, int tid_in_socket) {
  const int per_socket = get_work_per_socket(work);
  const int socket_base = std::min(socket_id * per_socket, work);
  const Span in_socket = clamp_block(tid_in_socket, ceil_div(per_socket, nthreads_per_socket), per_socket);
  return {std::min(socket_base + in_socket.begin, work), std::min(socket_base + in_socket.end, work)};
}

std::pair<int, int> get_partition(int work, int nthreads_per_socket, int tid_in_socket) {
  return get_partition(work, get_socket_num(), nthreads_per_socket, tid_in_socket);
}

std::pair<int, int> get_partition(int work) {
  return get_partition(work, get_num_threads_per_socket(), get_thread_num_in_socket());
}

// ---- 2-D ----------------------------------------------------------------------------------

ThreadGrid choose_thread_grid(int m, int n, double aspect_ratio, bool m_align, int T) {
  // Start from a single row of T blocks and walk the divisors of T upwards as the number of
  // block rows; keep going only while the block shape gets strictly closer to the target.
  ThreadGrid g{1, T, block_extent(m, 1, m_align), block_extent(n, T, true)};
  double best = std::abs((double)g.bm / g.bn - aspect_ratio);

  for (int rows = 2; rows <= T; ++rows) {
    if (T % rows) continue;
    const int cols = T / rows;
    const int m_per_block = ceil_div(m, rows);
    if (m_align) {
      // blocks are already a single 16-row line: splitting further would leave rows idle
      if (aspect_ratio < 1 && g.bm == 16 && m_per_block < 16) continue;
      if (m_per_block <= 8) continue;
    }
    if (ceil_div(n, cols) <= 8) continue;

    ThreadGrid c{rows, cols, block_extent(m, rows, m_align), block_extent(n, cols, true)};
    const double delta = std::abs((double)c.bm / c.bn - aspect_ratio);
    if (!(delta < best)) break;
    best = delta;
    g = c;
  }
  return g;
}

void get_intra_socket_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                                  double aspect_ratio, bool m_align, int nthreads_per_socket,
                                  int tid_in_socket) {
  const ThreadGrid g = choose_thread_grid(m, n, aspect_ratio, m_align, nthreads_per_socket);
  const Span rows = clamp_block(tid_in_socket / g.nb, g.bm, m);
  const Span cols = clamp_block(tid_in_socket % g.nb, g.bn, n);
  *m_begin = rows.begin;
  *m_end = rows.end;
  *n_begin = cols.begin;
  *n_end = cols.end;
}

void get_intra_socket_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                                  double aspect_ratio, bool m_align) {
  get_intra_socket_2dpartition(m_begin, m_end, n_begin, n_end, m, n, aspect_ratio, m_align,
                               get_num_threads_per_socket(), get_thread_num_in_socket());
}

void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align, int socket_id, int nthreads_per_socket,
                     int tid_in_socket) {
  const int rows_per_socket = get_work_per_socket(m);
  get_intra_socket_2dpartition(m_begin, m_end, n_begin, n_end, rows_per_socket, n, aspect_ratio,
                               m_align, nthreads_per_socket, tid_in_socket);
  const int socket_base = std::min(socket_id * rows_per_socket, m);
  *m_begin = std::min(socket_base + *m_begin, m);
  *m_end = std::min(socket_base + *m_end, m);
}

void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align, int nthreads_per_socket, int tid_in_socket) {
  get_2dpartition(m_begin, m_end, n_begin, n_end, m, n, aspect_ratio, m_align, get_socket_num(),
                  nthreads_per_socket, tid_in_socket);
}

void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align) {
  get_2dpartition(m_begin, m_end, n_begin, n_end, m, n, aspect_ratio, m_align,
                  get_num_threads_per_socket(), get_thread_num_in_socket());
}
