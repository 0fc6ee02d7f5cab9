// Work partitioning of the benchmark: how a 1-D range or an m x n GEMM output is split first
// over sockets (data-parallel replicas) and then over the threads of a socket.  Function names,
// argument order and results are those of the reference (Partition.h:8-76, Partition.cc:25-247);
// the results are integers and must agree with it exactly.
//
// Overloads without socket / thread ids read them from the calling OpenMP thread, with threads
// numbered socket-major (thread id = socket * threads_per_socket + thread_in_socket).
#pragma once

#include <utility>

// number of sockets (replicas) the ranges are split over; set by the driver before use
extern int nsockets;

// Result of the thread-grid search: mb x nb thread blocks of bm x bn elements each.
struct ThreadGrid {
  int mb, nb, bm, bn;
};

// Chooses the mb x nb = T thread grid whose block shape bm/bn comes closest to aspect_ratio.
// bn is always a multiple of 16; bm too when m_align is set.
ThreadGrid choose_thread_grid(int m, int n, double aspect_ratio, bool m_align, int nthreads_per_socket);

int get_num_threads_per_socket();
int get_socket_num();
int get_thread_num_in_socket();

// ceil(work / nsockets)
int get_work_per_socket(int work);

// [begin, end) of `work` owned by one thread
std::pair<int, int> get_partition(int work);
std::pair<int, int> get_partition(int work, int nthreads_per_socket, int tid_in_socket);
std::pair<int, int> get_partition(int work, int socket_id, int nthreads_per_socket, int tid_in_socket);

// block of an m x n output owned by one thread of a socket that holds all m rows
void get_intra_socket_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                                  double aspect_ratio, bool m_align);
void get_intra_socket_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                                  double aspect_ratio, bool m_align, int nthreads_per_socket,
                                  int tid_in_socket);

// same, with the m rows first split evenly over the sockets
void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align);
void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align, int nthreads_per_socket, int tid_in_socket);
void get_2dpartition(int* m_begin, int* m_end, int* n_begin, int* n_end, int m, int n,
                     double aspect_ratio, bool m_align, int socket_id, int nthreads_per_socket,
                     int tid_in_socket);
