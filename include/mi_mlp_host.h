/*
 * mi_mlp_host.h -- C view of the benchmark's host-side helpers (libmi_mlp_host.so), for callers
 * that cannot include the C++ headers (tests through ctypes, other languages).  Each function
 * forwards to the C++ function of the same name in tbb_test_amd/host/, which keeps the
 * reference's signature; the reference counterpart is cited per function.  No GPU is involved.
 */
#ifndef MI_MLP_HOST_H
#define MI_MLP_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* sets the global `nsockets` the partition functions split over (Partition.cc:6) */
void mi_host_set_nsockets(int n);
/* Partition.cc:25-27 */
int mi_host_get_work_per_socket(int work);
/* Partition.cc:30-48; out2 = {begin, end} */
void mi_host_get_partition(int work, int socket_id, int nthreads_per_socket, int tid_in_socket, int* out2);
/* Partition.cc:75-166; out4 = {m_begin, m_end, n_begin, n_end} */
void mi_host_get_intra_socket_2dpartition(int m, int n, double aspect_ratio, int m_align,
                                          int nthreads_per_socket, int tid_in_socket, int* out4);
/* Partition.cc:193-222 */
void mi_host_get_2dpartition(int m, int n, double aspect_ratio, int m_align, int socket_id,
                             int nthreads_per_socket, int tid_in_socket, int* out4);
/* The OpenMP-id overloads (Partition.cc:8-23,29-32,57-73,168-191): runs an OpenMP parallel region
 * of nsockets * nthreads_per_socket threads and stores what thread t obtained at
 * out[4*t .. 4*t+3].  Returns the number of threads that actually ran. */
int mi_host_get_2dpartition_omp(int m, int n, double aspect_ratio, int m_align,
                                int nthreads_per_socket, int* out);
/* mlp_bench_common.cc:170-190; out3 = {idx_in_ring, prev_sid, next_sid} */
void mi_host_get_my_ring_info(int sid, int task, int* out3);

/* seeded fills (tbb_test_amd/host/Rand.h; replaces the MKL stream of Rand.cc:14-49) */
void mi_host_rand_seed(uint64_t seed);
void mi_host_rand_stream(uint64_t stream);
uint64_t mi_host_rand_raw(uint64_t seed, uint64_t stream, uint64_t counter);
void mi_host_rand_uniform(float* dst, size_t len, float low, float high);
void mi_host_rand_normal(float* dst, size_t len, float mean, float stddev);
/* Rand.cc:83-130; duplicates == 0 samples without replacement from [low, high] */
int mi_host_rand_ints(int* dst, int len, int low, int high, int duplicates);

/* Fills the benchmark's seeded inputs for a model (init_matrices of the driver) into dense
 * caller buffers: X[R*B x nf[0]], W = concatenation of W_l[nf[l+1] x nf[l]], dY[R*B x nf[L]]. */
void mi_host_init_problem(int L, const int* nfeatures, int batch_per_replica, int R, uint64_t seed,
                          float* X, float* W, float* dY);

#ifdef __cplusplus
}
#endif
#endif /* MI_MLP_HOST_H */
