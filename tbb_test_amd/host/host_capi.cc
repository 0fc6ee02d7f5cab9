// C exports of the host-side helpers (include/mi_mlp_host.h): thin forwards to the C++ API.
#include "mi_mlp_host.h"

#include <omp.h>

#include <stdexcept>

#include "mlp_bench_common.h"

extern "C" {

void mi_host_set_nsockets(int n) { nsockets = n; }

int mi_host_get_work_per_socket(int work) { return get_work_per_socket(work); }

void mi_host_get_partition(int work, int socket_id, int T, int t, int* out2) {
  std::pair<int, int> r = get_partition(work, socket_id, T, t);
  out2[0] = r.first;
  out2[1] = r.second;
}

void mi_host_get_intra_socket_2dpartition(int m, int n, double ar, int m_align, int T, int t, int* out4) {
  get_intra_socket_2dpartition(&out4[0], &out4[1], &out4[2], &out4[3], m, n, ar, m_align != 0, T, t);
}

void mi_host_get_2dpartition(int m, int n, double ar, int m_align, int sid, int T, int t, int* out4) {
  get_2dpartition(&out4[0], &out4[1], &out4[2], &out4[3], m, n, ar, m_align != 0, sid, T, t);
}

int mi_host_get_2dpartition_omp(int m, int n, double ar, int m_align, int T, int* out) {
  int ran = 0;
  const int total = nsockets * T;
#pragma omp parallel num_threads(total)
  {
    if (omp_get_num_threads() == total) {
      int* o = out + 4 * omp_get_thread_num();
      get_2dpartition(&o[0], &o[1], &o[2], &o[3], m, n, ar, m_align != 0);
#pragma omp atomic
      ran += 1;
    }
  }
  return ran;
}

void mi_host_get_my_ring_info(int sid, int task, int* out3) {
  get_my_ring_info(sid, task, &out3[0], &out3[1], &out3[2]);
}

void mi_host_rand_seed(uint64_t seed) { randSeed(seed); }
void mi_host_rand_stream(uint64_t stream) { randStream(stream); }
uint64_t mi_host_rand_raw(uint64_t seed, uint64_t stream, uint64_t counter) { return randRaw(seed, stream, counter); }
void mi_host_rand_uniform(float* dst, size_t len, float low, float high) { randFill(dst, len, low, high); }
void mi_host_rand_normal(float* dst, size_t len, float mean, float stddev) { randFillNormal(dst, len, mean, stddev); }

int mi_host_rand_ints(int* dst, int len, int low, int high, int duplicates) {
  try {
    randFill(dst, len, low, high, duplicates != 0);
  } catch (const std::invalid_argument&) {
    return -1;
  }
  return 0;
}

void mi_host_init_problem(int L, const int* nf, int B, int R, uint64_t seed, float* X, float* W, float* dY) {
  model = ModelConfig();
  model.nfeatures.assign(nf, nf + L + 1);
  model.batch_per_replica = B;
  model.nreplicas = R;
  model.seed = seed;
  allocate_matrices();
  init_matrices();
  const int rows = B * R;
  for (int i = 0; i < rows; ++i) {
    std::copy_n(activations[0]->rawData(i, 0), nf[0], X + (size_t)i * nf[0]);
    std::copy_n(upstream_grad->rawData(i, 0), nf[L], dY + (size_t)i * nf[L]);
  }
  size_t off = 0;
  for (int l = 0; l < L; ++l)
    for (int i = 0; i < nf[l + 1]; ++i, off += nf[l]) std::copy_n(weights[l]->rawData(i, 0), nf[l], W + off);
}

}  // extern "C"
