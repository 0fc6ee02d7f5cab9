#include "mlp_bench_common.h"

#include <algorithm>
#include <cmath>
#include <cstdio>

using namespace std;

ModelConfig model;
int nlayers = 0;
int nthreads = 1, nthreads_per_socket = 1;
int NWARMUP = 3, NITER = 10;

vector<array<double, NUM_BREAKDOWNS>> sum_times, sum_flops;
double wall_clock_time = 0;

vector<unique_ptr<Matrix<float, PAD>>> weights, biases, activations;
unique_ptr<Matrix<float, PAD>> upstream_grad;

vector<array<int, 8>> rings = {{0, 1, 2, 4, 7, 6, 5, 3}, {0, 3, 5, 6, 7, 4, 2, 1}};

bool named_config(const string& name, int nreplicas, ModelConfig* out) {
  struct Preset {
    const char* name;
    int layers, width, batch, replicas;
    bool bf16;
  };
  static const Preset presets[] = {
      {"C1", 3, 512, 256, 2, false},   {"C2", 8, 1024, 1024, 4, false}, {"C3", 4, 4096, 2048, 2, false},
      {"C4", 20, 2048, 256, 8, false}, {"C5", 8, 8192, 4096, 4, true},
  };
  ModelConfig m;
  m.name = name;
  if (name == "ref") {
    m.nfeatures = {1024, 1024, 1024, 1024, 1024, 1024, 1024, 1};
    m.batch_per_replica = 1024;
    m.nreplicas = nreplicas > 0 ? nreplicas : 1;
    m.nwarmup = 16;
    m.niter = 256;
    *out = m;
    return true;
  }
  for (const Preset& p : presets) {
    if (name != p.name) continue;
    m.nfeatures.assign(p.layers + 1, p.width);
    m.batch_per_replica = p.batch;
    m.nreplicas = nreplicas > 0 ? nreplicas : p.replicas;
    m.bf16 = p.bf16;
    *out = m;
    return true;
  }
  return false;
}

void allocate_matrices() {
  nlayers = (int)model.nfeatures.size() - 1;
  NWARMUP = model.nwarmup;
  NITER = model.niter;
  nsockets = model.nreplicas;
  const int batch = model.batch_per_replica * model.nreplicas;
  weights.clear();
  biases.clear();
  activations.clear();
  for (int l = 0; l <= nlayers; ++l)
    activations.emplace_back(new Matrix<float, PAD>(batch, model.nfeatures[l], "act" + to_string(l)));
  for (int l = 0; l < nlayers; ++l) {
    weights.emplace_back(new Matrix<float, PAD>(model.nfeatures[l + 1], model.nfeatures[l], "w" + to_string(l)));
    biases.emplace_back(new Matrix<float, PAD>(1, model.nfeatures[l + 1], "b" + to_string(l)));
  }
  upstream_grad.reset(new Matrix<float, PAD>(batch, model.nfeatures[nlayers], "dY"));
  sum_times.assign(nlayers, {});
  sum_flops.assign(nlayers, {});
}

void init_matrices() {
  randSeed(model.seed);
  randStream(0);
  activations[0]->randFill(-1.f, 1.f);
  for (int l = 0; l < nlayers; ++l) {
    const float a = (float)sqrt(6.0 / (model.nfeatures[l] + model.nfeatures[l + 1]));
    randStream(1 + l);
    weights[l]->randFill(-a, a);
    fill_n(biases[l]->rawData(0, 0), model.nfeatures[l + 1], 0.f);
  }
  randStream(1000);
  for (int i = 0; i < upstream_grad->nrows(); ++i)
    randFillNormal(upstream_grad->rawData(i, 0), (size_t)upstream_grad->ncols(), 0.f, 1.f);
}

namespace {
double rate(double work, double seconds, double unit) { return seconds > 0 ? work / seconds / unit : 0.0; }
}  // namespace

// Same per-layer / total layout as the reference's report (mlp_bench_common.cc:38-150).  The
// GEMM columns are TF/s of the whole device instead of GF/s per core, the update column is GB/s
// of the device instead of per socket, and the imbalance columns are gone (one device).  The
// reduce-scatter / all-gather columns are kept and read 0: on one GPU neither phase exists.
void report_timing() {
  array<double, NUM_BREAKDOWNS> total_t{}, total_w{};
  for (int l = 0; l < nlayers; ++l) {
    const auto& t = sum_times[l];
    const auto& w = sum_flops[l];
    printf(
        "[layer %d] fwd %g ms/iter (%g TF/s), wgt_grad %g ms/iter (%g TF/s), bwd %g ms/iter (%g TF/s), "
        "wgt_update %g ms/iter (%g GB/s), wgt_update_reduce_scatter %g ms/iter (%g GB/s), "
        "wgt_update_allgather %g ms/iter (%g GB/s)\n",
        l, t[FWD] / NITER * 1e3, rate(w[FWD], t[FWD], 1e12), t[WGT_GRAD] / NITER * 1e3,
        rate(w[WGT_GRAD], t[WGT_GRAD], 1e12), t[BWD] / NITER * 1e3, rate(w[BWD], t[BWD], 1e12),
        t[WGT_UPDATE] / NITER * 1e3, rate(w[WGT_UPDATE], t[WGT_UPDATE], 1e9),
        t[WGT_UPDATE_REDUCE_SCATTER] / NITER * 1e3,
        rate(w[WGT_UPDATE_REDUCE_SCATTER], t[WGT_UPDATE_REDUCE_SCATTER], 1e9),
        t[WGT_UPDATE_ALLGATHER] / NITER * 1e3, rate(w[WGT_UPDATE_ALLGATHER], t[WGT_UPDATE_ALLGATHER], 1e9));
    for (int i = 0; i < NUM_BREAKDOWNS; ++i) {
      total_t[i] += t[i];
      total_w[i] += w[i];
    }
  }
  printf(
      "total fwd %g ms/iter (%g TF/s), wgt_grad %g ms/iter (%g TF/s), bwd %g ms/iter (%g TF/s), "
      "wgt_update %g ms/iter (%g GB/s), wgt_update_reduce_scatter %g ms/iter (%g GB/s), "
      "wgt_update_allgather %g ms/iter (%g GB/s)\n",
      total_t[FWD] / NITER * 1e3, rate(total_w[FWD], total_t[FWD], 1e12), total_t[WGT_GRAD] / NITER * 1e3,
      rate(total_w[WGT_GRAD], total_t[WGT_GRAD], 1e12), total_t[BWD] / NITER * 1e3,
      rate(total_w[BWD], total_t[BWD], 1e12), total_t[WGT_UPDATE] / NITER * 1e3,
      rate(total_w[WGT_UPDATE], total_t[WGT_UPDATE], 1e9), total_t[WGT_UPDATE_REDUCE_SCATTER] / NITER * 1e3,
      rate(total_w[WGT_UPDATE_REDUCE_SCATTER], total_t[WGT_UPDATE_REDUCE_SCATTER], 1e9),
      total_t[WGT_UPDATE_ALLGATHER] / NITER * 1e3,
      rate(total_w[WGT_UPDATE_ALLGATHER], total_t[WGT_UPDATE_ALLGATHER], 1e9));
  printf("wall clock time %g ms/iter\n", wall_clock_time / NITER * 1e3);
}

// l1 / l2 norm and trace of every weight matrix, accumulated in double
// (the fingerprint printed by the reference, mlp_bench_common.cc:152-168).
void print_checksum() {
  for (int l = 0; l < nlayers; ++l) {
    const Matrix<float, PAD>& w = *weights[l];
    double l1 = 0, l2 = 0, trace = 0;
    for (int i = 0; i < w.nrows(); ++i) {
      for (int j = 0; j < w.ncols(); ++j) {
        const double v = w(i, j);
        l1 += fabs(v);
        l2 += v * v;
      }
      if (i < w.ncols()) trace += w(i, i);
    }
    printf("layer %d l1 %g l2 %g trace %g\n", l, l1, sqrt(l2), trace);
  }
}

void get_my_ring_info(int sid, int task, int* idx_in_ring, int* prev_sid, int* next_sid) {
  const int which = task % (int)rings.size();
  if (nsockets < 8) {
    // fewer sockets than the hypercube has corners: natural order, reversed for odd tasks
    const int up = (sid + 1) % nsockets, down = (sid + nsockets - 1) % nsockets;
    *idx_in_ring = sid;
    *prev_sid = which ? up : down;
    *next_sid = which ? down : up;
    return;
  }
  const array<int, 8>& ring = rings[which];
  const int pos = (int)(find(ring.begin(), ring.end(), sid) - ring.begin());
  *idx_in_ring = pos;
  *prev_sid = ring[(pos + nsockets - 1) % nsockets];
  *next_sid = ring[(pos + 1) % nsockets];
}
