// Shared state and reporting of the MLP benchmark driver: model description, host tensors,
// per-phase timing accumulators, seeded initialisation, the timing report and the weight
// checksum.  Mirrors the reference's mlp_bench_common.h:9-68 with two deliberate differences:
//   * the model (layer widths, batch, replicas, iteration counts) is chosen at run time, because
//     the benchmark is run on several configurations; the reference fixes it at compile time
//     (mlp_bench_common.h:26-28,38);
//   * the weights exist once.  The reference keeps nsockets stacked copies of every weight and
//     gradient matrix so that each NUMA node reads local memory (mlp_omp.cc:395-403); a GPU has
//     one HBM, and the per-replica gradients live only on the device.
#pragma once

#include <array>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "Matrix.h"
#include "Partition.h"

constexpr int PAD = 16;             // extra columns (and rows) of every host matrix
constexpr int CACHE_LINE_LEN = 16;  // floats per 64-byte line

enum Breakdown {
  FWD = 0,
  WGT_GRAD,
  BWD,
  WGT_UPDATE,
  WGT_UPDATE_REDUCE_SCATTER,
  WGT_UPDATE_ALLGATHER,
  NUM_BREAKDOWNS,
};

struct ModelConfig {
  std::string name = "custom";
  std::vector<int> nfeatures;  // nlayers + 1 widths
  int batch_per_replica = 1024;
  int nreplicas = 1;           // = nsockets of the reference
  bool bf16 = false;
  bool relu_last = false;
  float lr = 0.01f;
  std::uint64_t seed = 1;
  int nwarmup = 3, niter = 10;
};

// The five benchmark configurations ("C1".."C5") and the reference's own default model
// ("ref": 1024 x 6 -> 1, batch 1024 per socket, mlp_bench_common.h:26, mlp_omp.cc:386).
// Returns false for an unknown name.  nreplicas <= 0 keeps the configuration's own count.
bool named_config(const std::string& name, int nreplicas, ModelConfig* out);

extern ModelConfig model;
extern int nlayers;                       // model.nfeatures.size() - 1
extern int nthreads_per_socket, nthreads; // kept for the host-side partition API; 1 device "thread"
extern int NWARMUP, NITER;

// sum_times[layer][breakdown] in seconds over the timed iterations, sum_flops[layer][breakdown]
// in FLOP (bytes for the WGT_UPDATE* slots) -- the reference's arrays of the same names
// (mlp_bench_common.h:35-36) without the per-thread dimension: the device is one "thread".
extern std::vector<std::array<double, NUM_BREAKDOWNS>> sum_times, sum_flops;
extern double wall_clock_time;

// two counter-rotating rings over 8 sockets (mlp_bench_common.cc:13-14)
extern std::vector<std::array<int, 8>> rings;

extern std::vector<std::unique_ptr<Matrix<float, PAD>>> weights, biases, activations;
extern std::unique_ptr<Matrix<float, PAD>> upstream_grad;  // dY

// Allocates the host tensors for `model` (activations[0] = X, activations[nlayers] = output).
void allocate_matrices();

// Seeded inputs: X ~ U[-1,1] (stream 0), W_l ~ U[-a,a] with a = sqrt(6/(fan_in+fan_out))
// (stream 1+l), b = 0, dY ~ N(0,1) (stream 1000).
void init_matrices();

void report_timing();
void print_checksum();

// Ring neighbourhood of socket `sid` for all-reduce task `task` (even tasks use ring 0, odd
// tasks the reverse ring).
void get_my_ring_info(int sid, int task, int* idx_in_ring, int* prev_sid, int* next_sid);
