// mlp_hip: the MLP training-step benchmark on one MI355X -- the counterpart of the reference's
// mlp_omp / mlp_tbb executables (mlp_omp.cc:375-750), with the three GEMMs and the gradient
// reduce + SGD running as HIP kernels behind the C ABI of mi_mlp.h.
//
//   mlp_hip <nreplicas> [nthreads_per_socket] [options]
//
// The two positional arguments are the reference's (<nsockets> <nthreads_per_socket>,
// mlp_omp.cc:376-379); a replica takes the place of a socket and the thread count is accepted
// and ignored.  Options:
//   --config C1|C2|C3|C4|C5|ref   one of the benchmark configurations (default C2)
//   --layers L --width N --batch B   a custom square model instead
//   --lr X --seed S --warmup W --iters K --relu-last
//   --overlap     per-layer reduce+SGD on a second stream, overlapping the next layer's GEMMs
//   --no-graph    launch kernels one by one instead of replaying a captured HIP graph
//   --keep-weights  let the weights evolve from step to step (default: every timed step starts
//                 from the initial weights, so the values stay finite however many steps run)
//   --loss l2     derive dY from seeded labels with SquaredL2Distance + AveragedLoss
//                 (mlp_caffe2.py:221-239) instead of uploading a given dY; prints the loss
//   --trace FILE  after the timed loop run one more step with an event pair around every launch
//                 and write the timeline in the format of the reference's trace.log
//                 (mlp_tbb.cc:1379-1392)
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "mi_mlp.h"
#include "mlp_bench_common.h"

using namespace std;

namespace {

[[noreturn]] void die(const char* what) {
  fprintf(stderr, "%s: %s\n", what, mi_last_error());
  exit(-1);
}
#define MI_CHECK(call) \
  do {                 \
    if ((call) != MI_OK) die(#call); \
  } while (0)

double now() {
  return chrono::duration<double>(chrono::steady_clock::now().time_since_epoch()).count();
}

// Known-answer test of the device reduce + SGD, the start-up check of the reference
// (check_all_reduce_correctness, mlp_omp.cc:325-373): gradient of replica r is r + i + j, weight
// is i * j, lr = 1; every value is an integer below 2^24, so the expected result
// i*j - ((i + j) * R + R*(R-1)/2) is exact in fp32.  Runs over the padded rows of the layer-0
// shape, like the reference's all-reduce does.
void check_all_reduce_correctness(int rows, int cols, int R) {
  Matrix<float, PAD> w(rows, cols), g(rows * R, cols);
  w.newInput();
  g.newInput();
  for (int r = 0; r < R; ++r)
    for (int i = 0; i < rows; ++i)
      for (int j = 0; j < cols; ++j) {
        g(r * rows + i, j) = (float)(r + i + j);
        if (r == 0) w(i, j) = (float)i * (float)j;
      }
  const size_t n = (size_t)rows * w.ld();
  void *dw = nullptr, *dg = nullptr;
  MI_CHECK(mi_malloc(&dw, n * sizeof(float)));
  MI_CHECK(mi_malloc(&dg, n * R * sizeof(float)));
  MI_CHECK(mi_memcpy_h2d(dw, w.rawData(), n * sizeof(float)));
  MI_CHECK(mi_memcpy_h2d(dg, g.rawData(), n * R * sizeof(float)));
  MI_CHECK(mi_reduce_sgd_raw((float*)dw, (const float*)dg, n, n, R, 1.0f, nullptr));
  MI_CHECK(mi_stream_sync(nullptr));
  MI_CHECK(mi_memcpy_d2h(w.rawData(), dw, n * sizeof(float)));
  MI_CHECK(mi_free(dw));
  MI_CHECK(mi_free(dg));
  for (int i = 0; i < rows; ++i)
    for (int j = 0; j < cols; ++j) {
      const float expected = (float)i * (float)j - (float)((i + j) * R + (R - 1) * R / 2);
      const float actual = w(i, j);
      if (fabs(actual - expected) > 1e-5) {
        printf("all-reduce check failed: i %d j %d expected %f actual %f\n", i, j, expected, actual);
        exit(-1);
      }
    }
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2 || !isdigit((unsigned char)argv[1][0])) {
    fprintf(stderr, "%s <nreplicas> [nthreads_per_socket] [--config C1..C5|ref] [--layers L --width N --batch B] "
                    "[--lr X] [--seed S] [--warmup W] [--iters K] [--relu-last] [--overlap] [--no-graph] "
                    "[--keep-weights] [--loss l2] [--trace FILE]\n", argv[0]);
    exit(1);
  }
  const int nreplicas_arg = atoi(argv[1]);
  int argi = 2;
  if (argi < argc && isdigit((unsigned char)argv[argi][0])) nthreads_per_socket = atoi(argv[argi++]);
  nthreads = nthreads_per_socket * max(nreplicas_arg, 1);

  string config = "C2";
  int layers = 0, width = 0, batch = 0, warmup = -1, iters = -1;
  float lr = 0.01f;
  uint64_t seed = 1;
  unsigned flags = 0;
  bool keep_weights = false, relu_last = false;
  string loss, trace_path;
  for (; argi < argc; ++argi) {
    const string a = argv[argi];
    auto value = [&]() -> const char* {
      if (argi + 1 >= argc) { fprintf(stderr, "%s needs a value\n", a.c_str()); exit(1); }
      return argv[++argi];
    };
    if (a == "--config") config = value();
    else if (a == "--layers") layers = atoi(value());
    else if (a == "--width") width = atoi(value());
    else if (a == "--batch") batch = atoi(value());
    else if (a == "--lr") lr = (float)atof(value());
    else if (a == "--seed") seed = strtoull(value(), nullptr, 10);
    else if (a == "--warmup") warmup = atoi(value());
    else if (a == "--iters") iters = atoi(value());
    else if (a == "--relu-last") relu_last = true;
    else if (a == "--overlap") flags |= MI_FLAG_PER_LAYER_UPDATE;
    else if (a == "--no-graph") flags |= MI_FLAG_NO_GRAPH;
    else if (a == "--keep-weights") keep_weights = true;
    else if (a == "--loss") loss = value();
    else if (a == "--trace") trace_path = value();
    else { fprintf(stderr, "unknown option %s\n", a.c_str()); exit(1); }
  }

  if (layers > 0 || width > 0 || batch > 0) {
    if (layers <= 0 || width <= 0 || batch <= 0) { fprintf(stderr, "--layers, --width and --batch go together\n"); exit(1); }
    model = ModelConfig();
    model.nfeatures.assign(layers + 1, width);
    model.batch_per_replica = batch;
    model.nreplicas = max(nreplicas_arg, 1);
  } else if (!named_config(config, nreplicas_arg, &model)) {
    fprintf(stderr, "unknown config %s\n", config.c_str());
    exit(1);
  }
  model.lr = lr;
  model.seed = seed;
  model.relu_last = relu_last;
  if (warmup >= 0) model.nwarmup = warmup;
  if (iters > 0) model.niter = iters;
  if (relu_last) flags |= MI_FLAG_RELU_LAST;

  char devname[256];
  int cus = 0, mhz = 0;
  size_t mem = 0;
  MI_CHECK(mi_device_info(devname, sizeof devname, &cus, &mhz, &mem));
  printf("device %s, %d CUs, %d MHz, %.1f GiB\n", devname, cus, mhz, mem / 1073741824.0);

  /////////////////////////////////////////////////////////////////////////////
  // host tensors
  allocate_matrices();
  const int R = model.nreplicas, B = model.batch_per_replica;
  printf("config %s: %d layers, widths", model.name.c_str(), nlayers);
  for (int v : model.nfeatures) printf(" %d", v);
  printf(", batch %d x %d replicas, %s, lr %g, seed %llu, %d warm-up + %d timed steps\n", B, R,
         model.bf16 ? "bf16" : "fp32", model.lr, (unsigned long long)model.seed, NWARMUP, NITER);

  /////////////////////////////////////////////////////////////////////////////
  // check correctness of the device reduce
  check_all_reduce_correctness(model.nfeatures[1], model.nfeatures[0], R);

  /////////////////////////////////////////////////////////////////////////////
  // initialise values and move the model to the device
  init_matrices();
  mi_mlp* h = nullptr;
  MI_CHECK(mi_mlp_create(&h, nlayers, model.nfeatures.data(), B, R, model.bf16 ? MI_BF16 : MI_F32, flags));
  for (int l = 0; l < nlayers; ++l)
    MI_CHECK(mi_mlp_set_weights(h, l, weights[l]->rawData(), weights[l]->ld(), biases[l]->rawData()));
  MI_CHECK(mi_mlp_set_input(h, activations[0]->rawData(), activations[0]->ld()));
  if (loss == "l2") {
    // labels ~ U[-1, 1] on a stream of their own; the given dY is not used
    Matrix<float, PAD> labels(R * B, model.nfeatures[nlayers]);
    randStream(2000);
    labels.randFill(-1.f, 1.f);
    MI_CHECK(mi_mlp_set_labels(h, labels.rawData(), labels.ld()));
  } else if (loss.empty()) {
    MI_CHECK(mi_mlp_set_dy(h, upstream_grad->rawData(), upstream_grad->ld()));
  } else {
    fprintf(stderr, "unknown loss %s (known: l2)\n", loss.c_str());
    exit(1);
  }
  MI_CHECK(mi_mlp_snapshot_weights(h));

  size_t params = 0, stride = 0;
  MI_CHECK(mi_mlp_param_count(h, &params, &stride));

  /////////////////////////////////////////////////////////////////////////////
  // main computation: first the wall clock of the plain step loop, then the same loop once more
  // with per-kernel event timing for the breakdown
  for (int it = 0; it < NWARMUP + NITER; ++it) {
    if (it == NWARMUP) {
      MI_CHECK(mi_mlp_sync(h));
      wall_clock_time = now();
    }
    if (!keep_weights) MI_CHECK(mi_mlp_restore_weights(h));
    MI_CHECK(mi_mlp_step(h, model.lr));
  }
  MI_CHECK(mi_mlp_sync(h));
  wall_clock_time = now() - wall_clock_time;

  MI_CHECK(mi_mlp_enable_timing(h, 1));
  for (int it = 0; it < NITER; ++it) {
    if (!keep_weights) MI_CHECK(mi_mlp_restore_weights(h));
    MI_CHECK(mi_mlp_step(h, model.lr));
  }
  vector<double> ms((size_t)MI_NUM_BREAKDOWNS * nlayers);
  MI_CHECK(mi_mlp_get_timings(h, ms.data(), nullptr));
  const double rows = (double)R * B;
  for (int l = 0; l < nlayers; ++l) {
    const double gemm_flops = 2.0 * rows * model.nfeatures[l] * model.nfeatures[l + 1] * NITER;
    for (int b = 0; b < NUM_BREAKDOWNS; ++b) sum_times[l][b] = ms[(size_t)b * nlayers + l] * 1e-3;
    sum_flops[l][FWD] = sum_flops[l][WGT_GRAD] = sum_flops[l][BWD] = gemm_flops;
    // bytes the update has to move: R gradient copies in, W in, W out
    const double layer_params = (double)model.nfeatures[l] * model.nfeatures[l + 1] + model.nfeatures[l + 1];
    const double bytes = (R + 2) * 4.0 * layer_params * NITER;
    // the per-kernel timing pass always runs the update as one launch over all layers (overlapping
    // launches cannot be timed one by one), whatever schedule the timed loop used: layer 0 carries it
    sum_flops[0][WGT_UPDATE] += bytes;
  }

  /////////////////////////////////////////////////////////////////////////////
  // report timing
  report_timing();
  double gemm_flop_step = 0;
  for (int l = 0; l < nlayers; ++l) gemm_flop_step += 3 * 2.0 * rows * model.nfeatures[l] * model.nfeatures[l + 1];
  const double step_ms = wall_clock_time / NITER * 1e3;
  printf("step %g ms, %g TFLOP/s over the whole step (GEMM FLOP model 3*2*batch*sum N_l*N_l+1 = %g GFLOP), "
         "update moves %g MB per step\n", step_ms, gemm_flop_step / step_ms / 1e9, gemm_flop_step / 1e9,
         (R + 2) * 4.0 * params / 1e6);

  if (!loss.empty()) {
    vector<double> per(R);
    double total = 0;
    MI_CHECK(mi_mlp_get_loss(h, per.data(), &total));
    printf("loss %.9g (per replica:", total);
    for (double v : per) printf(" %.9g", v);
    printf(")\n");
  }
  if (!trace_path.empty()) {
    MI_CHECK(mi_mlp_enable_timing(h, 0));
    if (!keep_weights) MI_CHECK(mi_mlp_restore_weights(h));
    MI_CHECK(mi_mlp_trace_step(h, model.lr, trace_path.c_str()));
    printf("timeline of one step written to %s\n", trace_path.c_str());
  }

  /////////////////////////////////////////////////////////////////////////////
  // print check sum for correctness check
  for (int l = 0; l < nlayers; ++l) MI_CHECK(mi_mlp_get_weight(h, l, weights[l]->rawData(), weights[l]->ld()));
  print_checksum();

  MI_CHECK(mi_mlp_destroy(h));
  return 0;
}
