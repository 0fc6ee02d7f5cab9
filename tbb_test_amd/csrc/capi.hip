// Implementation of the C ABI declared in include/mi_mlp.h: argument checking, device state of
// one model (parameter arena, R gradient arenas, activations), the step schedule, event timing
// and HIP-graph replay.  The arithmetic lives in gemm_f32.hip, gemm_bf16.hip and reduce_sgd.hip.
#include <hip/hip_runtime.h>
#include <cstdlib>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "kernels.h"
#include "mi_mlp.h"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(MI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define MI_HIP(call)                                  \
  do {                                                \
    hipError_t e_ = (call);                           \
    if (e_ != hipSuccess) return hip_fail(e_, #call); \
  } while (0)

#define MI_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return fail(MI_ERR_INVALID, __VA_ARGS__); \
  } while (0)

// Tuning hooks, process-wide: forced tile configuration per fp32 GEMM kind (nt, nn, tn) and of the
// bf16 kernel; 0 = automatic.  A change bumps the epoch, and a handle whose captured graph is older
// re-captures before its next replay.
std::atomic<int> g_variant[3] = {{0}, {0}, {0}};
std::atomic<int> g_hvariant{0};
std::atomic<int> g_variant_epoch{0};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace

// ------------------------------------------------------------------------------------------------
// model state

struct mi_mlp {
  int L = 0, B = 0, R = 0, dtype = MI_F32;
  unsigned flags = 0;
  int MB = 0;  // rows of every activation = R * B
  std::vector<int> nf;
  size_t P = 0;        // parameter count, padding excluded
  size_t stride = 0;   // floats per arena (segments padded to 256 bytes)
  std::vector<size_t> woff, boff;  // float offsets of W_l / b_l inside an arena
  float* params = nullptr;    // [stride]
  float* grads = nullptr;     // [R * stride]
  uint16_t* params16 = nullptr;  // bf16 copy of params (dtype bf16)
  uint16_t* params16T = nullptr; // bf16 W_l^T [N_l x N_{l+1}] at the same arena offsets (dtype bf16)
  float* params_saved = nullptr;    // snapshot of params (mi_mlp_snapshot_weights)
  uint16_t* params16_saved = nullptr;
  uint16_t* params16T_saved = nullptr;
  std::vector<uint16_t*> actsT;  // bf16 only: per-replica transposed activations [R][N_l x B], l < L
  // Gradient buffers: dZ_l lives in dz[l % ndz]; ndz = 3 (a rotation: dZ_l is dead once wgrad(l) and
  // dgrad(l) have read it) or, with MI_FLAG_KEEP_GRADIENTS, one buffer per layer.
  int ndz = 3;
  // bf16 only: per-replica transposed gradients [R][max N x B]; dZ_l^T lives in dzT[l % ndz] like
  // dZ_l in dz[l % ndz].  *_fused: the producing GEMM wrote the transposed copy in its epilogue.
  std::vector<uint16_t*> dzT;
  std::vector<char> actsT_fused;  // [L]
  std::vector<char> dzT_fused;  // [ndz]: state of the slot, what op_wgrad decides on
  std::vector<char> dzT_fused_layer;  // [L]: whether dZ_l^T last came out of a GEMM epilogue (mi_mlp_get_schedule)
  // bf16 only: the per-replica transposed copy of the uploaded dY, made once by mi_mlp_set_dy (the
  // weight gradient of the last layer reads it every step; the rotation buffers get overwritten)
  uint16_t* dyT = nullptr;
  bool dyT_valid = false;
  // bf16 only: column sums of dZ_l per block of 128 rows, written by the epilogue of the GEMM that
  // produced dZ_l (slot l % ndz, [MB / 128][max N] floats); folded into the bias gradient by op_wgrad
  std::vector<float*> colpart;
  std::vector<char> colpart_valid;
  std::vector<void*> acts;    // L+1 buffers [MB x nf[l]], fp32 or bf16
  void* dy = nullptr;         // upstream gradient [MB x nf[L]]
  std::vector<void*> dz;      // [ndz] buffers of [MB x max width]
  void* dx = nullptr;         // gradient w.r.t. the input [MB x nf[0]]
  float* staging = nullptr;   // fp32 bounce buffer for bf16 uploads/downloads [MB x max width] or one W
  size_t staging_elems = 0;
  hipStream_t stream = nullptr, stream2 = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  std::vector<hipEvent_t> ev_layer;  // per layer: input-gradient GEMM of layer l done (dZ_{l-1} ready, W_l free)
  std::vector<hipEvent_t> ev_wgrad;  // per layer: weight-gradient GEMM of layer l done (dZ_l free)


  // loss front-end: when labels are set, every step derives dY from the forward output
  float* labels = nullptr;         // [MB x nf[L]] fp32
  double* loss_partials = nullptr; // [R x LOSS_CHUNKS] partial sums of 0.5 * (pred - label)^2 of the last step
  bool use_loss = false;

  // timeline of one step (mi_mlp_trace_step)
  bool tracing = false;
  struct TraceItem { hipEvent_t a, b; int breakdown, layer, stream_id; };
  std::vector<TraceItem> trace_items;

  // timing
  bool timing = false;
  struct Pair { hipEvent_t a, b; int slot; };
  std::vector<Pair> pending;
  std::vector<hipEvent_t> free_events;
  std::vector<double> ms;
  std::vector<long long> launches;

  // graph replay
  hipGraphExec_t graph_exec = nullptr;
  int graph_epoch = 0;  // g_variant_epoch at capture time
  int eager_steps = 0;
  // g_variant_epoch of the last untimed eager step (-1: none yet).  A capture follows only such a
  // step: it has launched every kernel of the schedule once, so that the one-time kernel attribute
  // calls (more than 64 KB of dynamic LDS) are behind us when the capture begins.
  int warm_epoch = -1;
  // -lr on the device: the update kernels of a step read it from here, so that a captured graph
  // follows a learning-rate schedule without being captured again
  float* neg_lr_dev = nullptr;
  float neg_lr_value = 0.0f;
  bool neg_lr_valid = false;
  // what the last enqueue_step decided (mi_mlp_get_schedule)
  bool last_dual = false, last_per_layer = false, last_paired = false;

  size_t esize() const { return dtype == MI_BF16 ? 2 : 4; }
  size_t maxw() const {
    size_t m = 0;
    for (int v : nf) m = v > (int)m ? (size_t)v : m;
    return m;
  }
};

namespace {

int check_handle(mi_mlp* h) {
  if (!h) return fail(MI_ERR_INVALID, "null handle");
  return MI_OK;
}
int check_layer(mi_mlp* h, int l, int hi_inclusive) {
  if (!h) return fail(MI_ERR_INVALID, "null handle");
  if (l < 0 || l > hi_inclusive) return fail(MI_ERR_INVALID, "layer index %d out of range [0,%d]", l, hi_inclusive);
  return MI_OK;
}

// event timing ------------------------------------------------------------------------------------
int harvest(mi_mlp* h) {
  if (h->pending.empty()) return MI_OK;
  MI_HIP(hipStreamSynchronize(h->stream));
  if (h->stream2) MI_HIP(hipStreamSynchronize(h->stream2));
  for (auto& p : h->pending) {
    float t = 0.0f;
    MI_HIP(hipEventElapsedTime(&t, p.a, p.b));
    h->ms[p.slot] += (double)t;
    h->launches[p.slot] += 1;
    h->free_events.push_back(p.a);
    h->free_events.push_back(p.b);
  }
  h->pending.clear();
  return MI_OK;
}

int get_event(mi_mlp* h, hipEvent_t* ev) {
  if (h->free_events.empty()) {
    MI_HIP(hipEventCreate(ev));
  } else {
    *ev = h->free_events.back();
    h->free_events.pop_back();
  }
  return MI_OK;
}

constexpr int TRACE_LOSS = 100;   // pseudo-breakdown of the loss kernel in a timeline
constexpr int TRACE_PAIR = 101;   // weight gradient + input gradient of a layer in one launch
constexpr int LOSS_CHUNKS = 64;   // partial sums per replica

struct TimedScope {
  mi_mlp* h;
  hipStream_t s;
  mi::LaunchEvents ev{nullptr, nullptr, 0};
  int breakdown, layer;
  int status = MI_OK;
  bool on;
  TimedScope(mi_mlp* h_, hipStream_t s_, int breakdown_, int layer_)
      : h(h_), s(s_), breakdown(breakdown_), layer(layer_), on(h_->tracing || (h_->timing && breakdown_ < MI_NUM_BREAKDOWNS)) {
    if (!on) return;
    if (h->pending.size() >= 8192) status = harvest(h);
    if (status == MI_OK) status = get_event(h, &ev.start);
    if (status == MI_OK) status = get_event(h, &ev.stop);
    if (status == MI_OK) mi::launch_events = &ev;  // the kernels of this scope carry the events
  }
  ~TimedScope() {
    if (mi::launch_events == &ev) mi::launch_events = nullptr;
  }
  int finish() {
    if (!on || status != MI_OK) return status;
    mi::launch_events = nullptr;
    if (ev.launches == 0) {  // nothing was launched (empty operand): nothing to time
      h->free_events.push_back(ev.start);
      h->free_events.push_back(ev.stop);
      return MI_OK;
    }
    if (h->tracing) h->trace_items.push_back({ev.start, ev.stop, breakdown, layer, s == h->stream ? 0 : 1});
    else h->pending.push_back({ev.start, ev.stop, breakdown * h->L + (layer < 0 ? 0 : layer)});
    return MI_OK;
  }
};

// operations on the handle ----------------------------------------------------------------------
const void* dz_of_layer(mi_mlp* h, int l) {
  // gradient w.r.t. the pre-activation output of layer l
  if (l == h->L - 1 && !(h->flags & MI_FLAG_RELU_LAST)) return h->dy;
  return h->dz[l % h->ndz];
}

int op_forward(mi_mlp* h, int l, hipStream_t s) {
  const int relu = (l < h->L - 1) || (h->flags & MI_FLAG_RELU_LAST);
  TimedScope ts(h, s, MI_FWD, l);
  if (ts.status) return ts.status;
  hipError_t e;
  if (h->dtype == MI_F32) {
    e = mi::sgemm_nt(h->MB, h->nf[l + 1], h->nf[l], (const float*)h->acts[l], h->nf[l], h->params + h->woff[l],
                     h->nf[l], (float*)h->acts[l + 1], h->nf[l + 1], h->params + h->boff[l], relu, s, g_variant[0]);
  } else {
    // the activation a later weight-gradient GEMM reads K-contiguous is also written transposed
    bool wrote = false;
    uint16_t* ct = (l + 1 < h->L) ? h->actsT[l + 1] : nullptr;
    e = mi::hgemm_nt(1, h->MB, h->nf[l + 1], h->nf[l], (const uint16_t*)h->acts[l], h->nf[l], 0,
                     h->params16 + h->woff[l], h->nf[l], 0, h->acts[l + 1], h->nf[l + 1], 0, 1, h->params + h->boff[l],
                     relu, nullptr, 0, s, g_hvariant, ct, h->B, &wrote);
    if (l + 1 < h->L) h->actsT_fused[l + 1] = wrote;
  }
  if (e != hipSuccess) return hip_fail(e, "forward GEMM launch");
  return ts.finish();
}

int op_wgrad(mi_mlp* h, int l, hipStream_t s, bool with_bias) {
  const float* g0 = h->grads + h->woff[l];
  TimedScope ts(h, s, MI_WGT_GRAD, l);
  if (ts.status) return ts.status;
  hipError_t e;
  if (h->dtype == MI_F32) {
    e = mi::sgemm_tn(h->R, h->nf[l + 1], h->nf[l], h->B, (const float*)dz_of_layer(h, l), h->nf[l + 1],
                     (const float*)h->acts[l], h->nf[l], const_cast<float*>(g0), h->nf[l], (long long)h->stride,
                     with_bias ? h->grads + h->boff[l] : nullptr, (long long)h->stride, s,
                     g_variant[2]);
  } else {
    // K-contiguous copies of both operands, per replica: A_l^T [N_l x B] and dZ_l^T [N_{l+1} x B]
    const int B = h->B, nin = h->nf[l], nout = h->nf[l + 1];
    // (each copy comes from the epilogue of the GEMM that produced the operand when that was
    // possible, else from a transpose here)
    uint16_t* dzt = h->dzT[l % h->ndz];
    e = hipSuccess;
    // the uploaded dY is the last layer's dZ as it stands (no ReLU after the last layer, no loss front-end)
    const bool dy_cached = l == h->L - 1 && h->dyT_valid && !h->use_loss && !(h->flags & MI_FLAG_RELU_LAST);
    if (dy_cached) dzt = h->dyT;
    if (!h->actsT_fused[l])
      e = mi::transpose_bf16(h->R, B, nin, (const uint16_t*)h->acts[l], nin, (long long)B * nin, h->actsT[l], B,
                             (long long)nin * B, s);
    const bool dz_fused = l < h->L - 1 && h->dzT_fused[l % h->ndz];  // the last layer's dZ is the given or derived dY
    if (e == hipSuccess && !dz_fused && !dy_cached)
      e = mi::transpose_bf16(h->R, B, nout, (const uint16_t*)dz_of_layer(h, l), nout, (long long)B * nout, dzt, B,
                             (long long)nout * B, s);
    if (e == hipSuccess)
      e = mi::hgemm_nt(h->R, nout, nin, B, dzt, B, (long long)nout * B, h->actsT[l], B, (long long)nin * B,
                       const_cast<float*>(g0), nin, (long long)h->stride, 0, nullptr, 0, nullptr, 0, s, g_hvariant);
    if (e == hipSuccess && with_bias) {
      // bias gradient: from the column sums the producing GEMM left behind, else a pass over dZ^T
      if (l < h->L - 1 && h->colpart_valid[l % h->ndz] && B % 128 == 0)
        e = mi::colsum_fold(h->R, nout, B / 128, h->colpart[l % h->ndz], h->grads + h->boff[l], (long long)h->stride, s);
      else
        e = mi::rowsum_bf16(h->R, nout, B, dzt, B, (long long)nout * B, h->grads + h->boff[l], (long long)h->stride, s);
    }
  }
  if (e != hipSuccess) return hip_fail(e, "weight-gradient GEMM launch");
  return ts.finish();
}

int op_bgrad(mi_mlp* h, int l, hipStream_t s) {
  if (h->dtype != MI_F32) {
    const int B = h->B, nout = h->nf[l + 1];
    hipError_t eb = mi::transpose_bf16(h->R, B, nout, (const uint16_t*)dz_of_layer(h, l), nout, (long long)B * nout,
                                       h->dzT[l % h->ndz], B, (long long)nout * B, s);
    if (eb == hipSuccess)
      eb = mi::rowsum_bf16(h->R, nout, B, h->dzT[l % h->ndz], B, (long long)nout * B, h->grads + h->boff[l],
                           (long long)h->stride, s);
    if (eb != hipSuccess) return hip_fail(eb, "bias-gradient launch");
    return MI_OK;
  }
  hipError_t e = mi::colsum_f32(h->R, h->nf[l + 1], h->B, (const float*)dz_of_layer(h, l), h->nf[l + 1],
                                h->grads + h->boff[l], (long long)h->stride, s);
  if (e != hipSuccess) return hip_fail(e, "bias-gradient launch");
  return MI_OK;
}

int op_dgrad(mi_mlp* h, int l, hipStream_t s) {
  TimedScope ts(h, s, MI_BWD, l);
  if (ts.status) return ts.status;
  void* out = (l == 0) ? h->dx : h->dz[(l - 1) % h->ndz];
  const void* mask = (l == 0) ? nullptr : h->acts[l];
  hipError_t e;
  if (h->dtype == MI_F32) {
    e = mi::sgemm_nn(h->MB, h->nf[l], h->nf[l + 1], (const float*)dz_of_layer(h, l), h->nf[l + 1],
                     h->params + h->woff[l], h->nf[l], (float*)out, h->nf[l], (const float*)mask, h->nf[l], s,
                     g_variant[1]);
  } else {
    bool wrote = false, wrote_cs = false;
    uint16_t* ct = (l > 0) ? h->dzT[(l - 1) % h->ndz] : nullptr;  // dZ_{l-1}^T for the weight gradient of layer l-1
    float* cp = (l > 0 && h->B % 128 == 0) ? h->colpart[(l - 1) % h->ndz] : nullptr;  // and its column sums
    e = mi::hgemm_nt(1, h->MB, h->nf[l], h->nf[l + 1], (const uint16_t*)dz_of_layer(h, l), h->nf[l + 1], 0,
                     h->params16T + h->woff[l], h->nf[l + 1], 0, out, h->nf[l], 0, mask ? 2 : 3, nullptr, 0,
                     (const uint16_t*)mask, h->nf[l], s, g_hvariant, ct, h->B, &wrote, cp, &wrote_cs);
    if (l > 0) {
      h->dzT_fused[(l - 1) % h->ndz] = wrote;
      h->dzT_fused_layer[l - 1] = wrote;
      h->colpart_valid[(l - 1) % h->ndz] = wrote_cs;
    }
  }
  if (e != hipSuccess) return hip_fail(e, "input-gradient GEMM launch");
  return ts.finish();
}

// Weight gradient and input gradient of layer l in one launch (small fp32 layers only, see
// small_model()).  Booked as one weight-gradient scope in a timeline.
int op_backward_pair(mi_mlp* h, int l, hipStream_t s) {
  TimedScope ts(h, s, TRACE_PAIR, l);
  if (ts.status) return ts.status;
  float* out = (float*)((l == 0) ? h->dx : h->dz[(l - 1) % h->ndz]);
  const float* mask = (l == 0) ? nullptr : (const float*)h->acts[l];
  hipError_t e = mi::sgemm_backward_pair(h->R, h->MB, h->nf[l + 1], h->nf[l], (const float*)dz_of_layer(h, l),
                                         (const float*)h->acts[l], h->params + h->woff[l], h->grads + h->woff[l],
                                         (long long)h->stride, h->grads + h->boff[l], (long long)h->stride, out, mask, s);
  if (e != hipSuccess) return hip_fail(e, "backward pair launch");
  return ts.finish();
}

// A model all of whose backward GEMMs are small enough for the paired launch: its step is a chain
// of launches of a few microseconds each, so the schedule that counts is the one with the fewest
// launches -- one stream, weight and input gradient of a layer in one launch, one update launch.
bool small_model(const mi_mlp* h) {
  if (h->dtype != MI_F32) return false;
  for (int k = 0; k < 3; ++k)
    if (g_variant[k].load() != 0) return false;  // a forced tile configuration is honoured by the separate launches
  for (int l = 0; l < h->L; ++l)
    if (!mi::sgemm_backward_pair_fits(h->R, h->MB, h->nf[l + 1], h->nf[l])) return false;
  return true;
}

// beside_gemm: the launch shares the GPU with a GEMM of the same step on the other stream
int op_update(mi_mlp* h, int l_or_all, float lr, hipStream_t s, bool beside_gemm = false) {
  TimedScope ts(h, s, MI_WGT_UPDATE, l_or_all >= 0 ? l_or_all : -1);
  if (ts.status) return ts.status;
  hipError_t e = hipSuccess;
  if (!h->params16T) {
    // fp32 model: one flat launch over the layer's segment (W_l | b_l) or over the whole arena
    size_t off = 0, n = h->stride;
    if (l_or_all >= 0) {
      off = h->woff[l_or_all];
      n = (l_or_all + 1 < h->L ? h->woff[l_or_all + 1] : h->stride) - off;
    }
    e = mi::reduce_sgd(h->params + off, nullptr, h->grads + off, n, h->stride, h->R, lr, s, h->neg_lr_dev);
    if (e != hipSuccess) return hip_fail(e, "reduce+SGD launch");
    return ts.finish();
  }
  // bf16 model, per layer: W_l with both bf16 copies (W for the forward GEMM, W^T for the
  // input-gradient GEMM) written in the same pass, the bias segment by extra workgroups of the same launch.
  // Shapes the tiled kernel cannot take use the flat kernel and a transpose launch.
  const int first = l_or_all >= 0 ? l_or_all : 0, last = l_or_all >= 0 ? l_or_all : h->L - 1;
  for (int l = first; l <= last && e == hipSuccess; ++l) {
    const size_t wo = h->woff[l], bo = h->boff[l];
    const size_t seg_end = l + 1 < h->L ? h->woff[l + 1] : h->stride;
    const int rows = h->nf[l + 1], cols = h->nf[l];
    if (mi::reduce_sgd_tiled_fits(h->params + wo, h->params16 + wo, h->params16T + wo, h->grads + wo, rows, cols,
                                  h->stride, seg_end - bo, h->R)) {
      // the arena pads W_l to 64 floats, and rows * cols is a multiple of 64 here: b_l follows W_l directly
      e = mi::reduce_sgd_tiled(h->params + wo, h->params16 + wo, h->params16T + wo, h->grads + wo, rows, cols,
                               h->stride, seg_end - bo, h->R, lr, s, h->neg_lr_dev, beside_gemm);
    } else {
      e = mi::reduce_sgd(h->params + wo, h->params16 + wo, h->grads + wo, seg_end - wo, h->stride, h->R, lr, s,
                         h->neg_lr_dev);
      if (e == hipSuccess)
        e = mi::transpose_bf16(1, rows, cols, h->params16 + wo, cols, 0, h->params16T + wo, rows, 0, s);
    }
  }
  if (e != hipSuccess) return hip_fail(e, "reduce+SGD launch");
  return ts.finish();
}

// dZ of the last layer when it carries a ReLU: dY masked by the sign of the output
__global__ __launch_bounds__(256) void mask_copy_kernel(float* __restrict__ dst, const float* __restrict__ g,
                                                        const float* __restrict__ act, size_t n) {
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    dst[i] = act[i] > 0.0f ? g[i] : 0.0f;
}
// the same on bf16 words, compared after widening to fp32 (so zeros, negatives and NaN drop the
// gradient exactly as in the fp32 kernel)
__global__ __launch_bounds__(256) void mask_copy_bf16_kernel(uint16_t* __restrict__ dst, const uint16_t* __restrict__ g,
                                                             const uint16_t* __restrict__ act, size_t n) {
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) {
    const float a = __uint_as_float((unsigned)act[i] << 16);
    dst[i] = a > 0.0f ? g[i] : (uint16_t)0;
  }
}

int op_last_mask(mi_mlp* h, hipStream_t s) {
  if (!(h->flags & MI_FLAG_RELU_LAST)) return MI_OK;
  const size_t n = (size_t)h->MB * h->nf[h->L];
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (h->dtype == MI_F32)
    mi::launch_kernel(mask_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (float*)h->dz[(h->L - 1) % h->ndz],
                      (const float*)h->dy, (const float*)h->acts[h->L], n);
  else
    mi::launch_kernel(mask_copy_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                      (uint16_t*)h->dz[(h->L - 1) % h->ndz], (const uint16_t*)h->dy, (const uint16_t*)h->acts[h->L], n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "mask launch");
  return MI_OK;
}

// Loss front-end (SquaredL2Distance + AveragedLoss of the Caffe2 harness, mlp_caffe2.py:221-239):
// dY = (pred - label) / B, and per replica the partial sums of 0.5 * (pred - label)^2.  Block
// (c, r) owns a contiguous slice of replica r's elements; threads accumulate in double in a fixed
// order and the block folds through LDS, so the result does not depend on scheduling.
template <bool BF16>
__global__ __launch_bounds__(256) void l2_loss_kernel(void* __restrict__ dy, const void* __restrict__ pred,
                                                      const float* __restrict__ label, size_t per_replica,
                                                      float inv_b, double* __restrict__ partials) {
  __shared__ double red[256];
  const size_t chunk = (per_replica + gridDim.x - 1) / gridDim.x;
  const size_t lo = (size_t)blockIdx.y * per_replica + (size_t)blockIdx.x * chunk;
  size_t hi = lo + chunk;
  const size_t end = (size_t)(blockIdx.y + 1) * per_replica;
  if (hi > end) hi = end;
  double acc = 0.0;
  for (size_t i = lo + threadIdx.x; i < hi; i += 256) {
    float p;
    if (BF16) p = __uint_as_float((unsigned)reinterpret_cast<const uint16_t*>(pred)[i] << 16);
    else p = reinterpret_cast<const float*>(pred)[i];
    const float d = p - label[i];
    acc += 0.5 * (double)d * (double)d;
    const float g = d * inv_b;
    if (BF16) {
      unsigned u = __float_as_uint(g);
      if ((u & 0x7fffffffu) > 0x7f800000u) u = (u >> 16) | 0x40u;
      else u = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
      reinterpret_cast<uint16_t*>(dy)[i] = (uint16_t)u;
    } else {
      reinterpret_cast<float*>(dy)[i] = g;
    }
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) partials[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = red[0];
}

int op_loss(mi_mlp* h, hipStream_t s) {
  if (!h->labels) return fail(MI_ERR_INVALID, "no labels set (mi_mlp_set_labels)");
  TimedScope ts(h, s, TRACE_LOSS, 0);
  if (ts.status) return ts.status;
  const size_t per_replica = (size_t)h->B * h->nf[h->L];
  const float inv_b = 1.0f / (float)h->B;
  if (h->dtype == MI_F32)
    mi::launch_kernel(l2_loss_kernel<false>, dim3(LOSS_CHUNKS, h->R), dim3(256), 0, s, h->dy, h->acts[h->L], h->labels,
                       per_replica, inv_b, h->loss_partials);
  else
    mi::launch_kernel(l2_loss_kernel<true>, dim3(LOSS_CHUNKS, h->R), dim3(256), 0, s, h->dy, h->acts[h->L], h->labels,
                       per_replica, inv_b, h->loss_partials);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "loss launch");
  h->dyT_valid = false;  // dY was rewritten on the device: the transposed copy made at upload is stale
  return ts.finish();
}

__global__ void set_scalar_kernel(float* dst, float v) { *dst = v; }

// Makes *neg_lr_dev = -lr for the update launches that follow on the handle's streams.  Called
// outside any capture (the value is not part of the graph) and only when lr changes.  Ordered:
// it runs on the main stream, which every step joins the second stream into at its end.
int ensure_lr(mi_mlp* h, float lr) {
  if (h->neg_lr_valid && h->neg_lr_value == -lr) return MI_OK;
  hipLaunchKernelGGL(set_scalar_kernel, dim3(1), dim3(1), 0, h->stream, h->neg_lr_dev, -lr);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "learning-rate launch");
  h->neg_lr_value = -lr;
  h->neg_lr_valid = true;
  return MI_OK;
}

// ---- loss front-end on caller-owned buffers, allocating nothing --------------------------------
// The partial sums of l2_loss_kernel are the one scratch buffer of the loss path (the handle keeps
// them in loss_partials, allocated by mi_mlp_set_labels).  mi_l2_loss_static keeps them in this
// device-resident array instead, so that callers which cannot allocate can use the loss kernel.
// In host code the array's name is only a stand-in: the address of each device's copy is asked
// for once per device (static_scratch_of) and that pointer is what the kernels receive.
constexpr int LOSS_STATIC_MAX_REPLICAS = 1024;
static __device__ __align__(256) double g_loss_scratch[(size_t)LOSS_STATIC_MAX_REPLICAS * LOSS_CHUNKS];  // 512 KB per device

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
double* g_scratch_ptr[MAX_DEVICES] = {};  // per device: address of that device's g_loss_scratch

int static_scratch_of_current_device(double** out) {
  int dev = -1;
  MI_HIP(hipGetDevice(&dev));
  MI_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "device index %d beyond the %d this library tracks", dev, MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    MI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_loss_scratch)));
    MI_REQUIRE(p != nullptr, "hipGetSymbolAddress returned a null address for the loss scratch");
    g_scratch_ptr[dev] = static_cast<double*>(p);
  }
  *out = g_scratch_ptr[dev];
  return MI_OK;
}

// loss[r] = (sum of replica r's partial sums, in chunk order) / B -- the fold mi_mlp_get_loss does
// on the host, same order and same operations, so both give the same bits.
__global__ __launch_bounds__(64) void loss_fold_kernel(const double* __restrict__ partials, double* __restrict__ loss,
                                                       int R, double batch) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= R) return;
  double acc = 0.0;
  for (int c = 0; c < LOSS_CHUNKS; ++c) acc += partials[(size_t)r * LOSS_CHUNKS + c];
  loss[r] = acc / batch;
}

// Enqueues one whole step.
//
// Backward runs on two streams: the input-gradient GEMMs form the dependent chain on the main
// stream, the weight-gradient GEMMs (which nothing in the backward pass depends on) trail them on
// the second stream.  The two kinds are independent per layer, so the workgroups of one kernel move
// onto CUs as the other kernel's workgroups drain, which hides the prologue and epilogue that a
// chain of dependent one-tile-per-CU launches cannot hide.  dZ_l rotates through three buffers so
// that dgrad(l-1) may overwrite nothing wgrad(l) still reads; dgrad(l) additionally waits for
// wgrad(l+2), the last reader of the buffer it writes.  MI_FLAG_SERIAL_BACKWARD keeps everything on
// one stream.  With MI_FLAG_PER_LAYER_UPDATE the update of layer l follows wgrad(l) on the second
// stream as soon as dgrad(l), the last reader of W_l, is done; otherwise one update over all
// layers closes the step.
int enqueue_step(mi_mlp* h, float lr) {
  hipStream_t s = h->stream;
  int rc;
  for (int l = 0; l < h->L; ++l)
    if ((rc = op_forward(h, l, s))) return rc;
  if (h->use_loss)
    if ((rc = op_loss(h, s))) return rc;
  if ((rc = op_last_mask(h, s))) return rc;
  // While per-kernel event timing is on, everything runs back to back on one stream with one
  // update launch: durations of kernels that overlap cannot be attributed to a kernel.
  // (per-kernel timing keeps the separate launches so that every phase has its own figures)
  const bool paired = small_model(h) && !h->timing;
  const bool per_layer = (h->flags & MI_FLAG_PER_LAYER_UPDATE) != 0 && !h->timing && !paired;
  // Two backward streams pay while a GEMM launch leaves CUs idle at its start and end, i.e. up to
  // a few tiles per CU (configs 2 and 4: 256 tiles of 128 x 128 per input-gradient launch, 3-5 %
  // faster with two streams).  GEMMs with many tiles per CU only get in each other's way (config
  // 3, 1024 tiles: 11.32 ms with one backward stream, 11.47 ms with two; config 5: 45.9 / 47.1 ms).
  const bool crowded = (long long)(h->MB / 128) * (long long)(h->maxw() / 128) >= 1024;
  const bool dual = !(h->flags & MI_FLAG_SERIAL_BACKWARD) && !h->timing && !crowded && !paired;
  if (!h->timing) {  // the per-kernel timing pass is not the schedule mi_mlp_get_schedule reports
    h->last_dual = dual;
    h->last_per_layer = per_layer;
    h->last_paired = paired;
  }
  hipStream_t s2 = dual ? h->stream2 : s;
  if (dual) {  // fork: dZ_{L-1} and all activations are ready
    MI_HIP(hipEventRecord(h->ev_fork, s));
    MI_HIP(hipStreamWaitEvent(s2, h->ev_fork, 0));
  }
  for (int l = h->L - 1; l >= 0; --l) {
    if (paired) {
      if ((rc = op_backward_pair(h, l, s))) return rc;
      continue;
    }
    // One backward stream, bf16: the input gradient goes first, so that the update of layer l,
    // which starts when both GEMMs of the layer are done, runs beside the input gradient of layer
    // l-1 and not beside its weight gradient -- there the update (which also writes the two bf16
    // weight copies) and the weight gradient both live on HBM writes (config 5: 43.8 -> 43.4 ms on
    // one box; the fp32 config 3 is 0.3 % faster the other way round and keeps it).  dZ, its
    // transposed copy and the column-sum partials rotate through buffers indexed by layer, so the
    // order within a layer is free.
    const bool dgrad_first = !dual && h->dtype == MI_BF16;
    if (!dgrad_first) {
      if ((rc = op_wgrad(h, l, s2, true))) return rc;
      if (dual) {
        MI_HIP(hipEventRecord(h->ev_wgrad[l], s2));
        if (l + 2 <= h->L - 1) MI_HIP(hipStreamWaitEvent(s, h->ev_wgrad[l + 2], 0));
      }
    }
    if ((rc = op_dgrad(h, l, s))) return rc;
    if (dgrad_first)
      if ((rc = op_wgrad(h, l, s, true))) return rc;
    if (dual || per_layer) {
      MI_HIP(hipEventRecord(h->ev_layer[l], s));
      if (s2 != s) MI_HIP(hipStreamWaitEvent(s2, h->ev_layer[l], 0));  // wgrad(l-1) needs dZ_{l-1}; update(l) needs W_l free
    }
    if (per_layer) {
      hipStream_t su = dual ? s2 : h->stream2;
      if (!dual) MI_HIP(hipStreamWaitEvent(su, h->ev_layer[l], 0));
      // every layer's update but the last one's (layer 0) runs under the GEMMs of the layers below
      if ((rc = op_update(h, l, lr, su, /*beside_gemm=*/su != s && l > 0))) return rc;
    }
  }
  if (dual || per_layer) {
    MI_HIP(hipEventRecord(h->ev_join, h->stream2));
    MI_HIP(hipStreamWaitEvent(s, h->ev_join, 0));
  }
  if (!per_layer)
    if ((rc = op_update(h, -1, lr, s))) return rc;
  return MI_OK;
}

void drop_graph(mi_mlp* h) {
  if (h->graph_exec) {
    (void)hipGraphExecDestroy(h->graph_exec);
    h->graph_exec = nullptr;
  }
}

// host <-> device copies of one [rows x cols] matrix with arbitrary host leading dimension
int upload_matrix(mi_mlp* h, void* dst, const float* src, int rows, int cols, int ld, bool as_bf16) {
  MI_REQUIRE(src != nullptr, "null host pointer");
  MI_REQUIRE(ld >= cols, "leading dimension %d smaller than %d columns", ld, cols);
  if (!as_bf16) {
    MI_HIP(hipMemcpy2DAsync(dst, (size_t)cols * 4, src, (size_t)ld * 4, (size_t)cols * 4, rows,
                            hipMemcpyHostToDevice, h->stream));
    MI_HIP(hipStreamSynchronize(h->stream));
    return MI_OK;
  }
  MI_REQUIRE((size_t)rows * cols <= h->staging_elems, "staging buffer too small");
  MI_HIP(hipMemcpy2DAsync(h->staging, (size_t)cols * 4, src, (size_t)ld * 4, (size_t)cols * 4, rows,
                          hipMemcpyHostToDevice, h->stream));
  hipError_t e = mi::convert_f32_to_bf16((uint16_t*)dst, h->staging, (size_t)rows * cols, h->stream);
  if (e != hipSuccess) return hip_fail(e, "convert launch");
  MI_HIP(hipStreamSynchronize(h->stream));
  return MI_OK;
}

int download_matrix(mi_mlp* h, float* dst, const void* src, int rows, int cols, int ld, bool from_bf16) {
  MI_REQUIRE(dst != nullptr, "null host pointer");
  MI_REQUIRE(ld >= cols, "leading dimension %d smaller than %d columns", ld, cols);
  MI_HIP(hipStreamSynchronize(h->stream));
  if (h->stream2) MI_HIP(hipStreamSynchronize(h->stream2));
  const void* from = src;
  if (from_bf16) {
    MI_REQUIRE((size_t)rows * cols <= h->staging_elems, "staging buffer too small");
    hipError_t e = mi::convert_bf16_to_f32(h->staging, (const uint16_t*)src, (size_t)rows * cols, h->stream);
    if (e != hipSuccess) return hip_fail(e, "convert launch");
    from = h->staging;
  }
  MI_HIP(hipMemcpy2DAsync(dst, (size_t)ld * 4, from, (size_t)cols * 4, (size_t)cols * 4, rows,
                          hipMemcpyDeviceToHost, h->stream));
  MI_HIP(hipStreamSynchronize(h->stream));
  return MI_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------------
extern "C" {

const char* mi_last_error(void) { return g_last_error.c_str(); }

int mi_device_info(char* name, int name_len, int* num_cus, int* clock_mhz, size_t* hbm_bytes) {
  int dev = 0, count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) return fail(MI_ERR_NO_DEVICE, "no HIP device visible");
  MI_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MI_HIP(hipGetDeviceProperties(&prop, dev));
  if (name && name_len > 0) snprintf(name, (size_t)name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (num_cus) *num_cus = prop.multiProcessorCount;
  if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
  if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
  return MI_OK;
}

int mi_malloc(void** dptr, size_t bytes) {
  MI_REQUIRE(dptr != nullptr, "null output pointer");
  *dptr = nullptr;
  if (bytes == 0) return MI_OK;
  MI_HIP(hipMalloc(dptr, bytes));
  return MI_OK;
}
int mi_free(void* dptr) {
  if (dptr) MI_HIP(hipFree(dptr));
  return MI_OK;
}
int mi_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes) MI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return MI_OK;
}
int mi_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes) MI_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return MI_OK;
}
int mi_memset(void* dptr, int byte, size_t bytes) {
  if (bytes) MI_HIP(hipMemset(dptr, byte, bytes));
  return MI_OK;
}
int mi_stream_sync(void* stream) {
  MI_HIP(hipStreamSynchronize(as_stream(stream)));
  return MI_OK;
}

int mi_set_gemm_variant(int kind, int variant) {
  MI_REQUIRE(kind >= 0 && kind < 3, "kind must be 0 (nt), 1 (nn) or 2 (tn)");
  g_variant[kind].store(variant);
  g_variant_epoch.fetch_add(1);
  return MI_OK;
}

// ---- raw operations -----------------------------------------------------------------------------

static int check_gemm(int M, int N, int K, const void* A, int lda, int min_lda, const void* B, int ldb, int min_ldb,
                      const void* C, int ldc) {
  MI_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative dimension (M=%d N=%d K=%d)", M, N, K);
  if (M == 0 || N == 0) return MI_OK;
  MI_REQUIRE(C != nullptr, "null C");
  MI_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "null operand");
  MI_REQUIRE(lda >= min_lda, "lda %d < %d", lda, min_lda);
  MI_REQUIRE(ldb >= min_ldb, "ldb %d < %d", ldb, min_ldb);
  MI_REQUIRE(ldc >= N, "ldc %d < N %d", ldc, N);
  return MI_OK;
}

int mi_sgemm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                const float* bias, int relu, void* stream) {
  if (int rc = check_gemm(M, N, K, A, lda, K, B, ldb, K, C, ldc)) return rc;
  hipError_t e = mi::sgemm_nt(M, N, K, A, lda, B, ldb, C, ldc, bias, relu, as_stream(stream), g_variant[0]);
  if (e != hipSuccess) return hip_fail(e, "mi_sgemm_nt launch");
  return MI_OK;
}

int mi_sgemm_nn(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                const float* mask_src, int ldmask, void* stream) {
  if (int rc = check_gemm(M, N, K, A, lda, K, B, ldb, N, C, ldc)) return rc;
  MI_REQUIRE(!mask_src || ldmask >= N, "ldmask %d < N %d", ldmask, N);
  hipError_t e = mi::sgemm_nn(M, N, K, A, lda, B, ldb, C, ldc, mask_src, ldmask, as_stream(stream), g_variant[1]);
  if (e != hipSuccess) return hip_fail(e, "mi_sgemm_nn launch");
  return MI_OK;
}

int mi_sgemm_tn(int R, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                long long strideC, float* colsum, long long stride_colsum, void* stream) {
  MI_REQUIRE(R >= 0, "negative replica count");
  if (R == 0) return MI_OK;
  if (int rc = check_gemm(M, N, K, A, lda, M, B, ldb, N, C, ldc)) return rc;
  MI_REQUIRE(R == 1 || strideC >= (long long)(M > 0 ? (size_t)(M - 1) * ldc + N : 0), "strideC overlaps replicas");
  MI_REQUIRE(!colsum || R == 1 || stride_colsum >= M, "stride_colsum overlaps replicas");
  hipError_t e = mi::sgemm_tn(R, M, N, K, A, lda, B, ldb, C, ldc, strideC, colsum, stride_colsum, as_stream(stream),
                              g_variant[2]);
  if (e != hipSuccess) return hip_fail(e, "mi_sgemm_tn launch");
  return MI_OK;
}

int mi_reduce_sgd_raw(float* W, const float* G, size_t n, size_t replica_stride, int R, float lr, void* stream) {
  MI_REQUIRE(R >= 1, "R must be at least 1 (got %d)", R);
  if (n == 0) return MI_OK;
  MI_REQUIRE(W && G, "null pointer");
  MI_REQUIRE(R == 1 || replica_stride >= n, "replica_stride %zu < n %zu", replica_stride, n);
  hipError_t e = mi::reduce_sgd(W, nullptr, G, n, replica_stride, R, lr, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "mi_reduce_sgd_raw launch");
  return MI_OK;
}

int mi_reduce_sgd_bf16_raw(float* W, void* W_bf16, const float* G, size_t n, size_t replica_stride, int R, float lr,
                           void* stream) {
  MI_REQUIRE(R >= 1, "R must be at least 1 (got %d)", R);
  if (n == 0) return MI_OK;
  MI_REQUIRE(W && G && W_bf16, "null pointer");
  MI_REQUIRE(R == 1 || replica_stride >= n, "replica_stride %zu < n %zu", replica_stride, n);
  hipError_t e = mi::reduce_sgd(W, (uint16_t*)W_bf16, G, n, replica_stride, R, lr, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "mi_reduce_sgd_bf16_raw launch");
  return MI_OK;
}

int mi_reduce_sgd_bf16t_raw(float* W, void* W_bf16, void* Wt_bf16, const float* G, int rows, int cols,
                            size_t replica_stride, int R, float lr, void* stream) {
  MI_REQUIRE(R >= 1, "R must be at least 1 (got %d)", R);
  MI_REQUIRE(rows >= 0 && cols >= 0, "negative size");
  if (rows == 0 || cols == 0) return MI_OK;
  MI_REQUIRE(W && G && W_bf16 && Wt_bf16, "null pointer");
  const size_t n = (size_t)rows * cols;
  MI_REQUIRE(R == 1 || replica_stride >= n, "replica_stride %zu < rows * cols %zu", replica_stride, n);
  hipStream_t s = as_stream(stream);
  hipError_t e;
  if (mi::reduce_sgd_tiled_fits(W, (uint16_t*)W_bf16, (uint16_t*)Wt_bf16, G, rows, cols, replica_stride, 0, R)) {
    e = mi::reduce_sgd_tiled(W, (uint16_t*)W_bf16, (uint16_t*)Wt_bf16, G, rows, cols, replica_stride, 0, R, lr, s);
  } else {  // any shape: flat update, then a transpose of the bf16 copy
    e = mi::reduce_sgd(W, (uint16_t*)W_bf16, G, n, replica_stride, R, lr, s);
    if (e == hipSuccess)
      e = mi::transpose_bf16(1, rows, cols, (const uint16_t*)W_bf16, cols, 0, (uint16_t*)Wt_bf16, rows, 0, s);
  }
  if (e != hipSuccess) return hip_fail(e, "mi_reduce_sgd_bf16t_raw launch");
  return MI_OK;
}

static int check_hgemm(int M, int N, int K, const void* A, int lda, const void* B, int ldb, const void* C, int ldc) {
  MI_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative dimension (M=%d N=%d K=%d)", M, N, K);
  if (M == 0 || N == 0) return MI_OK;
  MI_REQUIRE(C != nullptr, "null C");
  MI_REQUIRE(K == 0 || (A != nullptr && B != nullptr), "null operand");
  MI_REQUIRE(lda >= K && ldb >= K, "both operands are K-contiguous: lda %d, ldb %d must be >= K %d", lda, ldb, K);
  MI_REQUIRE(ldc >= N, "ldc %d < N %d", ldc, N);
  return MI_OK;
}

int mi_hgemm_nt(int M, int N, int K, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                const float* bias, int relu, void* stream) {
  if (int rc = check_hgemm(M, N, K, A, lda, B, ldb, C, ldc)) return rc;
  hipError_t e = mi::hgemm_nt(1, M, N, K, (const uint16_t*)A, lda, 0, (const uint16_t*)B, ldb, 0, C, ldc, 0, 1, bias,
                              relu, nullptr, 0, as_stream(stream), g_hvariant);
  if (e != hipSuccess) return hip_fail(e, "mi_hgemm_nt launch");
  return MI_OK;
}

int mi_hgemm_nn(int M, int N, int K, const void* A, int lda, const void* Bt, int ldbt, void* C, int ldc,
                const void* mask_src, int ldmask, void* stream) {
  if (int rc = check_hgemm(M, N, K, A, lda, Bt, ldbt, C, ldc)) return rc;
  MI_REQUIRE(!mask_src || ldmask >= N, "ldmask %d < N %d", ldmask, N);
  hipError_t e = mi::hgemm_nt(1, M, N, K, (const uint16_t*)A, lda, 0, (const uint16_t*)Bt, ldbt, 0, C, ldc, 0,
                              mask_src ? 2 : 3, nullptr, 0, (const uint16_t*)mask_src, ldmask, as_stream(stream),
                              g_hvariant);
  if (e != hipSuccess) return hip_fail(e, "mi_hgemm_nn launch");
  return MI_OK;
}

int mi_hgemm_tn(int R, int M, int N, int K, const void* At, int ldat, long long strideAt, const void* Bt, int ldbt,
                long long strideBt, float* C, int ldc, long long strideC, void* stream) {
  MI_REQUIRE(R >= 0, "negative replica count");
  if (R == 0) return MI_OK;
  if (int rc = check_hgemm(M, N, K, At, ldat, Bt, ldbt, C, ldc)) return rc;
  MI_REQUIRE(R == 1 || strideC >= (long long)(M > 0 ? (size_t)(M - 1) * ldc + N : 0), "strideC overlaps replicas");
  hipError_t e = mi::hgemm_nt(R, M, N, K, (const uint16_t*)At, ldat, strideAt, (const uint16_t*)Bt, ldbt, strideBt, C,
                              ldc, strideC, 0, nullptr, 0, nullptr, 0, as_stream(stream), g_hvariant);
  if (e != hipSuccess) return hip_fail(e, "mi_hgemm_tn launch");
  return MI_OK;
}

int mi_transpose_bf16(int batch, int rows, int cols, const void* src, int ld_src, long long batch_src, void* dst,
                      int ld_dst, long long batch_dst, void* stream) {
  MI_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "negative size");
  if (batch == 0 || rows == 0 || cols == 0) return MI_OK;
  MI_REQUIRE(src && dst, "null pointer");
  MI_REQUIRE(ld_src >= cols && ld_dst >= rows, "leading dimension too small");
  hipError_t e = mi::transpose_bf16(batch, rows, cols, (const uint16_t*)src, ld_src, batch_src, (uint16_t*)dst, ld_dst,
                                    batch_dst, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "mi_transpose_bf16 launch");
  return MI_OK;
}

int mi_rowsum_bf16(int batch, int rows, int cols, const void* src, int ld, long long batch_src, float* out,
                   long long stride_out, void* stream) {
  MI_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "negative size");
  if (batch == 0 || rows == 0) return MI_OK;
  MI_REQUIRE(out && (cols == 0 || src), "null pointer");
  hipError_t e = mi::rowsum_bf16(batch, rows, cols, (const uint16_t*)src, ld, batch_src, out, stride_out,
                                 as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "mi_rowsum_bf16 launch");
  return MI_OK;
}

int mi_set_hgemm_variant(int variant) {
  g_hvariant.store(variant);
  g_variant_epoch.fetch_add(1);
  return MI_OK;
}

int mi_probe_mfma_rate(int dtype, int operands, double* tflops, void* stream) {
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "dtype must be MI_F32 or MI_BF16 (got %d)", dtype);
  MI_REQUIRE(operands >= 0 && operands <= 3, "operands must be 0 (zeros), 1 (ones), 2 (random) or 3 (random, 32x32x16 bf16 MFMAs), got %d", operands);
  MI_REQUIRE(tflops != nullptr, "null result pointer");
  hipError_t e = mi::probe_mfma_rate(dtype == MI_BF16, operands, tflops, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "mi_probe_mfma_rate");
  return MI_OK;
}

int mi_convert_f32_to_bf16(void* dst, const float* src, size_t n, void* stream) {
  MI_REQUIRE(n == 0 || (dst && src), "null pointer");
  hipError_t e = mi::convert_f32_to_bf16((uint16_t*)dst, src, n, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "convert launch");
  return MI_OK;
}
int mi_convert_bf16_to_f32(float* dst, const void* src, size_t n, void* stream) {
  MI_REQUIRE(n == 0 || (dst && src), "null pointer");
  hipError_t e = mi::convert_bf16_to_f32(dst, (const uint16_t*)src, n, as_stream(stream));
  if (e != hipSuccess) return hip_fail(e, "convert launch");
  return MI_OK;
}

// ---- handle -------------------------------------------------------------------------------------

int mi_mlp_create(mi_mlp** out, int L, const int* nfeatures, int batch_per_replica, int R, int dtype,
                  unsigned flags) {
  MI_REQUIRE(out != nullptr, "null output handle");
  *out = nullptr;
  MI_REQUIRE(L >= 1 && L <= 4096, "layer count %d out of range", L);
  MI_REQUIRE(nfeatures != nullptr, "null nfeatures");
  MI_REQUIRE(batch_per_replica >= 1 && R >= 1, "batch_per_replica and R must be positive");
  MI_REQUIRE((long long)batch_per_replica * R <= 0x7fffffffLL, "R * batch overflows int");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "unknown dtype %d", dtype);
  for (int l = 0; l <= L; ++l) MI_REQUIRE(nfeatures[l] >= 1, "nfeatures[%d] = %d must be positive", l, nfeatures[l]);

  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) return fail(MI_ERR_NO_DEVICE, "no HIP device visible");

  mi_mlp* h = new (std::nothrow) mi_mlp;
  MI_REQUIRE(h != nullptr, "out of host memory");
  h->L = L;
  h->B = batch_per_replica;
  h->R = R;
  h->MB = batch_per_replica * R;
  h->dtype = dtype;
  h->flags = flags;
  h->nf.assign(nfeatures, nfeatures + L + 1);
  h->ndz = (flags & MI_FLAG_KEEP_GRADIENTS) ? std::max(L, 3) : 3;
  h->woff.resize(L);
  h->boff.resize(L);
  size_t off = 0;
  for (int l = 0; l < L; ++l) {
    h->woff[l] = off;
    off = round_up(off + (size_t)h->nf[l + 1] * h->nf[l], 64);
    h->boff[l] = off;
    off = round_up(off + (size_t)h->nf[l + 1], 64);
    h->P += (size_t)h->nf[l + 1] * h->nf[l] + h->nf[l + 1];
  }
  h->stride = off;
  h->ms.assign((size_t)MI_NUM_BREAKDOWNS * L, 0.0);
  h->launches.assign((size_t)MI_NUM_BREAKDOWNS * L, 0);

  int rc = MI_OK;
  auto alloc = [&](void** p, size_t bytes) {
    if (rc != MI_OK) return;
    hipError_t e = hipMalloc(p, bytes);
    if (e != hipSuccess) { rc = hip_fail(e, "hipMalloc"); return; }
    e = hipMemset(*p, 0, bytes);
    if (e != hipSuccess) rc = hip_fail(e, "hipMemset");
  };
  const size_t es = h->esize();
  alloc((void**)&h->params, h->stride * 4);
  alloc((void**)&h->neg_lr_dev, 256);
  alloc((void**)&h->grads, h->stride * 4 * (size_t)R);
  if (dtype == MI_BF16) {
    alloc((void**)&h->params16, h->stride * 2);
    alloc((void**)&h->params16T, h->stride * 2);
    h->actsT.assign(L, nullptr);
    for (int l = 0; l < L; ++l) alloc((void**)&h->actsT[l], (size_t)h->MB * h->nf[l] * 2);
    h->dzT.assign(h->ndz, nullptr);
    h->dzT_fused.assign(h->ndz, 0);
    h->dzT_fused_layer.assign(L, 0);
    for (int i = 0; i < h->ndz; ++i) alloc((void**)&h->dzT[i], (size_t)h->MB * h->maxw() * 2);
    alloc((void**)&h->dyT, (size_t)h->MB * h->nf[L] * 2);
    h->colpart.assign(h->ndz, nullptr);
    h->colpart_valid.assign(h->ndz, 0);
    for (int i = 0; i < h->ndz; ++i) alloc((void**)&h->colpart[i], ((size_t)h->MB / 128 + 1) * h->maxw() * 4);
    h->actsT_fused.assign(L, 0);
    size_t wmax = 0;
    for (int l = 0; l < L; ++l) wmax = std::max(wmax, (size_t)h->nf[l] * h->nf[l + 1]);
    h->staging_elems = std::max((size_t)h->MB * h->maxw(), wmax);
    alloc((void**)&h->staging, h->staging_elems * 4);
  }
  h->acts.assign(L + 1, nullptr);
  for (int l = 0; l <= L; ++l) alloc(&h->acts[l], (size_t)h->MB * h->nf[l] * es);
  alloc(&h->dy, (size_t)h->MB * h->nf[L] * es);
  h->dz.assign(h->ndz, nullptr);
  for (int i = 0; i < h->ndz; ++i) alloc(&h->dz[i], (size_t)h->MB * h->maxw() * es);
  alloc(&h->dx, (size_t)h->MB * h->nf[0] * es);
  if (rc == MI_OK && hipDeviceSynchronize() != hipSuccess) rc = fail(MI_ERR_HIP, "hipDeviceSynchronize failed");
  if (rc == MI_OK && hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking) != hipSuccess)
    rc = fail(MI_ERR_HIP, "hipStreamCreate failed");
  if (rc == MI_OK) {
    if (hipStreamCreateWithFlags(&h->stream2, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&h->ev_join, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&h->ev_fork, hipEventDisableTiming) != hipSuccess)
      rc = fail(MI_ERR_HIP, "second stream setup failed");
    h->ev_layer.assign(L, nullptr);
    h->ev_wgrad.assign(L, nullptr);
    for (int l = 0; l < L && rc == MI_OK; ++l)
      if (hipEventCreateWithFlags(&h->ev_layer[l], hipEventDisableTiming) != hipSuccess ||
          hipEventCreateWithFlags(&h->ev_wgrad[l], hipEventDisableTiming) != hipSuccess)
        rc = fail(MI_ERR_HIP, "hipEventCreate failed");
  }
  if (rc != MI_OK) {
    std::string keep = g_last_error;
    mi_mlp_destroy(h);
    g_last_error = keep;
    return rc;
  }
  *out = h;
  return MI_OK;
}

int mi_mlp_destroy(mi_mlp* h) {
  if (!h) return MI_OK;
  if (h->stream) (void)hipStreamSynchronize(h->stream);
  if (h->stream2) (void)hipStreamSynchronize(h->stream2);
  drop_graph(h);
  for (auto& p : h->pending) {
    (void)hipEventDestroy(p.a);
    (void)hipEventDestroy(p.b);
  }
  for (auto e : h->free_events) (void)hipEventDestroy(e);
  for (auto e : h->ev_layer)
    if (e) (void)hipEventDestroy(e);
  for (auto e : h->ev_wgrad)
    if (e) (void)hipEventDestroy(e);
  if (h->ev_join) (void)hipEventDestroy(h->ev_join);
  if (h->ev_fork) (void)hipEventDestroy(h->ev_fork);
  (void)hipFree(h->params);
  (void)hipFree(h->neg_lr_dev);
  (void)hipFree(h->grads);
  (void)hipFree(h->params16);
  (void)hipFree(h->params_saved);
  (void)hipFree(h->params16_saved);
  (void)hipFree(h->params16T);
  (void)hipFree(h->params16T_saved);
  for (auto a : h->actsT) (void)hipFree(a);
  for (auto a : h->dzT) (void)hipFree(a);
  (void)hipFree(h->dyT);
  for (auto a : h->colpart) (void)hipFree(a);
  for (void* a : h->acts) (void)hipFree(a);
  (void)hipFree(h->dy);
  for (void* a : h->dz) (void)hipFree(a);
  (void)hipFree(h->dx);
  (void)hipFree(h->staging);
  (void)hipFree(h->labels);
  (void)hipFree(h->loss_partials);
  for (auto& t : h->trace_items) {
    (void)hipEventDestroy(t.a);
    (void)hipEventDestroy(t.b);
  }
  if (h->stream) (void)hipStreamDestroy(h->stream);
  if (h->stream2) (void)hipStreamDestroy(h->stream2);
  delete h;
  return MI_OK;
}

int mi_mlp_set_weights(mi_mlp* h, int l, const float* W, int ld, const float* b) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  if (int rc = upload_matrix(h, h->params + h->woff[l], W, h->nf[l + 1], h->nf[l], ld, false)) return rc;
  if (b) {
    // on the handle's stream (the streams are non-blocking: a null-stream copy would not be
    // ordered against work still in flight on them)
    MI_HIP(hipMemcpyAsync(h->params + h->boff[l], b, (size_t)h->nf[l + 1] * 4, hipMemcpyHostToDevice, h->stream));
    MI_HIP(hipStreamSynchronize(h->stream));
  } else {
    MI_HIP(hipMemsetAsync(h->params + h->boff[l], 0, (size_t)h->nf[l + 1] * 4, h->stream));
    MI_HIP(hipStreamSynchronize(h->stream));
  }
  if (h->params16) {
    const size_t n = (size_t)h->nf[l + 1] * h->nf[l];
    hipError_t e = mi::convert_f32_to_bf16(h->params16 + h->woff[l], h->params + h->woff[l], n, h->stream);
    if (e == hipSuccess)
      e = mi::transpose_bf16(1, h->nf[l + 1], h->nf[l], h->params16 + h->woff[l], h->nf[l], 0,
                             h->params16T + h->woff[l], h->nf[l + 1], 0, h->stream);
    if (e != hipSuccess) return hip_fail(e, "bf16 weight copy");
    MI_HIP(hipStreamSynchronize(h->stream));
  }
  return MI_OK;
}

// bf16 models: the K-contiguous per-replica copy a weight-gradient GEMM reads, made once at upload
// for the two operands that no GEMM of the step produces (the input X and a given dY)
static int transposed_copy(mi_mlp* h, const void* src, int cols, uint16_t* dst) {
  hipError_t e = mi::transpose_bf16(h->R, h->B, cols, (const uint16_t*)src, cols, (long long)h->B * cols, dst, h->B,
                                    (long long)cols * h->B, h->stream);
  if (e != hipSuccess) return hip_fail(e, "transpose launch");
  MI_HIP(hipStreamSynchronize(h->stream));
  return MI_OK;
}

int mi_mlp_set_input(mi_mlp* h, const float* X, int ld) {
  if (int rc = check_handle(h)) return rc;
  if (int rc = upload_matrix(h, h->acts[0], X, h->MB, h->nf[0], ld, h->dtype == MI_BF16)) return rc;
  if (h->dtype == MI_BF16) {
    if (int rc = transposed_copy(h, h->acts[0], h->nf[0], h->actsT[0])) return rc;
    h->actsT_fused[0] = 1;  // nothing in a step writes X, so the copy stays valid
  }
  return MI_OK;
}

int mi_mlp_set_dy(mi_mlp* h, const float* dY, int ld) {
  if (int rc = check_handle(h)) return rc;
  if (h->use_loss) {  // a given upstream gradient replaces the loss front-end
    MI_HIP(hipStreamSynchronize(h->stream));
    MI_HIP(hipStreamSynchronize(h->stream2));
    h->use_loss = false;
    drop_graph(h);
  }
  if (int rc = upload_matrix(h, h->dy, dY, h->MB, h->nf[h->L], ld, h->dtype == MI_BF16)) return rc;
  if (h->dtype == MI_BF16) {
    if (int rc = transposed_copy(h, h->dy, h->nf[h->L], h->dyT)) return rc;
    h->dyT_valid = true;
  }
  return MI_OK;
}

int mi_mlp_set_labels(mi_mlp* h, const float* Y, int ld) {
  if (int rc = check_handle(h)) return rc;
  MI_HIP(hipStreamSynchronize(h->stream));
  MI_HIP(hipStreamSynchronize(h->stream2));
  const size_t n = (size_t)h->MB * h->nf[h->L];
  if (!h->labels) MI_HIP(hipMalloc((void**)&h->labels, n * 4));
  if (!h->loss_partials) {
    MI_HIP(hipMalloc((void**)&h->loss_partials, sizeof(double) * LOSS_CHUNKS * h->R));
    MI_HIP(hipMemset(h->loss_partials, 0, sizeof(double) * LOSS_CHUNKS * h->R));
  }
  if (int rc = upload_matrix(h, h->labels, Y, h->MB, h->nf[h->L], ld, false)) return rc;
  if (!h->use_loss) drop_graph(h);
  h->use_loss = true;
  return MI_OK;
}

int mi_loss_backward(mi_mlp* h) {
  if (int rc = check_handle(h)) return rc;
  return op_loss(h, h->stream);
}

int mi_mlp_get_loss(mi_mlp* h, double* loss_per_replica, double* total) {
  if (int rc = check_handle(h)) return rc;
  MI_REQUIRE(h->loss_partials != nullptr, "no labels set (mi_mlp_set_labels)");
  MI_HIP(hipStreamSynchronize(h->stream));
  MI_HIP(hipStreamSynchronize(h->stream2));
  std::vector<double> part((size_t)LOSS_CHUNKS * h->R);
  MI_HIP(hipMemcpy(part.data(), h->loss_partials, part.size() * sizeof(double), hipMemcpyDeviceToHost));
  double sum = 0.0;
  for (int r = 0; r < h->R; ++r) {
    double acc = 0.0;
    for (int c = 0; c < LOSS_CHUNKS; ++c) acc += part[(size_t)r * LOSS_CHUNKS + c];
    acc /= (double)h->B;
    if (loss_per_replica) loss_per_replica[r] = acc;
    sum += acc;
  }
  if (total) *total = sum;
  return MI_OK;
}

int mi_l2_loss_static(int dtype, int R, int batch_per_replica, int N, const void* pred, const float* label, void* dy,
                      double* loss_per_replica, void* stream) {
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "dtype must be MI_F32 or MI_BF16 (got %d)", dtype);
  MI_REQUIRE(R >= 1 && batch_per_replica >= 1 && N >= 1, "R, batch_per_replica and N must be positive (got %d, %d, %d)",
             R, batch_per_replica, N);
  MI_REQUIRE(R <= LOSS_STATIC_MAX_REPLICAS, "R = %d exceeds the %d replicas the static scratch holds", R,
             LOSS_STATIC_MAX_REPLICAS);
  MI_REQUIRE(pred && label && dy && loss_per_replica, "null pointer");
  double* scratch = nullptr;
  if (int rc = static_scratch_of_current_device(&scratch)) return rc;
  hipStream_t s = as_stream(stream);
  const size_t per_replica = (size_t)batch_per_replica * N;
  const float inv_b = 1.0f / (float)batch_per_replica;
  // every block of the grid stores its partial sum, so the scratch needs no clearing between calls
  if (dtype == MI_F32)
    mi::launch_kernel(l2_loss_kernel<false>, dim3(LOSS_CHUNKS, R), dim3(256), 0, s, dy, pred, label, per_replica, inv_b,
                      scratch);
  else
    mi::launch_kernel(l2_loss_kernel<true>, dim3(LOSS_CHUNKS, R), dim3(256), 0, s, dy, pred, label, per_replica, inv_b,
                      scratch);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "loss launch");
  mi::launch_kernel(loss_fold_kernel, dim3((R + 63) / 64), dim3(64), 0, s, (const double*)scratch, loss_per_replica, R,
                    (double)batch_per_replica);
  e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "loss fold launch");
  return MI_OK;
}

int mi_mlp_trace_step(mi_mlp* h, float lr, const char* path) {
  if (int rc = check_handle(h)) return rc;
  MI_REQUIRE(path != nullptr, "null path");
  MI_REQUIRE(!h->timing, "per-kernel timing and the step timeline cannot be on together");
  MI_HIP(hipStreamSynchronize(h->stream));
  MI_HIP(hipStreamSynchronize(h->stream2));
  hipEvent_t base = nullptr;
  if (int rc = get_event(h, &base)) return rc;
  h->tracing = true;
  h->trace_items.clear();
  int rc = MI_OK;
  if (hipEventRecord(base, h->stream) != hipSuccess) rc = fail(MI_ERR_HIP, "hipEventRecord failed");
  if (rc == MI_OK) rc = ensure_lr(h, lr);
  if (rc == MI_OK) rc = enqueue_step(h, lr);
  h->tracing = false;
  h->eager_steps++;
  hipError_t e1 = hipStreamSynchronize(h->stream), e2 = hipStreamSynchronize(h->stream2);
  if (rc == MI_OK && e1 != hipSuccess) rc = hip_fail(e1, "hipStreamSynchronize");
  if (rc == MI_OK && e2 != hipSuccess) rc = hip_fail(e2, "hipStreamSynchronize");
  FILE* f = rc == MI_OK ? fopen(path, "w") : nullptr;
  if (rc == MI_OK && !f) rc = fail(MI_ERR_INVALID, "cannot open %s for writing", path);
  if (f) {
    // Same record layout as the reference's trace.log (mlp_tbb.cc:85-104,1379-1392): an array of
    // begin/end records, ts in microseconds.  pid 0 is the GPU, tid the stream (0 main, 1 second).
    static const char* kNames[] = {"FC", "FCWgtGradient", "FCBwdGradient", "ReduceScatterAllGather"};
    fprintf(f, "[\n");
    for (size_t i = 0; i < h->trace_items.size() && rc == MI_OK; ++i) {
      const auto& t = h->trace_items[i];
      float t0 = 0.0f, t1 = 0.0f;
      if (hipEventElapsedTime(&t0, base, t.a) != hipSuccess || hipEventElapsedTime(&t1, base, t.b) != hipSuccess) {
        rc = fail(MI_ERR_HIP, "hipEventElapsedTime failed");
        break;
      }
      char name[64];
      if (t.breakdown == TRACE_LOSS) snprintf(name, sizeof name, "L2Loss_0");
      else if (t.breakdown == TRACE_PAIR) snprintf(name, sizeof name, "FCWgtGradient+FCBwdGradient_%d_0", t.layer);
      else if (t.layer < 0) snprintf(name, sizeof name, "%s_all_0", kNames[t.breakdown]);
      else snprintf(name, sizeof name, "%s_%d_0", kNames[t.breakdown], t.layer);
      fprintf(f, "{\n \"ts\": %.3f,\n \"pid\": 0,\n \"tid\": %d,\n \"name\": \"%s\",\n \"ph\": \"B\"\n},\n", t0 * 1e3,
              t.stream_id, name);
      fprintf(f, "{\n \"ts\": %.3f,\n \"pid\": 0,\n \"tid\": %d,\n \"ph\": \"E\"\n}%s\n", t1 * 1e3, t.stream_id,
              i + 1 < h->trace_items.size() ? "," : "");
    }
    fprintf(f, "]\n");
    fclose(f);
  }
  for (auto& t : h->trace_items) {
    h->free_events.push_back(t.a);
    h->free_events.push_back(t.b);
  }
  h->trace_items.clear();
  h->free_events.push_back(base);
  return rc;
}

int mi_fc_forward(mi_mlp* h, int l) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  return op_forward(h, l, h->stream);
}
int mi_fc_wgrad(mi_mlp* h, int l) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  if (l == h->L - 1)
    if (int rc = op_last_mask(h, h->stream)) return rc;
  return op_wgrad(h, l, h->stream, true);
}
int mi_fc_bgrad(mi_mlp* h, int l) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  if (l == h->L - 1)
    if (int rc = op_last_mask(h, h->stream)) return rc;
  return op_bgrad(h, l, h->stream);
}
int mi_fc_dgrad(mi_mlp* h, int l) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  if (l == h->L - 1)
    if (int rc = op_last_mask(h, h->stream)) return rc;
  return op_dgrad(h, l, h->stream);
}
int mi_reduce_sgd(mi_mlp* h, float lr) {
  if (int rc = check_handle(h)) return rc;
  if (int rc = ensure_lr(h, lr)) return rc;
  return op_update(h, -1, lr, h->stream);
}
int mi_reduce_sgd_layer(mi_mlp* h, int l, float lr) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  if (int rc = ensure_lr(h, lr)) return rc;
  return op_update(h, l, lr, h->stream);
}

int mi_mlp_step(mi_mlp* h, float lr) {
  if (int rc = check_handle(h)) return rc;
  const bool use_graph = !(h->flags & MI_FLAG_NO_GRAPH) && !h->timing;
  const int epoch_now = g_variant_epoch.load();
  if (h->graph_exec && h->graph_epoch != epoch_now) drop_graph(h);
  if (!use_graph || h->warm_epoch != epoch_now) {
    // Eager: the first step, every step of a handle without graph or with per-kernel timing on, and
    // the first untimed step after a change of the forced tile variants.  Such a step performs the
    // one-time kernel attribute setup of the kernels it launches, which must not happen inside a
    // stream capture; a timed step launches other kernels (separate launches, one stream) and so
    // does not count.
    h->eager_steps++;
    if (int rc = ensure_lr(h, lr)) return rc;
    if (int rc = enqueue_step(h, lr)) return rc;
    if (!h->timing) h->warm_epoch = epoch_now;
    return MI_OK;
  }
  if (int rc = ensure_lr(h, lr)) return rc;
  if (!h->graph_exec) {
    hipGraph_t graph = nullptr;
    MI_HIP(hipStreamBeginCapture(h->stream, hipStreamCaptureModeThreadLocal));
    int rc = enqueue_step(h, lr);
    hipError_t e = hipStreamEndCapture(h->stream, &graph);
    if (rc != MI_OK) {
      if (graph) (void)hipGraphDestroy(graph);
      return rc;
    }
    if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture");
    e = hipGraphInstantiate(&h->graph_exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
      h->graph_exec = nullptr;
      return hip_fail(e, "hipGraphInstantiate");
    }
    h->graph_epoch = epoch_now;
  }
  MI_HIP(hipGraphLaunch(h->graph_exec, h->stream));
  return MI_OK;
}

int mi_mlp_sync(mi_mlp* h) {
  if (int rc = check_handle(h)) return rc;
  MI_HIP(hipStreamSynchronize(h->stream));
  if (h->stream2) MI_HIP(hipStreamSynchronize(h->stream2));
  return MI_OK;
}

int mi_mlp_get_activation(mi_mlp* h, int l, float* dst, int ld) {
  if (int rc = check_layer(h, l, h ? h->L : 0)) return rc;
  return download_matrix(h, dst, h->acts[l], h->MB, h->nf[l], ld, h->dtype == MI_BF16);
}
int mi_mlp_get_weight(mi_mlp* h, int l, float* dst, int ld) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  return download_matrix(h, dst, h->params + h->woff[l], h->nf[l + 1], h->nf[l], ld, false);
}
int mi_mlp_get_bias(mi_mlp* h, int l, float* dst) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  return download_matrix(h, dst, h->params + h->boff[l], 1, h->nf[l + 1], h->nf[l + 1], false);
}
int mi_mlp_get_wgrad(mi_mlp* h, int l, int r, float* dst, int ld) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  MI_REQUIRE(r >= 0 && r < h->R, "replica index %d out of range [0,%d)", r, h->R);
  return download_matrix(h, dst, h->grads + (size_t)r * h->stride + h->woff[l], h->nf[l + 1], h->nf[l], ld, false);
}
int mi_mlp_get_bgrad(mi_mlp* h, int l, int r, float* dst) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  MI_REQUIRE(r >= 0 && r < h->R, "replica index %d out of range [0,%d)", r, h->R);
  return download_matrix(h, dst, h->grads + (size_t)r * h->stride + h->boff[l], 1, h->nf[l + 1], h->nf[l + 1], false);
}
int mi_mlp_get_dx(mi_mlp* h, float* dst, int ld) {
  if (int rc = check_handle(h)) return rc;
  return download_matrix(h, dst, h->dx, h->MB, h->nf[0], ld, h->dtype == MI_BF16);
}

int mi_mlp_snapshot_weights(mi_mlp* h) {
  if (int rc = check_handle(h)) return rc;
  if (!h->params_saved) MI_HIP(hipMalloc((void**)&h->params_saved, h->stride * 4));
  MI_HIP(mi::device_copy(h->params_saved, h->params, h->stride * 4, h->stream));
  if (h->params16) {
    if (!h->params16_saved) MI_HIP(hipMalloc((void**)&h->params16_saved, h->stride * 2));
    if (!h->params16T_saved) MI_HIP(hipMalloc((void**)&h->params16T_saved, h->stride * 2));
    MI_HIP(mi::device_copy(h->params16_saved, h->params16, h->stride * 2, h->stream));
    MI_HIP(mi::device_copy(h->params16T_saved, h->params16T, h->stride * 2, h->stream));
  }
  return MI_OK;
}

int mi_mlp_restore_weights(mi_mlp* h) {
  if (int rc = check_handle(h)) return rc;
  MI_REQUIRE(h->params_saved != nullptr, "no snapshot taken");
  MI_HIP(mi::device_copy(h->params, h->params_saved, h->stride * 4, h->stream));
  if (h->params16) {
    MI_HIP(mi::device_copy(h->params16, h->params16_saved, h->stride * 2, h->stream));
    MI_HIP(mi::device_copy(h->params16T, h->params16T_saved, h->stride * 2, h->stream));
  }
  return MI_OK;
}

int mi_mlp_get_dz(mi_mlp* h, int l, float* dst, int ld) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  return download_matrix(h, dst, dz_of_layer(h, l), h->MB, h->nf[l + 1], ld, h->dtype == MI_BF16);
}

int mi_mlp_get_schedule(mi_mlp* h, int* info) {
  if (int rc = check_handle(h)) return rc;
  MI_REQUIRE(info != nullptr, "null output pointer");
  MI_REQUIRE(h->eager_steps > 0, "no step has run yet");
  info[0] = h->last_dual ? 1 : 0;
  info[1] = h->last_per_layer ? 1 : 0;
  info[2] = h->graph_exec ? 1 : 0;
  int fused = 0;
  if (h->dtype == MI_BF16) {
    for (int l = 1; l < h->L; ++l) fused += h->actsT_fused[l] ? 1 : 0;  // A_l^T written by forward(l-1)
    for (int l = 0; l + 1 < h->L; ++l) fused += h->dzT_fused_layer[l] ? 1 : 0;  // dZ_l^T written by dgrad(l+1)
  }
  info[3] = fused;
  info[4] = h->last_paired ? 1 : 0;
  return MI_OK;
}

int mi_mlp_get_weight_shadow(mi_mlp* h, int l, int transposed, float* dst, int ld) {
  if (int rc = check_layer(h, l, h ? h->L - 1 : 0)) return rc;
  MI_REQUIRE(h->dtype == MI_BF16, "only bf16 models keep bf16 weight copies");
  if (transposed) return download_matrix(h, dst, h->params16T + h->woff[l], h->nf[l], h->nf[l + 1], ld, true);
  return download_matrix(h, dst, h->params16 + h->woff[l], h->nf[l + 1], h->nf[l], ld, true);
}

int mi_mlp_param_count(mi_mlp* h, size_t* params, size_t* replica_stride) {
  if (int rc = check_handle(h)) return rc;
  if (params) *params = h->P;
  if (replica_stride) *replica_stride = h->stride;
  return MI_OK;
}

int mi_mlp_enable_timing(mi_mlp* h, int on) {
  if (int rc = check_handle(h)) return rc;
  if (!on)
    if (int rc = harvest(h)) return rc;
  h->timing = on != 0;
  return MI_OK;
}
int mi_mlp_reset_timings(mi_mlp* h) {
  if (int rc = check_handle(h)) return rc;
  if (int rc = harvest(h)) return rc;
  std::fill(h->ms.begin(), h->ms.end(), 0.0);
  std::fill(h->launches.begin(), h->launches.end(), 0);
  return MI_OK;
}
int mi_mlp_get_timings(mi_mlp* h, double* ms, long long* launches) {
  if (int rc = check_handle(h)) return rc;
  if (int rc = harvest(h)) return rc;
  if (ms) std::memcpy(ms, h->ms.data(), h->ms.size() * sizeof(double));
  if (launches) std::memcpy(launches, h->launches.data(), h->launches.size() * sizeof(long long));
  return MI_OK;
}

}  // extern "C"
