/*
 * mi_mlp.h -- C ABI of libmi_mlp.so: the MI355X (gfx950) implementation of the tbb_test MLP
 * training step (forward GEMM, the two backward GEMMs, gradient reduce + SGD).
 *
 * The reference has no FFI: its hot path is three cblas_sgemm call sites and two hand-written
 * all-reduce functions, called from the iteration loop of mlp_omp.cc / mlp_tbb.cc.  Each entry
 * point below names the reference call site it stands in for.
 *
 * Conventions
 *   - every function returns MI_OK (0) or a negative mi_status; mi_last_error() gives the text
 *     of the most recent failure on the calling thread.  Nothing here aborts the process.
 *   - all matrices are row-major with an explicit leading dimension in ELEMENTS.
 *   - "device pointer" = memory of the current HIP device (hipMalloc, mi_malloc, or a
 *     torch tensor's data_ptr()); "host pointer" = ordinary pageable or pinned host memory.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Raw operations are
 *     asynchronous with respect to the host.
 *   - a handle is not thread-safe; distinct handles may be used from distinct threads (the
 *     library's own process-wide state -- kernel attributes per device, the tuning hooks -- is
 *     synchronised; mi_last_error() is per thread).
 */
#ifndef MI_MLP_H
#define MI_MLP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mi_status {
  MI_OK = 0,
  MI_ERR_INVALID = -1,     /* bad argument (shape, alignment, null pointer, index out of range) */
  MI_ERR_HIP = -2,         /* a HIP runtime call failed; mi_last_error() carries hipGetErrorString */
  MI_ERR_NO_DEVICE = -3,   /* no gfx950 device visible */
  MI_ERR_UNSUPPORTED = -4  /* valid request this build does not implement */
} mi_status;

typedef enum mi_dtype {
  MI_F32 = 0, /* fp32 storage, fp32 MFMA */
  MI_BF16 = 1 /* bf16 activations and weight shadow, fp32 MFMA accumulation, fp32 master weights,
                 fp32 gradients and reduce */
} mi_dtype;

/* mi_mlp_create flags */
#define MI_FLAG_RELU_LAST 0x1u   /* ReLU after the last layer too (c2_bench/mlp_caffe2.py:215-217);
                                    default: ReLU between layers only */
#define MI_FLAG_NO_GRAPH 0x2u    /* mi_mlp_step launches kernels one by one instead of replaying a
                                    captured HIP graph */
#define MI_FLAG_PER_LAYER_UPDATE 0x4u /* reduce + SGD of layer l+1 is issued right after layer
                                    l+1's input-gradient GEMM on a second stream, so it overlaps
                                    layer l's GEMMs -- the schedule of OVERLAP_ALL_REDUCE,
                                    mlp_omp.cc:601-615,692-723 -- instead of one launch over all
                                    layers at the end of the step */

#define MI_FLAG_SERIAL_BACKWARD 0x8u /* keep the whole backward pass on one stream; default: the
                                    weight-gradient GEMMs run on a second stream next to the chain
                                    of input-gradient GEMMs (they are independent per layer),
                                    except for models whose GEMMs have four or more 128 x 128
                                    tiles per CU and fill the device on their own */

#define MI_FLAG_KEEP_GRADIENTS 0x10u /* every layer's dZ (gradient w.r.t. the layer's pre-activation
                                    output) keeps a buffer of its own, so that mi_mlp_get_dz answers
                                    for every layer after a whole step; default: three buffers in
                                    rotation.  Same kernels, same stream dependencies, same results;
                                    costs (L-3) * R*B * max width elements of HBM.  For verification. */

/* Timing slots, same names and order as the reference's enum Breakdown
 * (mlp_bench_common.h:12-20). */
enum {
  MI_FWD = 0,
  MI_WGT_GRAD,
  MI_BWD,
  MI_WGT_UPDATE,
  MI_WGT_UPDATE_REDUCE_SCATTER, /* always 0 on one GPU: there is no scatter phase */
  MI_WGT_UPDATE_ALLGATHER,      /* always 0 on one GPU: there is one copy of W    */
  MI_NUM_BREAKDOWNS
};

/* ------------------------------------------------------------------------------------------ */
/* library / device                                                                           */

const char* mi_last_error(void);

/* Name, compute-unit count, peak engine clock (MHz) and memory size of the current device. */
int mi_device_info(char* name, int name_len, int* num_cus, int* clock_mhz, size_t* hbm_bytes);

/* Thin device-memory helpers so that a host program needs no HIP headers. */
int mi_malloc(void** dptr, size_t bytes);
int mi_free(void* dptr);
int mi_memcpy_h2d(void* dst, const void* src, size_t bytes);
int mi_memcpy_d2h(void* dst, const void* src, size_t bytes);
int mi_memset(void* dptr, int byte, size_t bytes);
int mi_stream_sync(void* stream);

/* Tuning hook: force tile configuration `variant` of the MFMA GEMM for kind 0 (nt), 1 (nn) or
 * 2 (tn); 0 restores the automatic choice.  A shape the forced configuration cannot tile falls
 * back to the any-shape kernel.  Process-wide; a handle that already captured its step graph
 * captures it again before the next replay.  Not meant for production callers. */
int mi_set_gemm_variant(int kind, int variant);

/* ------------------------------------------------------------------------------------------ */
/* raw operations on device pointers: one per reference call site                             */

/*
 * Forward:  C[M x N] = A[M x K] * B[N x K]^T (+ bias[N]) , optional ReLU.
 * Replaces cblas_sgemm(RowMajor, NoTrans, Trans, ...) at mlp_omp.cc:474-488 / mlp_tbb.cc:860-874
 * (A = activations[l], B = weights[l], C = activations[l+1]); one call covers the whole
 * M = R*B batch instead of one call per thread block.  bias may be NULL.
 */
int mi_sgemm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                int ldc, const float* bias, int relu, void* stream);

/*
 * Input gradient:  C[M x N] = A[M x K] * B[K x N], optionally multiplied element-wise by
 * [mask_src > 0] (mask_src[M x N], leading dimension ldmask; NULL = no mask).
 * Replaces cblas_sgemm(RowMajor, NoTrans, NoTrans, ...) at mlp_omp.cc:657-671 /
 * mlp_tbb.cc:1144-1158 (A = dY of layer l, B = weights[l], C = dX).
 */
int mi_sgemm_nn(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                int ldc, const float* mask_src, int ldmask, void* stream);

/*
 * Weight gradient, one GEMM per replica in a single launch:
 *   for r in [0, R):  C_r[M x N] = A[r*K .. (r+1)*K, 0..M)^T * B[r*K .. (r+1)*K, 0..N)
 *                     colsum_r[M] = sum over those K rows of A          (if colsum != NULL)
 * with C_r = C + r*strideC and colsum_r = colsum + r*stride_colsum (strides in elements).
 * Replaces cblas_sgemm(RowMajor, Trans, NoTrans, ...) at mlp_omp.cc:565-580 /
 * mlp_tbb.cc:1029-1043, including the split of the batch (k) over sockets at
 * mlp_omp.cc:529-531: replica r = socket r, A = dY of layer l, B = activations[l],
 * C_r = the socket's own slice of weight_grads[l].  colsum is the bias gradient.
 */
int mi_sgemm_tn(int R, int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                float* C, int ldc, long long strideC, float* colsum, long long stride_colsum,
                void* stream);

/*
 * Gradient reduce with the SGD update fused in, over a flat array of n floats:
 *   W[i] = fma(-lr, G[i] + G[stride+i] + ... + G[(R-1)*stride+i], W[i])
 * fp32 adds in replica order, one fused multiply-add (the arithmetic of mlp_omp.cc:140-143 and
 * :242-250).  Replaces update_weight_reduce_scatter + update_weight_allgather
 * (mlp_omp.cc:56-169,171-295; mlp_tbb.cc:142-456): with all R replicas' gradients resident in
 * one HBM there is nothing to scatter or gather, and one W instead of R copies.
 */
int mi_reduce_sgd_raw(float* W, const float* G, size_t n, size_t replica_stride, int R, float lr,
                      void* stream);

/* Same, additionally writing the updated weights rounded to bf16 (round-to-nearest-even) into
 * W_bf16[n] (the operand copy the bf16 GEMMs read). */
int mi_reduce_sgd_bf16_raw(float* W, void* W_bf16, const float* G, size_t n, size_t replica_stride,
                           int R, float lr, void* stream);

/* Same for one dense weight matrix W [rows x cols], additionally writing the transposed bf16 copy
 * Wt_bf16 [cols x rows] in the same pass (the operand of the bf16 input-gradient GEMM) -- the GPU
 * form of the reference forwarding each updated chunk to its consumers inside the update pass
 * (mlp_omp.cc:240-252).  rows and cols multiples of 64 with 16-byte aligned pointers run as one
 * tiled kernel; anything else as the flat update followed by a transpose. */
int mi_reduce_sgd_bf16t_raw(float* W, void* W_bf16, void* Wt_bf16, const float* G, int rows, int cols,
                            size_t replica_stride, int R, float lr, void* stream);

/*
 * bf16 variants of the three GEMMs (bf16 stored as 16-bit words, fp32 accumulation on
 * v_mfma_f32_16x16x32_bf16 for the large shapes, v_mfma_f32_32x32x16_bf16 otherwise).  A bf16 MFMA reads 8 consecutive k per lane, so every operand must be
 * K-contiguous; where the fp32 call site reads a row-contiguous operand, the bf16 entry point
 * takes its transposed copy (mi_transpose_bf16 makes one):
 *   mi_hgemm_nt  forward          C[M x N] (bf16) = A[M x K] * B[N x K]^T + bias, optional ReLU
 *   mi_hgemm_nn  input gradient   C[M x N] (bf16) = A[M x K] * B[K x N], given Bt = B^T [N x K],
 *                                 zeroed where mask_src (bf16, [M x N]) <= 0 if mask_src != NULL
 *   mi_hgemm_tn  weight gradient  C_r[M x N] (fp32) = A_r^T * B_r over the K rows of replica r,
 *                                 given At_r = A_r^T [M x K] and Bt_r = B_r^T [N x K]; replica r's
 *                                 operands start at At + r*strideAt, Bt + r*strideBt (elements)
 */
int mi_hgemm_nt(int M, int N, int K, const void* A, int lda, const void* B, int ldb, void* C,
                int ldc, const float* bias, int relu, void* stream);
int mi_hgemm_nn(int M, int N, int K, const void* A, int lda, const void* Bt, int ldbt, void* C,
                int ldc, const void* mask_src, int ldmask, void* stream);
int mi_hgemm_tn(int R, int M, int N, int K, const void* At, int ldat, long long strideAt,
                const void* Bt, int ldbt, long long strideBt, float* C, int ldc, long long strideC,
                void* stream);
/* dst[z][c][r] = src[z][r][c] for z < batch: 16-bit elements, leading dimensions and batch
 * strides in elements. */
int mi_transpose_bf16(int batch, int rows, int cols, const void* src, int ld_src, long long batch_src,
                      void* dst, int ld_dst, long long batch_dst, void* stream);
/* out[z*stride_out + r] = sum over c of src[z][r][c] (fp32 sums of a bf16 matrix): the bias
 * gradient from a transposed gradient copy. */
int mi_rowsum_bf16(int batch, int rows, int cols, const void* src, int ld, long long batch_src,
                   float* out, long long stride_out, void* stream);
/* Tuning hook for the bf16 kernel, like mi_set_gemm_variant. */
int mi_set_hgemm_variant(int variant);

/*
 * Measurement aid without a counterpart in the reference: the rate, in TFLOP/s, of a loop of
 * independent MFMAs on register operands (v_mfma_f32_32x32x2_f32 for MI_F32,
 * v_mfma_f32_16x16x32_bf16, the instruction of the large bf16 GEMMs, for MI_BF16) with no memory
 * traffic, i.e. what the matrix cores of this device sustain at best.  operands: 0 = zeros,
 * 1 = ones, 2 = pseudo-random values in [-1, 1) -- the bf16 rate is power-limited and depends on
 * them -- 3 = the same random values through v_mfma_f32_32x32x16_bf16 (MI_BF16; for fp32 the same
 * as 2), which sustains less on this device.  Blocks until the measurement is
 * done (about 0.4 s; the rate is the average over the second half, so that idle clocks do not
 * enter); allocates and frees a small device buffer.
 */
int mi_probe_mfma_rate(int dtype, int operands, double* tflops, void* stream);

/* fp32 <-> bf16 conversion of n contiguous elements on the device. */
int mi_convert_f32_to_bf16(void* dst_bf16, const float* src, size_t n, void* stream);
int mi_convert_bf16_to_f32(float* dst, const void* src_bf16, size_t n, void* stream);

/* ------------------------------------------------------------------------------------------ */
/* handle API: the whole model resident in HBM                                                */

typedef struct mi_mlp mi_mlp;

/*
 * Allocates the model on the current device: L fully-connected layers of widths
 * nfeatures[0..L] (layer l maps nfeatures[l] -> nfeatures[l+1], weight W_l is
 * [nfeatures[l+1] x nfeatures[l]] as at mlp_omp.cc:395-396), R data-parallel replicas of
 * batch_per_replica rows each (replica r owns rows [r*B, (r+1)*B) of every activation, the
 * split of Partition.cc:25-27).  Device state: one parameter arena (all W_l and b_l), R gradient
 * arenas of the same layout, L+1 activation buffers and three rotating dZ buffers (bf16 models
 * add the bf16 weight copies W, W^T and the transposed operand copies of the weight gradient).
 * Stands in for the allocation block of main(), mlp_omp.cc:390-409.
 */
int mi_mlp_create(mi_mlp** h, int L, const int* nfeatures, int batch_per_replica, int R, int dtype,
                  unsigned flags);
int mi_mlp_destroy(mi_mlp* h);

/* Host -> device uploads.  ld in elements; b may be NULL (bias = 0).  Stand in for
 * init_matrices(), mlp_bench_common.cc:16-33.  bf16 models convert on the device and also make the
 * K-contiguous copies their GEMMs read (W^T at mi_mlp_set_weights, the per-replica X^T and dY^T at
 * mi_mlp_set_input / mi_mlp_set_dy), so that a step moves none of these again. */
int mi_mlp_set_weights(mi_mlp* h, int l, const float* W, int ld, const float* b);
int mi_mlp_set_input(mi_mlp* h, const float* X, int ld);
int mi_mlp_set_dy(mi_mlp* h, const float* dY, int ld);

/* Per-operation entry points, asynchronous on the handle's stream.  Backward runs from the
 * last layer down; mi_fc_dgrad(l) consumes the gradient produced by mi_fc_dgrad(l+1) (or the
 * uploaded dY for l = L-1). */
int mi_fc_forward(mi_mlp* h, int l); /* mlp_omp.cc:441-510 */
int mi_fc_wgrad(mi_mlp* h, int l);   /* mlp_omp.cc:513-600, all R replicas; also the bias gradient */
int mi_fc_bgrad(mi_mlp* h, int l);   /* bias gradient alone (column sums of the layer's dZ) */
int mi_fc_dgrad(mi_mlp* h, int l);   /* mlp_omp.cc:619-691 */
int mi_reduce_sgd(mi_mlp* h, float lr);                /* all layers, one launch */
int mi_reduce_sgd_layer(mi_mlp* h, int l, float lr);   /* one layer (W_l and b_l) */

/* One full step: forward over all layers, backward over all layers, reduce + SGD
 * (the body of the iteration loop, mlp_omp.cc:435-737). Asynchronous; mi_mlp_sync waits. */
int mi_mlp_step(mi_mlp* h, float lr);
int mi_mlp_sync(mi_mlp* h);

/* Device -> host downloads (synchronous).  Activations and gradients come back as fp32 whatever
 * the handle's dtype.  l in [0, L] for activations (0 = input), r in [0, R). */
int mi_mlp_get_activation(mi_mlp* h, int l, float* dst, int ld);
int mi_mlp_get_weight(mi_mlp* h, int l, float* dst, int ld);
int mi_mlp_get_bias(mi_mlp* h, int l, float* dst);
int mi_mlp_get_wgrad(mi_mlp* h, int l, int r, float* dst, int ld);
int mi_mlp_get_bgrad(mi_mlp* h, int l, int r, float* dst);
int mi_mlp_get_dx(mi_mlp* h, float* dst, int ld);
/* Gradient with respect to the pre-activation output of layer l, [R*B x N_{l+1}]: the uploaded dY
 * for l = L-1, otherwise what mi_fc_dgrad(l+1) produced.  dZ_l lives in buffer l mod 3 of a
 * rotation of three, so the value is meaningful from mi_fc_dgrad(l+1) until mi_fc_dgrad(l-2)
 * overwrites it (after a whole step: layers 0, 1, 2 and L-1); with MI_FLAG_KEEP_GRADIENTS every
 * layer keeps its own buffer and the value stays until the next step. */
int mi_mlp_get_dz(mi_mlp* h, int l, float* dst, int ld);

/* Device-side copy of all weights and biases (snapshot) and its inverse (restore), both
 * asynchronous on the handle's stream.  A benchmark loop restores before every step so that the
 * values stay finite over any number of sum-reduced SGD steps; the reference gets the same effect
 * by benchmarking with alpha = 1e-10 (mlp_omp.cc:609,699,718). */
int mi_mlp_snapshot_weights(mi_mlp* h);
int mi_mlp_restore_weights(mi_mlp* h);

/* bf16 models: the bf16 copy of W_l that the forward GEMM reads (transposed = 0, [N_{l+1} x N_l])
 * or the transposed copy W_l^T that the input-gradient GEMM reads (transposed = 1,
 * [N_l x N_{l+1}]), widened to fp32.  Both are rewritten by every update.  Synchronous. */
int mi_mlp_get_weight_shadow(mi_mlp* h, int l, int transposed, float* dst, int ld);

/* What the last mi_mlp_step / mi_mlp_trace_step outside per-kernel timing actually did (the
 * scheduling flags are requests; the library also looks at the shapes):
 *   info[0]  1 = backward pass on two streams, 0 = on one
 *   info[1]  1 = one update launch per layer on the second stream, 0 = one launch at the end
 *   info[2]  1 = steps replay a captured HIP graph
 *   info[3]  bf16 models: how many of the 2(L-1) transposed operand copies of the weight-gradient
 *            GEMMs were written by the epilogue of the GEMM that produced the operand (the rest
 *            came from separate transpose launches); 0 for fp32 models
 *   info[4]  1 = small fp32 model: weight gradient and input gradient of a layer share one launch,
 *            everything on one stream with one update launch (fewest launches; the scheduling
 *            flags have nothing to overlap there)
 * info must have room for 5 ints. */
int mi_mlp_get_schedule(mi_mlp* h, int* info);

/* Number of parameters P = sum_l (N_l*N_{l+1} + N_{l+1}) and the padded element stride between
 * consecutive replicas' gradient arenas. */
int mi_mlp_param_count(mi_mlp* h, size_t* params, size_t* replica_stride);

/*
 * Per-phase device timing with HIP events on the handle's stream (the role of sum_times /
 * dsecnd() in mlp_omp.cc:490-508,582-600,673-691,161-168).  While enabled, every kernel of
 * mi_mlp_step and of the per-operation entry points carries a start and a stop event on its
 * dispatch, so the figures are kernel execution times without launch gaps.
 * While timing is enabled the step runs serially on one stream with a single update launch,
 * whatever the scheduling flags say, because overlapping kernels cannot be timed individually.
 * mi_mlp_get_timings synchronises and writes accumulated milliseconds as
 * ms[breakdown * L + layer]; the single all-layer reduce launch is booked under
 * MI_WGT_UPDATE, layer 0.  launches[] (same indexing, may be NULL) receives launch counts.
 */
int mi_mlp_enable_timing(mi_mlp* h, int on);
int mi_mlp_reset_timings(mi_mlp* h);
int mi_mlp_get_timings(mi_mlp* h, double* ms, long long* launches);

/*
 * Loss front-end: SquaredL2Distance + AveragedLoss per replica as in the Caffe2 harness
 * (mlp_caffe2.py:221-239): loss_r = (1/B) sum_{i in replica r} 0.5 * |pred_i - label_i|^2, the
 * total is the sum over replicas, and the upstream gradient is dY = (pred - label) / B.
 * mi_mlp_set_labels uploads Y [R*B x N_L] (fp32 on the device for both dtypes) and switches the
 * handle to "loss mode": every mi_mlp_step then derives dY from its own forward output.
 * mi_mlp_set_dy switches back to a given dY.  mi_loss_backward is the per-operation entry point
 * (after mi_fc_forward(L-1), before the backward calls).  mi_mlp_get_loss synchronises and
 * returns the losses of the last step (either pointer may be NULL).
 */
int mi_mlp_set_labels(mi_mlp* h, const float* Y, int ld);
int mi_loss_backward(mi_mlp* h);
int mi_mlp_get_loss(mi_mlp* h, double* loss_per_replica, double* total);

/*
 * The loss front-end on caller-owned device buffers, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference; it is mi_loss_backward + mi_mlp_get_loss without a
 * handle: the same kernel, same arithmetic and same summation order, hence the same bits.
 *   dy[i]               = (pred[i] - label[i]) / batch_per_replica          (dtype of pred)
 *   loss_per_replica[r] = (1/B) sum over replica r's rows of 0.5 * |pred_i - label_i|^2  (device, R doubles)
 * pred, label and dy are dense [R*batch_per_replica x N]; pred and dy are fp32 (MI_F32) or bf16
 * (MI_BF16), label is fp32.  The kernel's partial sums live in a device-resident static array of
 * 512 KB (64 doubles per replica) that each GPU the library runs on holds until the process ends;
 * the call performs no hipMalloc / hipFree and fails with MI_ERR_INVALID for R > 1024.  The address
 * of the array is looked up on the first call on each device: make that call outside a graph
 * capture.  All calls on one GPU share the array, so calls that overlap in time on one GPU (two
 * streams, two threads) race; calls ordered on one stream do not.  Asynchronous on `stream`.
 */
int mi_l2_loss_static(int dtype, int R, int batch_per_replica, int N, const void* pred, const float* label,
                      void* dy, double* loss_per_replica, void* stream);

/*
 * Runs one step (like mi_mlp_step, eagerly, on the configured two-stream schedule) with an event
 * pair around every launch and writes the timeline to `path` in the format of the reference's
 * trace.log (mlp_tbb.cc:85-104,1379-1392: a JSON array of begin/end records with ts in
 * microseconds, loadable in a Chrome-trace viewer).  Names follow the reference's tasks
 * (mlp_tbb.cc:176-178,325-327,840,982,1104): FC_<l>_0, FCWgtGradient_<l>_0, FCBwdGradient_<l>_0;
 * the fused reduce + SGD launch of layer l is ReduceScatterAllGather_<l>_0 (_all_ when one launch
 * covers every layer), the loss kernel L2Loss_0; small fp32 models, whose two backward GEMMs of a
 * layer share a launch, show FCWgtGradient+FCBwdGradient_<l>_0 instead of the two.  pid 0 is the GPU, tid 0 / 1 the main / second
 * stream.  The step updates the weights like any other.
 */
int mi_mlp_trace_step(mi_mlp* h, float lr, const char* path);

#ifdef __cplusplus
}
#endif
#endif /* MI_MLP_H */
