/*
 * dragon_hip.h - C ABI of the MI355X (gfx950) kernel library behind Dragon's
 * kernels:: / math:: interface for LayerNorm, GroupNorm, BatchNorm, Moments,
 * Softmax / LogSoftmax and their siblings on the same reduction skeleton
 * (L1/L2Norm, ReduceSum, softmax cross-entropy loss).
 *
 * Each entry point replaces one function template of the reference (cited as
 * file:line relative to the reference tree). A `kernels::X<T, AccT, HIPContext>`
 * specialisation is a one-line forward to the entry point of the same name:
 * plain device pointers, 64-bit sizes, a dtype tag instead of the template
 * arguments, a layout tag instead of the "NCHW"/"NHWC" string, the context's
 * HIP stream, and (where a split reduction needs it) a scratch buffer the
 * caller takes from the context's workspace.
 *
 * Conventions
 *  - All tensor pointers are device pointers on the current device.
 *  - `dtype` is the I/O type T. Statistics, affine parameters and parameter
 *    gradients are AccT = float for f16/bf16/f32 and double for f64
 *    (dragon/utils/math/types.h:69-152).
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *  - Kernels are enqueued asynchronously; nothing here allocates, frees or
 *    synchronises, and every function is re-entrant.
 *  - Return value: 0 on success, a negative dragon_hip_status on an argument
 *    error (nothing was enqueued), a positive hipError_t when the runtime
 *    refused a launch. The reference aborts through LOG(FATAL) on every error
 *    (dragon/utils/logging.h:56-71); the HIPContext specialisation maps a
 *    non-zero status to that.
 *  - `scratch` may be NULL when the matching *_scratch_bytes() query returns 0;
 *    otherwise it must hold at least that many bytes, 256-byte aligned, and
 *    must not be shared by kernels running concurrently on other streams.
 */
#ifndef DRAGON_HIP_H_
#define DRAGON_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  DRAGON_HIP_F16 = 0,  /* dragon::float16  (dragon/core/types.h:36-38) */
  DRAGON_HIP_BF16 = 1, /* dragon::bfloat16 (dragon/core/types.h:40-42) */
  DRAGON_HIP_F32 = 2,
  DRAGON_HIP_F64 = 3,
  DRAGON_HIP_I32 = 4, /* class-index targets of the loss kernels only */
  DRAGON_HIP_I64 = 5
} dragon_hip_dtype;

typedef enum {
  DRAGON_HIP_NCHW = 0, /* data_format == "NCHW": x is [N, C, S]  */
  DRAGON_HIP_NHWC = 1  /* data_format == "NHWC": x is [N, S, C]  */
} dragon_hip_layout;

typedef enum {
  DRAGON_HIP_OK = 0,
  DRAGON_HIP_EINVAL = -1,   /* bad size, layout, null pointer or misalignment */
  DRAGON_HIP_EDTYPE = -2,   /* dtype not in dragon_hip_dtype                  */
  DRAGON_HIP_ESCRATCH = -3, /* scratch missing or too small                   */
  DRAGON_HIP_ENODEVICE = -4, /* no gfx950 device visible                      */
  DRAGON_HIP_ETIMEOUT = -5, /* reserved: no entry point returns it             */
  DRAGON_HIP_ELIMIT = -6    /* the shape needs more scratch than the static
                               buffer of a *_noalloc entry point holds         */
} dragon_hip_status;

/* Human-readable text for a status returned by any function below. */
const char* dragon_hip_status_string(int status);

/* ------------------------------------------------------------------------ */
/* Device-context plumbing: what a HIPContext needs so that the host layer   */
/* includes no HIP header. Mirrors the static/member set every Dragon device */
/* context provides (dragon/core/context_cuda.h:156-332; leanest precedent   */
/* dragon/core/context_mlu.h:124-284).                                       */
/* ------------------------------------------------------------------------ */
int dragon_hip_device_count(int* count);
int dragon_hip_set_device(int device);
int dragon_hip_get_device(int* device);
int dragon_hip_device_name(int device, char* buf, size_t buf_bytes);
int dragon_hip_device_capability(int device, int* major, int* minor);
int dragon_hip_device_sync(void);  /* every stream of the current device */
int dragon_hip_mem_info(size_t* free_bytes, size_t* total_bytes);
/* Streams are non-blocking and all at the default priority. */
int dragon_hip_stream_create(void** stream);
int dragon_hip_stream_destroy(void* stream);
int dragon_hip_stream_sync(void* stream);  /* Context::SynchronizeStream */
int dragon_hip_stream_query(void* stream, int* done); /* 1 when all work on it has finished */
int dragon_hip_malloc(void** ptr, size_t bytes);       /* Context::New    */
int dragon_hip_free(void* ptr);                        /* Context::Delete */
int dragon_hip_host_malloc(void** ptr, size_t bytes);  /* pinned host memory */
int dragon_hip_host_free(void* ptr);
int dragon_hip_memset_async(void* ptr, int value, size_t bytes, void* stream);
/* kind: 0 host->host, 1 host->device, 2 device->host, 3 device->device */
int dragon_hip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);
int dragon_hip_event_create(void** event);
int dragon_hip_event_destroy(void* event);
int dragon_hip_event_record(void* event, void* stream);
int dragon_hip_event_sync(void* event);
int dragon_hip_event_elapsed_ms(void* start, void* stop, float* ms);

/* ------------------------------------------------------------------------ */
/* math:: helpers the operator bodies call on AccT buffers                   */
/* ------------------------------------------------------------------------ */

/* math::InvStd<T, Context>, dragon/utils/math/elementwise.h:48 (CPU
 * dragon/utils/math/cpu/elementwise.cc:187-201): y = 1 / sqrt(x + eps).
 * y may alias x (the operators run it in place on the variance buffer). */
int dragon_hip_inv_std(int dtype, int64_t N, float eps, const void* x, void* y, void* stream);

/* math::Axpby<T, Context>, dragon/utils/math/cpu/blas.cc:125-136:
 * y = alpha * x + beta * y (running-statistics update, batch_norm_op.cc:60-63). */
int dragon_hip_axpby(int dtype, int64_t N, float alpha, const void* x, float beta, void* y, void* stream);

/* math::Copy / Set / Square / Sub as used at batch_norm_op.cc:45-47,148-165. */
int dragon_hip_copy(int dtype, int64_t N, const void* x, void* y, void* stream);
int dragon_hip_set(int dtype, int64_t N, float value, void* y, void* stream);
int dragon_hip_square(int dtype, int64_t N, const void* x, void* y, void* stream);
int dragon_hip_sub(int dtype, int64_t N, const void* a, const void* b, void* y, void* stream);

/* ------------------------------------------------------------------------ */
/* kernels::Moments, dragon/kernels/math/op_kernels.h:106-115                */
/* (CPU dragon/kernels/math/cpu/moments_kernel.cc:10-189): mean and BIASED   */
/* variance over `axes` of a row-major tensor of shape `dims`. mean / var    */
/* are AccT with one element per kept index, in row-major order.             */
/* ------------------------------------------------------------------------ */
size_t dragon_hip_moments_scratch_bytes(int dtype, int num_dims, const int64_t* dims,
                                        int num_axes, const int64_t* axes);
int dragon_hip_moments(int dtype, int num_dims, const int64_t* dims, int num_axes,
                       const int64_t* axes, const void* x, void* mean, void* var,
                       void* scratch, size_t scratch_bytes, void* stream);

/* math::ReduceSum / ReduceSumSqr / ReduceL1, dragon/utils/math/reduce.h:50-80
 * (CPU dragon/utils/math/cpu/reduce.cc:62-236): y = scale * sum f(x) over
 * `axes` with f = identity, square or absolute value. y is T with the kept
 * extents in order (as Moments); the sum is held in AccT and rounded once.
 * Scratch: dragon_hip_reduce_scratch_bytes (same planner as Moments). */
size_t dragon_hip_reduce_scratch_bytes(int dtype, int num_dims, const int64_t* dims, int num_axes,
                                       const int64_t* axes);
int dragon_hip_reduce_sum(int dtype, int num_dims, const int64_t* dims, int num_axes,
                          const int64_t* axes, float scale, const void* x, void* y, void* scratch,
                          size_t scratch_bytes, void* stream);
int dragon_hip_reduce_sum_sqr(int dtype, int num_dims, const int64_t* dims, int num_axes,
                              const int64_t* axes, float scale, const void* x, void* y,
                              void* scratch, size_t scratch_bytes, void* stream);
int dragon_hip_reduce_l1(int dtype, int num_dims, const int64_t* dims, int num_axes,
                         const int64_t* axes, float scale, const void* x, void* y, void* scratch,
                         size_t scratch_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* kernels::LayerNorm, dragon/kernels/normalization/op_kernels.h:191-202     */
/* (CPU dragon/kernels/normalization/cpu/layer_norm_kernel.cc:10-62).        */
/* x, y: T[N, C]; gamma, beta: AccT[C]; mu, rsig: AccT[N].                   */
/* ------------------------------------------------------------------------ */
int dragon_hip_layer_norm(int dtype, int64_t N, int64_t C, float eps, const void* x,
                          const void* gamma, const void* beta, void* mu, void* rsig,
                          void* y, void* stream);

/* ------------------------------------------------------------------------ */
/* kernels::GroupNorm, dragon/kernels/normalization/op_kernels.h:111-124     */
/* (CPU dragon/kernels/normalization/cpu/group_norm_kernel.cc:11-31,88-110). */
/* x, y: T[N,G,D,S] (NCHW) or T[N,S,G,D] (NHWC); mu, rsig: AccT[N*G];        */
/* gamma, beta: AccT[G*D].                                                   */
/* ------------------------------------------------------------------------ */
int dragon_hip_group_norm(int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
                          const void* x, const void* mu, const void* rsig, const void* gamma,
                          const void* beta, void* y, void* stream);

/* kernels::GroupNormGrad, dragon/kernels/normalization/op_kernels.h:126-143
 * (CPU group_norm_kernel.cc:33-84,112-147). Also LayerNorm backward with
 * G = S = 1, D = C, layout NHWC (dragon/operators/normalization/layer_norm_op.h:39-54).
 * ds, db: AccT[N*G] each, written by the call; ds == db means db = ds + N*G
 * (group_norm_kernel.cc:131). dgamma, dbeta: AccT[G*D]. All four are
 * overwritten (the reference zero-fills them first, :132-135). */
size_t dragon_hip_group_norm_grad_scratch_bytes(int dtype, int64_t N, int64_t G, int64_t D,
                                                int64_t S, int layout);
int dragon_hip_group_norm_grad(int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
                               const void* x, const void* mu, const void* rsig,
                               const void* gamma, const void* dy, void* ds, void* db,
                               void* dgamma, void* dbeta, void* dx, void* scratch,
                               size_t scratch_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* BatchNorm family, dragon/kernels/normalization/op_kernels.h:36-109        */
/* (CPU dragon/kernels/normalization/cpu/batch_norm_kernel.cc).              */
/* x, y, dy, dx: T[N,C,S] (NCHW) or T[N,S,C] (NHWC); every [C] vector AccT.  */
/* ------------------------------------------------------------------------ */

/* kernels::BatchNormExpectation (op_kernels.h:36-46): ex = sum(x)/normalizer,
 * ex2 = sum(x*x)/normalizer per channel. */
size_t dragon_hip_batch_norm_reduce_scratch_bytes(int dtype, int64_t N, int64_t C, int64_t S,
                                                  int layout);
int dragon_hip_batch_norm_expectation(int dtype, int64_t N, int64_t C, int64_t S,
                                      float normalizer, int layout, const void* x, void* ex,
                                      void* ex2, void* scratch, size_t scratch_bytes,
                                      void* stream);

/* kernels::BatchNorm (op_kernels.h:48-62): scale = gamma*rsig,
 * bias = beta - scale*mu, y = x*scale[c] + bias[c]. Aliasing conventions of
 * batch_norm_kernel.cc:244-248: scale == rsig means a 3C buffer
 * {rsig, scale, bias}; scale == bias means bias = scale + C. */
int dragon_hip_batch_norm(int dtype, int64_t N, int64_t C, int64_t S, int layout, const void* x,
                          const void* mu, const void* rsig, const void* gamma,
                          const void* beta, void* scale, void* bias, void* y, void* stream);

/* kernels::BatchNormWGrad (op_kernels.h:64-76): dgamma[c] = sum dy*(x-mu)*rsig,
 * dbeta[c] = sum dy; dgamma == dbeta means dbeta = dgamma + C (:296).
 * Scratch size: dragon_hip_batch_norm_reduce_scratch_bytes. */
int dragon_hip_batch_norm_wgrad(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                const void* x, const void* mu, const void* rsig, const void* dy,
                                void* dgamma, void* dbeta, void* scratch, size_t scratch_bytes,
                                void* stream);

/* kernels::BatchNormTrainingGrad (op_kernels.h:78-93):
 * dx = gamma*rsig*(dy - ((x-mu)*rsig*dgamma + dbeta)/normalizer);
 * dgamma == dbeta means dbeta = dgamma + C (:353). */
int dragon_hip_batch_norm_training_grad(int dtype, int64_t N, int64_t C, int64_t S,
                                        float normalizer, int layout, const void* x,
                                        const void* mu, const void* rsig, const void* gamma,
                                        const void* dgamma, const void* dbeta, const void* dy,
                                        void* dx, void* stream);

/* kernels::BatchNormInferenceGrad (op_kernels.h:95-109): dx = gamma*rsig*dy;
 * dgamma != NULL additionally runs BatchNormWGrad (:406-409). */
int dragon_hip_batch_norm_inference_grad(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                         const void* x, const void* mu, const void* rsig,
                                         const void* gamma, const void* dy, void* dgamma,
                                         void* dbeta, void* dx, void* scratch,
                                         size_t scratch_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Softmax family, dragon/kernels/activation/op_kernels.h:211-247            */
/* (CPU dragon/kernels/activation/cpu/softmax_kernel.cc:10-157).             */
/* Tensors are T[N, C, S]: the reduced axis has length C and element stride  */
/* S. y may alias x; dx may alias dy (softmax_op.cc:46-60).                  */
/* 16-bit I/O accumulates in fp32.                                           */
/* scratch may be NULL. With dragon_hip_softmax_scratch_bytes(...) bytes of it  */
/* (0 for shapes that need none) rows of many thousands of packets, e.g.      */
/* vocabulary-sized rows, are processed by several workgroups per row that     */
/* exchange their partial results through it; without it they take the         */
/* one-workgroup-per-row kernels. The context's workspace is what the          */
/* reference's launchers would pass (ctx->workspace()).                        */
/* ------------------------------------------------------------------------ */
size_t dragon_hip_softmax_scratch_bytes(int dtype, int64_t N, int64_t S, int64_t C);
int dragon_hip_softmax(int dtype, int64_t N, int64_t S, int64_t C, const void* x, void* y,
                       void* scratch, size_t scratch_bytes, void* stream);
int dragon_hip_log_softmax(int dtype, int64_t N, int64_t S, int64_t C, const void* x, void* y,
                           void* scratch, size_t scratch_bytes, void* stream);
int dragon_hip_softmax_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dy,
                            const void* y, void* dx, void* scratch, size_t scratch_bytes,
                            void* stream);
int dragon_hip_log_softmax_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dy,
                                const void* y, void* dx, void* scratch, size_t scratch_bytes,
                                void* stream);

/* ------------------------------------------------------------------------ */
/* L1Norm / L2Norm, dragon/kernels/normalization/op_kernels.h:145-189        */
/* (CPU dragon/kernels/normalization/cpu/lp_norm_kernel.cc:10-157).          */
/* Tensors are T[N, C, S], reduction along C (element stride S):             */
/*   l1  norm = max(sum|x| / normalizer, epsilon)                            */
/*   l2  norm = max(sqrt(sum x^2 / normalizer), epsilon)                     */
/*   y = x / norm;  dx = dy / norm - g(x) * (sum(dy*x) / normalizer) / norm^(p+1) */
/* with g = sign for l1 and identity for l2. normalizer is C for the "MEAN"  */
/* reduction and 1 for "SUM" (lp_norm_op.cc:14-35). y may alias x and dx may  */
/* alias dy. 16-bit I/O accumulates in fp32.                                 */
/* ------------------------------------------------------------------------ */
int dragon_hip_l1_norm(int dtype, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                       const void* x, void* y, void* stream);
int dragon_hip_l2_norm(int dtype, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                       const void* x, void* y, void* stream);
int dragon_hip_l1_norm_grad(int dtype, int64_t N, int64_t S, int64_t C, float normalizer,
                            float epsilon, const void* dy, const void* x, void* dx, void* stream);
int dragon_hip_l2_norm_grad(int dtype, int64_t N, int64_t S, int64_t C, float normalizer,
                            float epsilon, const void* dy, const void* x, void* dx, void* stream);

/* ------------------------------------------------------------------------ */
/* Softmax cross-entropy loss, dragon/kernels/loss/op_kernels.h              */
/* (CPU dragon/kernels/loss/cpu/cross_entropy_kernel.cc,                     */
/* generic_loss_kernel.cc). dtype is F32 or F64 (dtypes::Loss,               */
/* dragon/core/types.h:90); target_dtype is I32 or I64. A target outside     */
/* [0, C) other than ignore_index is treated as ignored.                     */
/* ------------------------------------------------------------------------ */

/* CrossEntropy, dense targets (op_kernels.h:51-57; cpu :10-15):
 * loss[i] = -target[i] * log(max(input[i], FLT_MIN)). */
int dragon_hip_cross_entropy(int dtype, int64_t N, const void* input, const void* target,
                             void* loss, void* stream);

/* CrossEntropy, class-index targets over input T[N, C, S] (op_kernels.h:59-69;
 * cpu :17-42): per (n, s) loss = -log(max(input[n, target, s], FLT_MIN)) and
 * mask = 1, or loss = mask = 0 where target == ignore_index. loss, mask: T[N*S]. */
int dragon_hip_sparse_cross_entropy(int dtype, int target_dtype, int64_t N, int64_t S, int64_t C,
                                    int64_t ignore_index, const void* input, const void* target,
                                    void* loss, void* mask, void* stream);

/* SoftmaxCrossEntropyGrad (op_kernels.h:179-189; cpu :80-108): dx holds a copy
 * of the probabilities on entry; subtracts 1 at the target class, or clears
 * the whole class axis where the target is ignored; writes mask T[N*S]. */
int dragon_hip_softmax_cross_entropy_grad(int dtype, int target_dtype, int64_t N, int64_t S,
                                          int64_t C, int64_t ignore_index, const void* input,
                                          const void* target, void* dx, void* mask, void* stream);

/* ReduceLoss / ReduceLossGrad (op_kernels.h:95-113; generic_loss_kernel.cc:31-60):
 *   inv_scale = sum(mask[0, num_masks)) if num_masks > 0 and normalizer < 0, else normalizer
 *   ReduceLoss      y[0] = sum(x[0, N)) * (1 / max(inv_scale, 1))
 *   ReduceLossGrad  dx[0, N) *= dl[0] / max(inv_scale, 0.5)
 * Scratch: dragon_hip_reduce_loss_scratch_bytes(dtype). */
size_t dragon_hip_reduce_loss_scratch_bytes(int dtype);
int dragon_hip_reduce_loss(int dtype, int64_t N, int64_t num_masks, float normalizer,
                           const void* x, const void* mask, void* y, void* scratch,
                           size_t scratch_bytes, void* stream);
int dragon_hip_reduce_loss_grad(int dtype, int64_t N, int64_t num_masks, float normalizer,
                                const void* dl, const void* mask, void* dx, void* scratch,
                                size_t scratch_bytes, void* stream);

/* BroadcastLossGrad (op_kernels.h:25-32; generic_loss_kernel.cc:10-25):
 * dx[n, c, s] *= dl[n, s]. */
int dragon_hip_broadcast_loss_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dl,
                                   void* dx, void* stream);

/* SoftmaxCrossEntropyLossOp / ...GradientOp bodies for class-index targets
 * (dragon/operators/loss/cross_entropy_softmax_loss_op.cc:8-143) as one call
 * each. reduction: 0 NONE, 1 SUM, 2 MEAN, 3 BATCH_MEAN, 4 VALID.
 *   forward   prob = softmax(x) (the op's "X_norm"), loss = T[N*S] for NONE,
 *             else the reduced scalar T[1]
 *   backward  dx = (prob - onehot(target)) * w, w = 0 at ignored positions,
 *             dl[n, s] for NONE, else dl[0] / max(normalizer or valid count, 0.5)
 * Scratch: forward dragon_hip_softmax_cross_entropy_loss_scratch_bytes(dtype, N, S, C),
 * backward dragon_hip_reduce_loss_scratch_bytes(dtype). */
size_t dragon_hip_softmax_cross_entropy_loss_scratch_bytes(int dtype, int64_t N, int64_t S,
                                                           int64_t C);
int dragon_hip_softmax_cross_entropy_loss_forward(int dtype, int target_dtype, int64_t N, int64_t S,
                                                  int64_t C, int64_t ignore_index, int reduction,
                                                  const void* x, const void* target, void* prob,
                                                  void* loss, void* scratch, size_t scratch_bytes,
                                                  void* stream);
int dragon_hip_softmax_cross_entropy_loss_backward(int dtype, int target_dtype, int64_t N,
                                                   int64_t S, int64_t C, int64_t ignore_index,
                                                   int reduction, const void* prob,
                                                   const void* target, const void* dl, void* dx,
                                                   void* scratch, size_t scratch_bytes,
                                                   void* stream);

/* ------------------------------------------------------------------------ */
/* Operator-level fused entry points: one call for a kernel sequence that a  */
/* Dragon operator body issues back to back, so that x is read once where    */
/* the chip can hold the reduction unit on-die. Results equal the sequence.  */
/* ------------------------------------------------------------------------ */

/* GroupNormOp body, dragon/operators/normalization/group_norm_op.cc:26-51:
 * Moments -> InvStd -> GroupNorm. Writes mu, rsig (AccT[N*G]) and y. */
size_t dragon_hip_group_norm_forward_scratch_bytes(int dtype, int64_t N, int64_t G, int64_t D,
                                                   int64_t S, int layout);
int dragon_hip_group_norm_forward(int dtype, int64_t N, int64_t G, int64_t D, int64_t S,
                                  int layout, float eps, const void* x, const void* gamma,
                                  const void* beta, void* mu, void* rsig, void* y,
                                  void* scratch, size_t scratch_bytes, void* stream);

/* BatchNormOp::RunTraining body without sync,
 * dragon/operators/normalization/batch_norm_op.cc:49-82: Moments -> Axpby x2
 * (running statistics, biased variance, y = (1-momentum)*stat + momentum*y)
 * -> InvStd -> BatchNorm. Writes mu, rsig (AccT[C]), params (AccT[2C] =
 * {scale, bias}), y, and updates running_mean / running_var in place. */
int dragon_hip_batch_norm_training_forward(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                           float momentum, float eps, const void* x,
                                           const void* gamma, const void* beta,
                                           void* running_mean, void* running_var, void* mu,
                                           void* rsig, void* params, void* y, void* scratch,
                                           size_t scratch_bytes, void* stream);

/* BatchNormGradientOp::RunTraining body without sync,
 * dragon/operators/normalization/batch_norm_op.cc:118-190: BatchNormWGrad ->
 * BatchNormTrainingGrad in one call, so that x and dy are read once where a
 * channel slice fits the registers. Writes dgamma, dbeta (AccT[C]; dgamma ==
 * dbeta means dbeta = dgamma + C) and dx.
 * Scratch size: dragon_hip_batch_norm_reduce_scratch_bytes. */
int dragon_hip_batch_norm_training_backward(int dtype, int64_t N, int64_t C, int64_t S,
                                            float normalizer, int layout, const void* x,
                                            const void* mu, const void* rsig, const void* gamma,
                                            const void* dy, void* dgamma, void* dbeta, void* dx,
                                            void* scratch, size_t scratch_bytes, void* stream);

/* dragon_hip_batch_norm_training_forward for callers that cannot allocate
 * device memory and have no workspace to pass: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc. No counterpart in the
 * reference, whose operators always take scratch from the context's workspace.
 * Same arguments without the scratch pair, same kernels, same results; the
 * scratch is a static device array of DRAGON_HIP_STATIC_SCRATCH_BYTES inside
 * the library (each device that runs the library holds it until the process
 * ends). Shapes for which dragon_hip_batch_norm_reduce_scratch_bytes() exceeds
 * that return DRAGON_HIP_ELIMIT and enqueue nothing. The call allocates and
 * frees nothing on the device. All calls on one device share the one array:
 * two calls that overlap in time on one device (different streams or threads)
 * race on it and must be ordered by the caller. */
#define DRAGON_HIP_STATIC_SCRATCH_BYTES (4u << 20)
int dragon_hip_batch_norm_training_forward_noalloc(int dtype, int64_t N, int64_t C, int64_t S,
                                                   int layout, float momentum, float eps,
                                                   const void* x, const void* gamma,
                                                   const void* beta, void* running_mean,
                                                   void* running_var, void* mu, void* rsig,
                                                   void* params, void* y, void* stream);

/* The single-read paths (BatchNorm training forward / backward on NCHW with S
 * a whole number of 16-byte packets, GroupNorm groups beyond one workgroup,
 * softmax rows of many thousands of packets when scratch is passed) keep the
 * slices of a reduction unit in the registers of several workgroups, which
 * exchange partial results inside one kernel and wait for each other. The wait
 * is bounded; a workgroup whose wait runs out writes nothing for its slice and
 * flags it in the call's scratch, and a second launch enqueued behind the first
 * finishes every flagged slice, so the outputs of a call are always complete
 * in stream order and no status is sticky. A wait can only run out when other
 * work keeps part of the grid off the device (e.g. a second such kernel on
 * another stream); the call is then correct but slow. No counterpart in the
 * reference.
 * dragon_hip_exchange_timed_out: how many slices of the current device had to
 * be finished that way since the last reset (a diagnostic; copies one word from
 * the device, so it waits for the null stream). Synchronise the streams of
 * interest first.
 * (The count is cleared, and the length of the wait set, by the test hook
 * dragon_hip_exchange_reset, declared apart in dragon_hip_testing.h.)
 * dragon_hip_exchange_plan: how the path would cut `units` reduction units,
 * each `nseg` runs of `seglen` contiguous elements, with `tensors` (1 or 2)
 * tensors held in registers: returns 1 and fills slices (per unit),
 * slice_packets (16-byte packets per slice), packets_per_thread and grid (the
 * workgroups it asks for; a unit never has more slices than that), or returns
 * 0 when the shape is left to the split path. */
int dragon_hip_exchange_timed_out(void);
int dragon_hip_exchange_plan(int dtype, int64_t units, int64_t nseg, int64_t seglen, int tensors,
                             int* slices, int* slice_packets, int* packets_per_thread, int* grid);

/* dragon_hip_group_norm_grad with a phase clock: where the call takes the persistent row
 * kernel of the LayerNorm backward (G = S = 1, rows of up to 16384 elements that are not
 * short), every workgroup of that kernel leaves six 64-bit words in `stamps` (device memory
 * with room for `workgroups` workgroups, zero-filled by the caller; workgroup b writes words
 * 6b .. 6b+5): the device's 100 MHz clock at its start, when its first row had arrived and
 * been summed, when its row loop ended, and at its end; then the XCD it ran on and the rows
 * its first row group handled. Other paths, or too few `workgroups`, record nothing.
 * No counterpart in the reference; it is how the benchmark shows where the microseconds of
 * this kernel go (first loads, row loop, partial row) and how evenly the dies finish. */
int dragon_hip_group_norm_grad_timeline(int dtype, int64_t N, int64_t G, int64_t D, int64_t S,
                                        int layout, const void* x, const void* mu, const void* rsig,
                                        const void* gamma, const void* dy, void* ds, void* db,
                                        void* dgamma, void* dbeta, void* dx, void* scratch,
                                        size_t scratch_bytes, void* stamps, size_t workgroups,
                                        void* stream);

/* dragon_hip_plan_name: which kernels an entry point would launch for a shape,
 * as text "flavour:kernel[threads];kernel[threads];..." in launch order (a
 * "key=value:" item in front of a kernel is a number its plan depends on). No
 * counterpart in the reference; it is for tests that pin the routing of a
 * shape without a GPU: the entry point itself runs in a plan-only mode that
 * launches nothing and touches no device, with every tensor assumed 16-byte
 * aligned and not in place, and scratch assumed large enough.
 * `op` is the entry point's name without the prefix: "layer_norm",
 * "layer_norm_grad" (group_norm_grad with G = S = 1), "group_norm_forward",
 * "group_norm_grad", "batch_norm_training_forward", "batch_norm_training_backward",
 * "softmax", "log_softmax", "softmax_grad", "log_softmax_grad", "l1_norm",
 * "l2_norm", "l1_norm_grad", "l2_norm_grad", "softmax_cross_entropy_loss_forward",
 * "softmax_cross_entropy_loss_backward" (int64 targets, VALID reduction).
 * `dims` holds the entry point's sizes in its own order: (N, C) for the two
 * LayerNorm ops, (N, G, D, S) for GroupNorm, (N, C, S) for BatchNorm, (N, S, C)
 * for the rest; `layout` matters where the entry point takes one.
 * Returns the length of the text written to `buf` (truncated to buf_bytes - 1),
 * or a negative dragon_hip_status for an unknown op or a shape the entry point
 * rejects. Counts that depend on the device (the grid of a persistent kernel,
 * slices per unit) are those of an MI355X when no device is visible. */
int dragon_hip_plan_name(const char* op, int dtype, int layout, const int64_t* dims, int num_dims,
                         char* buf, size_t buf_bytes);

/* ------------------------------------------------------------------------ */
/* Measurement utility (no counterpart in the reference): a streaming read    */
/* (mode 0: dst receives at most one word), copy (mode 1), fill (mode 2) or    */
/* two reads and one write (mode 3: src holds two tensors of `bytes` bytes     */
/* back to back, dst their xor) of `bytes` bytes (a multiple of 16, 16-byte    */
/* aligned buffers) with 128-bit accesses, several in flight per thread.       */
/* Gives the achieved streaming ceiling of the device at the read : write      */
/* mixes of the kernels here, and a known-size kernel for calibrating          */
/* profiler byte counters.                                                     */
/* ------------------------------------------------------------------------ */
int dragon_hip_stream_probe(int mode, const void* src, void* dst, size_t bytes, void* stream);
/* The same with the probe's shape chosen by the caller: `threads` per workgroup and
 * 16-byte loads `in_flight` per thread, one of (64, 1|2|4), (256, 1|2|4|8), (512, 2),
 * (1024, 2); dragon_hip_stream_probe is (256, 4). Which shape streams fastest depends on
 * the tensor size, so a benchmark that wants a ceiling for a kernel takes the best of them
 * at that kernel's tensor size. */
int dragon_hip_stream_probe_shape(int mode, int threads, int in_flight, const void* src, void* dst,
                                  size_t bytes, void* stream);
/* Two reads and one write (mode 3 above) streamed the way a *persistent* kernel does it:
 * `per_cu` workgroups of `threads` threads per compute unit walk chunks of
 * threads x in_flight packets with a grid stride, `depth` (0 .. 3) chunks requested ahead
 * into registers; `barrier` adds a workgroup barrier per chunk, as a row reduction has;
 * `store_waves` lets the second half of each workgroup do nothing but write out what the
 * first half leaves in LDS (then threads / 2 load). Shapes: threads 256, 512 or 1024,
 * in_flight 1 or 2. It measures what the structure of the kernels that must be persistent
 * (those that carry per-column sums across rows) costs against the one-chunk-per-workgroup
 * probes. */
int dragon_hip_stream_probe_persistent(int threads, int in_flight, int per_cu, int depth, int barrier,
                                       int store_waves, const void* src, void* dst, size_t bytes,
                                       void* stream);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* DRAGON_HIP_H_ */
