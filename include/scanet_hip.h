/*
 * scanet_hip.h -- C ABI of the MI355X (gfx950) execution backend for scanet's
 * compiled training / inference step.
 *
 * The library replaces what scanet3 reaches through TensorFlow-Java: graph
 * construction + Session.run for the step that `Optimizer.compileBackprop`
 * builds, the forward/loss functions, and the parameter averaging of
 * `Optimizer.aggregateParams`.  Every entry point notes the reference
 * interface it stands in for (paths under src/main/scala/scanet/).
 *
 * Conventions
 *   - every function returns 0 on success, a negative SN_E_* code on failure;
 *     sn_last_error() gives the message of the calling thread's last failure
 *     (the reference turns a TF status into an exception, native/package.scala:6-10);
 *   - handles are owned by the caller and must be destroyed by it;
 *   - a context, and everything created from it, is used by one host thread at
 *     a time (the reference hands a Session to one thread at a time,
 *     core/Session.scala:147-166); different contexts may run concurrently;
 *   - all work of a context is issued on that context's HIP stream; calls that
 *     return host values (a loss, a count, a d2h copy) wait for the stream,
 *     the others are asynchronous and ordered;
 *   - pointers named *_dev are device addresses (from sn_buffer_alloc or any
 *     other HIP allocation on the context's device), pointers named *_host are
 *     ordinary host memory;
 *   - tensors are dense, row-major float32; images are NHWC
 *     (core/TensorType.scala:170-174, math/nn/AllKernels.scala:129-133).
 */
#ifndef SCANET_HIP_H
#define SCANET_HIP_H

#include <stddef.h>
#include <stdint.h>

/* Every function below is exported; nothing else in the library is. */
#if defined(__GNUC__) || defined(__clang__)
#define SN_API __attribute__((visibility("default")))
#else
#define SN_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef struct sn_ctx sn_ctx;
typedef struct sn_model sn_model;
typedef struct sn_replica sn_replica;

enum {
  SN_OK = 0,
  SN_E_INVALID = -1,     /* bad argument / unsupported combination (reference: require(..) failures) */
  SN_E_HIP = -2,         /* a HIP runtime call failed */
  SN_E_OOM = -3,         /* device or host allocation failed */
  SN_E_STATE = -4        /* object used after destroy / wrong context */
};

/* ---- layer list (the layers under models/layer/, flattened as layer/Composed.scala:89-99 does) ---- */
enum { SN_LAYER_DENSE = 0, SN_LAYER_BIAS = 1, SN_LAYER_ACTIVATE = 2, SN_LAYER_FLATTEN = 3,
       SN_LAYER_CONV2D = 4, SN_LAYER_POOL2D = 5, SN_LAYER_LSTM = 6, SN_LAYER_SIMPLE_RNN = 7, SN_LAYER_BATCHNORM = 8 };
/* models/Activation.scala:32-83 */
enum { SN_ACT_IDENTITY = 0, SN_ACT_SIGMOID = 1, SN_ACT_TANH = 2, SN_ACT_RELU = 3, SN_ACT_SOFTMAX = 4 };
/* models/Loss.scala:18-57 */
enum { SN_LOSS_IDENTITY = 0, SN_LOSS_MSE = 1, SN_LOSS_BINARY_CROSSENTROPY = 2, SN_LOSS_CATEGORICAL_CROSSENTROPY = 3 };
/* math/nn/AllKernels.scala:25-103 */
/* `Reduce` of `pool2D` (math/nn/AllKernels.scala:383-397).  The reference's Pool2D LAYER never hands its `reduce` to
 * the kernel (layer/Pool2D.scala:36-42), so every model it builds max-pools; a binding that mirrors the layer as it is
 * passes SN_POOL_MAX whatever the layer says, one that mirrors the kernel function passes the argument through. */
enum { SN_POOL_MAX = 0, SN_POOL_AVG = 1 };
enum { SN_PAD_VALID = 0, SN_PAD_SAME = 1, SN_PAD_EXPLICIT = 2 /* Conv2D only: pad_top .. pad_right below */ };
/* models/Regularization.scala:16-44 */
enum { SN_REG_NONE = 0, SN_REG_L1 = 1, SN_REG_L2 = 2 };
/* optimizers/{SGD,AdaGrad,AdaDelta,RMSProp,Adam,Nadam,Adamax,AMSGrad}.scala */
enum { SN_OPT_SGD = 0, SN_OPT_ADAGRAD = 1, SN_OPT_ADADELTA = 2, SN_OPT_RMSPROP = 3,
       SN_OPT_ADAM = 4, SN_OPT_NADAM = 5, SN_OPT_ADAMAX = 6, SN_OPT_AMSGRAD = 7 };
/* math/rand/AllKernels.scala:45-50 (Dist) */
enum { SN_RANDOM_UNIFORM = 0, SN_RANDOM_NORMAL = 1, SN_RANDOM_TRUNCATED_NORMAL = 2 };
/* error terms of the regression estimators (estimators/package.scala:56-70) */
enum { SN_ERROR_SQUARED = 0, SN_ERROR_ABSOLUTE = 1 };
/* model flags */
enum {
  SN_FLAG_GEMM_BF16 = 1,       /* Dense GEMMs take bf16 inputs (fp32 accumulate, fp32 master weights) */
  SN_FLAG_STABLE_SOFTMAX = 2   /* subtract the row maximum before exp (the reference does not, Activation.scala:63-69) */
};

/* One entry of the flattened layer list.  `Dense(n, act)` of the reference is the
 * three entries DENSE, BIAS, ACTIVATE (layer/Dense.scala:30-40), `Conv2D(..)` is
 * CONV2D [, BIAS] [, ACTIVATE] (layer/Conv2D.scala:54-68); parameter paths are
 * "<index in this list>/weights" exactly as Composed.params builds them. */
typedef struct sn_layer_desc {
  int32_t kind;          /* SN_LAYER_* */
  int32_t units;         /* Dense outputs / Bias features / Conv2D filters / LSTM or SimpleRNN units */
  int32_t activation;    /* ACTIVATE: SN_ACT_*  (LSTM: cell activation, must be SN_ACT_TANH; SIMPLE_RNN: the cell's
                            activation, layer/RNN.scala:115,162) */
  float act_param;       /* ReLU threshold (Activation.scala:79-82) */
  int32_t kernel_h, kernel_w;   /* Conv2D kernel / Pool2D window */
  int32_t stride_h, stride_w;
  int32_t padding;       /* SN_PAD_* */
  int32_t reg_kind;      /* Dense/Bias: SN_REG_*; LSTM / SIMPLE_RNN: `kernelReg`; BATCHNORM: `betaRegularizer` (the reference adds
                            betaRegularizer(gamma) twice and never uses gammaRegularizer, layer/BatchNorm.scala:158-160; the library
                            does the same).  Bias and BatchNorm penalties count only while the model is trainable: sn_loss, the
                            frozen model's loss, leaves them out (layer/Bias.scala:35-36) */
  float reg_lambda;
  int32_t use_bias;      /* LSTM: per-gate bias vectors (layer/RNN.scala:215); SIMPLE_RNN: the cell's Bias (RNN.scala:116) */
  int32_t return_sequence; /* LSTM / SIMPLE_RNN: `returnSequence` (layer/RNN.scala:27,74-77): the output is every step's
                              output, (batch, time, units), instead of the last one */
  float bn_momentum;     /* BATCHNORM (layer/BatchNorm.scala:64-76, axes = Seq(-1)): decay of the moving statistics */
  float bn_epsilon;      /* BATCHNORM: added to the variance */
  int32_t pad_top, pad_bottom, pad_left, pad_right; /* CONV2D with SN_PAD_EXPLICIT: `Explicit((top, bottom), (left, right))`,
                            output size ceil((in + pads - window) / stride) + 1 (math/nn/AllKernels.scala:67-91) */
  int32_t bn_fused;      /* BATCHNORM: `fused` of the reference: -1 None, 0 Some(false), 1 Some(true).  As in the reference
                            (layer/BatchNorm.scala:98-133) rank-4 input takes the FusedBatchNormV3 branch unless fused =
                            Some(false), every other rank the generic form (math/nn/AllKernels.scala:663-684), and
                            Some(true) with another rank fails.  The fused branch is built AS THE REFERENCE WIRES THE
                            OP'S OUTPUTS (math/nn/AllKernels.scala:437-448): same output as the generic form, but the
                            moving variance follows the batch mean and the gradient op receives the unbiased batch
                            variance as its mean and the batch mean as its variance. */
  int32_t recurrent_reg_kind;   /* LSTM / SIMPLE_RNN: `recurrentReg` and `biasReg` (layer/RNN.scala:120-122,233-235) */
  float recurrent_reg_lambda;
  int32_t bias_reg_kind;
  float bias_reg_lambda;
  int32_t pool_reduce;   /* POOL2D: SN_POOL_*.  AVG divides by the number of window cells inside the input (TF AvgPool) */
  int32_t stateful;      /* LSTM / SIMPLE_RNN: `stateful` (layer/RNN.scala:27,34,66-67): the state the last time step leaves
                            (LSTM "cell_state" and "hidden_state", simple cell "0/state"; (batch, units), zeros at first) is a
                            non-trainable parameter that the next sn_step starts from; sn_replicas_average re-initialises it */
} sn_layer_desc;

/* An `Algorithm` case class (optimizers/Algorithm.scala:6-11).  Field use per kind:
 *   SGD      rate, beta1 = momentum, nesterov
 *   AdaGrad  rate, epsilon
 *   AdaDelta rate, beta1 = rho, epsilon
 *   RMSProp  rate, beta1 = rho, epsilon
 *   Adam / AMSGrad  rate, beta1, beta2, epsilon
 *   Nadam    beta1, beta2, epsilon, init_acc
 *   Adamax   rate, beta1, beta2, epsilon, init_acc                              */
typedef struct sn_optimizer_desc {
  int32_t kind;          /* SN_OPT_* */
  float rate;
  float beta1;
  float beta2;
  float epsilon;
  float init_acc;        /* initial value of every state tensor (Nadam.scala:26-35, Adamax.scala:30-39) */
  int32_t nesterov;
  int32_t maximize;      /* 0: w' = w - delta (`Optimizer.minimize`); 1: w' = w + delta (`Optimizer.maximize`,
                            optimizers/Optimizer.scala:186,326-336) */
} sn_optimizer_desc;

#define SN_MAX_RANK 8
#define SN_MAX_OPT_STATES 3
#define SN_MAX_AVG_INPUTS 32

/* One parameter tensor of a model, in flat-buffer order. */
typedef struct sn_param_info {
  char path[96];                 /* reference path, e.g. "0/weights", "0/forget/0/kernel_weights" */
  int64_t offset;                /* first element inside the replica's flat parameter buffer */
  int64_t size;                  /* number of elements */
  int32_t rank;
  int64_t dims[SN_MAX_RANK];
  int32_t trainable;             /* 0: layer state (BatchNorm moving statistics, `ParamDef.trainable = false`): no gradient,
                                    no optimizer state; the step replaces it with the layer's own update
                                    (optimizers/Optimizer.scala:118-122,142-144) */
  int32_t aggregated;            /* `ParamDef.aggregation`: 1 Some(Avg), averaged by sn_replicas_average; 0 None (the carried
                                    state of a stateful RNN), re-initialised to zeros there (Optimizer.scala:205-210) */
} sn_param_info;

/* ---------------------------------------------------------------- context / errors */

/* Replaces `new Session()` = Graph + TF Session (core/Session.scala:57-63).
 * `stream` is a hipStream_t to issue all work on, or NULL to let the context
 * create (and own) one. */
SN_API int sn_ctx_create(int device, void* stream, sn_ctx** out);
/* Replaces Session.close (core/Session.scala:106). Waits for outstanding work. */
SN_API int sn_ctx_destroy(sn_ctx* ctx);
/* Message of the calling thread's most recent failing call (never NULL). */
SN_API const char* sn_last_error(void);
/* Blocks until everything issued on the context's stream has finished.
 * Like every call that synchronises the compute stream and hands results back (sn_copy_d2h, sn_params_get /
 * sn_optstate_get / sn_grads_get, sn_count_correct, sn_error_sum, sn_train_epoch_host, the profile readers, a step or
 * gradient call that returns its loss), it returns SN_E_STATE once if a recurrent layer's one-launch forward or backward kernel gave up waiting for its neighbour workgroups
 * since the previous synchronisation (only possible when something else occupies compute units of the same GPU):
 * the results computed since then are invalid, the context stays usable and from then on runs recurrent layers with one
 * launch per time step.  The optimizer update of a training step whose passes gave up does not run: weights and
 * optimizer state keep the values they had before that step (and before every later step until the error is
 * reported); a stateful recurrent layer's carried state is undefined after such a step.  The wait is a bounded number of polls
 * (environment variable SCANET_SEQUENCE_SPIN_LIMIT, default 2000000, 0 = give up at the first wait; read when a context first launches that
 * kernel; SCANET_SEQUENCE_COHERENT=1 makes the kernel hand its state over with device-coherent accesses even
 * between workgroups of one XCD). */
SN_API int sn_sync(sn_ctx* ctx);
/* Name, HBM bytes and compute-unit count of the context's device
 * (reference: core/Devices.scala:23-37 lists TF devices). */
SN_API int sn_device_info(sn_ctx* ctx, char* name, int name_cap, int64_t* hbm_bytes, int32_t* compute_units);

/* ---------------------------------------------------------------- tensors / memory */

/* Replaces TF_AllocateTensor / TF_DeleteTensor (native/RawTensors.scala:81-88,106-115)
 * for device-resident tensors. */
SN_API int sn_buffer_alloc(sn_ctx* ctx, size_t bytes, void** out_dev);
SN_API int sn_buffer_free(sn_ctx* ctx, void* dev);
/* Pinned host memory a JVM can wrap as a read-only DirectBuffer
 * (native/RawTensors.scala:24-30, core/TensorCodec.scala:12-22). */
SN_API int sn_host_alloc(sn_ctx* ctx, size_t bytes, void** out_host);
SN_API int sn_host_free(sn_ctx* ctx, void* host);
/* Replaces the feed / fetch halves of Session.Runner (core/Session.scala:83-95).
 * h2d is asynchronous when src is pinned; d2h returns after the data has arrived. */
SN_API int sn_copy_h2d(sn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
SN_API int sn_copy_d2h(sn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);
SN_API int sn_fill(sn_ctx* ctx, float* dst_dev, float value, int64_t n);

/* ---------------------------------------------------------------- model = compiled step */

/* Replaces building `model.withLoss(loss)` and compiling its functions
 * (models/Model.scala:84-119, optimizers/Optimizer.scala:163-194, core/TF.scala:391-438).
 * `input_dims` is the shape of ONE sample (e.g. {784}, {28,28,1}, {64,32}); `batch`
 * is the largest number of rows any call will pass. */
SN_API int sn_model_create(sn_ctx* ctx, const sn_layer_desc* layers, int32_t n_layers, int32_t loss,
                    const int64_t* input_dims, int32_t input_rank, int32_t batch, uint32_t flags,
                    sn_model** out);
SN_API int sn_model_destroy(sn_model* model);
/* `model.params(input)` restricted to trainable weights (models/Model.scala:18;
 * optimizers/Optimizer.scala:117-122), in flat-buffer order. */
SN_API int sn_model_param_count(sn_model* model, int32_t* n_tensors, int64_t* flat_elems);
SN_API int sn_model_param_info(sn_model* model, int32_t index, sn_param_info* out);
/* `model.outputShape(input)` for one sample (models/Model.scala:41). */
SN_API int sn_model_output_shape(sn_model* model, int32_t* rank, int64_t* dims);

/* ---------------------------------------------------------------- replica = params + optimizer state */

/* One partition's training state: the flat weight, gradient and optimizer-state
 * buffers that optimizeOnPartition threads through its loop
 * (optimizers/Optimizer.scala:117-131). Weights start at zero, optimizer state at
 * `opt->init_acc` (ParamDef.initialize). `opt` may be NULL for inference only. */
SN_API int sn_replica_create(sn_model* model, const sn_optimizer_desc* opt, sn_replica** out);
SN_API int sn_replica_destroy(sn_replica* rep);
/* `.initParams(Params)` / reading `TrainedModel.params` (optimizers/Optimizer.scala:276-277,103). */
SN_API int sn_params_set(sn_replica* rep, int32_t index, const float* src_host, int64_t n);
SN_API int sn_params_get(sn_replica* rep, int32_t index, float* dst_host, int64_t n);
/* Optimizer state tensor `<path>/<state name>` (optimizers/Optimizer.scala:118-121); slot order is
 * the order of the algorithm's `params` (e.g. Adam: 0 momentum, 1 velocity). */
SN_API int sn_optstate_set(sn_replica* rep, int32_t index, int32_t slot, const float* src_host, int64_t n);
SN_API int sn_optstate_get(sn_replica* rep, int32_t index, int32_t slot, float* dst_host, int64_t n);
/* Gradient of the last sn_step / sn_grad for one tensor (`LossModel.grad`, models/Model.scala:107-111). */
SN_API int sn_grads_get(sn_replica* rep, int32_t index, float* dst_host, int64_t n);
/* Device views of the flat buffers: slot -2 weights, -1 gradients, 0.. optimizer state tensors. */
SN_API int sn_replica_flat(sn_replica* rep, int32_t slot, float** out_dev, int64_t* n);

/* One call of the compiled backprop function (optimizers/Optimizer.scala:142-143, 169-194):
 * forward, loss, gradients of every weight, optimizer update w' = w - delta with iteration
 * number `iter` (1-based). `rows` <= batch. If `loss_host` is not NULL the loss of this batch
 * (before the update) is written there and the call waits for the device; with NULL the kernels that
 * only finish the loss value (its final reduction, the penalty terms) are not launched. */
SN_API int sn_step(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int32_t iter, float* loss_host);
/* `LossModel.grad` (models/Model.scala:107-111): gradients only, no update. */
SN_API int sn_grad(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, float* loss_host);
/* `model.result` (models/Model.scala:35-36) of the frozen model, the one `LossModel.trained` hands to
 * `TrainedModel` (Model.scala:126-127): out_dev receives rows x output elements.  BatchNorm reads its
 * moving statistics. */
SN_API int sn_forward(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev);
/* Output of `model.resultStateful` (models/Model.scala:38-41) for the model as the optimizer compiles it:
 * BatchNorm normalises with the statistics of these `rows`.  The next state it would return is not applied;
 * only sn_step and the epoch calls move layer state. */
SN_API int sn_forward_training(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev);
/* sn_forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  What is tested is that the call leaves
 * the device's free memory unchanged; recording it into a graph is not.  Same result as sn_forward, but every
 * intermediate of the pass (layer outputs, pooling offsets, BatchNorm vectors, the GEMM workspace) lives in one
 * 64 MiB device array that is part of the library image (each GPU the library runs on holds its copy until the
 * process ends), and the call makes no hipMalloc / hipFree.  Fails with SN_E_INVALID when `rows` of this model need
 * more than 64 MiB, for models with recurrent layers and for SN_FLAG_GEMM_BF16.  Per-kernel timing is off inside the
 * call.  All calls on one GPU share the array: calls that overlap on one GPU (two contexts, two streams) race. */
SN_API int sn_forward_static(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev);
/* `LossModel.loss` (models/Model.scala:101-102) of the frozen model. */
SN_API int sn_loss(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, float* loss_host);
/* Per-batch body of `estimators.accuracy` (estimators/package.scala:28-32): rows whose every
 * rounded (half to even) output equals the label. */
SN_API int sn_count_correct(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int64_t* count_host);
/* Per-batch body of `estimators.MSE` / `RMSE` / `MAE` (estimators/package.scala:50-101, `errorSum`): the sum over
 * every output element of (predicted - expected)^2 or |predicted - expected| for the frozen model; the caller
 * adds the sums of its batches and divides by the row count as the reference does. */
SN_API int sn_error_sum(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int32_t kind, float* sum_host);
/* `optimizeOnPartition` (optimizers/Optimizer.scala:106-161) over a device-resident partition of
 * `total_rows` samples: every full batch in order with iter = global_iter + i + 1, partial batch
 * skipped (optimizers/Iterators.scala:90), then the loss of the last batch under the updated
 * weights. Fails with SN_E_INVALID when the partition holds no full batch. */
SN_API int sn_train_epoch(sn_replica* rep, const float* x_dev, const float* y_dev, int64_t total_rows, int32_t batch,
                   int32_t global_iter, int32_t* iterations_host, float* loss_host);

/* The same epoch over a partition in HOST memory (best allocated with sn_host_alloc: pinned memory makes the copies
 * asynchronous): runs of consecutive batches (1, 2, 4, ... up to 32 MiB or 64 batches) are copied to the device on a
 * second stream while the run before trains.  Replaces the
 * TensorIterator -> feed path of optimizeOnPartition (optimizers/Iterators.scala:39-83, Optimizer.scala:136-157).
 * Results are those of sn_train_epoch on a device-resident copy of the same partition. */
SN_API int sn_train_epoch_host(sn_replica* rep, const float* x_host, const float* y_host, int64_t total_rows, int32_t batch,
                               int32_t global_iter, int32_t* iterations_host, float* loss_host);

/* `aggregateParams` (optimizers/Optimizer.scala:196-230) for K replicas of one model: weights and
 * every optimizer-state tensor become the uniform mean AddN(..)/K (models/Aggregation.scala:16-19)
 * and are written back to all K replicas (the next epoch's broadcast, Optimizer.scala:72-73); tensors
 * without an aggregation (the carried state of a stateful RNN, layer/RNN.scala:188,302-303) are
 * re-initialised to zeros in every replica (Optimizer.scala:207-210).
 * DEVIATION for K > 2: the reference only ever averages PAIRS -- Spark's treeReduce folds
 * avg2(l, r) = AddN(l, r) / 2 and (l.loss + r.loss) / 2 in an order Spark chooses, so three partitions
 * end up weighted 1/4, 1/4, 1/2 in arrival order.  K = 2 is the reference's avg2 bit for bit; for K > 2 this
 * call takes the uniform mean the build target names, no reference test runs more than one partition, and
 * parity is unpinned.  A caller that wants one particular pairwise fold calls sn_average with k = 2 on the
 * flat views (sn_replica_flat) in its own order. */
SN_API int sn_replicas_average(sn_replica* const* reps, int32_t k);

/* ---------------------------------------------------------------- flat kernels (the memory-bound pair) */

/* One fused `Algorithm.build` + `w - delta` over a flat vector (optimizers/Optimizer.scala:181-188):
 * w[i], state*[i] updated in place from g[i]. Unused state pointers may be NULL. */
SN_API int sn_optimizer_update(sn_ctx* ctx, const sn_optimizer_desc* opt, float* w_dev, const float* g_dev,
                        float* s0_dev, float* s1_dev, float* s2_dev, int64_t n, int32_t iter);
/* `Aggregation.Avg` over k inputs (models/Aggregation.scala:16-19): out = (in[0] + .. + in[k-1]) / k,
 * accumulated left to right. `inputs_host` is a host array of k device pointers; out may alias in[0]. */
SN_API int sn_average(sn_ctx* ctx, const float* const* inputs_host, int32_t k, int64_t n, float* out_dev);

/* `rand(shape, dist, seed, scale, shift)` (math/rand/AllKernels.scala:68-81), the draw under every seeded
 * initializer of models/Initializer.scala:48-219: n values of the TensorFlow op the reference lowers to
 * (RandomUniform in [0,1), RandomStandardNormal, TruncatedNormal at two standard deviations) for op seed
 * `seed` (non-zero), then `* scale` and `+ shift` where the pointers are not NULL. The stream is the one
 * TensorFlow's CPU kernels produce, so the same seed gives the reference's initial weights. */
SN_API int sn_random_fill(sn_ctx* ctx, float* dst_dev, int64_t n, int32_t dist, uint64_t seed, const float* scale_host,
                          const float* shift_host);

/* ---------------------------------------------------------------- per-kernel timing */

/* When enabled every kernel launch of the context is bracketed by HIP events on the context's
 * stream (the reference only has wall-clock per epoch, optimizers/Optimizer.scala:74,87-89). */
SN_API int sn_profile_enable(sn_ctx* ctx, int32_t on);
SN_API int sn_profile_reset(sn_ctx* ctx);
/* Number of distinct kernel names seen since the last reset (waits for the stream). */
SN_API int sn_profile_count(sn_ctx* ctx, int32_t* n);
SN_API int sn_profile_get(sn_ctx* ctx, int32_t index, char* name, int32_t name_cap, double* total_ms, int64_t* launches);

#ifdef __cplusplus
}
#endif
#endif /* SCANET_HIP_H */
