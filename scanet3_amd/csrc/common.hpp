// Internal declarations shared by the HIP translation units of libscanet_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/scanet_hip.h"

namespace sn {

// ---- error handling -------------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define SN_HIP(expr)                                                                         \
  do {                                                                                       \
    hipError_t e__ = (expr);                                                                 \
    if (e__ != hipSuccess) (void)hipGetLastError(); /* or the next launch check finds it */  \
    if (e__ != hipSuccess)                                                                   \
      return sn::fail(e__ == hipErrorOutOfMemory ? SN_E_OOM : SN_E_HIP, "%s failed: %s (%s:%d)", #expr, \
                      hipGetErrorString(e__), __FILE__, __LINE__);                           \
  } while (0)

#define SN_TRY(expr)           \
  do {                         \
    int r__ = (expr);          \
    if (r__ != SN_OK) return r__; \
  } while (0)

#define SN_REQUIRE(cond, ...)                                \
  do {                                                       \
    if (!(cond)) return sn::fail(SN_E_INVALID, __VA_ARGS__); \
  } while (0)

// ---- per-kernel timing ----------------------------------------------------------------
struct ProfileEntry {
  double total_ms = 0.0;
  int64_t launches = 0;
};

struct PendingEvent {
  hipEvent_t start, stop;
  std::string name;
};

}  // namespace sn

// The reduction of partial sums that a launcher left to its caller because sn_ctx::defer asked for it:
// dst[o] = sum over `parts` partial results partial[p * outs + o] (o < outs), added in the order of the kernel that would
// otherwise have run right away: kind 1 = splitk_reduce4_kernel's (eight interleaved chains, then a pairwise tree),
// kind 2 = gemm_small_reduce_kernel's (64 interleaved chains, then a chain).  The training step hands these to the
// launch that also applies the optimizer (launch_finish), so a filter gradient is summed and used in one pass.
struct DeferredReduce {
  int kind = 0;
  const float* partial = nullptr;
  int parts = 0, outs = 0;
  float* dst = nullptr;
};
constexpr int MAX_DEFERRED = 4, MAX_FINISH_HOLES = 4;

struct sn_ctx {
  uint32_t magic;
  int device;
  hipStream_t stream;
  bool owns_stream;
  int compute_units;
  int live_models = 0;  // models created from this context and not yet destroyed
  // Recurrent sequence kernels (one launch for all time steps): arrival counters of their row groups in device memory,
  // a word in pinned host memory that such a kernel sets when it gives up waiting for its neighbours, and how many
  // polls it waits before it does.  Allocated by the first launch that needs them.
  unsigned* seq_arrived = nullptr;
  int64_t seq_next = 0;            // first word of the area no launch has used since it was last cleared
  int* seq_gave_up = nullptr;      // host address
  int* seq_gave_up_dev = nullptr;  // the same word as the device sees it
  DeferredReduce* defer = nullptr;   // set by a caller that takes the next partial-sum reduction on itself (cleared by the launcher that fills it)
  int* seq_failed_dev = nullptr;   // device memory: set with it, read by the optimizer launch that follows a recurrent pass
  unsigned seq_spin_limit = 0;
  int seq_force_coherent = 0;      // hand over as if every row group were spread over several XCDs
  bool seq_disabled = false;       // a one-launch kernel gave up once: from then on the per-step kernels run
  // timing
  bool profiling;
  std::vector<sn::PendingEvent> pending;
  std::vector<hipEvent_t> event_pool;
  std::map<std::string, sn::ProfileEntry> profile;
  std::vector<std::string> profile_names;  // stable order for sn_profile_get
  // kernels whose dynamic-LDS limit has been raised on this context's device, with the size granted
  std::map<const void*, size_t> lds_limit;
};

namespace sn {

constexpr uint32_t CTX_MAGIC = 0x534e4358u;  // "SNCX"
constexpr uint32_t MODEL_MAGIC = 0x534e4d44u;
constexpr uint32_t REPLICA_MAGIC = 0x534e5250u;

// Brackets one kernel launch with events when the context is profiling.
struct LaunchScope {
  sn_ctx* ctx;
  hipEvent_t start = nullptr, stop = nullptr;
  std::string name;
  LaunchScope(sn_ctx* c, const char* n);
  LaunchScope(sn_ctx* c, const char* n, int m, int nn, int k);  // name becomes "n[MxNxK]"
  void begin();
  ~LaunchScope();
};
int profile_drain(sn_ctx* ctx);
// Hands a sequence-kernel launch its own all-zero block for `groups` row groups out of the context's area (set up on
// first use).  The area is cleared in one go whenever it has been used up, so a launch costs no fill of its own.
int seq_sync_take(sn_ctx* ctx, int groups, unsigned** block);
// Words of a context's sequence-kernel area: one block of SEQ_GROUP_WORDS per row group (arrival counter, XCD word,
// spread flag; a block of its own so that the pollers of different row groups do not meet on one cache line), then the
// abort word's block.
constexpr int SEQ_GROUP_WORDS = 64, SEQ_MAX_GROUPS = 1023, SEQ_COUNTERS = (SEQ_MAX_GROUPS + 1) * SEQ_GROUP_WORDS;
// After a stream synchronisation: SN_E_STATE (once) if a sequence kernel gave up waiting since the last check.
int check_async(sn_ctx* ctx);
// looks up this device's address of the library's static scratch array (model.hip); `device` must be current
int static_scratch_init(int device);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Kernels that use more than 64 KiB of dynamic LDS must have their limit raised once per device; remembered per context.
inline int allow_dynamic_lds(sn_ctx* ctx, const void* kernel, size_t bytes) {
  auto it = ctx->lds_limit.find(kernel);
  if (it != ctx->lds_limit.end() && it->second >= bytes) return SN_OK;
  SN_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  ctx->lds_limit[kernel] = bytes;
  return SN_OK;
}
inline int64_t align_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- optimizer / averaging kernels (optim_kernels.hip) ---------------------------------
// Scalars every algorithm needs, evaluated once per step on the host in float32.
struct OptScalars {
  float rate, b1, b2, eps;
  float one_minus_b1, one_minus_b2;  // `1f.const - beta` evaluated in float32
  float bc1, bc2;                    // 1 - beta^iter, the divisor of `boost`
  int nesterov;
  int maximize;                      // w + delta instead of w - delta (`Optimizer.maximize`, optimizers/Optimizer.scala:186)
};
OptScalars make_opt_scalars(const sn_optimizer_desc& d, int iter);
int opt_state_count(int kind);
// wbf (optional): the updated weights are also written as bf16, element for element
// skip_if (optional, device memory): the launch leaves everything as it is when *skip_if is not zero
int launch_optimizer(sn_ctx* ctx, const sn_optimizer_desc& d, float* w, const float* g, float* s0, float* s1, float* s2,
                     int64_t n, int iter, void* wbf = nullptr, const int* skip_if = nullptr);
// One launch that finishes a training step: the deferred reductions d[0..n_d) land in the gradient buffer g (their
// targets lie inside it), and every element of the flat buffers [0, n) gets its optimizer update, the reduced ones from
// the sums just made.  Same arithmetic and order as the reduction kernels followed by launch_optimizer.
// holes: n_holes pairs [first, end) of elements the update leaves alone (tensors that are not trainable)
int launch_finish(sn_ctx* ctx, const sn_optimizer_desc& d, float* w, float* g, float* s0, float* s1, float* s2, int64_t n, int iter,
                  const DeferredReduce* defs, int n_defs, const int* skip_if, const int64_t* holes = nullptr, int n_holes = 0);
// Runs a deferred reduction on its own (when no optimizer launch follows that could take it).
int launch_deferred_reduce(sn_ctx* ctx, const DeferredReduce& d);
struct AvgInputs {
  const float* p[SN_MAX_AVG_INPUTS];
};
int launch_average(sn_ctx* ctx, const AvgInputs& in, int k, int64_t n, float* out, float* const* extra_out, int n_extra);
int launch_fill(sn_ctx* ctx, float* dst, float v, int64_t n);

// ---- elementwise / row kernels (elementwise_kernels.hip) -------------------------------
int launch_bias_act(sn_ctx* ctx, const float* x, const float* bias, float* y, int64_t rows, int cols, int act, float act_param);
int launch_act_bwd(sn_ctx* ctx, const float* y, const float* dy, float* dx, int64_t n, int act, float act_param);
int launch_softmax_fwd(sn_ctx* ctx, const float* z, float* p, int rows, int cols, bool stable);
int launch_softmax_bwd(sn_ctx* ctx, const float* p, const float* dp, float* dz, int rows, int cols);
// loss value (sum of per-element terms / divisor) into *loss_dev and d loss / d p into dp (dp may be null)
// loss kinds beyond the public SN_LOSS_*: plain sums of the error terms the regression estimators use
constexpr int LOSS_SUM_SQUARED_ERROR = 100, LOSS_SUM_ABSOLUTE_ERROR = 101;
// loss_dev == nullptr: only dp is wanted (the per-block partial sums are still written, the final reduction is skipped)
int launch_loss(sn_ctx* ctx, int kind, const float* p, const float* y, float* dp, float* loss_dev, float* partials,
                int rows, int cols);
// training step of a Softmax output under CategoricalCrossentropy: p, loss value and dz in one kernel per row
// (row_loss: `rows` floats of scratch; loss_dev == nullptr: the loss value is not wanted, its final reduction is skipped)
// dz_bf (optional): bf16 [rows, cols], the same dz rounded to bf16 (what a bf16 Dense layer below would cast it to next)
// p may be null when nobody reads the probabilities and cols <= 1024 (rows held in registers)
int launch_softmax_cce(sn_ctx* ctx, const float* z, const float* y, float* p, float* dz, float* loss_dev, float* row_loss, int rows,
                       int cols, bool stable, void* dz_bf = nullptr);
// The same when the logits still lie as `parts` partial sums [part][rows * cols] of a Dense layer's forward product (at most
// SOFTMAX_PARTIALS_MAX_COLS columns): the kernel adds them in the order of that product's own reduction, adds the bias
// (may be null), writes the logits to z_out and goes on as launch_softmax_cce.
constexpr int SOFTMAX_PARTIALS_MAX_COLS = 16;
int launch_softmax_cce_partials(sn_ctx* ctx, const float* partial, int parts, const float* bias, float* z_out, const float* y, float* p,
                                float* dz, float* loss_dev, float* row_loss, int rows, int cols, bool stable);
// out[c] = sum over rows of dy[r*ld + c]; `ws` (optional) lets many rows be summed in parallel slices
int launch_col_sum(sn_ctx* ctx, const float* dy, int64_t ld, float* out, int64_t rows, int cols, float* ws, int64_t ws_elems);
// partials: at least 1024 floats of scratch
int launch_penalty(sn_ctx* ctx, const float* w, int64_t n, int reg_kind, float lambda, float* loss_dev, float* partials);
int launch_penalty_grad(sn_ctx* ctx, const float* w, float* g, int64_t n, int reg_kind, float lambda);
int launch_count_correct(sn_ctx* ctx, const float* p, const float* y, int rows, int cols, unsigned long long* count_dev);
int launch_pool_fwd(sn_ctx* ctx, bool avg, const float* x, float* y, uint8_t* arg, int n, int h, int w, int c, int ho, int wo,
                       int kh, int kw, int sh, int sw, int pt, int pl);
// y_in (optional): the pooled tensor when it is the output of a layer with activation `act`; the kernel then
// returns act'(y_in) * gradient, i.e. that layer's pre-activation gradient, saving a pass over the tensor
int launch_pool_bwd(sn_ctx* ctx, bool avg, const float* dy, const uint8_t* arg, float* dx, int n, int h, int w, int c, int ho,
                       int wo, int kh, int kw, int sh, int sw, int pt, int pl, const float* y_in = nullptr, int act = SN_ACT_IDENTITY,
                       float act_param = 0.f);
struct LstmGateArgs {
  const float* z;       // [rows, 4H] pre-activations incl. bias, gate order forget,input,gate,output
  const float* c_prev;  // [rows, H] or null (zeros)
  float* gates;         // [rows, 4H] activated f,i,g,o
  float* c;             // [rows, H]
  float* h;             // [rows, H]
};
int launch_lstm_gates_fwd(sn_ctx* ctx, const LstmGateArgs& a, int rows, int hidden);
struct LstmGateBwdArgs {
  const float* gates;   // activated f,i,g,o of this step
  const float* c;       // c_t
  const float* c_prev;  // c_{t-1} or null
  const float* dh;      // [rows,H]
  float* dc;            // [rows,H] in: dc_t carried from t+1 (or zeros), out: dc_{t-1}
  float* dz;            // [rows,4H]
  int dc_is_zero;       // first backward step: treat dc as zeros on input
  int dh_parts = 1;     // dh is the sum of this many arrays, dh_part_stride elements apart (added in order); 0: none
  int64_t dh_part_stride = 0;
  const float* dy_seq = nullptr;  // this step's slice of the gradient of a returned sequence: row r at dy_seq + r * dy_seq_ld
  int64_t dy_seq_ld = 0;
};
// out[r, t, :] = slices[(first + t) * slice_stride + r * H ...]: time-major step outputs as the (batch, time, units)
// tensor `returnSequence` hands to the next layer (layer/RNN.scala:74-77)
int launch_sequence_gather(sn_ctx* ctx, const float* slices, int64_t slice_stride, int first, float* out, int rows, int T, int H);
// dst[r, :] (= or +=) src[r * src_ld ...] for rows x H values: one time step cut out of a (batch, time, units) gradient
int launch_step_slice_add(sn_ctx* ctx, float* dst, const float* src, int64_t src_ld, int rows, int H, bool accumulate);
int launch_lstm_gates_bwd(sn_ctx* ctx, const LstmGateBwdArgs& a, int rows, int hidden);

// ---- Dense(H, act) >> Dense(C, Softmax) + CategoricalCrossentropy in two launches (mlp2_kernels.hip): forward, loss terms
// and every gradient.  scratch_a / scratch_b: what mlp2_fused_ok asks for; row_loss: `rows` floats.
bool mlp2_fused_ok(int rows_max, int K, int H, int C, int64_t scratch_a_elems, int64_t scratch_b_elems);
int launch_mlp2_grad(sn_ctx* ctx, const float* x, const float* y, const float* w1, const float* b1, const float* w2, const float* b2, int rows,
                     int K, int H, int C, int act1, float act1_param, bool stable, float* h, float* z2, float* p, float* scratch_a,
                     float* scratch_b, float* row_loss, float* loss_dev, float* g_w1, float* g_b1, float* g_w2, float* g_b2,
                     const struct Mlp2Update* update = nullptr);
// The optimizer update riding in the second launch: every thread that finishes a gradient value applies it to its
// parameter on the spot (same arithmetic as the streaming optimizer kernels), so a training step is two launches.  w, g
// and the state buffers are the replica's flat buffers; the gradient pointers above must point into g.
struct Mlp2Update {
  int kind = -1, n_states = 0;
  OptScalars p;
  float* w = nullptr;
  const float* g = nullptr;
  float* s0 = nullptr;
  float* s1 = nullptr;
  float* s2 = nullptr;
};

// ---- seeded random tensors (random_kernels.hip): scale / shift may be null
int launch_random_fill(sn_ctx* ctx, float* out, int64_t n, int dist, uint64_t seed, const float* scale, const float* shift);

// ---- batch normalisation over the last axis (batchnorm_kernels.hip) ---------------------
struct BatchNormArgs {
  const float* gamma;        // [C]
  const float* beta;         // [C]
  const float* moving_mean;  // [C], read by the frozen form
  const float* moving_var;
  float* mean;               // [C] statistics the output was built from (batch or moving), kept for the gradient
  float* var;
  float* r;                  // 1/sqrt(var + epsilon)
  float* inv;                // r * gamma
  float* k1;                 // [C] scratch of the gradient
  float* k2;
  float epsilon, momentum;
  // The FusedBatchNormV3 branch as the reference wires the op's outputs (math/nn/AllKernels.scala:437-448): the
  // gradient op is handed the unbiased batch variance where it expects the mean and the batch mean where it expects
  // the variance, and the moving variance follows the batch mean.  g_* hold those substituted statistics.
  bool fused_wiring = false;
  float* g_mean = nullptr;   // [C] var * n / max(n - 1, 1)
  float* g_r = nullptr;      // 1/sqrt(mean + epsilon)
  float* g_inv = nullptr;    // g_r * gamma
};
// workspace (elements) the reductions need for a [rows, cols] activation
int64_t batchnorm_workspace_elems(const sn_ctx* ctx, int64_t rows, int cols);
// y = (x*inv - mean*inv) + beta; training: batch statistics, else the moving ones
int launch_batchnorm_fwd(sn_ctx* ctx, const float* x, float* y, int64_t rows, int cols, const BatchNormArgs& a, bool training, float* ws,
                         int64_t ws_elems);
// gradients of beta, gamma and (dx != null) the input, through the batch statistics; with below_act the input
// gradient also passes through the activation that produced x (x is that activation's output)
int launch_batchnorm_bwd(sn_ctx* ctx, const float* x, const float* dy, float* dx, int64_t rows, int cols, const BatchNormArgs& a,
                         float* dbeta, float* dgamma, float* ws, int64_t ws_elems, int below_act = SN_ACT_IDENTITY,
                         float below_act_param = 0.f);
// moving = momentum*moving + (1-momentum)*batch
int launch_batchnorm_moving(sn_ctx* ctx, const BatchNormArgs& a, float* moving_mean, float* moving_var, int cols);

// ---- GEMM family (gemm_kernels.hip) ----------------------------------------------------
struct Epilogue {
  float* out = nullptr;
  int64_t ldo = 0;
  const float* bias = nullptr;  // per output column, may be null
  int act = SN_ACT_IDENTITY;    // identity / sigmoid / tanh / relu (softmax is a row kernel)
  float act_param = 0.f;
  // one row of the product goes elsewhere, untouched by bias and activation (the bias gradient that rides along
  // in a weight-gradient GEMM as an all-ones row of A)
  int row_index = -1;
  float* row_out = nullptr;
};
// C[M,N] = A[M,K] * B[K,N] with arbitrary element strides (covers NN, NT, TN).
struct GemmDesc {
  const float* a; int64_t a_sm, a_sk;   // A(m,k) = a[m*a_sm + k*a_sk]
  const float* b; int64_t b_sk, b_sn;   // B(k,n) = b[k*b_sk + n*b_sn]
  int m, n, k;
  bool a_ones_row = false;              // A's last row (index m-1) is all ones and is not read from `a`
};
// true when launch_gemm would take its 16-byte loaders for this problem (they have no all-ones row)
bool gemm_takes_fast_loaders(const sn_ctx* ctx, const GemmDesc& g, const float* workspace, int64_t workspace_elems);
int launch_gemm(sn_ctx* ctx, const GemmDesc& g, const Epilogue& ep, float* workspace, int64_t workspace_elems, bool bf16);
// Gradients of a Dense layer from many features onto at most 16 units, as row streams over X (fp32, contiguous
// [rows, in_f] / [in_f, out_f] / [rows, out_f] tensors); dense_skinny_shape says whether a shape is in their range.
bool dense_skinny_shape(int rows, int in_f, int out_f);
// (w and dx, both or neither: the same launch also writes the input gradient dx = dy . w^T)
int launch_dense_skinny_dw(sn_ctx* ctx, const float* x, const float* dy, float* dw, float* db, int rows, int in_f, int out_f,
                           const float* w = nullptr, float* dx = nullptr);
// The same layer forward for small batches (partial sums per feature chunk in the workspace, then a fixed-order reduction
// that applies e's bias and activation); dense_skinny_fwd_shape says whether shape and workspace are in its range.
// A Dense layer onto at most 4 units from at most 1024 features (a regression head behind a recurrent layer): forward in one
// launch, backward (activation gradient from the layer's output y, dX unless dx is null, dW, db unless null) in two.
bool dense_tiny_shape(int rows, int in_f, int out_f, int64_t ws_elems);
int launch_dense_tiny_fwd(sn_ctx* ctx, const float* x, const float* w, const Epilogue& e, int rows, int in_f, int out_f);
int launch_dense_tiny_bwd(sn_ctx* ctx, const float* x, const float* y, const float* dy, const float* w, float* dx, float* dw, float* db, int rows,
                          int in_f, int out_f, int act, float act_param, float* ws, int64_t ws_elems);
bool dense_skinny_fwd_shape(int rows, int in_f, int out_f, int64_t ws_elems);
int64_t dense_skinny_fwd_workspace(int rows, int in_f, int out_f);  // floats of workspace the forward form needs
// parts_left (optional): the reduction is not launched; *parts_left partial sums [part][rows * out_f] stay in ws for a
// launch of the caller's that adds them in the same order (launch_softmax_cce_partials)
int launch_dense_skinny_fwd(sn_ctx* ctx, const float* x, const float* w, const Epilogue& e, int rows, int in_f, int out_f, float* ws,
                            int64_t ws_elems, int* parts_left = nullptr);

// bf16 fast path (gemm_bf16.hip): the three products of a Dense layer on bf16 operands read as the tensors lie (no
// transposed copies), fp32 accumulation.  Besides or instead of the fp32 result (e.out, may be null) the epilogue can
// emit the result as bf16, which is how a Dense layer hands its output to the next one without a separate cast pass.
struct EpilogueBf16 {
  Epilogue e;                // e.out may be null when out_bf is set; e.act: identity or ReLU only
  void* out_bf = nullptr;    // bf16 [M, e.ldo]
  // Forward product that leaves as bf16 only (full 256 x 256 tiles, ReLU at 0): one bit per output value, set where
  // the value passed the ReLU, [M * N / 32] words in the order the kernel's lanes hold the values.
  void* signs_out = nullptr;
  // Gradient hand-over to the Dense layer below (dX products only; full 256 x 256 tiles, out_bf set, e.out null, no
  // bias, identity): the result is multiplied by that layer's ReLU gradient, read from the sign words its forward
  // product wrote (null: identity activation, nothing to multiply), before it is cast and stored, and col_partials
  // [M / 64, N] (optional) receives the column sums of every 64-row block of the fp32 values.
  bool grad_handover = false;
  const void* signs_in = nullptr;
  float* col_partials = nullptr;
};
// The three products of a Dense layer on bf16 copies of the tensors as they lie (no transposed copies):
//   FORWARD  C[M,N] = a[M,K] . b[K,N]      (X . W)
//   DX       C[M,N] = a[M,K] . b[N,K]^T    (dZ . W^T)
//   DW       C[M,N] = a[K,M]^T . b[K,N]    (X^T . dZ)
// lda / ldb are the row pitches of a and b as stored.
enum { GEMM_BF16_FORWARD = 0, GEMM_BF16_DX = 1, GEMM_BF16_DW = 2 };
int launch_gemm_bf16(sn_ctx* ctx, int product, const void* a, int64_t lda, const void* b, int64_t ldb, int M, int N, int K,
                     const EpilogueBf16& ep);
// true when an [M, N] forward result can leave as bf16 only and its dX counterpart can hand dZ over
bool gemm_bf16_full_tiles(const sn_ctx* ctx, int M, int N);
// bf16 copy out[rows,cols] of an fp32 matrix; with y or y_bf given the activation gradient act'(y) * src is what gets
// cast (and is written to dz in fp32 when dz != null).  col_partials (optional, [ceil(rows/64), cols]) receives the
// column sums of every 64-row block of the fp32 values.  y_bf: the layer output as bf16 [rows, cols], used in place of
// y when y is null (enough for ReLU at 0, whose gradient only needs the sign).
int launch_cast_bf16(sn_ctx* ctx, const float* src, int64_t ld, int rows, int cols, void* out, const float* y, int act, float act_param,
                     float* dz, float* col_partials = nullptr, const void* y_bf = nullptr);

// Division of an index below 2^31 by a divisor fixed for the launch, as a multiplication and a shift (the device has no
// integer divider: a division by a run-time value is some twenty instructions, and these kernels take three per element).
// d >= 1.  q = (hi32(x * mul) + x) >> shift with shift = ceil(log2 d), mul = floor(2^32 (2^shift - d) / d) + 1.
struct FastDiv {
  uint32_t mul, shift, d;
};
static inline FastDiv fast_div(uint32_t d) {
  uint32_t shift = 0;
  while ((1ull << shift) < d) ++shift;
  const uint64_t mul = ((1ull << 32) * ((1ull << shift) - d)) / d + 1;
  return FastDiv{(uint32_t)mul, shift, d};
}
__device__ __forceinline__ uint32_t div_by(uint32_t x, const FastDiv& f) { return (__umulhi(x, f.mul) + x) >> f.shift; }

struct ConvGeom {
  int n, h, w, cin;      // input
  int ho, wo, cout;      // output
  int kh, kw, sh, sw, pt, pl;
};
// Conv2D filter gradient of a layer with 32 input channels, 32 or 64 filters and no padding as one matrix-core tile per
// filter tap: `*parts` partial filters [part][kh*kw*cin*cout] are left in ws for the caller to add in part order.
bool conv_wgrad_taps_shape(const sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy);
int64_t conv_wgrad_taps_workspace(const sn_ctx* ctx, const ConvGeom& g);  // floats of workspace
int launch_conv_wgrad_taps(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy, float* ws, int64_t ws_elems, int* parts);
int launch_conv_fwd(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* w, const Epilogue& ep, float* ws, int64_t ws_elems);
int launch_conv_dgrad(sn_ctx* ctx, const ConvGeom& g, const float* dy, const float* w, float* dx, float* ws, int64_t ws_elems);
// A 2 x 2 max pooling right above a first-layer convolution, for launch_conv_wgrad's direct kernel: the pooling's output
// gradient dy [n, ho, wo, cout], its recorded first-maximum offsets (one byte per output value) and the convolution's saved
// output y with its activation; the kernel then forms the convolution's output gradient itself (no launch_pool_bwd).
struct PoolGrad {
  const float* dy = nullptr;
  const uint8_t* arg = nullptr;
  const float* y = nullptr;
  int ho = 0, wo = 0, sh = 1, sw = 1, pt = 0, pl = 0, act = 0;
  float act_param = 0.f;
};
bool conv_wgrad_is_direct(const sn_ctx* ctx, const ConvGeom& g, const float* ws, int64_t ws_elems, bool with_pool = false);
int launch_conv_wgrad(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy, float* dw, float* ws, int64_t ws_elems,
                      const PoolGrad* pool = nullptr);

// the same two products with LDS-direct loads into a three-stage ring (conv_ring_kernels.hip), for the shapes *_ok accepts
bool conv_ring_fwd_ok(const ConvGeom& g, const float* x, const float* w, const Epilogue& e);
int launch_conv_ring_fwd(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* w, const Epilogue& e);
bool conv_ring_dgrad_ok(const ConvGeom& g, const float* dy, const float* w);
int launch_conv_ring_dgrad(sn_ctx* ctx, const ConvGeom& g, const float* dy, const float* w, float* dx);

struct LstmWeights {
  const float* wk[4];  // [F,H] forget,input,gate,output
  const float* wr[4];  // [H,H]
  const float* b[4];   // [H] or null
};
struct LstmGrads {
  float* wk[4];
  float* wr[4];
  float* b[4];
};
// z[rows,4H] = [x_t, h_prev] * [Wk; Wr] + b   (x_t = x[:, t, :] of a [rows,T,F] tensor)
int launch_lstm_z(sn_ctx* ctx, const float* x, int t, int T, int F, const float* h_prev, int rows, int H, const LstmWeights& w,
                  float* z, float* ws, int64_t ws_elems, int gates = 4);
// dh_prev[rows,H] = dz[rows,4H] * Wr^T
int launch_lstm_dh(sn_ctx* ctx, const float* dz, int rows, int H, const LstmWeights& w, float* dh_prev, float* ws, int64_t ws_elems,
                   int gates = 4);
// dx[:, t, :] = dz * Wk^T
int launch_lstm_dx(sn_ctx* ctx, const float* dz, int rows, int H, int F, int t, int T, const LstmWeights& w, float* dx, float* ws,
                   int64_t ws_elems, int gates = 4);
// dWk = X^T dZ, dWr = Hprev^T dZ over all steps (dz_all, h_all time-major [T,rows,*]; h_all[t] = h_{t-1})
// The same gradient with all F + H rows x 128 columns per workgroup and one k range each (F <= 32, H in {64, 128, 256},
// gates * H a multiple of 128): `ranges_out` partial results [F + H + 1, gates * H] (last row: column sums of dz, the
// bias gradient) land in ws for the caller to add.  lstm_wgrad_rows_workspace: floats of ws it needs (0: shape not taken).
bool lstm_wgrad_rows_ok(const sn_ctx* ctx, const float* x, const float* h, const float* dz, int rows, int T, int F, int H, int gates);
int64_t lstm_wgrad_rows_workspace(const sn_ctx* ctx, int rows, int T, int F, int H, int gates);
int launch_lstm_wgrad_rows(sn_ctx* ctx, const float* x, const float* h, const float* dz, int rows, int T, int F, int H, int gates, float* ws,
                           int64_t ws_elems, int* ranges_out);
// adds `parts` partial sums [F + H + 1][gates * H] (rows: x features, h features, column sums of dz) into the layer's tensors
int launch_lstm_wgrad_reduce(sn_ctx* ctx, const float* ws, int parts, int F, int H, int gates, const LstmGrads& g);
int launch_lstm_wgrad(sn_ctx* ctx, const float* x, const float* h_prev_all, const float* dz_all, int rows, int T, int F, int H,
                      const LstmGrads& g, float* ws, int64_t ws_elems, int gates = 4);
// The simple recurrent cell is the same four products with one gate (gates = 1): its weights sit in slot 0.

int64_t gemm_workspace_elems(int m, int n, int k, int cu);

// ---- fused LSTM steps (lstm_kernels.hip) ------------------------------------------------
// true when the fused step kernels handle this layer (F % 4 == 0, H % 16 == 0, F + H <= 400, 16-byte aligned tensors)
bool lstm_step_fused_ok(int F, int H, const float* x, const LstmWeights& w, int gates = 4);
// gates, c_t, h_t of step t from x[:, t, :], h_prev, c_prev (both null at t == 0) in one kernel
// The step kernels read the weights from copies in their LDS order: pack_fwd ([Wk; Wr] of the 4 gates) and pack_dh
// (Wr of the 4 gates), lstm_pack_elems(F, H) floats each at most; rebuilt once per pass over the sequence.
int64_t lstm_pack_elems(int F, int H);
int launch_lstm_pack(sn_ctx* ctx, const LstmWeights& w, int F, int H, float* pack_fwd, float* pack_dh, int gates = 4);
// The simple cell's recurrences over all time steps in one launch (the LSTM sequence kernel's structure without gates).
// Forward: r_slices holds T + 1 slices, slice t + 1 = r_t, slice 0 read only if first_valid.  Backward: dr_slices holds T
// slices, slice T - 1 complete at launch, slice t - 1 = dr_t * Wr^T (+ dy_seq[:, t - 1, :] when given) for t = T-1 .. 1.
bool rnn_sequence_fwd_ok(sn_ctx* ctx, int rows, int F, int H, const float* x);
int launch_rnn_sequence_fwd(sn_ctx* ctx, const float* x, int T, int F, int first_valid, int rows, int H, const float* wk, const float* wr,
                            float* r_slices, int64_t slice);
bool rnn_sequence_bwd_ok(sn_ctx* ctx, int rows, int H, const float* wr);
// (with x, the forward slices r and a workspace the launch can carry the weight gradient, as launch_lstm_sequence_bwd does:
// H 64, 128, 192 or 256, the batch a multiple of 16, F a multiple of 4 up to 64)
int64_t rnn_sequence_bwd_wgrad_workspace(int rows, int T, int F, int H);
int launch_rnn_sequence_bwd(sn_ctx* ctx, float* dr_slices, const float* dy_seq, int T, int rows, int H, const float* wr, int64_t slice,
                            const float* x = nullptr, const float* r_slices = nullptr, int F = 0, float* ws = nullptr, int64_t ws_elems = 0,
                            int* wgrad_parts = nullptr);
// All T forward steps of an LSTM layer in one launch: the workgroups keep their weights in registers and hand h_t to each
// other through memory, one arrival counter per group of 32 batch rows.  h: T + 1 slices of `slice` floats, slice 0 the
// initial hidden state (read only if h0_valid); gates / c: T slices.  lstm_sequence_fwd_ok says whether the launch fits
// the device whole, which the hand-over needs.
bool lstm_sequence_fwd_ok(sn_ctx* ctx, int rows, int F, int H, const float* x, const LstmWeights& w);
int launch_lstm_sequence_fwd(sn_ctx* ctx, const float* x, int T, int F, int h0_valid, const float* c0, int rows, int H, const LstmWeights& w,
                             float* gates, float* c, float* h, int64_t slice);
// All reverse steps in one launch (H a power of two from 16 to 256): dz (T slices of 4 * slice floats) from the saved gates
// and cell states, the gradient of the last hidden state (dh_last, may be null) and of a returned sequence (dy_seq
// [rows, T, H], may be null).  lstm_sequence_bwd_ok: as for the forward launch.
bool lstm_sequence_bwd_ok(sn_ctx* ctx, int rows, int H, const LstmWeights& w);
// With x [rows, T, F], h (T + 1 slices, slice t = h_{t-1}) and a workspace the same launch also accumulates the weight
// gradient where the shape allows it (H 64, 128 or 256; F even up to 32 or a multiple of 4 up to 64): *wgrad_parts partial
// sums [F + H + 1][4H] are left in ws for launch_lstm_wgrad_reduce, or *wgrad_parts = 0 and the caller runs
// launch_lstm_wgrad.  lstm_sequence_bwd_wgrad_workspace: floats of ws that takes (0: the shape cannot).
int64_t lstm_sequence_bwd_wgrad_workspace(int rows, int T, int F, int H);
int launch_lstm_sequence_bwd(sn_ctx* ctx, const float* gates, const float* c, const float* c0, const float* dh_last, const float* dy_seq, int T,
                             int rows, int H, const LstmWeights& w, float* dz, int64_t slice, const float* x = nullptr, const float* h = nullptr,
                             int F = 0, float* ws = nullptr, int64_t ws_elems = 0, int* wgrad_parts = nullptr);
int launch_lstm_step_fwd(sn_ctx* ctx, const float* x, int t, int T, int F, const float* h_prev, const float* c_prev, int rows, int H,
                         const LstmWeights& w, const float* wpack, float* gates, float* c, float* h);
// dh_parts[g] (g = 0..3, part_stride elements apart) = dz[:, g*H:(g+1)*H] * Wr_g^T; their sum is dh_prev
int launch_lstm_step_dh(sn_ctx* ctx, const float* dz, int rows, int H, const float* wpack, float* dh_parts, int64_t part_stride,
                        int gates = 4);
// One launch per reverse LSTM step: gate gradients (g: gates, c, c_prev, dh parts, dy_seq, dz as for launch_lstm_gates_bwd;
// dc_in null = zeros, dc_out another buffer) and, unless wpack is null, the lstm_bwd_parts(H) partial products whose sum
// is dh_{t-1}, written out_part_stride elements apart.  wpack: launch_lstm_pack_bwd (at most lstm_pack_elems floats).
bool lstm_step_bwd_fused_ok(int H, const LstmWeights& w);
int lstm_bwd_parts(int H);
int launch_lstm_pack_bwd(sn_ctx* ctx, const LstmWeights& w, int H, float* pack);
int launch_lstm_step_bwd(sn_ctx* ctx, const LstmGateBwdArgs& g, const float* dc_in, float* dc_out, const float* wpack, float* dh_out,
                         int64_t out_part_stride, int rows, int H);
// simple cell: r_t[rows, H] = [x[:, t, :], r_prev] * [Wk; Wr] from the one-gate pack (r_prev null at t == 0)
int launch_rnn_step_fwd(sn_ctx* ctx, const float* x, int t, int T, int F, const float* r_prev, int rows, int H, const float* wpack, float* out);

}  // namespace sn
