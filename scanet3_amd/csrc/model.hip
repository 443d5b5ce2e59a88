// Host side of the compiled step: turns the flattened layer list into a plan of fused
// operations over a flat parameter buffer, and runs forward / loss / backward / update,
// the per-partition epoch loop and the replica average.
//
// Correspondence with the reference (paths under src/main/scala/scanet/):
//   plan building ........ models/layer/Composed.scala:22-53 (parameter paths, layer order)
//   sn_step .............. optimizers/Optimizer.scala:169-194 (compileBackprop)
//   sn_train_epoch ....... optimizers/Optimizer.scala:106-161 (optimizeOnPartition)
//   sn_replicas_average .. optimizers/Optimizer.scala:196-230 (aggregateParams)
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <mutex>

namespace sn {

enum OpKind { OP_DENSE, OP_CONV, OP_POOL, OP_FLATTEN, OP_BIASACT, OP_SOFTMAX, OP_LSTM, OP_SRNN, OP_BATCHNORM };

struct ParamDef {
  sn_param_info info;
  int reg_kind = SN_REG_NONE;
  float reg_lambda = 0.f;
  // Bias and BatchNorm add their penalty only while trainable (layer/Bias.scala:35-36, layer/BatchNorm.scala:158-160):
  // the frozen model a TrainedModel holds leaves it out; Dense and the RNN cells add theirs always.
  bool penalty_when_frozen = true;
};
// ParamDef.aggregation of the tensor is `Some(Avg)` (info.aggregated = 1) for everything but the carried state of a
// stateful RNN (layer/RNN.scala:188,302-303), which aggregateParams re-initialises (optimizers/Optimizer.scala:207-210).

struct Op {
  OpKind kind;
  std::vector<int64_t> in_dims, out_dims;  // per sample
  int64_t in_elems = 0, out_elems = 0;     // per sample
  int w = -1, b = -1;                      // parameter indices
  int act = SN_ACT_IDENTITY;
  float act_param = 0.f;
  // conv / pool geometry (per sample: h, w, c)
  int kh = 0, kw = 0, sh = 1, sw = 1, pt = 0, pl = 0;
  bool pool_avg = false;  // Pool2D: mean of the window instead of its maximum
  // lstm
  int T = 0, F = 0, H = 0;
  bool ret_seq = false;  // the layer's output is every step's output, [T, H] per sample (layer/RNN.scala:74-77)
  int lstm_p[4][3] = {{-1, -1, -1}, {-1, -1, -1}, {-1, -1, -1}, {-1, -1, -1}};  // gate x {kernel, recurrent, bias}
  // batch norm: beta, gamma, moving mean, moving variance
  int bn_p[4] = {-1, -1, -1, -1};
  // stateful RNN (layer/RNN.scala:27,34,66-67): parameter indices of the carried state, LSTM {cell_state, hidden_state},
  // simple cell {state, -}; -1 = the layer starts every batch from zeros
  int state_p[2] = {-1, -1};
  float bn_momentum = 0.99f, bn_epsilon = 1e-3f;
  bool bn_fused = false;  // the FusedBatchNormV3 branch (rank-4 input unless fused = Some(false)), wired as the reference wires it
  // buffers (indices into replica buffer table), assigned at replica creation
  int out_buf = -1;
};

}  // namespace sn

struct sn_model {
  uint32_t magic;
  sn_ctx* ctx;
  int loss;
  uint32_t flags;
  int batch;
  std::vector<int64_t> input_dims;
  int64_t in_elems;
  std::vector<sn::Op> ops;
  std::vector<sn::ParamDef> params;
  int64_t flat_elems;  // padded length of the flat parameter buffer
  std::vector<std::pair<int64_t, int64_t>> trainable_runs;  // [begin, end) element ranges the optimizer updates
  std::vector<int64_t> out_dims;
  int64_t out_elems;
  int64_t max_act_elems;   // per sample, over every op input/output
  int64_t workspace_elems;
  int live_replicas;
};

struct sn_replica {
  uint32_t magic;
  sn_model* model;
  sn_ctx* ctx;
  bool has_opt;
  sn_optimizer_desc opt;
  int n_states;
  float* w = nullptr;
  float* g = nullptr;
  float* s[SN_MAX_OPT_STATES] = {nullptr, nullptr, nullptr};
  std::vector<float*> act;      // per op output (null for views)
  std::vector<uint8_t*> arg;    // per op: max-pool argmax
  float* grad_buf[2] = {nullptr, nullptr};
  float* ws = nullptr;
  float* loss_dev = nullptr;
  float* loss_partials = nullptr;
  unsigned long long* count_dev = nullptr;
  // lstm scratch (one set, shared by every LSTM op; sized for the largest)
  float* lstm_z = nullptr;
  std::vector<float*> lstm_gates, lstm_c, lstm_h, lstm_dz;  // per op
  std::vector<float*> lstm_pk_fwd, lstm_pk_dh;              // per op: weights in the step kernels' LDS order
  float* lstm_dh[2] = {nullptr, nullptr};
  float* lstm_dc = nullptr;
  float* lstm_dc2 = nullptr;  // the fused backward step reads the carried cell gradient from one buffer and writes the other
  // bf16 operand copies of the Dense layers (SN_FLAG_GEMM_BF16): per op its input, its dZ and its weights as they lie,
  // and one bit per output value where a hidden ReLU layer's output lives as bf16 only (the sign its gradient needs)
  std::vector<uint16_t*> bf_x, bf_dz, bf_w;  // bf_w[i] points into bf_wflat
  uint16_t* bf_wflat = nullptr;              // bf16 copy of the flat parameter buffer (same offsets), written by the optimizer
  std::vector<uint32_t*> bf_signs;
  std::vector<float*> bn_buf;  // per batch-norm op: mean, var, 1/sqrt(var+eps), scale, two gradient vectors
  float* bf_colp = nullptr;  // per-64-row-block column sums of dZ (bias gradient of the bf16 Dense path)
  bool bf_weights_stale = true;  // weights changed since their bf16 copies were made
  // Training steps of a model whose whole flat buffer is one optimizer launch: the sums of the convolutions' partial
  // filter gradients wait for that launch (launch_finish) instead of running as launches of their own.  Every such
  // convolution has a workspace of its own (the shared one is overwritten by the next product).
  bool updated_in_pass = false;  // the gradient pass of this step has applied the optimizer itself
  int pass_iter = 0;             // iteration number of the update that follows the running gradient pass (0: none follows)
  bool leave_logit_parts = false;  // the running forward pass may leave the last Dense product's partial sums to the loss kernel
  int logit_parts = 0;             // how many it left in ws (0: the logits are complete)
  bool fuse_finish = false, defer_now = false;
  std::vector<float*> ws_defer;
  DeferredReduce deferred[MAX_DEFERRED];
  int n_deferred = 0;
  // host-fed epochs: two device slots per tensor, a copy stream, "slot filled" / "slot consumed" events
  float* stage_x[2] = {nullptr, nullptr};
  float* stage_y[2] = {nullptr, nullptr};
  int64_t stage_group = 1;  // full batches a staging slot holds
  hipStream_t copy_stream = nullptr;
  hipEvent_t ev_filled[2] = {nullptr, nullptr}, ev_consumed[2] = {nullptr, nullptr};
  // bf16 Dense models: a layer's optimizer launch runs on a second stream beside the gradient products of the layers
  // below it (a stream of memory traffic beside matrix-core work)
  hipStream_t update_stream = nullptr;
  hipEvent_t ev_layer_ready = nullptr, ev_updates_done = nullptr;
  bool side_updates = false;  // the running gradient pass updates each Dense layer as soon as its gradients are complete
  std::vector<void*> owned;
};

namespace sn {

static int check_model(sn_model* m) {
  if (!m || m->magic != MODEL_MAGIC) return fail(SN_E_STATE, "invalid or destroyed model handle");
  return SN_OK;
}
static int check_replica(sn_replica* r) {
  if (!r || r->magic != REPLICA_MAGIC) return fail(SN_E_STATE, "invalid or destroyed replica handle");
  return SN_OK;
}

static int64_t prod(const std::vector<int64_t>& d) {
  int64_t p = 1;
  for (auto v : d) p *= v;
  return p;
}

// Padding.size / TensorFlow's SAME rule (math/nn/AllKernels.scala:39-65): extra padding goes after.
static void conv_out(int padding, int in, int k, int s, int* out, int* pad_before, int lo = 0, int hi = 0) {
  if (padding == SN_PAD_EXPLICIT) {  // math/nn/AllKernels.scala:74-91
    const int span = in + lo + hi - k;
    *out = span < 0 ? 0 : (span + s - 1) / s + 1;
    *pad_before = lo;
  } else if (padding == SN_PAD_SAME) {
    *out = (in + s - 1) / s;
    const int total = std::max((*out - 1) * s + k - in, 0);
    *pad_before = total / 2;
  } else {
    *out = (in - k + 1 + s - 1) / s;  // ceil((in - k + 1) / s)
    *pad_before = 0;
  }
}

static int add_param(sn_model* m, const std::string& path, const std::vector<int64_t>& dims, int reg_kind, float reg_lambda,
                     bool trainable = true, bool penalty_when_frozen = true, bool aggregated = true) {
  ParamDef p;
  memset(&p.info, 0, sizeof(p.info));
  p.info.trainable = trainable ? 1 : 0;
  p.info.aggregated = aggregated ? 1 : 0;
  snprintf(p.info.path, sizeof(p.info.path), "%s", path.c_str());
  p.info.rank = (int32_t)dims.size();
  p.info.size = 1;
  for (size_t i = 0; i < dims.size(); ++i) {
    p.info.dims[i] = dims[i];
    p.info.size *= dims[i];
  }
  p.info.offset = m->flat_elems;
  p.reg_kind = reg_kind;
  p.reg_lambda = reg_lambda;
  p.penalty_when_frozen = penalty_when_frozen;
  m->flat_elems += align_up(p.info.size, 64);  // every tensor starts on a 256-byte boundary
  m->params.push_back(p);
  return (int)m->params.size() - 1;
}

static int build_plan(sn_model* m, const sn_layer_desc* layers, int n_layers) {
  std::vector<int64_t> cur = m->input_dims;
  const bool single = n_layers == 1;  // Composed(single) is the layer itself: no index prefix (Composed.scala:95-98)
  auto prefix = [&](int i) { return single ? std::string() : std::to_string(i) + "/"; };
  int64_t max_act = prod(cur);
  int64_t ws = 0;
  const int cu = m->ctx->compute_units;
  const int B = m->batch;
  int i = 0;
  while (i < n_layers) {
    const sn_layer_desc& L = layers[i];
    Op op;
    op.in_dims = cur;
    op.in_elems = prod(cur);
    switch (L.kind) {
      case SN_LAYER_DENSE: {
        SN_REQUIRE(cur.size() == 1, "layer %d: Dense expects a (batch, features) input, got rank %zu (add Flatten)", i, cur.size() + 1);
        SN_REQUIRE(L.units > 0, "layer %d: Dense needs units > 0", i);
        op.kind = OP_DENSE;
        op.w = add_param(m, prefix(i) + "weights", {cur[0], L.units}, L.reg_kind, L.reg_lambda);
        op.out_dims = {L.units};
        ++i;
        if (i < n_layers && layers[i].kind == SN_LAYER_BIAS) {
          SN_REQUIRE(layers[i].units == L.units, "layer %d: Bias has %d features, input has %d", i, layers[i].units, L.units);
          op.b = add_param(m, prefix(i) + "weights", {L.units}, layers[i].reg_kind, layers[i].reg_lambda, true, false);
          ++i;
        }
        if (i < n_layers && layers[i].kind == SN_LAYER_ACTIVATE && layers[i].activation != SN_ACT_SOFTMAX) {
          op.act = layers[i].activation;
          op.act_param = layers[i].act_param;
          ++i;
        }
        const int in_f = (int)cur[0], out_f = L.units;
        ws = std::max(ws, gemm_workspace_elems(B, out_f, in_f, cu));
        if (dense_skinny_fwd_shape(B, in_f, out_f, INT64_MAX)) ws = std::max(ws, dense_skinny_fwd_workspace(B, in_f, out_f));
        ws = std::max(ws, gemm_workspace_elems(in_f + 1, out_f, B, cu));  // + the bias-gradient row
        ws = std::max(ws, gemm_workspace_elems(B, in_f, out_f, cu));
        break;
      }
      case SN_LAYER_CONV2D: {
        SN_REQUIRE(cur.size() == 3, "layer %d: Conv2D input should have a shape (NHWC) but was rank %zu", i, cur.size() + 1);
        SN_REQUIRE(L.units > 0 && L.kernel_h > 0 && L.kernel_w > 0 && L.stride_h > 0 && L.stride_w > 0,
                   "layer %d: Conv2D needs positive filters, kernel and strides", i);
        SN_REQUIRE(L.padding >= SN_PAD_VALID && L.padding <= SN_PAD_EXPLICIT, "layer %d: unknown padding %d", i, L.padding);
        SN_REQUIRE(L.padding != SN_PAD_EXPLICIT || (L.pad_top >= 0 && L.pad_bottom >= 0 && L.pad_left >= 0 && L.pad_right >= 0),
                   "layer %d: explicit paddings must not be negative", i);
        op.kind = OP_CONV;
        op.kh = L.kernel_h; op.kw = L.kernel_w; op.sh = L.stride_h; op.sw = L.stride_w;
        int ho, wo;
        conv_out(L.padding, (int)cur[0], op.kh, op.sh, &ho, &op.pt, L.pad_top, L.pad_bottom);
        conv_out(L.padding, (int)cur[1], op.kw, op.sw, &wo, &op.pl, L.pad_left, L.pad_right);
        SN_REQUIRE(ho > 0 && wo > 0, "layer %d: Conv2D kernel larger than its input", i);
        op.w = add_param(m, prefix(i) + "weights", {op.kh, op.kw, cur[2], L.units}, SN_REG_NONE, 0.f);
        op.out_dims = {ho, wo, L.units};
        ++i;
        if (i < n_layers && layers[i].kind == SN_LAYER_BIAS) {
          SN_REQUIRE(layers[i].units == L.units, "layer %d: Bias has %d features, input has %d", i, layers[i].units, L.units);
          op.b = add_param(m, prefix(i) + "weights", {L.units}, layers[i].reg_kind, layers[i].reg_lambda, true, false);
          ++i;
        }
        if (i < n_layers && layers[i].kind == SN_LAYER_ACTIVATE && layers[i].activation != SN_ACT_SOFTMAX) {
          op.act = layers[i].activation;
          op.act_param = layers[i].act_param;
          ++i;
        }
        const int64_t K = (int64_t)op.kh * op.kw * cur[2];
        ws = std::max(ws, gemm_workspace_elems(B * ho * wo, L.units, (int)K, cu));
        ws = std::max(ws, gemm_workspace_elems((int)K, L.units, B * ho * wo, cu));
        ws = std::max(ws, gemm_workspace_elems(B * (int)cur[0] * (int)cur[1], (int)cur[2], op.kh * op.kw * L.units, cu));
        {
          const ConvGeom cg{B, (int)cur[0], (int)cur[1], (int)cur[2], (int)ho, (int)wo, L.units, op.kh, op.kw, op.sh, op.sw, op.pt, op.pl};
          if (cg.cin == 32) ws = std::max(ws, conv_wgrad_taps_workspace(m->ctx, cg));  // the filter gradient's tile-per-tap form
        }
        break;
      }
      case SN_LAYER_POOL2D: {
        SN_REQUIRE(cur.size() == 3, "layer %d: Pool2D input should have a shape (NHWC) but was rank %zu", i, cur.size() + 1);
        SN_REQUIRE(L.kernel_h > 0 && L.kernel_w > 0 && L.stride_h > 0 && L.stride_w > 0 && L.kernel_h * L.kernel_w <= 255,
                   "layer %d: Pool2D needs a positive window (at most 255 cells) and strides", i);
        SN_REQUIRE(L.padding == SN_PAD_VALID || L.padding == SN_PAD_SAME, "layer %d: only [Same, Valid] paddings are supported", i);
        SN_REQUIRE(L.pool_reduce == SN_POOL_MAX || L.pool_reduce == SN_POOL_AVG, "layer %d: unknown pooling reduction %d", i, L.pool_reduce);
        op.kind = OP_POOL;
        op.pool_avg = L.pool_reduce == SN_POOL_AVG;
        op.kh = L.kernel_h; op.kw = L.kernel_w; op.sh = L.stride_h; op.sw = L.stride_w;
        int ho, wo;
        conv_out(L.padding, (int)cur[0], op.kh, op.sh, &ho, &op.pt);
        conv_out(L.padding, (int)cur[1], op.kw, op.sw, &wo, &op.pl);
        SN_REQUIRE(ho > 0 && wo > 0, "layer %d: Pool2D window larger than its input", i);
        op.out_dims = {ho, wo, cur[2]};
        ++i;
        break;
      }
      case SN_LAYER_FLATTEN: {
        SN_REQUIRE(cur.size() >= 1, "layer %d: rank should be >= 2", i);
        op.kind = OP_FLATTEN;
        op.out_dims = {prod(cur)};
        ++i;
        break;
      }
      case SN_LAYER_BIAS:
      case SN_LAYER_ACTIVATE: {
        op.out_dims = cur;
        if (L.kind == SN_LAYER_ACTIVATE && L.activation == SN_ACT_SOFTMAX) {
          SN_REQUIRE(cur.size() == 1, "layer %d: Softmax expects a (batch, classes) input", i);
          op.kind = OP_SOFTMAX;
          ++i;
          break;
        }
        op.kind = OP_BIASACT;
        if (L.kind == SN_LAYER_BIAS) {
          SN_REQUIRE(L.units == cur.back(), "layer %d: Bias has %d features, input has %lld", i, L.units, (long long)cur.back());
          op.b = add_param(m, prefix(i) + "weights", {L.units}, L.reg_kind, L.reg_lambda, true, false);
          ++i;
          if (i < n_layers && layers[i].kind == SN_LAYER_ACTIVATE && layers[i].activation != SN_ACT_SOFTMAX) {
            op.act = layers[i].activation;
            op.act_param = layers[i].act_param;
            ++i;
          }
        } else {
          SN_REQUIRE(L.activation >= SN_ACT_IDENTITY && L.activation <= SN_ACT_RELU, "layer %d: unknown activation %d", i, L.activation);
          op.act = L.activation;
          op.act_param = L.act_param;
          ++i;
        }
        break;
      }
      case SN_LAYER_LSTM: {
        SN_REQUIRE(cur.size() == 2, "layer %d: RNN requires input to have Shape(batch, time, features)", i);
        SN_REQUIRE(L.units > 0, "layer %d: RNN Cell should contain at least one unit", i);
        SN_REQUIRE(L.activation == SN_ACT_TANH || L.activation == SN_ACT_IDENTITY,
                   "layer %d: only the default LSTM activations (tanh cell, sigmoid gates) are built", i);
        op.kind = OP_LSTM;
        op.T = (int)cur[0]; op.F = (int)cur[1]; op.H = L.units;
        static const char* gates[4] = {"forget", "input", "gate", "output"};  // layer/RNN.scala:285-289
        if (L.stateful) {  // `state ++ weights` (RNN.scala:32-35): (batch, units), Zeros, not trainable, no aggregation (:302-303)
          op.state_p[0] = add_param(m, prefix(i) + "cell_state", {B, op.H}, SN_REG_NONE, 0.f, false, false, false);
          op.state_p[1] = add_param(m, prefix(i) + "hidden_state", {B, op.H}, SN_REG_NONE, 0.f, false, false, false);
        }
        for (int gi = 0; gi < 4; ++gi) {
          const std::string gp = prefix(i) + gates[gi];
          // every gate is a SimpleRNNCell ?>> Bias with the layer's three regularizers (RNN.scala:270-283,198-199)
          op.lstm_p[gi][0] = add_param(m, gp + "/0/kernel_weights", {op.F, op.H}, L.reg_kind, L.reg_lambda);
          op.lstm_p[gi][1] = add_param(m, gp + "/0/recurrent_weights", {op.H, op.H}, L.recurrent_reg_kind, L.recurrent_reg_lambda);
          if (L.use_bias) op.lstm_p[gi][2] = add_param(m, gp + "/1/weights", {op.H}, L.bias_reg_kind, L.bias_reg_lambda, true, false);
        }
        op.ret_seq = L.return_sequence != 0;
        op.out_dims = op.ret_seq ? std::vector<int64_t>{op.T, L.units} : std::vector<int64_t>{L.units};  // RNN.scala:84-90
        ws = std::max(ws, gemm_workspace_elems(B, 4 * op.H, op.F + op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(B, op.H, 4 * op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(B, op.F, 4 * op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(op.F + op.H + 1, 4 * op.H, op.T * B, cu));
        ws = std::max(ws, lstm_wgrad_rows_workspace(m->ctx, B, op.T, op.F, op.H, 4));
        if (B <= 1024) ws = std::max(ws, lstm_sequence_bwd_wgrad_workspace(B, op.T, op.F, op.H));  // one partial per 16 rows: up to 64 of them
        ++i;
        break;
      }
      case SN_LAYER_BATCHNORM: {
        // BatchNorm(axes = Seq(-1)): the generic form (layer/BatchNorm.scala:123-143, math/nn/AllKernels.scala:663-684), or for
        // NHWC input unless fused = Some(false) the FusedBatchNormV3 branch (BatchNorm.scala:100-107,116-130)
        SN_REQUIRE(cur.size() >= 1, "layer %d: rank should be >= 2", i);
        SN_REQUIRE(L.bn_fused >= -1 && L.bn_fused <= 1, "layer %d: fused must be -1 (None), 0 or 1", i);
        op.bn_fused = cur.size() == 3 && L.bn_fused != 0;
        SN_REQUIRE(op.bn_fused || L.bn_fused != 1, "layer %d: Cannot use fused implementation with this input rank", i);  // BatchNorm.scala:131-133
        SN_REQUIRE(L.bn_epsilon > 0.f, "layer %d: epsilon must be positive", i);
        op.kind = OP_BATCHNORM;
        op.bn_momentum = L.bn_momentum;
        op.bn_epsilon = L.bn_epsilon;
        op.out_dims = cur;
        std::vector<int64_t> shape(cur.size() + 1, 1);  // every axis but the normalised one becomes 1 (BatchNorm.scala:80-88)
        shape.back() = cur.back();
        static const char* names[4] = {"beta", "gamma", "moving_mean", "moving_variance"};  // BatchNorm.scala:92-97,170-173
        // penalty = betaRegularizer(gamma) + betaRegularizer(gamma) while trainable (BatchNorm.scala:158-160): the beta
        // regularizer, on gamma, twice; doubling lambda is the same number bit for bit
        for (int k = 0; k < 4; ++k)
          op.bn_p[k] = add_param(m, prefix(i) + names[k], shape, k == 1 ? L.reg_kind : SN_REG_NONE, k == 1 ? 2.0f * L.reg_lambda : 0.f, k < 2, false);
        ws = std::max(ws, batchnorm_workspace_elems(m->ctx, (int64_t)B * (prod(cur) / cur.back()), (int)cur.back()));
        ++i;
        break;
      }
      case SN_LAYER_SIMPLE_RNN: {
        // RNN(SimpleRNNCell ?>> Bias ?>> activation), layer/RNN.scala:113-163; one "gate" whose weights use slot 0
        SN_REQUIRE(cur.size() == 2, "layer %d: RNN requires input to have Shape(batch, time, features)", i);
        SN_REQUIRE(L.units > 0, "layer %d: RNN Cell should contain at least one unit", i);
        SN_REQUIRE(L.activation >= SN_ACT_IDENTITY && L.activation <= SN_ACT_RELU, "layer %d: unknown cell activation %d", i, L.activation);
        op.kind = OP_SRNN;
        op.T = (int)cur[0]; op.F = (int)cur[1]; op.H = L.units;
        op.act = L.activation;
        op.act_param = L.act_param;
        if (L.stateful)  // the cell's previous product (RNN.scala:188,195-196)
          op.state_p[0] = add_param(m, prefix(i) + "0/state", {B, op.H}, SN_REG_NONE, 0.f, false, false, false);
        op.lstm_p[0][0] = add_param(m, prefix(i) + "0/kernel_weights", {op.F, op.H}, L.reg_kind, L.reg_lambda);  // RNN.scala:165-166,198-203
        op.lstm_p[0][1] = add_param(m, prefix(i) + "0/recurrent_weights", {op.H, op.H}, L.recurrent_reg_kind, L.recurrent_reg_lambda);
        if (L.use_bias) op.b = add_param(m, prefix(i) + "1/weights", {op.H}, L.bias_reg_kind, L.bias_reg_lambda, true, false);
        op.ret_seq = L.return_sequence != 0;
        op.out_dims = op.ret_seq ? std::vector<int64_t>{op.T, L.units} : std::vector<int64_t>{L.units};
        ws = std::max(ws, gemm_workspace_elems(B, op.H, op.F + op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(B, op.H, op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(B, op.F, op.H, cu));
        ws = std::max(ws, gemm_workspace_elems(op.F + op.H, op.H, op.T * B, cu));
        ws = std::max(ws, lstm_wgrad_rows_workspace(m->ctx, B, op.T, op.F, op.H, 1));
        if (B <= 1024) ws = std::max(ws, rnn_sequence_bwd_wgrad_workspace(B, op.T, op.F, op.H));
        ++i;
        break;
      }
      default:
        return fail(SN_E_INVALID, "layer %d: unknown layer kind %d", i, L.kind);
    }
    op.out_elems = prod(op.out_dims);
    max_act = std::max(max_act, op.out_elems);
    cur = op.out_dims;
    m->ops.push_back(op);
  }
  m->out_dims = cur;
  m->out_elems = prod(cur);
  m->max_act_elems = max_act;
  // runs of trainable tensors in the flat buffer (padding included): what one optimizer launch covers
  for (const ParamDef& p : m->params) {
    if (!p.info.trainable) continue;
    const int64_t end = p.info.offset + align_up(p.info.size, 64);
    if (!m->trainable_runs.empty() && m->trainable_runs.back().second == p.info.offset) m->trainable_runs.back().second = end;
    else m->trainable_runs.push_back({p.info.offset, end});
  }
  // column sums over many rows use the workspace too
  ws = std::max<int64_t>(ws, (int64_t)cu * 4 * 64 * 4);
  m->workspace_elems = ws;
  return SN_OK;
}

// ---------------------------------------------------------------------------- replica memory
template <class T>
static int dev_alloc(sn_replica* r, T** out, int64_t elems) {
  *out = nullptr;
  if (elems <= 0) return SN_OK;
  void* p = nullptr;
  SN_HIP(hipMalloc(&p, (size_t)elems * sizeof(T)));
  r->owned.push_back(p);
  *out = (T*)p;
  return SN_OK;
}

static bool dense_bf16_fast(const sn_model* m, const struct Op& op);
// A hidden Dense layer of the bf16 path whose successor is another one hands its output over as bf16 copies; its
// fp32 output has no other reader when the activation's gradient needs only the sign of the output (ReLU at zero) or nothing.
static bool hidden_f32_not_needed(const sn_model* m, size_t i) {
  if (i + 1 >= m->ops.size()) return false;
  const Op& op = m->ops[i];
  // ReLU with a threshold other than zero keeps its fp32 output: the gradient is (threshold < y) in fp32 (`Max.localGrad`),
  // clamped outputs equal the threshold exactly, and bf16 may round the threshold to either side of itself.
  const bool sign_is_enough = op.act == SN_ACT_IDENTITY || (op.act == SN_ACT_RELU && op.act_param == 0.f);
  return dense_bf16_fast(m, op) && dense_bf16_fast(m, m->ops[i + 1]) && sign_is_enough && m->batch % 8 == 0;
}

// ... and does so for a pass over `rows` rows when the [rows, out] result tiles exactly into the 256 x 256 tiles whose
// stores the bf16 kernel can park; the backward pass of the same rows then finds the layer's dZ handed over.
static bool hidden_bf16_only(const sn_replica* r, size_t i, int rows) {
  return hidden_f32_not_needed(r->model, i) && gemm_bf16_full_tiles(r->ctx, rows, (int)r->model->ops[i].out_elems);
}

// The bf16 kernel moves 16-byte chunks of 8 values along every operand row.
static bool dense_bf16_fast(const sn_model* m, const Op& op) {
  return (m->flags & SN_FLAG_GEMM_BF16) && op.kind == OP_DENSE && op.in_elems % 8 == 0 && op.out_elems % 8 == 0 && m->batch % 8 == 0;
}

static float* param_ptr(sn_replica* r, float* base, int idx) { return idx < 0 ? nullptr : base + r->model->params[idx].info.offset; }

static bool mlp2_path(const sn_model* m);
static int alloc_replica(sn_replica* r) {
  sn_model* m = r->model;
  const int64_t B = m->batch;
  SN_HIP(hipSetDevice(r->ctx->device));
  SN_TRY(dev_alloc(r, &r->w, m->flat_elems));
  SN_TRY(dev_alloc(r, &r->g, m->flat_elems));
  SN_TRY(launch_fill(r->ctx, r->w, 0.f, m->flat_elems));
  SN_TRY(launch_fill(r->ctx, r->g, 0.f, m->flat_elems));
  for (int s = 0; s < r->n_states; ++s) {
    SN_TRY(dev_alloc(r, &r->s[s], m->flat_elems));
    SN_TRY(launch_fill(r->ctx, r->s[s], r->opt.init_acc, m->flat_elems));
  }
  const size_t n_ops = m->ops.size();
  r->act.assign(n_ops, nullptr);
  r->arg.assign(n_ops, nullptr);
  r->lstm_gates.assign(n_ops, nullptr);
  r->lstm_c.assign(n_ops, nullptr);
  r->lstm_h.assign(n_ops, nullptr);
  r->lstm_dz.assign(n_ops, nullptr);
  r->lstm_pk_fwd.assign(n_ops, nullptr);
  r->lstm_pk_dh.assign(n_ops, nullptr);
  r->bn_buf.assign(n_ops, nullptr);
  r->bf_x.assign(n_ops, nullptr); r->bf_dz.assign(n_ops, nullptr); r->bf_w.assign(n_ops, nullptr); r->bf_signs.assign(n_ops, nullptr);
  int64_t lstm_z = 0, lstm_h = 0, bf_colp = 0, lstm_parts = 4;
  for (size_t i = 0; i < n_ops; ++i) {
    const Op& op = m->ops[i];
    if (op.kind == OP_FLATTEN) continue;  // a view of its input
    if (op.kind == OP_LSTM) {
      const int64_t bh = B * op.H;
      SN_TRY(dev_alloc(r, &r->lstm_gates[i], (int64_t)op.T * bh * 4));
      SN_TRY(dev_alloc(r, &r->lstm_c[i], (int64_t)op.T * bh));
      SN_TRY(dev_alloc(r, &r->lstm_h[i], (int64_t)(op.T + 1) * bh));  // slice 0 = zeros = h_{-1}
      SN_TRY(dev_alloc(r, &r->lstm_dz[i], (int64_t)op.T * bh * 4));
      SN_TRY(dev_alloc(r, &r->lstm_pk_fwd[i], lstm_pack_elems(op.F, op.H)));
      SN_TRY(dev_alloc(r, &r->lstm_pk_dh[i], lstm_pack_elems(op.F, op.H)));
      SN_TRY(launch_fill(r->ctx, r->lstm_h[i], 0.f, bh));
      lstm_z = std::max(lstm_z, bh * 4);
      lstm_h = std::max(lstm_h, bh);
      lstm_parts = std::max<int64_t>(lstm_parts, lstm_bwd_parts(op.H));
      if (op.ret_seq) SN_TRY(dev_alloc(r, &r->act[i], B * op.out_elems));
      continue;  // output = last slice of lstm_h unless the whole sequence is returned
    }
    SN_TRY(dev_alloc(r, &r->act[i], B * op.out_elems));
    if (op.kind == OP_BATCHNORM) SN_TRY(dev_alloc(r, &r->bn_buf[i], 9 * align_up(op.out_dims.back(), 64)));
    if (op.kind == OP_SRNN) {  // the carried state of every step and its gradient, time-major like the LSTM's
      const int64_t bh = B * op.H;
      SN_TRY(dev_alloc(r, &r->lstm_h[i], (int64_t)(op.T + 1) * bh));  // slice 0 = zeros = the initial state
      SN_TRY(dev_alloc(r, &r->lstm_dz[i], (int64_t)op.T * bh));
      SN_TRY(dev_alloc(r, &r->lstm_pk_fwd[i], lstm_pack_elems(op.F, op.H) / 4));  // one gate
      SN_TRY(dev_alloc(r, &r->lstm_pk_dh[i], lstm_pack_elems(op.F, op.H) / 4));
      SN_TRY(launch_fill(r->ctx, r->lstm_h[i], 0.f, bh));
    }
    if (op.kind == OP_POOL && !op.pool_avg) SN_TRY(dev_alloc(r, &r->arg[i], B * op.out_elems));
    if (dense_bf16_fast(m, op)) {
      SN_TRY(dev_alloc(r, &r->bf_x[i], B * op.in_elems));
      SN_TRY(dev_alloc(r, &r->bf_dz[i], B * op.out_elems));
      if (hidden_f32_not_needed(m, i) && op.act == SN_ACT_RELU) SN_TRY(dev_alloc(r, &r->bf_signs[i], ceil_div(B * op.out_elems, 32)));
      bf_colp = std::max(bf_colp, ceil_div(B, 64) * op.out_elems);
    }
  }
  SN_TRY(dev_alloc(r, &r->bf_colp, bf_colp));
  if (m->flags & SN_FLAG_GEMM_BF16) {
    SN_TRY(dev_alloc(r, &r->bf_wflat, m->flat_elems));
    for (size_t i = 0; i < n_ops; ++i)
      if (dense_bf16_fast(m, m->ops[i])) r->bf_w[i] = r->bf_wflat + m->params[m->ops[i].w].info.offset;
  }
  SN_TRY(dev_alloc(r, &r->lstm_z, lstm_z));
  SN_TRY(dev_alloc(r, &r->lstm_dh[0], lstm_h * lstm_parts));  // partial sums of the hidden gradient: per gate, or per slice of units
  SN_TRY(dev_alloc(r, &r->lstm_dh[1], lstm_h * lstm_parts));
  SN_TRY(dev_alloc(r, &r->lstm_dc, lstm_h));
  SN_TRY(dev_alloc(r, &r->lstm_dc2, lstm_h));
  SN_TRY(dev_alloc(r, &r->grad_buf[0], B * m->max_act_elems));
  SN_TRY(dev_alloc(r, &r->grad_buf[1], B * m->max_act_elems));
  SN_TRY(dev_alloc(r, &r->ws, m->workspace_elems));
  r->ws_defer.assign(n_ops, nullptr);
  bool penalties = false;
  for (const auto& p : m->params) penalties = penalties || p.reg_kind != SN_REG_NONE;
  // (several runs of trainable tensors, i.e. a BatchNorm's moving statistics in between: the launch skips the gaps)
  r->fuse_finish = r->has_opt && !(m->flags & SN_FLAG_GEMM_BF16) && !penalties && !mlp2_path(m) && !m->trainable_runs.empty() &&
                   m->trainable_runs.size() <= (size_t)MAX_FINISH_HOLES && m->workspace_elems > 0 && m->workspace_elems <= ((int64_t)64 << 20);
  if (r->fuse_finish) {
    int n_conv = 0;
    for (size_t i = 0; i < n_ops; ++i)
      if (m->ops[i].kind == OP_CONV && n_conv < MAX_DEFERRED) {
        SN_TRY(dev_alloc(r, &r->ws_defer[i], m->workspace_elems));
        ++n_conv;
      }
    r->fuse_finish = n_conv > 0;
  }
  SN_TRY(dev_alloc(r, &r->loss_dev, 1));
  SN_TRY(dev_alloc(r, &r->loss_partials, std::max<int64_t>(1024, m->batch)));
  SN_TRY(dev_alloc(r, &r->count_dev, 1));
  return SN_OK;
}

// ---------------------------------------------------------------------------- forward
static const float* op_output(sn_replica* r, int i, const float* x, int rows) {
  // output pointer of op i (x for i == -1)
  if (i < 0) return x;
  const Op& op = r->model->ops[i];
  if (op.kind == OP_FLATTEN) return op_output(r, i - 1, x, rows);
  if (op.kind == OP_LSTM && !op.ret_seq) return r->lstm_h[i] + (int64_t)op.T * r->model->batch * op.H;
  return r->act[i];
}

static LstmWeights lstm_weights(sn_replica* r, const Op& op, float* base) {
  LstmWeights w{};
  for (int gi = 0; gi < 4; ++gi) {
    w.wk[gi] = param_ptr(r, base, op.lstm_p[gi][0]);
    w.wr[gi] = param_ptr(r, base, op.lstm_p[gi][1]);
    w.b[gi] = param_ptr(r, base, op.lstm_p[gi][2]);
  }
  return w;
}

static BatchNormArgs batchnorm_args(sn_replica* r, const Op& op, int i) {
  const int64_t c = align_up(op.out_dims.back(), 64);
  float* b = r->bn_buf[i];
  return BatchNormArgs{param_ptr(r, r->w, op.bn_p[1]), param_ptr(r, r->w, op.bn_p[0]), param_ptr(r, r->w, op.bn_p[2]),
                       param_ptr(r, r->w, op.bn_p[3]), b, b + c, b + 2 * c, b + 3 * c, b + 4 * c, b + 5 * c, op.bn_epsilon, op.bn_momentum,
                       op.bn_fused, b + 6 * c, b + 7 * c, b + 8 * c};
}

// skip_last: leave out the last op (the training pass fuses a Softmax output into the loss kernel)
// training: the model as the optimizer compiles it; false = frozen, as a trained model predicts (models/Model.scala:126-127).
//           Only batch normalisation tells the two apart.
static int forward(sn_replica* r, const float* x, int rows, bool skip_last = false, bool training = false) {
  sn_model* m = r->model;
  sn_ctx* ctx = r->ctx;
  const bool bf16 = (m->flags & SN_FLAG_GEMM_BF16) != 0;
  if (bf16 && r->bf_weights_stale) {
    for (size_t i = 0; i < m->ops.size(); ++i)
      if (dense_bf16_fast(m, m->ops[i]))
        SN_TRY(launch_cast_bf16(ctx, param_ptr(r, r->w, m->ops[i].w), m->ops[i].out_elems, (int)m->ops[i].in_elems,
                                (int)m->ops[i].out_elems, r->bf_w[i], nullptr, 0, 0.f, nullptr));
    r->bf_weights_stale = false;
  }
  std::vector<char> bf_ready(m->ops.size() + 1, 0);  // op i's bf16 input copies were written by op i-1's epilogue
  for (size_t i = 0; i + (skip_last ? 1 : 0) < m->ops.size(); ++i) {
    const Op& op = m->ops[i];
    const float* in = op_output(r, (int)i - 1, x, rows);
    switch (op.kind) {
      case OP_DENSE: {
        const int in_f = (int)op.in_elems, out_f = (int)op.out_elems;
        Epilogue ep;
        ep.out = r->act[i]; ep.ldo = out_f; ep.bias = param_ptr(r, r->w, op.b); ep.act = op.act; ep.act_param = op.act_param;
        if (dense_bf16_fast(m, op) && rows % 8 == 0) {
          // the bf16 copy of X unless the layer below already wrote it from its epilogue, then Y = X . W on the matrix cores
          if (!bf_ready[i]) SN_TRY(launch_cast_bf16(ctx, in, in_f, rows, in_f, r->bf_x[i], nullptr, 0, 0.f, nullptr));
          EpilogueBf16 eb;
          eb.e = ep;
          const bool in_kernel_act = op.act == SN_ACT_IDENTITY || op.act == SN_ACT_RELU;
          if (!in_kernel_act) { eb.e.bias = nullptr; eb.e.act = SN_ACT_IDENTITY; }  // sigmoid / tanh: a pass of their own below
          if (in_kernel_act && i + 1 < m->ops.size() && dense_bf16_fast(m, m->ops[i + 1])) {
            eb.out_bf = r->bf_x[i + 1];
            bf_ready[i + 1] = true;
            if (hidden_bf16_only(r, i, rows)) {  // the next layer and the backward pass read the bf16 copy and the sign bits
              eb.e.out = nullptr;
              eb.signs_out = r->bf_signs[i];
            }
          }
          SN_TRY(launch_gemm_bf16(ctx, GEMM_BF16_FORWARD, r->bf_x[i], in_f, r->bf_w[i], out_f, rows, out_f, in_f, eb));
          if (!in_kernel_act) SN_TRY(launch_bias_act(ctx, r->act[i], ep.bias, r->act[i], rows, out_f, op.act, op.act_param));
        } else if (!bf16 && dense_tiny_shape(rows, in_f, out_f, m->workspace_elems)) {  // a few units behind a short row: one launch
          SN_TRY(launch_dense_tiny_fwd(ctx, in, param_ptr(r, r->w, op.w), ep, rows, in_f, out_f));
        } else if (!bf16 && r->ws && dense_skinny_fwd_shape(rows, in_f, out_f, m->workspace_elems)) {
          // the logits of a Softmax output under the fused loss kernel: that kernel adds the partial sums itself
          const bool leave = r->leave_logit_parts && i + 2 == m->ops.size() && op.act == SN_ACT_IDENTITY && out_f <= SOFTMAX_PARTIALS_MAX_COLS;
          SN_TRY(launch_dense_skinny_fwd(ctx, in, param_ptr(r, r->w, op.w), ep, rows, in_f, out_f, r->ws, m->workspace_elems,
                                         leave ? &r->logit_parts : nullptr));
        } else {
          GemmDesc g{in, in_f, 1, param_ptr(r, r->w, op.w), out_f, 1, rows, out_f, in_f};
          SN_TRY(launch_gemm(ctx, g, ep, r->ws, m->workspace_elems, bf16));
        }
        break;
      }
      case OP_CONV: {
        ConvGeom g{rows, (int)op.in_dims[0], (int)op.in_dims[1], (int)op.in_dims[2], (int)op.out_dims[0], (int)op.out_dims[1],
                   (int)op.out_dims[2], op.kh, op.kw, op.sh, op.sw, op.pt, op.pl};
        Epilogue ep;
        ep.out = r->act[i]; ep.ldo = g.cout; ep.bias = param_ptr(r, r->w, op.b); ep.act = op.act; ep.act_param = op.act_param;
        SN_TRY(launch_conv_fwd(ctx, g, in, param_ptr(r, r->w, op.w), ep, r->ws, m->workspace_elems));
        break;
      }
      case OP_POOL:
        SN_TRY(launch_pool_fwd(ctx, op.pool_avg, in, r->act[i], r->arg[i], rows, (int)op.in_dims[0], (int)op.in_dims[1], (int)op.in_dims[2],
                                  (int)op.out_dims[0], (int)op.out_dims[1], op.kh, op.kw, op.sh, op.sw, op.pt, op.pl));
        break;
      case OP_FLATTEN:
        break;
      case OP_BIASACT:
        SN_TRY(launch_bias_act(ctx, in, param_ptr(r, r->w, op.b), r->act[i], (int64_t)rows * (op.out_elems / op.out_dims.back()),
                               (int)op.out_dims.back(), op.act, op.act_param));
        break;
      case OP_SOFTMAX:
        SN_TRY(launch_softmax_fwd(ctx, in, r->act[i], rows, (int)op.out_elems, (m->flags & SN_FLAG_STABLE_SOFTMAX) != 0));
        break;
      case OP_LSTM: {
        // time-major slices are laid out with the model's batch capacity so addresses do not depend on `rows`
        const int64_t bh = (int64_t)m->batch * op.H;
        const LstmWeights w = lstm_weights(r, op, r->w);
        const bool fused = lstm_step_fused_ok(op.F, op.H, in, w);
        // stateful: the first step starts from the carried state (slice 0 of the hidden slices otherwise stays zero)
        const bool carried = op.state_p[0] >= 0;
        if (carried)
          SN_HIP(hipMemcpyAsync(r->lstm_h[i], param_ptr(r, r->w, op.state_p[1]), (size_t)rows * op.H * sizeof(float), hipMemcpyDeviceToDevice,
                                ctx->stream));
        if (fused && op.T > 1 && lstm_sequence_fwd_ok(ctx, rows, op.F, op.H, in, w)) {  // every step in one launch (it reads the weights as they lie)
          SN_TRY(launch_lstm_sequence_fwd(ctx, in, op.T, op.F, carried ? 1 : 0, carried ? param_ptr(r, r->w, op.state_p[0]) : nullptr, rows, op.H,
                                          w, r->lstm_gates[i], r->lstm_c[i], r->lstm_h[i], bh));
          if (op.ret_seq) SN_TRY(launch_sequence_gather(ctx, r->lstm_h[i], bh, 1, r->act[i], rows, op.T, op.H));
          break;
        }
        if (fused) SN_TRY(launch_lstm_pack(ctx, w, op.F, op.H, r->lstm_pk_fwd[i], nullptr));  // the step kernels' LDS order
        for (int t = 0; t < op.T; ++t) {
          const float* h_prev = t == 0 && !carried ? nullptr : r->lstm_h[i] + (int64_t)t * bh;
          const float* c_prev = t == 0 ? (carried ? param_ptr(r, r->w, op.state_p[0]) : nullptr) : r->lstm_c[i] + (int64_t)(t - 1) * bh;
          if (fused) {
            SN_TRY(launch_lstm_step_fwd(ctx, in, t, op.T, op.F, h_prev, c_prev,
                                        rows, op.H, w, r->lstm_pk_fwd[i], r->lstm_gates[i] + (int64_t)t * bh * 4, r->lstm_c[i] + (int64_t)t * bh,
                                        r->lstm_h[i] + (int64_t)(t + 1) * bh));
            continue;
          }
          SN_TRY(launch_lstm_z(ctx, in, t, op.T, op.F, h_prev, rows, op.H, w, r->lstm_z, r->ws, m->workspace_elems));
          LstmGateArgs a{r->lstm_z, c_prev, r->lstm_gates[i] + (int64_t)t * bh * 4,
                         r->lstm_c[i] + (int64_t)t * bh, r->lstm_h[i] + (int64_t)(t + 1) * bh};
          SN_TRY(launch_lstm_gates_fwd(ctx, a, rows, op.H));
        }
        if (op.ret_seq) SN_TRY(launch_sequence_gather(ctx, r->lstm_h[i], bh, 1, r->act[i], rows, op.T, op.H));
        break;
      }
      case OP_BATCHNORM: {
        const int c = (int)op.out_dims.back();
        SN_TRY(launch_batchnorm_fwd(ctx, in, r->act[i], (int64_t)rows * (op.out_elems / c), c, batchnorm_args(r, op, (int)i), training, r->ws,
                                    m->workspace_elems));
        break;
      }
      case OP_SRNN: {
        // The state carried from step to step is the cell's product before bias and activation
        // (layer/RNN.scala:189-196), so the recurrence is r_t = x_t Wk + r_{t-1} Wr and only the last step's
        // output act(r + b) leaves the layer (RNN.scala:60-77 without returnSequence).
        const int64_t bh = (int64_t)m->batch * op.H;
        const LstmWeights w = lstm_weights(r, op, r->w);  // slot 0 only, no bias inside the recurrence
        const bool fused = lstm_step_fused_ok(op.F, op.H, in, w, 1);
        const bool carried = op.state_p[0] >= 0;  // stateful: slice 0 is the product the previous batch ended with
        if (carried)
          SN_HIP(hipMemcpyAsync(r->lstm_h[i], param_ptr(r, r->w, op.state_p[0]), (size_t)rows * op.H * sizeof(float), hipMemcpyDeviceToDevice,
                                ctx->stream));
        const bool whole = fused && op.T > 1 && rnn_sequence_fwd_ok(ctx, rows, op.F, op.H, in);
        if (whole)  // every step in one launch (it reads the weights as they lie)
          SN_TRY(launch_rnn_sequence_fwd(ctx, in, op.T, op.F, carried ? 1 : 0, rows, op.H, w.wk[0], w.wr[0], r->lstm_h[i], bh));
        else if (fused) SN_TRY(launch_lstm_pack(ctx, w, op.F, op.H, r->lstm_pk_fwd[i], nullptr, 1));  // the step kernel's LDS order
        for (int t = whole ? op.T : 0; t < op.T; ++t) {
          const float* r_prev = t == 0 && !carried ? nullptr : r->lstm_h[i] + (int64_t)t * bh;
          float* r_t = r->lstm_h[i] + (int64_t)(t + 1) * bh;
          if (fused) SN_TRY(launch_rnn_step_fwd(ctx, in, t, op.T, op.F, r_prev, rows, op.H, r->lstm_pk_fwd[i], r_t));
          else SN_TRY(launch_lstm_z(ctx, in, t, op.T, op.F, r_prev, rows, op.H, w, r_t, r->ws, m->workspace_elems, 1));
        }
        if (op.ret_seq) {  // every step's act(r_t + b), as (batch, time, units)
          SN_TRY(launch_sequence_gather(ctx, r->lstm_h[i], bh, 1, r->act[i], rows, op.T, op.H));
          SN_TRY(launch_bias_act(ctx, r->act[i], param_ptr(r, r->w, op.b), r->act[i], (int64_t)rows * op.T, op.H, op.act, op.act_param));
        } else {
          SN_TRY(launch_bias_act(ctx, r->lstm_h[i] + (int64_t)op.T * bh, param_ptr(r, r->w, op.b), r->act[i], rows, op.H, op.act,
                                 op.act_param));
        }
        break;
      }
    }
  }
  return SN_OK;
}

static int add_penalties(sn_replica* r, bool training) {
  for (auto& p : r->model->params)
    if (p.reg_kind != SN_REG_NONE && (training || p.penalty_when_frozen))
      SN_TRY(launch_penalty(r->ctx, r->w + p.info.offset, p.info.size, p.reg_kind, p.reg_lambda, r->loss_dev, r->loss_partials));
  return SN_OK;
}

// loss (+ penalty) into loss_dev; dp (may be null) receives d loss / d prediction
// want_value = false: only dp is wanted (a training step whose caller does not read the loss): the final reduction and
// the penalty terms, which only the value needs, are skipped
static int loss_of(sn_replica* r, const float* pred, const float* y, int rows, float* dp, bool training, bool want_value = true) {
  sn_model* m = r->model;
  if (m->loss == SN_LOSS_IDENTITY)
    SN_REQUIRE((int64_t)rows * m->out_elems == 1, "Identity loss needs a scalar model output");
  SN_TRY(launch_loss(r->ctx, m->loss, pred, y, dp, want_value ? r->loss_dev : nullptr, r->loss_partials, rows, (int)m->out_elems));
  return want_value ? add_penalties(r, training) : SN_OK;
}

// ---------------------------------------------------------------------------- backward
// The optimizer update of one bf16 Dense layer, as soon as its gradients are complete.  With more layers to come
// (`overlap`) the launch goes to the replica's second stream, behind an event that says the layer's products are done,
// and runs beside the products of the layers below; the last layer's goes to the compute stream.  Same kernel, same
// arithmetic as the one launch over the whole buffer: that one is a loop over elements, split here by layer.
static int update_dense_layer(sn_replica* r, const Op& op, bool overlap) {
  sn_model* m = r->model;
  sn_ctx* ctx = r->ctx;
  int64_t first = m->params[op.w].info.offset, end = first + m->params[op.w].info.size;
  if (op.b >= 0) {
    first = std::min<int64_t>(first, m->params[op.b].info.offset);
    end = std::max<int64_t>(end, m->params[op.b].info.offset + m->params[op.b].info.size);
  }
  hipStream_t compute = ctx->stream;
  if (overlap) {
    SN_HIP(hipEventRecord(r->ev_layer_ready, compute));
    SN_HIP(hipStreamWaitEvent(r->update_stream, r->ev_layer_ready, 0));
    ctx->stream = r->update_stream;
  }
  const int rc = launch_optimizer(ctx, r->opt, r->w + first, r->g + first, r->s[0] + first, r->s[1] ? r->s[1] + first : nullptr,
                                  r->s[2] ? r->s[2] + first : nullptr, end - first, r->pass_iter, r->bf_wflat ? r->bf_wflat + first : nullptr,
                                  ctx->seq_failed_dev);
  ctx->stream = compute;
  return rc;
}

// Starts at op `first` (the last op by default) whose output gradient lies in grad_buf[cur].
// first_dz_cast: the loss kernel has already left the bf16 copy of op `first`'s output gradient in bf_dz[first]
static int backward(sn_replica* r, const float* x, int rows, int first = -1, int cur = 0, bool first_dz_cast = false) {
  sn_model* m = r->model;
  sn_ctx* ctx = r->ctx;
  const bool bf16 = (m->flags & SN_FLAG_GEMM_BF16) != 0;
  if (first < 0) first = (int)m->ops.size() - 1;
  bool act_grad_done = false;  // the op above already applied this op's activation gradient
  bool pool_pending = false;   // the max pooling above a first-layer convolution left its backward pass to the filter gradient
  PoolGrad pool_grad;
  bool dz_handed_over = false;  // the bf16 Dense op above already wrote this op's dZ copies and bias-gradient block sums
  for (int i = first; i >= 0; --i) {  // grad_buf[cur] holds d loss / d (output of op i)
    const Op& op = m->ops[i];
    const float* in = op_output(r, i - 1, x, rows);
    float* dy = r->grad_buf[cur];
    float* dx = r->grad_buf[cur ^ 1];
    const bool need_dx = i > 0;
    switch (op.kind) {
      case OP_DENSE: {
        const int in_f = (int)op.in_elems, out_f = (int)op.out_elems;
        if (dense_bf16_fast(m, op) && rows % 8 == 0) {
          // one pass: dZ = act'(Y) * dY as bf16 (the fp32 dZ itself is not kept: its only other reader would be the bias
          // gradient, summed here per 64-row block from the fp32 values)
          const bool y_from_bf = hidden_bf16_only(r, (size_t)i, rows);
          const bool cast_by_loss = first_dz_cast && i == first;  // (an identity activation: dZ = dY; its column sums come from the fp32 dY)
          if (cast_by_loss) {
            if (op.b >= 0) SN_TRY(launch_col_sum(ctx, dy, out_f, param_ptr(r, r->g, op.b), rows, out_f, r->ws, m->workspace_elems));
          } else if (!dz_handed_over)
            SN_TRY(launch_cast_bf16(ctx, dy, out_f, rows, out_f, r->bf_dz[i],
                                    op.act != SN_ACT_IDENTITY && !y_from_bf ? r->act[i] : nullptr, op.act, op.act_param, nullptr,
                                    op.b >= 0 ? r->bf_colp : nullptr,
                                    op.act != SN_ACT_IDENTITY && y_from_bf ? r->bf_x[i + 1] : nullptr));
          dz_handed_over = false;
          if (op.b >= 0 && !cast_by_loss)
            SN_TRY(launch_col_sum(ctx, r->bf_colp, out_f, param_ptr(r, r->g, op.b), ceil_div(rows, 64), out_f, r->ws, m->workspace_elems));
          EpilogueBf16 ew;
          ew.e.out = param_ptr(r, r->g, op.w); ew.e.ldo = out_f;
          SN_TRY(launch_gemm_bf16(ctx, GEMM_BF16_DW, r->bf_x[i], in_f, r->bf_dz[i], out_f, in_f, out_f, rows, ew));  // dW = X^T . dZ
          if (need_dx) {
            EpilogueBf16 ex;
            ex.e.out = dx; ex.e.ldo = in_f;
            // A bf16 Dense layer below whose output only lives as a bf16 copy (ReLU at 0 or no activation) takes its dZ
            // straight from this product's epilogue: activation gradient, the bf16 cast and the bias gradient's block
            // sums, instead of an fp32 dX that a second kernel would read back, mask and cast.
            if (i > 0 && hidden_bf16_only(r, (size_t)i - 1, rows)) {
              const Op& below = m->ops[i - 1];
              ex.e.out = nullptr;
              ex.out_bf = r->bf_dz[i - 1];
              ex.grad_handover = true;
              ex.signs_in = below.act == SN_ACT_RELU ? r->bf_signs[i - 1] : nullptr;
              ex.col_partials = below.b >= 0 ? r->bf_colp : nullptr;
              dz_handed_over = true;
            }
            SN_TRY(launch_gemm_bf16(ctx, GEMM_BF16_DX, r->bf_dz[i], out_f, r->bf_w[i], out_f, rows, in_f, out_f, ex));  // dX = dZ . W^T
            cur ^= 1;
          }
          if (r->side_updates) SN_TRY(update_dense_layer(r, op, need_dx));  // (after dX: that product read the layer's bf16 weights)
          break;
        }
        if (!bf16 && r->ws && dense_tiny_shape(rows, in_f, out_f, m->workspace_elems)) {  // activation gradient, dX, dW and db in two launches
          SN_TRY(launch_dense_tiny_bwd(ctx, in, r->act[i], dy, param_ptr(r, r->w, op.w), need_dx ? dx : nullptr, param_ptr(r, r->g, op.w),
                                       param_ptr(r, r->g, op.b), rows, in_f, out_f, op.act, op.act_param, r->ws, m->workspace_elems));
          if (need_dx) cur ^= 1;
          break;
        }
        if (op.act != SN_ACT_IDENTITY) SN_TRY(launch_act_bwd(ctx, r->act[i], dy, dy, (int64_t)rows * out_f, op.act, op.act_param));
        if (!bf16 && dense_skinny_shape(rows, in_f, out_f)) {  // a few units behind many features: row streams, no matrix tiles
          // one launch for both gradients: the rows of dY are staged once
          SN_TRY(launch_dense_skinny_dw(ctx, in, dy, param_ptr(r, r->g, op.w), param_ptr(r, r->g, op.b), rows, in_f, out_f,
                                        need_dx ? param_ptr(r, r->w, op.w) : nullptr, need_dx ? dx : nullptr));
          if (need_dx) cur ^= 1;
          break;
        }
        {  // dW = X^T . dY (math/alg/AllKernels.scala:382-388)
          GemmDesc g{in, 1, in_f, dy, out_f, 1, in_f, out_f, rows};
          Epilogue ep;
          ep.out = param_ptr(r, r->g, op.w); ep.ldo = out_f;
          // the bias gradient (column sums of dY) is the product's row for an all-ones row of X^T: it rides along
          // unless the GEMM takes its 16-byte loaders, which have no such row
          // (with a single input feature X^T is also K-contiguous and takes another loader: plain column sums then)
          const bool ride = op.b >= 0 && in_f > 1 && !gemm_takes_fast_loaders(ctx, g, r->ws, m->workspace_elems);
          if (ride) {
            g.m = in_f + 1;
            g.a_ones_row = true;
            ep.row_index = in_f;
            ep.row_out = param_ptr(r, r->g, op.b);
          } else if (op.b >= 0) {
            SN_TRY(launch_col_sum(ctx, dy, out_f, param_ptr(r, r->g, op.b), rows, out_f, r->ws, m->workspace_elems));
          }
          SN_TRY(launch_gemm(ctx, g, ep, r->ws, m->workspace_elems, bf16));
        }
        if (need_dx) {  // dX = dY . W^T
          GemmDesc g{dy, out_f, 1, param_ptr(r, r->w, op.w), 1, out_f, rows, in_f, out_f};
          Epilogue ep;
          ep.out = dx; ep.ldo = in_f;
          SN_TRY(launch_gemm(ctx, g, ep, r->ws, m->workspace_elems, bf16));
          cur ^= 1;
        }
        break;
      }
      case OP_CONV: {
        ConvGeom g{rows, (int)op.in_dims[0], (int)op.in_dims[1], (int)op.in_dims[2], (int)op.out_dims[0], (int)op.out_dims[1],
                   (int)op.out_dims[2], op.kh, op.kw, op.sh, op.sw, op.pt, op.pl};
        const int64_t n_out = (int64_t)rows * op.out_elems;
        const PoolGrad* pool = pool_pending ? &pool_grad : nullptr;  // the pooling above left its backward pass to this product
        pool_pending = false;
        if (op.act != SN_ACT_IDENTITY && !act_grad_done && !pool) SN_TRY(launch_act_bwd(ctx, r->act[i], dy, dy, n_out, op.act, op.act_param));
        act_grad_done = false;
        if (op.b >= 0)
          SN_TRY(launch_col_sum(ctx, dy, g.cout, param_ptr(r, r->g, op.b), (int64_t)rows * g.ho * g.wo, g.cout, r->ws, m->workspace_elems));
        if (r->defer_now && r->ws_defer[i] && r->n_deferred < MAX_DEFERRED) {
          // the sum of this product's partial results waits for the optimizer launch of the step
          DeferredReduce& slot = r->deferred[r->n_deferred];
          slot = DeferredReduce{};
          ctx->defer = &slot;
          const int rc = launch_conv_wgrad(ctx, g, in, dy, param_ptr(r, r->g, op.w), r->ws_defer[i], m->workspace_elems, pool);
          ctx->defer = nullptr;
          SN_TRY(rc);
          if (slot.kind != 0) ++r->n_deferred;
        } else {
          SN_TRY(launch_conv_wgrad(ctx, g, in, dy, param_ptr(r, r->g, op.w), r->ws, m->workspace_elems, pool));
        }
        if (need_dx) {
          SN_TRY(launch_conv_dgrad(ctx, g, dy, param_ptr(r, r->w, op.w), dx, r->ws, m->workspace_elems));
          cur ^= 1;
        }
        break;
      }
      case OP_POOL:
        if (need_dx) {
          // a convolution with an activation right below: its activation gradient rides along (one pass less over the tensor)
          const Op& below = m->ops[i - 1];
          const bool fuse = below.kind == OP_CONV && below.act != SN_ACT_IDENTITY;
          // The first layer's convolution needs its output gradient for the filter gradient only (and has no bias to sum it
          // for): where that product runs as the direct kernel, the kernel forms the gradient itself from what this pooling
          // would have read, and the pooling's backward launch and the tensor it writes are not needed.
          if (i == 1 && below.kind == OP_CONV && below.b < 0 && !op.pool_avg && op.kh == 2 && op.kw == 2 && rows > 0) {
            const ConvGeom cg{rows, (int)below.in_dims[0], (int)below.in_dims[1], (int)below.in_dims[2], (int)below.out_dims[0],
                              (int)below.out_dims[1], (int)below.out_dims[2], below.kh, below.kw, below.sh, below.sw, below.pt, below.pl};
            const bool deferred = r->defer_now && r->ws_defer[0] && r->n_deferred < MAX_DEFERRED;
            const bool aligned = ((reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(r->arg[i]) | reinterpret_cast<uintptr_t>(r->act[i - 1])) & 15u) == 0;
            if (aligned && conv_wgrad_is_direct(ctx, cg, deferred ? r->ws_defer[0] : r->ws, m->workspace_elems, true)) {
              pool_grad.dy = dy; pool_grad.arg = r->arg[i]; pool_grad.y = r->act[i - 1];
              pool_grad.ho = (int)op.out_dims[0]; pool_grad.wo = (int)op.out_dims[1];
              pool_grad.sh = op.sh; pool_grad.sw = op.sw; pool_grad.pt = op.pt; pool_grad.pl = op.pl;
              pool_grad.act = below.act; pool_grad.act_param = below.act_param;
              pool_pending = true;
              break;
            }
          }
          SN_TRY(launch_pool_bwd(ctx, op.pool_avg, dy, r->arg[i], dx, rows, (int)op.in_dims[0], (int)op.in_dims[1], (int)op.in_dims[2],
                                    (int)op.out_dims[0], (int)op.out_dims[1], op.kh, op.kw, op.sh, op.sw, op.pt, op.pl,
                                    fuse ? r->act[i - 1] : nullptr, below.act, below.act_param));
          act_grad_done = fuse;
          cur ^= 1;
        }
        break;
      case OP_FLATTEN:
        break;
      case OP_BIASACT: {
        const int cols = (int)op.out_dims.back();
        const int64_t n_out = (int64_t)rows * op.out_elems;
        if (op.act != SN_ACT_IDENTITY) SN_TRY(launch_act_bwd(ctx, r->act[i], dy, dy, n_out, op.act, op.act_param));
        if (op.b >= 0) SN_TRY(launch_col_sum(ctx, dy, cols, param_ptr(r, r->g, op.b), n_out / cols, cols, r->ws, m->workspace_elems));
        break;
      }
      case OP_SOFTMAX:
        SN_TRY(launch_softmax_bwd(ctx, r->act[i], dy, dx, rows, (int)op.out_elems));
        cur ^= 1;
        break;
      case OP_LSTM: {
        // the weight-gradient GEMM reads the saved steps as one [T*rows, .] matrix, so the slices must be full
        SN_REQUIRE(rows == m->batch, "LSTM training needs rows == batch (%d), got %d", m->batch, rows);
        const int64_t bh = (int64_t)m->batch * op.H;
        const LstmWeights w = lstm_weights(r, op, r->w);
        const float* dh = op.ret_seq ? nullptr : dy;  // gradient of the last hidden state (a returned sequence adds its own per step)
        int hb = 0, dh_parts = op.ret_seq ? 0 : 1;
        const bool fused = lstm_step_fused_ok(op.F, op.H, in, w);
        // one launch per step (gate gradients + the product that carries dh back) where the layer's shape allows it
        const bool fused_bwd = fused && lstm_step_bwd_fused_ok(op.H, w);
        // every reverse step in one launch where the whole grid fits the device; the input gradients follow per step
        const bool whole = fused && op.T > 1 && lstm_sequence_bwd_ok(ctx, rows, op.H, w);
        LstmGrads gr;
        for (int gi = 0; gi < 4; ++gi) {
          gr.wk[gi] = param_ptr(r, r->g, op.lstm_p[gi][0]);
          gr.wr[gi] = param_ptr(r, r->g, op.lstm_p[gi][1]);
          gr.b[gi] = param_ptr(r, r->g, op.lstm_p[gi][2]);
        }
        int wgrad_parts = 0;  // > 0: the backward launch has left the weight gradient's partial sums in the workspace
        if (whole) {
          SN_TRY(launch_lstm_sequence_bwd(ctx, r->lstm_gates[i], r->lstm_c[i], param_ptr(r, r->w, op.state_p[0]), op.ret_seq ? nullptr : dy,
                                          op.ret_seq ? dy : nullptr, op.T, rows, op.H, w, r->lstm_dz[i], bh, in, r->lstm_h[i], op.F, r->ws,
                                          m->workspace_elems, &wgrad_parts));
          if (wgrad_parts > 0) SN_TRY(launch_lstm_wgrad_reduce(ctx, r->ws, wgrad_parts, op.F, op.H, 4, gr));  // before the workspace's next user
          if (need_dx)
            for (int t = op.T - 1; t >= 0; --t)
              SN_TRY(launch_lstm_dx(ctx, r->lstm_dz[i] + (int64_t)t * bh * 4, rows, op.H, op.F, t, op.T, w, dx, r->ws, m->workspace_elems));
        } else if (fused_bwd && op.T > 1) SN_TRY(launch_lstm_pack_bwd(ctx, w, op.H, r->lstm_pk_dh[i]));
        else if (fused && op.T > 1) SN_TRY(launch_lstm_pack(ctx, w, op.F, op.H, nullptr, r->lstm_pk_dh[i]));
        float* dcbuf[2] = {r->lstm_dc, r->lstm_dc2};
        int db = 0;
        for (int t = whole ? -1 : op.T - 1; t >= 0; --t) {
          LstmGateBwdArgs a{r->lstm_gates[i] + (int64_t)t * bh * 4, r->lstm_c[i] + (int64_t)t * bh,
                            t == 0 ? param_ptr(r, r->w, op.state_p[0]) : r->lstm_c[i] + (int64_t)(t - 1) * bh, dh, r->lstm_dc,
                            r->lstm_dz[i] + (int64_t)t * bh * 4, t == op.T - 1 ? 1 : 0, dh_parts, bh};
          if (op.ret_seq) {  // this step's own output gradient joins what the later steps carried back
            a.dy_seq = dy + (int64_t)t * op.H;
            a.dy_seq_ld = (int64_t)op.T * op.H;
          }
          if (fused_bwd) {
            SN_TRY(launch_lstm_step_bwd(ctx, a, t == op.T - 1 ? nullptr : dcbuf[db], dcbuf[db ^ 1], t > 0 ? r->lstm_pk_dh[i] : nullptr,
                                        r->lstm_dh[hb], bh, rows, op.H));
            db ^= 1;
            if (need_dx) SN_TRY(launch_lstm_dx(ctx, a.dz, rows, op.H, op.F, t, op.T, w, dx, r->ws, m->workspace_elems));
            dh = r->lstm_dh[hb];
            dh_parts = lstm_bwd_parts(op.H);
            hb ^= 1;
            continue;
          }
          SN_TRY(launch_lstm_gates_bwd(ctx, a, rows, op.H));
          if (need_dx) SN_TRY(launch_lstm_dx(ctx, a.dz, rows, op.H, op.F, t, op.T, w, dx, r->ws, m->workspace_elems));
          if (t > 0) {
            if (fused) {  // four per-gate partial products; the next gate-gradient kernel adds them
              SN_TRY(launch_lstm_step_dh(ctx, a.dz, rows, op.H, r->lstm_pk_dh[i], r->lstm_dh[hb], bh));
              dh_parts = 4;
            } else {
              SN_TRY(launch_lstm_dh(ctx, a.dz, rows, op.H, w, r->lstm_dh[hb], r->ws, m->workspace_elems));
              dh_parts = 1;
            }
            dh = r->lstm_dh[hb];
            hb ^= 1;
          }
        }
        if (wgrad_parts == 0) SN_TRY(launch_lstm_wgrad(ctx, in, r->lstm_h[i], r->lstm_dz[i], rows, op.T, op.F, op.H, gr, r->ws, m->workspace_elems));
        if (need_dx) cur ^= 1;
        break;
      }
      case OP_BATCHNORM: {
        const int c = (int)op.out_dims.back();
        // a convolution right below: its activation gradient rides along in the input-gradient pass (x is its output)
        const bool fuse = need_dx && m->ops[i - 1].kind == OP_CONV && m->ops[i - 1].act != SN_ACT_IDENTITY;
        SN_TRY(launch_batchnorm_bwd(ctx, in, dy, need_dx ? dx : nullptr, (int64_t)rows * (op.out_elems / c), c, batchnorm_args(r, op, i),
                                    param_ptr(r, r->g, op.bn_p[0]), param_ptr(r, r->g, op.bn_p[1]), r->ws, m->workspace_elems,
                                    fuse ? m->ops[i - 1].act : SN_ACT_IDENTITY, fuse ? m->ops[i - 1].act_param : 0.f));
        act_grad_done = fuse;
        if (need_dx) cur ^= 1;
        break;
      }
      case OP_SRNN: {
        SN_REQUIRE(rows == m->batch, "RNN training needs rows == batch (%d), got %d", m->batch, rows);
        const int64_t bh = (int64_t)m->batch * op.H;
        const LstmWeights w = lstm_weights(r, op, r->w);
        float* dr = r->lstm_dz[i] + (int64_t)(op.T - 1) * bh;
        if (op.ret_seq) {
          // every step has an output: dz = act'(out) * dout over the whole (batch, time, units) tensor, in place; each
          // step below adds its slice to the gradient carried back from the step after it
          SN_TRY(launch_act_bwd(ctx, r->act[i], dy, dy, (int64_t)rows * op.T * op.H, op.act, op.act_param));
          if (op.b >= 0)
            SN_TRY(launch_col_sum(ctx, dy, op.H, param_ptr(r, r->g, op.b), (int64_t)rows * op.T, op.H, r->ws, m->workspace_elems));
        } else {
          // bias and activation touch the last step only; every earlier step acts through the carried state
          SN_TRY(launch_act_bwd(ctx, r->act[i], dy, dr, (int64_t)rows * op.H, op.act, op.act_param));
          if (op.b >= 0) SN_TRY(launch_col_sum(ctx, dr, op.H, param_ptr(r, r->g, op.b), rows, op.H, r->ws, m->workspace_elems));
        }
        const bool fused = lstm_step_fused_ok(op.F, op.H, in, w, 1);
        const bool whole = fused && op.T > 1 && rnn_sequence_bwd_ok(ctx, rows, op.H, w.wr[0]);
        if (fused && op.T > 1 && !whole) SN_TRY(launch_lstm_pack(ctx, w, op.F, op.H, nullptr, r->lstm_pk_dh[i], 1));  // the step kernel's LDS order
        LstmGrads gr{};
        gr.wk[0] = param_ptr(r, r->g, op.lstm_p[0][0]);
        gr.wr[0] = param_ptr(r, r->g, op.lstm_p[0][1]);
        int wgrad_parts = 0;  // > 0: the backward launch has left the weight gradient's partial sums in the workspace
        if (whole) {  // every step in one launch (it adds a returned sequence's output gradients itself), then the input gradients
          dr = r->lstm_dz[i] + (int64_t)(op.T - 1) * bh;
          if (op.ret_seq) SN_TRY(launch_step_slice_add(ctx, dr, dy + (int64_t)(op.T - 1) * op.H, (int64_t)op.T * op.H, rows, op.H, false));
          SN_TRY(launch_rnn_sequence_bwd(ctx, r->lstm_dz[i], op.ret_seq ? dy : nullptr, op.T, rows, op.H, w.wr[0], bh, in, r->lstm_h[i], op.F,
                                         r->ws, m->workspace_elems, &wgrad_parts));
          if (wgrad_parts > 0) SN_TRY(launch_lstm_wgrad_reduce(ctx, r->ws, wgrad_parts, op.F, op.H, 1, gr));  // before the workspace's next user
          if (need_dx)
            for (int t = op.T - 1; t >= 0; --t)
              SN_TRY(launch_lstm_dx(ctx, r->lstm_dz[i] + (int64_t)t * bh, rows, op.H, op.F, t, op.T, w, dx, r->ws, m->workspace_elems, 1));
        }
        for (int t = whole ? -1 : op.T - 1; t >= 0; --t) {
          dr = r->lstm_dz[i] + (int64_t)t * bh;
          if (op.ret_seq) SN_TRY(launch_step_slice_add(ctx, dr, dy + (int64_t)t * op.H, (int64_t)op.T * op.H, rows, op.H, t < op.T - 1));
          if (need_dx) SN_TRY(launch_lstm_dx(ctx, dr, rows, op.H, op.F, t, op.T, w, dx, r->ws, m->workspace_elems, 1));
          if (t > 0) {
            if (fused) SN_TRY(launch_lstm_step_dh(ctx, dr, rows, op.H, r->lstm_pk_dh[i], dr - bh, 0, 1));
            else SN_TRY(launch_lstm_dh(ctx, dr, rows, op.H, w, dr - bh, r->ws, m->workspace_elems, 1));
          }
        }
        if (wgrad_parts == 0) SN_TRY(launch_lstm_wgrad(ctx, in, r->lstm_h[i], r->lstm_dz[i], rows, op.T, op.F, op.H, gr, r->ws, m->workspace_elems, 1));
        if (need_dx) cur ^= 1;
        break;
      }
    }
  }
  for (auto& p : m->params)
    if (p.reg_kind != SN_REG_NONE)
      SN_TRY(launch_penalty_grad(ctx, r->w + p.info.offset, r->g + p.info.offset, p.info.size, p.reg_kind, p.reg_lambda));
  return SN_OK;
}

static int check_rows(sn_replica* r, int rows) {
  SN_REQUIRE(rows >= 1 && rows <= r->model->batch, "rows must be in 1..%d (the model's batch), got %d", r->model->batch, rows);
  return SN_OK;
}

static int read_loss(sn_replica* r, float* loss_host) {
  if (!loss_host) return SN_OK;
  SN_HIP(hipMemcpyAsync(loss_host, r->loss_dev, sizeof(float), hipMemcpyDeviceToHost, r->ctx->stream));
  SN_HIP(hipStreamSynchronize(r->ctx->stream));
  return check_async(r->ctx);
}

// want_loss = false: the caller does not read this step's loss value (the steps inside an epoch, sn_step / sn_grad without a
// loss pointer), so the kernels that only finish the scalar are not launched
// Dense(H, act) >> Dense(C) >> Softmax under CategoricalCrossentropy, small enough for the two-launch training pass
static bool mlp2_path(const sn_model* m) {
  if (m->ops.size() != 3 || m->loss != SN_LOSS_CATEGORICAL_CROSSENTROPY || (m->flags & SN_FLAG_GEMM_BF16)) return false;
  const Op& d1 = m->ops[0];
  const Op& d2 = m->ops[1];
  if (d1.kind != OP_DENSE || d2.kind != OP_DENSE || d2.act != SN_ACT_IDENTITY || m->ops[2].kind != OP_SOFTMAX) return false;
  const int64_t scratch = (int64_t)m->batch * m->max_act_elems;
  return mlp2_fused_ok(m->batch, (int)d1.in_elems, (int)d1.out_elems, (int)d2.out_elems, scratch, scratch);
}

// for_update: the optimizer update of the same step follows (update()), which may then take over reductions this pass
// leaves open; without it (sn_grad) every gradient is complete when the pass returns.
static int grad_pass_body(sn_replica* r, const float* x, const float* y, int rows, bool want_loss);
// A training step of a model made of bf16 Dense layers only (and parameter-free ops), without penalties: every layer is
// updated as soon as its gradients are complete, on a second stream, and update() has nothing left to launch.
static int begin_side_updates(sn_replica* r, int rows, bool for_update) {
  sn_model* m = r->model;
  r->side_updates = false;
  if (!for_update || !r->has_opt || !(m->flags & SN_FLAG_GEMM_BF16) || rows % 8 != 0 || m->trainable_runs.size() != 1) return SN_OK;
  int dense = 0;
  for (const Op& op : m->ops) {
    if (op.kind == OP_DENSE) {
      if (!dense_bf16_fast(m, op)) return SN_OK;
      ++dense;
    } else if (op.kind != OP_SOFTMAX && op.kind != OP_FLATTEN) {
      return SN_OK;  // (layers with parameters or state of their own keep the one launch over the whole buffer)
    }
  }
  if (dense < 2) return SN_OK;
  for (const auto& p : m->params)
    if (p.reg_kind != SN_REG_NONE) return SN_OK;
  if (!r->update_stream) {
    hipStream_t st = nullptr;
    SN_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));  // (default priority, as the compute stream)
    hipEvent_t a = nullptr, b = nullptr;
    if (hipEventCreateWithFlags(&a, hipEventDisableTiming) != hipSuccess || hipEventCreateWithFlags(&b, hipEventDisableTiming) != hipSuccess) {
      if (a) (void)hipEventDestroy(a);
      (void)hipStreamDestroy(st);
      return fail(SN_E_HIP, "events for the update stream could not be created");
    }
    r->update_stream = st;
    r->ev_layer_ready = a;
    r->ev_updates_done = b;
  }
  r->side_updates = true;
  return SN_OK;
}
// update_iter > 0: the optimizer update with that iteration number follows (update()), and may be taken over by this pass
static int grad_pass(sn_replica* r, const float* x, const float* y, int rows, bool want_loss, int update_iter = 0) {
  const bool for_update = update_iter > 0;
  r->n_deferred = 0;
  r->updated_in_pass = false;
  r->pass_iter = update_iter;
  r->defer_now = for_update && r->fuse_finish;
  SN_TRY(begin_side_updates(r, rows, for_update));
  int rc = grad_pass_body(r, x, y, rows, want_loss);
  r->defer_now = false;
  if (rc != SN_OK) r->n_deferred = 0;
  if (r->side_updates) {  // the compute stream goes on only after every layer's update (also after a failed pass: nothing is left running)
    r->side_updates = false;
    const hipError_t e1 = hipEventRecord(r->ev_updates_done, r->update_stream);
    const hipError_t e2 = e1 == hipSuccess ? hipStreamWaitEvent(r->ctx->stream, r->ev_updates_done, 0) : e1;
    if (e2 != hipSuccess) {
      (void)hipStreamSynchronize(r->update_stream);
      if (rc == SN_OK) rc = fail(SN_E_HIP, "joining the update stream failed: %s", hipGetErrorString(e2));
    }
    if (rc == SN_OK) r->updated_in_pass = true;
    else r->bf_weights_stale = true;  // some layers may have moved: their bf16 copies are rebuilt from the fp32 weights
  }
  r->pass_iter = update_iter;  // (kept for update()'s check)
  return rc;
}
static int grad_pass_body(sn_replica* r, const float* x, const float* y, int rows, bool want_loss) {
  sn_model* m = r->model;
  const int last = (int)m->ops.size() - 1;
  if (mlp2_path(m)) {
    const Op& d1 = m->ops[0];
    const Op& d2 = m->ops[1];
    // A training step of a model without penalties: the second launch applies the optimizer to every gradient value it
    // finishes (the pass touches every parameter of the model exactly once), and update() has nothing left to launch.
    Mlp2Update u;
    const Mlp2Update* upd = nullptr;
    bool penalties = false;
    for (const auto& p : m->params) penalties = penalties || p.reg_kind != SN_REG_NONE;
    if (r->pass_iter > 0 && r->has_opt && !penalties) {
      u.kind = r->opt.kind;
      u.n_states = opt_state_count(r->opt.kind);
      u.p = make_opt_scalars(r->opt, r->pass_iter);
      u.w = r->w; u.g = r->g; u.s0 = r->s[0]; u.s1 = r->s[1]; u.s2 = r->s[2];
      upd = &u;
      r->updated_in_pass = true;
    }
    SN_TRY(launch_mlp2_grad(r->ctx, x, y, param_ptr(r, r->w, d1.w), param_ptr(r, r->w, d1.b), param_ptr(r, r->w, d2.w), param_ptr(r, r->w, d2.b), rows,
                            (int)d1.in_elems, (int)d1.out_elems, (int)d2.out_elems, d1.act, d1.act_param,
                            (m->flags & SN_FLAG_STABLE_SOFTMAX) != 0, r->act[0], r->act[1], r->act[2], r->grad_buf[0], r->grad_buf[1],
                            r->loss_partials, want_loss ? r->loss_dev : nullptr, param_ptr(r, r->g, d1.w), param_ptr(r, r->g, d1.b),
                            param_ptr(r, r->g, d2.w), param_ptr(r, r->g, d2.b), upd));
    if (want_loss) SN_TRY(add_penalties(r, true));
    for (auto& p : m->params)
      if (p.reg_kind != SN_REG_NONE)
        SN_TRY(launch_penalty_grad(r->ctx, r->w + p.info.offset, r->g + p.info.offset, p.info.size, p.reg_kind, p.reg_lambda));
    return SN_OK;
  }
  if (last >= 1 && m->ops[last].kind == OP_SOFTMAX && m->loss == SN_LOSS_CATEGORICAL_CROSSENTROPY) {
    // Softmax output under CategoricalCrossentropy: probabilities, loss and d loss / d logits in one kernel
    bool cast_by_loss = false;
    r->logit_parts = 0;
    r->leave_logit_parts = m->ops[last - 1].kind == OP_DENSE;
    const int rc = forward(r, x, rows, true, true);
    r->leave_logit_parts = false;
    SN_TRY(rc);
    if (r->logit_parts > 0) {
      const Op& d = m->ops[last - 1];
      SN_TRY(launch_softmax_cce_partials(r->ctx, r->ws, r->logit_parts, param_ptr(r, r->w, d.b), r->act[last - 1], y, nullptr, r->grad_buf[1],
                                         want_loss ? r->loss_dev : nullptr, r->loss_partials, rows, (int)m->ops[last].out_elems,
                                         (m->flags & SN_FLAG_STABLE_SOFTMAX) != 0));
    } else {
      // a bf16 Dense layer without activation right below: the kernel also writes the bf16 copy of dZ that layer's products read
      const Op& below = m->ops[last - 1];
      cast_by_loss = below.kind == OP_DENSE && below.act == SN_ACT_IDENTITY && dense_bf16_fast(m, below) && rows % 8 == 0 && r->bf_dz[last - 1];
      // (the probabilities have no reader in a gradient pass: rows that fit in registers do not store them)
      SN_TRY(launch_softmax_cce(r->ctx, op_output(r, last - 1, x, rows), y, (int)m->ops[last].out_elems <= 1024 ? nullptr : r->act[last], r->grad_buf[1],
                                want_loss ? r->loss_dev : nullptr,
                                r->loss_partials, rows, (int)m->ops[last].out_elems, (m->flags & SN_FLAG_STABLE_SOFTMAX) != 0,
                                cast_by_loss ? r->bf_dz[last - 1] : nullptr));
    }
    if (want_loss) SN_TRY(add_penalties(r, true));
    return backward(r, x, rows, last - 1, 1, cast_by_loss);
  }
  SN_TRY(forward(r, x, rows, false, true));
  const float* pred = op_output(r, (int)r->model->ops.size() - 1, x, rows);
  SN_TRY(loss_of(r, pred, y, rows, r->grad_buf[0], true, want_loss));
  SN_TRY(backward(r, x, rows));
  return SN_OK;
}

static int update(sn_replica* r, int iter) {
  SN_REQUIRE(r->has_opt, "replica was created without an optimizer");
  sn_model* m = r->model;
  // A one-launch recurrent kernel of an earlier pass that gave up is reported before anything moves (the flag sits in
  // pinned host memory: no synchronisation needed to look); one of THIS step's passes that gives up, which the host
  // cannot know yet, makes the optimizer launch below leave weights and optimizer state as they are.
  if (r->ctx->seq_gave_up && *(volatile int*)r->ctx->seq_gave_up != 0) {
    // kernels queued behind the one that gave up may do the same: let them end, so that this is reported once
    SN_HIP(hipStreamSynchronize(r->ctx->stream));
    return check_async(r->ctx);
  }
  // weights move by the algorithm, layer state by the layer's own rule (`nextWeights ++ nextState`, Optimizer.scala:142-144);
  // the statistics are those of the gradient pass that has just run.  In bf16 mode the optimizer writes the bf16 copy of
  // what it updates in the same pass (every Dense weight is trainable), so the copies stay current.
  if (r->updated_in_pass) {  // the gradient pass has applied the update itself (with this iteration number)
    SN_REQUIRE(r->pass_iter == iter, "update(%d) behind a gradient pass that was run for iteration %d", iter, r->pass_iter);
    r->updated_in_pass = false;
  } else if (r->n_deferred > 0) {  // one launch: the open gradient sums, then the update of the whole buffer
    const int nd = r->n_deferred;
    r->n_deferred = 0;
    int64_t holes[2 * MAX_FINISH_HOLES];
    int n_holes = 0;
    int64_t at = 0;
    for (const auto& run : m->trainable_runs) {  // what lies between the runs is not the optimizer's
      if (run.first > at) { holes[2 * n_holes] = at; holes[2 * n_holes + 1] = run.first; ++n_holes; }
      at = run.second;
    }
    SN_TRY(launch_finish(r->ctx, r->opt, r->w, r->g, r->s[0], r->s[1], r->s[2], at, iter, r->deferred, nd, r->ctx->seq_failed_dev, holes, n_holes));
  } else
  for (const auto& run : m->trainable_runs)
    SN_TRY(launch_optimizer(r->ctx, r->opt, r->w + run.first, r->g + run.first, r->s[0] + run.first, r->s[1] ? r->s[1] + run.first : nullptr,
                            r->s[2] ? r->s[2] + run.first : nullptr, run.second - run.first, iter,
                            r->bf_wflat ? r->bf_wflat + run.first : nullptr, r->ctx->seq_failed_dev));
  for (size_t i = 0; i < m->ops.size(); ++i) {
    const Op& op = m->ops[i];
    if (op.kind == OP_BATCHNORM)
      SN_TRY(launch_batchnorm_moving(r->ctx, batchnorm_args(r, op, (int)i), param_ptr(r, r->w, op.bn_p[2]),
                                     param_ptr(r, r->w, op.bn_p[3]), (int)op.out_dims.back()));
    if ((op.kind == OP_LSTM || op.kind == OP_SRNN) && op.state_p[0] >= 0) {
      // the state the last step left is where the next batch starts (layer/RNN.scala:66-72; LSTM: c and h, :338; simple
      // cell: its product, :195-196).  Training passes always run full batches, so whole slices move.
      const size_t bytes = (size_t)m->batch * op.H * sizeof(float);
      const int64_t bh = (int64_t)m->batch * op.H;
      const float* last_h = r->lstm_h[i] + (int64_t)op.T * bh;
      if (op.kind == OP_LSTM) {
        SN_HIP(hipMemcpyAsync(param_ptr(r, r->w, op.state_p[0]), r->lstm_c[i] + (int64_t)(op.T - 1) * bh, bytes, hipMemcpyDeviceToDevice, r->ctx->stream));
        SN_HIP(hipMemcpyAsync(param_ptr(r, r->w, op.state_p[1]), last_h, bytes, hipMemcpyDeviceToDevice, r->ctx->stream));
      } else {
        SN_HIP(hipMemcpyAsync(param_ptr(r, r->w, op.state_p[0]), last_h, bytes, hipMemcpyDeviceToDevice, r->ctx->stream));
      }
    }
  }
  return SN_OK;
}

static int tensor_io(sn_replica* r, float* base, int index, float* host, const float* src, int64_t n, bool weights_only = false) {
  sn_model* m = r->model;
  SN_REQUIRE(index >= 0 && index < (int)m->params.size(), "parameter index %d out of range (model has %zu)", index, m->params.size());
  const sn_param_info& p = m->params[index].info;
  SN_REQUIRE(!weights_only || p.trainable, "%s is layer state: it has no gradient and no optimizer state", p.path);
  SN_REQUIRE(n == p.size, "parameter %s holds %lld elements, caller passed %lld", p.path, (long long)p.size, (long long)n);
  SN_REQUIRE(base != nullptr, "replica has no such buffer");
  if (src) {
    SN_HIP(hipMemcpyAsync(base + p.offset, src, (size_t)n * sizeof(float), hipMemcpyHostToDevice, r->ctx->stream));
    SN_HIP(hipStreamSynchronize(r->ctx->stream));  // the caller may reuse `src` right away
  } else {
    SN_HIP(hipMemcpyAsync(host, base + p.offset, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, r->ctx->stream));
    SN_HIP(hipStreamSynchronize(r->ctx->stream));
    return check_async(r->ctx);  // what was read may come from a pass whose one-launch recurrent kernel gave up
  }
  return SN_OK;
}

}  // namespace sn

// ---- the forward pass for callers that cannot allocate -----------------------------------------------------------
// Every intermediate of the pass (layer outputs, pooling window offsets, BatchNorm vectors, the GEMM workspace)
// lives in one file-scope device array instead of the replica's own allocations.  Each device the library runs on
// holds its own copy of the array at its own address; the address is looked up once per device.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)64 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
static unsigned char* g_scratch_ptr[STATIC_SCRATCH_MAX_DEVICES];  // device address of `scratch` per device, null until looked up
static std::mutex g_scratch_mutex;

namespace sn {
// Called by sn_ctx_create with `device` current.
int static_scratch_init(int device) {
  SN_REQUIRE(device >= 0 && device < STATIC_SCRATCH_MAX_DEVICES, "device %d is beyond the %d the library keeps scratch addresses for", device,
             STATIC_SCRATCH_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device]) return SN_OK;
  unsigned char* ptr = nullptr;
  SN_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
  SN_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null address for the static scratch array");
  g_scratch_ptr[device] = ptr;
  return SN_OK;
}
}  // namespace sn

using namespace sn;

extern "C" {

int sn_model_create(sn_ctx* ctx, const sn_layer_desc* layers, int32_t n_layers, int32_t loss, const int64_t* input_dims,
                    int32_t input_rank, int32_t batch, uint32_t flags, sn_model** out) {
  SN_REQUIRE(out != nullptr, "sn_model_create: out is NULL");
  *out = nullptr;
  if (!ctx || ctx->magic != CTX_MAGIC) return fail(SN_E_STATE, "invalid or destroyed context handle");
  SN_REQUIRE(layers && n_layers >= 1, "at least 1 layer is required");
  SN_REQUIRE(loss >= SN_LOSS_IDENTITY && loss <= SN_LOSS_CATEGORICAL_CROSSENTROPY, "unknown loss %d", loss);
  SN_REQUIRE(input_dims && input_rank >= 1 && input_rank < SN_MAX_RANK, "input rank must be in 1..%d", SN_MAX_RANK - 1);
  SN_REQUIRE(batch >= 1, "batch must be positive");
  sn_model* m = new sn_model();
  m->magic = MODEL_MAGIC;
  m->ctx = ctx;
  m->loss = loss;
  m->flags = flags;
  m->batch = batch;
  m->flat_elems = 0;
  m->live_replicas = 0;
  for (int i = 0; i < input_rank; ++i) {
    if (input_dims[i] < 1) {
      delete m;
      return fail(SN_E_INVALID, "input dimension %d must be positive", i);
    }
    m->input_dims.push_back(input_dims[i]);
  }
  m->in_elems = prod(m->input_dims);
  int rc = build_plan(m, layers, n_layers);
  if (rc == SN_OK && (int64_t)batch * m->max_act_elems > (int64_t)INT32_MAX)
    rc = fail(SN_E_INVALID, "batch x largest activation exceeds 2^31 elements");
  if (rc != SN_OK) {
    delete m;
    return rc;
  }
  ctx->live_models++;
  *out = m;
  return SN_OK;
}

int sn_model_destroy(sn_model* model) {
  SN_TRY(check_model(model));
  if (model->live_replicas != 0) return fail(SN_E_STATE, "model still has %d live replicas", model->live_replicas);
  model->ctx->live_models--;
  model->magic = 0;
  delete model;
  return SN_OK;
}

int sn_model_param_count(sn_model* model, int32_t* n_tensors, int64_t* flat_elems) {
  SN_TRY(check_model(model));
  if (n_tensors) *n_tensors = (int32_t)model->params.size();
  if (flat_elems) *flat_elems = model->flat_elems;
  return SN_OK;
}

int sn_model_param_info(sn_model* model, int32_t index, sn_param_info* out) {
  SN_TRY(check_model(model));
  SN_REQUIRE(out != nullptr, "sn_model_param_info: out is NULL");
  SN_REQUIRE(index >= 0 && index < (int32_t)model->params.size(), "parameter index %d out of range", index);
  *out = model->params[index].info;
  return SN_OK;
}

int sn_model_output_shape(sn_model* model, int32_t* rank, int64_t* dims) {
  SN_TRY(check_model(model));
  if (rank) *rank = (int32_t)model->out_dims.size();
  if (dims)
    for (size_t i = 0; i < model->out_dims.size(); ++i) dims[i] = model->out_dims[i];
  return SN_OK;
}

int sn_replica_create(sn_model* model, const sn_optimizer_desc* opt, sn_replica** out) {
  SN_REQUIRE(out != nullptr, "sn_replica_create: out is NULL");
  *out = nullptr;
  SN_TRY(check_model(model));
  sn_replica* r = new sn_replica();
  r->magic = REPLICA_MAGIC;
  r->model = model;
  r->ctx = model->ctx;
  r->has_opt = opt != nullptr;
  r->n_states = 0;
  if (opt) {
    r->opt = *opt;
    r->n_states = opt_state_count(opt->kind);
    if (r->n_states < 0) {
      delete r;
      return fail(SN_E_INVALID, "unknown optimizer kind %d", opt->kind);
    }
  }
  int rc = alloc_replica(r);
  if (rc != SN_OK) {
    for (void* p : r->owned) (void)hipFree(p);
    delete r;
    return rc;
  }
  model->live_replicas++;
  *out = r;
  return SN_OK;
}

int sn_replica_destroy(sn_replica* rep) {
  SN_TRY(check_replica(rep));
  (void)hipStreamSynchronize(rep->ctx->stream);
  if (rep->copy_stream) {
    (void)hipStreamSynchronize(rep->copy_stream);
    for (int i = 0; i < 2; ++i) {
      (void)hipEventDestroy(rep->ev_filled[i]);
      (void)hipEventDestroy(rep->ev_consumed[i]);
    }
    (void)hipStreamDestroy(rep->copy_stream);
  }
  if (rep->update_stream) {
    (void)hipStreamSynchronize(rep->update_stream);
    (void)hipEventDestroy(rep->ev_layer_ready);
    (void)hipEventDestroy(rep->ev_updates_done);
    (void)hipStreamDestroy(rep->update_stream);
  }
  for (void* p : rep->owned) (void)hipFree(p);
  rep->model->live_replicas--;
  rep->magic = 0;
  delete rep;
  return SN_OK;
}

int sn_params_set(sn_replica* rep, int32_t index, const float* src_host, int64_t n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(src_host != nullptr, "sn_params_set: source is NULL");
  rep->bf_weights_stale = true;
  return tensor_io(rep, rep->w, index, nullptr, src_host, n);
}
int sn_params_get(sn_replica* rep, int32_t index, float* dst_host, int64_t n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(dst_host != nullptr, "sn_params_get: destination is NULL");
  return tensor_io(rep, rep->w, index, dst_host, nullptr, n);
}
int sn_optstate_set(sn_replica* rep, int32_t index, int32_t slot, const float* src_host, int64_t n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(src_host != nullptr, "sn_optstate_set: source is NULL");
  SN_REQUIRE(slot >= 0 && slot < rep->n_states, "optimizer has %d state tensors per weight, slot %d asked", rep->n_states, slot);
  return tensor_io(rep, rep->s[slot], index, nullptr, src_host, n, true);
}
int sn_optstate_get(sn_replica* rep, int32_t index, int32_t slot, float* dst_host, int64_t n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(dst_host != nullptr, "sn_optstate_get: destination is NULL");
  SN_REQUIRE(slot >= 0 && slot < rep->n_states, "optimizer has %d state tensors per weight, slot %d asked", rep->n_states, slot);
  return tensor_io(rep, rep->s[slot], index, dst_host, nullptr, n, true);
}
int sn_grads_get(sn_replica* rep, int32_t index, float* dst_host, int64_t n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(dst_host != nullptr, "sn_grads_get: destination is NULL");
  return tensor_io(rep, rep->g, index, dst_host, nullptr, n, true);
}

int sn_replica_flat(sn_replica* rep, int32_t slot, float** out_dev, int64_t* n) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(out_dev != nullptr, "sn_replica_flat: out is NULL");
  SN_REQUIRE(slot >= -2 && slot < rep->n_states, "slot %d out of range", slot);
  *out_dev = slot == -2 ? rep->w : (slot == -1 ? rep->g : rep->s[slot]);
  if (slot == -2) rep->bf_weights_stale = true;  // the caller may write through the view
  if (n) *n = rep->model->flat_elems;
  return SN_OK;
}

int sn_step(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int32_t iter, float* loss_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev, "sn_step: null batch pointer");
  SN_TRY(check_rows(rep, rows));
  SN_REQUIRE(iter >= 1, "iteration numbers start at 1, got %d", iter);
  SN_REQUIRE(rep->has_opt, "replica was created without an optimizer");
  SN_TRY(grad_pass(rep, x_dev, y_dev, rows, loss_host != nullptr, iter));
  SN_TRY(update(rep, iter));
  return read_loss(rep, loss_host);
}

int sn_grad(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, float* loss_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev, "sn_grad: null batch pointer");
  SN_TRY(check_rows(rep, rows));
  SN_TRY(grad_pass(rep, x_dev, y_dev, rows, loss_host != nullptr));
  return read_loss(rep, loss_host);
}

static int forward_to(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev, bool training) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && out_dev, "sn_forward: null pointer");
  SN_TRY(check_rows(rep, rows));
  SN_TRY(forward(rep, x_dev, rows, false, training));
  const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, x_dev, rows);
  SN_HIP(hipMemcpyAsync(out_dev, pred, (size_t)rows * rep->model->out_elems * sizeof(float), hipMemcpyDeviceToDevice, rep->ctx->stream));
  return SN_OK;
}
int sn_forward(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev) { return forward_to(rep, x_dev, rows, out_dev, false); }
int sn_forward_training(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev) {
  return forward_to(rep, x_dev, rows, out_dev, true);
}

int sn_forward_static(sn_replica* rep, const float* x_dev, int32_t rows, float* out_dev) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && out_dev, "sn_forward_static: null pointer");
  SN_TRY(check_rows(rep, rows));
  sn_model* m = rep->model;
  sn_ctx* ctx = rep->ctx;
  SN_REQUIRE((m->flags & SN_FLAG_GEMM_BF16) == 0, "sn_forward_static: models with SN_FLAG_GEMM_BF16 keep bf16 operand copies it has no room for");
  for (const Op& op : m->ops)
    SN_REQUIRE(op.kind != OP_LSTM && op.kind != OP_SRNN, "sn_forward_static: recurrent layers keep per-step state it has no room for");
  unsigned char* base = ctx->device >= 0 && ctx->device < STATIC_SCRATCH_MAX_DEVICES ? g_scratch_ptr[ctx->device] : nullptr;
  SN_REQUIRE(base != nullptr, "sn_forward_static: the scratch array of device %d was never looked up", ctx->device);
  // carve the array: every piece starts on a 256-byte boundary
  const size_t n_ops = m->ops.size();
  std::vector<float*> act(n_ops, nullptr), bn(n_ops, nullptr);
  std::vector<uint8_t*> arg(n_ops, nullptr);
  size_t used = 0;
  auto carve = [&](size_t bytes) {
    unsigned char* p = base + used;  // an address past the end is never used: the size check below comes first
    used += (size_t)align_up((int64_t)bytes, 256);
    return p;
  };
  for (size_t i = 0; i < n_ops; ++i) {
    const Op& op = m->ops[i];
    if (op.kind == OP_FLATTEN) continue;
    act[i] = (float*)carve((size_t)rows * op.out_elems * sizeof(float));
    if (op.kind == OP_BATCHNORM) bn[i] = (float*)carve((size_t)9 * align_up(op.out_dims.back(), 64) * sizeof(float));
    if (op.kind == OP_POOL && !op.pool_avg) arg[i] = (uint8_t*)carve((size_t)rows * op.out_elems);
  }
  float* ws = (float*)carve((size_t)m->workspace_elems * sizeof(float));
  SN_REQUIRE(used <= STATIC_SCRATCH_BYTES,
             "sn_forward_static: %d rows of this model need %zu bytes of intermediates, the static scratch array holds %zu", rows, used,
             STATIC_SCRATCH_BYTES);
  // The pass itself is sn_forward's, pointed at the static pieces.  Per-kernel timing creates events: off for this call.
  const bool profiling = ctx->profiling;
  ctx->profiling = false;
  std::swap(rep->act, act);
  std::swap(rep->arg, arg);
  std::swap(rep->bn_buf, bn);
  std::swap(rep->ws, ws);
  int rc = forward(rep, x_dev, rows, false, false);
  if (rc == SN_OK) {
    const float* pred = op_output(rep, (int)n_ops - 1, x_dev, rows);
    hipError_t e = hipMemcpyAsync(out_dev, pred, (size_t)rows * m->out_elems * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream);
    if (e != hipSuccess) rc = fail(SN_E_HIP, "hipMemcpyAsync failed: %s", hipGetErrorString(e));
  }
  std::swap(rep->act, act);
  std::swap(rep->arg, arg);
  std::swap(rep->bn_buf, bn);
  std::swap(rep->ws, ws);
  ctx->profiling = profiling;
  return rc;
}

int sn_loss(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, float* loss_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev && loss_host, "sn_loss: null pointer");
  SN_TRY(check_rows(rep, rows));
  SN_TRY(forward(rep, x_dev, rows));
  const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, x_dev, rows);
  SN_TRY(loss_of(rep, pred, y_dev, rows, nullptr, false));  // the frozen model of a TrainedModel (models/Model.scala:126-127)
  return read_loss(rep, loss_host);
}

int sn_count_correct(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int64_t* count_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev && count_host, "sn_count_correct: null pointer");
  SN_TRY(check_rows(rep, rows));
  SN_TRY(forward(rep, x_dev, rows));
  const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, x_dev, rows);
  // cleared by a kernel, not a memset node: the call may be recorded into a HIP graph (all-zero bits are 0.0f twice)
  SN_TRY(launch_fill(rep->ctx, (float*)rep->count_dev, 0.f, 2));
  const int cols = (int)rep->model->out_dims.back();
  SN_TRY(launch_count_correct(rep->ctx, pred, y_dev, (int)((int64_t)rows * rep->model->out_elems / cols), cols, rep->count_dev));
  unsigned long long c = 0;
  SN_HIP(hipMemcpyAsync(&c, rep->count_dev, sizeof(c), hipMemcpyDeviceToHost, rep->ctx->stream));
  SN_HIP(hipStreamSynchronize(rep->ctx->stream));
  SN_TRY(check_async(rep->ctx));
  *count_host = (int64_t)c;
  return SN_OK;
}

int sn_error_sum(sn_replica* rep, const float* x_dev, const float* y_dev, int32_t rows, int32_t kind, float* sum_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev && sum_host, "sn_error_sum: null pointer");
  SN_REQUIRE(kind == SN_ERROR_SQUARED || kind == SN_ERROR_ABSOLUTE, "unknown error kind %d", kind);
  SN_TRY(check_rows(rep, rows));
  SN_TRY(forward(rep, x_dev, rows));
  const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, x_dev, rows);
  SN_TRY(launch_loss(rep->ctx, kind == SN_ERROR_SQUARED ? LOSS_SUM_SQUARED_ERROR : LOSS_SUM_ABSOLUTE_ERROR, pred, y_dev, nullptr,
                     rep->loss_dev, rep->loss_partials, rows, (int)rep->model->out_elems));
  return read_loss(rep, sum_host);
}

int sn_train_epoch(sn_replica* rep, const float* x_dev, const float* y_dev, int64_t total_rows, int32_t batch, int32_t global_iter,
                   int32_t* iterations_host, float* loss_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_dev && y_dev, "sn_train_epoch: null partition pointer");
  SN_REQUIRE(batch >= 1 && batch <= rep->model->batch, "batch must be in 1..%d, got %d", rep->model->batch, batch);
  SN_REQUIRE(global_iter >= 0, "global_iter must not be negative");
  const int64_t n_batches = total_rows / batch;  // the partial batch is skipped (optimizers/Iterators.scala:90)
  SN_REQUIRE(n_batches >= 1, "partition of %lld rows holds no full batch of %d (the reference's iterator throws here)",
             (long long)total_rows, batch);
  const int64_t xs = rep->model->in_elems * batch, ys = rep->model->out_elems * batch;
  for (int64_t i = 0; i < n_batches; ++i) {
    SN_TRY(grad_pass(rep, x_dev + i * xs, y_dev + i * ys, batch, false, global_iter + (int)i + 1));  // the epoch's loss is evaluated after its last update
    SN_TRY(update(rep, global_iter + (int)i + 1));  // optimizers/Optimizer.scala:143
  }
  if (iterations_host) *iterations_host = (int32_t)n_batches;
  if (loss_host) {  // optimizers/Optimizer.scala:148: loss of the last batch under the updated weights
    const float* xl = x_dev + (n_batches - 1) * xs;
    const float* yl = y_dev + (n_batches - 1) * ys;
    SN_TRY(forward(rep, xl, batch, false, true));  // `lossModel.lossStateful`: not frozen (Optimizer.scala:163-167)
    const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, xl, batch);
    SN_TRY(loss_of(rep, pred, yl, batch, nullptr, true));
    SN_TRY(read_loss(rep, loss_host));
  }
  return SN_OK;
}

// One epoch over a partition that lives in HOST memory (the reference's TensorIterator copies every batch into a
// fresh tensor that the session then feeds, optimizers/Iterators.scala:57-78): batch i+1 travels to the device on a
// second stream while batch i trains.  Two device slots; a slot is refilled only after the step that read it.
int sn_train_epoch_host(sn_replica* rep, const float* x_host, const float* y_host, int64_t total_rows, int32_t batch,
                        int32_t global_iter, int32_t* iterations_host, float* loss_host) {
  SN_TRY(check_replica(rep));
  SN_REQUIRE(x_host && y_host, "sn_train_epoch_host: null partition pointer");
  SN_REQUIRE(batch >= 1 && batch <= rep->model->batch, "batch must be in 1..%d, got %d", rep->model->batch, batch);
  SN_REQUIRE(global_iter >= 0, "global_iter must not be negative");
  const int64_t n_batches = total_rows / batch;  // the partial batch is skipped (optimizers/Iterators.scala:90)
  SN_REQUIRE(n_batches >= 1, "partition of %lld rows holds no full batch of %d (the reference's iterator throws here)",
             (long long)total_rows, batch);
  hipStream_t compute = rep->ctx->stream;
  if (!rep->copy_stream) {
    // Staging buffers, events and the copy stream are made in locals and handed to the replica only when all of them
    // exist, so a failure half way leaves nothing behind and the next call starts over.
    float* sx[2] = {nullptr, nullptr};
    float* sy[2] = {nullptr, nullptr};
    hipEvent_t filled[2] = {nullptr, nullptr}, consumed[2] = {nullptr, nullptr};
    hipStream_t copy = nullptr;
    // A slot holds a run of consecutive batches (up to 32 MiB or 64 batches): one copy and one pair of events per run
    // instead of per step, which is what a small model's step would otherwise wait for.
    const size_t one = (size_t)(rep->model->in_elems + rep->model->out_elems) * rep->model->batch * sizeof(float);
    const int64_t group = std::max<int64_t>(1, std::min<int64_t>(64, (int64_t)(((size_t)32 << 20) / one)));
    const size_t xb = (size_t)rep->model->in_elems * rep->model->batch * sizeof(float) * group;
    const size_t yb = (size_t)rep->model->out_elems * rep->model->batch * sizeof(float) * group;
    hipError_t e = hipSetDevice(rep->ctx->device);
    for (int i = 0; i < 2 && e == hipSuccess; ++i) {
      e = hipMalloc((void**)&sx[i], xb);
      if (e == hipSuccess) e = hipMalloc((void**)&sy[i], yb);
      if (e == hipSuccess) e = hipEventCreateWithFlags(&filled[i], hipEventDisableTiming);
      if (e == hipSuccess) e = hipEventCreateWithFlags(&consumed[i], hipEventDisableTiming);
    }
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&copy, hipStreamNonBlocking);
    if (e != hipSuccess) {
      for (int i = 0; i < 2; ++i) {
        if (sx[i]) (void)hipFree(sx[i]);
        if (sy[i]) (void)hipFree(sy[i]);
        if (filled[i]) (void)hipEventDestroy(filled[i]);
        if (consumed[i]) (void)hipEventDestroy(consumed[i]);
      }
      return fail(e == hipErrorOutOfMemory ? SN_E_OOM : SN_E_HIP, "sn_train_epoch_host: setting up the staging slots failed: %s",
                  hipGetErrorString(e));
    }
    for (int i = 0; i < 2; ++i) {
      rep->stage_x[i] = sx[i];
      rep->stage_y[i] = sy[i];
      rep->owned.push_back(sx[i]);
      rep->owned.push_back(sy[i]);
      rep->ev_filled[i] = filled[i];
      rep->ev_consumed[i] = consumed[i];
    }
    rep->copy_stream = copy;
    rep->stage_group = group;
  }
  const int64_t xs = rep->model->in_elems * batch, ys = rep->model->out_elems * batch;
  // Runs of 1, 2, 4, ... up to stage_group batches: the first step waits for one batch only, later copies are long
  const int64_t G = rep->stage_group;
  auto fill = [&](int64_t first, int64_t nb, int slot) -> int {
    SN_HIP(hipMemcpyAsync(rep->stage_x[slot], x_host + first * xs, (size_t)(nb * xs) * sizeof(float), hipMemcpyHostToDevice, rep->copy_stream));
    SN_HIP(hipMemcpyAsync(rep->stage_y[slot], y_host + first * ys, (size_t)(nb * ys) * sizeof(float), hipMemcpyHostToDevice, rep->copy_stream));
    SN_HIP(hipEventRecord(rep->ev_filled[slot], rep->copy_stream));
    return SN_OK;
  };
  // earlier work on the compute stream may still read the slots (a previous epoch's last loss)
  SN_HIP(hipEventRecord(rep->ev_consumed[0], compute));
  SN_HIP(hipStreamWaitEvent(rep->copy_stream, rep->ev_consumed[0], 0));
  int64_t first = 0, nb = 1, last_first = 0;
  int slot = 0;
  // The caller may reuse its host buffers as soon as this function returns, also when it returns an error: whatever
  // path leaves it, the copies queued so far (and the steps they feed) have finished first.
  struct DrainOnExit {
    hipStream_t copy, compute;
    ~DrainOnExit() {
      (void)hipStreamSynchronize(compute);
      (void)hipStreamSynchronize(copy);
    }
  } drain{rep->copy_stream, compute};
  SN_TRY(fill(first, nb, slot));
  for (int64_t run = 0; first < n_batches; ++run) {
    const int64_t next_first = first + nb, next_nb = std::min(std::min(G, 2 * nb), n_batches - next_first);
    if (next_nb > 0) {  // the other slot was last read by the steps of run - 1, already queued on the compute stream
      if (run >= 1) SN_HIP(hipStreamWaitEvent(rep->copy_stream, rep->ev_consumed[slot ^ 1], 0));
      SN_TRY(fill(next_first, next_nb, slot ^ 1));
    }
    SN_HIP(hipStreamWaitEvent(compute, rep->ev_filled[slot], 0));
    for (int64_t j = 0; j < nb; ++j) {
      SN_TRY(grad_pass(rep, rep->stage_x[slot] + j * xs, rep->stage_y[slot] + j * ys, batch, false, global_iter + (int)(first + j) + 1));
      SN_TRY(update(rep, global_iter + (int)(first + j) + 1));  // optimizers/Optimizer.scala:143
    }
    SN_HIP(hipEventRecord(rep->ev_consumed[slot], compute));
    last_first = first;
    first = next_first;
    nb = next_nb;
    slot ^= 1;
  }
  const int last_slot = slot ^ 1;  // the slot of the run that held the last batch
  if (iterations_host) *iterations_host = (int32_t)n_batches;
  const float* last_x = rep->stage_x[last_slot] + (n_batches - 1 - last_first) * xs;
  const float* last_y = rep->stage_y[last_slot] + (n_batches - 1 - last_first) * ys;
  if (loss_host) {  // optimizers/Optimizer.scala:148: loss of the last batch under the updated weights
    SN_TRY(forward(rep, last_x, batch, false, true));
    const float* pred = op_output(rep, (int)rep->model->ops.size() - 1, last_x, batch);
    SN_TRY(loss_of(rep, pred, last_y, batch, nullptr, true));
    SN_TRY(read_loss(rep, loss_host));
  } else {
    SN_HIP(hipStreamSynchronize(compute));
    SN_TRY(check_async(rep->ctx));
  }
  SN_HIP(hipStreamSynchronize(rep->copy_stream));
  return SN_OK;
}

int sn_replicas_average(sn_replica* const* reps, int32_t k) {
  SN_REQUIRE(reps != nullptr, "sn_replicas_average: replica list is NULL");
  SN_REQUIRE(k >= 1 && k <= SN_MAX_AVG_INPUTS, "sn_replicas_average: k must be in 1..%d, got %d", SN_MAX_AVG_INPUTS, k);
  for (int i = 0; i < k; ++i) {
    SN_TRY(check_replica(reps[i]));
    SN_REQUIRE(reps[i]->model == reps[0]->model, "replica %d belongs to another model", i);
    // replicas of one model share its context, hence its stream: the launches below are ordered behind every replica's steps
    SN_REQUIRE(reps[i]->ctx == reps[0]->ctx, "replica %d lives in another context", i);
    SN_REQUIRE(reps[i]->n_states == reps[0]->n_states && (!reps[i]->has_opt || reps[i]->opt.kind == reps[0]->opt.kind),
               "replica %d uses another optimizer", i);
  }
  if (k == 1) return SN_OK;  // treeReduce of one partition never calls aggregateParams
  for (int i = 0; i < k; ++i) reps[i]->bf_weights_stale = true;
  sn_ctx* ctx = reps[0]->ctx;
  const int64_t n = reps[0]->model->flat_elems;
  for (int slot = -1; slot < reps[0]->n_states; ++slot) {
    AvgInputs in;
    float* outs[SN_MAX_AVG_INPUTS];
    for (int i = 0; i < k; ++i) {
      float* p = slot < 0 ? reps[i]->w : reps[i]->s[slot];
      in.p[i] = p;
      outs[i] = p;
    }
    SN_TRY(launch_average(ctx, in, k, n, outs[0], outs + 1, k - 1));
  }
  // tensors without an aggregation start over from their initializer, Zeros (optimizers/Optimizer.scala:207-210)
  for (const ParamDef& p : reps[0]->model->params)
    if (!p.info.aggregated)
      for (int i = 0; i < k; ++i) SN_TRY(launch_fill(ctx, reps[i]->w + p.info.offset, 0.f, p.info.size));
  return SN_OK;
}

}  // extern "C"
