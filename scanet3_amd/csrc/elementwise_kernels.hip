// Memory-bound layer kernels: bias + activation, activation backward, softmax rows,
// losses, column sums (bias gradients), regularisation, max and average pooling, LSTM gate maths
// and the accuracy count.  All arithmetic is float32 in the reference's operation
// order (no fused multiply-add; the file is compiled with -ffp-contract=off).
#include "common.hpp"

namespace sn {

// ---------------------------------------------------------------------------- helpers
__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float act_fwd(int act, float x, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return sigmoidf_(x);
    case SN_ACT_TANH: return tanhf(x);
    case SN_ACT_RELU: return fmaxf(param, x);  // Maximum(threshold, x), Activation.scala:79-82
    default: return x;
  }
}

// Gradient through an activation given its OUTPUT y (each rule below is the reference's
// localGrad with the recomputed forward value replaced by the stored one, which is the
// same float):
//   sigmoid: s*(1-s)*dy (AllKernels.scala:397-404)   tanh: (1 - y^2)*dy (:414-420)
//   relu: (threshold < x) * dy with x > threshold <=> y > threshold (:297-302)
__device__ __forceinline__ float act_bwd(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sum over a 256-thread block; result valid in every thread.
__device__ __forceinline__ float block_sum(float v, float* smem /* >= 4 floats */) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  float t = 0.f;
  const int nw = (blockDim.x + 63) >> 6;
  for (int i = 0; i < nw; ++i) t += smem[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* smem) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  float t = smem[0];
  const int nw = (blockDim.x + 63) >> 6;
  for (int i = 1; i < nw; ++i) t = fmaxf(t, smem[i]);
  return t;
}

static inline unsigned grid_for(sn_ctx* ctx, int64_t n, int per_block) {
  int64_t blocks = ceil_div(n, per_block);
  const int64_t cap = (int64_t)ctx->compute_units * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// ---------------------------------------------------------------------------- bias + activation
__global__ __launch_bounds__(256) void bias_act_kernel(const float* __restrict__ x, const float* __restrict__ bias,
                                                        float* __restrict__ y, int64_t n, int cols, int act, float param) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float v = x[i];
    if (bias) v = v + bias[i % cols];  // Bias.scala:32-33
    y[i] = act_fwd(act, v, param);
  }
}

int launch_bias_act(sn_ctx* ctx, const float* x, const float* bias, float* y, int64_t rows, int cols, int act, float act_param) {
  const int64_t n = rows * cols;
  if (n <= 0) return SN_OK;
  LaunchScope scope(ctx, "bias_activation");
  hipLaunchKernelGGL(bias_act_kernel, dim3(grid_for(ctx, n, 1024)), dim3(256), 0, ctx->stream, x, bias, y, n, cols, act, act_param);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

__global__ __launch_bounds__(256) void act_bwd_kernel(const float* __restrict__ y, const float* __restrict__ dy,
                                                       float* __restrict__ dx, int64_t n, int act, float param) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dx[i] = act_bwd(act, y[i], dy[i], param);
}

int launch_act_bwd(sn_ctx* ctx, const float* y, const float* dy, float* dx, int64_t n, int act, float act_param) {
  if (n <= 0) return SN_OK;
  LaunchScope scope(ctx, "activation_backward");
  hipLaunchKernelGGL(act_bwd_kernel, dim3(grid_for(ctx, n, 1024)), dim3(256), 0, ctx->stream, y, dy, dx, n, act, act_param);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- softmax
// One 256-thread block per row. p = exp(z) / sum(exp(z)) (Activation.scala:63-69); with
// `stable` the row maximum is subtracted first (same value in exact arithmetic).
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const float* __restrict__ z, float* __restrict__ p, int cols, int stable) {
  __shared__ float smem[4];
  const float* zr = z + (int64_t)blockIdx.x * cols;
  float* pr = p + (int64_t)blockIdx.x * cols;
  float mx = 0.f;
  if (stable) {
    float m = -INFINITY;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) m = fmaxf(m, zr[c]);
    mx = block_max(m, smem);
  }
  float s = 0.f;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float e = expf(zr[c] - mx);
    pr[c] = e;
    s += e;
  }
  const float total = block_sum(s, smem);
  for (int c = threadIdx.x; c < cols; c += blockDim.x) pr[c] = pr[c] / total;
}

int launch_softmax_fwd(sn_ctx* ctx, const float* z, float* p, int rows, int cols, bool stable) {
  if (rows <= 0) return SN_OK;
  LaunchScope scope(ctx, "softmax_forward");
  const int threads = cols <= 64 ? 64 : 256;
  hipLaunchKernelGGL(softmax_fwd_kernel, dim3(rows), dim3(threads), 0, ctx->stream, z, p, cols, stable ? 1 : 0);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// dz_i = p_i * dp_i - p_i * sum_j(p_j * dp_j): the Div/Sum/Exp chain of the reference
// (AllKernels.scala:196-201,214-227,237-244) with e/S written as p.
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const float* __restrict__ p, const float* __restrict__ dp,
                                                           float* __restrict__ dz, int cols) {
  __shared__ float smem[4];
  const int64_t base = (int64_t)blockIdx.x * cols;
  float s = 0.f;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) s += p[base + c] * dp[base + c];
  const float dot = block_sum(s, smem);
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float pi = p[base + c];
    dz[base + c] = pi * dp[base + c] - pi * dot;
  }
}

int launch_softmax_bwd(sn_ctx* ctx, const float* p, const float* dp, float* dz, int rows, int cols) {
  if (rows <= 0) return SN_OK;
  LaunchScope scope(ctx, "softmax_backward");
  const int threads = cols <= 64 ? 64 : 256;
  hipLaunchKernelGGL(softmax_bwd_kernel, dim3(rows), dim3(threads), 0, ctx->stream, p, dp, dz, cols);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- losses
// Stage 1: per-block partial sums of the per-element loss terms and, when dp != null,
// d loss / d p.  Stage 2 (one block) adds the partials in order and scales.
//   MSE  (Loss.scala:18-24):  mean((p-y)^2);        dp = ((p-y)*2) * (1/size)
//   BCE  (Loss.scala:26-42):  mean(-y log(p+e) - (1-y) log(1-(p-e)))
//   CCE  (Loss.scala:44-57):  -sum(y log(p+e)) / rows;  dp = (y * -(1/rows)) / (p+e)
constexpr int LOSS_BLOCKS_MAX = 1024;

__global__ __launch_bounds__(256) void loss_stage1_kernel(int kind, const float* __restrict__ p, const float* __restrict__ y,
                                                           float* __restrict__ dp, float* __restrict__ partials, int64_t n,
                                                           float inv_size, float neg_inv_rows) {
  __shared__ float smem[4];
  const float eps = 1e-8f;
  float s = 0.f;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float pi = p[i], yi = y[i];
    if (kind == SN_LOSS_MSE) {
      const float d = pi - yi;
      s += d * d;
      if (dp) dp[i] = (d * 2.0f) * inv_size;
    } else if (kind == SN_LOSS_BINARY_CROSSENTROPY) {
      const float left = yi * logf(pi + eps);
      const float right = (1.0f - yi) * logf(1.0f - (pi - eps));
      s += (-left - right);
      if (dp) {
        const float g = inv_size;
        const float dl = (yi * (-g)) / (pi + eps);
        const float dr = -(((1.0f - yi) * (-g)) / (1.0f - (pi - eps)));
        dp[i] = dl + dr;
      }
    } else if (kind == SN_LOSS_CATEGORICAL_CROSSENTROPY) {
      s += yi * logf(pi + eps);
      if (dp) dp[i] = (yi * neg_inv_rows) / (pi + eps);
    } else if (kind == LOSS_SUM_SQUARED_ERROR) {  // estimators/package.scala:56-62
      const float d = pi - yi;
      s += d * d;
    } else if (kind == LOSS_SUM_ABSOLUTE_ERROR) {  // estimators/package.scala:64-70
      s += fabsf(pi - yi);
    } else {  // identity: the prediction is the loss (Loss.scala:10-14); callers guarantee n == 1
      s += pi;
      if (dp) dp[i] = 1.0f;
    }
  }
  const float t = block_sum(s, smem);
  if (threadIdx.x == 0) partials[blockIdx.x] = t;
}

__global__ __launch_bounds__(256) void loss_stage2_kernel(int kind, const float* __restrict__ partials, int n_partials,
                                                           float* __restrict__ loss, float inv_size, float rows) {
  __shared__ float smem[4];
  float s = 0.f;
  for (int i = threadIdx.x; i < n_partials; i += blockDim.x) s += partials[i];
  const float t = block_sum(s, smem);
  if (threadIdx.x == 0) {
    if (kind == SN_LOSS_CATEGORICAL_CROSSENTROPY) *loss = (-t) / rows;
    else if (kind == SN_LOSS_IDENTITY || kind == LOSS_SUM_SQUARED_ERROR || kind == LOSS_SUM_ABSOLUTE_ERROR) *loss = t;
    else *loss = t * inv_size;
  }
}

int launch_loss(sn_ctx* ctx, int kind, const float* p, const float* y, float* dp, float* loss_dev, float* partials, int rows,
                int cols) {
  const int64_t n = (int64_t)rows * cols;
  SN_REQUIRE(n > 0, "loss over an empty batch");
  const unsigned blocks = (unsigned)std::min<int64_t>(LOSS_BLOCKS_MAX, std::max<int64_t>(1, ceil_div(n, 2048)));
  const float inv_size = 1.0f / (float)n;
  const float neg_inv_rows = -(1.0f / (float)rows);
  {
    LaunchScope scope(ctx, "loss_stage1");
    hipLaunchKernelGGL(loss_stage1_kernel, dim3(blocks), dim3(256), 0, ctx->stream, kind, p, y, dp, partials, n, inv_size,
                       neg_inv_rows);
  }
  if (loss_dev) {
    LaunchScope scope(ctx, "loss_stage2");
    hipLaunchKernelGGL(loss_stage2_kernel, dim3(1), dim3(256), 0, ctx->stream, kind, partials, (int)blocks, loss_dev, inv_size,
                       (float)rows);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// Softmax output + CategoricalCrossentropy in one pass per row (training step only): p, the row's loss term
// and dz = p*dp - p*sum(p*dp) with dp = (y * -(1/rows)) / (p + e), i.e. exactly what softmax_fwd_kernel,
// loss_stage1_kernel and softmax_bwd_kernel compute one after the other, without the dp round trip.
__global__ __launch_bounds__(256) void softmax_cce_kernel(const float* __restrict__ z, const float* __restrict__ y, float* __restrict__ p,
                                                           float* __restrict__ dz, float* __restrict__ row_loss, int cols, int stable,
                                                           float neg_inv_rows, __bf16* __restrict__ dz_bf) {
  __shared__ float smem[4];
  const int64_t base = (int64_t)blockIdx.x * cols;
  const float eps = 1e-8f;
  float mx = 0.f;
  if (stable) {
    float m = -INFINITY;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) m = fmaxf(m, z[base + c]);
    mx = block_max(m, smem);
  }
  float s = 0.f;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float e = expf(z[base + c] - mx);
    p[base + c] = e;  // re-read below by the thread that wrote it
    s += e;
  }
  const float total = block_sum(s, smem);
  float term = 0.f, dot = 0.f;
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float pi = p[base + c] / total, yi = y[base + c];
    p[base + c] = pi;
    term += yi * logf(pi + eps);
    dot += pi * ((yi * neg_inv_rows) / (pi + eps));
  }
  const float row_term = block_sum(term, smem);
  const float row_dot = block_sum(dot, smem);
  for (int c = threadIdx.x; c < cols; c += blockDim.x) {
    const float pi = p[base + c];
    const float dpi = (y[base + c] * neg_inv_rows) / (pi + eps);
    const float d = pi * dpi - pi * row_dot;
    dz[base + c] = d;
    if (dz_bf) dz_bf[base + c] = (__bf16)d;
  }
  if (threadIdx.x == 0) row_loss[blockIdx.x] = row_term;
}

// The same row kernel when a thread's share of the row (E values: columns threadIdx.x + k * blockDim.x) fits in registers:
// z and y are read once, p and dz written once; every sum sees the same values in the same order as above.
template <int E>
__global__ __launch_bounds__(256) void softmax_cce_reg_kernel(const float* __restrict__ z, const float* __restrict__ y, float* __restrict__ p,
                                                               float* __restrict__ dz, float* __restrict__ row_loss, int cols, int stable,
                                                               float neg_inv_rows, __bf16* __restrict__ dz_bf) {
  __shared__ float smem[4];
  const int64_t base = (int64_t)blockIdx.x * cols;
  const float eps = 1e-8f;
  float zv[E], yv[E];
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    zv[k] = c < cols ? z[base + c] : 0.f;
    yv[k] = c < cols ? y[base + c] : 0.f;
  }
  float mx = 0.f;
  if (stable) {
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < E; ++k)
      if ((int)(threadIdx.x + k * blockDim.x) < cols) m = fmaxf(m, zv[k]);
    mx = block_max(m, smem);
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < E; ++k) {
    if ((int)(threadIdx.x + k * blockDim.x) < cols) {
      zv[k] = expf(zv[k] - mx);
      s += zv[k];
    }
  }
  const float total = block_sum(s, smem);
  float term = 0.f, dot = 0.f;
#pragma unroll
  for (int k = 0; k < E; ++k) {
    if ((int)(threadIdx.x + k * blockDim.x) < cols) {
      const float pi = zv[k] / total;
      zv[k] = pi;
      term += yv[k] * logf(pi + eps);
      dot += pi * ((yv[k] * neg_inv_rows) / (pi + eps));
    }
  }
  const float row_term = block_sum(term, smem);
  const float row_dot = block_sum(dot, smem);
#pragma unroll
  for (int k = 0; k < E; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    if (c < cols) {
      const float pi = zv[k];
      const float dpi = (yv[k] * neg_inv_rows) / (pi + eps);
      const float d = pi * dpi - pi * row_dot;
      if (p) p[base + c] = pi;
      dz[base + c] = d;
      if (dz_bf) dz_bf[base + c] = (__bf16)d;
    }
  }
  if (threadIdx.x == 0) row_loss[blockIdx.x] = row_term;
}

// The row kernel for logits that still lie as partial sums [part][rows * cols] of the Dense product below (a product over
// many features that left one partial result per feature chunk).  64 lanes per logit walk every 64th part, their sums
// are added as a chain, then the bias: the order of the product's own reduction kernel.  The first wavefront then holds
// the row's logits, one per lane, and finishes as softmax_cce_reg_kernel<1> does with 64 threads.
__global__ __launch_bounds__(1024) void softmax_cce_partials_kernel(const float* __restrict__ partial, int parts, const float* __restrict__ bias,
                                                                     float* __restrict__ z_out, const float* __restrict__ y,
                                                                     float* __restrict__ p, float* __restrict__ dz, float* __restrict__ row_loss,
                                                                     int rows, int cols, int stable, float neg_inv_rows) {
  __shared__ float sm[64][SOFTMAX_PARTIALS_MAX_COLS];
  const int ol = threadIdx.x % cols, pl = threadIdx.x / cols;  // blockDim.x = 64 * cols
  const int64_t outs = (int64_t)rows * cols;
  const int64_t base = (int64_t)blockIdx.x * cols;
  {
    const int64_t o = base + ol;
    float s = 0.f;
    for (int i = pl; i < parts; i += 64 * 8) {  // 8 loads in flight, added in part order
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = i + 64 * u < parts ? partial[(int64_t)(i + 64 * u) * outs + o] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    sm[pl][ol] = s;
  }
  __syncthreads();
  if (threadIdx.x >= 64) return;
  const int c = threadIdx.x;
  const bool live = c < cols;
  float zv = 0.f, yv = 0.f;
  if (live) {
    float t = 0.f;
#pragma unroll 8
    for (int j = 0; j < 64; ++j) t += sm[j][c];
    if (bias) t = t + bias[c];
    z_out[base + c] = t;
    zv = t;
    yv = y[base + c];
  }
  const float eps = 1e-8f;
  float mx = 0.f;
  if (stable) mx = wave_max(live ? zv : -INFINITY);
  float s = 0.f;
  if (live) {
    zv = expf(zv - mx);
    s += zv;
  }
  const float total = 0.f + wave_sum(s);
  float term = 0.f, dot = 0.f;
  if (live) {
    const float pi = zv / total;
    zv = pi;
    term += yv * logf(pi + eps);
    dot += pi * ((yv * neg_inv_rows) / (pi + eps));
  }
  const float row_term = 0.f + wave_sum(term);
  const float row_dot = 0.f + wave_sum(dot);
  if (live) {
    const float pi = zv;
    const float dpi = (yv * neg_inv_rows) / (pi + eps);
    if (p) p[base + c] = pi;
    dz[base + c] = pi * dpi - pi * row_dot;
  }
  if (c == 0) row_loss[blockIdx.x] = row_term;
}

int launch_softmax_cce_partials(sn_ctx* ctx, const float* partial, int parts, const float* bias, float* z_out, const float* y, float* p,
                                float* dz, float* loss_dev, float* row_loss, int rows, int cols, bool stable) {
  SN_REQUIRE(rows > 0 && cols > 0 && cols <= SOFTMAX_PARTIALS_MAX_COLS && parts > 0, "softmax over partial sums: %d rows, %d columns, %d parts", rows, cols, parts);
  {
    LaunchScope scope(ctx, "small_output_reduce_softmax_crossentropy_fused");
    const float neg_inv_rows = -(1.0f / (float)rows);
    hipLaunchKernelGGL(softmax_cce_partials_kernel, dim3(rows), dim3(64 * cols), 0, ctx->stream, partial, parts, bias, z_out, y, p, dz, row_loss,
                       rows, cols, stable ? 1 : 0, neg_inv_rows);
  }
  if (loss_dev) {
    LaunchScope scope(ctx, "loss_stage2");
    hipLaunchKernelGGL(loss_stage2_kernel, dim3(1), dim3(256), 0, ctx->stream, (int)SN_LOSS_CATEGORICAL_CROSSENTROPY, (const float*)row_loss,
                       rows, loss_dev, 0.f, (float)rows);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_softmax_cce(sn_ctx* ctx, const float* z, const float* y, float* p, float* dz, float* loss_dev, float* row_loss, int rows,
                       int cols, bool stable, void* dz_bf) {
  SN_REQUIRE(rows > 0 && cols > 0, "loss over an empty batch");
  {
    LaunchScope scope(ctx, "softmax_crossentropy_fused");
    const int threads = cols <= 64 ? 64 : 256;
    const float neg_inv_rows = -(1.0f / (float)rows);
    SN_REQUIRE(p || cols <= 4 * threads, "softmax_crossentropy_fused: rows of %d values need the probabilities' buffer", cols);
#define SN_SOFTMAX_CCE_REG(E) \
  hipLaunchKernelGGL((softmax_cce_reg_kernel<E>), dim3(rows), dim3(threads), 0, ctx->stream, z, y, p, dz, row_loss, cols, stable ? 1 : 0, neg_inv_rows, \
                     (__bf16*)dz_bf)
    if (cols <= threads) SN_SOFTMAX_CCE_REG(1);
    else if (cols <= 2 * threads) SN_SOFTMAX_CCE_REG(2);
    else if (cols <= 4 * threads) SN_SOFTMAX_CCE_REG(4);
    else
      hipLaunchKernelGGL(softmax_cce_kernel, dim3(rows), dim3(threads), 0, ctx->stream, z, y, p, dz, row_loss, cols, stable ? 1 : 0, neg_inv_rows,
                         (__bf16*)dz_bf);
#undef SN_SOFTMAX_CCE_REG
  }
  if (loss_dev) {
    LaunchScope scope(ctx, "loss_stage2");
    hipLaunchKernelGGL(loss_stage2_kernel, dim3(1), dim3(256), 0, ctx->stream, (int)SN_LOSS_CATEGORICAL_CROSSENTROPY, (const float*)row_loss,
                       rows, loss_dev, 0.f, (float)rows);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- column sums (bias gradient)
// out[c] = sum_r dy[r, c] (Plus's gradient: Sum over the broadcast axes, AllKernels.scala:21-31).
// A block owns 64 columns; its 4 waves stride over the rows; partial sums meet in LDS.
// Rows r, r+4, ... below r1 of column c, added in that order; 8 loads are in flight at a time (one load per
// loop trip would make the loop as slow as 8 memory latencies per 8 rows).
__device__ __forceinline__ float sum_every_4th_row(const float* __restrict__ dy, int64_t ld, int c, int64_t r, int64_t r1) {
  float s = 0.f;
  for (; r + 28 < r1; r += 32) {
    float a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = dy[(r + 4 * u) * ld + c];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += a[u];
  }
  for (; r < r1; r += 4) s += dy[r * ld + c];
  return s;
}

__global__ __launch_bounds__(256) void col_sum_kernel(const float* __restrict__ dy, int64_t ld, float* __restrict__ out, int64_t rows,
                                                       int cols) {
  __shared__ float smem[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const float s = c < cols ? sum_every_4th_row(dy, ld, c, wave, rows) : 0.f;
  smem[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && c < cols) out[c] = ((smem[0][lane] + smem[1][lane]) + smem[2][lane]) + smem[3][lane];
}

// Many rows: the rows are cut into gridDim.y slices that write partial sums, which a second
// launch of col_sum_kernel adds up in slice order (deterministic, no atomics).
__global__ __launch_bounds__(256) void col_sum_split_kernel(const float* __restrict__ dy, int64_t ld, float* __restrict__ part,
                                                             int64_t rows, int cols, int64_t rows_per_slice) {
  __shared__ float smem[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < rows ? r0 + rows_per_slice : rows;
  const float s = c < cols ? sum_every_4th_row(dy, ld, c, r0 + wave, r1) : 0.f;
  smem[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && c < cols) part[(int64_t)blockIdx.y * cols + c] = ((smem[0][lane] + smem[1][lane]) + smem[2][lane]) + smem[3][lane];
}

// Wide matrices: a lane owns 4 consecutive columns (float4), a wavefront 256 columns = 1 KiB of a row, the
// block's 4 wavefronts take every 4th row of the slice, 4 rows in flight per lane.
typedef float cs_f4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void col_sum_wide_kernel(const float* __restrict__ dy, int64_t ld, float* __restrict__ part,
                                                            int64_t rows, int cols, int64_t rows_per_slice) {
  __shared__ cs_f4 smem[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * 4;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < rows ? r0 + rows_per_slice : rows;
  cs_f4 s = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {
    int64_t r = r0 + wave;
    for (; r + 12 < r1; r += 16) {
      const cs_f4 a = __builtin_nontemporal_load((const cs_f4*)(dy + r * ld + c));
      const cs_f4 b = __builtin_nontemporal_load((const cs_f4*)(dy + (r + 4) * ld + c));
      const cs_f4 d = __builtin_nontemporal_load((const cs_f4*)(dy + (r + 8) * ld + c));
      const cs_f4 e = __builtin_nontemporal_load((const cs_f4*)(dy + (r + 12) * ld + c));
      s = (((s + a) + b) + d) + e;
    }
    for (; r < r1; r += 4) s = s + *(const cs_f4*)(dy + r * ld + c);
  }
  smem[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && c < cols) *(cs_f4*)(part + (int64_t)blockIdx.y * cols + c) = ((smem[0][lane] + smem[1][lane]) + smem[2][lane]) + smem[3][lane];
}

int launch_col_sum(sn_ctx* ctx, const float* dy, int64_t ld, float* out, int64_t rows, int cols, float* ws, int64_t ws_elems) {
  if (cols <= 0) return SN_OK;
  if (cols >= 256 && cols % 4 == 0 && ld % 4 == 0 && rows >= 512 && ws && ws_elems >= 2 * (int64_t)cols &&
      (reinterpret_cast<uintptr_t>(dy) & 15u) == 0 && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0) {
    const unsigned cb = (unsigned)ceil_div(cols, 256);
    int64_t slices = std::min<int64_t>(ceil_div(rows, 64), ceil_div((int64_t)ctx->compute_units * 8, cb));
    slices = std::max<int64_t>(1, std::min<int64_t>(slices, ws_elems / cols));
    const int64_t per = ceil_div(rows, slices);
    slices = ceil_div(rows, per);
    LaunchScope scope(ctx, "bias_gradient");
    hipLaunchKernelGGL(col_sum_wide_kernel, dim3(cb, (unsigned)slices), dim3(256), 0, ctx->stream, dy, ld, ws, rows, cols, per);
    hipLaunchKernelGGL(col_sum_kernel, dim3((unsigned)ceil_div(cols, 64)), dim3(256), 0, ctx->stream, (const float*)ws, (int64_t)cols, out,
                       slices, cols);
    SN_HIP(hipGetLastError());
    return SN_OK;
  }
  const unsigned col_blocks = (unsigned)ceil_div(cols, 64);
  int64_t slices = 1;
  if (rows >= 512 && ws) {
    slices = std::min<int64_t>(ceil_div(rows, 128), ceil_div((int64_t)ctx->compute_units * 4, col_blocks));
    slices = std::min<int64_t>(slices, ws_elems / cols);
    if (slices < 1) slices = 1;
  }
  LaunchScope scope(ctx, "bias_gradient");
  if (slices <= 1) {
    hipLaunchKernelGGL(col_sum_kernel, dim3(col_blocks), dim3(256), 0, ctx->stream, dy, ld, out, rows, cols);
  } else {
    const int64_t per = ceil_div(rows, slices);
    slices = ceil_div(rows, per);
    hipLaunchKernelGGL(col_sum_split_kernel, dim3(col_blocks, (unsigned)slices), dim3(256), 0, ctx->stream, dy, ld, ws, rows, cols, per);
    hipLaunchKernelGGL(col_sum_kernel, dim3(col_blocks), dim3(256), 0, ctx->stream, (const float*)ws, (int64_t)cols, out, slices, cols);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- regularisation
// L2: lambda * sum(w^2) / 2 ; L1: lambda * sum(|w|) / 2 (Regularization.scala:30-44); added to *loss.
// Two stages like the losses: per-block partial sums, then one block adds them in order and finishes the term.
__global__ __launch_bounds__(256) void penalty_stage1_kernel(const float* __restrict__ w, int64_t n, int reg, float* __restrict__ partials) {
  __shared__ float smem[4];
  float s = 0.f;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) s += reg == SN_REG_L2 ? w[i] * w[i] : fabsf(w[i]);
  const float t = block_sum(s, smem);
  if (threadIdx.x == 0) partials[blockIdx.x] = t;
}

__global__ __launch_bounds__(256) void penalty_stage2_kernel(const float* __restrict__ partials, int n_partials, float lambda, float* loss) {
  __shared__ float smem[4];
  float s = 0.f;
  for (int i = threadIdx.x; i < n_partials; i += blockDim.x) s += partials[i];
  const float t = block_sum(s, smem);
  if (threadIdx.x == 0) *loss = *loss + (lambda * t) / 2.0f;
}

int launch_penalty(sn_ctx* ctx, const float* w, int64_t n, int reg_kind, float lambda, float* loss_dev, float* partials) {
  const unsigned blocks = (unsigned)std::min<int64_t>(LOSS_BLOCKS_MAX, std::max<int64_t>(1, ceil_div(n, 2048)));
  LaunchScope scope(ctx, "penalty");
  hipLaunchKernelGGL(penalty_stage1_kernel, dim3(blocks), dim3(256), 0, ctx->stream, w, n, reg_kind, partials);
  hipLaunchKernelGGL(penalty_stage2_kernel, dim3(1), dim3(256), 0, ctx->stream, (const float*)partials, (int)blocks, lambda, loss_dev);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// d penalty / d w: L2 through Pow's gradient (w*2)*(lambda/2); L1 through Abs's gradient, which in
// the reference is |parent| = lambda/2 for every element (AllKernels.scala:330-335).
__global__ __launch_bounds__(256) void penalty_grad_kernel(const float* __restrict__ w, float* __restrict__ g, int64_t n, int reg,
                                                            float lambda) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const float half = lambda / 2.0f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    g[i] = g[i] + (reg == SN_REG_L2 ? (w[i] * 2.0f) * half : fabsf(half));
}

int launch_penalty_grad(sn_ctx* ctx, const float* w, float* g, int64_t n, int reg_kind, float lambda) {
  if (n <= 0) return SN_OK;
  LaunchScope scope(ctx, "penalty_gradient");
  hipLaunchKernelGGL(penalty_grad_kernel, dim3(grid_for(ctx, n, 1024)), dim3(256), 0, ctx->stream, w, g, n, reg_kind, lambda);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- accuracy count
// rows where every rint(p) equals y (estimators/package.scala:28-32); rintf rounds half to even.
__global__ __launch_bounds__(256) void count_correct_kernel(const float* __restrict__ p, const float* __restrict__ y, int rows,
                                                             int cols, unsigned long long* count) {
  __shared__ float smem[4];
  float local = 0.f;
  for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < rows; r += gridDim.x * blockDim.x) {
    int matched = 0;
    for (int c = 0; c < cols; ++c) matched += (y[(int64_t)r * cols + c] == rintf(p[(int64_t)r * cols + c])) ? 1 : 0;
    local += matched == cols ? 1.f : 0.f;
  }
  const float t = block_sum(local, smem);  // exact: at most 2^24 rows per block
  if (threadIdx.x == 0 && t > 0.f) atomicAdd(count, (unsigned long long)t);
}

int launch_count_correct(sn_ctx* ctx, const float* p, const float* y, int rows, int cols, unsigned long long* count_dev) {
  if (rows <= 0) return SN_OK;
  LaunchScope scope(ctx, "count_correct");
  hipLaunchKernelGGL(count_correct_kernel, dim3(grid_for(ctx, rows, 256)), dim3(256), 0, ctx->stream, p, y, rows, cols, count_dev);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// Consecutive workgroup ids land on different XCDs (8, each with its own L2).  Stencil kernels whose neighbouring
// workgroups read overlapping rows use this block number instead: XCD x gets the x-th contiguous eighth of the
// blocks, so the shared rows are fetched into one L2 only.  The grid must be a multiple of 8.
__device__ __forceinline__ unsigned xcd_contiguous_block() {
  return (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
}
static inline unsigned grid_for_xcd(sn_ctx* ctx, int64_t n, int per_block) {
  return (grid_for(ctx, n, per_block) + 7u) & ~7u;
}

// ---------------------------------------------------------------------------- pooling (NHWC)
// Forward keeps, per output element, the window offset (r*kw + q) of the first maximum in
// row-major window order; padding cells never win (TF MaxPoolV2, math/nn/AllKernels.scala:270-303).
// V channels per thread (V = 4 needs c % 4 == 0 and 16-byte aligned tensors); I is the index type.
// AVG: the mean over the window's cells that lie inside the input instead (TF AvgPool, math/nn/AllKernels.scala:326-353);
// nothing is recorded for the backward pass.
template <int V, typename I, bool AVG>
__global__ __launch_bounds__(256) void pool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ arg,
                                                           int n, int h, int w, int c, int ho, int wo, int kh, int kw, int sh,
                                                           int sw, int pt, int pl) {
  const I cv = (I)(c / V);
  const I total = (I)n * ho * wo * cv;
  const I stride = (I)gridDim.x * blockDim.x;
  for (I i = (I)xcd_contiguous_block() * blockDim.x + threadIdx.x; i < total; i += stride) {
    const I ch = (i % cv) * V;
    I t = i / cv;
    const int ow = (int)(t % wo); t /= wo;
    const int oh = (int)(t % ho);
    const I b = t / ho;
    float best[V];
    int at[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { best[v] = AVG ? 0.f : -INFINITY; at[v] = 0; }
    int cells = 0;
    for (int r = 0; r < kh; ++r) {
      const int iy = oh * sh - pt + r;
      if (iy < 0 || iy >= h) continue;
      for (int q = 0; q < kw; ++q) {
        const int ix = ow * sw - pl + q;
        if (ix < 0 || ix >= w) continue;
        const float* src = x + ((b * h + iy) * w + ix) * c + ch;
        float val[V];
        if constexpr (V == 4) { const float4 f = *(const float4*)src; val[0] = f.x; val[1] = f.y; val[2] = f.z; val[3] = f.w; }
        else val[0] = *src;
        ++cells;
#pragma unroll
        for (int v = 0; v < V; ++v) {
          if constexpr (AVG) best[v] += val[v];
          else if (val[v] > best[v]) { best[v] = val[v]; at[v] = r * kw + q; }
        }
      }
    }
    if constexpr (AVG) {
      const float count = (float)(cells > 0 ? cells : 1);
#pragma unroll
      for (int v = 0; v < V; ++v) best[v] = best[v] / count;
    }
    const I o = i * V;
    if constexpr (V == 4) {
      *(float4*)(y + o) = make_float4(best[0], best[1], best[2], best[3]);
      if constexpr (!AVG) *(uint32_t*)(arg + o) = (uint32_t)at[0] | ((uint32_t)at[1] << 8) | ((uint32_t)at[2] << 16) | ((uint32_t)at[3] << 24);
    } else {
      y[o] = best[0];
      if constexpr (!AVG) arg[o] = (uint8_t)at[0];
    }
  }
}


// The same forward pass for 2x2 max windows, 4 channels per thread, 32-bit indices: the four window cells are requested
// together (cells outside the input re-read the tensor's first element and never win), then compared in window order.
__global__ __launch_bounds__(256) void pool2x2_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ arg,
                                                           int n, int h, int w, int c, int ho, int wo, int sh, int sw, int pt, int pl,
                                                           FastDiv by_cv, FastDiv by_wo, FastDiv by_ho) {
  const uint32_t cv = (uint32_t)(c / 4);
  const uint32_t total = (uint32_t)n * ho * wo * cv;
  const uint32_t stride = (uint32_t)gridDim.x * blockDim.x;
  for (uint32_t i = (uint32_t)xcd_contiguous_block() * blockDim.x + threadIdx.x; i < total; i += stride) {
    uint32_t t = div_by(i, by_cv);
    const uint32_t ch = (i - t * cv) * 4;
    uint32_t t2 = div_by(t, by_wo);
    const int ow = (int)(t - t2 * (uint32_t)wo);
    const uint32_t b = div_by(t2, by_ho);
    const int oh = (int)(t2 - b * (uint32_t)ho);
    float4 val[4];
    bool in[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int iy = oh * sh - pt + (k >> 1), ix = ow * sw - pl + (k & 1);
      in[k] = (unsigned)iy < (unsigned)h && (unsigned)ix < (unsigned)w;
      val[k] = *(const float4*)(x + (in[k] ? ((b * h + iy) * w + ix) * c + ch : 0u));
    }
    float best[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    uint32_t at[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float v[4] = {val[k].x, val[k].y, val[k].z, val[k].w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (in[k] && v[e] > best[e]) { best[e] = v[e]; at[e] = (uint32_t)k; }
    }
    const uint32_t o = i * 4;
    *(float4*)(y + o) = make_float4(best[0], best[1], best[2], best[3]);
    *(uint32_t*)(arg + o) = at[0] | (at[1] << 8) | (at[2] << 16) | (at[3] << 24);
  }
}

static bool pool_vec4(const void* a, const void* b, const void* m, int c) {
  return c % 4 == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0 && (reinterpret_cast<uintptr_t>(m) & 3u) == 0;
}

int launch_pool_fwd(sn_ctx* ctx, bool avg, const float* x, float* y, uint8_t* arg, int n, int h, int w, int c, int ho, int wo, int kh,
                    int kw, int sh, int sw, int pt, int pl) {
  const int64_t total = (int64_t)n * ho * wo * c;
  if (total <= 0) return SN_OK;
  const bool small = total < (1ll << 31) && (int64_t)n * h * w * c < (1ll << 31);
  const bool v4 = pool_vec4(x, y, arg, c);
  const dim3 grid(grid_for_xcd(ctx, v4 ? total / 4 : total, 256));
  LaunchScope scope(ctx, avg ? "avgpool_forward" : "maxpool_forward");
#define SN_POOL_FWD(V, I)                                                                                                              \
  do {                                                                                                                                 \
    if (avg) hipLaunchKernelGGL((pool_fwd_kernel<V, I, true>), grid, dim3(256), 0, ctx->stream, x, y, arg, n, h, w, c, ho, wo, kh, kw, sh, sw, pt, pl); \
    else hipLaunchKernelGGL((pool_fwd_kernel<V, I, false>), grid, dim3(256), 0, ctx->stream, x, y, arg, n, h, w, c, ho, wo, kh, kw, sh, sw, pt, pl);    \
  } while (0)
  if (v4 && small && !avg && kh == 2 && kw == 2)
    hipLaunchKernelGGL(pool2x2_fwd_kernel, grid, dim3(256), 0, ctx->stream, x, y, arg, n, h, w, c, ho, wo, sh, sw, pt, pl, fast_div((uint32_t)(c / 4)),
                       fast_div((uint32_t)wo), fast_div((uint32_t)ho));
  else if (v4 && small) SN_POOL_FWD(4, uint32_t);
  else if (v4) SN_POOL_FWD(4, uint64_t);
  else if (small) SN_POOL_FWD(1, uint32_t);
  else SN_POOL_FWD(1, uint64_t);
#undef SN_POOL_FWD
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// Backward as a gather: each input element adds the gradients of the windows whose recorded
// first maximum is this element (TF MaxPoolGradV2, math/nn/AllKernels.scala:305-324). No atomics.
// AVG: every window that covers the element hands it its gradient times 1 / (the window's cells inside the input)
// (TF AvgPoolGrad, math/nn/AllKernels.scala:355-381).
template <int V, typename I, bool AVG>
__global__ __launch_bounds__(256) void pool_bwd_kernel(const float* __restrict__ dy, const uint8_t* __restrict__ arg,
                                                           float* __restrict__ dx, int n, int h, int w, int c, int ho, int wo,
                                                           int kh, int kw, int sh, int sw, int pt, int pl,
                                                           const float* __restrict__ y_in, int act, float act_param) {
  const I cv = (I)(c / V);
  const I total = (I)n * h * w * cv;
  const I stride = (I)gridDim.x * blockDim.x;
  for (I i = (I)xcd_contiguous_block() * blockDim.x + threadIdx.x; i < total; i += stride) {
    const I ch = (i % cv) * V;
    I t = i / cv;
    const int ix = (int)(t % w); t /= w;
    const int iy = (int)(t % h);
    const I b = t / h;
    float s[V];
#pragma unroll
    for (int v = 0; v < V; ++v) s[v] = 0.f;
    // windows (oh, ow) with oh*sh - pt <= iy < oh*sh - pt + kh
    int oh_lo = iy + pt - kh + 1;
    oh_lo = oh_lo <= 0 ? 0 : (oh_lo + sh - 1) / sh;
    int oh_hi = (iy + pt) / sh;
    if (oh_hi > ho - 1) oh_hi = ho - 1;
    int ow_lo = ix + pl - kw + 1;
    ow_lo = ow_lo <= 0 ? 0 : (ow_lo + sw - 1) / sw;
    int ow_hi = (ix + pl) / sw;
    if (ow_hi > wo - 1) ow_hi = wo - 1;
    for (int oh = oh_lo; oh <= oh_hi; ++oh) {
      const int r = iy - (oh * sh - pt);
      const int y0 = oh * sh - pt;
      const int rows_in = (y0 + kh < h ? y0 + kh : h) - (y0 > 0 ? y0 : 0);
      for (int ow = ow_lo; ow <= ow_hi; ++ow) {
        const int q = ix - (ow * sw - pl);
        const I o = ((b * ho + oh) * wo + ow) * c + ch;
        if constexpr (AVG) {
          const int x0 = ow * sw - pl;
          const int cols_in = (x0 + kw < w ? x0 + kw : w) - (x0 > 0 ? x0 : 0);
          const float share = 1.0f / (float)(rows_in * cols_in);
          if constexpr (V == 4) {
            const float4 g = *(const float4*)(dy + o);
            s[0] += g.x * share; s[1] += g.y * share; s[2] += g.z * share; s[3] += g.w * share;
          } else {
            s[0] += dy[o] * share;
          }
          continue;
        }
        const uint32_t want = (uint32_t)(r * kw + q);
        if constexpr (V == 4) {
          const uint32_t a4 = *(const uint32_t*)(arg + o);
          const float4 g = *(const float4*)(dy + o);
          if ((a4 & 255u) == want) s[0] += g.x;
          if (((a4 >> 8) & 255u) == want) s[1] += g.y;
          if (((a4 >> 16) & 255u) == want) s[2] += g.z;
          if ((a4 >> 24) == want) s[3] += g.w;
        } else {
          if (arg[o] == want) s[0] += dy[o];
        }
      }
    }
    if (y_in) {  // the pooled tensor is the output y of a layer with an activation: hand back act'(y) * gradient
      if constexpr (V == 4) {
        const float4 yv = *(const float4*)(y_in + i * 4);
        s[0] = act_bwd(act, yv.x, s[0], act_param);
        s[1] = act_bwd(act, yv.y, s[1], act_param);
        s[2] = act_bwd(act, yv.z, s[2], act_param);
        s[3] = act_bwd(act, yv.w, s[3], act_param);
      } else {
        s[0] = act_bwd(act, y_in[i], s[0], act_param);
      }
    }
    if constexpr (V == 4) *(float4*)(dx + i * 4) = make_float4(s[0], s[1], s[2], s[3]);
    else dx[i] = s[0];
  }
}

// The same backward pass for 2x2 max windows, 4 channels per thread, 32-bit indices: an input element lies in at most 2 x 2
// windows (oh_hi - a, ow_hi - d for a, d in {0, 1}); their argmax words and gradients are requested together (windows that do
// not exist re-read the first element and are ignored) and added in the order of the general kernel (oh, then ow, ascending).
template <int S>  // both strides when they are equal and 1 or 2 (divisions by a constant), 0: read sh, sw
__global__ __launch_bounds__(256) void pool2x2_bwd_kernel(const float* __restrict__ dy, const uint8_t* __restrict__ arg,
                                                           float* __restrict__ dx, int n, int h, int w, int c, int ho, int wo, int sh_,
                                                           int sw_, int pt, int pl, const float* __restrict__ y_in, int act, float act_param,
                                                           FastDiv by_cv, FastDiv by_w, FastDiv by_h) {
  const int sh = S ? S : sh_, sw = S ? S : sw_;
  const uint32_t cv = (uint32_t)(c / 4);
  const uint32_t total = (uint32_t)n * h * w * cv;
  const uint32_t stride = (uint32_t)gridDim.x * blockDim.x;
  for (uint32_t i = (uint32_t)xcd_contiguous_block() * blockDim.x + threadIdx.x; i < total; i += stride) {
    uint32_t t = div_by(i, by_cv);
    const uint32_t ch = (i - t * cv) * 4;
    uint32_t t2 = div_by(t, by_w);
    const int ix = (int)(t - t2 * (uint32_t)w);
    const uint32_t b = div_by(t2, by_h);
    const int iy = (int)(t2 - b * (uint32_t)h);
    int oh_lo = iy + pt - 1;
    oh_lo = oh_lo <= 0 ? 0 : (oh_lo + sh - 1) / sh;
    int oh_hi = (iy + pt) / sh;
    if (oh_hi > ho - 1) oh_hi = ho - 1;
    int ow_lo = ix + pl - 1;
    ow_lo = ow_lo <= 0 ? 0 : (ow_lo + sw - 1) / sw;
    int ow_hi = (ix + pl) / sw;
    if (ow_hi > wo - 1) ow_hi = wo - 1;
    float4 yv = make_float4(0.f, 0.f, 0.f, 0.f);
    if (y_in) yv = *(const float4*)(y_in + i * 4);
    uint32_t a4[4], want[4];
    float4 g[4];
    bool on[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int oh = oh_lo + (k >> 1), ow = ow_lo + (k & 1);
      on[k] = oh <= oh_hi && ow <= ow_hi;
      const uint32_t o = on[k] ? ((b * ho + oh) * wo + ow) * c + ch : 0u;
      want[k] = (uint32_t)((iy - (oh * sh - pt)) * 2 + (ix - (ow * sw - pl)));
      a4[k] = *(const uint32_t*)(arg + o);
      g[k] = *(const float4*)(dy + o);
    }
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (!on[k]) continue;
      if ((a4[k] & 255u) == want[k]) s[0] += g[k].x;
      if (((a4[k] >> 8) & 255u) == want[k]) s[1] += g[k].y;
      if (((a4[k] >> 16) & 255u) == want[k]) s[2] += g[k].z;
      if ((a4[k] >> 24) == want[k]) s[3] += g[k].w;
    }
    if (y_in) {
      s[0] = act_bwd(act, yv.x, s[0], act_param);
      s[1] = act_bwd(act, yv.y, s[1], act_param);
      s[2] = act_bwd(act, yv.z, s[2], act_param);
      s[3] = act_bwd(act, yv.w, s[3], act_param);
    }
    *(float4*)(dx + i * 4) = make_float4(s[0], s[1], s[2], s[3]);
  }
}

int launch_pool_bwd(sn_ctx* ctx, bool avg, const float* dy, const uint8_t* arg, float* dx, int n, int h, int w, int c, int ho, int wo,
                    int kh, int kw, int sh, int sw, int pt, int pl, const float* y_in, int act, float act_param) {
  const int64_t total = (int64_t)n * h * w * c;
  if (total <= 0) return SN_OK;
  const bool small = total < (1ll << 31) && (int64_t)n * ho * wo * c < (1ll << 31);
  const bool v4 = pool_vec4(dy, dx, arg, c) && (reinterpret_cast<uintptr_t>(y_in) & 15u) == 0;
  const dim3 grid(grid_for_xcd(ctx, v4 ? total / 4 : total, 256));
  LaunchScope scope(ctx, avg ? (y_in ? "avgpool_activation_backward" : "avgpool_backward") : (y_in ? "maxpool_activation_backward" : "maxpool_backward"));
#define SN_POOL_BWD(V, I)                                                                                                     \
  do {                                                                                                                        \
    if (avg)                                                                                                                  \
      hipLaunchKernelGGL((pool_bwd_kernel<V, I, true>), grid, dim3(256), 0, ctx->stream, dy, arg, dx, n, h, w, c, ho, wo, kh, kw, sh, sw, \
                         pt, pl, y_in, act, act_param);                                                                       \
    else                                                                                                                      \
      hipLaunchKernelGGL((pool_bwd_kernel<V, I, false>), grid, dim3(256), 0, ctx->stream, dy, arg, dx, n, h, w, c, ho, wo, kh, kw, sh, sw, \
                         pt, pl, y_in, act, act_param);                                                                       \
  } while (0)
  if (v4 && small && !avg && kh == 2 && kw == 2)
  {
    const FastDiv by_cv = fast_div((uint32_t)(c / 4)), by_w = fast_div((uint32_t)w), by_h = fast_div((uint32_t)h);
    if (sh == 1 && sw == 1)
      hipLaunchKernelGGL(pool2x2_bwd_kernel<1>, grid, dim3(256), 0, ctx->stream, dy, arg, dx, n, h, w, c, ho, wo, sh, sw, pt, pl, y_in, act, act_param, by_cv, by_w, by_h);
    else if (sh == 2 && sw == 2)
      hipLaunchKernelGGL(pool2x2_bwd_kernel<2>, grid, dim3(256), 0, ctx->stream, dy, arg, dx, n, h, w, c, ho, wo, sh, sw, pt, pl, y_in, act, act_param, by_cv, by_w, by_h);
    else
      hipLaunchKernelGGL(pool2x2_bwd_kernel<0>, grid, dim3(256), 0, ctx->stream, dy, arg, dx, n, h, w, c, ho, wo, sh, sw, pt, pl, y_in, act, act_param, by_cv, by_w, by_h);
  }
  else if (v4 && small) SN_POOL_BWD(4, uint32_t);
  else if (v4) SN_POOL_BWD(4, uint64_t);
  else if (small) SN_POOL_BWD(1, uint32_t);
  else SN_POOL_BWD(1, uint64_t);
#undef SN_POOL_BWD
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---------------------------------------------------------------------------- LSTM gate maths
// c = c_prev * f + i * g ; h = o * tanh(c) (layer/RNN.scala:336-337), gates f,i,o = sigmoid, g = tanh.
__global__ __launch_bounds__(256) void lstm_gates_fwd_kernel(LstmGateArgs a, int rows, int hidden) {
  const int64_t total = (int64_t)rows * hidden;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / hidden;
    const int u = (int)(i % hidden);
    const int64_t zb = r * 4 * hidden + u;
    const float f = sigmoidf_(a.z[zb]);
    const float in = sigmoidf_(a.z[zb + hidden]);
    const float g = tanhf(a.z[zb + 2 * hidden]);
    const float o = sigmoidf_(a.z[zb + 3 * hidden]);
    const float cp = a.c_prev ? a.c_prev[i] : 0.f;
    const float c = cp * f + in * g;
    a.gates[zb] = f;
    a.gates[zb + hidden] = in;
    a.gates[zb + 2 * hidden] = g;
    a.gates[zb + 3 * hidden] = o;
    a.c[i] = c;
    a.h[i] = o * tanhf(c);
  }
}

int launch_lstm_gates_fwd(sn_ctx* ctx, const LstmGateArgs& a, int rows, int hidden) {
  const int64_t total = (int64_t)rows * hidden;
  if (total <= 0) return SN_OK;
  LaunchScope scope(ctx, "lstm_gates_forward");
  hipLaunchKernelGGL(lstm_gates_fwd_kernel, dim3(grid_for(ctx, total, 256)), dim3(256), 0, ctx->stream, a, rows, hidden);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// Reverse of the step above, by the reference's local gradient rules:
//   do = dh * tanh(c);  dc += (1 - tanh(c)^2) * (dh * o)
//   df = dc * c_prev;   di = dc * g;   dg = dc * i;   dc_prev = dc * f
//   dz_gate = act'(z_gate) * d_gate  (sigmoid: s(1-s), tanh: 1 - g^2)
__global__ __launch_bounds__(256) void lstm_gates_bwd_kernel(LstmGateBwdArgs a, int rows, int hidden) {
  const int64_t total = (int64_t)rows * hidden;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / hidden;
    const int u = (int)(i % hidden);
    const int64_t zb = r * 4 * hidden + u;
    const float f = a.gates[zb], in = a.gates[zb + hidden], g = a.gates[zb + 2 * hidden], o = a.gates[zb + 3 * hidden];
    const float tc = tanhf(a.c[i]);
    float dh = a.dh_parts > 0 ? a.dh[i] : 0.f;
    for (int p = 1; p < a.dh_parts; ++p) dh += a.dh[i + p * a.dh_part_stride];
    if (a.dy_seq) dh = dh + a.dy_seq[r * a.dy_seq_ld + u];
    const float d_o = dh * tc;
    float dc = a.dc_is_zero ? 0.f : a.dc[i];
    dc = dc + (1.0f - tc * tc) * (dh * o);
    const float cp = a.c_prev ? a.c_prev[i] : 0.f;
    const float df = dc * cp, di = dc * g, dg = dc * in;
    a.dc[i] = dc * f;
    a.dz[zb] = (f * (1.0f - f)) * df;
    a.dz[zb + hidden] = (in * (1.0f - in)) * di;
    a.dz[zb + 2 * hidden] = (1.0f - g * g) * dg;
    a.dz[zb + 3 * hidden] = (o * (1.0f - o)) * d_o;
  }
}

__global__ __launch_bounds__(256) void sequence_gather_kernel(const float* __restrict__ slices, int64_t slice_stride, int first,
                                                               float* __restrict__ out, int rows, int T, int H) {
  const int64_t total = (int64_t)rows * T * H;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int u = (int)(i % H);
    const int64_t rt = i / H;
    const int t = (int)(rt % T);
    const int64_t r = rt / T;
    out[i] = slices[(int64_t)(first + t) * slice_stride + r * H + u];
  }
}

int launch_sequence_gather(sn_ctx* ctx, const float* slices, int64_t slice_stride, int first, float* out, int rows, int T, int H) {
  const int64_t total = (int64_t)rows * T * H;
  if (total <= 0) return SN_OK;
  LaunchScope scope(ctx, "sequence_gather");
  hipLaunchKernelGGL(sequence_gather_kernel, dim3(grid_for(ctx, total, 1024)), dim3(256), 0, ctx->stream, slices, slice_stride, first, out, rows,
                     T, H);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

__global__ __launch_bounds__(256) void step_slice_add_kernel(float* __restrict__ dst, const float* __restrict__ src, int64_t src_ld,
                                                              int rows, int H, int accumulate) {
  const int64_t total = (int64_t)rows * H;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / H;
    const int u = (int)(i % H);
    const float v = src[r * src_ld + u];
    dst[i] = accumulate ? dst[i] + v : v;
  }
}

int launch_step_slice_add(sn_ctx* ctx, float* dst, const float* src, int64_t src_ld, int rows, int H, bool accumulate) {
  const int64_t total = (int64_t)rows * H;
  if (total <= 0) return SN_OK;
  LaunchScope scope(ctx, "sequence_step_gradient");
  hipLaunchKernelGGL(step_slice_add_kernel, dim3(grid_for(ctx, total, 1024)), dim3(256), 0, ctx->stream, dst, src, src_ld, rows, H,
                     accumulate ? 1 : 0);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_lstm_gates_bwd(sn_ctx* ctx, const LstmGateBwdArgs& a, int rows, int hidden) {
  const int64_t total = (int64_t)rows * hidden;
  if (total <= 0) return SN_OK;
  LaunchScope scope(ctx, "lstm_gates_backward");
  hipLaunchKernelGGL(lstm_gates_bwd_kernel, dim3(grid_for(ctx, total, 256)), dim3(256), 0, ctx->stream, a, rows, hidden);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
