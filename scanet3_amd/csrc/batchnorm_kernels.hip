// Batch normalisation over the last axis of a channels-last tensor viewed as [rows, C]
// (generic `batchNorm`, math/nn/AllKernels.scala:663-684, as the BatchNorm layer calls it for
// `axes = Seq(-1)`, models/layer/BatchNorm.scala:123-143).
//
//   training:  mean = sum(x)/rows, var = sum((x-mean)^2)/rows   (alg/AllKernels.scala:505-513)
//   frozen:    mean, var = the moving statistics
//   inv = rsqrt(var + eps) * gamma;  y = (x*inv - mean*inv) + beta
//
// All of it is memory bound: every pass reads the activation once with 8 row-loads in flight per
// lane; the per-channel reductions are cut into row slices so the grid covers the chip, and the
// slices are added in slice order by one thread per channel (deterministic, no atomics).
#include "common.hpp"

namespace sn {
namespace {

typedef float bn_f4 __attribute__((ext_vector_type(4)));

enum { BN_SUM = 0, BN_SQDIFF = 1, BN_GRAD = 2 };

// Block = 64 columns x 4 waves; wave w takes rows r0+w, r0+w+4, ... of its slice.
// BN_SUM:    part0 = sum x
// BN_SQDIFF: part0 = sum (x - mean)^2
// BN_GRAD:   part0 = sum dy, part1 = sum dy * (x - mean)
template <int MODE>
__global__ __launch_bounds__(256) void bn_reduce_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                         const float* __restrict__ mean, float* __restrict__ part0,
                                                         float* __restrict__ part1, int64_t rows, int cols, int64_t rows_per_slice) {
  __shared__ float smem[2][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < rows ? r0 + rows_per_slice : rows;
  float s0 = 0.f, s1 = 0.f;
  if (c < cols) {
    const float m = MODE == BN_SUM ? 0.f : mean[c];
    int64_t r = r0 + wave;
    for (; r + 28 < r1; r += 32) {
      float a[8], b[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) a[u] = x[(r + 4 * u) * cols + c];
      if (MODE == BN_GRAD) {
#pragma unroll
        for (int u = 0; u < 8; ++u) b[u] = dy[(r + 4 * u) * cols + c];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (MODE == BN_SUM) s0 += a[u];
        if (MODE == BN_SQDIFF) { const float d = a[u] - m; s0 += d * d; }
        if (MODE == BN_GRAD) { s0 += b[u]; s1 += b[u] * (a[u] - m); }
      }
    }
    for (; r < r1; r += 4) {
      const float a = x[r * cols + c];
      if (MODE == BN_SUM) s0 += a;
      if (MODE == BN_SQDIFF) { const float d = a - m; s0 += d * d; }
      if (MODE == BN_GRAD) { const float b = dy[r * cols + c]; s0 += b; s1 += b * (a - m); }
    }
  }
  smem[0][wave][lane] = s0;
  if (MODE == BN_GRAD) smem[1][wave][lane] = s1;
  __syncthreads();
  if (wave == 0 && c < cols) {
    part0[(int64_t)blockIdx.y * cols + c] = ((smem[0][0][lane] + smem[0][1][lane]) + smem[0][2][lane]) + smem[0][3][lane];
    if (MODE == BN_GRAD)
      part1[(int64_t)blockIdx.y * cols + c] = ((smem[1][0][lane] + smem[1][1][lane]) + smem[1][2][lane]) + smem[1][3][lane];
  }
}

// Few channels (C/4 divides 256): the tensor is read as one stream of float4; a thread's float4 index moves in steps
// of 256, so it stays on the same four channels and every wavefront load covers 1 KiB of consecutive memory.
// A block owns `per4` consecutive float4 (a multiple of 256); threads with equal t % (C/4) meet in LDS.
template <int MODE>
__global__ __launch_bounds__(256) void bn_reduce_v4_kernel(const bn_f4* __restrict__ x, const bn_f4* __restrict__ dy,
                                                            const float* __restrict__ mean, float* __restrict__ part0,
                                                            float* __restrict__ part1, int64_t n4, int cols, int64_t per4) {
  __shared__ bn_f4 smem[2][256];
  const int t = threadIdx.x, cg = cols / 4, g = t % cg;
  const int64_t begin = (int64_t)blockIdx.x * per4;
  const int64_t end = begin + per4 < n4 ? begin + per4 : n4;
  bn_f4 m = {0.f, 0.f, 0.f, 0.f};
  if (MODE != BN_SUM) m = *(const bn_f4*)(mean + 4 * g);
  bn_f4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
  int64_t i = begin + t;
  for (; i + 7 * 256 < end; i += 8 * 256) {
    bn_f4 a[8], b[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = __builtin_nontemporal_load(x + i + u * 256);
    if (MODE == BN_GRAD) {
#pragma unroll
      for (int u = 0; u < 8; ++u) b[u] = __builtin_nontemporal_load(dy + i + u * 256);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (MODE == BN_SUM) s0 = s0 + a[u];
      if (MODE == BN_SQDIFF) { const bn_f4 d = a[u] - m; s0 = s0 + d * d; }
      if (MODE == BN_GRAD) { s0 = s0 + b[u]; s1 = s1 + b[u] * (a[u] - m); }
    }
  }
  for (; i < end; i += 256) {
    const bn_f4 a = x[i];
    if (MODE == BN_SUM) s0 = s0 + a;
    if (MODE == BN_SQDIFF) { const bn_f4 d = a - m; s0 = s0 + d * d; }
    if (MODE == BN_GRAD) { const bn_f4 b = dy[i]; s0 = s0 + b; s1 = s1 + b * (a - m); }
  }
  smem[0][t] = s0;
  if (MODE == BN_GRAD) smem[1][t] = s1;
  __syncthreads();
  if (t < cg) {
    bn_f4 r0 = smem[0][t], r1 = smem[1][t];
    for (int j = t + cg; j < 256; j += cg) {
      r0 = r0 + smem[0][j];
      if (MODE == BN_GRAD) r1 = r1 + smem[1][j];
    }
    *(bn_f4*)(part0 + (int64_t)blockIdx.x * cols + 4 * t) = r0;
    if (MODE == BN_GRAD) *(bn_f4*)(part1 + (int64_t)blockIdx.x * cols + 4 * t) = r1;
  }
}

// Sum of one channel's slices by 16 threads: a block is 16 channels x 16 slice lanes; lane j adds slices j, j+16, ...
// (8 loads in flight), the 16 lane sums are added in lane order.  Every thread of the block must call it; the total is
// returned to all of them.  (One thread per channel would walk up to 1024 slices one memory latency after another.)
__device__ __forceinline__ float slices_total(const float* __restrict__ part, int slices, int cols, int c, float (*smem)[16]) {
  const int cl = threadIdx.x & 15, sl = threadIdx.x >> 4;
  float s = 0.f;
  if (c < cols) {
    int i = sl;
    for (; i + 7 * 16 < slices; i += 8 * 16) {
      float a[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) a[u] = part[(int64_t)(i + 16 * u) * cols + c];
#pragma unroll
      for (int u = 0; u < 8; ++u) s += a[u];
    }
    for (; i < slices; i += 16) s += part[(int64_t)i * cols + c];
  }
  __syncthreads();  // a previous call's readers are done with smem
  smem[sl][cl] = s;
  __syncthreads();
  float total = smem[0][cl];
#pragma unroll
  for (int j = 1; j < 16; ++j) total += smem[j][cl];
  return total;
}

// Finishing kernels: block = 16 channels x 16 slice lanes, grid = ceil(C/16).
__global__ __launch_bounds__(256) void bn_mean_kernel(const float* __restrict__ part, int slices, int cols, float n, float* __restrict__ mean) {
  __shared__ float smem[16][16];
  const int c = blockIdx.x * 16 + (threadIdx.x & 15);
  const float total = slices_total(part, slices, cols, c, smem);
  if (threadIdx.x < 16 && c < cols) mean[c] = total / n;
}

// var from the slices (training) or from the moving variance (part == null), then r = 1/sqrt(var+eps), inv = r*gamma
__global__ __launch_bounds__(256) void bn_scale_kernel(const float* __restrict__ part, int slices, int cols, float n, float eps,
                                                        const float* __restrict__ gamma, const float* __restrict__ moving_mean,
                                                        const float* __restrict__ moving_var, float* __restrict__ mean,
                                                        float* __restrict__ var, float* __restrict__ r, float* __restrict__ inv) {
  __shared__ float smem[16][16];
  const int c = blockIdx.x * 16 + (threadIdx.x & 15);
  float total = 0.f;
  if (part) total = slices_total(part, slices, cols, c, smem);  // uniform over the block
  if (threadIdx.x >= 16 || c >= cols) return;
  float v;
  if (part) {
    v = total / n;
  } else {
    v = moving_var[c];
    mean[c] = moving_mean[c];
  }
  var[c] = v;
  const float rr = 1.0f / sqrtf(v + eps);
  r[c] = rr;
  inv[c] = rr * gamma[c];
}

template <bool V4>
__global__ __launch_bounds__(256) void bn_apply_kernel(const float* __restrict__ x, const float* __restrict__ mean,
                                                        const float* __restrict__ inv, const float* __restrict__ beta,
                                                        float* __restrict__ y, int64_t n, int cols, int centred) {
  // generic form: (x*inv - mean*inv) + beta (math/nn/AllKernels.scala:676-683); the fused op: (x - mean)*inv + beta
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  if (V4) {
    const int64_t n4 = n / 4;
    // the column walks with the index: one division at the start, then an addition and a wrap per trip
    const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int c = (int)((i0 * 4) % cols);
    const int cstep = (int)((stride * 4) % cols);
    for (int64_t i = i0; i < n4; i += stride, c = c + cstep >= cols ? c + cstep - cols : c + cstep) {
      const bn_f4 xv = *(const bn_f4*)(x + i * 4), iv = *(const bn_f4*)(inv + c), mv = *(const bn_f4*)(mean + c), bv = *(const bn_f4*)(beta + c);
      bn_f4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = centred ? (xv[e] - mv[e]) * iv[e] + bv[e] : (xv[e] * iv[e] - mv[e] * iv[e]) + bv[e];
      *(bn_f4*)(y + i * 4) = o;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
      const int c = (int)(i % cols);
      y[i] = centred ? (x[i] - mean[c]) * inv[c] + beta[c] : (x[i] * inv[c] - mean[c] * inv[c]) + beta[c];
    }
  }
}

// The statistics the reference's wiring hands to the fused gradient op: "mean" = the unbiased variance, "variance" = the mean.
__global__ __launch_bounds__(256) void bn_fused_wiring_kernel(const float* __restrict__ mean, const float* __restrict__ var,
                                                               const float* __restrict__ gamma, float unbias, float eps,
                                                               float* __restrict__ g_mean, float* __restrict__ g_r,
                                                               float* __restrict__ g_inv, int cols) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  g_mean[c] = var[c] * unbias;
  const float rr = 1.0f / sqrtf(mean[c] + eps);   // NaN for a channel whose mean is below -epsilon, as in the reference
  g_r[c] = rr;
  g_inv[c] = rr * gamma[c];
}

// d beta = S1, d gamma = S2 * r; k1 = S1/n, k2 = r*r*S2/n for the input gradient
__global__ __launch_bounds__(256) void bn_grad_finish_kernel(const float* __restrict__ part0, const float* __restrict__ part1, int slices,
                                                              int cols, float n, const float* __restrict__ r, float* __restrict__ dbeta,
                                                              float* __restrict__ dgamma, float* __restrict__ k1, float* __restrict__ k2) {
  __shared__ float smem[16][16];
  const int c = blockIdx.x * 16 + (threadIdx.x & 15);
  const float s1 = slices_total(part0, slices, cols, c, smem);
  const float s2 = slices_total(part1, slices, cols, c, smem);
  if (threadIdx.x >= 16 || c >= cols) return;
  const float rr = r[c];
  dbeta[c] = s1;
  dgamma[c] = s2 * rr;
  k1[c] = s1 / n;
  k2[c] = rr * rr * s2 / n;
}

// Gradient of the activation that produced x (the layer below), from its output: models/Activation.scala:32-83.
__device__ __forceinline__ float below_act_grad(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

// dx = inv * (dy - k1 - (x - mean) * k2), then (act != identity) through the activation of the layer that wrote x
template <bool V4>
__global__ __launch_bounds__(256) void bn_dx_kernel(const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ mean,
                                                     const float* __restrict__ inv, const float* __restrict__ k1,
                                                     const float* __restrict__ k2, float* __restrict__ dx, int64_t n, int cols, int act,
                                                     float act_param) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  if (V4) {
    const int64_t n4 = n / 4;
    const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int c = (int)((i0 * 4) % cols);
    const int cstep = (int)((stride * 4) % cols);
    for (int64_t i = i0; i < n4; i += stride, c = c + cstep >= cols ? c + cstep - cols : c + cstep) {
      const bn_f4 xv = *(const bn_f4*)(x + i * 4), gv = *(const bn_f4*)(dy + i * 4), iv = *(const bn_f4*)(inv + c),
                  mv = *(const bn_f4*)(mean + c), a = *(const bn_f4*)(k1 + c), b = *(const bn_f4*)(k2 + c);
      bn_f4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = below_act_grad(act, xv[e], iv[e] * ((gv[e] - a[e]) - (xv[e] - mv[e]) * b[e]), act_param);
      *(bn_f4*)(dx + i * 4) = o;
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
      const int c = (int)(i % cols);
      dx[i] = below_act_grad(act, x[i], inv[c] * ((dy[i] - k1[c]) - (x[i] - mean[c]) * k2[c]), act_param);
    }
  }
}

// decayingAvg (alg/AllKernels.scala:541-544): moving = momentum*moving + (1-momentum)*batch
__global__ __launch_bounds__(256) void bn_moving_kernel(float* __restrict__ moving_mean, float* __restrict__ moving_var,
                                                         const float* __restrict__ mean, const float* __restrict__ var, int cols, float momentum) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  const float keep = 1.0f - momentum;
  moving_mean[c] = momentum * moving_mean[c] + keep * mean[c];
  moving_var[c] = momentum * moving_var[c] + keep * var[c];
}

unsigned grid_for(const sn_ctx* ctx, int64_t n, int per_block) {
  int64_t blocks = ceil_div(n, per_block);
  const int64_t cap = (int64_t)ctx->compute_units * 16;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1u : (unsigned)blocks;
}

int slices_for(const sn_ctx* ctx, int64_t rows, int cols) {
  const int64_t col_blocks = ceil_div((int64_t)cols, (int64_t)64);
  int64_t s = ceil_div((int64_t)ctx->compute_units * 4, col_blocks);
  const int64_t by_rows = ceil_div(rows, (int64_t)64);  // at least 64 rows (16 per wave) in a slice
  if (s > by_rows) s = by_rows;
  if (s > 1024) s = 1024;
  return s < 1 ? 1 : (int)s;
}

// the float4-stream reduction: C/4 divides 256 and enough data for more than one block
bool stream_form(int64_t rows, int cols) { return cols % 4 == 0 && cols <= 1024 && 256 % (cols / 4) == 0 && rows * cols >= 4 * 8 * 256; }
int stream_slices(const sn_ctx* ctx, int64_t n4) {
  int64_t s = ceil_div(n4, (int64_t)8 * 256);  // at least one full trip of 8 loads per thread
  const int64_t cap = (int64_t)ctx->compute_units * 4;
  if (s > cap) s = cap;
  return s < 1 ? 1 : (int)s;
}

// One reduction pass in whichever form fits; returns the number of slices written to part0 (and part1).
template <int MODE>
int reduce_pass(sn_ctx* ctx, const float* x, const float* dy, const float* mean, float* part0, int64_t part1_offset, int64_t rows,
                int cols, int* slices_out) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(part0)) & 15u) == 0;
  if (stream_form(rows, cols) && aligned && part1_offset % 4 == 0) {
    const int64_t n4 = rows * cols / 4;
    const int s = stream_slices(ctx, n4);
    const int64_t per4 = align_up(ceil_div(n4, (int64_t)s), 256);
    hipLaunchKernelGGL((bn_reduce_v4_kernel<MODE>), dim3((unsigned)s), dim3(256), 0, ctx->stream, (const bn_f4*)x, (const bn_f4*)dy, mean,
                       part0, part0 + part1_offset, n4, cols, per4);
    *slices_out = s;
  } else {
    const int s = slices_for(ctx, rows, cols);
    hipLaunchKernelGGL((bn_reduce_kernel<MODE>), dim3((unsigned)ceil_div((int64_t)cols, (int64_t)64), (unsigned)s), dim3(256), 0,
                       ctx->stream, x, dy, mean, part0, part0 + part1_offset, rows, cols, ceil_div(rows, (int64_t)s));
    *slices_out = s;
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int max_slices(const sn_ctx* ctx, int64_t rows, int cols) {
  int s = slices_for(ctx, rows, cols);
  if (stream_form(rows, cols)) s = std::max(s, stream_slices(ctx, rows * cols / 4));
  return s;
}

bool vec4_ok(int cols, std::initializer_list<const void*> ptrs) {
  if (cols % 4 != 0) return false;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15u) return false;
  return true;
}

}  // namespace

int64_t batchnorm_workspace_elems(const sn_ctx* ctx, int64_t rows, int cols) { return (int64_t)2 * max_slices(ctx, rows, cols) * cols; }

int launch_batchnorm_fwd(sn_ctx* ctx, const float* x, float* y, int64_t rows, int cols, const BatchNormArgs& a, bool training, float* ws,
                         int64_t ws_elems) {
  if (rows <= 0 || cols <= 0) return SN_OK;
  SN_REQUIRE(rows * cols <= (int64_t)INT32_MAX * 4, "batch norm over %lld elements exceeds one launch", (long long)(rows * cols));
  const int cb = (int)ceil_div((int64_t)cols, (int64_t)16);  // finishing kernels: 16 channels per block
  if (training) {
    const int64_t need = (int64_t)max_slices(ctx, rows, cols) * cols;
    SN_REQUIRE(need <= ws_elems, "batch norm needs %lld workspace elements, %lld given", (long long)need, (long long)ws_elems);
    int s = 0;
    {
      LaunchScope scope(ctx, "batchnorm_mean");
      SN_TRY(reduce_pass<BN_SUM>(ctx, x, nullptr, nullptr, ws, 0, rows, cols, &s));
      hipLaunchKernelGGL(bn_mean_kernel, dim3(cb), dim3(256), 0, ctx->stream, (const float*)ws, s, cols, (float)rows, a.mean);
    }
    {
      LaunchScope scope(ctx, "batchnorm_variance");
      SN_TRY(reduce_pass<BN_SQDIFF>(ctx, x, nullptr, a.mean, ws, 0, rows, cols, &s));
      hipLaunchKernelGGL(bn_scale_kernel, dim3(cb), dim3(256), 0, ctx->stream, (const float*)ws, s, cols, (float)rows, a.epsilon, a.gamma,
                         (const float*)nullptr, (const float*)nullptr, a.mean, a.var, a.r, a.inv);
    }
    if (a.fused_wiring) {
      LaunchScope scope(ctx, "batchnorm_fused_wiring");
      const float unbias = (float)rows / (float)(rows > 1 ? rows - 1 : 1);
      hipLaunchKernelGGL(bn_fused_wiring_kernel, dim3((unsigned)ceil_div((int64_t)cols, (int64_t)256)), dim3(256), 0, ctx->stream,
                         (const float*)a.mean, (const float*)a.var, a.gamma, unbias, a.epsilon, a.g_mean, a.g_r, a.g_inv, cols);
    }
  } else {
    LaunchScope scope(ctx, "batchnorm_frozen_scale");
    hipLaunchKernelGGL(bn_scale_kernel, dim3(cb), dim3(256), 0, ctx->stream, (const float*)nullptr, 0, cols, 1.0f, a.epsilon, a.gamma,
                       a.moving_mean, a.moving_var, a.mean, a.var, a.r, a.inv);
  }
  const int64_t n = rows * cols;
  LaunchScope scope(ctx, "batchnorm_apply");
  if (vec4_ok(cols, {x, y, a.mean, a.inv, a.beta}))
    hipLaunchKernelGGL((bn_apply_kernel<true>), dim3(grid_for(ctx, n / 4, 1024)), dim3(256), 0, ctx->stream, x, (const float*)a.mean,
                       (const float*)a.inv, a.beta, y, n, cols, a.fused_wiring ? 1 : 0);
  else
    hipLaunchKernelGGL((bn_apply_kernel<false>), dim3(grid_for(ctx, n, 1024)), dim3(256), 0, ctx->stream, x, (const float*)a.mean,
                       (const float*)a.inv, a.beta, y, n, cols, a.fused_wiring ? 1 : 0);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_batchnorm_bwd(sn_ctx* ctx, const float* x, const float* dy, float* dx, int64_t rows, int cols, const BatchNormArgs& a,
                         float* dbeta, float* dgamma, float* ws, int64_t ws_elems, int below_act, float below_act_param) {
  if (rows <= 0 || cols <= 0) return SN_OK;
  const int64_t half = (int64_t)max_slices(ctx, rows, cols) * cols;
  SN_REQUIRE(2 * half <= ws_elems, "batch norm gradient needs %lld workspace elements, %lld given", (long long)(2 * half), (long long)ws_elems);
  const int cb = (int)ceil_div((int64_t)cols, (int64_t)16);  // finishing kernels: 16 channels per block
  float* part1 = ws + half;
  const float* mean = a.fused_wiring ? a.g_mean : a.mean;
  const float* r = a.fused_wiring ? a.g_r : a.r;
  const float* inv = a.fused_wiring ? a.g_inv : a.inv;
  {
    LaunchScope scope(ctx, "batchnorm_gradient_sums");
    int s = 0;
    SN_TRY(reduce_pass<BN_GRAD>(ctx, x, dy, mean, ws, half, rows, cols, &s));
    hipLaunchKernelGGL(bn_grad_finish_kernel, dim3(cb), dim3(256), 0, ctx->stream, (const float*)ws, (const float*)part1, s, cols,
                       (float)rows, r, dbeta, dgamma, a.k1, a.k2);
  }
  if (dx) {
    const int64_t n = rows * cols;
    LaunchScope scope(ctx, "batchnorm_input_gradient");
    if (vec4_ok(cols, {x, dy, dx, mean, inv, a.k1, a.k2}))
      hipLaunchKernelGGL((bn_dx_kernel<true>), dim3(grid_for(ctx, n / 4, 1024)), dim3(256), 0, ctx->stream, x, dy, mean, inv,
                         (const float*)a.k1, (const float*)a.k2, dx, n, cols, below_act, below_act_param);
    else
      hipLaunchKernelGGL((bn_dx_kernel<false>), dim3(grid_for(ctx, n, 1024)), dim3(256), 0, ctx->stream, x, dy, mean, inv,
                         (const float*)a.k1, (const float*)a.k2, dx, n, cols, below_act, below_act_param);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_batchnorm_moving(sn_ctx* ctx, const BatchNormArgs& a, float* moving_mean, float* moving_var, int cols) {
  if (cols <= 0) return SN_OK;
  LaunchScope scope(ctx, "batchnorm_moving_statistics");
  hipLaunchKernelGGL(bn_moving_kernel, dim3((unsigned)ceil_div((int64_t)cols, (int64_t)256)), dim3(256), 0, ctx->stream, moving_mean,
                     moving_var, (const float*)a.mean, (const float*)(a.fused_wiring ? a.mean : a.var), cols, a.momentum);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
