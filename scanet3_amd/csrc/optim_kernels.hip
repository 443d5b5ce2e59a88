// Fused optimizer updates over a flat parameter vector and the K-replica average.
//
// Both families are pure streaming kernels: every element is read once and
// written once, so the bound is HBM bandwidth.  Bytes per element:
//   update:  4 * (2 + 2 * n_state)   (read w, g, states; write w, states)
//   average: 4 * (K + n_outputs)
// The arithmetic follows the reference's operation order exactly (one rounding
// per TensorFlow op, no fused multiply-add), see optimizers/*.scala.
#include "common.hpp"
#include "optim_update.hpp"

#include <cmath>

namespace sn {

typedef float f4 __attribute__((ext_vector_type(4)));

OptScalars make_opt_scalars(const sn_optimizer_desc& d, int iter) {
  OptScalars s;
  s.rate = d.rate;
  s.b1 = d.beta1;
  s.b2 = d.beta2;
  s.eps = d.epsilon;
  s.one_minus_b1 = 1.0f - d.beta1;
  s.one_minus_b2 = 1.0f - d.beta2;
  // `Pow(rate, iter.cast[Float])` (math/alg/AllKernels.scala:546-549), correctly rounded to float32
  s.bc1 = 1.0f - (float)std::pow((double)d.beta1, (double)iter);
  s.bc2 = 1.0f - (float)std::pow((double)d.beta2, (double)iter);
  s.nesterov = d.nesterov;
  s.maximize = d.maximize;
  return s;
}

int opt_state_count(int kind) {
  switch (kind) {
    case SN_OPT_SGD: case SN_OPT_ADAGRAD: case SN_OPT_RMSPROP: return 1;
    case SN_OPT_ADADELTA: case SN_OPT_ADAM: case SN_OPT_NADAM: case SN_OPT_ADAMAX: return 2;
    case SN_OPT_AMSGRAD: return 3;
  }
  return -1;
}

// A block owns T*U consecutive float4 of every array and touches ONE ARRAY AT A TIME: U loads of w,
// then U of g, ... then the stores array by array (measured on MI355X: 6.1 TB/s for Adam's 4 read + 3 write
// streams where the element-interleaved order reaches 5.6 TB/s).
// WBF: the updated weights also leave as bf16 (wbf, same element order), for the bf16 matrix products of the next pass.
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
template <int KIND, int U, int T, bool WBF>
__global__ __launch_bounds__(T) void optimizer_kernel_v4(f4* __restrict__ w, const f4* __restrict__ g, f4* __restrict__ s0,
                                                            f4* __restrict__ s1, f4* __restrict__ s2, int64_t n4,
                                                            OptScalars p, bf16x4_t* __restrict__ wbf, const int* __restrict__ skip_if) {
  constexpr int NS = n_states<KIND>();
  if (skip_if && *skip_if) return;  // the gradient pass in front of this update failed: nothing moves
  const int64_t base = (int64_t)blockIdx.x * (T * U) + threadIdx.x;
  if (U == 1 && base >= n4) return;  // one vector per thread: one early exit instead of a check around every access
#define SN_IN_RANGE(u) (U == 1 || base + (u) * T < n4)
  f4 vw[U], vg[U], a[U], b[U], c[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (SN_IN_RANGE(u)) vw[u] = __builtin_nontemporal_load(w + base + u * T);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (SN_IN_RANGE(u)) vg[u] = __builtin_nontemporal_load(g + base + u * T);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (SN_IN_RANGE(u)) a[u] = __builtin_nontemporal_load(s0 + base + u * T);
  if (NS > 1) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) b[u] = __builtin_nontemporal_load(s1 + base + u * T);
  }
  if (NS > 2) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) c[u] = __builtin_nontemporal_load(s2 + base + u * T);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float ww = vw[u][e], aa = a[u][e], bb = NS > 1 ? b[u][e] : 0.f, cc = NS > 2 ? c[u][e] : 0.f;
      update_one<KIND>(ww, vg[u][e], aa, bb, cc, p);
      vw[u][e] = ww;
      a[u][e] = aa;
      if (NS > 1) b[u][e] = bb;
      if (NS > 2) c[u][e] = cc;
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (SN_IN_RANGE(u)) __builtin_nontemporal_store(vw[u], w + base + u * T);
  if (WBF) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) {
        bf16x4_t h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = (__bf16)vw[u][e];
        wbf[base + u * T] = h;
      }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (SN_IN_RANGE(u)) __builtin_nontemporal_store(a[u], s0 + base + u * T);
  if (NS > 1) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) __builtin_nontemporal_store(b[u], s1 + base + u * T);
  }
  if (NS > 2) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) __builtin_nontemporal_store(c[u], s2 + base + u * T);
  }
}
#undef SN_IN_RANGE

// Scalar form for a misaligned buffer or the last n % 4 elements.
template <int KIND>
__global__ __launch_bounds__(256) void optimizer_kernel_scalar(float* __restrict__ w, const float* __restrict__ g,
                                                                float* __restrict__ s0, float* __restrict__ s1,
                                                                float* __restrict__ s2, int64_t n, OptScalars p,
                                                                __bf16* __restrict__ wbf, const int* __restrict__ skip_if) {
  constexpr int NS = n_states<KIND>();
  if (skip_if && *skip_if) return;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float ww = w[i], aa = s0[i], bb = NS > 1 ? s1[i] : 0.f, cc = NS > 2 ? s2[i] : 0.f;
    update_one<KIND>(ww, g[i], aa, bb, cc, p);
    w[i] = ww;
    if (wbf) wbf[i] = (__bf16)ww;
    s0[i] = aa;
    if (NS > 1) s1[i] = bb;
    if (NS > 2) s2[i] = cc;
  }
}

static bool aligned16(const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int KIND>
static int launch_opt_t(sn_ctx* ctx, const char* name, float* w, const float* g, float* s0, float* s1, float* s2, int64_t n,
                        const OptScalars& p, void* wbf, const int* skip_if) {
  // One vector per thread; threads per block measured per number of state tensors on 100 M elements (MI355X): 128 for one or
  // two states (SGD 308 us against 319 with 4 vectors x 256 threads, Adam 446 against 467), 64 for three (AMSGrad 596
  // against 614).  Many small blocks keep more independent request streams in flight than few large ones.
  constexpr int UNROLL = 1, THREADS = n_states<KIND>() <= 2 ? 128 : 64;
  const bool vec = aligned16(w) && aligned16(g) && aligned16(s0) && aligned16(s1) && aligned16(s2) && (reinterpret_cast<uintptr_t>(wbf) & 7u) == 0;
  const int64_t n4 = vec ? n / 4 : 0;
  if (n4 > 0) {
    const int64_t blocks = ceil_div(n4, (int64_t)THREADS * UNROLL);  // one pass, no grid-stride loop
    SN_REQUIRE(blocks <= 0x7fffffff, "optimizer update over %lld elements exceeds one launch", (long long)n);
    LaunchScope scope(ctx, name);
    if (wbf)
      hipLaunchKernelGGL((optimizer_kernel_v4<KIND, UNROLL, THREADS, true>), dim3((unsigned)blocks), dim3(THREADS), 0, ctx->stream, (f4*)w,
                         (const f4*)g, (f4*)s0, (f4*)s1, (f4*)s2, n4, p, (bf16x4_t*)wbf, skip_if);
    else
      hipLaunchKernelGGL((optimizer_kernel_v4<KIND, UNROLL, THREADS, false>), dim3((unsigned)blocks), dim3(THREADS), 0, ctx->stream, (f4*)w,
                         (const f4*)g, (f4*)s0, (f4*)s1, (f4*)s2, n4, p, (bf16x4_t*)nullptr, skip_if);
  }
  const int64_t done = n4 * 4;
  if (done < n) {
    const int64_t rest = n - done;
    int64_t blocks = ceil_div(rest, 256);
    const int64_t cap = (int64_t)ctx->compute_units * 8;
    if (blocks > cap) blocks = cap;
    LaunchScope scope(ctx, name);
    hipLaunchKernelGGL((optimizer_kernel_scalar<KIND>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, w + done, g + done,
                       s0 + done, s1 ? s1 + done : nullptr, s2 ? s2 + done : nullptr, rest, p, wbf ? (__bf16*)wbf + done : nullptr, skip_if);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_optimizer(sn_ctx* ctx, const sn_optimizer_desc& d, float* w, const float* g, float* s0, float* s1, float* s2,
                     int64_t n, int iter, void* wbf, const int* skip_if) {
  const int ns = opt_state_count(d.kind);
  SN_REQUIRE(ns > 0, "unknown optimizer kind %d", d.kind);
  SN_REQUIRE(w && g && s0 && (ns < 2 || s1) && (ns < 3 || s2), "optimizer kind %d needs %d state buffers", d.kind, ns);
  SN_REQUIRE(iter >= 1, "iteration numbers start at 1, got %d", iter);
  if (n <= 0) return SN_OK;
  const OptScalars p = make_opt_scalars(d, iter);
  switch (d.kind) {
    case SN_OPT_SGD: return launch_opt_t<SN_OPT_SGD>(ctx, "optimizer_sgd", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_ADAGRAD: return launch_opt_t<SN_OPT_ADAGRAD>(ctx, "optimizer_adagrad", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_ADADELTA: return launch_opt_t<SN_OPT_ADADELTA>(ctx, "optimizer_adadelta", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_RMSPROP: return launch_opt_t<SN_OPT_RMSPROP>(ctx, "optimizer_rmsprop", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_ADAM: return launch_opt_t<SN_OPT_ADAM>(ctx, "optimizer_adam", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_NADAM: return launch_opt_t<SN_OPT_NADAM>(ctx, "optimizer_nadam", w, g, s0, s1, s2, n, p, wbf, skip_if);
    case SN_OPT_ADAMAX: return launch_opt_t<SN_OPT_ADAMAX>(ctx, "optimizer_adamax", w, g, s0, s1, s2, n, p, wbf, skip_if);
    default: return launch_opt_t<SN_OPT_AMSGRAD>(ctx, "optimizer_amsgrad", w, g, s0, s1, s2, n, p, wbf, skip_if);
  }
}

// ---- the launch that finishes a training step ------------------------------------------------
// Sections of one grid: first the plain update of every float4 of the flat buffers that no deferred reduction owns
// (128 threads, one vector each, as optimizer_kernel_v4), then per deferred reduction the blocks that add its partial
// sums, in the order of the stand-alone reduction kernels, store the sums to the gradient buffer and update the
// parameters they belong to right away.
struct FinishPlan {
  DeferredReduce r[MAX_DEFERRED];
  int64_t first[MAX_DEFERRED];  // index in the flat buffers of r[i].dst[0]
  int block0[MAX_DEFERRED + 1]; // first block of reduction i; block0[0] = number of plain blocks
  int n;
  // ranges of the flat buffers the optimizer must leave alone (tensors that are not trainable: a BatchNorm's moving
  // statistics); tensors start on 256-byte boundaries, so no float4 straddles an end
  int64_t hole_first[MAX_FINISH_HOLES], hole_end[MAX_FINISH_HOLES];
  int n_holes;
};

template <int KIND>
__global__ __launch_bounds__(256) void finish_kernel(float* __restrict__ w, float* __restrict__ g, float* __restrict__ s0, float* __restrict__ s1,
                                                      float* __restrict__ s2, int64_t n, OptScalars p, FinishPlan plan,
                                                      const int* __restrict__ skip_if) {
  constexpr int NS = n_states<KIND>();
  __shared__ f4 part4[8][32];
  __shared__ float part1[64][4];
  const bool skip = skip_if && *skip_if;  // a failed pass: gradients are still summed, nothing is updated
  const int b = blockIdx.x;
  if (b < plan.block0[0]) {
    if (skip || threadIdx.x >= 128) return;
    const int64_t i4 = (int64_t)b * 128 + threadIdx.x, e = i4 * 4;
    if (e >= n) return;
    for (int k = 0; k < plan.n; ++k)
      if (e >= plan.first[k] && e < plan.first[k] + plan.r[k].outs) return;  // a reduction block updates these
    for (int k = 0; k < plan.n_holes; ++k)
      if (e >= plan.hole_first[k] && e < plan.hole_end[k]) return;           // not trainable
    if (e + 4 <= n) {
      f4 vw = *(const f4*)(w + e), vg = *(const f4*)(g + e), a = *(const f4*)(s0 + e), bb = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
      if (NS > 1) bb = *(const f4*)(s1 + e);
      if (NS > 2) c = *(const f4*)(s2 + e);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float ww = vw[q], aa = a[q], b2 = bb[q], cc = c[q];
        update_one<KIND>(ww, vg[q], aa, b2, cc, p);
        vw[q] = ww; a[q] = aa; bb[q] = b2; c[q] = cc;
      }
      *(f4*)(w + e) = vw;
      *(f4*)(s0 + e) = a;
      if (NS > 1) *(f4*)(s1 + e) = bb;
      if (NS > 2) *(f4*)(s2 + e) = c;
    } else {
      for (int64_t q = e; q < n; ++q) {
        float ww = w[q], aa = s0[q], b2 = NS > 1 ? s1[q] : 0.f, cc = NS > 2 ? s2[q] : 0.f;
        update_one<KIND>(ww, g[q], aa, b2, cc, p);
        w[q] = ww; s0[q] = aa;
        if (NS > 1) s1[q] = b2;
        if (NS > 2) s2[q] = cc;
      }
    }
    return;
  }
  int k = 0;
  while (k + 1 < plan.n && b >= plan.block0[k + 1]) ++k;
  const DeferredReduce& r = plan.r[k];
  const int lb = b - plan.block0[k];
  const int64_t flat0 = plan.first[k];
  if (r.kind == 1) {
    // splitk_reduce4_kernel's order: 8 groups of 32 lanes x 4 consecutive outputs; group q adds partials q, q + 8, ...
    const int64_t total4 = r.outs / 4;
    const int q = threadIdx.x >> 5, j = threadIdx.x & 31;
    const int64_t i = (int64_t)lb * 32 + j;
    const int64_t e = flat0 + i * 4;
    // the parameters and their optimizer state are requested first: they are back by the time the sums are made
    f4 vw = {0.f, 0.f, 0.f, 0.f}, a = {0.f, 0.f, 0.f, 0.f}, bb = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
    if (q == 0 && i < total4 && !skip) {
      vw = *(const f4*)(w + e);
      a = *(const f4*)(s0 + e);
      if (NS > 1) bb = *(const f4*)(s1 + e);
      if (NS > 2) c = *(const f4*)(s2 + e);
    }
    f4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < total4) {
      const f4* w4 = reinterpret_cast<const f4*>(r.partial) + i;
      int z = q;
      for (; z + 56 < r.parts; z += 64) {  // 8 loads of 16 bytes in flight, added in split order
        f4 pv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) pv[u] = w4[(int64_t)(z + 8 * u) * total4];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += pv[u];
      }
      for (; z < r.parts; z += 8) s += w4[(int64_t)z * total4];
    }
    part4[q][j] = s;
    __syncthreads();
    if (q == 0 && i < total4) {
      const f4 t = ((part4[0][j] + part4[1][j]) + (part4[2][j] + part4[3][j])) + ((part4[4][j] + part4[5][j]) + (part4[6][j] + part4[7][j]));
      *(f4*)(g + e) = t;
      if (!skip) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          float ww = vw[x], aa = a[x], b2 = bb[x], cc = c[x];
          update_one<KIND>(ww, t[x], aa, b2, cc, p);
          vw[x] = ww; a[x] = aa; bb[x] = b2; c[x] = cc;
        }
        *(f4*)(w + e) = vw;
        *(f4*)(s0 + e) = a;
        if (NS > 1) *(f4*)(s1 + e) = bb;
        if (NS > 2) *(f4*)(s2 + e) = c;
      }
    }
  } else {
    // gemm_small_reduce_kernel's order: a block owns 4 outputs, 64 lanes each walk every 64th partial
    const int ol = threadIdx.x & 3, pl = threadIdx.x >> 2;
    const int o = lb * 4 + ol;
    const int64_t e = flat0 + o;
    // the parameter and its optimizer state are requested first: they are back by the time the sum is made
    const bool updates = threadIdx.x < 4 && o < r.outs;
    float ww = 0.f, aa = 0.f, b2 = 0.f, cc = 0.f;
    if (updates && !skip) {
      ww = w[e]; aa = s0[e];
      if (NS > 1) b2 = s1[e];
      if (NS > 2) cc = s2[e];
    }
    float s = 0.f;
    if (o < r.outs) {
      for (int i = pl; i < r.parts; i += 64 * 16) {  // 16 loads in flight, added in part order
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = i + 64 * u < r.parts ? r.partial[(int64_t)(i + 64 * u) * r.outs + o] : 0.f;
#pragma unroll
        for (int u = 0; u < 16; ++u) s += v[u];
      }
    }
    part1[pl][ol] = s;
    __syncthreads();
    if (updates) {
      float t = 0.f;
#pragma unroll 8
      for (int j = 0; j < 64; ++j) t += part1[j][ol];
      g[e] = t;
      if (!skip) {
        update_one<KIND>(ww, t, aa, b2, cc, p);
        w[e] = ww; s0[e] = aa;
        if (NS > 1) s1[e] = b2;
        if (NS > 2) s2[e] = cc;
      }
    }
  }
}

template <int KIND>
static int launch_finish_t(sn_ctx* ctx, float* w, float* g, float* s0, float* s1, float* s2, int64_t n, const OptScalars& p, const FinishPlan& plan,
                           int blocks, const int* skip_if) {
  LaunchScope scope(ctx, "gradient_sums_and_optimizer");
  hipLaunchKernelGGL((finish_kernel<KIND>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, w, g, s0, s1, s2, n, p, plan, skip_if);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_finish(sn_ctx* ctx, const sn_optimizer_desc& d, float* w, float* g, float* s0, float* s1, float* s2, int64_t n, int iter,
                  const DeferredReduce* defs, int n_defs, const int* skip_if, const int64_t* holes, int n_holes) {
  const int ns = opt_state_count(d.kind);
  SN_REQUIRE(ns > 0, "unknown optimizer kind %d", d.kind);
  SN_REQUIRE(w && g && s0 && (ns < 2 || s1) && (ns < 3 || s2), "optimizer kind %d needs %d state buffers", d.kind, ns);
  SN_REQUIRE(iter >= 1, "iteration numbers start at 1, got %d", iter);
  SN_REQUIRE(n_defs >= 1 && n_defs <= MAX_DEFERRED, "launch_finish takes 1..%d deferred reductions, got %d", MAX_DEFERRED, n_defs);
  SN_REQUIRE(aligned16(w) && aligned16(g) && aligned16(s0) && aligned16(s1) && aligned16(s2), "launch_finish: buffers must be 16-byte aligned");
  SN_REQUIRE(n_holes >= 0 && n_holes <= MAX_FINISH_HOLES && (n_holes == 0 || holes), "launch_finish takes up to %d untouched ranges, got %d", MAX_FINISH_HOLES, n_holes);
  FinishPlan plan;
  plan.n = n_defs;
  plan.n_holes = n_holes;
  for (int i = 0; i < n_holes; ++i) {
    SN_REQUIRE(holes[2 * i] % 4 == 0 && holes[2 * i + 1] % 4 == 0 && holes[2 * i] <= holes[2 * i + 1] && holes[2 * i + 1] <= n,
               "launch_finish: untouched range %d is not made of whole float4s of the buffer", i);
    plan.hole_first[i] = holes[2 * i];
    plan.hole_end[i] = holes[2 * i + 1];
  }
  int64_t blocks = ceil_div(ceil_div(n, 4), 128);
  plan.block0[0] = (int)blocks;
  for (int i = 0; i < n_defs; ++i) {
    const DeferredReduce& r = defs[i];
    SN_REQUIRE((r.kind == 1 || r.kind == 2) && r.partial && r.dst && r.parts >= 1 && r.outs >= 4 && r.outs % 4 == 0, "launch_finish: malformed reduction %d", i);
    SN_REQUIRE(r.dst >= g && r.dst + r.outs <= g + n && (r.dst - g) % 4 == 0, "launch_finish: reduction %d does not write into the gradient buffer", i);
    plan.r[i] = r;
    plan.first[i] = r.dst - g;
    blocks += r.kind == 1 ? ceil_div(r.outs / 4, 32) : ceil_div(r.outs, 4);
    plan.block0[i + 1] = (int)blocks;
  }
  SN_REQUIRE(blocks <= 0x7fffffff, "launch_finish: %lld elements exceed one launch", (long long)n);
  const OptScalars p = make_opt_scalars(d, iter);
  switch (d.kind) {
    case SN_OPT_SGD: return launch_finish_t<SN_OPT_SGD>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_ADAGRAD: return launch_finish_t<SN_OPT_ADAGRAD>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_ADADELTA: return launch_finish_t<SN_OPT_ADADELTA>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_RMSPROP: return launch_finish_t<SN_OPT_RMSPROP>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_ADAM: return launch_finish_t<SN_OPT_ADAM>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_NADAM: return launch_finish_t<SN_OPT_NADAM>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    case SN_OPT_ADAMAX: return launch_finish_t<SN_OPT_ADAMAX>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
    default: return launch_finish_t<SN_OPT_AMSGRAD>(ctx, w, g, s0, s1, s2, n, p, plan, (int)blocks, skip_if);
  }
}

// the sums alone, when no optimizer launch follows
__global__ __launch_bounds__(256) void deferred_reduce_kernel(DeferredReduce r) {
  __shared__ f4 part4[8][32];
  __shared__ float part1[64][4];
  if (r.kind == 1) {
    const int64_t total4 = r.outs / 4;
    const int q = threadIdx.x >> 5, j = threadIdx.x & 31;
    const int64_t i = (int64_t)blockIdx.x * 32 + j;
    f4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < total4) {
      const f4* w4 = reinterpret_cast<const f4*>(r.partial) + i;
      int z = q;
      for (; z + 56 < r.parts; z += 64) {
        f4 a[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = w4[(int64_t)(z + 8 * u) * total4];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += a[u];
      }
      for (; z < r.parts; z += 8) s += w4[(int64_t)z * total4];
    }
    part4[q][j] = s;
    __syncthreads();
    if (q == 0 && i < total4)
      reinterpret_cast<f4*>(r.dst)[i] = ((part4[0][j] + part4[1][j]) + (part4[2][j] + part4[3][j])) + ((part4[4][j] + part4[5][j]) + (part4[6][j] + part4[7][j]));
  } else {
    const int ol = threadIdx.x & 3, pl = threadIdx.x >> 2;
    const int o = blockIdx.x * 4 + ol;
    float s = 0.f;
    if (o < r.outs) {
      for (int i = pl; i < r.parts; i += 64 * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = i + 64 * u < r.parts ? r.partial[(int64_t)(i + 64 * u) * r.outs + o] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
      }
    }
    part1[pl][ol] = s;
    __syncthreads();
    if (threadIdx.x < 4 && o < r.outs) {
      float t = 0.f;
#pragma unroll 8
      for (int j = 0; j < 64; ++j) t += part1[j][ol];
      r.dst[o] = t;
    }
  }
}

int launch_deferred_reduce(sn_ctx* ctx, const DeferredReduce& d) {
  SN_REQUIRE((d.kind == 1 || d.kind == 2) && d.partial && d.dst && d.outs % 4 == 0, "malformed deferred reduction");
  LaunchScope scope(ctx, d.kind == 1 ? "splitk_reduce" : "small_output_reduce");
  const int64_t blocks = d.kind == 1 ? ceil_div(d.outs / 4, 32) : ceil_div(d.outs, 4);
  hipLaunchKernelGGL(deferred_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, d);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ---- K-replica average --------------------------------------------------------------------
struct AvgOutputs {
  float* p[SN_MAX_AVG_INPUTS + 1];
};

// Block-contiguous like the optimizer kernel: a block owns AVG_T*U float4, reads them input by input.  Measured on 8 x 25 M
// (MI355X): 128 threads x 1 vector 6.18 TB/s, 64 x 1 6.20, 256 x 2 5.98, 256 x 1 5.54, 512 x 1 5.91; a plain copy
// kernel of the same shape reaches 6.15 TB/s on the same box.
constexpr int AVG_T = 128;
template <int K_STATIC, int U>
__global__ __launch_bounds__(AVG_T) void average_kernel_v4(AvgInputs in, int k, int64_t n4, AvgOutputs out, int n_out, float kf) {
  constexpr int T = AVG_T;
  const int64_t base = (int64_t)blockIdx.x * (T * U) + threadIdx.x;
  // with one vector per thread the bounds check is one early exit; a check around every load made the compiler wait for
  // each load before it issued the next
  if (U == 1 && base >= n4) return;
#define SN_IN_RANGE(u) (U == 1 || base + (u) * T < n4)
  f4 acc[U];
  if constexpr (K_STATIC > 0) {
    f4 v[K_STATIC][U];
#pragma unroll
    for (int r = 0; r < K_STATIC; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (SN_IN_RANGE(u)) v[r][u] = __builtin_nontemporal_load((const f4*)in.p[r] + base + u * T);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc[u] = v[0][u];
#pragma unroll
      for (int r = 1; r < K_STATIC; ++r) acc[u] = acc[u] + v[r][u];  // AddN, left to right
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) acc[u] = __builtin_nontemporal_load((const f4*)in.p[0] + base + u * T);
    for (int r = 1; r < k; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (SN_IN_RANGE(u)) acc[u] = acc[u] + __builtin_nontemporal_load((const f4*)in.p[r] + base + u * T);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) acc[u] = acc[u] / kf;  // `plus(inputs) / inputs.size` (models/Aggregation.scala:16-19)
  for (int o = 0; o < n_out; ++o)
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (SN_IN_RANGE(u)) __builtin_nontemporal_store(acc[u], (f4*)out.p[o] + base + u * T);
}
#undef SN_IN_RANGE

__global__ __launch_bounds__(256) void average_kernel_scalar(AvgInputs in, int k, int64_t first, int64_t n, AvgOutputs out,
                                                              int n_out, float kf) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float acc = in.p[0][i];
    for (int r = 1; r < k; ++r) acc = acc + in.p[r][i];
    acc = acc / kf;
    for (int o = 0; o < n_out; ++o) out.p[o][i] = acc;
  }
}

int launch_average(sn_ctx* ctx, const AvgInputs& in, int k, int64_t n, float* out, float* const* extra_out, int n_extra) {
  SN_REQUIRE(k >= 1 && k <= SN_MAX_AVG_INPUTS, "average takes 1..%d inputs, got %d", SN_MAX_AVG_INPUTS, k);
  SN_REQUIRE(n_extra >= 0 && n_extra <= SN_MAX_AVG_INPUTS, "too many average outputs");
  if (n <= 0) return SN_OK;
  AvgOutputs o;
  o.p[0] = out;
  for (int i = 0; i < n_extra; ++i) o.p[i + 1] = extra_out[i];
  const int n_out = 1 + n_extra;
  bool vec = aligned16(out);
  for (int i = 0; i < k; ++i) vec = vec && aligned16(in.p[i]);
  for (int i = 0; i < n_extra; ++i) vec = vec && aligned16(extra_out[i]);
  const int64_t n4 = vec ? n / 4 : 0;
  const float kf = (float)k;
  if (n4 > 0) {
    constexpr int U = 1;
    const int64_t blocks = ceil_div(n4, AVG_T * U);
    SN_REQUIRE(blocks <= 0x7fffffff, "average over %lld elements exceeds one launch", (long long)n);
    LaunchScope scope(ctx, "average_replicas");
    if (k == 8)
      hipLaunchKernelGGL((average_kernel_v4<8, U>), dim3((unsigned)blocks), dim3(AVG_T), 0, ctx->stream, in, k, n4, o, n_out, kf);
    else if (k == 4)
      hipLaunchKernelGGL((average_kernel_v4<4, U>), dim3((unsigned)blocks), dim3(AVG_T), 0, ctx->stream, in, k, n4, o, n_out, kf);
    else if (k == 2)
      hipLaunchKernelGGL((average_kernel_v4<2, U>), dim3((unsigned)blocks), dim3(AVG_T), 0, ctx->stream, in, k, n4, o, n_out, kf);
    else
      hipLaunchKernelGGL((average_kernel_v4<0, U>), dim3((unsigned)blocks), dim3(AVG_T), 0, ctx->stream, in, k, n4, o, n_out, kf);
  }
  if (n4 * 4 < n) {
    LaunchScope scope(ctx, "average_replicas");
    int64_t blocks = ceil_div(n - n4 * 4, 256);
    const int64_t cap = (int64_t)ctx->compute_units * 8;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(average_kernel_scalar, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, in, k, n4 * 4, n, o, n_out, kf);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

__global__ __launch_bounds__(256) void fill_kernel(float* dst, float v, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = v;
}

int launch_fill(sn_ctx* ctx, float* dst, float v, int64_t n) {
  if (n <= 0) return SN_OK;
  int64_t blocks = ceil_div(n, 256 * 4);
  const int64_t cap = (int64_t)ctx->compute_units * 8;
  if (blocks > cap) blocks = cap;
  LaunchScope scope(ctx, "fill");
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, dst, v, n);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
