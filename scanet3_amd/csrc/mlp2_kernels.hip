// Training pass of a small two-layer perceptron in two launches (gfx950):
//
//   Dense(H, act) >> Dense(C, Softmax) under CategoricalCrossentropy, H <= 64 hidden units, C <= 16 classes
//   (layer/Dense.scala:30-71, Activation.scala:46-83, Loss.scala:44-57; the reference's first benchmark configuration
//   784 -> 50 -> 10 at batch 1000).
//
// As a chain of general kernels this step is a dozen dependent launches of 3-9 us each.  Here
//   kernel 1 (one workgroup per 16 batch rows): z1 = x W1 on the matrix cores (v_mfma_f32_16x16x4_f32; the x tile in
//     LDS, each wavefront's 16 columns of W1 straight from memory into registers, 16 k-blocks ahead), h = act(z1 + b1),
//     z2 = h W2 + b2, softmax, the loss terms, dz2, dh = dz2 W2^T, dz1 = act'(h) dh, and this row block's terms of dW2,
//     db1 and db2; dz1 leaves in the order kernel 2's matrix-core fragments want it;
//   kernel 2 (one workgroup per 16 input features + one): dW1 = x^T dz1 on the matrix cores (the 16-feature slab of x
//     in LDS, dz1 fragments as 16-byte loads), and the sums of the row blocks' partial dW2 / db1 / db2 in block order.
// Every sum has a fixed order, so results do not depend on the launch.
#include "common.hpp"
#include "optim_update.hpp"

namespace sn {
namespace {

typedef float f4v __attribute__((ext_vector_type(4)));
constexpr int MR = 16;            // batch rows per workgroup of kernel 1 = one k-block of kernel 2
constexpr int MH = 64;            // hidden units, padded
constexpr int MC = 16;            // classes, padded
constexpr int CHUNK = 16;         // k-blocks of 16 whose B fragments are requested together (64 registers)
constexpr int XPITCH = 20;        // floats per row of kernel 2's x slab: the four row groups of a fragment read fall on different banks

struct Mlp2Args {
  const float* x;    // [rows, K]
  const float* y;    // [rows, C]
  const float* w1;   // [K, H]
  const float* b1;   // [H] or null
  const float* w2;   // [H, C]
  const float* b2;   // [C] or null
  float* h;          // [rows, H]
  float* z2;         // [rows, C]
  float* p;          // [rows, C]
  float* dz1f;       // [row blocks][4 column blocks][64 lanes][4]: dz1[16 kb + 4 (lane / 16) + j][16 cb + lane % 16]
  float* row_loss;   // [rows]
  float* part;       // [row blocks][H * C + H + C]: partial dW2, db1, db2
  float* g_w1; float* g_b1; float* g_w2; float* g_b2;   // gradients (b may be null)
  int rows, K, H, C, act1, stable;
  float act1_param, neg_inv_rows;
  Mlp2Update upd;    // kind >= 0: kernel 2 applies every gradient value it finishes to its parameter
};

// the optimizer update of the parameter whose gradient g_at[0] has just been stored
__device__ __forceinline__ void apply_update(const Mlp2Update& u, const float* g_at, float grad) {
  const int64_t off = g_at - u.g;
  float w = u.w[off], s0 = u.s0[off], s1 = u.n_states > 1 ? u.s1[off] : 0.f, s2 = u.n_states > 2 ? u.s2[off] : 0.f;
  update_any(u.kind, w, grad, s0, s1, s2, u.p);
  u.w[off] = w;
  u.s0[off] = s0;
  if (u.n_states > 1) u.s1[off] = s1;
  if (u.n_states > 2) u.s2[off] = s2;
}

__device__ __forceinline__ float act_fwd1(int act, float v, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));   // TF Sigmoid
    case SN_ACT_TANH: return tanhf(v);
    case SN_ACT_RELU: return fmaxf(param, v);               // Maximum(threshold, x), Activation.scala:79-82
    default: return v;
  }
}
__device__ __forceinline__ float act_bwd1(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

__global__ __launch_bounds__(256) void mlp2_rows_kernel(Mlp2Args a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int K16 = (a.K + 15) & ~15, KP = K16 + 4, kq = K16 / 4, nkb = K16 / 16;
  float* Xs = lds;                        // [MR][KP]
  float* Hs = lds + MR * KP;              // [MR][MH + 1]   h
  float* Ds = Hs + MR * (MH + 1);         // [MR][MH + 1]   dz1
  float* Z2 = Ds + MR * (MH + 1);         // [MR][MC + 1]   z2, then dz2
  float* W2s = Z2 + MR * (MC + 1);        // [H][C]         the second layer's weights (read H or C times per output below)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int blk = blockIdx.x, r0 = blk * MR;

  // ---- the x tile, every load in flight before the first LDS write: 16 threads per row, quads tid % 16 + 16 i
  {
    constexpr int NL = 16;  // 16 * 16 quads per row cover K up to 1024 in one pass
    const int row = tid >> 4, q0 = tid & 15;
    const bool row_on = r0 + row < a.rows;
    const float* xr = a.x + (int64_t)(row_on ? r0 + row : 0) * a.K;
    f4v v[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int q = q0 + 16 * i;
      v[i] = *(const f4v*)(xr + 4 * min(q, a.K / 4 - 1));   // clamped address; what lies outside the tile is zeroed below
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int q = q0 + 16 * i;
      if (q < kq) *(f4v*)(Xs + row * KP + 4 * q) = (row_on && 4 * q < a.K) ? v[i] : f4v{0.f, 0.f, 0.f, 0.f};
    }
  }
  for (int e = tid; e < a.H * a.C; e += 256) W2s[e] = a.w2[e];
  // ---- z1 = x W1: wavefront w owns hidden units 16 w .. 16 w + 15; lane (n = l % 16, g = l / 16) feeds
  // k = 16 kb + 4 g + j into the j-th MFMA of block kb
  const int n16 = lane & 15, g = lane >> 4, col = wave * 16 + n16;
  const bool col_on = col < a.H;
  const float* wcol = a.w1 + min(col, a.H - 1);
  auto load_chunk = [&](int c, float (&b)[CHUNK][4]) {
#pragma unroll
    for (int i = 0; i < CHUNK; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // Unconditional loads from clamped addresses, no select: past K the x tile holds zeros, so whatever B value meets
        // them adds nothing, and columns past H are never stored.  (A condition on the loaded value makes the compiler
        // move each load into its own branch and wait for it there: 196 loads one after the other.)
        const int k = 16 * (c * CHUNK + i) + 4 * g + j;
        b[i][j] = wcol[(int64_t)min(k, a.K - 1) * a.H];
      }
  };
  f4v acc = {0.f, 0.f, 0.f, 0.f};
  float bcur[CHUNK][4], bnext[CHUNK][4];
  const int nchunks = (nkb + CHUNK - 1) / CHUNK;
  load_chunk(0, bcur);
  __syncthreads();  // the x tile is in LDS
  const float* ap = Xs + n16 * KP + 4 * g;
  for (int c = 0; c < nchunks; ++c) {
    if (c + 1 < nchunks) load_chunk(c + 1, bnext);
    if ((c + 1) * CHUNK <= nkb) {  // a full chunk: straight-line code, so that the LDS reads run ahead of the MFMAs
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        const f4v av = *(const f4v*)(ap + 16 * (c * CHUNK + i));
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bcur[i][j], acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        const int kb = c * CHUNK + i;
        if (kb < nkb) {
          const f4v av = *(const f4v*)(ap + 16 * kb);
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bcur[i][j], acc, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < CHUNK; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) bcur[i][j] = bnext[i][j];
  }
  // ---- h = act(z1 + b1): accumulator element v of lane (n, g) is row 4 g + v, column 16 w + n
  {
    const float bias = (a.b1 && col_on) ? a.b1[col] : 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = 4 * g + v;
      float hv = 0.f;
      if (col_on && r0 + row < a.rows) {
        hv = act_fwd1(a.act1, a.b1 ? acc[v] + bias : acc[v], a.act1_param);
        a.h[(int64_t)(r0 + row) * a.H + col] = hv;
      }
      Hs[row * (MH + 1) + col] = hv;
    }
  }
  __syncthreads();
  // ---- z2 = h W2 + b2 (Dense.scala:57-61, Bias.scala:32-33): one thread per (row, class)
  for (int e = tid; e < MR * a.C; e += 256) {
    const int row = e / a.C, c = e - row * a.C;
    float s = 0.f;
#pragma unroll 8
    for (int j = 0; j < a.H; ++j) s += Hs[row * (MH + 1) + j] * W2s[j * a.C + c];
    if (a.b2) s = s + a.b2[c];
    Z2[row * (MC + 1) + c] = s;
    if (r0 + row < a.rows) a.z2[(int64_t)(r0 + row) * a.C + c] = s;
  }
  __syncthreads();
  // ---- softmax, loss term and d loss / d z2 per row (Activation.scala:63-69, Loss.scala:44-57, general form with epsilon):
  // 16 lanes per row, one class each; the row sums are butterflies over the 16 lanes (a fixed order)
  {
    const int row = tid >> 4, c = tid & 15;
    const bool on = c < a.C && r0 + row < a.rows;
    const float eps = 1e-8f;
    auto sum16 = [](float v) {
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, 16);
      return v;
    };
    const float z = on ? Z2[row * (MC + 1) + c] : 0.f;
    const float yi = on ? a.y[(int64_t)(r0 + row) * a.C + c] : 0.f;
    float mx = 0.f;
    if (a.stable) {
      mx = on ? z : -INFINITY;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 16));
    }
    const float e = on ? expf(z - mx) : 0.f;
    const float total = sum16(e);
    const float pi = on ? e / total : 0.f;
    const float dpi = on ? (yi * a.neg_inv_rows) / (pi + eps) : 0.f;
    const float term = sum16(on ? yi * logf(pi + eps) : 0.f);
    const float dot = sum16(pi * dpi);
    if (on) a.p[(int64_t)(r0 + row) * a.C + c] = pi;
    if (c < a.C) Z2[row * (MC + 1) + c] = on ? pi * dpi - pi * dot : 0.f;   // dz2 (zeros for rows past the batch)
    if (c == 0 && r0 + row < a.rows) a.row_loss[r0 + row] = term;
  }
  __syncthreads();
  // ---- dh = dz2 W2^T, dz1 = act'(h) dh; dz1 leaves in fragment order (zeros outside the matrix)
  for (int e = tid; e < MR * MH; e += 256) {
    const int row = e / MH, j = e - row * MH;
    float d = 0.f;
    if (j < a.H && r0 + row < a.rows) {
      float s = 0.f;
#pragma unroll 4
      for (int c = 0; c < a.C; ++c) s += Z2[row * (MC + 1) + c] * W2s[j * a.C + c];
      d = act_bwd1(a.act1, Hs[row * (MH + 1) + j], s, a.act1_param);
    }
    Ds[row * (MH + 1) + j] = d;
    a.dz1f[(((int64_t)blk * 4 + (j >> 4)) * 64 + (row >> 2) * 16 + (j & 15)) * 4 + (row & 3)] = d;
  }
  __syncthreads();
  // ---- this row block's terms of dW2 = h^T dz2, db1 = column sums of dz1, db2 = column sums of dz2
  float* part = a.part + (int64_t)blk * (a.H * a.C + a.H + a.C);
  for (int e = tid; e < a.H * a.C + a.H + a.C; e += 256) {
    float s = 0.f;
    if (e < a.H * a.C) {
      const int j = e / a.C, c = e - j * a.C;
      for (int row = 0; row < MR; ++row) s += Hs[row * (MH + 1) + j] * Z2[row * (MC + 1) + c];
    } else if (e < a.H * a.C + a.H) {
      const int j = e - a.H * a.C;
      for (int row = 0; row < MR; ++row) s += Ds[row * (MH + 1) + j];
    } else {
      const int c = e - a.H * a.C - a.H;
      for (int row = 0; row < MR; ++row) s += Z2[row * (MC + 1) + c];
    }
    part[e] = s;
  }
}

__global__ __launch_bounds__(256) void mlp2_weights_kernel(Mlp2Args a, int nblk, int nslab) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if ((int)blockIdx.x == nslab) {
    // sums of the row blocks' partial dW2 / db1 / db2, in block order, 8 loads in flight
    const int np = a.H * a.C + a.H + a.C;
    for (int e = tid; e < np; e += 256) {
      float s = 0.f;
      int b = 0;
      for (; b + 8 <= nblk; b += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = a.part[(int64_t)(b + u) * np + e];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
      }
      for (; b < nblk; ++b) s += a.part[(int64_t)b * np + e];
      float* at = nullptr;
      if (e < a.H * a.C) at = a.g_w2 + e;
      else if (e < a.H * a.C + a.H) at = a.g_b1 ? a.g_b1 + (e - a.H * a.C) : nullptr;
      else at = a.g_b2 ? a.g_b2 + (e - a.H * a.C - a.H) : nullptr;
      if (at) {
        *at = s;
        if (a.upd.kind >= 0) apply_update(a.upd, at, s);
      }
    }
    return;
  }
  // ---- dW1[f0 .. f0 + 15, :] = x[:, f0 .. f0 + 15]^T dz1
  const int f0 = blockIdx.x * 16, rows16 = nblk * MR;
  float* Xs = lds;  // [rows16][XPITCH]
  for (int base = 0; base < rows16 * 4; base += 256 * 8) {  // 16-byte loads, 8 in flight per thread
    f4v v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = base + u * 256 + tid, row = idx >> 2, q = idx & 3;
      v[u] = *(const f4v*)(a.x + (int64_t)min(row, a.rows - 1) * a.K + min(f0 + 4 * q, a.K - 4));   // zeroed below where outside
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = base + u * 256 + tid, row = idx >> 2, q = idx & 3;
      if (idx < rows16 * 4) *(f4v*)(Xs + row * XPITCH + 4 * q) = (row < a.rows && f0 + 4 * q < a.K) ? v[u] : f4v{0.f, 0.f, 0.f, 0.f};
    }
  }
  const int n16 = lane & 15, g = lane >> 4;
  const f4v* bsrc = (const f4v*)a.dz1f + (int64_t)wave * 64 + lane;  // k-block kb: + kb * 256
  auto load_chunk = [&](int c, f4v (&b)[CHUNK]) {
#pragma unroll
    for (int i = 0; i < CHUNK; ++i) {
      const int kb = c * CHUNK + i;
      b[i] = bsrc[(int64_t)min(kb, nblk - 1) * 256];   // clamped address, no select: k-blocks past the last are not multiplied
    }
  };
  f4v acc = {0.f, 0.f, 0.f, 0.f};
  f4v bcur[CHUNK], bnext[CHUNK];
  const int nchunks = (nblk + CHUNK - 1) / CHUNK;
  load_chunk(0, bcur);
  __syncthreads();
  const float* ap = Xs + (4 * g) * XPITCH + n16;   // feature n16 of rows 16 kb + 4 g + j
  for (int c = 0; c < nchunks; ++c) {
    if (c + 1 < nchunks) load_chunk(c + 1, bnext);
    if ((c + 1) * CHUNK <= nblk) {  // a full chunk: straight-line code, so that the LDS reads run ahead of the MFMAs
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        float av[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) av[j] = ap[(16 * (c * CHUNK + i) + j) * XPITCH];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bcur[i][j], acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < CHUNK; ++i) {
        const int kb = c * CHUNK + i;
        if (kb < nblk) {
          float av[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) av[j] = ap[(16 * kb + j) * XPITCH];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bcur[i][j], acc, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < CHUNK; ++i) bcur[i] = bnext[i];
  }
  // accumulator element v of lane (n, g): feature f0 + 4 g + v, hidden unit 16 wave + n
  const int col = wave * 16 + n16;
  if (col < a.H) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int f = f0 + 4 * g + v;
      if (f < a.K) {
        float* at = a.g_w1 + (int64_t)f * a.H + col;
        *at = acc[v];
        if (a.upd.kind >= 0) apply_update(a.upd, at, acc[v]);
      }
    }
  }
}

__global__ __launch_bounds__(256) void mlp2_loss_kernel(const float* __restrict__ row_loss, int rows, float* __restrict__ loss) {
  __shared__ float sm[4];
  float s = 0.f;
  for (int i = threadIdx.x; i < rows; i += 256) s += row_loss[i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) *loss = (-(((sm[0] + sm[1]) + sm[2]) + sm[3])) / (float)rows;   // -Sum(y log(p + eps)) / B, Loss.scala:44-57
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
size_t rows_lds(int K) { return ((size_t)MR * (((K + 15) & ~15) + 4) + 2 * MR * (MH + 1) + MR * (MC + 1) + MH * MC) * sizeof(float); }
size_t weights_lds(int rows) { return (size_t)ceil_div(rows, MR) * MR * XPITCH * sizeof(float); }

}  // namespace

// Shapes the fused pass takes: K a multiple of 4 up to 1024, H <= 64, C <= 16, up to 1792 rows (the x slab of kernel 2
// must fit LDS), and room in the two scratch buffers.
bool mlp2_fused_ok(int rows_max, int K, int H, int C, int64_t scratch_a_elems, int64_t scratch_b_elems) {
  const int64_t nblk = ceil_div(rows_max, MR);
  return K % 4 == 0 && K >= 4 && K <= 1024 && H >= 1 && H <= MH && C >= 1 && C <= MC && rows_max <= 1792 &&
         scratch_a_elems >= nblk * 4 * 64 * 4 && scratch_b_elems >= nblk * ((int64_t)H * C + H + C);
}

int launch_mlp2_grad(sn_ctx* ctx, const float* x, const float* y, const float* w1, const float* b1, const float* w2, const float* b2, int rows,
                     int K, int H, int C, int act1, float act1_param, bool stable, float* h, float* z2, float* p, float* scratch_a,
                     float* scratch_b, float* row_loss, float* loss_dev, float* g_w1, float* g_b1, float* g_w2, float* g_b2,
                     const Mlp2Update* update) {
  SN_REQUIRE(rows > 0, "loss over an empty batch");
  SN_REQUIRE(aligned16(x) && aligned16(scratch_a), "mlp2: x and the scratch buffers must be 16-byte aligned");
  Mlp2Args a{x, y, w1, b1, w2, b2, h, z2, p, scratch_a, row_loss, scratch_b, g_w1, g_b1, g_w2, g_b2,
             rows, K, H, C, act1, stable ? 1 : 0, act1_param, -(1.0f / (float)rows), update ? *update : Mlp2Update{}};
  const int nblk = (int)ceil_div(rows, MR), nslab = (int)ceil_div(K, 16);
  {
    LaunchScope scope(ctx, "mlp2_rows_forward_backward", rows, H, K);
    SN_TRY(allow_dynamic_lds(ctx, (const void*)mlp2_rows_kernel, rows_lds(1024)));
    hipLaunchKernelGGL(mlp2_rows_kernel, dim3((unsigned)nblk), dim3(256), rows_lds(K), ctx->stream, a);
  }
  {
    LaunchScope scope(ctx, update ? "mlp2_weight_gradients_and_optimizer" : "mlp2_weight_gradients", K, H, rows);
    SN_TRY(allow_dynamic_lds(ctx, (const void*)mlp2_weights_kernel, weights_lds(1792)));
    hipLaunchKernelGGL(mlp2_weights_kernel, dim3((unsigned)(nslab + 1)), dim3(256), weights_lds(rows), ctx->stream, a, nblk, nslab);
  }
  if (loss_dev) {
    LaunchScope scope(ctx, "loss_stage2");
    hipLaunchKernelGGL(mlp2_loss_kernel, dim3(1), dim3(256), 0, ctx->stream, (const float*)row_loss, rows, loss_dev);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
