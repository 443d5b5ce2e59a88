// MFMA GEMM family for gfx950: one LDS-tiled kernel template whose operand tiles are
// gathered by small "loader" functors, so the same matrix-core inner loop serves
//   - Dense forward / dX / dW (strided operands: NN, NT, TN),
//   - Conv2D forward, input gradient and filter gradient as implicit GEMMs over NHWC,
//   - the LSTM step (4-gate GEMM over [x_t, h_{t-1}]), its dh/dx and its weight gradients.
// fp32 path: v_mfma_f32_32x32x2_f32.  bf16 path (Dense, on request): operands are rounded to
// bf16 while they are staged into LDS and multiplied with v_mfma_f32_32x32x16_bf16, fp32 accumulate.
//
// Block = 256 threads = 4 wavefronts in a 2x2 arrangement; block tile BM x BN (64 or 128 each),
// K step 16; each wavefront owns (BM/2) x (BN/2) as 32x32 MFMA tiles.  Small-output problems
// are split along K over gridDim.z; partial tiles go to a workspace and a second kernel adds
// them in split order (deterministic) and applies the epilogue.
#include "common.hpp"

#include <type_traits>

namespace sn {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int BK = 16;
constexpr int THREADS = 256;

// ============================================================================ loaders
// A loader describes one operand as a function (outer index, k) -> value, where the outer
// index is the row m of A or the column n of B.  K_CONTIG tells the tile copy which index
// should run fastest across lanes so that global loads coalesce.
//   Cursor   per-element state
//   init     position a cursor at (outer, k)
//   load     value at the cursor (0 outside the matrix or past k_end)
//   advance  move the cursor dk along k
// The kernel drives a loader through a second, finer interface that separates what is the same for the
// whole workgroup in one k tile (struct Tile: the tile's first k and whatever follows from it, kept in
// scalar registers) from what belongs to the thread (Cursor):
//   init4(c, outer, k_begin, kk)   kk = the thread's fixed k offset inside every tile
//   tile_init / tile_advance        uniform state for the tile starting at k0, then k0 += BK
//   thread_advance                  per-thread part of moving on one tile (nothing for the FAST loaders)
//   load_t / load4_t                value(s) at (cursor, tile)
// Loaders written against the cursor interface only get the second one from SN_CURSOR_ONLY_API; the FAST
// loaders implement it directly with 32-bit offsets, a per-thread validity mask and no branches.
#define SN_CURSOR_ONLY_API                                                                                         \
  static constexpr bool FAST = false;                                                                              \
  struct Tile {};                                                                                                  \
  __device__ __forceinline__ void tile_init(Tile&, int) const {}                                                   \
  __device__ __forceinline__ void tile_advance(Tile&) const {}                                                     \
  __device__ __forceinline__ void thread_advance(Cursor& c) const { advance(c, BK); }                              \
  __device__ __forceinline__ void init4(Cursor& c, int outer, int kb, int kk) const { init(c, outer, kb + kk); }   \
  __device__ __forceinline__ float load_t(const Cursor& c, const Tile&, int k_end) const { return load(c, k_end); } \
  __device__ __forceinline__ bool load4_t(const Cursor& c, const Tile&, int k_end, float (&v)[4]) const { load4(c, k_end, v); return true; }

// 16-byte load without a branch: a lane whose element lies outside the matrix reads the first 16 bytes of
// the tensor instead (always mapped, 16-byte aligned) and discards them.  Offsets are 32-bit: the host only
// picks the FAST loaders for tensors below 2 GiB.
constexpr int64_t FAST_SPAN = (int64_t)1 << 31;
// Returns `valid` and leaves the select to the caller, who applies it when the values go to LDS one K tile later: a select
// right here would make the loads' consumer sit directly behind them, and the wait for the data would land in front of
// the current tile's MFMAs instead of behind them.
__device__ __forceinline__ bool sel_load4(const float* base, uint32_t byte_off, bool valid, float (&v)[4]) {
  const f4v r = *(const f4v*)((const char*)base + (valid ? byte_off : 0u));
  v[0] = r[0];
  v[1] = r[1];
  v[2] = r[2];
  v[3] = r[3];
  return valid;
}
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ONES: the loader knows one extra outer index that reads as all ones (a separate type, so the plain loader's
// cursor and loads stay as lean as they were)
template <bool KC, bool ONES = false>
struct StridedLoader {
  static constexpr bool K_CONTIG = KC;
  const float* p;
  int64_t s_outer, s_k;
  int outer_n;
  int ones_outer = -1;  // this outer index (just past the matrix) reads as all ones; -1: none
  struct Cursor {
    const float* ptr;
    int k;
    bool ones;
  };
  __device__ __forceinline__ void init(Cursor& c, int outer, int k) const {
    c.ptr = outer < outer_n ? p + (int64_t)outer * s_outer : nullptr;
    c.k = k;
    c.ones = ONES && outer == ones_outer;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (ONES && c.ones) return c.k < k_end ? 1.0f : 0.f;
    return (c.ptr && c.k < k_end) ? c.ptr[(int64_t)c.k * s_k] : 0.f;
  }
  // 4 values along the contiguous index (k when KC, the outer index otherwise); vec4_ok() guarantees that the
  // four are inside or outside the matrix together and 16-byte aligned
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.ptr && c.k < k_end) r = *(const f4v*)(c.ptr + (int64_t)c.k * s_k);
    // the ones row starts a group of 4 outer indices (outer_n % 4 == 0) whose other three lie outside the matrix;
    // along k (KC) it is four ones
    if (ONES && c.ones && c.k < k_end) r = KC ? f4v{1.f, 1.f, 1.f, 1.f} : f4v{1.f, 0.f, 0.f, 0.f};
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int K) const {
    const bool aligned = (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
    return KC ? (s_k == 1 && s_outer % 4 == 0 && K % 4 == 0 && aligned) : (s_outer == 1 && s_k % 4 == 0 && outer_n % 4 == 0 && aligned);
  }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const { c.k += dk; }
  SN_CURSOR_ONLY_API
};

// ---- Conv2D forward: A(m,k) = x[b, oh*sh-pt+r, ow*sw-pl+q, ci], m=(b,oh,ow), k=(r,q,ci)
struct ConvFwdA {
  static constexpr bool K_CONTIG = true;
  const float* x;
  ConvGeom g;
  int M;
  struct Cursor {
    const float* img;  // x + b*h*w*cin, null when the row is outside the matrix
    int iy0, ix0, r, q, ci, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int m, int k) const {
    c.k = k;
    if (m >= M) { c.img = nullptr; c.iy0 = c.ix0 = c.r = c.q = c.ci = 0; return; }
    const int ow = m % g.wo;
    const int t = m / g.wo;
    const int oh = t % g.ho;
    const int b = t / g.ho;
    c.img = x + (int64_t)b * g.h * g.w * g.cin;
    c.iy0 = oh * g.sh - g.pt;
    c.ix0 = ow * g.sw - g.pl;
    c.ci = k % g.cin;
    const int rq = k / g.cin;
    c.q = rq % g.kw;
    c.r = rq / g.kw;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (!c.img || c.k >= k_end) return 0.f;
    const int iy = c.iy0 + c.r, ix = c.ix0 + c.q;
    if (iy < 0 || iy >= g.h || ix < 0 || ix >= g.w) return 0.f;
    return c.img[((int64_t)iy * g.w + ix) * g.cin + c.ci];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {  // ci .. ci+3 of one pixel
    f4v r = {0.f, 0.f, 0.f, 0.f};
    const int iy = c.iy0 + c.r, ix = c.ix0 + c.q;
    if (c.img && c.k < k_end && iy >= 0 && iy < g.h && ix >= 0 && ix < g.w) r = *(const f4v*)(c.img + ((int64_t)iy * g.w + ix) * g.cin + c.ci);
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const { return g.cin % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0; }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const {
    c.k += dk;
    c.ci += dk;
    while (c.ci >= g.cin) {
      c.ci -= g.cin;
      if (++c.q == g.kw) { c.q = 0; ++c.r; }
    }
  }
  SN_CURSOR_ONLY_API
};

// ---- Conv2D input gradient: dx[b,iy,ix,ci] = sum_{r,q,co} dy[b,(iy+pt-r)/sh,(ix+pl-q)/sw,co] * w[r,q,ci,co]
struct ConvDgradA {  // m=(b,iy,ix), k=(r,q,co)
  static constexpr bool K_CONTIG = true;
  const float* dy;
  ConvGeom g;
  int M;
  struct Cursor {
    const float* img;  // dy + b*ho*wo*cout
    int ty, tx, r, q, co, k;  // ty = iy + pt, tx = ix + pl
  };
  __device__ __forceinline__ void init(Cursor& c, int m, int k) const {
    c.k = k;
    if (m >= M) { c.img = nullptr; c.ty = c.tx = c.r = c.q = c.co = 0; return; }
    const int ix = m % g.w;
    const int t = m / g.w;
    const int iy = t % g.h;
    const int b = t / g.h;
    c.img = dy + (int64_t)b * g.ho * g.wo * g.cout;
    c.ty = iy + g.pt;
    c.tx = ix + g.pl;
    c.co = k % g.cout;
    const int rq = k / g.cout;
    c.q = rq % g.kw;
    c.r = rq / g.kw;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (!c.img || c.k >= k_end) return 0.f;
    const int ny = c.ty - c.r, nx = c.tx - c.q;
    if (ny < 0 || nx < 0) return 0.f;
    const int oy = ny / g.sh, ox = nx / g.sw;
    if (oy * g.sh != ny || ox * g.sw != nx || oy >= g.ho || ox >= g.wo) return 0.f;
    return c.img[((int64_t)oy * g.wo + ox) * g.cout + c.co];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {  // co .. co+3 of one output pixel
    f4v r = {0.f, 0.f, 0.f, 0.f};
    const int ny = c.ty - c.r, nx = c.tx - c.q;
    if (c.img && c.k < k_end && ny >= 0 && nx >= 0) {
      if (g.sh == 1 && g.sw == 1) {  // unit strides (the same for every lane): no divisions
        if (ny < g.ho && nx < g.wo) r = *(const f4v*)(c.img + (ny * g.wo + nx) * g.cout + c.co);
      } else {
        const int oy = ny / g.sh, ox = nx / g.sw;
        if (oy * g.sh == ny && ox * g.sw == nx && oy < g.ho && ox < g.wo) r = *(const f4v*)(c.img + ((int64_t)oy * g.wo + ox) * g.cout + c.co);
      }
    }
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const { return g.cout % 4 == 0 && (reinterpret_cast<uintptr_t>(dy) & 15u) == 0; }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const {
    c.k += dk;
    c.co += dk;
    while (c.co >= g.cout) {
      c.co -= g.cout;
      if (++c.q == g.kw) { c.q = 0; ++c.r; }
    }
  }
  SN_CURSOR_ONLY_API
};

struct ConvDgradB {  // outer n = ci, k=(r,q,co): w[((r*kw+q)*cin + ci)*cout + co]
  static constexpr bool K_CONTIG = true;
  const float* w;
  ConvGeom g;
  struct Cursor {
    int ci, rq, co, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int n, int k) const {
    c.k = k;
    c.ci = n < g.cin ? n : -1;
    c.co = k % g.cout;
    c.rq = k / g.cout;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (c.ci < 0 || c.k >= k_end) return 0.f;
    return w[((int64_t)c.rq * g.cin + c.ci) * g.cout + c.co];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.ci >= 0 && c.k < k_end) r = *(const f4v*)(w + ((int64_t)c.rq * g.cin + c.ci) * g.cout + c.co);
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const { return g.cout % 4 == 0 && (reinterpret_cast<uintptr_t>(w) & 15u) == 0; }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const {
    c.k += dk;
    c.co += dk;
    while (c.co >= g.cout) { c.co -= g.cout; ++c.rq; }
  }
  SN_CURSOR_ONLY_API
};

// ---- Conv2D filter gradient: dw[r,q,ci,co] = sum_{b,oh,ow} x[b,oh*sh-pt+r,ow*sw-pl+q,ci] * dy[b,oh,ow,co]
struct ConvWgradA {  // m=(r,q,ci) (ci fastest -> contiguous), k=(b,oh,ow)
  static constexpr bool K_CONTIG = false;
  const float* x;
  ConvGeom g;
  int M;
  struct Cursor {
    int r, q, ci;  // ci < 0: row outside the matrix
    int b, oh, ow, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int m, int k) const {
    c.k = k;
    if (m >= M) { c.ci = -1; c.r = c.q = 0; }
    else {
      c.ci = m % g.cin;
      const int rq = m / g.cin;
      c.q = rq % g.kw;
      c.r = rq / g.kw;
    }
    c.ow = k % g.wo;
    const int t = k / g.wo;
    c.oh = t % g.ho;
    c.b = t / g.ho;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (c.ci < 0 || c.k >= k_end) return 0.f;
    const int iy = c.oh * g.sh - g.pt + c.r, ix = c.ow * g.sw - g.pl + c.q;
    if (iy < 0 || iy >= g.h || ix < 0 || ix >= g.w) return 0.f;
    return x[(((int64_t)c.b * g.h + iy) * g.w + ix) * g.cin + c.ci];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {  // rows (r,q,ci..ci+3) at one k
    f4v r = {0.f, 0.f, 0.f, 0.f};
    const int iy = c.oh * g.sh - g.pt + c.r, ix = c.ow * g.sw - g.pl + c.q;
    if (c.ci >= 0 && c.k < k_end && iy >= 0 && iy < g.h && ix >= 0 && ix < g.w)
      r = *(const f4v*)(x + (((int64_t)c.b * g.h + iy) * g.w + ix) * g.cin + c.ci);
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const { return g.cin % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0; }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const {
    c.k += dk;
    c.ow += dk;
    while (c.ow >= g.wo) {
      c.ow -= g.wo;
      if (++c.oh == g.ho) { c.oh = 0; ++c.b; }
    }
  }
  SN_CURSOR_ONLY_API
};

// ---- LSTM step: A(m,k) = k < F ? x[m, t, k] : h_prev[m, k-F]
struct LstmZA {
  static constexpr bool K_CONTIG = true;
  const float* x;       // [rows, T, F]
  const float* h_prev;  // [rows, H] or null (zeros)
  int rows, T, F, H, t;
  struct Cursor {
    int m, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int m, int k) const { c.m = m < rows ? m : -1; c.k = k; }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (c.m < 0 || c.k >= k_end) return 0.f;
    if (c.k < F) return x[((int64_t)c.m * T + t) * F + c.k];
    return h_prev ? h_prev[(int64_t)c.m * H + (c.k - F)] : 0.f;
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.m >= 0 && c.k < k_end) {
      if (c.k < F) r = *(const f4v*)(x + ((int64_t)c.m * T + t) * F + c.k);
      else if (h_prev) r = *(const f4v*)(h_prev + (int64_t)c.m * H + (c.k - F));
    }
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const {
    return F % 4 == 0 && H % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(h_prev) & 15u) == 0;
  }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const { c.k += dk; }
  SN_CURSOR_ONLY_API
};

// B(k,n) with n = gate*H + u: k < F ? Wk_gate[k, u] : Wr_gate[k-F, u]
struct LstmZB {
  static constexpr bool K_CONTIG = false;
  LstmWeights w;
  int F, H, G;  // G gates side by side (4 for the LSTM, 1 for the simple cell)
  struct Cursor {
    const float* wk;  // column base inside the gate's kernel matrix, null outside
    const float* wr;
    int k;
  };
  __device__ __forceinline__ void init(Cursor& c, int n, int k) const {
    c.k = k;
    if (n >= G * H) { c.wk = c.wr = nullptr; return; }
    const int gate = n / H, u = n % H;
    c.wk = w.wk[gate] + u;
    c.wr = w.wr[gate] + u;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (!c.wk || c.k >= k_end) return 0.f;
    return c.k < F ? c.wk[(int64_t)c.k * H] : c.wr[(int64_t)(c.k - F) * H];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {  // units u..u+3 of one gate
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.wk && c.k < k_end) r = c.k < F ? *(const f4v*)(c.wk + (int64_t)c.k * H) : *(const f4v*)(c.wr + (int64_t)(c.k - F) * H);
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const {
    bool ok = H % 4 == 0;
    for (int g = 0; g < G; ++g) ok = ok && (reinterpret_cast<uintptr_t>(w.wk[g]) & 15u) == 0 && (reinterpret_cast<uintptr_t>(w.wr[g]) & 15u) == 0;
    return ok;
  }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const { c.k += dk; }
  SN_CURSOR_ONLY_API
};

// B(k,n) = W_gate[n, u], k = gate*H + u (transposed gate weights: dh = dz Wr^T, dx = dz Wk^T)
struct LstmWT {
  static constexpr bool K_CONTIG = true;
  const float* w[4];
  int n_rows, H, G;  // W_gate is [n_rows, H]; G gates
  struct Cursor {
    int n, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int n, int k) const { c.n = n < n_rows ? n : -1; c.k = k; }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (c.n < 0 || c.k >= k_end) return 0.f;
    const int gate = c.k / H, u = c.k - gate * H;
    return w[gate][(int64_t)c.n * H + u];
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.n >= 0 && c.k < k_end) {
      const int gate = c.k / H, u = c.k - gate * H;
      r = *(const f4v*)(w[gate] + (int64_t)c.n * H + u);
    }
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const {
    bool ok = H % 4 == 0;
    for (int g = 0; g < G; ++g) ok = ok && (reinterpret_cast<uintptr_t>(w[g]) & 15u) == 0;
    return ok;
  }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const { c.k += dk; }
  SN_CURSOR_ONLY_API
};

// Weight gradients of all steps at once: A(m,k), k = t*rows + b:
//   m < F: x[b, t, m];  F <= m < F+H: h_{t-1}[b, m-F];  m == F+H: 1 (bias row)
struct LstmWgradA {
  static constexpr bool K_CONTIG = false;
  const float* x;           // [rows, T, F]
  const float* h_prev_all;  // [T, rows, H], slice t holds h_{t-1}
  int rows, T, F, H, M;
  struct Cursor {
    int m, t, b, k;
  };
  __device__ __forceinline__ void init(Cursor& c, int m, int k) const {
    c.m = m < M ? m : -1;
    c.k = k;
    c.t = k / rows;
    c.b = k - c.t * rows;
  }
  __device__ __forceinline__ float load(const Cursor& c, int k_end) const {
    if (c.m < 0 || c.k >= k_end) return 0.f;
    if (c.m < F) return x[((int64_t)c.b * T + c.t) * F + c.m];
    if (c.m < F + H) return h_prev_all[((int64_t)c.t * rows + c.b) * H + (c.m - F)];
    return 1.0f;
  }
  __device__ __forceinline__ void load4(const Cursor& c, int k_end, float (&v)[4]) const {  // rows m..m+3 at one k
    f4v r = {0.f, 0.f, 0.f, 0.f};
    if (c.m >= 0 && c.k < k_end) {
      if (c.m < F) r = *(const f4v*)(x + ((int64_t)c.b * T + c.t) * F + c.m);
      else if (c.m < F + H) r = *(const f4v*)(h_prev_all + ((int64_t)c.t * rows + c.b) * H + (c.m - F));
      else r[0] = 1.0f;  // the bias row; rows F+H+1.. lie outside the matrix
    }
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  bool vec4_ok(int) const {
    return F % 4 == 0 && H % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(h_prev_all) & 15u) == 0;
  }
  __device__ __forceinline__ void advance(Cursor& c, int dk) const {
    c.k += dk;
    c.b += dk;
    while (c.b >= rows) { c.b -= rows; ++c.t; }
  }
  SN_CURSOR_ONLY_API
};

// ============================================================================ FAST loaders
// Strided operand with unit stride along its contiguous index: value(outer, k) = p[outer*s_outer + k*s_k].
template <bool KC>
struct FlatLoader {
  static constexpr bool K_CONTIG = KC, FAST = true;
  const float* p;
  int s_outer, s_k;  // elements; one of them is 1
  int outer_n;
  struct Cursor {
    uint32_t base;  // byte offset of (outer, kk)
    int kk;         // < 0: outside the matrix
  };
  struct Tile {
    int k0;
    uint32_t koff;  // byte offset of k0
  };
  __device__ __forceinline__ void init4(Cursor& c, int outer, int, int kk) const {
    c.kk = outer < outer_n ? kk : -0x40000000;
    c.base = ((uint32_t)outer * (uint32_t)s_outer + (uint32_t)kk * (uint32_t)s_k) * 4u;
  }
  __device__ __forceinline__ void tile_init(Tile& t, int k0) const { t.k0 = k0; t.koff = (uint32_t)k0 * (uint32_t)s_k * 4u; }
  __device__ __forceinline__ void tile_advance(Tile& t) const { t.k0 += BK; t.koff += (uint32_t)BK * (uint32_t)s_k * 4u; }
  __device__ __forceinline__ void thread_advance(Cursor&) const {}
  __device__ __forceinline__ bool load4_t(const Cursor& c, const Tile& t, int k_end, float (&v)[4]) const {
    return sel_load4(p, c.base + t.koff, c.kk >= 0 && t.k0 + c.kk < k_end, v);
  }
  __device__ __forceinline__ float load_t(const Cursor&, const Tile&, int) const { return 0.f; }  // FAST loaders run VEC = 4 only
  static bool ok(const float* p, int64_t s_outer, int64_t s_k, int outer_n, int K) {
    if (!aligned16(p) || s_outer < 0 || s_k < 0 || ((int64_t)outer_n * s_outer + (int64_t)K * s_k) * 4 >= FAST_SPAN) return false;
    return KC ? (s_k == 1 && s_outer % 4 == 0 && K % 4 == 0) : (s_outer == 1 && s_k % 4 == 0 && outer_n % 4 == 0);
  }
};

// A operand of a convolution seen as a product: row m is a position (b, iy, ix) of the iteration space
// (the output for the forward pass, the input for the input gradient), k = (tap r, tap q, channel) with the
// channel fastest and the channel count a multiple of BK, so that a k tile lies inside one tap:
//   value = src[b, iy*sy + oy + r*ty, ix*sx + ox + q*tx, channel]   (0 outside the source image)
// forward: src = x, (sy, sx) = strides, (oy, ox) = -padding, (ty, tx) = (+1, +1);
// input gradient with unit strides: src = dy, (sy, sx) = (1, 1), (oy, ox) = +padding, (ty, tx) = (-1, -1).
// Which taps fall inside the image is fixed per row: a 32-bit mask computed once per thread.
struct TapLoader {
  static constexpr bool K_CONTIG = true, FAST = true;
  const float* src;
  int M, ih, iw;       // iteration space
  int sy, sx, oy, ox, ty, tx;
  int H, W, C;         // source image
  int kh, kw;
  struct Cursor {
    uint32_t base;  // byte offset of (b, y0, x0, kk), possibly outside the tensor (then no tap is valid there)
    uint32_t mask;  // bit r*kw+q: tap inside the image
    int kk;
  };
  struct Tile {
    int k0, r, q, c0, rq;
    uint32_t tapoff;  // byte offset of (r*ty, q*tx, c0) relative to (y0, x0, 0)
  };
  __device__ __forceinline__ void init4(Cursor& c, int m, int, int kk) const {
    c.kk = kk;
    c.mask = 0;
    c.base = 0;
    if (m >= M) return;
    const int ix = m % iw;
    const int t = m / iw;
    const int iy = t % ih;
    const int b = t / ih;
    const int y0 = iy * sy + oy, x0 = ix * sx + ox;
    c.base = (uint32_t)(((b * H + y0) * W + x0) * C + kk) * 4u;
    for (int r = 0; r < kh; ++r)
      for (int q = 0; q < kw; ++q)
        if ((unsigned)(y0 + r * ty) < (unsigned)H && (unsigned)(x0 + q * tx) < (unsigned)W) c.mask |= 1u << (r * kw + q);
  }
  __device__ __forceinline__ void set_tap(Tile& t) const { t.tapoff = (uint32_t)((t.r * ty * W + t.q * tx) * C + t.c0) * 4u; }
  __device__ __forceinline__ void tile_init(Tile& t, int k0) const {
    t.k0 = k0;
    t.rq = k0 / C;
    t.c0 = k0 - t.rq * C;
    t.r = t.rq / kw;
    t.q = t.rq - t.r * kw;
    set_tap(t);
  }
  __device__ __forceinline__ void tile_advance(Tile& t) const {
    t.k0 += BK;
    t.c0 += BK;
    if (t.c0 >= C) {
      t.c0 = 0;
      ++t.rq;
      if (++t.q == kw) { t.q = 0; ++t.r; }
    }
    set_tap(t);
  }
  __device__ __forceinline__ void thread_advance(Cursor&) const {}
  __device__ __forceinline__ bool load4_t(const Cursor& c, const Tile& t, int k_end, float (&v)[4]) const {
    return sel_load4(src, c.base + t.tapoff, ((c.mask >> (t.rq & 31)) & 1u) != 0 && t.k0 + c.kk < k_end, v);
  }
  __device__ __forceinline__ float load_t(const Cursor&, const Tile&, int) const { return 0.f; }
  static bool ok(const float* src, int n, int H, int W, int C, int kh, int kw) {
    return C % BK == 0 && kh * kw <= 32 && aligned16(src) && (int64_t)n * H * W * C * 4 < FAST_SPAN;
  }
};

// B operand of the input gradient: column n = ci, k = (r, q, co): w[((r*kw+q)*cin + ci)*cout + co], cout % BK == 0
struct DgradWLoader {
  static constexpr bool K_CONTIG = true, FAST = true;
  const float* w;
  int cin, cout;
  struct Cursor {
    uint32_t base;  // byte offset of (tap 0, ci, kk)
    int kk;         // < 0: outside the matrix
  };
  struct Tile {
    int k0, c0, rq;
    uint32_t koff;
  };
  __device__ __forceinline__ void init4(Cursor& c, int n, int, int kk) const {
    c.kk = n < cin ? kk : -0x40000000;
    c.base = (uint32_t)(n * cout + kk) * 4u;
  }
  __device__ __forceinline__ void tile_init(Tile& t, int k0) const {
    t.k0 = k0;
    t.rq = k0 / cout;
    t.c0 = k0 - t.rq * cout;
    t.koff = (uint32_t)(t.rq * cin * cout + t.c0) * 4u;
  }
  __device__ __forceinline__ void tile_advance(Tile& t) const {
    t.k0 += BK;
    t.c0 += BK;
    if (t.c0 >= cout) { t.c0 = 0; ++t.rq; }
    t.koff = (uint32_t)(t.rq * cin * cout + t.c0) * 4u;
  }
  __device__ __forceinline__ void thread_advance(Cursor&) const {}
  __device__ __forceinline__ bool load4_t(const Cursor& c, const Tile& t, int k_end, float (&v)[4]) const {
    return sel_load4(w, c.base + t.koff, c.kk >= 0 && t.k0 + c.kk < k_end, v);
  }
  __device__ __forceinline__ float load_t(const Cursor&, const Tile&, int) const { return 0.f; }
};

// A operand of the filter gradient: row m = (r, q, ci) with ci fastest (4 consecutive ci per load), k = output
// pixel (b, oh, ow): x[b, oh*sh - pt + r, ow*sw - pl + q, ci].  Every thread keeps its own pixel and moves it
// BK pixels per tile, carrying into the next output row / image by additions only.
struct WgradXLoader {
  static constexpr bool K_CONTIG = false, FAST = true;
  const float* x;
  ConvGeom g;
  int M;
  int interior;  // no padding: every tap of every output pixel lies inside the image, no bounds checks
  struct Cursor {
    uint32_t off;  // byte offset of the element
    int ow, oh, iy, ix, kk;  // kk < 0: row outside the matrix
  };
  struct Tile {
    int k0;
  };
  __device__ __forceinline__ void init4(Cursor& c, int m, int kb, int kk) const {
    c.kk = m < M ? kk : -0x40000000;
    const int ci = m % g.cin;
    const int rq = m / g.cin;
    const int q = rq % g.kw, r = rq / g.kw;
    const int p = kb + kk;
    c.ow = p % g.wo;
    const int t = p / g.wo;
    c.oh = t % g.ho;
    const int b = t / g.ho;
    c.iy = c.oh * g.sh - g.pt + r;
    c.ix = c.ow * g.sw - g.pl + q;
    c.off = (uint32_t)(((b * g.h + c.iy) * g.w + c.ix) * g.cin + ci) * 4u;
  }
  __device__ __forceinline__ void tile_init(Tile& t, int k0) const { t.k0 = k0; }
  __device__ __forceinline__ void tile_advance(Tile& t) const { t.k0 += BK; }
  __device__ __forceinline__ void thread_advance(Cursor& c) const {
    c.ow += BK;
    c.ix += BK * g.sw;
    c.off += (uint32_t)(BK * g.sw * g.cin) * 4u;
    while (c.ow >= g.wo) {  // next output row: back wo pixels, down sh input rows
      c.ow -= g.wo;
      c.ix -= g.wo * g.sw;
      c.off += (uint32_t)((g.sh * g.w - g.wo * g.sw) * g.cin) * 4u;
      c.iy += g.sh;
      if (++c.oh == g.ho) {  // next image
        c.oh = 0;
        c.iy -= g.ho * g.sh;
        c.off += (uint32_t)((g.h - g.ho * g.sh) * g.w * g.cin) * 4u;
      }
    }
  }
  __device__ __forceinline__ bool load4_t(const Cursor& c, const Tile& t, int k_end, float (&v)[4]) const {
    const bool inside = interior || ((unsigned)c.iy < (unsigned)g.h && (unsigned)c.ix < (unsigned)g.w);
    return sel_load4(x, c.off, c.kk >= 0 && t.k0 + c.kk < k_end && inside, v);
  }
  __device__ __forceinline__ float load_t(const Cursor&, const Tile&, int) const { return 0.f; }
  static bool ok(const float* x, const ConvGeom& g) {
    return g.cin % 4 == 0 && aligned16(x) && ((int64_t)g.n + 1) * g.h * g.w * g.cin * 4 < FAST_SPAN;
  }
};

// ============================================================================ epilogues
__device__ __forceinline__ float ep_act(int act, float v, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
    case SN_ACT_TANH: return tanhf(v);
    case SN_ACT_RELU: return fmaxf(param, v);
    default: return v;
  }
}

// The same activation over N values with ONE dispatch on `act`: a switch per value costs a handful of scalar branches
// each, which in a 16-value accumulator tile is more instruction-fetch stalls than arithmetic.
template <int N>
__device__ __forceinline__ void ep_act_block(int act, float (&v)[N], float param) {
  switch (act) {
    case SN_ACT_SIGMOID:
#pragma unroll
      for (int k = 0; k < N; ++k) v[k] = 1.0f / (1.0f + expf(-v[k]));
      break;
    case SN_ACT_TANH:
#pragma unroll
      for (int k = 0; k < N; ++k) v[k] = tanhf(v[k]);
      break;
    case SN_ACT_RELU:
#pragma unroll
      for (int k = 0; k < N; ++k) v[k] = fmaxf(param, v[k]);
      break;
    default: break;
  }
}

struct StdEpilogue {
  Epilogue e;
  __device__ __forceinline__ void store(int m, int n, float acc) const {
    if (m == e.row_index) {
      e.row_out[n] = acc;
      return;
    }
    float v = acc;
    if (e.bias) v = v + e.bias[n];
    e.out[(int64_t)m * e.ldo + n] = ep_act(e.act, v, e.act_param);
  }
};

// A lane's 16 accumulator values of one 32x32 MFMA tile: column n, rows row0 + 8*(v/4) + v%4 (v = 0..15), rows >= M dropped.
template <class EP>
__device__ __forceinline__ void store16(const EP& ep, int row0, int n, const f16v& acc, int M) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = row0 + (v >> 2) * 8 + (v & 3);
    if (row < M) ep.store(row, n, acc[v]);
  }
}
// The plain epilogue reads the column's bias once and dispatches on the activation once for the 16 values: inside an
// instantiation the activation is a compile-time constant, so the 16 stores carry no scalar branches.
template <int ACT>
__device__ __forceinline__ float ep_act_const(float v, float param) {
  if constexpr (ACT == SN_ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
  else if constexpr (ACT == SN_ACT_TANH) return tanhf(v);
  else if constexpr (ACT == SN_ACT_RELU) return fmaxf(param, v);
  else return v;
}

template <int ACT>
__device__ __forceinline__ void store16_act(const Epilogue& e, int row0, int n, const f16v& acc, int M) {
  const bool has_bias = e.bias != nullptr;
  const float b = has_bias ? e.bias[n] : 0.f;
  float* out = e.out + (int64_t)row0 * e.ldo + n;
  // One value at a time, each behind its own row check: a straight run of 16 stores lets the compiler compute all 16
  // addresses and read all 16 accumulators up front, which doubles the kernel's registers and costs the split-K launches
  // their occupancy (measured: filter gradient 31 -> 37 us).
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int dr = (k >> 2) * 8 + (k & 3);
    if (row0 + dr >= M) continue;
    if (row0 + dr == e.row_index) {
      e.row_out[n] = acc[k];
    } else {
      const float x = has_bias ? acc[k] + b : acc[k];
      out[(int64_t)dr * e.ldo] = ep_act_const<ACT>(x, e.act_param);
    }
  }
}

__device__ __forceinline__ void store16(const StdEpilogue& ep, int row0, int n, const f16v& acc, int M) {
  switch (ep.e.act) {
    case SN_ACT_SIGMOID: store16_act<SN_ACT_SIGMOID>(ep.e, row0, n, acc, M); break;
    case SN_ACT_TANH: store16_act<SN_ACT_TANH>(ep.e, row0, n, acc, M); break;
    case SN_ACT_RELU: store16_act<SN_ACT_RELU>(ep.e, row0, n, acc, M); break;
    default: store16_act<SN_ACT_IDENTITY>(ep.e, row0, n, acc, M); break;
  }
}

struct LstmZEpilogue {  // z[m, n] = acc + b_gate[u]
  float* z;
  const float* b[4];
  int H, G;
  __device__ __forceinline__ void store(int m, int n, float acc) const {
    const int gate = n / H, u = n - gate * H;
    float v = acc;
    if (b[gate]) v = v + b[gate][u];
    z[(int64_t)m * G * H + n] = v;
  }
};

struct LstmWgradEpilogue {  // rows: F kernel rows, H recurrent rows, 1 bias row; columns gate*H + u
  LstmGrads g;
  int F, H;
  __device__ __forceinline__ void store(int m, int n, float acc) const {
    const int gate = n / H, u = n - gate * H;
    if (m < F) g.wk[gate][(int64_t)m * H + u] = acc;
    else if (m < F + H) g.wr[gate][(int64_t)(m - F) * H + u] = acc;
    else if (g.b[gate]) g.b[gate][u] = acc;
  }
};

struct DxScatterEpilogue {  // dx[m, t, n] of a [rows, T, F] tensor
  float* dx;
  int T, F, t;
  __device__ __forceinline__ void store(int m, int n, float acc) const { dx[((int64_t)m * T + t) * F + n] = acc; }
};

// ============================================================================ the kernel
template <bool KC, int BT>
__device__ __forceinline__ int lds_index(int outer, int k) {
  // K-contiguous operands are staged as [outer][BK+1], the others as [BK][BT+1]; either way
  // both the staging writes and the MFMA operand reads are free of systematic bank conflicts.
  return KC ? outer * (BK + 1) + k : k * (BT + 1) + outer;
}

template <bool BF16>
struct LdsElem { typedef float type; };
template <>
struct LdsElem<true> { typedef __bf16 type; };

// VEC = 4: every tile copy moves 4 values per load along the operand's contiguous index (the host checks
// vec4_ok() of both loaders); VEC = 1 is the general element-wise form.
template <int BM, int BN, bool BF16, int VEC, class AL, class BL, class EP>
__global__ __launch_bounds__(THREADS) void gemm_kernel(int M, int N, int K, int k_per_split, AL al, BL bl, EP ep, float* ws, int splits) {
  typedef typename LdsElem<BF16>::type lds_t;
  // the 4 waves form a 2x2 grid over the tile, or 4x1 when the tile is a single MFMA block wide
  constexpr int WAVES_N = BN >= 64 ? 2 : 1, WAVES_M = 4 / WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
  // a B tile of fewer than THREADS vectors is copied by the first B_ACTIVE threads only
  constexpr int B_ACTIVE = BN * BK / VEC < THREADS ? BN * BK / VEC : THREADS;
  constexpr int EA = BM * BK / (THREADS * VEC), EB = BN * BK / (B_ACTIVE * VEC);
  static_assert(TM >= 1 && TN >= 1 && EA >= 1, "tile too small for four waves");
  __shared__ lds_t As[BM * (BK + 1)];
  __shared__ lds_t Bs[BN * (BK + 1)];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool b_on = tid < B_ACTIVE;
  // Split-K launches use a flat grid: consecutive workgroup ids land on different XCDs (8, each with its own L2),
  // so XCD x takes the splits x, x+8, ... and walks all output tiles of one split before the next: the tiles
  // that re-read the same K range of A and B then share one L2 instead of fetching it once per XCD.
  int bm = blockIdx.y, bn = blockIdx.x, bz = blockIdx.z;
  if (splits > 1) {
    const int tiles_n = (N + BN - 1) / BN, tiles_mn = tiles_n * ((M + BM - 1) / BM);
    const int slot = blockIdx.x >> 3;
    bz = (blockIdx.x & 7) + 8 * (slot / tiles_mn);
    if (bz >= splits) return;
    const int tile = slot % tiles_mn;
    bm = tile / tiles_n;
    bn = tile - bm * tiles_n;
  }
  const int m0 = bm * BM, n0 = bn * BN;
  const int k_begin = bz * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);

  typename AL::Cursor ca[EA];
  typename BL::Cursor cb[EB];
  typename AL::Tile ta;
  typename BL::Tile tb;
  int ia[EA], ib[EB];  // LDS slot of the first value of each vector; the others follow one slot apart
#pragma unroll
  for (int e = 0; e < EA; ++e) {
    int mm, kk;
    if (AL::K_CONTIG) { constexpr int KV = BK / VEC; kk = (tid % KV) * VEC; mm = tid / KV + e * (THREADS / KV); }
    else { constexpr int OV = BM / VEC; mm = (tid % OV) * VEC; kk = tid / OV + e * (THREADS / OV); }
    al.init4(ca[e], m0 + mm, k_begin, kk);
    ia[e] = lds_index<AL::K_CONTIG, BM>(mm, kk);
  }
#pragma unroll
  for (int e = 0; e < EB; ++e) {
    int nn, kk;
    if (BL::K_CONTIG) { constexpr int KV = BK / VEC; kk = (tid % KV) * VEC; nn = tid / KV + e * (B_ACTIVE / KV); }
    else { constexpr int OV = BN / VEC; nn = (tid % OV) * VEC; kk = tid / OV + e * (B_ACTIVE / OV); }
    if (!b_on) { nn = 0; kk = 0; }
    bl.init4(cb[e], n0 + nn, k_begin, kk);
    ib[e] = lds_index<BL::K_CONTIG, BN>(nn, kk);
  }
  al.tile_init(ta, k_begin);
  bl.tile_init(tb, k_begin);

  f16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // both staging layouts put consecutive values of the contiguous index one LDS slot apart
  float ra[EA][VEC], rb[EB][VEC];
  bool va[EA], vb[EB];  // false: the vector lies outside the operand and goes to LDS as zeros
  auto fetch = [&]() {  // loads the tile the loaders point at (zeros past k_end), then moves them on
#pragma unroll
    for (int e = 0; e < EA; ++e) {
      va[e] = true;
      if constexpr (VEC == 4) va[e] = al.load4_t(ca[e], ta, k_end, ra[e]);
      else ra[e][0] = al.load_t(ca[e], ta, k_end);
      al.thread_advance(ca[e]);
    }
    if (b_on) {
#pragma unroll
      for (int e = 0; e < EB; ++e) {
        vb[e] = true;
        if constexpr (VEC == 4) vb[e] = bl.load4_t(cb[e], tb, k_end, rb[e]);
        else rb[e][0] = bl.load_t(cb[e], tb, k_end);
        bl.thread_advance(cb[e]);
      }
    }
    al.tile_advance(ta);
    bl.tile_advance(tb);
  };
  fetch();

  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
  const int l32 = lane & 31, lhi = lane >> 5;

  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
#pragma unroll
    for (int e = 0; e < EA; ++e)
#pragma unroll
      for (int i = 0; i < VEC; ++i) As[ia[e] + i] = (lds_t)(va[e] ? ra[e][i] : 0.f);
    if (b_on) {
#pragma unroll
      for (int e = 0; e < EB; ++e)
#pragma unroll
        for (int i = 0; i < VEC; ++i) Bs[ib[e] + i] = (lds_t)(vb[e] ? rb[e][i] : 0.f);
    }
    __syncthreads();
    if (k0 + BK < k_end) fetch();  // the next tile's global loads fly while this one is multiplied
    if constexpr (!BF16) {
#pragma unroll
      for (int ks = 0; ks < BK; ks += 2) {
        const int k = ks + lhi;
        float av[TM], bv[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) av[i] = As[lds_index<AL::K_CONTIG, BM>(wm + i * 32 + l32, k)];
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = Bs[lds_index<BL::K_CONTIG, BN>(wn + j * 32 + l32, k)];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
      }
    } else {
      // 32x32x16 bf16: lane supplies k = 8*(lane/32) .. +7 of row/col lane%32
      bf16x8 av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 8; ++v) av[i][v] = As[lds_index<AL::K_CONTIG, BM>(wm + i * 32 + l32, lhi * 8 + v)];
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 8; ++v) bv[j][v] = Bs[lds_index<BL::K_CONTIG, BN>(wn + j * 32 + l32, lhi * 8 + v)];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  // accumulator element v of lane l sits at row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn + j * 32 + l32;
      if (col >= N) continue;
      const int row0 = m0 + wm + i * 32 + lhi * 4;
      if (ws) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = row0 + (v >> 2) * 8 + (v & 3);
          if (row < M) ws[((int64_t)bz * M + row) * N + col] = acc[i][j][v];
        }
      } else {
        store16(ep, row0, col, acc[i][j], M);
      }
    }
}

// Adds the split-K partial tiles.  Eight lanes share one output: lane g adds splits g, g+8, ... in order, then the
// eight partial sums are combined pairwise (a fixed tree), so the result does not depend on the launch shape.
template <class EP>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int splits, int M, int N, EP ep) {
  const int64_t total = (int64_t)M * N;
  const int g = threadIdx.x >> 5, j = threadIdx.x & 31;  // 8 groups of 32 consecutive outputs
  for (int64_t base = (int64_t)blockIdx.x * 32; base < total; base += (int64_t)gridDim.x * 32) {
    const int64_t i = base + j;
    float s = 0.f;
    if (i < total) {
      int z = g;
      for (; z + 120 < splits; z += 128) {  // 16 loads in flight, added in split order
        float a[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) a[u] = ws[(int64_t)(z + 8 * u) * total + i];
#pragma unroll
        for (int u = 0; u < 16; ++u) s += a[u];
      }
      for (; z + 24 < splits; z += 32) {  // 4 loads in flight
        float a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) a[u] = ws[(int64_t)(z + 8 * u) * total + i];
#pragma unroll
        for (int u = 0; u < 4; ++u) s += a[u];
      }
      for (; z < splits; z += 8) s += ws[(int64_t)z * total + i];
    }
    __shared__ float part[8][32];
    part[g][j] = s;
    __syncthreads();
    if (g == 0 && i < total) {
      const float t = ((part[0][j] + part[1][j]) + (part[2][j] + part[3][j])) + ((part[4][j] + part[5][j]) + (part[6][j] + part[7][j]));
      ep.store((int)(i / N), (int)(i % N), t);
    }
    __syncthreads();
  }
}

// The same reduction when M*N is a multiple of 4 (every partial tile then starts on a 16-byte boundary): a lane owns 4
// consecutive outputs and reads them as one 16-byte load per split; every output sees the same additions in the same order.
template <class EP>
__global__ __launch_bounds__(256) void splitk_reduce4_kernel(const float* __restrict__ ws, int splits, int M, int N, EP ep) {
  const int64_t total4 = (int64_t)M * N / 4;
  const int g = threadIdx.x >> 5, j = threadIdx.x & 31;  // 8 groups of 32 lanes x 4 consecutive outputs
  for (int64_t base = (int64_t)blockIdx.x * 32; base < total4; base += (int64_t)gridDim.x * 32) {
    const int64_t i = base + j;
    f4v s = {0.f, 0.f, 0.f, 0.f};
    if (i < total4) {
      const f4v* w4 = reinterpret_cast<const f4v*>(ws) + i;
      int z = g;
      for (; z + 56 < splits; z += 64) {  // 8 loads of 16 bytes in flight, added in split order
        f4v a[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = w4[(int64_t)(z + 8 * u) * total4];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += a[u];
      }
      for (; z < splits; z += 8) s += w4[(int64_t)z * total4];
    }
    __shared__ f4v part4[8][32];
    part4[g][j] = s;
    __syncthreads();
    if (g == 0 && i < total4) {
      const f4v t = ((part4[0][j] + part4[1][j]) + (part4[2][j] + part4[3][j])) + ((part4[4][j] + part4[5][j]) + (part4[6][j] + part4[7][j]));
      // row and column of the first of the four outputs by one division (32-bit where the index allows: a 64-bit division
      // is some hundred instructions on this device), the others by stepping
      const int64_t o0 = i * 4;
      int m, n;
      if (o0 < ((int64_t)1 << 31)) {
        const uint32_t q = (uint32_t)o0 / (uint32_t)N;
        m = (int)q;
        n = (int)((uint32_t)o0 - q * (uint32_t)N);
      } else {
        m = (int)(o0 / N);
        n = (int)(o0 % N);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ep.store(m, n, t[e]);
        if (++n == N) { n = 0; ++m; }
      }
    }
    __syncthreads();
  }
}

// ============================================================================ small output, long reduction
// C[M,N] with M*N <= 1024 and K in the thousands (first-layer filter gradients, Dense layers onto a few
// classes): too little output for MFMA tiles to occupy the chip. Workgroups stride over 64-long slices of K,
// stage them in LDS, keep up to four outputs per thread in registers and leave one partial sum per workgroup
// and output; a second kernel adds the partials in a fixed order.
constexpr int SMALL_SLICE = 64, SMALL_MAX_OUT = 512, SMALL_MAX_DIM = 128, SMALL_MIN_K = 2048;

template <class AL, class BL>
__global__ __launch_bounds__(256) void gemm_small_kernel(int M, int N, int K, AL al, BL bl, float* __restrict__ partial) {
  extern __shared__ float small_lds[];
  float* As = small_lds;                    // [SMALL_SLICE][M]
  float* Bs = small_lds + SMALL_SLICE * M;  // [SMALL_SLICE][N]
  const int tid = threadIdx.x, outs = M * N;
  int om[4], on[4];
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = tid + j * 256;
    om[j] = o < outs ? o / N : 0;
    on[j] = o < outs ? o % N : 0;
  }
  const int slices = (K + SMALL_SLICE - 1) / SMALL_SLICE;
  for (int sl = blockIdx.x; sl < slices; sl += gridDim.x) {
    const int k0 = sl * SMALL_SLICE;
    // batches of 8 loads per thread are issued before any of them is stored, so their latencies overlap
    for (int base = 0; base < SMALL_SLICE * M; base += 256 * 8) {
      float v[8];
      int at[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = base + u * 256 + tid;
        int m, p;
        if (AL::K_CONTIG) { p = e % SMALL_SLICE; m = e / SMALL_SLICE; }
        else { m = e % M; p = e / M; }
        at[u] = e < SMALL_SLICE * M ? p * M + m : -1;
        typename AL::Cursor c;
        al.init(c, at[u] >= 0 ? m : M, k0 + p);
        v[u] = al.load(c, K);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (at[u] >= 0) As[at[u]] = v[u];
    }
    for (int base = 0; base < SMALL_SLICE * N; base += 256 * 8) {
      float v[8];
      int at[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = base + u * 256 + tid;
        int n, p;
        if (BL::K_CONTIG) { p = e % SMALL_SLICE; n = e / SMALL_SLICE; }
        else { n = e % N; p = e / N; }
        at[u] = e < SMALL_SLICE * N ? p * N + n : -1;
        typename BL::Cursor c;
        bl.init(c, at[u] >= 0 ? n : N, k0 + p);
        v[u] = bl.load(c, K);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (at[u] >= 0) Bs[at[u]] = v[u];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if ((tid & ~63) + j * 256 >= outs) break;  // the same for every lane of a wave
      float a = acc[j];
#pragma unroll 8
      for (int p = 0; p < SMALL_SLICE; ++p) a += As[p * M + om[j]] * Bs[p * N + on[j]];
      acc[j] = a;
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = tid + j * 256;
    if (o < outs) partial[(int64_t)blockIdx.x * outs + o] = acc[j];  // [part][output]: a workgroup's outputs leave as one run
  }
}

// Adds the partial sums [parts][M*N] in a fixed order: a workgroup owns 4 outputs, 64 lanes each walk every 64th part.
template <class EP>
__global__ __launch_bounds__(256) void gemm_small_reduce_kernel(const float* __restrict__ partial, int parts, int M, int N, EP ep) {
  __shared__ float sm[64][4];
  const int outs = M * N;
  const int ol = threadIdx.x & 3, pl = threadIdx.x >> 2;
  const int o = blockIdx.x * 4 + ol;
  float s = 0.f;
  if (o < outs) {
    for (int i = pl; i < parts; i += 64 * 8) {  // 8 loads in flight, added in part order
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = i + 64 * u < parts ? partial[(int64_t)(i + 64 * u) * outs + o] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
  }
  sm[pl][ol] = s;
  __syncthreads();
  if (threadIdx.x < 4 && o < outs) {
    float t = 0.f;
#pragma unroll 8
    for (int j = 0; j < 64; ++j) t += sm[j][ol];
    ep.store(o / N, o % N, t);
  }
}

static int small_parts(int m, int n, int k, int cu, int64_t ws_elems) {
  if ((int64_t)m * n > SMALL_MAX_OUT || m > SMALL_MAX_DIM || n > SMALL_MAX_DIM || k < SMALL_MIN_K) return 0;
  int64_t parts = std::min<int64_t>(ceil_div(k, SMALL_SLICE), (int64_t)4 * cu);
  if (ws_elems >= 0) parts = std::min<int64_t>(parts, ws_elems / ((int64_t)m * n));
  return parts >= 32 ? (int)parts : 0;
}

// ============================================================================ dispatch
constexpr int SPLIT_WG_PER_CU = 8, SPLIT_MAX = 256, SPLIT_MIN_K = 256;
int64_t gemm_workspace_elems(int m, int n, int k, int cu) {
  // room for the partial sums of the small-output kernel, or for the largest split count launch_tiles may pick
  const int parts = small_parts(m, n, k, cu, -1);
  if (parts) return (int64_t)parts * m * n;
  const int64_t tiles = ceil_div(m, 64) * ceil_div(n, 64);
  if (tiles >= cu || k < SPLIT_MIN_K) return 0;
  int64_t splits = std::min<int64_t>(ceil_div((int64_t)SPLIT_WG_PER_CU * cu, tiles), std::max<int64_t>(1, k / 32));
  splits = std::min<int64_t>(splits, SPLIT_MAX);
  return splits * (int64_t)m * n;
}

template <int BM, int BN, bool BF16, class AL, class BL, class EP>
static int launch_tiles(sn_ctx* ctx, const char* name, int M, int N, int K, const AL& al, const BL& bl, const EP& ep, float* ws,
                        int64_t ws_elems) {
  const int64_t tiles = ceil_div(M, BM) * ceil_div(N, BN);
  int splits = 1;
  if (tiles * 2 <= ctx->compute_units && K >= SPLIT_MIN_K && ws) {  // a split costs a second pass over M*N*splits floats
    // These kernels are a chain of load, stage, multiply per K tile: what hides its latency is other workgroups on
    // the same CU, so aim for 8 per CU (measured: 2 per CU runs the LeNet filter gradient in 52 us, 8 per CU in 31).
    int64_t s = std::min<int64_t>(ceil_div((int64_t)SPLIT_WG_PER_CU * ctx->compute_units, tiles), std::max<int64_t>(1, K / 32));
    s = std::min<int64_t>(s, SPLIT_MAX);
    s = std::min<int64_t>(s, ws_elems / ((int64_t)M * N));
    splits = (int)std::max<int64_t>(1, s);
  }
  // XCD x takes the splits x, x + 8, ...: a count that is no multiple of 8 gives some XCDs a split more than others
  // (26 splits of the LSTM weight gradient: two XCDs with 4, six with 3; with 24: 255 -> 226 us)
  if (splits > 8) splits = splits / 8 * 8;
  int k_per_split = (int)align_up(ceil_div(K, splits), BK);
  splits = (int)ceil_div(K, k_per_split);
  const dim3 grid = splits > 1 ? dim3((unsigned)(8 * ceil_div(N, BN) * ceil_div(M, BM) * ceil_div(splits, 8)))
                               : dim3((unsigned)ceil_div(N, BN), (unsigned)ceil_div(M, BM), 1);
  {
    LaunchScope scope(ctx, name, M, N, K);
    if constexpr (AL::FAST && BL::FAST) {  // the caller has checked what 16-byte loads need
      hipLaunchKernelGGL((gemm_kernel<BM, BN, BF16, 4, AL, BL, EP>), grid, dim3(THREADS), 0, ctx->stream, M, N, K, k_per_split, al, bl, ep,
                         splits > 1 ? ws : nullptr, splits);
    } else {
      if (al.vec4_ok(K) && bl.vec4_ok(K))
        hipLaunchKernelGGL((gemm_kernel<BM, BN, BF16, 4, AL, BL, EP>), grid, dim3(THREADS), 0, ctx->stream, M, N, K, k_per_split, al, bl, ep,
                           splits > 1 ? ws : nullptr, splits);
      else
        hipLaunchKernelGGL((gemm_kernel<BM, BN, BF16, 1, AL, BL, EP>), grid, dim3(THREADS), 0, ctx->stream, M, N, K, k_per_split, al, bl, ep,
                           splits > 1 ? ws : nullptr, splits);
    }
  }
  if (splits > 1) {
    const int64_t total = (int64_t)M * N;
    if constexpr (std::is_same<EP, StdEpilogue>::value) {
      // a caller that applies the optimizer next takes the sum of the partial tiles into that launch
      if (ctx->defer && total % 4 == 0 && total >= 4096 && total < ((int64_t)1 << 30) && aligned16(ws) && !ep.e.bias && ep.e.act == SN_ACT_IDENTITY &&
          ep.e.row_index < 0 && ep.e.ldo == N) {
        *ctx->defer = DeferredReduce{1, ws, splits, (int)total, ep.e.out};
        ctx->defer = nullptr;
        SN_HIP(hipGetLastError());
        return SN_OK;
      }
    }
    LaunchScope scope(ctx, "splitk_reduce");
    if (total % 4 == 0 && total >= 4096 && aligned16(ws)) {
      const int64_t blocks = std::min<int64_t>(ceil_div(total / 4, 32), (int64_t)ctx->compute_units * 16);
      hipLaunchKernelGGL((splitk_reduce4_kernel<EP>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const float*)ws, splits, M, N, ep);
    } else {
      const int64_t blocks = std::min<int64_t>(ceil_div(total, 32), (int64_t)ctx->compute_units * 16);
      hipLaunchKernelGGL((splitk_reduce_kernel<EP>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const float*)ws, splits, M, N, ep);
    }
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

template <bool BF16, class AL, class BL, class EP>
static int launch_any(sn_ctx* ctx, const char* name, int M, int N, int K, const AL& al, const BL& bl, const EP& ep, float* ws,
                      int64_t ws_elems) {
  if (M <= 0 || N <= 0) return SN_OK;
  SN_REQUIRE(K > 0, "%s: empty reduction dimension", name);
  if constexpr (!(AL::FAST && BL::FAST)) {
   if (const int parts = ws ? small_parts(M, N, K, ctx->compute_units, ws_elems) : 0) {
    {
      LaunchScope scope(ctx, name, M, N, K);
      hipLaunchKernelGGL((gemm_small_kernel<AL, BL>), dim3((unsigned)parts), dim3(256), (size_t)SMALL_SLICE * (M + N) * sizeof(float),
                         ctx->stream, M, N, K, al, bl, ws);
    }
    LaunchScope scope(ctx, "small_output_reduce");
    hipLaunchKernelGGL((gemm_small_reduce_kernel<EP>), dim3((unsigned)ceil_div(M * N, 4)), dim3(256), 0, ctx->stream, (const float*)ws,
                       parts, M, N, ep);
    SN_HIP(hipGetLastError());
    return SN_OK;
   }
  }
  bool big_m = M > 64, big_n = N > 64;
  // 128-wide tiles only when they still cover every CU at least twice; otherwise more, smaller workgroups
  if (ceil_div(M, big_m ? 128 : 64) * ceil_div(N, big_n ? 128 : 64) < (int64_t)2 * ctx->compute_units) big_m = big_n = false;
  if (N <= 32 && M > 64) return launch_tiles<128, 32, BF16>(ctx, name, M, N, K, al, bl, ep, ws, ws_elems);
  if (big_m && big_n) return launch_tiles<128, 128, BF16>(ctx, name, M, N, K, al, bl, ep, ws, ws_elems);
  if (big_m) return launch_tiles<128, 64, BF16>(ctx, name, M, N, K, al, bl, ep, ws, ws_elems);
  if (big_n) return launch_tiles<64, 128, BF16>(ctx, name, M, N, K, al, bl, ep, ws, ws_elems);
  return launch_tiles<64, 64, BF16>(ctx, name, M, N, K, al, bl, ep, ws, ws_elems);
}

static bool fast_pair_ok(const sn_ctx* ctx, const GemmDesc& g, const float* ws, int64_t ws_elems) {
  if (g.a_ones_row || (ws && small_parts(g.m, g.n, g.k, ctx->compute_units, ws_elems))) return false;
  const bool akc = g.a_sk == 1, bkc = g.b_sk == 1 && g.b_sn != 1;
  const bool a_ok = akc ? FlatLoader<true>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k) : FlatLoader<false>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k);
  const bool b_ok = bkc ? FlatLoader<true>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k) : FlatLoader<false>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k);
  return a_ok && b_ok;
}

bool gemm_takes_fast_loaders(const sn_ctx* ctx, const GemmDesc& g, const float* workspace, int64_t workspace_elems) {
  return fast_pair_ok(ctx, g, workspace, workspace_elems);
}

template <bool BF16>
static int launch_gemm_t(sn_ctx* ctx, const GemmDesc& g, const Epilogue& e, float* ws, int64_t ws_elems) {
  StdEpilogue ep{e};
  const char* name = BF16 ? "gemm_bf16" : "gemm_f32";
  const bool akc = g.a_sk == 1, bkc = g.b_sk == 1 && g.b_sn != 1;
  // FAST loaders whenever both operands allow 16-byte loads, unless the small-output kernel (cursor loaders) takes the problem
  if (fast_pair_ok(ctx, g, ws, ws_elems)) {
    if (akc && bkc && FlatLoader<true>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k) && FlatLoader<true>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k)) {
      FlatLoader<true> al{g.a, (int)g.a_sm, (int)g.a_sk, g.m}, bl{g.b, (int)g.b_sn, (int)g.b_sk, g.n};
      return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
    }
    if (akc && !bkc && FlatLoader<true>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k) && FlatLoader<false>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k)) {
      FlatLoader<true> al{g.a, (int)g.a_sm, (int)g.a_sk, g.m};
      FlatLoader<false> bl{g.b, (int)g.b_sn, (int)g.b_sk, g.n};
      return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
    }
    if (!akc && bkc && FlatLoader<false>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k) && FlatLoader<true>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k)) {
      FlatLoader<false> al{g.a, (int)g.a_sm, (int)g.a_sk, g.m};
      FlatLoader<true> bl{g.b, (int)g.b_sn, (int)g.b_sk, g.n};
      return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
    }
    if (!akc && !bkc && FlatLoader<false>::ok(g.a, g.a_sm, g.a_sk, g.m, g.k) && FlatLoader<false>::ok(g.b, g.b_sn, g.b_sk, g.n, g.k)) {
      FlatLoader<false> al{g.a, (int)g.a_sm, (int)g.a_sk, g.m}, bl{g.b, (int)g.b_sn, (int)g.b_sk, g.n};
      return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
    }
  }
  if (g.a_ones_row) {  // the weight-gradient form: A = X^T (outer index contiguous) plus the ones row, B = dY (row major)
    SN_REQUIRE(!akc && !bkc, "gemm: the all-ones row is built for A^T-major A and row-major B only");
    StridedLoader<false, true> al{g.a, g.a_sm, g.a_sk, g.m - 1, g.m - 1};
    StridedLoader<false> bl{g.b, g.b_sn, g.b_sk, g.n};
    return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
  }
  if (akc && bkc) {
    StridedLoader<true> al{g.a, g.a_sm, g.a_sk, g.m}, bl{g.b, g.b_sn, g.b_sk, g.n};
    return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
  } else if (akc) {
    StridedLoader<true> al{g.a, g.a_sm, g.a_sk, g.m};
    StridedLoader<false> bl{g.b, g.b_sn, g.b_sk, g.n};
    return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
  } else if (bkc) {
    StridedLoader<false> al{g.a, g.a_sm, g.a_sk, g.m};
    StridedLoader<true> bl{g.b, g.b_sn, g.b_sk, g.n};
    return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
  }
  StridedLoader<false> al{g.a, g.a_sm, g.a_sk, g.m}, bl{g.b, g.b_sn, g.b_sk, g.n};
  return launch_any<BF16>(ctx, name, g.m, g.n, g.k, al, bl, ep, ws, ws_elems);
}

int launch_gemm(sn_ctx* ctx, const GemmDesc& g, const Epilogue& ep, float* workspace, int64_t workspace_elems, bool bf16) {
  SN_REQUIRE(g.a && g.b && ep.out, "gemm: null operand");
  return bf16 ? launch_gemm_t<true>(ctx, g, ep, workspace, workspace_elems) : launch_gemm_t<false>(ctx, g, ep, workspace, workspace_elems);
}

// ---------------------------------------------------------------------------- Conv2D
// First-layer convolutions (1 to 4 input channels): K = kh*kw*cin is a few dozen, far too short for MFMA tiles
// to pay for their set-up, and the layer is bound by writing its output.  Direct form: the filter sits in LDS,
// 8 neighbouring lanes share one output pixel and own 4 output channels each (so a pixel's channels leave as
// one contiguous run), every lane gathers the pixel's K inputs itself (they stay in L1).
constexpr int DIRECT_MAX_K = 64;
__global__ __launch_bounds__(256) void conv_direct_fwd_kernel(ConvGeom g, const float* __restrict__ x, const float* __restrict__ w,
                                                               Epilogue e, int pixels) {
  extern __shared__ __attribute__((aligned(16))) float wl[];  // [K][cout]
  const int K = g.kh * g.kw * g.cin;
  for (int i = threadIdx.x; i < K * g.cout; i += 256) wl[i] = w[i];
  __syncthreads();
  const int quads = g.cout / 4;  // channel quads per pixel
  const int64_t total = (int64_t)pixels * quads;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
    const int cq = (int)(t % quads);
    const int p = (int)(t / quads);
    const int ow = p % g.wo;
    const int t2 = p / g.wo;
    const int oh = t2 % g.ho;
    const int b = t2 / g.ho;
    const int iy0 = oh * g.sh - g.pt, ix0 = ow * g.sw - g.pl;
    const float* img = x + (int64_t)b * g.h * g.w * g.cin;
    f4v acc = {0.f, 0.f, 0.f, 0.f};
    int k = 0;
    for (int r = 0; r < g.kh; ++r) {
      const int iy = iy0 + r;
      for (int q = 0; q < g.kw; ++q) {
        const int ix = ix0 + q;
        const bool in = (unsigned)iy < (unsigned)g.h && (unsigned)ix < (unsigned)g.w;
        for (int ci = 0; ci < g.cin; ++ci, ++k) {
          const float xv = in ? img[(iy * g.w + ix) * g.cin + ci] : 0.f;
          const f4v wv = *(const f4v*)(wl + k * g.cout + cq * 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(xv, wv[i], acc[i]);  // fused like the matrix cores; k in (r, q, ci) order
        }
      }
    }
    const int col = cq * 4;
    f4v out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = acc[i];
      if (e.bias) v = v + e.bias[col + i];
      out[i] = ep_act(e.act, v, e.act_param);
    }
    *(f4v*)(e.out + (int64_t)p * e.ldo + col) = out;
  }
}

// U pixels of one lane (p0, p0 + slots, ...; all inside the band): taps outermost, so a tap's weights are used U times.
template <int MT, int U>
__device__ __forceinline__ void fwd_rows_pixels(const float* lds, const int* origin, const int (&off)[MT], const f4v (&wr)[MT], const f4v& bias,
                                                const Epilogue& e, float* outb, int p0, int slots) {
  f4v acc[U];
  int base[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    base[u] = origin[p0 + u * slots];
    acc[u] = f4v{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float xv = lds[base[u] + off[m]];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[u][i] = __builtin_fmaf(xv, wr[m][i], acc[u][i]);
    }
  }
  float v[U * 4];
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[u * 4 + i] = acc[u][i] + bias[i];
  }
  ep_act_block<U * 4>(e.act, v, e.act_param);  // one dispatch on the activation for all of the lane's pixels
#pragma unroll
  for (int u = 0; u < U; ++u) *(f4v*)(outb + (int64_t)(p0 + u * slots) * e.ldo) = f4v{v[u * 4], v[u * 4 + 1], v[u * 4 + 2], v[u * 4 + 3]};
}

// What a launch of the two direct first-layer kernels below fixes and the device would otherwise divide out per thread
// (the device has no integer divider): the LDS offset of tap m = (r, q, ci) from a position's top-left input element
// (taps >= kh*kw*cin repeat tap 0), and the divisors of the index arithmetic.
constexpr int WGRAD_DIRECT_MAX_TAPS = 36;
struct DirectConvPlan {
  int off[WGRAD_DIRECT_MAX_TAPS];
  FastDiv by_cv, by_wo, by_row_elems, by_cin, by_cout;
};
static DirectConvPlan direct_conv_plan(const ConvGeom& g, int lw) {
  DirectConvPlan plan;
  const int M = g.kh * g.kw * g.cin, row_elems = lw * g.cin;
  for (int m = 0; m < WGRAD_DIRECT_MAX_TAPS; ++m) {
    const int mm = m < M ? m : 0;
    const int ci = mm % g.cin, rq = mm / g.cin;
    plan.off[m] = (rq / g.kw) * row_elems + (rq % g.kw) * g.cin + ci;
  }
  plan.by_cv = fast_div((uint32_t)std::max(1, g.cout / 4));
  plan.by_wo = fast_div((uint32_t)g.wo);
  plan.by_row_elems = fast_div((uint32_t)row_elems);
  plan.by_cin = fast_div((uint32_t)g.cin);
  plan.by_cout = fast_div((uint32_t)g.cout);
  return plan;
}

// The same layer when the filter count is 4 << j (j = 0..6) and there are at most 18 taps: a workgroup takes a band of
// output rows of one image and keeps the input rows under it in LDS, zero-padded; a lane owns 4 filters, holds their
// weights for every tap in registers and walks pixels, so a pixel costs its taps' LDS reads (shared by the lanes of the
// pixel) and 4 FMAs per tap; the pixel's channels leave as one contiguous run.  Same (r, q, ci) accumulation order.
// Rows m >= taps of the register arrays carry zero weights (they re-read tap 0), so the tap loop has no branch.
template <int MT>
__global__ __launch_bounds__(256) void conv_direct_fwd_rows_kernel(ConvGeom g, const float* __restrict__ x, const float* __restrict__ w,
                                                                    Epilogue e, int rows_per_band, int bands_per_image, int items, int lw,
                                                                    int qshift, int staged_full, DirectConvPlan plan) {
  extern __shared__ float fw_lds[];
  const int tid = threadIdx.x;
  const int M = g.kh * g.kw * g.cin;
  const int row_elems = lw * g.cin;
  const int quads = 1 << qshift;
  const int col = (tid & (quads - 1)) * 4;
  const int slot = tid >> qshift, slots = 256 >> qshift;
  f4v wr[MT];
  int off[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    off[m] = plan.off[m];
    const f4v zero = {0.f, 0.f, 0.f, 0.f};
    wr[m] = m < M ? *(const f4v*)(w + (int64_t)m * g.cout + col) : zero;
  }
  f4v bias = {0.f, 0.f, 0.f, 0.f};
  if (e.bias) {
#pragma unroll
    for (int i = 0; i < 4; ++i) bias[i] = e.bias[col + i];
  }
  int* origin = reinterpret_cast<int*>(fw_lds + staged_full);
  constexpr int U = 4;  // pixels per lane in flight
  for (int item = blockIdx.x; item < items; item += gridDim.x) {
    const int b = item / bands_per_image, band = item % bands_per_image;
    const int oh0 = band * rows_per_band;
    const int oh1 = oh0 + rows_per_band < g.ho ? oh0 + rows_per_band : g.ho;
    const int iy0 = oh0 * g.sh - g.pt;
    const int staged = ((oh1 - oh0 - 1) * g.sh + g.kh) * row_elems;
    const int P = (oh1 - oh0) * g.wo;
    __syncthreads();  // the previous item's readers are done with the staged rows
    for (int el = tid; el < staged; el += 256) {
      const int row = (int)div_by((uint32_t)el, plan.by_row_elems), rem = el - row * row_elems;
      const int px = (int)div_by((uint32_t)rem, plan.by_cin);
      const int iy = iy0 + row, ix = px - g.pl, ci = rem - px * g.cin;
      fw_lds[el] = ((unsigned)iy < (unsigned)g.h && (unsigned)ix < (unsigned)g.w) ? x[(((int64_t)b * g.h + iy) * g.w + ix) * g.cin + ci] : 0.f;
    }
    for (int p = tid; p < P; p += 256) {
      const int prow = (int)div_by((uint32_t)p, plan.by_wo);
      origin[p] = prow * g.sh * row_elems + (p - prow * g.wo) * g.sw * g.cin;
    }
    __syncthreads();
    float* outb = e.out + (((int64_t)b * g.ho + oh0) * g.wo) * e.ldo + col;
    int p0 = slot;
    for (; p0 + (U - 1) * slots < P; p0 += slots * U) fwd_rows_pixels<MT, U>(fw_lds, origin, off, wr, bias, e, outb, p0, slots);
    for (; p0 < P; p0 += slots) fwd_rows_pixels<MT, 1>(fw_lds, origin, off, wr, bias, e, outb, p0, slots);
  }
}

static bool conv_fwd_rows(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* w, const Epilogue& e, int* rc) {
  const int N = g.cout, K = g.kh * g.kw * g.cin;
  const int64_t pixels = (int64_t)g.n * g.ho * g.wo;
  if (g.cin > 4 || K > 18 || N % 4 != 0 || N > 256 || ((N / 4) & (N / 4 - 1)) != 0 || pixels < 2048) return false;
  if (e.ldo % 4 != 0 || !aligned16(e.out) || !aligned16(w)) return false;
  int qshift = 0;
  while ((4 << qshift) < N) ++qshift;
  const int lw = (g.wo - 1) * g.sw + g.kw;
  // a band holds at least ~4 pixels per lane, so staging its input rows is a small part of the work
  const int rows_per_band = (int)std::min<int64_t>(g.ho, std::max<int64_t>(1, ceil_div((int64_t)1024, (int64_t)(N / 4) * g.wo)));
  const int bands = (int)ceil_div((int64_t)g.ho, (int64_t)rows_per_band);
  const int64_t items = (int64_t)g.n * bands;
  const int64_t staged = (int64_t)((rows_per_band - 1) * g.sh + g.kh) * lw * g.cin;
  const int64_t lds_floats = staged + (int64_t)rows_per_band * g.wo;
  if (lds_floats * 4 > 48 * 1024 || items >= (int64_t)1 << 30) return false;
  const unsigned blocks = (unsigned)std::min<int64_t>(items, (int64_t)ctx->compute_units * 8);
  const DirectConvPlan plan = direct_conv_plan(g, lw);
  LaunchScope scope(ctx, "conv2d_forward_direct", (int)pixels, N, K);
#define SN_FWD_ROWS(MT)                                                                                                                  \
  hipLaunchKernelGGL((conv_direct_fwd_rows_kernel<MT>), dim3(blocks), dim3(256), (size_t)lds_floats * sizeof(float), ctx->stream, g, x, w, e, \
                     rows_per_band, bands, (int)items, lw, qshift, (int)staged, plan)
  if (K <= 9) SN_FWD_ROWS(9);
  else SN_FWD_ROWS(18);
#undef SN_FWD_ROWS
  *rc = hipGetLastError() == hipSuccess ? SN_OK : fail(SN_E_HIP, "conv2d_forward_direct: launch failed");
  return true;
}

int launch_conv_fwd(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* w, const Epilogue& e, float* ws, int64_t ws_elems) {
  const int M = g.n * g.ho * g.wo, N = g.cout, K = g.kh * g.kw * g.cin;
  int rows_rc = SN_OK;
  if (conv_fwd_rows(ctx, g, x, w, e, &rows_rc)) return rows_rc;
  if (g.cin <= 4 && K <= DIRECT_MAX_K && N % 4 == 0 && (size_t)K * N * sizeof(float) <= 48 * 1024 && e.ldo % 4 == 0 && aligned16(e.out) && M > 0) {
    const int64_t total = (int64_t)M * (N / 4);
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(total, 256), (int64_t)ctx->compute_units * 32);
    LaunchScope scope(ctx, "conv2d_forward_direct", M, N, K);
    hipLaunchKernelGGL(conv_direct_fwd_kernel, dim3(blocks), dim3(256), (size_t)K * N * sizeof(float), ctx->stream, g, x, w, e, M);
    SN_HIP(hipGetLastError());
    return SN_OK;
  }
  if (conv_ring_fwd_ok(g, x, w, e)) return launch_conv_ring_fwd(ctx, g, x, w, e);
  StdEpilogue ep{e};
  if (TapLoader::ok(x, g.n, g.h, g.w, g.cin, g.kh, g.kw) && FlatLoader<false>::ok(w, 1, g.cout, N, K)) {
    TapLoader al{x, M, g.ho, g.wo, g.sh, g.sw, -g.pt, -g.pl, 1, 1, g.h, g.w, g.cin, g.kh, g.kw};
    FlatLoader<false> bl{w, 1, g.cout, N};
    return launch_any<false>(ctx, "conv2d_forward", M, N, K, al, bl, ep, ws, ws_elems);
  }
  ConvFwdA al{x, g, M};
  StridedLoader<false> bl{w, 1, (int64_t)g.cout, N};  // filter [kh,kw,cin,cout] is a row-major [K, cout] matrix
  return launch_any<false>(ctx, "conv2d_forward", M, N, K, al, bl, ep, ws, ws_elems);
}

int launch_conv_dgrad(sn_ctx* ctx, const ConvGeom& g, const float* dy, const float* w, float* dx, float* ws, int64_t ws_elems) {
  const int M = g.n * g.h * g.w, N = g.cin, K = g.kh * g.kw * g.cout;
  Epilogue e;
  e.out = dx;
  e.ldo = g.cin;
  if (conv_ring_dgrad_ok(g, dy, w)) return launch_conv_ring_dgrad(ctx, g, dy, w, dx);
  StdEpilogue ep{e};
  if (g.sh == 1 && g.sw == 1 && TapLoader::ok(dy, g.n, g.ho, g.wo, g.cout, g.kh, g.kw) && aligned16(w) &&
      (int64_t)K * g.cin * 4 < FAST_SPAN) {
    TapLoader al{dy, M, g.h, g.w, 1, 1, g.pt, g.pl, -1, -1, g.ho, g.wo, g.cout, g.kh, g.kw};
    DgradWLoader bl{w, g.cin, g.cout};
    return launch_any<false>(ctx, "conv2d_input_gradient", M, N, K, al, bl, ep, ws, ws_elems);
  }
  ConvDgradA al{dy, g, M};
  ConvDgradB bl{w, g};
  return launch_any<false>(ctx, "conv2d_input_gradient", M, N, K, al, bl, ep, ws, ws_elems);
}

// Filter gradient of a first-layer convolution (a few input channels, at most 64 filters): M = kh*kw*cin is a few
// dozen rows, N = cout a few dozen columns and K = every output position of the batch, so the work is reading dy
// once.  Direct form: a workgroup takes a band of output rows of one image, keeps the input rows under it in LDS
// (zero-padded, so taps need no bounds checks), a group of `1 << cshift` >= cout lanes owns one output position at a
// time, each lane one filter, and keeps all M sums of that filter in registers.  The lanes' sums meet in LDS and
// leave as one partial [M][cout] per workgroup; gemm_small_reduce_kernel adds the partials in a fixed order.

// POOL: the convolution's output gradient is not in memory yet.  A 2 x 2 max pooling sits right above the layer and the
// kernel computes dy[position, filter] itself from the pooling's output gradient, the recorded first-maximum offsets and
// the convolution's saved output (for its activation gradient), exactly as pool2x2_bwd_kernel does: an element lies in at
// most 2 x 2 windows, whose contributions are added in (oh, ow) order, then act'(y) multiplies.  One launch and one pass
// over the tensor less for a first layer, whose input gradient nobody needs.
__device__ __forceinline__ float pool_grad_act_bwd(int act, float y, float dy, float param) {  // elementwise_kernels.hip: act_bwd
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

template <int MT, bool POOL>  // MT: upper bound of kh*kw*cin
__global__ __launch_bounds__(256) void conv_wgrad_direct_kernel(ConvGeom g, const float* __restrict__ x, const float* __restrict__ dy,
                                                                 float* __restrict__ partial, int rows_per_band, int bands_per_image,
                                                                 int items, int lw, int cshift, int staged_full, PoolGrad pg, DirectConvPlan plan) {
  extern __shared__ float wg_lds[];
  const int tid = threadIdx.x;
  const int M = g.kh * g.kw * g.cin;
  const int row_elems = lw * g.cin;
  int off[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) off[m] = plan.off[m];
  const FastDiv by_cv = plan.by_cv, by_wo = plan.by_wo;
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;
  const int lanes = 1 << cshift;
  const int c = tid & (lanes - 1);
  const int slot = tid >> cshift, slots = 256 >> cshift;
  const bool live = c < g.cout;
  const int cc = live ? c : 0;
  for (int item = blockIdx.x; item < items; item += gridDim.x) {
    const int b = item / bands_per_image, band = item % bands_per_image;
    const int oh0 = band * rows_per_band;
    const int oh1 = oh0 + rows_per_band < g.ho ? oh0 + rows_per_band : g.ho;
    const int iy0 = oh0 * g.sh - g.pt;
    const int staged = ((oh1 - oh0 - 1) * g.sh + g.kh) * row_elems;
    const int P = (oh1 - oh0) * g.wo;
    const float* dyb = dy + ((int64_t)b * g.ho + oh0) * g.wo * g.cout;
    constexpr int U = 16;  // positions per lane whose dy loads are in flight together
    int* origin = reinterpret_cast<int*>(wg_lds + staged_full);  // per position of the band: LDS offset of its top-left input element
    float* dcv = wg_lds + staged_full + rows_per_band * g.wo;    // POOL: the band's output gradient [P][cout]
    __syncthreads();  // the previous item's readers are done with the staged rows
    for (int e = tid; e < staged; e += 256) {
      const int row = (int)div_by((uint32_t)e, plan.by_row_elems), rem = e - row * row_elems;
      const int px = (int)div_by((uint32_t)rem, plan.by_cin);
      const int iy = iy0 + row, ix = px - g.pl, ci = rem - px * g.cin;
      wg_lds[e] = ((unsigned)iy < (unsigned)g.h && (unsigned)ix < (unsigned)g.w) ? x[(((int64_t)b * g.h + iy) * g.w + ix) * g.cin + ci] : 0.f;
    }
    for (int p = tid; p < P; p += 256) {  // once per position, not per lane
      const int prow = (int)div_by((uint32_t)p, by_wo);
      origin[p] = prow * g.sh * row_elems + (p - prow * g.wo) * g.sw * g.cin;
    }
    if constexpr (POOL) {
      // the band's output gradient [P][cout], four filters per thread: position (iy, ix) of the convolution's output = of the
      // pooling's input lies in the windows oh_lo + {0, 1} x ow_lo + {0, 1} (those that exist)
      // (index arithmetic is what this phase costs: divisions by the launch's constants are multiplications, those by the
      // pooling's stride shifts for strides 1 and 2, element offsets 32-bit)
      const int cv = g.cout >> 2;
      auto by_stride = [](int v, int st) { return st == 1 ? v : (st == 2 ? v >> 1 : v / st); };  // v >= 0
      const uint32_t img_y = (uint32_t)b * g.ho, img_p = (uint32_t)b * pg.ho;
      for (int e = tid; e < P * cv; e += 256) {
        const int p = (int)div_by((uint32_t)e, by_cv), ch = (e - p * cv) * 4;
        const int prow = (int)div_by((uint32_t)p, by_wo);
        const int iy = oh0 + prow, ix = p - prow * g.wo;
        int oh_lo = iy + pg.pt - 1;
        oh_lo = oh_lo <= 0 ? 0 : by_stride(oh_lo + pg.sh - 1, pg.sh);
        int oh_hi = by_stride(iy + pg.pt, pg.sh);
        if (oh_hi > pg.ho - 1) oh_hi = pg.ho - 1;
        int ow_lo = ix + pg.pl - 1;
        ow_lo = ow_lo <= 0 ? 0 : by_stride(ow_lo + pg.sw - 1, pg.sw);
        int ow_hi = by_stride(ix + pg.pl, pg.sw);
        if (ow_hi > pg.wo - 1) ow_hi = pg.wo - 1;
        const f4v yv = *(const f4v*)(pg.y + (((img_y + iy) * g.wo + ix) * g.cout + ch));
        uint32_t a4[4], want[4];
        f4v gk[4];
        bool on[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {  // windows that do not exist re-read the first element and are ignored
          const int oh = oh_lo + (k >> 1), ow = ow_lo + (k & 1);
          on[k] = oh <= oh_hi && ow <= ow_hi;
          const uint32_t o = on[k] ? ((img_p + oh) * pg.wo + ow) * g.cout + ch : (uint32_t)ch;
          want[k] = (uint32_t)((iy - (oh * pg.sh - pg.pt)) * 2 + (ix - (ow * pg.sw - pg.pl)));
          a4[k] = *(const uint32_t*)(pg.arg + o);
          gk[k] = *(const f4v*)(pg.dy + o);
        }
        f4v sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (!on[k]) continue;
          if ((a4[k] & 255u) == want[k]) sum[0] += gk[k][0];
          if (((a4[k] >> 8) & 255u) == want[k]) sum[1] += gk[k][1];
          if (((a4[k] >> 16) & 255u) == want[k]) sum[2] += gk[k][2];
          if ((a4[k] >> 24) == want[k]) sum[3] += gk[k][3];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) dcv[p * g.cout + ch + q] = pool_grad_act_bwd(pg.act, yv[q], sum[q], pg.act_param);
      }
    }
    __syncthreads();
    for (int p0 = slot; p0 < P; p0 += slots * U) {
      float d[U];
      int base[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = p0 + u * slots;
        const bool in = p < P;
        const int pp = in ? p : 0;
        float v;
        if constexpr (POOL) v = dcv[pp * g.cout + cc];  // formed below, once per band
        else v = dyb[(int64_t)pp * g.cout + cc];  // always a valid address: no branch around the load
        d[u] = (in && live) ? v : 0.f;
        base[u] = origin[pp];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int m = 0; m < MT; ++m)  // rows m >= M repeat tap 0 and are dropped at the end: no branch between the LDS reads
          acc[m] = __builtin_fmaf(wg_lds[base[u] + off[m]], d[u], acc[m]);
      }
    }
  }
  __syncthreads();
  // [slot][m][lane] -> one sum per (m, filter), slots added in order
#pragma unroll
  for (int m = 0; m < MT; ++m)
    if (m < M) wg_lds[(slot * M + m) * lanes + c] = acc[m];
  __syncthreads();
  const int outs = M * g.cout;
  for (int o = tid; o < outs; o += 256) {
    const int m = (int)div_by((uint32_t)o, plan.by_cout), co = o - m * g.cout;
    float t = 0.f;
    for (int sl = 0; sl < slots; ++sl) t += wg_lds[(sl * M + m) * lanes + co];
    partial[(int64_t)blockIdx.x * outs + o] = t;
  }
}

// true when launch_conv_wgrad takes the direct kernel for this layer (which can also stand in for a max pooling's backward
// pass above it: launch_conv_wgrad's `pool` argument)
bool conv_wgrad_is_direct(const sn_ctx* ctx, const ConvGeom& g, const float* ws, int64_t ws_elems, bool with_pool) {
  const int M = g.kh * g.kw * g.cin, N = g.cout;
  const int64_t K = (int64_t)g.n * g.ho * g.wo;
  if (!ws || g.cin > 4 || M > WGRAD_DIRECT_MAX_TAPS || N > 64 || K < SMALL_MIN_K) return false;
  const int64_t room = std::min<int64_t>((int64_t)4 * ctx->compute_units, ws_elems / ((int64_t)M * N));
  if (room < 32) return false;
  const int lw = (g.wo - 1) * g.sw + g.kw;
  const int rows_per_band = (int)std::min<int64_t>(g.ho, std::max<int64_t>(1, ceil_div((int64_t)g.n * g.ho, room)));
  const int bands = (int)ceil_div((int64_t)g.ho, (int64_t)rows_per_band);
  const int64_t staged = (int64_t)((rows_per_band - 1) * g.sh + g.kh) * lw * g.cin;
  const int64_t lds_floats = std::max<int64_t>(staged + (int64_t)rows_per_band * g.wo * (with_pool ? 1 + N : 1), (int64_t)256 * M);
  return lds_floats * 4 <= 48 * 1024 && (int64_t)g.n * bands < (int64_t)1 << 30 && (!with_pool || (N % 4 == 0 && (int64_t)g.n * g.ho * g.wo * N < ((int64_t)1 << 32)));  // (32-bit element offsets there)
}

static bool conv_wgrad_direct(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy, float* dw, float* ws, int64_t ws_elems, int* rc,
                              const PoolGrad* pool) {
  const int M = g.kh * g.kw * g.cin, N = g.cout;
  const int64_t K = (int64_t)g.n * g.ho * g.wo;
  if (!ws || g.cin > 4 || M > WGRAD_DIRECT_MAX_TAPS || N > 64 || K < SMALL_MIN_K) return false;
  const int64_t room = std::min<int64_t>((int64_t)4 * ctx->compute_units, ws_elems / ((int64_t)M * N));
  if (room < 32) return false;
  int cshift = 0;
  while ((1 << cshift) < N) ++cshift;
  const int lw = (g.wo - 1) * g.sw + g.kw;
  int rows_per_band = (int)std::min<int64_t>(g.ho, std::max<int64_t>(1, ceil_div((int64_t)g.n * g.ho, room)));
  const int bands = (int)ceil_div((int64_t)g.ho, (int64_t)rows_per_band);
  const int64_t items = (int64_t)g.n * bands;
  const int64_t staged = (int64_t)((rows_per_band - 1) * g.sh + g.kh) * lw * g.cin;
  const int64_t lds_floats = std::max<int64_t>(staged + (int64_t)rows_per_band * g.wo * (pool ? 1 + N : 1), (int64_t)256 * M);
  if (lds_floats * 4 > 48 * 1024 || items >= (int64_t)1 << 30) return false;
  const int parts = (int)std::min<int64_t>(items, room);
  {
    LaunchScope scope(ctx, pool ? "maxpool_backward_and_conv2d_filter_gradient_direct" : "conv2d_filter_gradient_direct", M, N, (int)K);
    const PoolGrad pg = pool ? *pool : PoolGrad{};
    const DirectConvPlan plan = direct_conv_plan(g, lw);
#define SN_WGRAD_DIRECT(MT)                                                                                                             \
  do {                                                                                                                                  \
    if (pool)                                                                                                                           \
      hipLaunchKernelGGL((conv_wgrad_direct_kernel<MT, true>), dim3((unsigned)parts), dim3(256), (size_t)lds_floats * sizeof(float),    \
                         ctx->stream, g, x, dy, ws, rows_per_band, bands, (int)items, lw, cshift, (int)staged, pg, plan);               \
    else                                                                                                                                \
      hipLaunchKernelGGL((conv_wgrad_direct_kernel<MT, false>), dim3((unsigned)parts), dim3(256), (size_t)lds_floats * sizeof(float),   \
                         ctx->stream, g, x, dy, ws, rows_per_band, bands, (int)items, lw, cshift, (int)staged, pg, plan);               \
  } while (0)
    if (M <= 9) SN_WGRAD_DIRECT(9);
    else if (M <= 18) SN_WGRAD_DIRECT(18);
    else SN_WGRAD_DIRECT(36);
#undef SN_WGRAD_DIRECT
  }
  if (ctx->defer && (M * N) % 4 == 0) {  // the caller's optimizer launch adds the partials
    *ctx->defer = DeferredReduce{2, ws, parts, M * N, dw};
    ctx->defer = nullptr;
    *rc = hipGetLastError() == hipSuccess ? SN_OK : fail(SN_E_HIP, "conv2d_filter_gradient_direct: launch failed");
    return true;
  }
  Epilogue e;
  e.out = dw;
  e.ldo = g.cout;
  StdEpilogue ep{e};
  LaunchScope scope(ctx, "small_output_reduce");
  hipLaunchKernelGGL((gemm_small_reduce_kernel<StdEpilogue>), dim3((unsigned)ceil_div(M * N, 4)), dim3(256), 0, ctx->stream, (const float*)ws,
                     parts, M, N, ep);
  *rc = hipGetLastError() == hipSuccess ? SN_OK : fail(SN_E_HIP, "conv2d_filter_gradient_direct: launch failed");
  return true;
}

int launch_conv_wgrad(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy, float* dw, float* ws, int64_t ws_elems,
                      const PoolGrad* pool) {
  const int M = g.kh * g.kw * g.cin, N = g.cout, K = g.n * g.ho * g.wo;
  int rc = SN_OK;
  if (conv_wgrad_direct(ctx, g, x, dy, dw, ws, ws_elems, &rc, pool)) return rc;
  SN_REQUIRE(pool == nullptr, "conv2d_filter_gradient: only the direct kernel takes a pooling's gradient (ask conv_wgrad_is_direct first)");
  if (ws && aligned16(ws) && conv_wgrad_taps_shape(ctx, g, x, dy) && conv_wgrad_taps_workspace(ctx, g) <= ws_elems) {
    // a tile per filter tap: a few dozen partial filters instead of the 64 x 64 tiling's hundreds
    int parts = 0;
    SN_TRY(launch_conv_wgrad_taps(ctx, g, x, dy, ws, ws_elems, &parts));
    const int64_t total = (int64_t)M * N;  // a multiple of 1024
    if (ctx->defer && total >= 4096) {  // a caller that applies the optimizer next takes the sum into that launch
      *ctx->defer = DeferredReduce{1, ws, parts, (int)total, dw};
      ctx->defer = nullptr;
      return SN_OK;
    }
    Epilogue e;
    e.out = dw;
    e.ldo = g.cout;
    StdEpilogue ep{e};
    LaunchScope scope(ctx, "splitk_reduce");
    const int64_t blocks = std::min<int64_t>(ceil_div(total / 4, 32), (int64_t)ctx->compute_units * 16);
    hipLaunchKernelGGL((splitk_reduce4_kernel<StdEpilogue>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (const float*)ws, parts, M, N, ep);
    SN_HIP(hipGetLastError());
    return SN_OK;
  }
  if (!(ws && small_parts(M, N, K, ctx->compute_units, ws_elems)) && WgradXLoader::ok(x, g) && FlatLoader<false>::ok(dy, 1, g.cout, N, K)) {
    const int interior = g.pt == 0 && g.pl == 0 && (g.ho - 1) * g.sh + g.kh <= g.h && (g.wo - 1) * g.sw + g.kw <= g.w;
    WgradXLoader al{x, g, M, interior};
    FlatLoader<false> bl{dy, 1, g.cout, N};
    Epilogue e;
    e.out = dw;
    e.ldo = g.cout;
    StdEpilogue ep{e};
    return launch_any<false>(ctx, "conv2d_filter_gradient", M, N, K, al, bl, ep, ws, ws_elems);
  }
  ConvWgradA al{x, g, M};
  StridedLoader<false> bl{dy, 1, (int64_t)g.cout, N};
  Epilogue e;
  e.out = dw;
  e.ldo = g.cout;
  StdEpilogue ep{e};
  return launch_any<false>(ctx, "conv2d_filter_gradient", M, N, K, al, bl, ep, ws, ws_elems);
}

// ---------------------------------------------------------------------------- LSTM
int launch_lstm_z(sn_ctx* ctx, const float* x, int t, int T, int F, const float* h_prev, int rows, int H, const LstmWeights& w,
                  float* z, float* ws, int64_t ws_elems, int gates) {
  LstmZA al{x, h_prev, rows, T, F, H, t};
  LstmZB bl{w, F, H, gates};
  LstmZEpilogue ep{z, {w.b[0], w.b[1], w.b[2], w.b[3]}, H, gates};
  return launch_any<false>(ctx, "lstm_gate_gemm", rows, gates * H, F + H, al, bl, ep, ws, ws_elems);
}

int launch_lstm_dh(sn_ctx* ctx, const float* dz, int rows, int H, const LstmWeights& w, float* dh_prev, float* ws, int64_t ws_elems,
                   int gates) {
  StridedLoader<true> al{dz, (int64_t)gates * H, 1, rows};
  LstmWT bl{{w.wr[0], w.wr[1], w.wr[2], w.wr[3]}, H, H, gates};
  Epilogue e;
  e.out = dh_prev;
  e.ldo = H;
  StdEpilogue ep{e};
  return launch_any<false>(ctx, "lstm_hidden_gradient", rows, H, gates * H, al, bl, ep, ws, ws_elems);
}

int launch_lstm_dx(sn_ctx* ctx, const float* dz, int rows, int H, int F, int t, int T, const LstmWeights& w, float* dx, float* ws,
                   int64_t ws_elems, int gates) {
  StridedLoader<true> al{dz, (int64_t)gates * H, 1, rows};
  LstmWT bl{{w.wk[0], w.wk[1], w.wk[2], w.wk[3]}, F, H, gates};
  DxScatterEpilogue ep{dx, T, F, t};
  return launch_any<false>(ctx, "lstm_input_gradient", rows, F, gates * H, al, bl, ep, ws, ws_elems);
}

int launch_lstm_wgrad_reduce(sn_ctx* ctx, const float* ws, int parts, int F, int H, int gates, const LstmGrads& g) {
  LstmWgradEpilogue ep{g, F, H};
  const int Mo = F + H + 1, No = gates * H;
  const int64_t total = (int64_t)Mo * No;
  LaunchScope scope(ctx, "splitk_reduce");
  if (total % 4 == 0) {
    const int64_t blocks = std::min<int64_t>(ceil_div(total / 4, 32), (int64_t)ctx->compute_units * 16);
    hipLaunchKernelGGL((splitk_reduce4_kernel<LstmWgradEpilogue>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, ws, parts, Mo, No, ep);
  } else {
    const int64_t blocks = std::min<int64_t>(ceil_div(total, 32), (int64_t)ctx->compute_units * 16);
    hipLaunchKernelGGL((splitk_reduce_kernel<LstmWgradEpilogue>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, ws, parts, Mo, No, ep);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_lstm_wgrad(sn_ctx* ctx, const float* x, const float* h_prev_all, const float* dz_all, int rows, int T, int F, int H,
                      const LstmGrads& g, float* ws, int64_t ws_elems, int gates) {
  const bool has_bias = g.b[0] != nullptr;
  if (ws && lstm_wgrad_rows_ok(ctx, x, h_prev_all, dz_all, rows, T, F, H, gates) &&
      lstm_wgrad_rows_workspace(ctx, rows, T, F, H, gates) <= ws_elems && aligned16(ws)) {
    // all F + H rows x 128 columns per workgroup, one k range each; then the ranges are added into the layer's tensors
    int ranges = 0;
    SN_TRY(launch_lstm_wgrad_rows(ctx, x, h_prev_all, dz_all, rows, T, F, H, gates, ws, ws_elems, &ranges));
    return launch_lstm_wgrad_reduce(ctx, ws, ranges, F, H, gates, g);
  }
  const int M = F + H + (has_bias ? 1 : 0);
  LstmWgradA al{x, h_prev_all, rows, T, F, H, M};
  StridedLoader<false> bl{dz_all, 1, (int64_t)gates * H, gates * H};
  LstmWgradEpilogue ep{g, F, H};
  return launch_any<false>(ctx, "lstm_weight_gradient", M, gates * H, T * rows, al, bl, ep, ws, ws_elems);
}

// ============================================================================ Dense onto a few units: backward
// A Dense layer from tens of thousands of features onto at most 16 units (a classifier head behind Flatten) with a
// batch of a few hundred rows: its gradients are memory-bound streams over X and dX (one read and one write of a
// [rows, features] tensor), with a launch that fills the chip along the feature axis.
constexpr int SKINNY_MAX_UNITS = 16, SKINNY_MIN_FEATURES = 2048, SKINNY_MAX_ROWS = 2048;

// dW[i, n] = sum_b X[b, i] dY[b, n] (math/alg/AllKernels.scala:382-388, the left operand's gradient of a matrix product
// seen from the weights), db[n] = sum_b dY[b, n] and, with DX, the layer's input gradient dX[b, i] = sum_n dY[b, n] W[i, n]
// (the right operand's side) in one launch on the matrix cores (v_mfma_f32_16x16x4_f32), without LDS: a wavefront owns
// 16 features and walks all rows.  dW tile [16 features][16 units] += A B with A[m = feature][k = row] = X[row, feature] and
// B[k = row][n = unit] = dY[row, unit]: lane (c = l % 16, g = l / 16) loads X[4 s + g, feature c] and dY[4 s + g, unit c]
// for step s, 32 steps in flight.  dX tile [16 rows][16 features] = A B with A[m = row][k = unit] = dY[row, unit] and
// B[k = unit][n = feature] = W[feature, unit], written while the rows of X are on their way.  The lanes of one
// wavefront together hold every value of dY, so the bias gradient is their sum (workgroup 0, wavefront 0).
// An accumulator value v of lane (c, g) is element [4 g + v][c] of its tile.
template <bool DX>
__global__ __launch_bounds__(256) void dense_skinny_grad_mfma_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                                      float* __restrict__ dw, float* __restrict__ db, int rows, int in_f,
                                                                      int out_f, const float* __restrict__ w, float* __restrict__ dx) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int i0 = (blockIdx.x * 4 + wave) * 16;
  if (i0 >= in_f) return;
  const int feat = i0 + c;
  const bool live = feat < in_f;
  const bool unit = c < out_f;
  // a lane's element of row b lies at the tensor's base (the same for all lanes) + a 32-bit byte offset: one register per
  // address instead of two (the host has checked that the tensors are below 4 GiB)
  const uint32_t xlane = (uint32_t)(live ? feat : 0) * 4u, dlane = (uint32_t)(unit ? c : 0) * 4u;
  const uint32_t xrow = (uint32_t)in_f * 4u, drow = (uint32_t)out_f * 4u;
  auto x_at = [&](int b) { return *(const float*)((const char*)x + (xlane + (uint32_t)b * xrow)); };
  auto dy_at = [&](int b) { return *(const float*)((const char*)dy + (dlane + (uint32_t)b * drow)); };
  constexpr int S = 32;  // steps (of 4 rows) in flight
  const int steps = (rows + 3) >> 2;
  float xv[S], dv[S];
#pragma unroll
  for (int u = 0; u < S; ++u) {
    const int b = 4 * u + g;
    xv[u] = (live && b < rows) ? x_at(b) : 0.f;
  }
#pragma unroll
  for (int u = 0; u < S; ++u) {
    const int b = 4 * u + g;
    dv[u] = (unit && b < rows) ? dy_at(b) : 0.f;
  }
  if constexpr (DX) {
    const int nq = (out_f + 3) >> 2;
    float wk[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) wk[q] = (live && 4 * q + g < out_f) ? w[(int64_t)feat * out_f + 4 * q + g] : 0.f;
    for (int r0 = 0; r0 < rows; r0 += 16) {
      f4v t = {0.f, 0.f, 0.f, 0.f};
      const int row = r0 + c;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (q < nq) {
          const float a = (row < rows && 4 * q + g < out_f) ? dy[(int64_t)row * out_f + 4 * q + g] : 0.f;
          t = __builtin_amdgcn_mfma_f32_16x16x4f32(a, wk[q], t, 0, 0, 0);
        }
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int b = r0 + 4 * g + v;
        if (live && b < rows) *(float*)((char*)dx + (xlane + (uint32_t)b * xrow)) = t[v];
      }
    }
  }
  f4v acc = {0.f, 0.f, 0.f, 0.f};
  float bsum = 0.f;
  for (int s0 = 0; s0 < steps; s0 += S) {
    if (s0 != 0) {
#pragma unroll
      for (int u = 0; u < S; ++u) {
        const int b = 4 * (s0 + u) + g;
        xv[u] = (live && b < rows) ? x_at(b) : 0.f;
        dv[u] = (unit && b < rows) ? dy_at(b) : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < S; ++u) {
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u], dv[u], acc, 0, 0, 0);
      bsum += dv[u];
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int f = i0 + 4 * g + v;
    if (unit && f < in_f) dw[(int64_t)f * out_f + c] = acc[v];
  }
  if (db && blockIdx.x == 0 && wave == 0) {  // rows 4 s + g of unit c were this lane's: the four row groups meet by shuffles
    const float s1 = __shfl(bsum, c + 16, 64), s2 = __shfl(bsum, c + 32, 64), s3 = __shfl(bsum, c + 48, 64);
    if (g == 0 && unit) db[c] = ((bsum + s1) + s2) + s3;
  }
}

bool dense_skinny_shape(int rows, int in_f, int out_f) {
  return rows >= 4 && rows <= SKINNY_MAX_ROWS && out_f >= 1 && out_f <= SKINNY_MAX_UNITS && in_f >= SKINNY_MIN_FEATURES &&
         (int64_t)rows * in_f < ((int64_t)1 << 30);
}

int launch_dense_skinny_dw(sn_ctx* ctx, const float* x, const float* dy, float* dw, float* db, int rows, int in_f, int out_f, const float* w,
                           float* dx) {
  SN_REQUIRE(dense_skinny_shape(rows, in_f, out_f), "dense_weight_gradient_rows: shape outside the kernel's range");
  SN_REQUIRE((w != nullptr) == (dx != nullptr), "dense_weight_gradient_rows: the input gradient needs the weights and a place to go");
  const unsigned blocks = (unsigned)ceil_div(in_f, 64);
  LaunchScope scope(ctx, dx ? "dense_weight_and_input_gradient_rows" : "dense_weight_gradient_rows", in_f, out_f, rows);
  if (dx)
    hipLaunchKernelGGL((dense_skinny_grad_mfma_kernel<true>), dim3(blocks), dim3(256), 0, ctx->stream, x, dy, dw, db, rows, in_f, out_f, w, dx);
  else
    hipLaunchKernelGGL((dense_skinny_grad_mfma_kernel<false>), dim3(blocks), dim3(256), 0, ctx->stream, x, dy, dw, db, rows, in_f, out_f, w, dx);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// The same layer forward for a batch of at most SKINNY_FWD_MAX_ROWS rows: Y = X W is 4 B of X per 2 out_f flops.  A workgroup
// owns SKINNY_FWD_CHUNK consecutive features: its wavefronts fetch their rows of that chunk in one go (a lane takes two
// neighbouring features, so a wavefront reads 512 contiguous bytes per row, all rows in flight), the chunk turns in
// LDS ([row][129]: rows on different banks), then thread (row pair, unit quad) adds its 128 products per output in feature order and the
// workgroup leaves one partial [rows][out_f]; gemm_small_reduce_kernel adds the partials in a fixed order and applies the
// bias and the activation.
constexpr int SKINNY_FWD_CHUNK = 64, SKINNY_FWD_MAX_ROWS = 112, SKINNY_FWD_ROWS_PER_WAVE = SKINNY_FWD_MAX_ROWS / 4;

template <int NQ>
__global__ __launch_bounds__(256) void dense_skinny_fwd_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ partial,
                                                                int rows, int in_f, int out_f) {
  constexpr int KC = SKINNY_FWD_CHUNK, PITCH = KC + 1, R = SKINNY_FWD_ROWS_PER_WAVE;
  extern __shared__ __attribute__((aligned(16))) float skinny_fwd_lds[];
  float* xs = skinny_fwd_lds;                                  // [rows][PITCH]
  f4v* wsm = reinterpret_cast<f4v*>(skinny_fwd_lds + ((rows * PITCH + 3) & ~3));  // [KC][NQ]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i0 = blockIdx.x * KC;
  constexpr int FL = KC / 64;     // features per lane: 1 or 2
  const int fa = i0 + FL * lane;  // this lane's first feature
  // whole chunks of rows that start on 8-byte boundaries take 8-byte loads without a branch (rows past the batch re-read the last row)
  const bool whole = FL == 2 && i0 + KC <= in_f && (in_f & 1) == 0 && (reinterpret_cast<uintptr_t>(x) & 7) == 0;
  float2 xv[R];
  if (FL == 1) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int b = wave + 4 * u < rows ? wave + 4 * u : rows - 1;
      xv[u].x = fa < in_f ? x[(int64_t)b * in_f + fa] : 0.f;
      xv[u].y = 0.f;
    }
  } else if (whole) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int b = wave + 4 * u < rows ? wave + 4 * u : rows - 1;
      xv[u] = *reinterpret_cast<const float2*>(x + (int64_t)b * in_f + fa);
    }
  } else {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int b = wave + 4 * u < rows ? wave + 4 * u : rows - 1;
      const float* rp = x + (int64_t)b * in_f;
      xv[u].x = fa < in_f ? rp[fa] : 0.f;
      xv[u].y = fa + 1 < in_f ? rp[fa + 1] : 0.f;
    }
  }
  {  // the chunk's weight rows, units padded to quads with zeros; features past in_f are zero rows
    float* wflat = reinterpret_cast<float*>(wsm);
    constexpr int total = KC * NQ * 4;
    for (int base = 0; base < total; base += 256 * 8) {  // 8 loads per thread are issued before any of them is stored
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = base + u * 256 + (int)threadIdx.x;
        const int k = e / (NQ * 4), n = e % (NQ * 4);
        v[u] = (e < total && i0 + k < in_f && n < out_f) ? w[(int64_t)(i0 + k) * out_f + n] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = base + u * 256 + (int)threadIdx.x;
        if (e < total) wflat[e] = v[u];
      }
    }
  }
#pragma unroll
  for (int u = 0; u < R; ++u) {
    const int b = wave + 4 * u;
    if (b < rows) {
      xs[b * PITCH + FL * lane] = xv[u].x;
      if (FL == 2) xs[b * PITCH + FL * lane + 1] = xv[u].y;
    }
  }
  __syncthreads();
  // thread (row pair, unit quad): a weight quad read from LDS serves both rows; at most 56 pairs x 4 quads = 224 threads
  float* out = partial + (int64_t)blockIdx.x * rows * out_f;
  const int item = threadIdx.x;
  if (item < ((rows + 1) / 2) * NQ) {
    const int b = (item / NQ) * 2, q = item % NQ;
    const bool second = b + 1 < rows;
    const float* xr0 = xs + b * PITCH;
    const float* xr1 = xs + (second ? b + 1 : b) * PITCH;
    f4v acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 16
    for (int k = 0; k < KC; ++k) {
      const float x0 = xr0[k], x1 = xr1[k];
      const f4v wk = wsm[k * NQ + q];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        acc0[c] = __builtin_fmaf(x0, wk[c], acc0[c]);
        acc1[c] = __builtin_fmaf(x1, wk[c], acc1[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (q * 4 + c < out_f) {
        out[b * out_f + q * 4 + c] = acc0[c];
        if (second) out[(b + 1) * out_f + q * 4 + c] = acc1[c];
      }
    }
  }
}

int64_t dense_skinny_fwd_workspace(int rows, int in_f, int out_f) { return ceil_div(in_f, SKINNY_FWD_CHUNK) * rows * out_f; }

static size_t skinny_fwd_lds_bytes(int rows, int out_f) {
  return ((size_t)((rows * (SKINNY_FWD_CHUNK + 1) + 3) & ~3) + (size_t)SKINNY_FWD_CHUNK * ((out_f + 3) / 4) * 4) * sizeof(float);
}

bool dense_skinny_fwd_shape(int rows, int in_f, int out_f, int64_t ws_elems) {
  return rows >= 1 && rows <= SKINNY_FWD_MAX_ROWS && out_f >= 1 && out_f <= SKINNY_MAX_UNITS && in_f >= SKINNY_MIN_FEATURES &&
         skinny_fwd_lds_bytes(rows, out_f) <= 64 * 1024 && dense_skinny_fwd_workspace(rows, in_f, out_f) <= ws_elems;
}

int launch_dense_skinny_fwd(sn_ctx* ctx, const float* x, const float* w, const Epilogue& e, int rows, int in_f, int out_f, float* ws,
                            int64_t ws_elems, int* parts_left) {
  SN_REQUIRE(ws && dense_skinny_fwd_shape(rows, in_f, out_f, ws_elems), "dense_forward_rows: shape outside the kernel's range");
  const int nq = (out_f + 3) / 4;
  const int parts = (int)ceil_div(in_f, SKINNY_FWD_CHUNK);
  const size_t lds = skinny_fwd_lds_bytes(rows, out_f);
  {
    LaunchScope scope(ctx, "dense_forward_rows", rows, out_f, in_f);
#define SN_SKINNY_FWD(NQ) \
  hipLaunchKernelGGL((dense_skinny_fwd_kernel<NQ>), dim3((unsigned)parts), dim3(256), lds, ctx->stream, x, w, ws, rows, in_f, out_f)
    switch (nq) {
      case 1: SN_SKINNY_FWD(1); break;
      case 2: SN_SKINNY_FWD(2); break;
      case 3: SN_SKINNY_FWD(3); break;
      default: SN_SKINNY_FWD(4); break;
    }
#undef SN_SKINNY_FWD
  }
  if (parts_left) {  // the caller's next launch adds the partial sums itself
    *parts_left = parts;
    SN_HIP(hipGetLastError());
    return SN_OK;
  }
  StdEpilogue ep{e};
  LaunchScope scope(ctx, "small_output_reduce");
  hipLaunchKernelGGL((gemm_small_reduce_kernel<StdEpilogue>), dim3((unsigned)ceil_div(rows * out_f, 4)), dim3(256), 0, ctx->stream,
                     (const float*)ws, parts, rows, out_f, ep);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// ============================================================================ Dense onto a few units from a short row
// A Dense(1..4) head behind a recurrent layer (512 x 256 -> 1): as GEMMs its three products are a split-K launch plus a
// reduction launch each, every one of them at the floor of what a launch costs.  Here the forward pass is one launch (a
// wavefront per row: 64 lanes walk the row, a butterfly adds them in a fixed order, lane 0 applies bias and activation)
// and the backward pass two: a workgroup takes 16 rows, turns dY into dZ = act'(Y) dY itself, writes dX = dZ W^T
// (AllKernels.scala:382-388) and leaves its share of dW = X^T dZ and db as one partial [in_f + 1][out_f];
// gemm_small_reduce_kernel adds the partials in a fixed order.
constexpr int TINY_MAX_UNITS = 4, TINY_MAX_FEATURES = 1024, TINY_MIN_FEATURES = 16, TINY_ROWS = 16, TINY_MAX_ROWS = 16384;

bool dense_tiny_shape(int rows, int in_f, int out_f, int64_t ws_elems) {
  return rows >= 1 && rows <= TINY_MAX_ROWS && out_f >= 1 && out_f <= TINY_MAX_UNITS && in_f >= TINY_MIN_FEATURES && in_f <= TINY_MAX_FEATURES &&
         ceil_div(rows, TINY_ROWS) * (int64_t)(in_f + 1) * out_f <= ws_elems;
}

template <int N>
__global__ __launch_bounds__(256) void dense_tiny_fwd_kernel(const float* __restrict__ x, const float* __restrict__ w, StdEpilogue ep, int rows,
                                                             int in_f) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float s[N];
#pragma unroll
  for (int n = 0; n < N; ++n) s[n] = 0.f;
  const float* xr = x + (int64_t)row * in_f;
  for (int i = lane; i < in_f; i += 64) {
    const float xv = xr[i];
#pragma unroll
    for (int n = 0; n < N; ++n) s[n] = __builtin_fmaf(xv, w[i * N + n], s[n]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
#pragma unroll
    for (int n = 0; n < N; ++n) s[n] += __shfl_xor(s[n], off, 64);
  if (lane == 0) {
#pragma unroll
    for (int n = 0; n < N; ++n) ep.store(row, n, s[n]);
  }
}

// the activation's gradient from its output (AllKernels.scala:297-302, 397-404, 414-420)
__device__ __forceinline__ float tiny_act_bwd(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

template <int N>
__global__ __launch_bounds__(256) void dense_tiny_bwd_kernel(const float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ dy,
                                                             const float* __restrict__ w, float* __restrict__ dx, float* __restrict__ partial,
                                                             int rows, int in_f, int act, float act_param, int with_bias) {
  __shared__ float dzs[TINY_ROWS][N];
  const int tid = threadIdx.x, r0 = blockIdx.x * TINY_ROWS, nr = min(TINY_ROWS, rows - r0);
  if (tid < TINY_ROWS * N) {
    const int r = tid / N, n = tid % N;
    const int64_t o = (int64_t)(r0 + r) * N + n;
    dzs[r][n] = r < nr ? tiny_act_bwd(act, y[o], dy[o], act_param) : 0.f;  // rows past the batch add nothing
  }
  __syncthreads();
  float* part = partial + (int64_t)blockIdx.x * (in_f + with_bias) * N;
  for (int i = tid; i < in_f; i += 256) {
    float wr[N], acc[N], xv[TINY_ROWS];
#pragma unroll
    for (int n = 0; n < N; ++n) {
      wr[n] = w[i * N + n];
      acc[n] = 0.f;
    }
#pragma unroll
    for (int r = 0; r < TINY_ROWS; ++r) xv[r] = x[(int64_t)(r0 + (r < nr ? r : nr - 1)) * in_f + i];  // every load in flight
#pragma unroll
    for (int r = 0; r < TINY_ROWS; ++r) {
      float s = 0.f;
#pragma unroll
      for (int n = 0; n < N; ++n) {
        acc[n] = __builtin_fmaf(xv[r], dzs[r][n], acc[n]);
        s = __builtin_fmaf(dzs[r][n], wr[n], s);
      }
      if (dx && r < nr) dx[(int64_t)(r0 + r) * in_f + i] = s;
    }
#pragma unroll
    for (int n = 0; n < N; ++n) part[i * N + n] = acc[n];
  }
  if (with_bias && tid < N) {
    float s = 0.f;
    for (int r = 0; r < TINY_ROWS; ++r) s += dzs[r][tid];
    part[in_f * N + tid] = s;
  }
}

int launch_dense_tiny_fwd(sn_ctx* ctx, const float* x, const float* w, const Epilogue& e, int rows, int in_f, int out_f) {
  SN_REQUIRE(dense_tiny_shape(rows, in_f, out_f, (int64_t)1 << 40), "dense_forward_row_dots: shape outside the kernel's range");
  StdEpilogue ep{e};
  LaunchScope scope(ctx, "dense_forward_row_dots", rows, out_f, in_f);
  const unsigned blocks = (unsigned)ceil_div(rows, 4);
#define SN_TINY_FWD(N) hipLaunchKernelGGL((dense_tiny_fwd_kernel<N>), dim3(blocks), dim3(256), 0, ctx->stream, x, w, ep, rows, in_f)
  switch (out_f) {
    case 1: SN_TINY_FWD(1); break;
    case 2: SN_TINY_FWD(2); break;
    case 3: SN_TINY_FWD(3); break;
    default: SN_TINY_FWD(4); break;
  }
#undef SN_TINY_FWD
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_dense_tiny_bwd(sn_ctx* ctx, const float* x, const float* y, const float* dy, const float* w, float* dx, float* dw, float* db, int rows,
                          int in_f, int out_f, int act, float act_param, float* ws, int64_t ws_elems) {
  SN_REQUIRE(ws && dense_tiny_shape(rows, in_f, out_f, ws_elems), "dense_backward_rows16: shape outside the kernel's range");
  const int parts = (int)ceil_div(rows, TINY_ROWS), with_bias = db ? 1 : 0;
  {
    LaunchScope scope(ctx, "dense_backward_rows16", rows, in_f, out_f);
#define SN_TINY_BWD(N)                                                                                                                \
  hipLaunchKernelGGL((dense_tiny_bwd_kernel<N>), dim3((unsigned)parts), dim3(256), 0, ctx->stream, x, y, dy, w, dx, ws, rows, in_f, act, \
                     act_param, with_bias)
    switch (out_f) {
      case 1: SN_TINY_BWD(1); break;
      case 2: SN_TINY_BWD(2); break;
      case 3: SN_TINY_BWD(3); break;
      default: SN_TINY_BWD(4); break;
    }
#undef SN_TINY_BWD
  }
  Epilogue e;
  e.out = dw; e.ldo = out_f;
  if (db) {
    e.row_index = in_f;
    e.row_out = db;
  }
  StdEpilogue ep{e};
  LaunchScope scope(ctx, "small_output_reduce");
  const int M = in_f + with_bias;
  hipLaunchKernelGGL((gemm_small_reduce_kernel<StdEpilogue>), dim3((unsigned)ceil_div(M * out_f, 4)), dim3(256), 0, ctx->stream, (const float*)ws,
                     parts, M, out_f, ep);
  SN_HIP(hipGetLastError());
  return SN_OK;
}


}  // namespace sn
