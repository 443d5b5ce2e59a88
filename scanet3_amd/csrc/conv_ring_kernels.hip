// Conv2D forward and input gradient as implicit fp32 GEMMs whose operand tiles travel HBM/L2 -> LDS with LDS-direct
// 16-byte loads into two alternating LDS buffers (gfx950).
//
//   C[M, N] = A[M, K] * B[K, N],  row m = a position (b, iy, ix) of the iteration space, k = (tap r, tap q, channel)
//   with the channel fastest and the channel count a multiple of 32, so that a K stage of 32 lies inside one tap:
//     A(m, k) = src[b, iy*sy + oy + r*ty, ix*sx + ox + q*tx, channel]   (0 outside the source image)
//   forward:        src = x,  (sy, sx) = strides, (oy, ox) = -padding, (ty, tx) = (+1, +1), B = the filter as [K][N]
//   input gradient: src = dy, unit strides, (oy, ox) = +padding, (ty, tx) = (-1, -1), B(k, n) = w[tap, n, channel]
//
// Workgroup = 4 wavefronts, each owning one 32 x 32 accumulator tile (v_mfma_f32_32x32x2_f32): block tile 64 x 64
// (2 x 2 wavefronts), or 64 x 32 with two wavefronts per tile that split every stage's k-values.  A stage is 32 k-values: every tile row is 128 bytes = eight 16-byte
// chunks, stored at chunk position (chunk ^ (row & 7)) so that the 16-byte fragment reads are conflict free.  Lanes
// with l/32 = 0 read chunks 0, 2, 4, 6 and lanes with l/32 = 1 chunks 1, 3, 5, 7: MFMA t of chunk pair j multiplies
// k = 8j + t and k = 8j + 4 + t, one 16-byte LDS read per operand for four MFMAs.  An operand that is not
// K-contiguous in memory (the forward filter, [K][N]) is staged as it lies, four k rows per load, and read one value
// per MFMA.  Rows outside the matrix and taps outside the image are loads with an out-of-range offset: the buffer
// descriptor's range check answers them with zeros and no memory traffic.
// One barrier per stage: it publishes stage s and frees the buffer stage s+1 is then loaded into.  (A third buffer and a
// prefetch distance of two stages were measured: no faster, and the smaller footprint lets four workgroups share a CU,
// which for LeNet's 827 tiles is the difference between one round of workgroups and two.)
#include "common.hpp"

namespace sn {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int RK = 32;                     // k-values per stage
constexpr int STAGES = 2;
constexpr uint32_t OOB = 0x80000000u;      // beyond any operand (tensors are checked to be < 2 GiB)
constexpr int BO_BLOCK = 1024 + 128;       // bytes between the 4-row blocks of an outer-contiguous B stage

struct RingArgs {
  const float* src;
  uint32_t src_bytes;
  int M, ih, iw;            // iteration space: rows m = (b, iy, ix)
  int sy, sx, oy, ox, ty, tx;
  int H, W, C;              // source image
  int kh, kw;
  const float* b;
  uint32_t b_bytes;
  int N;
  int b_tap_stride, b_n_stride;  // K-contiguous B: element (n, tap, channel) at tap * b_tap_stride + n * b_n_stride + channel
  Epilogue ep;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

template <int ACT>
__device__ __forceinline__ float act_const(float v, float param) {
  if constexpr (ACT == SN_ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
  else if constexpr (ACT == SN_ACT_TANH) return tanhf(v);
  else if constexpr (ACT == SN_ACT_RELU) return fmaxf(param, v);
  else return v;
}

// A lane's 16 values of one 32x32 tile: column n, rows row0 + 8*(v/4) + v%4
template <int ACT>
__device__ __forceinline__ void store_tile(const Epilogue& e, int row0, int n, const f16v& acc, int M) {
  const float b = e.bias ? e.bias[n] : 0.f;
  float* out = e.out + (int64_t)row0 * e.ldo + n;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int dr = (k >> 2) * 8 + (k & 3);
    if (row0 + dr < M) out[(int64_t)dr * e.ldo] = act_const<ACT>(e.bias ? acc[k] + b : acc[k], e.act_param);
  }
}

// s_waitcnt immediate: vmcnt = N, the other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt out of range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// WAVES_M x WAVES_N wavefronts of one 32 x 32 tile each.  B_KC: B is K-contiguous in memory.  ACT: the epilogue's
// activation, a compile-time constant so that the kernel carries one store sequence only.
// WAVES_K = 2: two wavefronts per tile, each multiplying one half of every stage's 32 k-values (chunk pairs 0-1 and
// 2-3); the second hands its sums over through LDS at the end.  Twice the wavefronts per SIMD for the same matrix work:
// a wavefront's chain per stage (wait, barrier, fragment reads, MFMAs) gets shorter against the matrix cores' time.
template <int WAVES_M, int WAVES_N, bool B_KC, int ACT, int WAVES_K = 1>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * WAVES_K) void conv_ring_kernel(RingArgs a) {
  constexpr int NT = WAVES_M * WAVES_N, NW = NT * WAVES_K, BM = 32 * WAVES_M, BN = 32 * WAVES_N, NJ = 4 / WAVES_K;
  static_assert(WAVES_K == 1 || WAVES_K == 2, "one or two wavefronts per tile");
  constexpr int A_STAGE = BM * 128;                                  // bytes
  constexpr int B_STAGE = B_KC ? BN * 128 : (RK / 4) * BO_BLOCK;
  constexpr int A_ISSUES = BM / 8 / NW;                              // 1 KiB loads per wavefront and stage
  constexpr int B_ISSUES_ALL = B_KC ? BN / 8 : RK / 4;               // per workgroup
  constexpr int B_ISSUES = B_ISSUES_ALL / NW;                        // per wavefront
  static_assert(B_KC || BN == 64, "the outer-contiguous B stage is laid out for 64 columns");
  static_assert(B_ISSUES_ALL % NW == 0 && (BM / 8) % NW == 0, "every wavefront issues the same number of loads per stage");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* sA = smem;                       // [STAGES][A_STAGE]
  char* sB = smem + STAGES * A_STAGE;    // [STAGES][B_STAGE]

  // Consecutive workgroup ids land on different XCDs (8, each with its own L2): give every XCD a contiguous run of row
  // tiles, whose gathers overlap in the source image.
  const int tiles = a.tiles_m * a.tiles_n, per_xcd = (tiles + 7) >> 3;
  const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || tile >= tiles) return;
  const int tm = tile / a.tiles_n, tn = tile - tm * a.tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(a.src, a.src_bytes), rsB = make_rsrc(a.b, a.b_bytes);

  // ---- per-lane part of the A gather: issue i of this wavefront fills tile rows (wave * A_ISSUES + i) * 8 + lane / 8.
  // One division per lane; the following issues' rows lie 8 further on and are reached by carries.
  uint32_t abase[A_ISSUES], amask[A_ISSUES];
  {
    const int row0 = wave * A_ISSUES * 8 + (lane >> 3);
    int m = m0 + row0;
    int ix = m % a.iw, t = m / a.iw, iy = t % a.ih, b = t / a.ih;
    const uint32_t chunk = (uint32_t)((lane & 7) ^ (row0 & 7)) * 16u;  // rows 8 apart share row & 7
#pragma unroll
    for (int i = 0; i < A_ISSUES; ++i) {
      const int y0 = iy * a.sy + a.oy, x0 = ix * a.sx + a.ox;
      abase[i] = (uint32_t)(((b * a.H + y0) * a.W + x0) * a.C) * 4u + chunk;
      uint32_t cols = 0, mask = 0;
      for (int q = 0; q < a.kw; ++q) cols |= ((unsigned)(x0 + q * a.tx) < (unsigned)a.W ? 1u : 0u) << q;
      for (int r = 0; r < a.kh; ++r)
        if ((unsigned)(y0 + r * a.ty) < (unsigned)a.H) mask |= cols << (r * a.kw);
      amask[i] = m < a.M ? mask : 0u;
      m += 8;
      ix += 8;
      while (ix >= a.iw) {
        ix -= a.iw;
        if (++iy == a.ih) { iy = 0; ++b; }
      }
    }
  }
  // ---- per-lane part of the B loads
  uint32_t bbase[B_ISSUES];
#pragma unroll
  for (int i = 0; i < B_ISSUES; ++i) {
    const int q = wave * B_ISSUES + i;
    if constexpr (B_KC) {
      const int row = q * 8 + (lane >> 3), n = n0 + row;
      bbase[i] = n < a.N ? (uint32_t)(n * a.b_n_stride) * 4u + (uint32_t)((lane & 7) ^ (row & 7)) * 16u : OOB;
    } else {  // four k rows of BN floats per issue: lane -> (k row lane / 16, 4 columns lane % 16)
      const int n = n0 + (lane & 15) * 4;
      bbase[i] = n < a.N ? (uint32_t)((q * 4 + (lane >> 4)) * a.N + n) * 4u : OOB;
    }
  }
  const int cpt = a.C / RK;               // stages per tap
  const int nk = a.kh * a.kw * cpt;
  // the stage about to be loaded: tap (r, q) = rq, channel offset c0; everything else follows by additions
  int ld_rq = 0, ld_q = 0, ld_c = 0;
  uint32_t ld_tap_a = 0;                  // byte offset of tap (r, q), channel 0 relative to (y0, x0, 0) in the source
  uint32_t ld_k_b = 0;                    // byte offset of the stage inside B
  const uint32_t a_step_q = (uint32_t)(a.tx * a.C) * 4u, a_step_r = (uint32_t)((a.ty * a.W - a.kw * a.tx) * a.C) * 4u;
  const uint32_t b_step = B_KC ? RK * 4u : (uint32_t)(RK * a.N) * 4u;
  const uint32_t b_step_tap = B_KC ? (uint32_t)(a.b_tap_stride - a.C) * 4u : 0u;  // on top of the cpt channel steps
  auto issue_next = [&](int buf) {
    const uint32_t ta = ld_tap_a + (uint32_t)ld_c * 4u;
#pragma unroll
    for (int i = 0; i < A_ISSUES; ++i) {
      const uint32_t off = ((amask[i] >> ld_rq) & 1u) ? abase[i] + ta : OOB;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_ptr)(sA + buf * A_STAGE + (wave * A_ISSUES + i) * 1024), 16, (int)off, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < B_ISSUES; ++i) {
      const int qq = wave * B_ISSUES + i;
      const uint32_t off = bbase[i] == OOB ? OOB : bbase[i] + ld_k_b;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_ptr)(sB + buf * B_STAGE + qq * (B_KC ? 1024 : BO_BLOCK)), 16, (int)off, 0, 0, 0);
    }
    ld_c += RK;
    ld_k_b += b_step;
    if (ld_c == a.C) {  // next tap
      ld_c = 0;
      ++ld_rq;
      ld_k_b += b_step_tap;
      ld_tap_a += a_step_q;
      if (++ld_q == a.kw) { ld_q = 0; ld_tap_a += a_step_r; }
    }
  };

  f16v acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  const int kgrp = wave / NT, wtile = wave - kgrp * NT;
  const int wm = (wtile / WAVES_N) * 32, wn = (wtile % WAVES_N) * 32;  // (the barrier below is a no-op cost for one wavefront)
  const int arow = wm + l32, brow = wn + l32;
  const int aoff = arow * 128, asw = arow & 7;
  const int boff = brow * 128, bsw = brow & 7;

  // LDS byte addresses of this lane's fragments inside a stage (the chunk swizzle folded in)
  typedef __attribute__((address_space(3))) char lds_char;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_char*)smem;
  uint32_t a_at[NJ], b_at[NJ];
#pragma unroll
  for (int jj = 0; jj < NJ; ++jj) {
    const int j = kgrp * NJ + jj;
    a_at[jj] = lds0 + (uint32_t)(aoff + (((2 * j + lhi) ^ asw) << 4));
    b_at[jj] = lds0 + (uint32_t)(STAGES * A_STAGE) + (B_KC ? (uint32_t)(boff + (((2 * j + lhi) ^ bsw) << 4)) : (uint32_t)((2 * j + lhi) * BO_BLOCK + brow * 4));
  }

  // Two buffers, one barrier per stage.  The barrier at the top of stage s says two things: everybody's loads of stage s
  // have landed (each wavefront waits for its own first), and everybody has finished reading stage s - 1, whose buffer
  // the loads of stage s + 1 are then issued into.  The fragment reads are written as assembly: the compiler cannot tell
  // which LDS-direct load a plain LDS read might depend on and would make every read wait for the loads just issued.
  // The wait between reads and MFMAs names the fragment registers as in/out operands so that no MFMA moves in front of it.
  issue_next(0);
  for (int s = 0; s < nk; ++s) {
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    if (s + 1 < nk) issue_next((s + 1) & 1);
    const uint32_t oa = (uint32_t)((s & 1) * A_STAGE), ob = (uint32_t)((s & 1) * B_STAGE);
    f4v af[NJ], bf[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) asm volatile("ds_read_b128 %0, %1" : "=v"(af[j]) : "v"(a_at[j] + oa));
    if constexpr (B_KC) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) asm volatile("ds_read_b128 %0, %1" : "=v"(bf[j]) : "v"(b_at[j] + ob));
    } else {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        float b0, b1, b2, b3;
        asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %4 offset:256\n\tds_read_b32 %2, %4 offset:512\n\tds_read_b32 %3, %4 offset:768"
                     : "=&v"(b0), "=&v"(b1), "=&v"(b2), "=&v"(b3)
                     : "v"(b_at[j] + ob));
        bf[j] = f4v{b0, b1, b2, b3};
      }
    }
    if constexpr (NJ == 4)
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(af[0]), "+v"(af[1]), "+v"(af[2]), "+v"(af[3]), "+v"(bf[0]), "+v"(bf[1]), "+v"(bf[2]), "+v"(bf[3]));
    else
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]), "+v"(bf[0]), "+v"(bf[1]));
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[j][t], bf[j][t], acc, 0, 0, 0);
  }

  if constexpr (WAVES_K == 2) {
    // every wavefront has read its last fragments and no load is in flight: the stage buffers carry the hand-over,
    // value v of lane l of tile t at float (t * 16 + v) * 64 + l
    static_assert(NT * 16 * 64 * 4 <= STAGES * A_STAGE, "the hand-over fits the A stages");
    __builtin_amdgcn_s_barrier();
    float* ex = reinterpret_cast<float*>(smem) + wtile * 1024 + lane;
    if (kgrp == 1) {
#pragma unroll
      for (int v = 0; v < 16; ++v) ex[v * 64] = acc[v];
    }
    __syncthreads();
    if (kgrp == 1) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] += ex[v * 64];
  }

  const int col = n0 + wn + l32;
  if (col < a.N) store_tile<ACT>(a.ep, m0 + wm + lhi * 4, col, acc, a.M);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int WAVES_M, int WAVES_N, bool B_KC, int ACT, int WAVES_K = 1>
int launch_ring_act(sn_ctx* ctx, const char* name, RingArgs& a, int K) {
  constexpr int BM = 32 * WAVES_M, BN = 32 * WAVES_N;
  a.tiles_m = (int)ceil_div(a.M, BM);
  a.tiles_n = (int)ceil_div(a.N, BN);
  const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
  const size_t smem = (size_t)STAGES * (BM * 128 + (B_KC ? BN * 128 : (RK / 4) * BO_BLOCK));
  LaunchScope scope(ctx, name, a.M, a.N, K);
  hipLaunchKernelGGL((conv_ring_kernel<WAVES_M, WAVES_N, B_KC, ACT, WAVES_K>), dim3((unsigned)(8 * ceil_div(tiles, 8))),
                     dim3(64 * WAVES_M * WAVES_N * WAVES_K), smem, ctx->stream, a);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

template <int WAVES_M, int WAVES_N, bool B_KC>
int launch_ring(sn_ctx* ctx, const char* name, RingArgs& a, int K) {
  switch (a.ep.act) {
    case SN_ACT_SIGMOID: return launch_ring_act<WAVES_M, WAVES_N, B_KC, SN_ACT_SIGMOID>(ctx, name, a, K);
    case SN_ACT_TANH: return launch_ring_act<WAVES_M, WAVES_N, B_KC, SN_ACT_TANH>(ctx, name, a, K);
    case SN_ACT_RELU: return launch_ring_act<WAVES_M, WAVES_N, B_KC, SN_ACT_RELU>(ctx, name, a, K);
    default: return launch_ring_act<WAVES_M, WAVES_N, B_KC, SN_ACT_IDENTITY>(ctx, name, a, K);
  }
}

}  // namespace

// Shapes the ring kernels take: channels of the gathered tensor a multiple of 32, at most 32 taps, 16-byte aligned
// tensors below 2 GiB, no all-ones row riding along in the epilogue.
bool conv_ring_fwd_ok(const ConvGeom& g, const float* x, const float* w, const Epilogue& e) {
  return g.cin % RK == 0 && g.cout % 4 == 0 && g.kh * g.kw <= 32 && aligned16(x) && aligned16(w) && e.row_index < 0 &&
         (int64_t)g.n * g.h * g.w * g.cin * 4 < (int64_t)OOB && (int64_t)g.kh * g.kw * g.cin * g.cout * 4 < (int64_t)OOB &&
         (int64_t)g.n * g.ho * g.wo >= 64;
}

int launch_conv_ring_fwd(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* w, const Epilogue& e) {
  RingArgs a{};
  a.src = x;
  a.src_bytes = (uint32_t)((int64_t)g.n * g.h * g.w * g.cin * 4);
  a.M = g.n * g.ho * g.wo; a.ih = g.ho; a.iw = g.wo;
  a.sy = g.sh; a.sx = g.sw; a.oy = -g.pt; a.ox = -g.pl; a.ty = 1; a.tx = 1;
  a.H = g.h; a.W = g.w; a.C = g.cin; a.kh = g.kh; a.kw = g.kw;
  a.b = w;
  a.b_bytes = (uint32_t)((int64_t)g.kh * g.kw * g.cin * g.cout * 4);
  a.N = g.cout;
  a.ep = e;
  return launch_ring<2, 2, false>(ctx, "conv2d_forward", a, g.kh * g.kw * g.cin);
}

bool conv_ring_dgrad_ok(const ConvGeom& g, const float* dy, const float* w) {
  return g.sh == 1 && g.sw == 1 && g.cout % RK == 0 && g.kh * g.kw <= 32 && aligned16(dy) && aligned16(w) &&
         (int64_t)g.n * g.ho * g.wo * g.cout * 4 < (int64_t)OOB && (int64_t)g.kh * g.kw * g.cin * g.cout * 4 < (int64_t)OOB &&
         (int64_t)g.n * g.h * g.w >= 128;
}

int launch_conv_ring_dgrad(sn_ctx* ctx, const ConvGeom& g, const float* dy, const float* w, float* dx) {
  RingArgs a{};
  a.src = dy;
  a.src_bytes = (uint32_t)((int64_t)g.n * g.ho * g.wo * g.cout * 4);
  a.M = g.n * g.h * g.w; a.ih = g.h; a.iw = g.w;
  a.sy = 1; a.sx = 1; a.oy = g.pt; a.ox = g.pl; a.ty = -1; a.tx = -1;
  a.H = g.ho; a.W = g.wo; a.C = g.cout; a.kh = g.kh; a.kw = g.kw;
  a.b = w;
  a.b_bytes = (uint32_t)((int64_t)g.kh * g.kw * g.cin * g.cout * 4);
  a.N = g.cin;
  a.b_tap_stride = g.cin * g.cout;   // w[tap, n, channel]
  a.b_n_stride = g.cout;
  a.ep.out = dx;
  a.ep.ldo = g.cin;
  const int K = g.kh * g.kw * g.cout;
  // (two-wavefront workgroups, 32 x 64 and 64 x 32, were measured on LeNet's second convolution: forward 35 us against 31,
  // input gradient the same 30 us)
  // 32 columns: 64 x 32 tiles, two wavefronts per 32 x 32 tile (the input gradient has no activation).  On LeNet's
  // second convolution 29.1 us against 30.2 for 128 x 32 tiles of one wavefront each (128 x 32 with two: 29.4); the same
  // split of the forward product's 64 x 64 tiles gained nothing there (30.2 us either way) and is not used.
  if (g.cin <= 32) return launch_ring_act<2, 1, true, SN_ACT_IDENTITY, 2>(ctx, "conv2d_input_gradient", a, K);
  return launch_ring<2, 2, true>(ctx, "conv2d_input_gradient", a, K);
}

}  // namespace sn
