// Conv2D filter gradient for 32 input channels as fp32 matrix-core tiles per filter tap (gfx950).
//
//   dW[r, q, ci, co] = sum over (b, oh, ow) of x[b, oh*sh + r, ow*sw + q, ci] * dy[b, oh, ow, co]
//   (math/nn/AllKernels.scala:211-261: the filter's side of Conv2D's gradient), no padding.
//
// As a GEMM the product is [kh*kw*32] x [cout] over tens of thousands of positions: the output is tiny, so filling the
// chip means many partial results.  Tiled 64 x 64 with a split of the positions, 256 partial filters leave and come back
// for one result.  Here a workgroup owns the [32 channels] x [cout] tiles of ONE tap (conv_wgrad_taps_kernel) or of the
// up to three taps of one filter row (conv_wgrad_tap_rows_kernel, the form taken where it applies) and a contiguous range
// of the output rows (b, oh); the workgroups of a range are neighbours on one XCD, so a range's x and dy are read from
// memory once and from L2 by the other taps, and the number of partial filters is the number of ranges (a few dozen).
//
// Neither operand goes through LDS.  With the position as the k index both operands of v_mfma_f32_32x32x2_f32 are rows of
// the tensors as they lie: lane l holds A[m = l % 32][k = l / 32] = x[position p + l / 32][channel l % 32] and
// B[k = l / 32][n = l % 32] = dy[position p + l / 32][unit n0 + l % 32], so one 4-byte buffer load per lane (two runs
// of 128 bytes per wavefront) feeds an operand of one MFMA.  A wavefront walks its rows two positions at a time (the
// odd position at a row's end is a load beyond the buffer's range: zeros, no traffic) with a ring of loads in flight;
// the wavefronts of a workgroup split its range, and their accumulators meet in LDS at the end.
#include "common.hpp"

namespace sn {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));

constexpr uint32_t OOB = 0x80000000u;  // beyond any operand (tensors are checked to be < 2 GiB)
constexpr int TAP_CIN = 32;            // input channels (the m index of a tile)
constexpr int TAP_RING = 16;           // position pairs in flight per wavefront
constexpr int TAP_PITCH = 65;          // LDS row pitch of the accumulator exchange (floats)

struct TapArgs {
  const float* x;
  uint32_t x_bytes;
  const float* dy;
  uint32_t dy_bytes;
  float* partial;  // [ranges][kh*kw*32*cout]
  int h, w, ho, wo, kh, kw, sh, sw, cout;
  int rows;        // n * ho output rows
  int ranges;      // row ranges (= partial results)
  int ranges_per_xcd;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tap_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float tap_load(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, (int)voff, (int)soff, 0));
}

// The stream of position pairs of a wavefront: rows [row, row_end), pairs 0 .. pairs_per_row - 1 of each.
struct PairStream {
  int row, row_end, img, oh, j;
  uint32_t x_base, dy_base;  // byte offsets of the row's first position
};

template <int NT>  // 32-unit tiles of the output channels: cout = 32 * NT
__global__ __launch_bounds__(256) void conv_wgrad_taps_kernel(TapArgs a) {
  extern __shared__ __attribute__((aligned(16))) float tap_lds[];  // [4 wavefronts][32][TAP_PITCH] (cout <= 64)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // everything a row range depends on is scalar
  const int taps = a.kh * a.kw;
  // workgroups b, b + 8, ... share an XCD (and its L2): an XCD takes whole ranges, all taps of each
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int local = slot / taps, tap = slot - local * taps;
  if (local >= a.ranges_per_xcd) return;
  const int range = local * 8 + xcd;
  if (range >= a.ranges) return;
  const int r = tap / a.kw, q = tap - r * a.kw;
  // rows of this range, then of this wavefront
  const int g0 = (int)((int64_t)a.rows * range / a.ranges), g1 = (int)((int64_t)a.rows * (range + 1) / a.ranges);
  const int row0 = g0 + (int)((int64_t)(g1 - g0) * wave / 4), row1 = g0 + (int)((int64_t)(g1 - g0) * (wave + 1) / 4);
  const int pairs_per_row = (a.wo + 1) >> 1;
  const bool odd = (a.wo & 1) != 0;
  const __amdgpu_buffer_rsrc_t rx = tap_rsrc(a.x, a.x_bytes), rd = tap_rsrc(a.dy, a.dy_bytes);
  const uint32_t half = (uint32_t)(lane >> 5), col = (uint32_t)(lane & 31);
  const uint32_t vx = (half * (uint32_t)a.sw * TAP_CIN + col) * 4u, vd = (half * (uint32_t)a.cout + col) * 4u;
  const uint32_t vx_tail = half ? OOB : vx, vd_tail = half ? OOB : vd;  // the pair at an odd row's end has one position
  const uint32_t x_pair = 2u * (uint32_t)a.sw * TAP_CIN * 4u, dy_pair = 2u * (uint32_t)a.cout * 4u;

  PairStream s;
  s.row = row0; s.row_end = row1; s.j = 0;
  s.img = row0 / a.ho; s.oh = row0 - s.img * a.ho;
  auto row_bases = [&]() {
    s.x_base = (uint32_t)(((s.img * a.h + s.oh * a.sh + r) * a.w + q) * TAP_CIN) * 4u;
    s.dy_base = (uint32_t)(s.row * a.wo) * (uint32_t)a.cout * 4u;
  };
  row_bases();
  float xa[TAP_RING], db[TAP_RING][NT];
  auto issue = [&](int u) {  // requests the stream's next pair into slot u (zeros once the stream has ended)
    const bool live = s.row < s.row_end;
    const bool tail = odd && s.j == pairs_per_row - 1;
    const uint32_t ox = live ? (tail ? vx_tail : vx) : OOB, od = live ? (tail ? vd_tail : vd) : OOB;
    const uint32_t sx = s.x_base + (uint32_t)s.j * x_pair, sd = s.dy_base + (uint32_t)s.j * dy_pair;
    xa[u] = tap_load(rx, ox, sx);
#pragma unroll
    for (int t = 0; t < NT; ++t) db[u][t] = tap_load(rd, od + 128u * t, sd);
    if (live) {
      if (++s.j == pairs_per_row) {
        s.j = 0;
        ++s.row;
        if (++s.oh == a.ho) { s.oh = 0; ++s.img; }
        row_bases();
      }
    }
  };
#pragma unroll
  for (int u = 0; u < TAP_RING; ++u) issue(u);
  f16v acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
  const int total_pairs = (row1 - row0) * pairs_per_row;
  for (int i = 0; i < total_pairs; i += TAP_RING) {
#pragma unroll
    for (int u = 0; u < TAP_RING; ++u) {
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[u], db[u][t], acc[t], 0, 0, 0);
      issue(u);
    }
  }
  // the four wavefronts' tiles meet in LDS and are added in wavefront order; value v of lane l is element
  // [8 (v / 4) + 4 (l / 32) + v % 4][l % 32] of its tile
  float* mine = tap_lds + wave * 32 * TAP_PITCH;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) mine[(8 * (v >> 2) + 4 * (int)half + (v & 3)) * TAP_PITCH + 32 * t + (int)col] = acc[t][v];
  __syncthreads();
  float* out = a.partial + ((int64_t)range * taps + tap) * TAP_CIN * a.cout;
  for (int e = threadIdx.x; e < TAP_CIN * a.cout; e += 256) {
    const int m = e / a.cout, n = e - m * a.cout;
    const float* p = tap_lds + m * TAP_PITCH + n;
    out[e] = ((p[0] + p[32 * TAP_PITCH]) + p[2 * 32 * TAP_PITCH]) + p[3 * 32 * TAP_PITCH];
  }
}

// The same product with the taps of one filter row (kw <= 3, unit stride along the row) in one workgroup of 8 wavefronts,
// so that what is loaded serves up to three taps.  A row of the output is walked in slots of two positions; slot i loads
//   D_i = dy[2i, 2i+1],  E_i = x[columns 2i, 2i+1]  and  O_i = x[columns 2i+1, 2i+2]
// and multiplies  tap 0: E_i D_i,  tap 1: O_i D_i,  tap 2: E_i D_(i-1)  (x column = position + tap).  With three taps a
// row has one slot more than pairs of positions; its D is beyond the row and loads as zeros, which also makes the D_(i-1)
// of the next row's first slot zero.  Positions beyond the row's end and columns beyond the image load as zeros.
constexpr int ROWTAP_RING = 12;    // slots in flight per wavefront (4 loads each)
constexpr int ROWTAP_WAVES = 8;
constexpr int ROWTAP_PITCH = 33;

template <int KW, int NT>
__global__ __launch_bounds__(ROWTAP_WAVES * 64) void conv_wgrad_tap_rows_kernel(TapArgs a) {
  __shared__ float ex[ROWTAP_WAVES * 32 * ROWTAP_PITCH];  // one 32 x 32 tile per wavefront
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // everything a row range depends on is scalar
  const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
  const int local = slot_id / a.kh, r = slot_id - local * a.kh;
  if (local >= a.ranges_per_xcd) return;
  const int range = local * 8 + xcd;
  if (range >= a.ranges) return;
  const int slots = ((a.wo + 1) >> 1) + (KW == 3 ? 1 : 0);
  // the slots of all rows, in order, are dealt out evenly: a wavefront's run may start and end inside a row
  // (32-bit arithmetic: the host has checked rows * slots < 2^31): the first all % shares wavefronts take one slot more
  const uint32_t all = (uint32_t)a.rows * (uint32_t)slots, shares = (uint32_t)a.ranges * ROWTAP_WAVES, share = (uint32_t)range * ROWTAP_WAVES + wave;
  const uint32_t each = all / shares, extra = all - each * shares;
  const uint32_t first = each * share + (share < extra ? share : extra);
  const int total = (int)(each + (share < extra ? 1u : 0u));
  const int row0 = (int)(first / (uint32_t)slots);
  const __amdgpu_buffer_rsrc_t rx = tap_rsrc(a.x, a.x_bytes), rd = tap_rsrc(a.dy, a.dy_bytes);
  const int half = lane >> 5, col = lane & 31;
  const uint32_t vx = (uint32_t)(half * TAP_CIN + col) * 4u, vd = (uint32_t)(half * a.cout + col) * 4u;
  const uint32_t x_pair = 2u * TAP_CIN * 4u, dy_pair = 2u * (uint32_t)a.cout * 4u;

  int s_row = row0, s_i = (int)first - row0 * slots, s_left = total;
  int s_img = row0 / a.ho, s_oh = row0 - s_img * a.ho;
  uint32_t x_base, dy_base;
  auto row_bases = [&]() {
    x_base = (uint32_t)(((s_img * a.h + s_oh * a.sh + r) * a.w) * TAP_CIN) * 4u;
    dy_base = (uint32_t)(s_row * a.wo) * (uint32_t)a.cout * 4u;
  };
  row_bases();
  // Ring entry e holds a slot's E, O and D.  Slot k of the run lies in entry k % RING; its D stays there one slot longer
  // than its E and O, as the D_(i-1) of slot k + 1: entry e is refilled after the slot in entry e + 1 has been multiplied.
  float xe[ROWTAP_RING], xo[ROWTAP_RING], db[ROWTAP_RING][NT];
  const int full_slots = a.wo >> 1;  // slots of a row whose two positions (and all the x columns they need) exist
  auto issue = [&](int e) {  // requests the stream's next slot into ring entry e (zeros once the stream has ended)
    // (the same in every lane; said explicitly, so that the loads take them as scalar offsets whatever unit computed them)
    const uint32_t sx = (uint32_t)__builtin_amdgcn_readfirstlane((int)(x_base + (uint32_t)s_i * x_pair));
    const uint32_t sd = (uint32_t)__builtin_amdgcn_readfirstlane((int)(dy_base + (uint32_t)s_i * dy_pair));
    if (s_left > 0 && s_i < full_slots) {  // nothing to mask: no vector instruction but the loads
#pragma unroll
      for (int t = 0; t < NT; ++t) db[e][t] = tap_load(rd, vd + 128u * t, sd);
      xe[e] = tap_load(rx, vx, sx);
      if (KW >= 2) xo[e] = tap_load(rx, vx, sx + TAP_CIN * 4u);
    } else {
      const bool live = s_left > 0;
      const int p0 = 2 * s_i + half;  // this lane's position, and its x column for tap 0
      const uint32_t od = (live && p0 < a.wo) ? vd : OOB;
      const uint32_t oe = (live && p0 < a.w) ? vx : OOB;
      const uint32_t oo = (live && p0 + 1 < a.w) ? vx : OOB;
#pragma unroll
      for (int t = 0; t < NT; ++t) db[e][t] = tap_load(rd, od + 128u * t, sd);
      xe[e] = tap_load(rx, oe, sx);
      if (KW >= 2) xo[e] = tap_load(rx, oo, sx + TAP_CIN * 4u);
    }
    // the stream moves on (beyond its end it walks on: those slots load nothing)
    --s_left;
    const bool wrap = s_i + 1 == slots;
    const bool wrap_img = wrap && s_oh + 1 == a.ho;
    s_i = wrap ? 0 : s_i + 1;
    s_row += wrap ? 1 : 0;
    s_oh = wrap_img ? 0 : s_oh + (wrap ? 1 : 0);
    s_img += wrap_img ? 1 : 0;
    row_bases();
  };
  // the D before the run's first slot goes where slot -1 would lie: zeros, or (a run that starts inside a row) loaded
#pragma unroll
  for (int t = 0; t < NT; ++t) db[ROWTAP_RING - 1][t] = 0.f;
  if (KW == 3 && s_i > 0) {
    const uint32_t od = 2 * (s_i - 1) + half < a.wo ? vd : OOB;
#pragma unroll
    for (int t = 0; t < NT; ++t) db[ROWTAP_RING - 1][t] = tap_load(rd, od + 128u * t, dy_base + (uint32_t)(s_i - 1) * dy_pair);
  }
#pragma unroll
  for (int e = 0; e < ROWTAP_RING - 1; ++e) issue(e);
  f16v acc[KW][NT];
#pragma unroll
  for (int k = 0; k < KW; ++k)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[k][t][v] = 0.f;
  auto multiply = [&](int e) {
    const int before = (e + ROWTAP_RING - 1) % ROWTAP_RING;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(xe[e], db[e][t], acc[0][t], 0, 0, 0);
      if (KW >= 2) acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(xo[e], db[e][t], acc[1][t], 0, 0, 0);
      if (KW == 3) acc[2][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(xe[e], db[before][t], acc[2][t], 0, 0, 0);
    }
  };
  const int turns = total / ROWTAP_RING;  // whole turns of the ring: straight-line code but for the rows' ends
  for (int i = 0; i < turns; ++i) {
#pragma unroll
    for (int e = 0; e < ROWTAP_RING; ++e) {
      multiply(e);
      issue((e + ROWTAP_RING - 1) % ROWTAP_RING);
    }
  }
#pragma unroll
  for (int e = 0; e < ROWTAP_RING - 1; ++e)  // what is left of the run: at most RING - 1 slots, all of them requested
    if (turns * ROWTAP_RING + e < total) multiply(e);
  // tile by tile the wavefronts' accumulators meet in LDS and are added in wavefront order; value v of lane l is element
  // [8 (v / 4) + 4 (l / 32) + v % 4][l % 32] of its tile
  float* mine = ex + wave * 32 * ROWTAP_PITCH;
  float* out = a.partial + ((int64_t)range * a.kh + r) * KW * TAP_CIN * a.cout;
#pragma unroll
  for (int k = 0; k < KW; ++k) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (k + t > 0) __syncthreads();  // the sums of the tile before have been read
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[(8 * (v >> 2) + 4 * half + (v & 3)) * ROWTAP_PITCH + col] = acc[k][t][v];
      __syncthreads();
      for (int e = threadIdx.x; e < 32 * 32; e += ROWTAP_WAVES * 64) {
        const int m = e >> 5, n = e & 31;
        const float* p = ex + m * ROWTAP_PITCH + n;
        float sum = p[0];
#pragma unroll
        for (int w = 1; w < ROWTAP_WAVES; ++w) sum += p[w * 32 * ROWTAP_PITCH];
        out[(k * TAP_CIN + m) * a.cout + 32 * t + n] = sum;
      }
    }
  }
}

int rowtap_ranges_per_xcd(const sn_ctx* ctx, const ConvGeom& g) {
  // one workgroup of 8 wavefronts per compute unit, an XCD's share of them split into whole ranges of kh filter rows
  return std::max(1, ctx->compute_units / 8) / g.kh;
}
bool rowtap_shape(const sn_ctx* ctx, const ConvGeom& g) {
  const int per = rowtap_ranges_per_xcd(ctx, g);
  return g.kw <= 3 && g.sw == 1 && per >= 1 && (int64_t)g.n * g.ho >= (int64_t)per * 8 * ROWTAP_WAVES * 2;
}

int tap_ranges_per_xcd(const sn_ctx* ctx, const ConvGeom& g) {
  // two workgroups per compute unit, an XCD's share of them split into whole ranges of kh * kw taps
  const int per_xcd = std::max(1, 2 * ctx->compute_units / 8);
  return per_xcd / (g.kh * g.kw);
}

}  // namespace

bool conv_wgrad_taps_shape(const sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy) {
  if (g.cin != TAP_CIN || (g.cout != 32 && g.cout != 64) || g.pt != 0 || g.pl != 0) return false;
  if ((int64_t)g.n * g.ho * (g.wo / 2 + 2) >= ((int64_t)1 << 31)) return false;
  if ((g.ho - 1) * g.sh + g.kh > g.h || (g.wo - 1) * g.sw + g.kw > g.w || g.n <= 0 || g.ho <= 0 || g.wo <= 0) return false;
  const int64_t x_bytes = (int64_t)g.n * g.h * g.w * g.cin * 4, dy_bytes = (int64_t)g.n * g.ho * g.wo * g.cout * 4;
  if (x_bytes >= ((int64_t)1 << 31) || dy_bytes >= ((int64_t)1 << 31)) return false;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy)) & 3u) return false;
  if ((int64_t)g.n * g.ho * g.wo < 8192) return false;  // too few positions for partial results to be worth their sum
  if (rowtap_shape(ctx, g)) return true;
  const int per = tap_ranges_per_xcd(ctx, g);
  return per >= 1 && (int64_t)g.n * g.ho >= (int64_t)per * 8 * 4 * 2;  // rows for every wavefront of every range
}

int64_t conv_wgrad_taps_workspace(const sn_ctx* ctx, const ConvGeom& g) {
  const int per = std::max(tap_ranges_per_xcd(ctx, g), rowtap_ranges_per_xcd(ctx, g));
  return (int64_t)per * 8 * g.kh * g.kw * g.cin * g.cout;
}

// Leaves `*parts` partial filters [part][kh*kw*cin*cout] in ws; the caller adds them (in part order).
int launch_conv_wgrad_taps(sn_ctx* ctx, const ConvGeom& g, const float* x, const float* dy, float* ws, int64_t ws_elems, int* parts) {
  SN_REQUIRE(conv_wgrad_taps_shape(ctx, g, x, dy), "conv2d_filter_gradient_taps: shape outside the kernel's range");
  SN_REQUIRE(ws && conv_wgrad_taps_workspace(ctx, g) <= ws_elems, "conv2d_filter_gradient_taps: workspace too small");
  TapArgs a;
  a.x = x; a.x_bytes = (uint32_t)((int64_t)g.n * g.h * g.w * g.cin * 4);
  a.dy = dy; a.dy_bytes = (uint32_t)((int64_t)g.n * g.ho * g.wo * g.cout * 4);
  a.partial = ws;
  a.h = g.h; a.w = g.w; a.ho = g.ho; a.wo = g.wo; a.kh = g.kh; a.kw = g.kw; a.sh = g.sh; a.sw = g.sw; a.cout = g.cout;
  a.rows = g.n * g.ho;
  if (rowtap_shape(ctx, g)) {  // the taps of a filter row together
    a.ranges_per_xcd = rowtap_ranges_per_xcd(ctx, g);
    a.ranges = a.ranges_per_xcd * 8;
    const unsigned blocks = (unsigned)(8 * a.ranges_per_xcd * g.kh);
    LaunchScope scope(ctx, "conv2d_filter_gradient_tap_rows", g.kh * g.kw * g.cin, g.cout, g.n * g.ho * g.wo);
#define SN_ROWTAP(KW)                                                                                                    \
  do {                                                                                                                   \
    if (g.cout == 64) hipLaunchKernelGGL((conv_wgrad_tap_rows_kernel<KW, 2>), dim3(blocks), dim3(ROWTAP_WAVES * 64), 0, ctx->stream, a); \
    else hipLaunchKernelGGL((conv_wgrad_tap_rows_kernel<KW, 1>), dim3(blocks), dim3(ROWTAP_WAVES * 64), 0, ctx->stream, a);               \
  } while (0)
    if (g.kw == 3) SN_ROWTAP(3);
    else if (g.kw == 2) SN_ROWTAP(2);
    else SN_ROWTAP(1);
#undef SN_ROWTAP
    *parts = a.ranges;
    SN_HIP(hipGetLastError());
    return SN_OK;
  }
  a.ranges_per_xcd = tap_ranges_per_xcd(ctx, g);
  a.ranges = a.ranges_per_xcd * 8;
  const unsigned blocks = (unsigned)(8 * a.ranges_per_xcd * g.kh * g.kw);
  const size_t lds = (size_t)4 * 32 * TAP_PITCH * sizeof(float);
  LaunchScope scope(ctx, "conv2d_filter_gradient_taps", g.kh * g.kw * g.cin, g.cout, g.n * g.ho * g.wo);
  if (g.cout == 64) hipLaunchKernelGGL((conv_wgrad_taps_kernel<2>), dim3(blocks), dim3(256), lds, ctx->stream, a);
  else hipLaunchKernelGGL((conv_wgrad_taps_kernel<1>), dim3(blocks), dim3(256), lds, ctx->stream, a);
  *parts = a.ranges;
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
