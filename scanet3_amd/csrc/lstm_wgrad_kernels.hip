// Weight gradient of a recurrent layer over all time steps: dW[m, n] = sum_k A[k, m] * dZ[k, n] with k = (t, batch row),
// A[k, .] = [x_t | h_{t-1}] of that row (F + H values) and dZ[k, .] the gradient of its G*H pre-activations (G = 4 gates for
// the LSTM, 1 for the simple cell).  The bias gradient is the column sum of dZ.  (layer/RNN.scala:320-338 through
// math/alg/AllKernels.scala:382-388: matmul's gradient wrt its right operand, summed over the unrolled steps.)
//
// Shape of the problem at LSTM(256), batch 512, 64 steps, 32 features: 288 x 1024 outputs, k = 32768.  Both operands are
// contiguous along their OUTPUT index, which is the order v_mfma_f32_32x32x2_f32 wants across its lanes, so a stage of 16
// k-rows goes to LDS as it lies (`global_load_lds_dwordx4`, no staging registers) and a fragment is one ds_read_b32 per
// lane.  A workgroup owns ALL F + H rows x 128 columns for one range of k: wavefront w keeps 32 columns x (1 + H/32) row
// tiles of accumulators (144 registers at H = 256), reads one B fragment and 1 + H/32 A fragments per k-pair, and adds the
// B fragments it passes into the bias row.  Work items = (column tiles) x (k ranges), one per CU, all the same size: no
// padded rows (the tiled GEMM pays 320 rows for 289) and no second round.  Three LDS stages: the loads of stage s + 3 are
// issued at the barrier that frees stage s, two stages ahead of their use.  The k ranges leave one partial [F + H + 1, G*H]
// each; splitk_reduce4_kernel adds them in a fixed order into the layer's gradient tensors.
#include "common.hpp"

namespace sn {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;
__device__ __align__(16) const float wgrad_zero_chunk[4] = {0.f, 0.f, 0.f, 0.f};  // what the padding of the feature tile reads

constexpr int WK = 16;    // k-rows per stage
constexpr int WBN = 128;  // columns per workgroup
constexpr int WRING = 3;  // LDS stages

struct WgradArgs {
  const float* x;    // [rows, T, F]
  const float* h;    // [T * rows, H]: row k = h_{t-1} of batch row b, k = t * rows + b
  const float* dz;   // [T * rows, N]
  float* partial;    // [ranges, F + H + 1, N]
  int rows, T, F, H, N;
  int n_tiles, ranges;
  int stages_total;  // T * rows / WK
  int stages_per_range;
};

template <int HT>  // H / 32
__global__ __launch_bounds__(256) void lstm_wgrad_rows_kernel(WgradArgs a) {
  constexpr int H = 32 * HT, MT = 1 + HT;
  constexpr int AX_BYTES = WK * 128, AH_BYTES = WK * H * 4, B_BYTES = WK * WBN * 4;
  constexpr int STAGE = AX_BYTES + AH_BYTES + B_BYTES;
  constexpr int H_ISSUES = AH_BYTES / 1024 / 4;  // per wavefront
  constexpr int IPW = 1 + H_ISSUES + 2;          // LDS-bound loads per wavefront and stage
  extern __shared__ __attribute__((aligned(16))) char wg_smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const int item = blockIdx.x;
  const int nt = item % a.n_tiles, range = item / a.n_tiles;
  const int n0 = nt * WBN;
  const int s_begin = range * a.stages_per_range;
  const int nst = min(a.stages_per_range, a.stages_total - s_begin);
  if (nst <= 0) return;

  // ---- global -> LDS, stage s of this range into ring slot s % WRING
  auto issue_stage = [&](int s) {
    char* base = wg_smem + (s % WRING) * STAGE;
    const int64_t k0 = (int64_t)(s_begin + s) * WK;
    {  // feature tile [WK][32]: this wavefront's half of the k-rows (wavefronts 0/2 and 1/3 load the same halves)
      const int krow = 8 * (wave & 1) + (lane >> 3), c = lane & 7;
      const int k = (int)k0 + krow;  // T * rows < 2^31 (checked by the host)
      const int t = k / a.rows, b = k - t * a.rows;
      const float* src = 4 * c < a.F ? a.x + ((int64_t)b * a.T + t) * a.F + 4 * c : wgrad_zero_chunk;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(base + 1024 * (wave & 1)), 16, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < H_ISSUES; ++q) {  // hidden tile [WK][H]
      const int byte = (wave * H_ISSUES + q) * 1024 + 16 * lane;
      const float* src = a.h + (k0 + byte / (H * 4)) * H + (byte % (H * 4)) / 4;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(base + AX_BYTES + (wave * H_ISSUES + q) * 1024), 16, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {  // dZ tile [WK][128]
      const int j = wave * 2 + q;
      const float* src = a.dz + (k0 + 2 * j + lhi) * a.N + n0 + 4 * l32;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(base + AX_BYTES + AH_BYTES + j * 1024), 16, 0, 0);
    }
  };

  // ---- LDS -> fragments of k-pair p (k-rows 2p, 2p + 1) of the stage in slot `slot`
  float fa[2][MT], fb[2];
  auto read_pair = [&](int set, int slot, int p) {
    const char* base = wg_smem + slot * STAGE;
    const int krow = 2 * p + lhi;
    fb[set] = *(const float*)(base + AX_BYTES + AH_BYTES + krow * (WBN * 4) + (wave * 32 + l32) * 4);
    fa[set][0] = *(const float*)(base + krow * 128 + l32 * 4);
#pragma unroll
    for (int i = 1; i < MT; ++i) fa[set][i] = *(const float*)(base + AX_BYTES + krow * (H * 4) + ((i - 1) * 32 + l32) * 4);
  };

  f16v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  float bsum = 0.f;

  // prologue: up to three stages in flight, the first one landed
#pragma unroll
  for (int s = 0; s < WRING; ++s)
    if (s < nst) issue_stage(s);
  if (nst >= 3) __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * IPW));       // vmcnt(2 IPW): all but the last two stages' loads
  else if (nst == 2) __builtin_amdgcn_s_waitcnt(0x0f70 | IPW);
  else __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();
  read_pair(0, 0, 0);

  for (int s = 0; s < nst; ++s) {
    const int slot = s % WRING;
#pragma unroll
    for (int p = 0; p < WK / 2; ++p) {
      const int cur = p & 1;
      if (p + 1 < WK / 2) {
        read_pair(cur ^ 1, slot, p + 1);
      } else {
        // every fragment of this stage is in registers (or on its way: lgkmcnt(0)); the next stage must have landed
        if (s + 2 < nst) __builtin_amdgcn_s_waitcnt(0x0070 | IPW);   // lgkmcnt(0), vmcnt(IPW): the stage after next may still fly
        else __builtin_amdgcn_s_waitcnt(0x0070);                      // lgkmcnt(0), vmcnt(0)
        __syncthreads();
        if (s + WRING < nst) issue_stage(s + WRING);                  // into the slot this stage leaves
        if (s + 1 < nst) read_pair(cur ^ 1, (s + 1) % WRING, 0);
      }
      bsum += fb[cur];
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][i], fb[cur], acc[i], 0, 0, 0);
    }
  }

  // ---- this range's partial: rows 0..F-1 (features), F..F+H-1 (hidden), F+H (column sums of dZ)
  const int M_out = a.F + a.H + 1;
  float* out = a.partial + (int64_t)range * M_out * a.N + n0 + wave * 32 + l32;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int r = 8 * (v >> 2) + 4 * lhi + (v & 3);
      if (i == 0) {
        if (r < a.F) out[(int64_t)r * a.N] = acc[0][v];
      } else {
        out[(int64_t)(a.F + (i - 1) * 32 + r) * a.N] = acc[i][v];
      }
    }
  }
  const float both = bsum + __shfl_xor(bsum, 32, 64);  // even k-rows in lanes 0..31, odd ones in 32..63
  if (lhi == 0) out[(int64_t)(a.F + a.H) * a.N] = both;
}

int ranges_for(const sn_ctx* ctx, int rows, int T, int N) {
  const int n_tiles = N / WBN;
  const int stages_total = (int)((int64_t)rows * T / WK);
  int ranges = ctx->compute_units / n_tiles;
  if (ranges < 1) ranges = 1;
  if (ranges > stages_total / 8) ranges = stages_total / 8;  // at least 8 stages per range
  return ranges;
}

}  // namespace

bool lstm_wgrad_rows_ok(const sn_ctx* ctx, const float* x, const float* h, const float* dz, int rows, int T, int F, int H, int gates) {
  const int N = gates * H;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(dz)) & 15u) == 0;
  return aligned && F >= 4 && F <= 32 && F % 4 == 0 && (H == 64 || H == 128 || H == 256) && N % WBN == 0 && ((int64_t)rows * T) % WK == 0 &&
         (int64_t)rows * T >= 64 * WK && (int64_t)rows * T < ((int64_t)1 << 31) && ranges_for(ctx, rows, T, N) >= 2;
}

int64_t lstm_wgrad_rows_workspace(const sn_ctx* ctx, int rows, int T, int F, int H, int gates) {
  const int N = gates * H;
  if (!(F >= 4 && F <= 32 && F % 4 == 0 && (H == 64 || H == 128 || H == 256) && N % WBN == 0 && ((int64_t)rows * T) % WK == 0 && (int64_t)rows * T >= 64 * WK)) return 0;
  return (int64_t)ranges_for(ctx, rows, T, N) * (F + H + 1) * N;
}

// Writes `*ranges` partial results [F + H + 1, gates * H] to ws (the caller adds them).
int launch_lstm_wgrad_rows(sn_ctx* ctx, const float* x, const float* h, const float* dz, int rows, int T, int F, int H, int gates, float* ws,
                           int64_t ws_elems, int* ranges_out) {
  SN_REQUIRE(lstm_wgrad_rows_ok(ctx, x, h, dz, rows, T, F, H, gates), "lstm_weight_gradient_rows: shape rows=%d T=%d F=%d H=%d is not in range", rows, T, F, H);
  WgradArgs a;
  a.x = x; a.h = h; a.dz = dz; a.partial = ws;
  a.rows = rows; a.T = T; a.F = F; a.H = H; a.N = gates * H;
  a.n_tiles = a.N / WBN;
  a.stages_total = (int)((int64_t)rows * T / WK);
  int ranges = ranges_for(ctx, rows, T, a.N);
  a.stages_per_range = (int)ceil_div(a.stages_total, ranges);
  ranges = (int)ceil_div(a.stages_total, a.stages_per_range);
  a.ranges = ranges;
  SN_REQUIRE(ws && (int64_t)ranges * (F + H + 1) * a.N <= ws_elems, "lstm_weight_gradient_rows: workspace of %lld floats is too small", (long long)ws_elems);
  *ranges_out = ranges;
  const int ht = H / 32;
  const size_t smem = (size_t)WRING * (WK * 128 + WK * H * 4 + WK * WBN * 4);
  LaunchScope scope(ctx, "lstm_weight_gradient_rows", F + H + 1, a.N, rows * T);
  const dim3 grid((unsigned)(a.n_tiles * ranges));
  if (ht == 8) {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)lstm_wgrad_rows_kernel<8>, smem));
    hipLaunchKernelGGL(lstm_wgrad_rows_kernel<8>, grid, dim3(256), smem, ctx->stream, a);
  } else if (ht == 4) {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)lstm_wgrad_rows_kernel<4>, smem));
    hipLaunchKernelGGL(lstm_wgrad_rows_kernel<4>, grid, dim3(256), smem, ctx->stream, a);
  } else {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)lstm_wgrad_rows_kernel<2>, smem));
    hipLaunchKernelGGL(lstm_wgrad_rows_kernel<2>, grid, dim3(256), smem, ctx->stream, a);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
