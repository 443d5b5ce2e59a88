// bf16 matrix-core GEMM for the wide Dense layers (fp32 master data, bf16 operands, fp32 accumulate).
//
// Canonical form: C[M,N] = A[M,K] * Bt[N,K]^T with BOTH operands K-contiguous bf16, so every
// global load is a 16-byte chunk of 8 consecutive k and goes to LDS unchanged.  The three Dense
// products map onto it with bf16 copies kept in both orientations:
//   forward  Y  = X  W      A = X   [rows,in]   Bt = W^T  [out,in]
//   dX          = dY W^T    A = dY  [rows,out]  Bt = W    [in,out]
//   dW          = X^T dY    A = X^T [in,rows]   Bt = dY^T [out,rows]
// cast_transpose_kernel writes the two bf16 orientations of an fp32 matrix in one pass (optionally
// applying the activation gradient on the way), which is all the extra traffic this path costs.
//
// Kernel shape (WT = 128): 256 threads = 4 wavefronts (2x2), block tile 256x256, K step 64,
// wavefront tile 128x128 = 4x4 v_mfma_f32_32x32x16_bf16 (256 accumulator registers per lane,
// one wavefront per SIMD).  LDS holds two stages of A and B tiles (2 x 64 KiB of the 160 KiB);
// rows are 128 bytes and their 16-byte chunks are XOR-swizzled so that the ds_read_b128 fragment
// loads are conflict free.  Tiles travel HBM/L2 -> LDS with `buffer_load_dwordx4 ... lds`: no
// staging registers, no ds_write instructions, and out-of-range rows / the k tail arrive as zeros
// from the buffer descriptor's range check.  The loads of stage k+2 are issued right after the
// barrier that publishes stage k+1, so they have a whole stage of MFMAs (about 2048 cycles) to land.
// WT = 64 is the same kernel with a 128x128 block tile for outputs too small to fill 256 CUs.
#include "common.hpp"

namespace sn {

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int GBK = 64;  // k per stage: 8 chunks of 8 bf16 = 128 bytes per tile row

// Byte offset of 16-byte chunk `chunk` of tile row `row`.  The XOR pattern puts any 8 consecutive rows of one
// logical chunk on 8 different 16-byte bank groups of a 128-byte line, and any 16 consecutive rows on 16
// different groups of a 256-byte double line, so ds_read_b128 / ds_write_b128 stay conflict free whether the
// LDS serves 8 or 16 lanes per cycle.
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row & 7) ^ ((row >> 3) & 1))) << 4); }

// Activations of the bf16 path: hardware exp2 / reciprocal (about 1e-6 relative), far inside bf16's 4e-3
// and small enough to sit 256 times in an unrolled epilogue.
__device__ __forceinline__ float fast_sigmoid(float v) { return __frcp_rn(1.0f + __expf(-v)); }
__device__ __forceinline__ float fast_tanh(float v) { return 1.0f - 2.0f * __frcp_rn(1.0f + __expf(2.0f * v)); }

__device__ __forceinline__ float bf_act(int act, float v, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return fast_sigmoid(v);
    case SN_ACT_TANH: return fast_tanh(v);
    case SN_ACT_RELU: return fmaxf(param, v);
    default: return v;
  }
}

// Raw buffer descriptor over [p, p + bytes): loads whose offset falls outside return zero, which is
// how partial tiles (rows past M or N, the k tail) are handled without a branch.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
constexpr uint32_t OOB = 0x80000000u;  // beyond any operand (operands are checked to be < 2 GiB)

typedef __attribute__((address_space(3))) void* lds_ptr;

// Epilogue modes: 0..3 = the activation (SN_ACT_*) as a compile-time constant, -1 = decide at run time (edge tiles).
__device__ __forceinline__ float bf_act_grad(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

// Per-wavefront LDS staging area for the transposed bf16 copy: [WT columns][WT rows + 4] bf16.
template <int WT>
constexpr int tr_pitch() { return WT * 2 + 8; }  // bytes per staged column

constexpr int MODE_HANDOVER = 8;  // EpilogueBf16::grad_handover (full tiles only)

template <int MODE, bool FULL, int TI>
__device__ __forceinline__ void store_tile(const f16v (&acc)[TI][TI], const EpilogueBf16& ep, int mbase, int nbase, int lane, int M,
                                           int N, char* stage) {
  // mbase/nbase: origin of this wavefront's (32 TI) x (32 TI) tile.  Lane l holds column l%32 of every 32x32
  // sub-tile and rows 8*(v/4) + 4*(l/32) + v%4 for accumulator element v.
  constexpr int WT = 32 * TI;
  constexpr int PITCH = tr_pitch<WT>();
  const int l32 = lane & 31, lhi = lane >> 5;
  const int row0 = mbase + lhi * 4, col0 = nbase + l32;
  const int ldo = (int)ep.e.ldo;
  const int64_t origin = (int64_t)row0 * ldo + col0;
  float* out = ep.e.out ? ep.e.out + origin : nullptr;
  bf16* obf = ep.out_bf ? (bf16*)ep.out_bf + origin : nullptr;
  const bool transposed = ep.out_bf_t != nullptr;
  // Hand-over mode: the 4 rows a lane holds per (i, vq) are 8 contiguous bytes of the transposed output copy of the layer
  // below; a column's 4 TI masks are requested one column ahead of their use (requesting the whole tile's masks up front
  // was measured and is slower).
  constexpr bool HAND = MODE == MODE_HANDOVER;
  constexpr int MT = HAND ? TI : 1;
  const bf16* ym = (HAND && ep.grad_mask_t) ? (const bf16*)ep.grad_mask_t + (int64_t)col0 * ep.ld_t + row0 : nullptr;
  bf16x4 mk[2][MT][4];
  if (HAND && ym) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) mk[0][i][vq] = *(const bf16x4*)(ym + i * 32 + vq * 8);
    }
  }
#pragma unroll
  for (int j = 0; j < TI; ++j) {
    if (!FULL && col0 + j * 32 >= N) continue;
    const float bias = ep.e.bias ? ep.e.bias[col0 + j * 32] : 0.f;
    if (HAND && ym && j + 1 < TI) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) mk[(j + 1) & 1][i][vq] = *(const bf16x4*)(ym + (int64_t)(j + 1) * 32 * ep.ld_t + i * 32 + vq * 8);
      }
    }
    float csum[(TI + 1) / 2];
#pragma unroll
    for (int b = 0; b < (TI + 1) / 2; ++b) csum[b] = 0.f;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
      // keep the scheduler from hoisting every tile's loads to the top: the accumulators fill the register file
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        bf16x4 packed;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = i * 32 + vq * 8 + e;
          float x = acc[i][j][vq * 4 + e];
          if (HAND) {
            if (ym) x = (ep.e.act_param < (float)mk[j & 1][HAND ? i : 0][vq][e] ? 1.0f : 0.0f) * x;
            csum[i / 2] += x;
          }
          if (FULL || row0 + r < M) {
            if (ep.e.bias) x = x + bias;
            if (MODE == SN_ACT_SIGMOID) x = fast_sigmoid(x);
            else if (MODE == SN_ACT_TANH) x = fast_tanh(x);
            else if (MODE == SN_ACT_RELU) x = fmaxf(ep.e.act_param, x);
            else if (MODE < 0) x = bf_act(ep.e.act, x, ep.e.act_param);
            if (out) out[r * ldo + j * 32] = x;
            if (obf) obf[r * ldo + j * 32] = (bf16)x;
          }
          packed[e] = (bf16)x;
        }
        // 4 consecutive rows of one column are 8 contiguous bytes of the transposed tile
        if (transposed) *(bf16x4*)(stage + (j * 32 + l32) * PITCH + (i * 32 + vq * 8 + lhi * 4) * 2) = packed;
      }
    }
    if (HAND && ep.col_partials) {  // this column's sums over the wavefront's 64-row blocks: the two half-waves hold 4 rows of every 8 each
#pragma unroll
      for (int b = 0; b < (TI + 1) / 2; ++b) {
        const float t = csum[b] + __shfl_xor(csum[b], 32, 64);
        if (lhi == 0) ep.col_partials[(int64_t)(mbase / 64 + b) * N + col0 + j * 32] = t;
      }
    }
  }
  if (transposed) {
    // C^T leaves through LDS so that every store instruction writes whole 16-byte chunks of contiguous rows:
    // a lane takes 8 rows of one column, 64 lanes cover 64 / (WT/8) columns.
    constexpr int CH = WT / 8;         // 16-byte chunks per staged column
    constexpr int CPI = 64 / CH;       // columns per store instruction
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's staging writes are done (LDS is in-order per wave)
    const int ch = lane % CH, cc = lane / CH;
    bf16* obt = (bf16*)ep.out_bf_t;
#pragma unroll 4
    for (int c = 0; c < WT; c += CPI) {
      const int col = c + cc;
      const bf16x8 v = *(const bf16x8*)(stage + col * PITCH + ch * 16);
      if (FULL || (nbase + col < N && mbase + ch * 8 < M))
        *(bf16x8*)(obt + (int64_t)(nbase + col) * ep.ld_t + mbase + ch * 8) = v;
    }
  }
}

template <int WT, int MODE>
__device__ __forceinline__ void gemm_bf16_tn_body(const bf16* __restrict__ A, int64_t lda, const bf16* __restrict__ Bt, int64_t ldb,
                                                  int M, int N, int K, const EpilogueBf16& ep, int tiles_m, int tiles_n) {
  constexpr int BT = 2 * WT;        // block tile edge
  constexpr int TI = WT / 32;       // MFMA tiles per wavefront edge
  constexpr int ISSUES = BT / 32;   // LDS-load issues per wavefront per operand per stage (8 rows of 128 B each)
  constexpr int STAGE = BT * 128;   // bytes of one operand tile
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* sA = smem;                  // [2][STAGE]
  char* sB = smem + 2 * STAGE;      // [2][STAGE]

  // Tile order.  Consecutive workgroup ids land on different XCDs (8, each with its own L2), so first give
  // every XCD a contiguous run of tile numbers, then walk the tiles in groups of 4 tile-rows, column by
  // column: the 32 tiles an XCD works on at a time then form a 4 x 8 patch that shares 4 A panels and
  // 8 B panels in that XCD's L2.
  int t = blockIdx.x;
  const int total = tiles_m * tiles_n;
  if ((total & 7) == 0) t = (t & 7) * (total >> 3) + (t >> 3);
  constexpr int GROUP = 4;
  const int per_group = GROUP * tiles_n;
  const int first_m = (t / per_group) * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int tm = first_m + (t % per_group) % gsz, tn = (t % per_group) / gsz;
  const int m0 = tm * BT, n0 = tn * BT;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS load targets go through M0
  const int l32 = lane & 31, lhi = lane >> 5;
  const int wm = (wave >> 1) * WT, wn = (wave & 1) * WT;

  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(A, (uint32_t)(((int64_t)(M - 1) * lda + K) * 2));
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(Bt, (uint32_t)(((int64_t)(N - 1) * ldb + K) * 2));

  // Staging map: issue q of wavefront w fills tile rows w*(BT/4) + 8q .. +7 (1 KiB of LDS, lane l at +16 l).
  // LDS position (row r, physical chunk p) must hold logical chunk p ^ f(r), so that is what the lane fetches.
  const int srow = lane >> 3, pchunk = lane & 7;
  int lchunk[2];  // logical chunk for even / odd 8-row groups (f(r) = (r & 7) ^ ((r >> 3) & 1))
  lchunk[0] = pchunk ^ srow;
  lchunk[1] = pchunk ^ srow ^ 1;
  const int r0 = wave * (BT / 4) + srow;                     // tile row of issue 0; issue q adds 8q
  const int qa = (M - m0 - r0 + 7) >> 3, qb = (N - n0 - r0 + 7) >> 3;  // issues q >= qa / qb fall past the matrix
  const uint32_t a0 = (uint32_t)(((int64_t)(m0 + r0) * lda) * 2), b0 = (uint32_t)(((int64_t)(n0 + r0) * ldb) * 2);
  const uint32_t astep = (uint32_t)(lda * 16), bstep = (uint32_t)(ldb * 16);  // 8 rows in bytes
  // One 1 KiB LDS-bound load: issue q of this wavefront for stage k0 of operand A / B.  A k0 at or past K
  // gives out-of-range offsets, which the buffer load answers with zeros and no memory traffic.
  // K is a multiple of 8, so a 16-byte chunk lies inside or outside its row as a whole.
  auto issue_a = [&](int q, int k0, int buf) {
    const int kc = k0 + lchunk[q & 1] * 8;
    const uint32_t off = (q < qa && kc < K) ? a0 + q * astep + (uint32_t)kc * 2 : OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_ptr)(sA + buf * STAGE + wave * (BT / 4) * 128 + q * 1024), 16, (int)off, 0, 0, 0);
  };
  auto issue_b = [&](int q, int k0, int buf) {
    const int kc = k0 + lchunk[q & 1] * 8;
    const uint32_t off = (q < qb && kc < K) ? b0 + q * bstep + (uint32_t)kc * 2 : OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_ptr)(sB + buf * STAGE + wave * (BT / 4) * 128 + q * 1024), 16, (int)off, 0, 0, 0);
  };

  f16v acc[TI][TI];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TI; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  bf16x8 f0a[TI], f0b[TI], f1a[TI], f1b[TI];
  // Fragment r of k sub-step s (16 k-values) of the stage in buffer `buf`, in the order the MFMAs of the next
  // sub-step want them: A0, B0 .. B(TI-1), A1 .. A(TI-1).
#define SN_READ_ONE(FA, FB, buf, s, r)                                                                              \
  {                                                                                                                 \
    if ((r) == 0) FA[0] = *(const bf16x8*)(sA + (buf) * STAGE + swz(wm + l32, (s) * 2 + lhi));                       \
    else if ((r) <= TI) FB[(r) - 1] = *(const bf16x8*)(sB + (buf) * STAGE + swz(wn + ((r) - 1) * 32 + l32, (s) * 2 + lhi)); \
    else FA[(r) - TI] = *(const bf16x8*)(sA + (buf) * STAGE + swz(wm + ((r) - TI) * 32 + l32, (s) * 2 + lhi));       \
  }
#define SN_FENCE() __builtin_amdgcn_sched_barrier(0)
  // One k sub-step: TI*TI MFMAs in pairs; behind each pair go two fragment reads for the next sub-step
  // (DO_READ) and this pair's share of the stage loads of operand LOAD (0 none, 1 A, 2 B), so that LDS reads
  // and global loads are issued in the shadow of the matrix cores instead of between their bursts.
  constexpr int NG = TI * TI / 2, PPR = TI / 2, LPG = ISSUES / NG;
#define SN_SUBSTEP(CA, CB, NA, NB, DO_READ, rbuf, rs, LOAD, lk0, lbuf)                                               \
  {                                                                                                                 \
    _Pragma("unroll") for (int g = 0; g < NG; ++g) {                                                                 \
      const int i_ = g / PPR, j_ = (g % PPR) * 2;                                                                   \
      acc[i_][j_] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(CA[i_], CB[j_], acc[i_][j_], 0, 0, 0);                   \
      acc[i_][j_ + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(CA[i_], CB[j_ + 1], acc[i_][j_ + 1], 0, 0, 0);       \
      if (DO_READ) {                                                                                                \
        _Pragma("unroll") for (int r_ = 2 * g; r_ < 2 * g + 2; ++r_)                                                 \
          if (r_ < 2 * TI) SN_READ_ONE(NA, NB, rbuf, rs, r_);                                                       \
      }                                                                                                             \
      if ((LOAD) == 1) { _Pragma("unroll") for (int q_ = g * LPG; q_ < (g + 1) * LPG; ++q_) issue_a(q_, lk0, lbuf); } \
      if ((LOAD) == 2) { _Pragma("unroll") for (int q_ = g * LPG; q_ < (g + 1) * LPG; ++q_) issue_b(q_, lk0, lbuf); } \
      SN_FENCE();                                                                                                   \
    }                                                                                                               \
  }
  // all of this wavefront's LDS-bound loads have landed, then everybody's
#define SN_PUBLISH()                      \
  {                                       \
    __builtin_amdgcn_s_waitcnt(0);        \
    __syncthreads();                      \
  }

  // Pipeline over k stages of 64 (4 sub-steps of 16) and two LDS buffers.  One barrier per stage, before
  // sub-step 3: it publishes stage kt+1 and frees the current buffer.  The A half of stage kt+2 is loaded
  // into the freed buffer during sub-step 3, the B half during sub-step 0 of the next stage, one load
  // behind every MFMA pair; sub-step 3 also covers the first fragment reads of stage kt+1.
  const int nk = (K + GBK - 1) / GBK;
#pragma unroll
  for (int q = 0; q < ISSUES; ++q) { issue_a(q, 0, 0); issue_b(q, 0, 0); }
  SN_PUBLISH();
#pragma unroll
  for (int q = 0; q < ISSUES; ++q) issue_a(q, GBK, 1);
#pragma unroll
  for (int r = 0; r < 2 * TI; ++r) SN_READ_ONE(f0a, f0b, 0, 0, r);
  SN_FENCE();
  for (int kt = 0; kt + 1 < nk; ++kt) {
    const int buf = kt & 1;
    SN_SUBSTEP(f0a, f0b, f1a, f1b, true, buf, 1, 2, (kt + 1) * GBK, buf ^ 1);
    SN_SUBSTEP(f1a, f1b, f0a, f0b, true, buf, 2, 0, 0, 0);
    SN_SUBSTEP(f0a, f0b, f1a, f1b, true, buf, 3, 0, 0, 0);
    SN_PUBLISH();
    SN_SUBSTEP(f1a, f1b, f0a, f0b, true, buf ^ 1, 0, 1, (kt + 2) * GBK, buf);
  }
  {
    const int buf = (nk - 1) & 1;
    SN_SUBSTEP(f0a, f0b, f1a, f1b, true, buf, 1, 0, 0, 0);
    SN_SUBSTEP(f1a, f1b, f0a, f0b, true, buf, 2, 0, 0, 0);
    SN_SUBSTEP(f0a, f0b, f1a, f1b, true, buf, 3, 0, 0, 0);
    SN_SUBSTEP(f1a, f1b, f0a, f0b, false, 0, 0, 0, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0);  // the zero-filling loads past the last stage have landed before LDS is reused
#undef SN_READ_ONE
#undef SN_SUBSTEP
#undef SN_FENCE
#undef SN_PUBLISH

  // accumulator element v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
  char* stage = smem + wave * (WT * tr_pitch<WT>());
  if (ep.out_bf_t) __syncthreads();  // the staging areas overlay the operand tiles other wavefronts may still be reading
  // The epilogue mode is a template parameter of the KERNEL (the host picks it): with one full-tile and one
  // edge-tile instantiation per kernel the accumulators stay in registers; a run-time switch over all modes
  // inside one kernel makes the compiler demote them to scratch memory.
  // The 256x256 kernel is only launched on outputs it tiles exactly: adding the bounds-checked variant next to
  // the full-tile one also pushes its 256 accumulators out of the register file.
  if (WT == 128 || (m0 + BT <= M && n0 + BT <= N)) store_tile<MODE, true, TI>(acc, ep, m0 + wm, n0 + wn, lane, M, N, stage);
  else store_tile<-1, false, TI>(acc, ep, m0 + wm, n0 + wn, lane, M, N, stage);  // edge tiles: bounds-checked, mode picked at run time
}

// 256x256 tiles: 256 accumulator registers per lane, one wavefront per SIMD
template <int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_bf16_tn_256(const bf16* __restrict__ A, int64_t lda, const bf16* __restrict__ Bt, int64_t ldb, int M, int N, int K,
                      EpilogueBf16 ep, int tiles_m, int tiles_n) {
  gemm_bf16_tn_body<128, MODE>(A, lda, Bt, ldb, M, N, K, ep, tiles_m, tiles_n);
}
// 128x128 tiles: two workgroups per CU
template <int MODE>
__global__ __launch_bounds__(256, 2)
void gemm_bf16_tn_128(const bf16* __restrict__ A, int64_t lda, const bf16* __restrict__ Bt, int64_t ldb, int M, int N, int K,
                      EpilogueBf16 ep, int tiles_m, int tiles_n) {
  gemm_bf16_tn_body<64, MODE>(A, lda, Bt, ldb, M, N, K, ep, tiles_m, tiles_n);
}

template <int MODE>
static int launch_mode(sn_ctx* ctx, const bf16* a, int64_t lda, const bf16* bt, int64_t ldb, int M, int N, int K, const EpilogueBf16& ep) {
  const int64_t big_tiles = ceil_div(M, 256) * ceil_div(N, 256);
  if (big_tiles >= ctx->compute_units && M % 256 == 0 && N % 256 == 0) {
    const size_t smem = 4 * 128 * tr_pitch<128>() > 4 * 256 * 128 ? 4 * 128 * tr_pitch<128>() : 4 * 256 * 128;
    SN_TRY(allow_dynamic_lds(ctx, (const void*)gemm_bf16_tn_256<MODE>, smem));
    const int tm = (int)ceil_div(M, 256), tn = (int)ceil_div(N, 256);
    LaunchScope scope(ctx, MODE == MODE_HANDOVER ? "gemm_bf16_256_handover" : "gemm_bf16_256", M, N, K);
    hipLaunchKernelGGL(gemm_bf16_tn_256<MODE>, dim3((unsigned)(tm * tn)), dim3(256), smem, ctx->stream, a, lda, bt, ldb, M, N, K, ep, tm, tn);
  } else {
    const size_t smem = 4 * 64 * tr_pitch<64>() > 4 * 128 * 128 ? 4 * 64 * tr_pitch<64>() : 4 * 128 * 128;
    SN_TRY(allow_dynamic_lds(ctx, (const void*)gemm_bf16_tn_128<MODE>, smem));
    const int tm = (int)ceil_div(M, 128), tn = (int)ceil_div(N, 128);
    LaunchScope scope(ctx, MODE == MODE_HANDOVER ? "gemm_bf16_128_handover" : "gemm_bf16_128", M, N, K);
    hipLaunchKernelGGL(gemm_bf16_tn_128<MODE>, dim3((unsigned)(tm * tn)), dim3(256), smem, ctx->stream, a, lda, bt, ldb, M, N, K, ep, tm, tn);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_gemm_bf16_tn(sn_ctx* ctx, const void* a, int64_t lda, const void* bt, int64_t ldb, int M, int N, int K, const EpilogueBf16& ep) {
  SN_REQUIRE(a && bt && (ep.e.out || ep.out_bf || ep.out_bf_t), "gemm_bf16: null operand");
  SN_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0, "gemm_bf16: K and the row pitches must be multiples of 8 (got K=%d)", K);
  SN_REQUIRE(((int64_t)M * lda + K) * 2 < (int64_t)1 << 31 && ((int64_t)N * ldb + K) * 2 < (int64_t)1 << 31,
             "gemm_bf16: an operand of %d x %d / %d x %d bf16 exceeds the 2 GiB a buffer descriptor may span", M, K, N, K);
  SN_REQUIRE((int64_t)M * ep.e.ldo < (int64_t)1 << 31 && (int64_t)N * ep.ld_t < (int64_t)1 << 31,
             "gemm_bf16: output of %d rows x pitch %lld exceeds 2^31 elements", M, (long long)ep.e.ldo);
  if (M <= 0 || N <= 0) return SN_OK;
  const bf16* A = (const bf16*)a;
  const bf16* B = (const bf16*)bt;
  if (ep.grad_handover) {
    SN_REQUIRE(M % 128 == 0 && N % 128 == 0 && ep.out_bf_t && ep.e.act == SN_ACT_IDENTITY && !ep.e.bias && ep.ld_t % 4 == 0,
               "gemm_bf16: the gradient hand-over needs full 128 x 128 tiles, a transposed output and a plain product (got %d x %d)", M, N);
    return launch_mode<MODE_HANDOVER>(ctx, A, lda, B, ldb, M, N, K, ep);
  }
  switch (ep.e.act) {
    case SN_ACT_SIGMOID: return launch_mode<SN_ACT_SIGMOID>(ctx, A, lda, B, ldb, M, N, K, ep);
    case SN_ACT_TANH: return launch_mode<SN_ACT_TANH>(ctx, A, lda, B, ldb, M, N, K, ep);
    case SN_ACT_RELU: return launch_mode<SN_ACT_RELU>(ctx, A, lda, B, ldb, M, N, K, ep);
    default: return launch_mode<SN_ACT_IDENTITY>(ctx, A, lda, B, ldb, M, N, K, ep);
  }
}

// ---------------------------------------------------------------------------- fp32 -> bf16 in both orientations
// out[r][c] and out_t[c][r] (either may be null) from src[r*ld + c]; when y != null the value cast is
// the activation gradient act'(y) * src, which is also written back to dz (fp32) when dz != null.
__global__ __launch_bounds__(256) void cast_transpose_kernel(const float* __restrict__ src, int64_t ld, int rows, int cols,
                                                              bf16* __restrict__ out, bf16* __restrict__ out_t,
                                                              const float* __restrict__ y, const bf16* __restrict__ y_bf, int act,
                                                              float act_param, float* __restrict__ dz, float* __restrict__ col_partials) {
  // 64x64 tile; a thread handles 4 consecutive columns of 4 rows (float4 in, 8-byte bf16x4 out), and on the
  // transposed side 4 consecutive rows of one column.  cols and rows are multiples of 4 (checked by the caller).
  __shared__ bf16 tile[64][68];
  __shared__ float colp[16][64];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tc = (threadIdx.x & 15) * 4, tr = threadIdx.x >> 4;
  f4 csum = {0.f, 0.f, 0.f, 0.f};  // this thread's 4 rows of its 4 columns (fp32 values, before rounding)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + tr + 16 * i, c = c0 + tc;
    f4 v = {0.f, 0.f, 0.f, 0.f};
    if (r < rows && c < cols) {
      v = *(const f4*)(src + (int64_t)r * ld + c);
      if (y || y_bf) {
        f4 yy;
        if (y) yy = *(const f4*)(y + (int64_t)r * ld + c);
        else {  // the layer's output only exists as the bf16 copy its successor reads (pitch = cols)
          const bf16x4 yb = *(const bf16x4*)(y_bf + (int64_t)r * cols + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) yy[e] = (float)yb[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = bf_act_grad(act, yy[e], v[e], act_param);
        if (dz) *(f4*)(dz + (int64_t)r * ld + c) = v;
      }
      bf16x4 b;
#pragma unroll
      for (int e = 0; e < 4; ++e) b[e] = (bf16)v[e];
      if (out) *(bf16x4*)(out + (int64_t)r * cols + c) = b;
    }
    csum += v;
#pragma unroll
    for (int e = 0; e < 4; ++e) tile[tr + 16 * i][tc + e] = (bf16)v[e];
  }
  if (!out_t) return;
  if (col_partials) {
#pragma unroll
    for (int e = 0; e < 4; ++e) colp[tr][tc + e] = csum[e];
  }
  __syncthreads();
  if (col_partials && threadIdx.x < 64 && c0 + threadIdx.x < cols) {  // column sums of this 64-row block, rows in a fixed order
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) t += colp[j][threadIdx.x];
    col_partials[(int64_t)blockIdx.y * cols + c0 + threadIdx.x] = t;
  }
  if (!out_t) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + tr + 16 * i, r = r0 + tc;  // column c of the source, rows r..r+3
    if (c < cols && r < rows) {
      bf16x4 b;
#pragma unroll
      for (int e = 0; e < 4; ++e) b[e] = tile[tc + e][tr + 16 * i];
      *(bf16x4*)(out_t + (int64_t)c * rows + r) = b;
    }
  }
}

int launch_cast_transpose(sn_ctx* ctx, const float* src, int64_t ld, int rows, int cols, void* out, void* out_t, const float* y,
                          int act, float act_param, float* dz, float* col_partials, const void* y_bf) {
  if (rows <= 0 || cols <= 0) return SN_OK;
  SN_REQUIRE(rows % 4 == 0 && cols % 4 == 0 && ld % 4 == 0, "cast_bf16: rows, cols and pitch must be multiples of 4");
  LaunchScope scope(ctx, (y || y_bf) ? "activation_backward_cast_bf16" : "cast_bf16");
  hipLaunchKernelGGL(cast_transpose_kernel, dim3((unsigned)ceil_div(cols, 64), (unsigned)ceil_div(rows, 64)), dim3(256), 0, ctx->stream,
                     src, ld, rows, cols, (bf16*)out, (bf16*)out_t, y, (const bf16*)y_bf, act, act_param, dz, col_partials);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
