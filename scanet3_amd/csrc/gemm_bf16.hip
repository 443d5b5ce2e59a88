// bf16 matrix-core GEMM for the wide Dense layers (fp32 master data, bf16 operands, fp32 accumulate).
//
// C[M,N] = sum_k A(m,k) B(n,k).  Each operand is either k-major (rows of its output index, k contiguous:
// element (r,k) at p[r*ld + k]) or index-major (rows of k, the output index contiguous: element (r,k) at
// p[k*ld + r]), so the three Dense products read the tensors as they lie and no transposed copy exists:
//   forward  Y  = X  W      A = X  [rows,in]  k-major       B = W  [in,out]    index-major
//   dX          = dZ W^T    A = dZ [rows,out] k-major       B = W  [in,out]    k-major
//   dW          = X^T dZ    A = X  [rows,in]  index-major   B = dZ [rows,out]  index-major
//
// Kernel shape: 256 threads = 4 wavefronts (2x2), wavefront tile (32 TM) x (32 TN) of v_mfma_f32_32x32x16_bf16
// (TM = TN = 4: 256 accumulator registers per lane, one wavefront per SIMD), k stage 64, two LDS stages.  Tiles
// travel HBM/L2 -> LDS with `buffer_load_dwordx4 ... lds` (no staging registers; rows past the matrix and the
// k tail arrive as zeros from the buffer descriptor's range check).  A k-major tile is [rows][128 B] with
// XOR-swizzled 16-byte chunks and feeds the matrix cores through ds_read_b128; an index-major tile is
// [64 k][rows * 2 B] with XOR-swizzled 32-byte pairs and is read with ds_read_b64_tr_b16, which hands every
// lane four consecutive k of its own row.  A workgroup walks several output tiles (persistent grid) and the stage
// ring runs on across tile boundaries: the first stages of the next tile load while a tile's results leave.
#include "common.hpp"

#include <type_traits>

namespace sn {

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s4v __attribute__((ext_vector_type(4)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int GBK = 64;  // k per stage

// k-major tile: byte offset of 16-byte chunk `chunk` of tile row `row`.  Any 8 consecutive rows of one logical
// chunk land on 8 different 16-byte bank groups of a 128-byte line, any 16 on 16 groups of a 256-byte double line.
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row & 7) ^ ((row >> 3) & 1))) << 4); }
// index-major tile: 16-byte chunk c of k-row k sits at chunk c ^ mn_xor(k) of that row.  The four k-rows a
// transposing read touches per 16 lanes move their 32-byte pairs to four different bank groups, whether the LDS
// serves 16 lanes (128 B) or 32 lanes (256 B) per cycle.
__device__ __forceinline__ int mn_xor(int k) { return (0x6530 >> ((k & 3) * 4) & 7) << 1; }  // pair index ^ {0, 3, 5, 6}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
constexpr uint32_t OOB = 0x80000000u;  // beyond any operand (operands are checked to be < 2 GiB)

typedef __attribute__((address_space(3))) void* lds_ptr;
typedef __attribute__((address_space(3))) s4v* lds_s4p;

__device__ __forceinline__ float bf_act_grad(int act, float y, float dy, float param) {
  switch (act) {
    case SN_ACT_SIGMOID: return (y * (1.0f - y)) * dy;
    case SN_ACT_TANH: return (1.0f - y * y) * dy;
    case SN_ACT_RELU: return (param < y ? 1.0f : 0.0f) * dy;
    default: return dy;
  }
}

// One transposing read, written as assembly: the compiler puts `s_waitcnt vmcnt(0)` in front of the builtin form
// whenever an LDS-bound global load is in flight (it cannot tell which one the read depends on), which would end the
// overlap of loads and matrix work.  The result is valid only after the `s_waitcnt lgkmcnt` the kernel issues itself.
// offset = BUF * STAGE + S * 16 * RB + H * 4 * RB must be an immediate: one case per (buffer, sub-step, half).
template <int RB, int STAGE>
__device__ __forceinline__ s4v tr_read(uint32_t addr, int buf, int s, int h) {
  s4v v;
#define SN_TR_CASE(B, S, H) \
  case ((B) * 8 + (S) * 2 + (H)): asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"((B) * STAGE + (S) * 16 * RB + (H) * 4 * RB)); break;
  switch (buf * 8 + s * 2 + h) {
    SN_TR_CASE(0, 0, 0) SN_TR_CASE(0, 0, 1) SN_TR_CASE(0, 1, 0) SN_TR_CASE(0, 1, 1) SN_TR_CASE(0, 2, 0) SN_TR_CASE(0, 2, 1) SN_TR_CASE(0, 3, 0) SN_TR_CASE(0, 3, 1)
    SN_TR_CASE(1, 0, 0) SN_TR_CASE(1, 0, 1) SN_TR_CASE(1, 1, 0) SN_TR_CASE(1, 1, 1) SN_TR_CASE(1, 2, 0) SN_TR_CASE(1, 2, 1) SN_TR_CASE(1, 3, 0) SN_TR_CASE(1, 3, 1)
    default: __builtin_unreachable();
  }
#undef SN_TR_CASE
  return v;
}
// s_waitcnt lgkmcnt(N) that the fragment halves named as operands are ordered behind
template <int N> __device__ __forceinline__ void wait_lgkm(s4v& a, s4v& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N> __device__ __forceinline__ void wait_lgkm(s4v& a, s4v& b, s4v& c, s4v& d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N> __device__ __forceinline__ void wait_lgkm(s4v& a, s4v& b, s4v& c, s4v& d, s4v& e, s4v& f) {
  asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f) : "n"(N));
}
template <typename... T>
__device__ __forceinline__ void wait_lgkm_n(int n, T&... h) {
  switch (n) {
    case 0: wait_lgkm<0>(h...); break;   case 1: wait_lgkm<1>(h...); break;   case 2: wait_lgkm<2>(h...); break;
    case 3: wait_lgkm<3>(h...); break;   case 4: wait_lgkm<4>(h...); break;   case 5: wait_lgkm<5>(h...); break;
    case 6: wait_lgkm<6>(h...); break;   case 7: wait_lgkm<7>(h...); break;   case 8: wait_lgkm<8>(h...); break;
    case 9: wait_lgkm<9>(h...); break;   case 10: wait_lgkm<10>(h...); break; case 11: wait_lgkm<11>(h...); break;
    case 12: wait_lgkm<12>(h...); break; case 13: wait_lgkm<13>(h...); break; case 14: wait_lgkm<14>(h...); break;
    default: wait_lgkm<15>(h...); break;
  }
}

// The fragment reads of a sub-step, in issue order: behind MFMA pair g first the B fragments j with j NG / TN == g,
// then A fragment i if g is the last pair of row i.  wait_before(g) = how many transposing reads (two per
// index-major fragment; the compiler keeps its own count for k-major ones) may still be in flight when pair g of the
// NEXT sub-step starts, such that the index-major fragments that pair multiplies have landed; -1: nothing to wait
// for, or an earlier pair of the sub-step already waited for as much.
template <int TM, int TN, bool AMN, bool BMN>
struct FragSchedule {
  static constexpr int NG = TM * TN / 2, PPR = TN / 2;
  // position in issue order of A fragment i / B fragment j, and the number of transposing reads issued up to and
  // including each position
  static constexpr int pos_a(int i) { int p = 0; for (int g = 0; g < NG; ++g) { for (int j = 0; j < TN; ++j) if ((j * NG) / TN == g) ++p; if (g % PPR == PPR - 1) { if (g / PPR == i) return p; ++p; } } return -1; }
  static constexpr int pos_b(int jq) { int p = 0; for (int g = 0; g < NG; ++g) { for (int j = 0; j < TN; ++j) if ((j * NG) / TN == g) { if (j == jq) return p; ++p; } if (g % PPR == PPR - 1) ++p; } return -1; }
  static constexpr int reads_through(int pos) {  // transposing reads issued at positions 0 .. pos
    int p = 0, n = 0;
    for (int g = 0; g < NG; ++g) { for (int j = 0; j < TN; ++j) if ((j * NG) / TN == g) { if (p <= pos && BMN) n += 2; ++p; } if (g % PPR == PPR - 1) { if (p <= pos && AMN) n += 2; ++p; } }
    return n;
  }
  static constexpr int reads_in_groups_before(int gi) {  // transposing reads issued behind pairs 0 .. gi-1
    int n = 0;
    for (int g = 0; g < gi; ++g) { for (int j = 0; j < TN; ++j) if ((j * NG) / TN == g && BMN) n += 2; if (g % PPR == PPR - 1 && AMN) n += 2; }
    return n;
  }
  static constexpr int latest_needed(int gi) {  // last position among the index-major fragments pair gi multiplies, -1 if none
    const int i = gi / PPR, j = (gi % PPR) * 2;
    int latest = -1;
    if (AMN && pos_a(i) > latest) latest = pos_a(i);
    if (BMN && pos_b(j) > latest) latest = pos_b(j);
    if (BMN && pos_b(j + 1) > latest) latest = pos_b(j + 1);
    return latest;
  }
  static constexpr int wait_before(int gi) {
    const int latest = latest_needed(gi);
    if (latest < 0) return -1;
    for (int g = 0; g < gi; ++g) if (latest_needed(g) >= latest) return -1;
    const int total = reads_through(TM + TN - 1);
    const int n = (total - reads_through(latest)) + reads_in_groups_before(gi);
    return n > 15 ? 15 : n;
  }
};

// Epilogue modes (compile-time).
constexpr int MODE_F32 = 0;       // fp32 result (+ bias, ReLU), optionally a bf16 copy; any shape (bounds-checked unless FULL)
constexpr int MODE_BF16 = 1;      // bf16 result only (+ bias, ReLU at 0) and the ReLU's sign bits, full tiles
constexpr int MODE_HANDOVER = 2;  // MODE_BF16 for a dX product that writes the dZ of the layer below (see GemmBf16Args)

struct GemmBf16Args {
  const bf16* a; const bf16* b;
  int64_t lda, ldb;
  int M, N, K;
  int tiles_m, tiles_n;
  float* out;            // fp32 [M, ldo] (MODE_F32)
  bf16* out_bf;          // bf16 [M, ldo]
  int64_t ldo;
  const float* bias;     // per column, may be null
  float relu_at;         // threshold of the ReLU (ACT = relu)
  // MODE_BF16 with ReLU: one bit per output value, 1 where the value passed the ReLU, in the order the lanes of the
  // 256 x 256 tiling hold them ([tile][wavefront][8 words][lane]); MODE_HANDOVER reads the same words back.
  uint32_t* signs_out;
  const uint32_t* signs_in;
  float* col_partials;   // MODE_HANDOVER: [M / 64, N] column sums of every 64-row block of the fp32 values
};

template <int TM, int TN, bool AMN, bool BMN, int MODE, int ACT, bool FULL>
__device__ __forceinline__ void gemm_bf16_body(const GemmBf16Args& g) {
  constexpr int BM = 64 * TM, BN = 64 * TN;        // block tile
  constexpr int STAGE_A = BM * 128, STAGE_B = BN * 128;  // bytes of one operand stage, either layout
  constexpr int IA = 2 * TM, IB = 2 * TN;          // LDS-load issues per wavefront, operand and stage (1 KiB each)
  static_assert(MODE == MODE_F32 || (TM == 4 && TN == 4 && FULL), "the bf16-only epilogues are built for full 256 x 256 tiles");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const sA = smem;                 // [2][STAGE_A]
  char* const sB = smem + 2 * STAGE_A;   // [2][STAGE_B]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS load targets go through M0
  const int l32 = lane & 31, lhi = lane >> 5;
  const int wm = (wave >> 1) * (32 * TM), wn = (wave & 1) * (32 * TN);
  const int M = g.M, N = g.N, K = g.K;
  const int nk = ((K + GBK - 1) / GBK + 1) & ~1;  // stages per tile, padded to an even count (a padding stage loads zeros)

  // ------------------------------------------------------------------ this workgroup's tiles
  // Consecutive workgroup ids land on different XCDs (8, each with its own L2): every XCD gets a contiguous run of
  // tile numbers, and tile numbers walk the output in groups of 4 tile-rows, column by column, so the tiles an XCD
  // works on at a time form a patch that shares few A and B panels in its L2.
  const int total = g.tiles_m * g.tiles_n;
  int first, stride, count;
  if ((gridDim.x & 7) == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
    const int base = total >> 3, rem = total & 7;
    const int lo = xcd * base + min(xcd, rem), n_x = base + (xcd < rem ? 1 : 0);
    first = lo + slot; stride = slots; count = slot < n_x ? (n_x - slot + slots - 1) / slots : 0;
  } else {
    first = blockIdx.x; stride = gridDim.x; count = (int)blockIdx.x < total ? (total - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
  }
  if (count == 0) return;
  auto tile_origin = [&](int t, int& m0, int& n0) {
    constexpr int GROUP = 4;
    const int per_group = GROUP * g.tiles_n;
    const int first_m = (t / per_group) * GROUP;
    const int gsz = min(g.tiles_m - first_m, GROUP);
    m0 = (first_m + (t % per_group) % gsz) * BM;
    n0 = ((t % per_group) / gsz) * BN;
  };

  // ------------------------------------------------------------------ global -> LDS
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.a, (uint32_t)((AMN ? (int64_t)(K - 1) * g.lda + M : (int64_t)(M - 1) * g.lda + K) * 2));
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.b, (uint32_t)((BMN ? (int64_t)(K - 1) * g.ldb + N : (int64_t)(N - 1) * g.ldb + K) * 2));
  // A load cursor: where the next stage of this operand comes from.  base[p]: this lane's byte offset for issue 0
  // (p = parity of the issue number) at k = 0 of the cursor's tile; issue q adds q * qstep, stage k0 adds k0 * kmul.
  struct Cursor { uint32_t base[2]; int k0; int next_tile; };
  // k-major: issue q of wavefront w fills tile rows w*(rows/4) + 8q .. +7; LDS position (row, physical chunk p) holds
  // logical chunk p ^ f(row).  Rows past the matrix lie past the descriptor's range by themselves (ld >= K); a chunk
  // past K inside a row does not, so that is checked per issue.
  // index-major: issue q fills k-rows w*16 + kpi*q .. of the stage (kpi = 1024 / row bytes); LDS position (k, physical
  // chunk p) holds logical chunk p ^ mn_xor(k).  k-rows past K are out of range by themselves; a chunk past the last
  // column is not, so the lane's base is out of range then.
  auto setup = [&](auto MN_, auto T_, Cursor& c, int origin, int64_t ld, int extent, int klane[2]) {
    constexpr bool MN = decltype(MN_)::value;
    constexpr int T = decltype(T_)::value;
    if (c.next_tile >= count) { c.base[0] = c.base[1] = OOB; c.k0 = 0; return; }
    if (!MN) {
      const int srow = lane >> 3, pchunk = lane & 7;
      const int row = wave * (16 * T) + srow;
      klane[0] = (pchunk ^ srow) * 8; klane[1] = (pchunk ^ srow ^ 1) * 8;
      const uint32_t rowoff = (uint32_t)(((int64_t)(origin + row) * ld) * 2);
      c.base[0] = rowoff + klane[0] * 2; c.base[1] = rowoff + klane[1] * 2;
    } else {
      constexpr int RB = 128 * T;          // bytes per k-row of the tile
      constexpr int CPR = RB / 16;         // chunks per k-row
      constexpr int KPI = 1024 / RB;       // k-rows per issue
      const int kb = wave * 16 + lane / CPR, pc = lane % CPR;
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int k = kb + KPI * p;        // k-row of issue p within the stage; issue q is 2-periodic in k & 3 (KPI = 2) or constant (KPI = 4)
        const int col = origin + 8 * (pc ^ mn_xor(k));
        c.base[p] = col < extent ? (uint32_t)(((int64_t)kb * ld + col) * 2) : OOB;
      }
      klane[0] = klane[1] = 0;
    }
    c.k0 = 0;
  };
  int klaneA[2], klaneB[2];
  const uint32_t qstepA = AMN ? (uint32_t)((1024 / (128 * TM)) * g.lda * 2) : (uint32_t)(g.lda * 16);
  const uint32_t qstepB = BMN ? (uint32_t)((1024 / (128 * TN)) * g.ldb * 2) : (uint32_t)(g.ldb * 16);
  const uint32_t kmulA = AMN ? (uint32_t)(g.lda * 2) : 2u, kmulB = BMN ? (uint32_t)(g.ldb * 2) : 2u;
  Cursor ca, cb;
  ca.next_tile = cb.next_tile = 0;
  auto cursor_tile_a = [&]() {
    int m0 = 0, n0 = 0;
    if (ca.next_tile < count) tile_origin(first + ca.next_tile * stride, m0, n0);
    setup(std::integral_constant<bool, AMN>{}, std::integral_constant<int, TM>{}, ca, m0, g.lda, M, klaneA);
    ++ca.next_tile;
  };
  auto cursor_tile_b = [&]() {
    int m0 = 0, n0 = 0;
    if (cb.next_tile < count) tile_origin(first + cb.next_tile * stride, m0, n0);
    setup(std::integral_constant<bool, BMN>{}, std::integral_constant<int, TN>{}, cb, n0, g.ldb, N, klaneB);
    ++cb.next_tile;
  };
  cursor_tile_a();
  cursor_tile_b();
  auto issue_a = [&](int q, int buf) {
    uint32_t off = ca.base[q & 1] + (uint32_t)q * qstepA + (uint32_t)ca.k0 * kmulA;
    if (!AMN && ca.k0 + klaneA[q & 1] >= K) off = OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_ptr)(sA + buf * STAGE_A + wave * (STAGE_A / 4) + q * 1024), 16, (int)off, 0, 0, 0);
  };
  auto issue_b = [&](int q, int buf) {
    uint32_t off = cb.base[q & 1] + (uint32_t)q * qstepB + (uint32_t)cb.k0 * kmulB;
    if (!BMN && cb.k0 + klaneB[q & 1] >= K) off = OOB;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_ptr)(sB + buf * STAGE_B + wave * (STAGE_B / 4) + q * 1024), 16, (int)off, 0, 0, 0);
  };
  // after the last issue of a stage the cursor moves one stage on; the pipeline below moves it to the workgroup's
  // next tile (cursor_tile_*) between the stages where the loads cross a tile boundary
  auto advance_a = [&]() { ca.k0 += GBK; };
  auto advance_b = [&]() { cb.k0 += GBK; };

  // ------------------------------------------------------------------ LDS -> fragments
  // k-major fragment of sub-step s: ds_read_b128 of chunk 2s + lane/32 of row (32 i + lane%32): per-lane offsets per s.
  // index-major fragment: two transposing reads; lane l (16-lane group gq = l/16, source role r = l%16) addresses the
  // four rows m = 16 (gq & 1) + 4 (r & 3) .. +3 of k-row 16 s + 8 (gq >> 1) + 4 h + r / 4 (h = first / second read) and
  // receives row 16 (gq & 1) + r of k-rows 16 s + 8 (l / 32) + 4 h .. +3: the k-values the k-major fragment of the
  // other operand holds in the same order.
  int fa_off[4], fb_off[4];  // k-major: per s; index-major: per i (or j)
  {
    const int f = (l32 & 7) ^ ((l32 >> 3) & 1);
    const int gq = lane >> 4, r = lane & 15;
    const int xl = mn_xor(r >> 2);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (!AMN) fa_off[s] = (wm + l32) * 128 + (((s * 2 + lhi) ^ f) << 4);
      else fa_off[s] = s < TM ? ((8 * (gq >> 1) + (r >> 2)) * (128 * TM) + ((((wm >> 3) + 4 * s + 2 * (gq & 1) + ((r & 3) >> 1)) ^ xl) << 4) + (r & 1) * 8) : 0;
      if (!BMN) fb_off[s] = (wn + l32) * 128 + (((s * 2 + lhi) ^ f) << 4);
      else fb_off[s] = s < TN ? ((8 * (gq >> 1) + (r >> 2)) * (128 * TN) + ((((wn >> 3) + 4 * s + 2 * (gq & 1) + ((r & 3) >> 1)) ^ xl) << 4) + (r & 1) * 8) : 0;
    }
  }
  const uint32_t lds_a = (uint32_t)(size_t)(lds_ptr)sA, lds_b = (uint32_t)(size_t)(lds_ptr)sB;
  auto read_a_km = [&](int buf, int s, int i) -> bf16x8 { return *(const bf16x8*)(sA + buf * STAGE_A + fa_off[s] + i * 4096); };
  auto read_b_km = [&](int buf, int s, int j) -> bf16x8 { return *(const bf16x8*)(sB + buf * STAGE_B + fb_off[s] + j * 4096); };
  auto read_a_mn = [&](int buf, int s, int i, int h) -> s4v { return tr_read<128 * TM, STAGE_A>(lds_a + fa_off[i], buf, s, h); };
  auto read_b_mn = [&](int buf, int s, int j, int h) -> s4v { return tr_read<128 * TN, STAGE_B>(lds_b + fb_off[j], buf, s, h); };

  f16v acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  };
  zero_acc();

  // the row pitch as a per-lane value the compiler cannot fold: row offsets are then made where they are used
  // instead of as hundreds of scalars computed (and spilled) up front
  uint32_t ldo_v = (uint32_t)g.ldo;
  asm volatile("" : "+v"(ldo_v));

  // B fragments are double-buffered; an A fragment's register is free again as soon as the last MFMA of its row of
  // sub-tiles has been issued, so the A fragments of the next sub-step are read into the same registers.
  // k-major fragments as the compiler's own loads; index-major ones as the two halves the transposing reads deliver
  bf16x8 fa[AMN ? 1 : TM], fb[2][BMN ? 1 : TN];
  s4v fa_lo[AMN ? TM : 1], fa_hi[AMN ? TM : 1], fb_lo[2][BMN ? TN : 1], fb_hi[2][BMN ? TN : 1];
  auto frag_of = [&](const s4v& lo, const s4v& hi) -> bf16x8 {
    const s8v v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
  };
#define SN_FENCE() __builtin_amdgcn_sched_barrier(0)
  constexpr int NG = TM * TN / 2, PPR = TN / 2;
  typedef FragSchedule<TM, TN, AMN, BMN> Sched;
  // One k sub-step: TM*TN MFMAs in pairs (row of sub-tiles by row) from the A fragments and B fragment set CUR;
  // behind each pair go this pair's share of the fragment reads for the next sub-step (buffer RBUF, sub-step RS:
  // B fragment j behind pair j NG / TN, A fragment i behind the last pair of row i) and of the stage loads of operand
  // LOAD (0 none, 1 A, 2 B) into buffer LBUF.
  auto substep = [&](auto CUR_, auto DO_READ_, auto RBUF_, auto RS_, auto LOAD_, auto LBUF_) {
    constexpr int CUR = decltype(CUR_)::value, RBUF = decltype(RBUF_)::value, RS = decltype(RS_)::value;
    constexpr int LOAD = decltype(LOAD_)::value, LBUF = decltype(LBUF_)::value;
    constexpr bool DO_READ = decltype(DO_READ_)::value;
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
      const int i_ = gi / PPR, j_ = (gi % PPR) * 2;
      if constexpr (AMN || BMN) {
        const int w = Sched::wait_before(gi);
        if (w >= 0) {
          if constexpr (AMN && BMN) wait_lgkm_n(w, fa_lo[i_], fa_hi[i_], fb_lo[CUR][j_], fb_hi[CUR][j_], fb_lo[CUR][j_ + 1], fb_hi[CUR][j_ + 1]);
          else if constexpr (AMN) wait_lgkm_n(w, fa_lo[i_], fa_hi[i_]);
          else wait_lgkm_n(w, fb_lo[CUR][j_], fb_hi[CUR][j_], fb_lo[CUR][j_ + 1], fb_hi[CUR][j_ + 1]);
        }
      }
      const bf16x8 av = AMN ? frag_of(fa_lo[AMN ? i_ : 0], fa_hi[AMN ? i_ : 0]) : fa[AMN ? 0 : i_];
      const bf16x8 bv0 = BMN ? frag_of(fb_lo[CUR][BMN ? j_ : 0], fb_hi[CUR][BMN ? j_ : 0]) : fb[CUR][BMN ? 0 : j_];
      const bf16x8 bv1 = BMN ? frag_of(fb_lo[CUR][BMN ? j_ + 1 : 0], fb_hi[CUR][BMN ? j_ + 1 : 0]) : fb[CUR][BMN ? 0 : j_ + 1];
      acc[i_][j_] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv0, acc[i_][j_], 0, 0, 0);
      acc[i_][j_ + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv1, acc[i_][j_ + 1], 0, 0, 0);
      if constexpr (DO_READ) {
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
          if ((jj * NG) / TN == gi) {
            if constexpr (BMN) { fb_lo[CUR ^ 1][jj] = read_b_mn(RBUF, RS, jj, 0); fb_hi[CUR ^ 1][jj] = read_b_mn(RBUF, RS, jj, 1); }
            else fb[CUR ^ 1][jj] = read_b_km(RBUF, RS, jj);
          }
        if ((gi % PPR) == PPR - 1) {
          if constexpr (AMN) { fa_lo[i_] = read_a_mn(RBUF, RS, i_, 0); fa_hi[i_] = read_a_mn(RBUF, RS, i_, 1); }
          else fa[i_] = read_a_km(RBUF, RS, i_);
        }
      }
      if constexpr (LOAD == 1) {
#pragma unroll
        for (int q_ = gi * (IA / NG); q_ < (gi + 1) * (IA / NG); ++q_) issue_a(q_, LBUF);
      }
      if constexpr (LOAD == 2) {
#pragma unroll
        for (int q_ = gi * (IB / NG); q_ < (gi + 1) * (IB / NG); ++q_) issue_b(q_, LBUF);
      }
      SN_FENCE();
    }
    if constexpr (LOAD == 1) advance_a();
    if constexpr (LOAD == 2) advance_b();
  };
  // all of this wavefront's LDS-bound loads have landed, then everybody's
  auto publish = [&]() {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  };
  // One stage out of buffer BUF: sub-steps 0..3.  The barrier before sub-step 3 publishes the next stage (other
  // buffer) and frees this one: the A half of the stage after next is loaded into it during sub-step 3, the B half
  // during sub-step 0 of the next stage, one load behind every MFMA pair; sub-step 3 also reads the first fragments
  // of the next stage.
  auto stage = [&](auto BUF_) {
    constexpr int BUF = decltype(BUF_)::value;
    typedef std::integral_constant<int, 0> I0; typedef std::integral_constant<int, 1> I1; typedef std::integral_constant<int, 2> I2;
    typedef std::integral_constant<int, 3> I3; typedef std::true_type Y;
    typedef std::integral_constant<int, BUF> B; typedef std::integral_constant<int, BUF ^ 1> NB;
    substep(I0{}, Y{}, B{}, I1{}, I2{}, NB{});
    substep(I1{}, Y{}, B{}, I2{}, I0{}, I0{});
    substep(I0{}, Y{}, B{}, I3{}, I0{}, I0{});
    publish();
    substep(I1{}, Y{}, NB{}, I0{}, I1{}, B{});
  };

  // ------------------------------------------------------------------ epilogues
  // An accumulator value is fetched where it is used: left to itself the register allocator copies all 256 of them
  // out of the accumulator file in front of the epilogue and spills everything else to make room.
  auto acc_at = [&](int i, int j, int v) -> float {
    float x;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[i][j][v]));
    return x;
  };
  const float* bias = g.bias;
  // MODE_F32: bias, activation, fp32 store (and the optional bf16 copy) straight from the accumulators
  auto store_f32 = [&](int m0, int n0) {
    const int row0 = m0 + wm + lhi * 4, col0 = n0 + wn + l32;
    const uint32_t origin = (uint32_t)row0 * (uint32_t)g.ldo + (uint32_t)col0;
    float* const out = g.out;
    bf16* const obf = g.out_bf;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (!FULL && col0 + j * 32 >= N) continue;
      const float bj = bias ? bias[col0 + j * 32] : 0.f;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        __builtin_amdgcn_sched_barrier(0);  // keeps the scheduler from hoisting every sub-tile's address arithmetic to the top
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = i * 32 + (v >> 2) * 8 + (v & 3);
          float x = acc_at(i, j, v);
          if (FULL || row0 + r < M) {
            if (bias) x = x + bj;
            if (ACT == SN_ACT_RELU) x = fmaxf(g.relu_at, x);
            const uint32_t at = origin + (uint32_t)r * ldo_v + j * 32;
            if (out) out[at] = x;
            if (obf) obf[at] = (bf16)x;
          }
        }
      }
    }
  };
  // MODE_BF16 / MODE_HANDOVER: bias, ReLU and its sign bits (or the ReLU gradient of the layer below and the column
  // sums of what passes), the bf16 cast and two-byte stores, 64 contiguous bytes per row and instruction.
  uint32_t sw[8];  // MODE_HANDOVER: the tile's sign words, requested one stage ahead of the epilogue
  auto request_signs = [&](int t) {
    if constexpr (MODE == MODE_HANDOVER) {
      if (g.signs_in) {
        const uint32_t* sp = g.signs_in + ((int64_t)(t * 4 + wave) * 8) * 64 + lane;
#pragma unroll
        for (int w = 0; w < 8; ++w) sw[w] = sp[w * 64];
      }
    }
  };
  auto store_bf16 = [&](int t, int m0, int n0) {
    if constexpr (MODE != MODE_F32) {
      const uint32_t origin = (uint32_t)(m0 + wm + lhi * 4) * (uint32_t)g.ldo + (uint32_t)(n0 + wn + l32);
      bf16* const o = g.out_bf;
      const bool masked = MODE == MODE_HANDOVER && g.signs_in != nullptr;
      uint32_t bits = 0;
      float csum[TN][TM / 2];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const float bj = (MODE == MODE_BF16 && bias) ? bias[n0 + wn + l32 + j * 32] : 0.f;
          uint32_t word = MODE == MODE_HANDOVER ? sw[(i * TN + j) >> 1] : 0u;
          if (i % 2 == 0) csum[j][i / 2] = 0.f;
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float x = acc_at(i, j, v);
            if constexpr (MODE == MODE_BF16) {
              if (bias) x = x + bj;
              if (ACT == SN_ACT_RELU) {
                // bits = 2 bits + (0 < x): the compare's lane mask is the add's carry-in
                if (g.signs_out) asm volatile("v_cmp_lt_f32 vcc, 0, %1\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(bits) : "v"(x) : "vcc");
                x = fmaxf(0.f, x);
              }
            } else {
              // word += word shifts the next sign bit into the carry, which keeps or clears the value
              if (masked) asm volatile("v_add_co_u32 %0, vcc, %0, %0\n\tv_cndmask_b32 %1, 0, %1, vcc" : "+v"(word), "+v"(x) : : "vcc");
              csum[j][i / 2] += x;
            }
            o[origin + (uint32_t)(i * 32 + (v >> 2) * 8 + (v & 3)) * ldo_v + j * 32] = (bf16)x;
          }
          if constexpr (MODE == MODE_HANDOVER) sw[(i * TN + j) >> 1] = word;
          if constexpr (MODE == MODE_BF16) {
            if (ACT == SN_ACT_RELU && g.signs_out && ((i * TN + j) & 1)) {
              g.signs_out[((int64_t)(t * 4 + wave) * 8 + ((i * TN + j) >> 1)) * 64 + lane] = bits;
              bits = 0;
            }
          }
        }
      }
      if constexpr (MODE == MODE_HANDOVER) {
        if (g.col_partials) {  // the two half-waves hold 4 rows of every 8 each
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int b = 0; b < TM / 2; ++b) {
              const float tsum = csum[j][b] + __shfl_xor(csum[j][b], 32, 64);
              if (lhi == 0) g.col_partials[(int64_t)((m0 + wm) / 64 + b) * N + n0 + wn + l32 + j * 32] = tsum;
            }
        }
      }
    }
  };

  // ------------------------------------------------------------------ the pipeline
  typedef std::integral_constant<int, 0> Z0;
  typedef std::integral_constant<int, 1> Z1;
  // first tile: stage 0 complete and the A half of stage 1 in flight, fragments of sub-step 0 read
#pragma unroll
  for (int q = 0; q < IA; ++q) issue_a(q, 0);
  advance_a();
#pragma unroll
  for (int q = 0; q < IB; ++q) issue_b(q, 0);
  advance_b();
  publish();
#pragma unroll
  for (int q = 0; q < IA; ++q) issue_a(q, 1);
  advance_a();
#pragma unroll
  for (int jj = 0; jj < TN; ++jj) {
    if constexpr (BMN) { fb_lo[0][jj] = read_b_mn(0, 0, jj, 0); fb_hi[0][jj] = read_b_mn(0, 0, jj, 1); }
    else fb[0][jj] = read_b_km(0, 0, jj);
  }
#pragma unroll
  for (int ii = 0; ii < TM; ++ii) {
    if constexpr (AMN) { fa_lo[ii] = read_a_mn(0, 0, ii, 0); fa_hi[ii] = read_a_mn(0, 0, ii, 1); }
    else fa[ii] = read_a_km(0, 0, ii);
  }
  if constexpr (AMN || BMN) __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the steady-state waits count from a full sub-step of reads
  SN_FENCE();
  // Stage kt loads the B half of stage kt + 1 and the A half of stage kt + 2, so in a tile's last pair of stages
  // (nk - 2, nk - 1) every A load and the second B load belong to the next tile: the A cursor changes tile in front
  // of that pair, the B cursor between its two stages.
  if (nk == 2) cursor_tile_a();  // the prologue's second A load already was the next tile's
  for (int it = 0; it < count; ++it) {
    const int t = first + it * stride;
    int m0, n0;
    tile_origin(t, m0, n0);
    for (int kp = 0; kp < nk / 2 - 1; ++kp) {
      stage(Z0{});
      stage(Z1{});
    }
    if (nk > 2) cursor_tile_a();
    if (MODE == MODE_HANDOVER) request_signs(t);
    stage(Z0{});
    cursor_tile_b();
    stage(Z1{});
    if (nk == 2) cursor_tile_a();
    // the first loads of the next tile are in flight while this one's results leave
    if constexpr (MODE == MODE_F32) store_f32(m0, n0);
    else store_bf16(t, m0, n0);
    zero_acc();
  }
  __builtin_amdgcn_s_waitcnt(0);  // the zero-filling loads past the last stage have landed before the workgroup leaves
#undef SN_FENCE
}

template <int TM, int TN, bool AMN, bool BMN, int MODE, int ACT, bool FULL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_bf16_one(GemmBf16Args g) {  // one workgroup per CU: up to 512 registers per lane
  gemm_bf16_body<TM, TN, AMN, BMN, MODE, ACT, FULL>(g);
}
template <int TM, int TN, bool AMN, bool BMN, int MODE, int ACT, bool FULL>
__global__ __launch_bounds__(256, 2)
void gemm_bf16_two(GemmBf16Args g) {  // two workgroups per CU (128 x 128 tiles)
  gemm_bf16_body<TM, TN, AMN, BMN, MODE, ACT, FULL>(g);
}

template <int TM, int TN, bool AMN, bool BMN, int MODE, int ACT, bool FULL>
static int launch_shape(sn_ctx* ctx, const GemmBf16Args& g0, const char* label) {
  GemmBf16Args g = g0;
  constexpr int BM = 64 * TM, BN = 64 * TN;
  g.tiles_m = (int)ceil_div(g.M, BM);
  g.tiles_n = (int)ceil_div(g.N, BN);
  const int total = g.tiles_m * g.tiles_n;
  const size_t smem = 2 * 128 * (BM + BN);
  constexpr bool TWO = TM == 2 && TN == 2;
  const int slots = ctx->compute_units * (TWO ? 2 : 1);
  const int grid = total < slots ? total : slots;
  if constexpr (TWO) {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)gemm_bf16_two<TM, TN, AMN, BMN, MODE, ACT, FULL>, smem));
    LaunchScope scope(ctx, label, g.M, g.N, g.K);
    hipLaunchKernelGGL((gemm_bf16_two<TM, TN, AMN, BMN, MODE, ACT, FULL>), dim3((unsigned)grid), dim3(256), smem, ctx->stream, g);
  } else {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)gemm_bf16_one<TM, TN, AMN, BMN, MODE, ACT, FULL>, smem));
    LaunchScope scope(ctx, label, g.M, g.N, g.K);
    hipLaunchKernelGGL((gemm_bf16_one<TM, TN, AMN, BMN, MODE, ACT, FULL>), dim3((unsigned)grid), dim3(256), smem, ctx->stream, g);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// MODE_F32 for any shape: the largest tile that still gives every CU one, bounds-checked unless the 256 x 256 tiling is exact.
template <bool AMN, bool BMN, int ACT>
static int launch_f32(sn_ctx* ctx, const GemmBf16Args& g) {
  const int cus = ctx->compute_units;
  const int64_t t44 = ceil_div(g.M, 256) * ceil_div(g.N, 256), t24 = ceil_div(g.M, 128) * ceil_div(g.N, 256);
  if (t44 >= cus) {
    if (g.M % 256 == 0 && g.N % 256 == 0) return launch_shape<4, 4, AMN, BMN, MODE_F32, ACT, true>(ctx, g, "gemm_bf16_256x256");
    return launch_shape<4, 4, AMN, BMN, MODE_F32, ACT, false>(ctx, g, "gemm_bf16_256x256");
  }
  if (t24 >= cus) return launch_shape<2, 4, AMN, BMN, MODE_F32, ACT, false>(ctx, g, "gemm_bf16_128x256");
  return launch_shape<2, 2, AMN, BMN, MODE_F32, ACT, false>(ctx, g, "gemm_bf16_128x128");
}

int launch_gemm_bf16(sn_ctx* ctx, int product, const void* a, int64_t lda, const void* b, int64_t ldb, int M, int N, int K,
                     const EpilogueBf16& ep) {
  SN_REQUIRE(a && b && (ep.e.out || ep.out_bf), "gemm_bf16: null operand");
  SN_REQUIRE(product == GEMM_BF16_FORWARD || product == GEMM_BF16_DX || product == GEMM_BF16_DW, "gemm_bf16: unknown product %d", product);
  const bool amn = product == GEMM_BF16_DW, bmn = product != GEMM_BF16_DX;
  SN_REQUIRE(M % 8 == 0 && N % 8 == 0 && K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0,
             "gemm_bf16: M, N, K and the row pitches must be multiples of 8 (got %d x %d x %d)", M, N, K);
  SN_REQUIRE(((amn ? (int64_t)K : (int64_t)M) * lda + 512) * 2 < (int64_t)1 << 31 && ((bmn ? (int64_t)K : (int64_t)N) * ldb + 512) * 2 < (int64_t)1 << 31,
             "gemm_bf16: an operand of %d x %d x %d exceeds the 2 GiB a buffer descriptor may span", M, N, K);
  SN_REQUIRE((int64_t)M * ep.e.ldo < (int64_t)1 << 31, "gemm_bf16: output of %d rows x pitch %lld exceeds 2^31 elements", M, (long long)ep.e.ldo);
  SN_REQUIRE(ep.e.act == SN_ACT_IDENTITY || ep.e.act == SN_ACT_RELU, "gemm_bf16: only ReLU rides in the epilogue (got activation %d)", ep.e.act);
  if (M <= 0 || N <= 0) return SN_OK;
  GemmBf16Args g;
  g.a = (const bf16*)a; g.b = (const bf16*)b; g.lda = lda; g.ldb = ldb; g.M = M; g.N = N; g.K = K; g.tiles_m = g.tiles_n = 0;
  g.out = ep.e.out; g.out_bf = (bf16*)ep.out_bf; g.ldo = ep.e.ldo; g.bias = ep.e.bias; g.relu_at = ep.e.act_param;
  g.signs_out = (uint32_t*)ep.signs_out; g.signs_in = (const uint32_t*)ep.signs_in; g.col_partials = ep.col_partials;
  const bool relu = ep.e.act == SN_ACT_RELU;
  const bool tiles_256 = M % 256 == 0 && N % 256 == 0 && (int64_t)(M / 256) * (N / 256) >= ctx->compute_units;
  if (ep.grad_handover) {
    SN_REQUIRE(product == GEMM_BF16_DX && tiles_256 && g.out_bf && !g.out && !relu && !g.bias,
               "gemm_bf16: the gradient hand-over needs a plain dX product on full 256 x 256 tiles (got %d x %d)", M, N);
    return launch_shape<4, 4, false, false, MODE_HANDOVER, SN_ACT_IDENTITY, true>(ctx, g, "gemm_bf16_256x256_handover");
  }
  if (product == GEMM_BF16_FORWARD && !g.out && tiles_256 && (!relu || g.relu_at == 0.f)) {  // a hidden layer whose output lives as bf16 only
    if (relu) return launch_shape<4, 4, false, true, MODE_BF16, SN_ACT_RELU, true>(ctx, g, "gemm_bf16_256x256_bf16out");
    return launch_shape<4, 4, false, true, MODE_BF16, SN_ACT_IDENTITY, true>(ctx, g, "gemm_bf16_256x256_bf16out");
  }
  SN_REQUIRE(g.out != nullptr, "gemm_bf16: this shape needs an fp32 output (bf16-only results are for full 256 x 256 tiles)");
  if (product == GEMM_BF16_FORWARD) return relu ? launch_f32<false, true, SN_ACT_RELU>(ctx, g) : launch_f32<false, true, SN_ACT_IDENTITY>(ctx, g);
  SN_REQUIRE(!relu && !g.bias, "gemm_bf16: gradient products take no bias and no activation");
  if (product == GEMM_BF16_DX) return launch_f32<false, false, SN_ACT_IDENTITY>(ctx, g);
  return launch_f32<true, true, SN_ACT_IDENTITY>(ctx, g);
}

// true when a forward product of this shape can leave as bf16 only (and its dX counterpart can hand dZ over)
bool gemm_bf16_full_tiles(const sn_ctx* ctx, int M, int N) {
  return M % 256 == 0 && N % 256 == 0 && (int64_t)(M / 256) * (N / 256) >= ctx->compute_units;
}

// ---------------------------------------------------------------------------- fp32 -> bf16
// out[r][c] from src[r*ld + c]; when y or y_bf is given the value cast is the activation gradient act'(y) * src
// (also written back to dz in fp32 when dz != null); col_partials (optional, [ceil(rows/64), cols]) receives the
// column sums of every 64-row block of the fp32 values.
__global__ __launch_bounds__(256) void cast_bf16_kernel(const float* __restrict__ src, int64_t ld, int rows, int cols, bf16* __restrict__ out,
                                                         const float* __restrict__ y, const bf16* __restrict__ y_bf, int act, float act_param,
                                                         float* __restrict__ dz, float* __restrict__ col_partials) {
  // 64x64 tile; a thread handles 4 consecutive columns of 4 rows (float4 in, 8-byte bf16x4 out).
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
      bf16x4 bq;
#pragma unroll
      for (int e = 0; e < 4; ++e) bq[e] = (bf16)v[e];
      *(bf16x4*)(out + (int64_t)r * cols + c) = bq;
    }
    csum += v;
  }
  if (!col_partials) return;
#pragma unroll
  for (int e = 0; e < 4; ++e) colp[tr][tc + e] = csum[e];
  __syncthreads();
  if (threadIdx.x < 64 && c0 + threadIdx.x < cols) {  // column sums of this 64-row block, rows in a fixed order
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) t += colp[j][threadIdx.x];
    col_partials[(int64_t)blockIdx.y * cols + c0 + threadIdx.x] = t;
  }
}

int launch_cast_bf16(sn_ctx* ctx, const float* src, int64_t ld, int rows, int cols, void* out, const float* y, int act, float act_param,
                     float* dz, float* col_partials, const void* y_bf) {
  if (rows <= 0 || cols <= 0) return SN_OK;
  SN_REQUIRE(out != nullptr, "cast_bf16: null output");
  SN_REQUIRE(rows % 4 == 0 && cols % 4 == 0 && ld % 4 == 0, "cast_bf16: rows, cols and pitch must be multiples of 4");
  LaunchScope scope(ctx, (y || y_bf) ? "activation_backward_cast_bf16" : "cast_bf16");
  hipLaunchKernelGGL(cast_bf16_kernel, dim3((unsigned)ceil_div(cols, 64), (unsigned)ceil_div(rows, 64)), dim3(256), 0, ctx->stream,
                     src, ld, rows, cols, (bf16*)out, y, (const bf16*)y_bf, act, act_param, dz, col_partials);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
