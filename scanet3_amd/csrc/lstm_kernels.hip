// Recurrent-layer kernels for gfx950 (LSTM and the simple cell).
//
// One recurrent step multiplies a [rows, F+H] operand by weights that stay the same for the whole sequence and is far
// too small to fill the chip as a tiled GEMM followed by an element-wise pass.  Two families live here:
//   * one launch per direction for ALL time steps (lstm_sequence_fwd_kernel, lstm_sequence_bwd_kernel,
//     rnn_sequence_kernel): a workgroup owns 16 batch rows x 16 hidden units for the whole sequence, keeps its weights in
//     registers and its cell state (or cell gradient) too, fetches the step's operand rows with LDS-direct loads, and the
//     unit groups of a row group hand h_t (backward: dz_t) to each other through the XCD's L2 with an arrival counter;
//   * one launch per step (lstm_step_fwd_kernel, lstm_step_bwd_kernel, step_product_kernel), used where the first family
//     does not fit the device or the shape: a workgroup owns 32 batch rows x 64 output columns, stages the WHOLE reduction
//     dimension of both operands in LDS with every global load in flight at once, multiplies with
//     v_mfma_f32_16x16x4_f32 and finishes the step in its epilogue (forward, layer/RNN.scala:303-340: the 64 columns are
//     the four gates of 16 hidden units, so the workgroup applies the gate activations and writes gates, c_t and h_t
//     itself; backward: gate gradients and the dz * Wr^T product share a kernel, cut into partial dh per unit slice).
#include "common.hpp"

namespace sn {
namespace {

typedef float f4v __attribute__((ext_vector_type(4)));
constexpr int RB = 32;        // batch rows per workgroup
constexpr int ZP = 17;        // row pitch of the pre-activation exchange area
constexpr int MAX_K = 400;    // 32*(K+4) + 64*K floats of LDS must fit in 160 KiB

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

__host__ __device__ inline int round16(int k) { return (k + 15) & ~15; }

// acc[r] += A[row block rb0 + r][:] * B[:, column block cb]  (blocks of 16 rows / 16 columns).
// As: [RB][K16+4].  Bs: [column blocks][K16/4][16 columns][4 consecutive k].  Lane (row = l%16, g = l/16) feeds
// k = 16 kb + 4 g + j into the j-th MFMA of block kb, so both operands come from one 16-byte LDS read each.
template <int NRB>
__device__ __forceinline__ void multiply_blocks(const float* As, const float* Bs, int K16, int cb, int rb0, int lane, f4v (&acc)[NRB]) {
  const int row = lane & 15, g = lane >> 4;
  const float* ap = As + (rb0 * 16 + row) * (K16 + 4) + 4 * g;
  const float* bp = Bs + (((int64_t)cb * (K16 / 4) + g) * 16 + row) * 4;
#pragma unroll 2
  for (int kb = 0; kb < K16 / 16; ++kb) {
    f4v a[NRB];
#pragma unroll
    for (int r = 0; r < NRB; ++r) a[r] = *(const f4v*)(ap + r * 16 * (K16 + 4) + 16 * kb);
    const f4v b = *(const f4v*)(bp + kb * 256);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < NRB; ++r) acc[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r][j], b[j], acc[r], 0, 0, 0);
  }
}

// ---------------------------------------------------------------------------- forward step
struct StepFwdArgs {
  const float* x;       // [rows, T, F]
  const float* h_prev;  // [rows, H] or null (first step: h_{-1} = 0 drops out of the product)
  const float* c_prev;  // [rows, H] or null
  LstmWeights w;
  const float* wpack;   // the weights in LDS order (pack_fwd_kernel)
  float* gates;         // [rows, 4H] activated forget, input, gate, output
  float* c;             // [rows, H]
  float* h;             // [rows, H]
  int rows, T, F, H, t;
};

// Weights in the order the step kernel's LDS wants them, rebuilt once per pass over the sequence (they change once
// per training step, the step kernel runs T times): [unit group of 16][gate][k/4][16 units][4 consecutive k],
// k over [Wk; Wr] padded with zeros to a multiple of 16.  The step kernel then copies its slab with contiguous
// 16-byte loads instead of gathering 4-byte values from 4 rows per cell.
__global__ __launch_bounds__(256) void pack_fwd_kernel(LstmWeights w, int F, int H, int G, float* __restrict__ out) {
  const int K = F + H, kq = round16(K) / 4;
  const int64_t cells = (int64_t)(H / 16) * G * kq * 16;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < cells; e += (int64_t)gridDim.x * 256) {
    const int bu = (int)(e & 15);
    int64_t t = e >> 4;
    const int q = (int)(t % kq); t /= kq;
    const int gate = (int)(t % G);
    const int cg = (int)(t / G);
    f4v v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = 4 * q + j;
      if (k < F) v[j] = w.wk[gate][(int64_t)k * H + cg * 16 + bu];
      else if (k < K) v[j] = w.wr[gate][(int64_t)(k - F) * H + cg * 16 + bu];
    }
    *(f4v*)(out + e * 4) = v;
  }
}

// [gate][unit block of 16][n/4][16 units][4 consecutive n] of the recurrent weights Wr_gate[u][n], n padded to 16
__global__ __launch_bounds__(256) void pack_dh_kernel(LstmWeights w, int H, int G, float* __restrict__ out) {
  const int kq = round16(H) / 4;
  const int64_t cells = (int64_t)G * (H / 16) * kq * 16;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < cells; e += (int64_t)gridDim.x * 256) {
    const int bu = (int)(e & 15);
    int64_t t = e >> 4;
    const int q = (int)(t % kq); t /= kq;
    const int ublk = (int)(t % (H / 16));
    const int gate = (int)(t / (H / 16));
    f4v v = {0.f, 0.f, 0.f, 0.f};
    if (4 * q < H) v = *(const f4v*)(w.wr[gate] + (int64_t)(ublk * 16 + bu) * H + 4 * q);  // H % 16 == 0: whole quads
    *(f4v*)(out + e * 4) = v;
  }
}

// 16 hidden units (x 4 gates) per workgroup: one gate per wavefront, two row blocks each.
__global__ __launch_bounds__(256) void lstm_step_fwd_kernel(StepFwdArgs a) {
  constexpr int UB = 16;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int K = a.h_prev ? a.F + a.H : a.F;
  const int K16 = round16(K), KP = K16 + 4, kq = K16 / 4;
  float* As = lds;                 // [RB][KP]
  constexpr int NCB = UB / 4, NRB = NCB / 2;  // column blocks of 16 (column = gate * UB + unit); row blocks per wavefront
  const int kq_full = round16(a.F + a.H) / 4;  // quads per gate in the packed weights (the first step uses only F/4 of them)
  float* Bs = lds + RB * KP;       // [NCB][kq][16 columns][4]
  float* Zx = lds;                 // [4 gates][RB][ZP], over the operand slabs once every wavefront has finished multiplying
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r0 = blockIdx.y * RB, u0 = blockIdx.x * UB;

  // ---- stage both operands.  Every global load of a pass is issued before the first LDS write, and one
  // pass covers F + H up to 384 (NA = 12 row vectors, NB = 24 weight cells per thread), so the whole tile
  // costs one memory latency.
  // Index maps without divisions: 8 threads per operand row take 16-byte vectors q = tid%8 + 8i; for the
  // weights a thread owns unit tid%16 and the k quads q = tid/16 + 16i of every gate, gathering the 4 values
  // of one LDS cell, so consecutive lanes write consecutive cells and read 64-byte runs of each weight row.
  constexpr int NA = 12, NQ = 6;  // enough for MAX_K: 8 * NA and 16 * NQ quads
  for (int pass = 0; pass * 8 * NA < kq; ++pass) {
    f4v va[NA], vb[NCB][NQ];
    const int arow = tid >> 3, bu = tid & 15;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int q = (pass * NA + i) * 8 + (tid & 7), k = q * 4;
      va[i] = f4v{0.f, 0.f, 0.f, 0.f};
      if (q < kq && r0 + arow < a.rows && k < K)
        va[i] = k < a.F ? *(const f4v*)(a.x + ((int64_t)(r0 + arow) * a.T + a.t) * a.F + k)
                        : *(const f4v*)(a.h_prev + (int64_t)(r0 + arow) * a.H + (k - a.F));
    }
    if (pass * 16 * NQ < kq) {
#pragma unroll
      for (int cbi = 0; cbi < NCB; ++cbi) {  // column block = gate; the packed slab has the LDS cell order
        const float* slab = a.wpack + ((int64_t)blockIdx.x * 4 + cbi) * kq_full * 64;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
          const int q = (pass * NQ + i) * 16 + (tid >> 4);
          vb[cbi][i] = f4v{0.f, 0.f, 0.f, 0.f};
          if (q < kq) vb[cbi][i] = *(const f4v*)(slab + (q * 16 + bu) * 4);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int q = (pass * NA + i) * 8 + (tid & 7);
      if (q < kq) *(f4v*)(As + arow * KP + q * 4) = va[i];
    }
    if (pass * 16 * NQ < kq) {
#pragma unroll
      for (int cbi = 0; cbi < NCB; ++cbi)
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
          const int q = (pass * NQ + i) * 16 + (tid >> 4);
          if (q < kq) *(f4v*)(Bs + ((cbi * kq + q) * 16 + bu) * 4) = vb[cbi][i];
        }
    }
  }
  __syncthreads();

  const int cb = wave % NCB, rb0 = (wave / NCB) * NRB;
  f4v acc[NRB];
#pragma unroll
  for (int r = 0; r < NRB; ++r) acc[r] = f4v{0.f, 0.f, 0.f, 0.f};
  multiply_blocks<NRB>(As, Bs, K16, cb, rb0, lane, acc);

  // ---- pre-activations to the exchange area: element v of a lane is row 4*(l/16) + v of its block, column l%16
  __syncthreads();
  {
    const int col = cb * 16 + (lane & 15), gate = col / UB, u = col % UB, g = lane >> 4;
    const float bias = a.w.b[gate] ? a.w.b[gate][u0 + u] : 0.f;
#pragma unroll
    for (int r = 0; r < NRB; ++r)
#pragma unroll
      for (int v = 0; v < 4; ++v) Zx[(gate * RB + (rb0 + r) * 16 + 4 * g + v) * ZP + u] = acc[r][v] + bias;
  }
  __syncthreads();
  // ---- c = c_prev * f + i * g ; h = o * tanh(c)   (layer/RNN.scala:336-337)
#pragma unroll
  for (int e = tid; e < RB * UB; e += 256) {
    const int row = e / UB, u = e % UB;
    if (r0 + row >= a.rows) continue;
    const float f = sigmoidf_(Zx[(0 * RB + row) * ZP + u]);
    const float in = sigmoidf_(Zx[(1 * RB + row) * ZP + u]);
    const float g = tanhf(Zx[(2 * RB + row) * ZP + u]);
    const float o = sigmoidf_(Zx[(3 * RB + row) * ZP + u]);
    const int64_t i = (int64_t)(r0 + row) * a.H + u0 + u;
    const int64_t zb = (int64_t)(r0 + row) * 4 * a.H + u0 + u;
    const float cp = a.c_prev ? a.c_prev[i] : 0.f;
    const float c = cp * f + in * g;
    a.gates[zb] = f;
    a.gates[zb + a.H] = in;
    a.gates[zb + 2 * a.H] = g;
    a.gates[zb + 3 * a.H] = o;
    a.c[i] = c;
    a.h[i] = o * tanhf(c);
  }
}

// ---------------------------------------------------------------------------- all forward steps in one launch
// A workgroup owns 16 batch rows x 16 hidden units for the whole sequence (512 x 256 gives 512 workgroups, two or more
// per CU, so one multiplies while its neighbour on the CU waits).  Wavefront w owns gate w: its [K x 16] weights are read
// once per launch, as they lie, into registers in MFMA operand order; the cell states of the workgroup's cells live in
// registers; per step only the 16 rows of [x_t, h_{t-1}] are fetched, straight into LDS (LDS-direct loads), multiplied on
// v_mfma_f32_16x16x4_f32, and the four gates meet in LDS.  h_t is handed from the unit groups of a row group to each
// other through memory: after its stores of step t have been acknowledged a workgroup adds 1 to the row group's arrival
// counter; before step t + 1 it waits until the counter shows every workgroup of the group.  That needs all workgroups
// of the launch on the device at once, which the host checks against the device's occupancy before it picks this
// kernel.  The wait is bounded all the same: a workgroup that polls `spin_limit` times in vain (or sees that another
// one did) raises the abort word, reports through `gave_up` / `failed` and leaves, and so does every other workgroup at
// its next wait.  About 4.4 us per step at 512 x 256 x 288 (one launch per step: 11.2 us).
//
// The hand-over avoids device-scope fences, which on this hardware write back and invalidate a whole L2 and cost tens
// of microseconds per step here.  Two forms instead, chosen per row group:
//   within one XCD   plain stores and loads.  The XCD's L2 is the one cache between its CUs: a store acknowledged
//                    (s_waitcnt vmcnt(0)) is in L2, and a load of a line this CU's vector L1 does not hold finds it
//                    there.  That the L1 does not hold it rests on two things: every h (dz, r) slice is written once
//                    and read once per launch, at addresses nobody has read before in this launch; and the vector L1
//                    is write-through WITHOUT write-allocate, so the 64 bytes a workgroup itself stored into a
//                    128-byte line of the slice did not bring that line into its L1 (the other half of the line comes
//                    from a neighbour workgroup and must be read from L2).  The second premise is a property of this
//                    hardware that the kernel relies on and cannot check; the parity tests (both forms, several
//                    steps with different data per step) are what pins it.
//   across XCDs      every access is itself coherent at device scope: h_t is written with device-scope atomic stores
//                    (write-through), read with loads that carry the same coherence bit (sc1).  About twice the time.
// Workgroup ids are mapped to (row group, unit group) so that a row group's workgroups have ids congruent mod 8, which
// the dispatcher places on one XCD.  That is not taken on trust: each workgroup reads the XCD it runs on from the
// hardware register, the members of a row group compare theirs in a first arrival before any hand-over, and one
// mismatch switches the whole row group to the second form.  Each row group's counter, XCD word and flag have 256 bytes
// of their own (all counters in one line made every polling workgroup of the launch meet on that line), and the counter
// itself is only touched with device-scope atomics.
__device__ __forceinline__ f4v load_coherent(const float* p) {
  f4v v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
template <int N>
__device__ __forceinline__ void wait_coherent_loads(f4v (&v)[N]) {  // ties the wait to the registers the loads fill
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(v[i]));
}

struct SeqFwdArgs {
  const float* x;        // [rows, T, F]
  const float* c0;       // [rows, H] or null: zeros
  const float* wk[4];    // [F, H] forget, input, gate, output
  const float* wr[4];    // [H, H]
  const float* bias[4];
  float* gates;          // T slices of 4 * slice floats: activated forget, input, gate, output of [rows, 4H]
  float* c;              // T slices
  float* h;              // T + 1 slices, slice t + 1 = h_t; slice 0 is read only if h0_valid
  int64_t slice;
  int h0_valid;
  int rows, T, F, H;
  int row_groups, unit_groups;
  unsigned* sync;        // zero at launch: per row group a block of SEQ_GROUP_WORDS (arrival counter, XCD word, spread flag), then the abort word
  unsigned spin_limit;
  int* gave_up;          // host-visible
  int* failed;           // the same flag in device memory: the optimizer launch of the step looks at it
  int force_coherent;    // take the across-XCD form everywhere
};

// Waits (thread 0 polls) until *count >= target.  Returns nonzero in every thread if the wait was given up.
__device__ __forceinline__ int wait_arrivals(unsigned* count, unsigned target, unsigned* abort_word, unsigned spin_limit, int* gave_up, int* failed, int* stop) {
  if (threadIdx.x == 0) {
    unsigned spins = 0;
    int bad = spin_limit == 0u;  // a limit of zero gives up at the first wait whatever the counter shows (how a test forces this path)
    while (!bad && __hip_atomic_load(count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      // (every workgroup of the launch watches the one abort word: a look every 16th round keeps them off each other)
      if (++spins > spin_limit || ((spins & 15u) == 0u && __hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
        bad = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (bad) {
      __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(failed, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    *stop = bad;
  }
  __syncthreads();
  return *stop;
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;
__device__ __align__(16) const float seq_zero_chunk[4] = {0.f, 0.f, 0.f, 0.f};  // what the k padding and an absent h_{-1} read

// LDS-direct loads of blocks KB .. NKB - 1 of a 16-row operand: block kb = 64 bytes of every row, 1 KiB of LDS
template <int KB, int NKB, int AUX>
__device__ __forceinline__ void load_row_blocks(global_ptr_t ap, float* aw) {
  if constexpr (KB < NKB) {
    __builtin_amdgcn_global_load_lds(ap, (lds_ptr_t)(aw + KB * (256 - 16)), 16, 64 * KB, AUX);
    load_row_blocks<KB + 1, NKB, AUX>(ap, aw);
  }
}

// base + a per-lane BYTE offset of 32 bits: the form the compiler turns into "scalar base + one offset register" accesses
template <typename T>
__device__ __forceinline__ T* at_bytes(T* uniform_base, unsigned byte_offset) {
  return (T*)((char*)uniform_base + byte_offset);
}
template <typename T>
__device__ __forceinline__ const T* at_bytes(const T* uniform_base, unsigned byte_offset) {
  return (const T*)((const char*)uniform_base + byte_offset);
}


// Shape of the kernel: a workgroup owns 16 batch rows x 16 hidden units, so that two or more workgroups share a CU and one
// of them multiplies while another waits for its hand-over.  Wavefront w owns gate w: its [K x 16] weights stay in
// registers in MFMA operand order.  The 16 rows of [x_t, h_{t-1}] arrive through LDS-direct loads (one load = 16 rows x
// 16 k = 1 KiB of LDS, lane p to bytes 16 p .. 16 p + 15: four neighbouring lanes fetch 64 contiguous bytes of a row, and
// chunk c of row r lands in slot c ^ (r / 4) so that the reads of one chunk index over 16 rows hit 16 different bank
// groups); the wavefronts share the blocks, each requests every fourth one.
constexpr int SRB = 16;  // batch rows per workgroup of the one-launch kernels

template <int NKB>  // 16-long blocks of k over [x_t, h_{t-1}], padded with zeros
__global__ __launch_bounds__(256) void lstm_sequence_fwd_kernel(SeqFwdArgs a) {
  constexpr int UB = 16;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ int stop;
  float* As = lds;              // [NKB][16 rows x 16 k]
  float* Zx = lds + NKB * 256;  // [4 gates][16 rows][ZP]
  const int K = a.F + a.H;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // id -> (row group, unit group): ids congruent mod 8 share an XCD, so XCD x takes the row groups x, x + 8, ...
  const int slot = blockIdx.x >> 3;
  const int rg = (blockIdx.x & 7) + 8 * (slot / a.unit_groups), ug = slot % a.unit_groups;
  if (rg >= a.row_groups) return;  // the grid is rounded up to whole rounds of 8 row groups
  const int r0 = rg * SRB, u0 = ug * UB;
  unsigned* my_count = a.sync + rg * SEQ_GROUP_WORDS;
  unsigned* my_xcd = my_count + 1;
  unsigned* my_spread = my_count + 2;
  unsigned* abort_word = a.sync + a.row_groups * SEQ_GROUP_WORDS;

  // ---- arrival 0 (the placement check): do the members of this row group share an XCD?
  if (tid == 0) {
    const unsigned mine = 1u + (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u);  // HW_REG_XCC_ID, 4 bits
    unsigned seen = 0u;
    __hip_atomic_compare_exchange_strong(my_xcd, &seen, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((seen != 0u && seen != mine) || a.force_coherent) __hip_atomic_store(my_spread, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the flag is acknowledged before this workgroup counts itself in, so whoever has seen the full count sees the flag
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
    __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  const int row16 = lane & 15, g = lane >> 4;
  // weights of gate `wave`: lane (unit = row16, g) holds k = 16 kb + 4 g .. + 3 for every kb, k over [Wk; Wr], zeros past K
  // (read once per launch, straight from the layer's tensors: 16 lanes fetch 64 contiguous bytes of a weight row)
  f4v bw[NKB];
  {
    const float* wkc = a.wk[wave] + u0 + row16;
    const float* wrc = a.wr[wave] + u0 + row16;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = 16 * kb + 4 * g + j;
        bw[kb][j] = k < a.F ? wkc[(int64_t)k * a.H] : (k < K ? wrc[(int64_t)(k - a.F) * a.H] : 0.f);
      }
  }
  // the cell this thread finishes per step: row tid / 16, unit tid % 16
  const int crow = tid >> 4, cu = tid & 15;
  const bool live = r0 + crow < a.rows;
  const int64_t ci = (int64_t)(live ? r0 + crow : 0) * a.H + u0 + cu, zi = (int64_t)(live ? r0 + crow : 0) * 4 * a.H + u0 + cu;
  float c_reg = a.c0 ? a.c0[ci] : 0.f;
  float bias[4];
#pragma unroll
  for (int gate = 0; gate < 4; ++gate) bias[gate] = a.bias[gate] ? a.bias[gate][u0 + cu] : 0.f;
  // operand loads: lane p fetches chunk (p % 4) ^ (p / 16) of row p / 4 (rows past the batch: the last row again)
  const int chunk = (lane & 3) ^ (lane >> 4);
  const int64_t arow = min(r0 + (lane >> 2), a.rows - 1);
  const float* xrow = a.x + arow * a.T * a.F;
  const float* ar = As + (row16 * 4 + (g ^ (row16 >> 2))) * 4;

  bool spread = true;  // until arrival 0 is complete (the first wait below), write as if the row group were spread out
  for (int t = 0; t < a.T; ++t) {
    const bool with_h = t > 0 || a.h0_valid;
    if (t > 0) {  // h_{t-1} is complete once every unit group of this row group has arrived t + 1 times (arrival 0 included)
      if (wait_arrivals(my_count, (unsigned)a.unit_groups * (unsigned)(t + 1), abort_word, a.spin_limit, a.gave_up, a.failed, &stop)) return;
      if (t == 1) spread = __hip_atomic_load(my_spread, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
    }
    const float* xt = xrow + (int64_t)t * a.F;
    const float* ht = a.h + (int64_t)t * a.slice + arow * a.H - a.F;  // indexed by k
    const bool coherent = spread && t > 0;  // slice 0 was written before this launch
#pragma unroll
    for (int i = 0; i < (NKB + 3) / 4; ++i) {
      const int kb = wave + 4 * i;  // uniform in the wavefront
      if (kb >= NKB) break;
      const int k0 = 16 * kb + 4 * chunk;
      const float* src = k0 < a.F ? xt + k0 : (k0 < K && with_h ? ht + k0 : seq_zero_chunk);
      if (coherent) __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(As + kb * 256), 16, 0, 16);  // sc1: coherent at device scope
      else __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(As + kb * 256), 16, 0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the compiler does not order LDS reads behind these loads by itself)
    __syncthreads();
    f4v acc[2] = {f4v{0.f, 0.f, 0.f, 0.f}, f4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      const f4v av = *(const f4v*)(ar + kb * 256);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[kb & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[v], bw[kb][v], acc[kb & 1], 0, 0, 0);
    }
    // pre-activations to the exchange area: element v of a lane is row 4 g + v, unit row16 of gate `wave`
#pragma unroll
    for (int v = 0; v < 4; ++v) Zx[(wave * SRB + 4 * g + v) * ZP + row16] = acc[0][v] + acc[1][v];
    __syncthreads();  // (also: every wavefront has read As)
    // ---- c = c_prev * f + i * g ; h = o * tanh(c)   (layer/RNN.scala:336-337)
    if (live) {
      const float f = sigmoidf_(Zx[(0 * SRB + crow) * ZP + cu] + bias[0]);
      const float in = sigmoidf_(Zx[(1 * SRB + crow) * ZP + cu] + bias[1]);
      const float gg = tanhf(Zx[(2 * SRB + crow) * ZP + cu] + bias[2]);
      const float o = sigmoidf_(Zx[(3 * SRB + crow) * ZP + cu] + bias[3]);
      float* gt = a.gates + (int64_t)t * 4 * a.slice + zi;
      const float c = c_reg * f + in * gg;
      c_reg = c;
      gt[0] = f;
      gt[a.H] = in;
      gt[2 * a.H] = gg;
      gt[3 * a.H] = o;
      a.c[(int64_t)t * a.slice + ci] = c;
      float* hout = a.h + (int64_t)(t + 1) * a.slice + ci;
      if (spread) __hip_atomic_store(hout, o * tanhf(c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else *hout = o * tanhf(c);
    }
    // ---- hand h_t over: every wavefront waits until its stores have been acknowledged, then one thread counts the
    // workgroup in
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));  // vmcnt(0)
    __syncthreads();  // (also: Zx is free again)
    if (tid == 0 && t + 1 < a.T) __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ---------------------------------------------------------------------------- one product per step, whole K in LDS
// out_z[m, u] = sum_k A[m, k] * W_z[u, k] for z = blockIdx.z, where a row of A is [a0 row (k0 values), a1 row (k1 values)]
// and W_z comes packed as [unit block of 16][k/4][16 units][4 consecutive k] with `kq_pack` quads per unit block.
//   LSTM backward:      A = dz of gate z (a0 = dz + z*H, a1 = null), W = recurrent weights, out = partial dh of gate z
//   simple cell forward: A = [x_t, r_{t-1}], W = [Wk; Wr] columns, out = r_t            (layer/RNN.scala:189-196)
//   simple cell backward: A = dr_t, W = recurrent weights, out = dr_{t-1}
struct StepMulArgs {
  const float* a0;
  int64_t ld0;          // row stride of a0
  int k0;
  const float* a1;      // or null
  int64_t ld1;
  int k1;
  int64_t a0_z_stride;  // added to a0 per blockIdx.z
  const float* wpack;
  int kq_pack;          // quads per unit block in the pack (>= the quads this launch reads)
  int64_t pack_z_stride;
  float* out;           // [rows, out_ld]
  int64_t out_ld, out_z_stride;
  int rows, cols;
};

// CBT output units per workgroup: 64 (one column block per wavefront, two row blocks each) or 32 (half the LDS).
template <int CBT>
__global__ __launch_bounds__(256) void step_product_kernel(StepMulArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int K = a.k0 + (a.a1 ? a.k1 : 0), K16 = round16(K), KP = K16 + 4, kq = K16 / 4;
  float* As = lds;            // [RB][KP]
  constexpr int NCB = CBT / 16, NRB = NCB / 2;
  float* Bs = lds + RB * KP;  // [NCB][kq][16 units][4]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r0 = blockIdx.y * RB, u0 = blockIdx.x * CBT, z = blockIdx.z;
  const float* a0 = a.a0 + (int64_t)z * a.a0_z_stride;
  const float* wp = a.wpack + (int64_t)z * a.pack_z_stride;

  // Staging as in the forward kernel: one pass (K up to 384) with every load in flight before the LDS writes.
  constexpr int NA = 12, NQ = 6;
  for (int pass = 0; pass * 8 * NA < kq; ++pass) {
    f4v va[NA], vb[NCB][NQ];
    const int arow = tid >> 3, bu = tid & 15;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int q = (pass * NA + i) * 8 + (tid & 7), k = q * 4;
      va[i] = f4v{0.f, 0.f, 0.f, 0.f};
      if (q < kq && r0 + arow < a.rows && k < K)
        va[i] = k < a.k0 ? *(const f4v*)(a0 + (int64_t)(r0 + arow) * a.ld0 + k) : *(const f4v*)(a.a1 + (int64_t)(r0 + arow) * a.ld1 + (k - a.k0));
    }
    if (pass * 16 * NQ < kq) {
#pragma unroll
      for (int wv = 0; wv < NCB; ++wv)
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
          const int q = (pass * NQ + i) * 16 + (tid >> 4), ublk = (u0 >> 4) + wv;
          vb[wv][i] = f4v{0.f, 0.f, 0.f, 0.f};
          if (q < kq && ublk * 16 < a.cols) vb[wv][i] = *(const f4v*)(wp + (((int64_t)ublk * a.kq_pack + q) * 16 + bu) * 4);
        }
    }
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int q = (pass * NA + i) * 8 + (tid & 7);
      if (q < kq) *(f4v*)(As + arow * KP + q * 4) = va[i];
    }
    if (pass * 16 * NQ < kq) {
#pragma unroll
      for (int wv = 0; wv < NCB; ++wv)
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
          const int q = (pass * NQ + i) * 16 + (tid >> 4);
          if (q < kq) *(f4v*)(Bs + ((wv * kq + q) * 16 + bu) * 4) = vb[wv][i];
        }
    }
  }
  __syncthreads();

  const int cb = wave % NCB, rb0 = (wave / NCB) * NRB;
  f4v acc[NRB];
#pragma unroll
  for (int r = 0; r < NRB; ++r) acc[r] = f4v{0.f, 0.f, 0.f, 0.f};
  multiply_blocks<NRB>(As, Bs, K16, cb, rb0, lane, acc);

  const int col = u0 + cb * 16 + (lane & 15), g = lane >> 4;
  if (col < a.cols) {
    float* out = a.out + (int64_t)z * a.out_z_stride;
#pragma unroll
    for (int r = 0; r < NRB; ++r)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int row = r0 + (rb0 + r) * 16 + 4 * g + v;
        if (row < a.rows) out[(int64_t)row * a.out_ld + col] = acc[r][v];
      }
  }
}

// ---------------------------------------------------------------------------- the simple cell's steps in one launch
// The simple cell's two recurrences are one product per step with nothing around it:
//   forward   r_t     = [x_t, r_{t-1}] * [Wk; Wr]                         (layer/RNN.scala:189-196), t = 0 .. T-1
//   backward  dr_{t-1} = dr_t * Wr^T (+ the output gradient of step t-1 when the layer returns its sequence), t = T-1 .. 1
// so one kernel runs either for all steps, built like the LSTM's one-launch kernels: a workgroup owns 16 batch rows x 16
// units, each of its wavefronts multiplies a quarter of k (weights in registers, its blocks of the operand rows through
// LDS-direct loads into LDS of its own), the four partial sums meet in LDS, and the unit groups of a row group hand the
// step's result to each other through memory with the same arrival counter, placement check, bounded wait and two
// hand-over forms.  Every slice is written once and read once per launch, so within an XCD plain loads find it in L2.
struct SeqMulArgs {
  const float* x;       // forward: [rows, T, F]; backward: null
  float* rec;           // slices of `slice` floats; forward: slice t + 1 = r_t (slice 0 read only if first_valid),
                        // backward: slice t = dr_t, slice T - 1 complete at launch
  const float* dy_seq;  // backward, returned sequence: [rows, T, H] added to slice t - 1 as it is written; or null
  const float* wk;      // forward: [F, H] kernel weights; backward: null
  const float* wr;      // [H, H] recurrent weights
  int64_t slice;
  int first_valid;
  int rows, T, F, H;    // backward: F = 0
  int row_groups, unit_groups;
  unsigned* sync;
  unsigned spin_limit;
  int* gave_up;
  int* failed;
  int force_coherent;
  // backward with the weight gradient riding along (XW > 0 instantiations)
  const float* wg_x;    // [rows, T, wg_F]
  const float* wg_r;    // the forward pass's slices: slice t = r_{t-1}
  float* wpartial;      // [row_groups][wg_F + H + 1][H]
  int wg_F;
};

// XW > 0 (backward only; H a multiple of 64, the batch a multiple of 16 rows): the launch also accumulates the layer's weight
// gradient dW[m, n] = sum over (t, row) of [x_t | r_{t-1}][row, m] * dr_t[row, n], as lstm_sequence_bwd_body does for the
// LSTM: the workgroup keeps the [F + H, 16] block that belongs to its rows and units in accumulator registers (wavefront w
// the 64-feature run w of r, one wavefront the x features), takes dr_t of its own cells from LDS the moment it has
// computed them (slice T - 1, which is complete at launch, from memory), the operand rows straight from memory a step
// ahead, and multiplies right behind its arrival signal.  One partial [F + H + 1, H] per row group leaves at the end (its
// last row, the place of a bias gradient, is not written: the simple cell's bias acts on the last step only).
template <bool BACKWARD, int NKBW, int XW = 0>  // NKBW: 16-long blocks of k per wavefront (4 NKBW blocks cover K, padded with zeros)
__global__ __launch_bounds__(256) void rnn_sequence_kernel(SeqMulArgs a) {
  constexpr int UB = 16;
  constexpr bool WG = BACKWARD && XW > 0;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ int stop;
  float* Ps = lds;                 // [4 quarters of k][SRB][ZP] partial sums
  float* As = lds + 4 * SRB * ZP;  // (16-byte aligned) [wavefront][k block][16 rows x 16 k]
  float* Dzs = As + 4 * NKBW * 256;  // [SRB][16]: dr of this workgroup's cells (weight gradient only)
  const int K = a.F + a.H;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int slot = blockIdx.x >> 3;
  const int rg = (blockIdx.x & 7) + 8 * (slot / a.unit_groups), ug = slot % a.unit_groups;
  if (rg >= a.row_groups) return;
  const int r0 = rg * SRB, u0 = ug * UB;
  unsigned* my_count = a.sync + rg * SEQ_GROUP_WORDS;
  unsigned* my_xcd = my_count + 1;
  unsigned* my_spread = my_count + 2;
  unsigned* abort_word = a.sync + a.row_groups * SEQ_GROUP_WORDS;

  if (tid == 0) {  // arrival 0 (the placement check): do the members of this row group share an XCD?
    const unsigned mine = 1u + (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u);  // HW_REG_XCC_ID, 4 bits
    unsigned seen = 0u;
    __hip_atomic_compare_exchange_strong(my_xcd, &seen, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((seen != 0u && seen != mine) || a.force_coherent) __hip_atomic_store(my_spread, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
    __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  const int row16 = lane & 15, g = lane >> 4;
  // wavefront w multiplies k blocks w NKBW .. w NKBW + NKBW - 1; its part of the unit block's weights stays in registers in
  // MFMA operand order, read once per launch from the layer's own tensors: forward B[k][u] = [Wk; Wr][k][u] (16 lanes fetch
  // 64 contiguous bytes of a weight row), backward B[k = n][u] = Wr[u][n] (a lane's 4 k-values are 16 contiguous bytes)
  f4v bw[NKBW];
#pragma unroll
  for (int i = 0; i < NKBW; ++i) {
    const int k0 = 16 * (wave * NKBW + i) + 4 * g;
    if (BACKWARD) {
      bw[i] = k0 < K ? *(const f4v*)(a.wr + (int64_t)(u0 + row16) * a.H + k0) : f4v{0.f, 0.f, 0.f, 0.f};
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + j;
        bw[i][j] = k < a.F ? a.wk[(int64_t)k * a.H + u0 + row16] : (k < K ? a.wr[(int64_t)(k - a.F) * a.H + u0 + row16] : 0.f);
      }
    }
  }
  // the element this thread finishes per step: row tid / 16, unit tid % 16
  const int crow = tid >> 4, cu = tid & 15;
  const bool live = r0 + crow < a.rows;
  const int64_t ci = (int64_t)(live ? r0 + crow : 0) * a.H + u0 + cu;
  // operand loads (see lstm_sequence_fwd_kernel): lane p fetches chunk (p % 4) ^ (p / 16) of row p / 4
  const int chunk = (lane & 3) ^ (lane >> 4);
  const int64_t arow = min(r0 + (lane >> 2), a.rows - 1);
  const float* xrow = BACKWARD ? nullptr : a.x + arow * a.T * a.F;
  float* aw = As + wave * NKBW * 256;
  const float* ar = aw + (row16 * 4 + (g ^ (row16 >> 2))) * 4;

  const int steps = BACKWARD ? a.T - 1 : a.T;
  bool spread = true;  // until arrival 0 is complete (the first wait below)
  // ---- weight gradient: accumulators, operand rows, the step of slice T - 1
  typedef float xwv __attribute__((ext_vector_type(WG ? XW : 2)));
  constexpr int XWAVE = NKBW % 4;  // the wavefront that takes the x features: the first one without a run of r, if there is one
  f4v accr[4], accx[WG ? XW : 1], ah[4];
  xwv ax[4];
  const bool x_lane = XW * row16 < a.wg_F;
  unsigned hoff = 4u * (g * a.H + 4 * row16), xoff = 4u * (g * a.T * a.wg_F + (x_lane ? XW * row16 : 0));
  auto request_operands = [&](int tt) {  // [x_tt | r_{tt-1}] of rows g + 4 i
    const float* hs = a.wg_r + (int64_t)tt * a.slice + r0 * a.H + 64 * min(wave, NKBW - 1);
    const float* xs = a.wg_x + ((int64_t)r0 * a.T + tt) * a.wg_F;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ah[i] = *(const f4v*)at_bytes(hs + 4 * i * a.H, hoff);
      ax[i] = *(const xwv*)at_bytes(xs + (int64_t)4 * i * a.T * a.wg_F, xoff);
    }
  };
  auto weight_gradient_step = [&]() {  // += [x | r]^T (16 rows) * dr (the tile in LDS)
    const float* dzr = Dzs + g * 16 + row16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float b = dzr[4 * i * 16];
      if (wave < NKBW) {
#pragma unroll
        for (int j = 0; j < 4; ++j) accr[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[i][j], b, accr[j], 0, 0, 0);
      }
      if (wave == XWAVE) {
#pragma unroll
        for (int j = 0; j < XW; ++j) accx[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(x_lane ? ax[i][j] : 0.f, b, accx[j], 0, 0, 0);
      }
    }
  };
  if constexpr (WG) {
#pragma unroll
    for (int j = 0; j < 4; ++j) accr[j] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < XW; ++j) accx[j] = f4v{0.f, 0.f, 0.f, 0.f};
    request_operands(a.T - 1);
    Dzs[crow * 16 + cu] = live ? a.rec[(int64_t)(a.T - 1) * a.slice + ci] : 0.f;
    __syncthreads();
    weight_gradient_step();
    request_operands(a.T - 2);
  }
  for (int s = 0; s < steps; ++s) {
    if constexpr (WG) asm volatile("" : "+v"(hoff), "+v"(xoff));  // (keeps the offsets one register each: see lstm_sequence_bwd_body)
    const int t = BACKWARD ? a.T - 1 - s : s;  // the step whose operand slice is read
    if (s > 0) {  // the slice is complete once every unit group of this row group has arrived s + 1 times (arrival 0 included)
      if (wait_arrivals(my_count, (unsigned)a.unit_groups * (unsigned)(s + 1), abort_word, a.spin_limit, a.gave_up, a.failed, &stop)) return;
      if (s == 1) spread = __hip_atomic_load(my_spread, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
    }
    const bool with_rec = BACKWARD || s > 0 || a.first_valid;
    const bool coherent = spread && s > 0;  // the first slice was written before this launch
    const float* xt = BACKWARD ? nullptr : xrow + (int64_t)t * a.F;
    const float* rt = a.rec + (int64_t)t * a.slice + arow * a.H - a.F;  // indexed by k
#pragma unroll
    for (int i = 0; i < NKBW; ++i) {
      const int k0 = 16 * (wave * NKBW + i) + 4 * chunk;
      const float* src = k0 < a.F ? xt + k0 : (k0 < K && with_rec ? rt + k0 : seq_zero_chunk);
      if (coherent) __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(aw + i * 256), 16, 0, 16);  // sc1: coherent at device scope
      else __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(aw + i * 256), 16, 0, 0);
    }
    // the blocks are this wavefront's own: no barrier, block i is multiplied once all but the loads behind it have landed
    f4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NKBW; ++i) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKBW - 1 - i) : "memory");
      const f4v av = *(const f4v*)(ar + i * 256);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[v], bw[i][v], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) Ps[(wave * SRB + 4 * g + v) * ZP + row16] = acc[v];
    __syncthreads();
    const int to = BACKWARD ? t - 1 : t + 1;
    if (live) {
      float val = (Ps[crow * ZP + cu] + Ps[(SRB + crow) * ZP + cu]) + (Ps[(2 * SRB + crow) * ZP + cu] + Ps[(3 * SRB + crow) * ZP + cu]);
      if (BACKWARD && a.dy_seq) val = val + a.dy_seq[((int64_t)(r0 + crow) * a.T + to) * a.H + u0 + cu];
      float* out = a.rec + (int64_t)to * a.slice + ci;
      if (spread) __hip_atomic_store(out, val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else *out = val;
      if constexpr (WG) Dzs[crow * 16 + cu] = val;
    } else if constexpr (WG) {
      Dzs[crow * 16 + cu] = 0.f;
    }
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));  // vmcnt(0): the stores are acknowledged
    __syncthreads();  // (also: Ps is free again, the dr tile is published)
    if (tid == 0 && s + 1 < steps) __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if constexpr (WG) {  // slice `to` is this workgroup's own: its share of the weight gradient while the others arrive
      weight_gradient_step();
      if (to > 0) request_operands(to - 1);
    }
  }
  if constexpr (WG) {  // this row group's partial: rows 0..F-1 (x), F..F+H-1 (r)
    const int N = a.H;
    float* out = a.wpartial + (int64_t)rg * (a.wg_F + a.H + 1) * N + u0 + row16;
    if (wave == XWAVE) {
#pragma unroll
      for (int j = 0; j < XW; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = XW * (4 * g + v) + j;
          if (m < a.wg_F) out[(int64_t)m * N] = accx[j][v];
        }
    }
    if (wave < NKBW) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) out[(int64_t)(a.wg_F + 64 * wave + 4 * (4 * g + v) + j) * N] = accr[j][v];
    }
  }
}

// ---------------------------------------------------------------------------- backward step, fused
// One launch per reverse time step: the gate gradients of step t (element-wise) and the product that carries the
// hidden gradient back, dh_{t-1} = sum over gates of dz_gate * Wr_gate^T.  A workgroup owns BR batch rows x BU hidden
// units: it turns those cells' dh, dc and saved gates into dz (written out for the weight-gradient GEMM and kept in
// LDS as the product's A operand, k = gate * BU + unit), and multiplies by the matching K slice of the recurrent
// weights, which travels to LDS with LDS-direct loads while the element-wise part runs.  Every workgroup so
// contributes one K slice of dh_{t-1} for its rows: the H / BU partial results are written side by side and the next
// (earlier) step adds them in slice order.  Every cell belongs to exactly one workgroup per column chunk.
//   do = dh * tanh(c);  dc += (1 - tanh(c)^2) * (dh * o)
//   df = dc * c_prev;   di = dc * g;   dg = dc * i;   dc_prev = dc * f
//   dz_gate = act'(z_gate) * d_gate  (sigmoid: s(1-s), tanh: 1 - g^2)
constexpr int BR = 16, BU = 32, BK4 = 4 * BU, BKP = BK4 + 4, BN_MAX = 128;

struct StepBwdArgs {
  const float* gates;    // [rows, 4H] activated f, i, g, o of this step
  const float* c;        // c_t
  const float* c_prev;   // c_{t-1} or null (zeros)
  const float* dh;       // dh_parts arrays, dh_part_stride elements apart, added in order; may be null with dh_parts == 0
  int dh_parts;
  int64_t dh_part_stride;
  const float* dy_seq;   // optional: this step's slice of the gradient of a returned sequence, row r at dy_seq + r * dy_seq_ld
  int64_t dy_seq_ld;
  const float* dc_in;    // dc carried from step t+1, or null (zeros)
  float* dc_out;         // dc for step t-1 (a different buffer than dc_in: other workgroups still read that one)
  float* dz;             // [rows, 4H]
  const float* wpack;    // recurrent weights in LDS order (pack_bwd_kernel), null: no product (first time step)
  float* dh_out;         // [H / BU][part_stride] partial dh_{t-1}
  int64_t out_part_stride;
  int rows, H;
};

// [slice of BU units][column block of 16 inputs n][k quad q of the slice's 4*BU k][16 columns][4 consecutive k]:
// k = gate * BU + unit, value Wr_gate[n][slice * BU + unit]
__global__ __launch_bounds__(256) void pack_bwd_kernel(LstmWeights w, int H, float* __restrict__ out) {
  const int64_t cells = (int64_t)(H / BU) * (H / 16) * (BK4 / 4) * 16;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < cells; e += (int64_t)gridDim.x * 256) {
    const int col = (int)(e & 15);
    int64_t t = e >> 4;
    const int q = (int)(t % (BK4 / 4)); t /= (BK4 / 4);
    const int cb = (int)(t % (H / 16));
    const int slice = (int)(t / (H / 16));
    const int gate = (4 * q) / BU, ul = (4 * q) % BU;
    *(f4v*)(out + e * 4) = *(const f4v*)(w.wr[gate] + (int64_t)(cb * 16 + col) * H + slice * BU + ul);
  }
}

__global__ __launch_bounds__(256) void lstm_step_bwd_kernel(StepBwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* As = lds;              // [BR][BKP]
  float* Bs = lds + BR * BKP;   // [column blocks of this chunk][BK4 / 4][16][4]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int slice = blockIdx.x, r0 = blockIdx.y * BR, n0 = blockIdx.z * BN_MAX;
  const int ncols = min(BN_MAX, a.H - n0), ncb = ncols / 16;  // H % 16 == 0
  const bool product = a.wpack != nullptr;

  // ---- everything the workgroup's cells need is requested first (two cells per thread, every load in flight at once),
  // the weight slab right behind it, so the element-wise arithmetic runs while the slab is still on its way
  constexpr int CELLS = BR * BU / 256, MAX_PARTS = 8;
  float f[CELLS], in[CELLS], gg[CELLS], o[CELLS], cc[CELLS], cp[CELLS], dcv[CELLS], dyv[CELLS], dhp[CELLS][MAX_PARTS];
  bool live[CELLS];
#pragma unroll
  for (int ci = 0; ci < CELLS; ++ci) {
    const int e = tid + ci * 256, row = e / BU, ul = e % BU;
    live[ci] = r0 + row < a.rows;
    const int64_t i = (int64_t)(live[ci] ? r0 + row : 0) * a.H + slice * BU + ul;
    const int64_t zb = (int64_t)(live[ci] ? r0 + row : 0) * 4 * a.H + slice * BU + ul;
    f[ci] = a.gates[zb];
    in[ci] = a.gates[zb + a.H];
    gg[ci] = a.gates[zb + 2 * a.H];
    o[ci] = a.gates[zb + 3 * a.H];
    cc[ci] = a.c[i];
    cp[ci] = a.c_prev ? a.c_prev[i] : 0.f;
    dcv[ci] = a.dc_in ? a.dc_in[i] : 0.f;
    dyv[ci] = a.dy_seq ? a.dy_seq[(int64_t)(live[ci] ? r0 + row : 0) * a.dy_seq_ld + slice * BU + ul] : 0.f;
#pragma unroll
    for (int p = 0; p < MAX_PARTS; ++p) dhp[ci][p] = p < a.dh_parts ? a.dh[i + p * a.dh_part_stride] : 0.f;
  }
  // the weight slab for this slice and column chunk: one contiguous run in the pack, copied 1 KiB per issue
  if (product) {
    const float* slab = a.wpack + ((int64_t)slice * (a.H / 16) + n0 / 16) * (BK4 / 4) * 64;
    const uint32_t bytes = (uint32_t)ncb * (BK4 / 4) * 64 * 4;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(slab), 0, (int)bytes, 0x00020000);
    for (uint32_t off = (uint32_t)wave * 1024u; off < bytes; off += 4096u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)((char*)Bs + off), 16, (int)(off + lane * 16), 0, 0, 0);
  }

  // ---- gate gradients of this workgroup's cells (only column chunk 0 writes them out: the chunks share the cells)
  const bool writer = blockIdx.z == 0;
#pragma unroll
  for (int ci = 0; ci < CELLS; ++ci) {
    const int e = tid + ci * 256, row = e / BU, ul = e % BU;
    float dzf = 0.f, dzi = 0.f, dzg = 0.f, dzo = 0.f;
    if (live[ci]) {
      const int u = slice * BU + ul;
      const int64_t i = (int64_t)(r0 + row) * a.H + u;
      const int64_t zb = (int64_t)(r0 + row) * 4 * a.H + u;
      const float tc = tanhf(cc[ci]);
      float dh = dhp[ci][0];
#pragma unroll
      for (int p = 1; p < MAX_PARTS; ++p)
        if (p < a.dh_parts) dh += dhp[ci][p];
      for (int p = MAX_PARTS; p < a.dh_parts; ++p) dh += a.dh[i + p * a.dh_part_stride];  // more slices than registers hold
      if (a.dy_seq) dh = dh + dyv[ci];
      const float d_o = dh * tc;
      float dc = dcv[ci] + (1.0f - tc * tc) * (dh * o[ci]);
      const float df = dc * cp[ci], di = dc * gg[ci], dg = dc * in[ci];
      dzf = (f[ci] * (1.0f - f[ci])) * df;
      dzi = (in[ci] * (1.0f - in[ci])) * di;
      dzg = (1.0f - gg[ci] * gg[ci]) * dg;
      dzo = (o[ci] * (1.0f - o[ci])) * d_o;
      if (writer) {
        a.dc_out[i] = dc * f[ci];
        a.dz[zb] = dzf;
        a.dz[zb + a.H] = dzi;
        a.dz[zb + 2 * a.H] = dzg;
        a.dz[zb + 3 * a.H] = dzo;
      }
    }
    float* arow = As + row * BKP + ul;
    arow[0] = dzf;
    arow[BU] = dzi;
    arow[2 * BU] = dzg;
    arow[3 * BU] = dzo;
  }
  if (!product) return;
  __builtin_amdgcn_s_waitcnt(0);  // this wavefront's LDS-direct loads have landed
  __syncthreads();

  // ---- dh partial [BR x ncols] = As [BR x BK4] * Bs: wavefront w takes column blocks w, w + 4, ...
  const int c16 = lane & 15, g = lane >> 4;
  f4v acc[BN_MAX / 64];
#pragma unroll
  for (int j = 0; j < BN_MAX / 64; ++j) acc[j] = f4v{0.f, 0.f, 0.f, 0.f};
  const float* ap = As + c16 * BKP + 4 * g;
#pragma unroll 2
  for (int kb = 0; kb < BK4 / 16; ++kb) {
    const f4v av = *(const f4v*)(ap + 16 * kb);
    f4v bv[BN_MAX / 64];
#pragma unroll
    for (int j = 0; j < BN_MAX / 64; ++j) {
      const int cb = wave + 4 * j;
      bv[j] = cb < ncb ? *(const f4v*)(Bs + (((int64_t)cb * (BK4 / 4) + kb * 4 + g) * 16 + c16) * 4) : f4v{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
      for (int j = 0; j < BN_MAX / 64; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[v], bv[j][v], acc[j], 0, 0, 0);
  }
  float* out = a.dh_out + (int64_t)slice * a.out_part_stride;
#pragma unroll
  for (int j = 0; j < BN_MAX / 64; ++j) {
    const int cb = wave + 4 * j;
    if (cb >= ncb) continue;
    const int col = n0 + cb * 16 + c16;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = r0 + 4 * g + v;
      if (row < a.rows) out[(int64_t)row * a.H + col] = acc[j][v];
    }
  }
}

// ---------------------------------------------------------------------------- all backward steps in one launch
// The reverse recurrence, built like lstm_sequence_fwd_kernel: a workgroup owns 16 batch rows x 16 hidden units for the
// whole sequence, keeps dc of its cells and the recurrent weights of its units (all 4H k-values) in registers.
// What the unit groups of a row group hand to each other is dz_t itself, which has to be written anyway (the
// weight-gradient GEMM reads it): a workgroup turns dh_t, dc and the saved gates of its cells into its 64 columns of
// dz_t, counts itself in, waits for the others, reads the 16 complete rows of dz_t and multiplies them by its weight
// slab, which is dh_{t-1} of its own cells and never leaves the workgroup.  Every dz slice is written once and read
// once per launch, so the two hand-over forms of the forward kernel apply unchanged (plain accesses within an XCD,
// device-coherent ones otherwise), and so do the placement check and the bounded wait.
//   do = dh * tanh(c);  dc += (1 - tanh(c)^2) * (dh * o)
//   df = dc * c_prev;   di = dc * g;   dg = dc * i;   dc_prev = dc * f
//   dz_gate = act'(z_gate) * d_gate;   dh_{t-1}[r, u] = sum_{gate, n} dz_t[r, gate H + n] * Wr_gate[u][n]
// Wavefront w multiplies the rows by gate w's quarter of the 4H k-values; the four partial sums meet in LDS and are
// added in a fixed order.
struct SeqBwdArgs {
  const float* gates;    // T slices of 4 * slice floats: activated forget, input, gate, output of [rows, 4H]
  const float* c;        // T slices
  const float* c0;       // [rows, H] or null: zeros
  const float* dh_last;  // [rows, H] gradient of h_{T-1}, or null
  const float* dy_seq;   // [rows, T, H] gradient of a returned sequence (every step adds its own slice), or null
  const float* wr[4];    // [H, H] recurrent weights of forget, input, gate, output
  float* dz;             // T slices of 4 * slice floats
  int64_t slice;
  int rows, T, H;
  int row_groups, unit_groups;
  unsigned* sync;        // zero at launch, as in SeqFwdArgs
  unsigned spin_limit;
  int* gave_up;
  int* failed;
  int force_coherent;
  // the weight gradient riding along (XW > 0 instantiations only)
  const float* x;        // [rows, T, F]
  const float* h;        // T + 1 slices, slice t = h_{t-1}
  float* wpartial;       // [row_groups][F + H + 1][4H]: every row group's own sum over its rows and all steps
  int F;
};

// The weight gradient can ride along (XW > 0: x features per lane, 2 or 4; H a multiple of 64).  dW[m, n] = sum over
// (t, row) of [x_t | h_{t-1}][row, m] * dz_t[row, n], and a workgroup holds its 16 rows x 64 columns of dz_t the moment it
// has computed them: it keeps the [F + H, 64] block of the sum that belongs to its rows and columns in accumulator
// registers for the whole launch.  Per step the dz tile goes to LDS (the B operand: lane (n, g) reads row g + 4 i), the
// operand rows come straight from memory a step ahead (lane (m, g) holds 4 consecutive features of row g + 4 i, so MFMA
// (j, i) multiplies features {4 m + j} by rows {g + 4 i}: accumulator tile j collects every fourth feature), and the
// multiplications run between the workgroup's arrival and its wait for the others, where its wavefronts would idle.
// Wavefront w owns a 64-feature run of h (all its gate tiles, or a share of them when H < 256) and the x features of gate
// tile w.  The bias gradient is each thread's running sum of its own four dz values, added over the 16 rows at the end.
// What leaves is one partial [F + H + 1, 4H] per row group, which splitk_reduce adds in a fixed order.
constexpr int DZP = 80;  // row pitch of the dz tile in LDS: rows g and g + 1 land in different halves of the banks

template <int NKB, int XW>  // 16-long k blocks per wavefront: H = 16 NKB
__device__ __forceinline__ void lstm_sequence_bwd_body(const SeqBwdArgs& a) {
  constexpr int UB = 16, H = 16 * NKB;
  constexpr bool WG = XW > 0;
  constexpr int S = WG ? NKB / 4 : 1;  // 64-feature runs of h = gate tiles per wavefront
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ int stop;
  float* Ps = lds;                 // [4 quarters of k][SRB][ZP] partial dh
  float* As = lds + 4 * SRB * ZP;  // (16-byte aligned) [wavefront][k block][16 rows x 16 k]: dz_t as the loads deliver it
  float* Dzs = As + SRB * 4 * H;   // [SRB][DZP]: this workgroup's own 64 columns of dz_t (weight gradient only)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int slot = blockIdx.x >> 3;
  const int rg = (blockIdx.x & 7) + 8 * (slot / a.unit_groups), ug = slot % a.unit_groups;
  if (rg >= a.row_groups) return;
  const int r0 = rg * SRB, u0 = ug * UB;
  unsigned* my_count = a.sync + rg * SEQ_GROUP_WORDS;
  unsigned* my_xcd = my_count + 1;
  unsigned* my_spread = my_count + 2;
  unsigned* abort_word = a.sync + a.row_groups * SEQ_GROUP_WORDS;

  if (tid == 0) {  // arrival 0 (the placement check): do the members of this row group share an XCD?
    const unsigned mine = 1u + (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u);  // HW_REG_XCC_ID, 4 bits
    unsigned seen = 0u;
    __hip_atomic_compare_exchange_strong(my_xcd, &seen, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((seen != 0u && seen != mine) || a.force_coherent) __hip_atomic_store(my_spread, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
    __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  const int row16 = lane & 15, g = lane >> 4;
  // Wavefront w multiplies the k-values of gate w (k = w H .. w H + H - 1).  Its part of the unit group's weights stays in
  // registers in MFMA operand order: lane (unit, g) holds Wr_w[unit][n = 16 kb + 4 g .. + 3] of block kb, 16 contiguous
  // bytes of the layer's own tensor, read once per launch.
  f4v bw[NKB];
  {
    const float* wrow = a.wr[wave] + (int64_t)(u0 + row16) * H + 4 * g;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) bw[kb] = *(const f4v*)(wrow + 16 * kb);
  }
  // the cell this thread owns: row tid / 16, unit tid % 16
  const int crow = tid >> 4, cu = tid & 15;
  const bool live = r0 + crow < a.rows;
  // per-lane offsets are unsigned 32-bit byte counts (the launch checks the sizes): with a uniform base per access they
  // travel as one register and the base in scalar registers
  const unsigned cr = live ? r0 + crow : 0;
  unsigned ci = 4u * (cr * H + u0 + cu), zi = 4u * (cr * 4 * H + u0 + cu);
  const int64_t yi = (int64_t)cr * a.T * H + u0 + cu;
  float f, in, gg, o, cc, cp, dyv, dh, dcv = 0.f;
  {
    const int t = a.T - 1;
    const float* gt = a.gates + (int64_t)t * 4 * a.slice;
    f = *at_bytes(gt, zi);
    in = *at_bytes(gt + H, zi);
    gg = *at_bytes(gt + 2 * H, zi);
    o = *at_bytes(gt + 3 * H, zi);
    cc = *at_bytes(a.c + (int64_t)t * a.slice, ci);
    cp = t > 0 ? *at_bytes(a.c + (int64_t)(t - 1) * a.slice, ci) : (a.c0 ? *at_bytes(a.c0, ci) : 0.f);
    dyv = a.dy_seq ? a.dy_seq[yi + (int64_t)t * H] : 0.f;
    dh = a.dh_last ? *at_bytes(a.dh_last, ci) : 0.f;
  }
  // One load instruction brings a 16-row x 16-k block of dz_t to 1 KiB of LDS, lane p to bytes 16 p .. 16 p + 15: four
  // neighbouring lanes fetch the 64 contiguous bytes of one row (rows past the batch: the last row again, their results
  // belong to no cell), and chunk c of row r lands in slot c ^ (r / 4) of the row so that the 16 lanes that later read
  // one chunk index of 16 rows hit 16 different bank groups.
  unsigned a_off = 4u * ((unsigned)min(r0 + (lane >> 2), a.rows - 1) * 4 * H + 4 * ((lane & 3) ^ (lane >> 4)));
  float* aw = As + wave * NKB * 256;
  const float* ar = aw + (row16 * 4 + (g ^ (row16 >> 2))) * 4;
  bool spread = true;  // until arrival 0 is complete (the first wait below), write as if the row group were spread out
  // ---- weight gradient: accumulators, operand addresses and the operand rows of the first step
  const int sw = wave / (4 / S), nt0 = (wave % (4 / S)) * S;  // this wavefront's run of h features and its first gate tile
  f4v acch[WG ? 4 : 1][S], accx[WG ? XW : 1];
  typedef float xwv __attribute__((ext_vector_type(WG ? XW : 2)));
  f4v ah[4];
  xwv ax[4];
  float bsum[4] = {0.f, 0.f, 0.f, 0.f};
  const bool x_lane = XW * row16 < a.F;  // lanes past the last feature load the row's first ones and multiply zeros
  // (the batch is a multiple of 16 rows here: row g + 4 i is a uniform distance from row g, one per-lane offset serves all four)
  unsigned hoff = 4u * (g * H + 4 * row16), xoff = 4u * (g * a.T * a.F + (x_lane ? XW * row16 : 0));
  auto request_operands = [&](int t) {  // [x_t | h_{t-1}] of rows g + 4 i: 16 bytes of h and XW floats of x per lane and row
    const float* hs = a.h + (int64_t)t * a.slice + r0 * H + 64 * sw;
    const float* xs = a.x + ((int64_t)r0 * a.T + t) * a.F;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ah[i] = *(const f4v*)at_bytes(hs + 4 * i * H, hoff);
      ax[i] = *(const xwv*)at_bytes(xs + (int64_t)4 * i * a.T * a.F, xoff);
    }
  };
  if constexpr (WG) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int n = 0; n < S; ++n) acch[j][n] = f4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < XW; ++j) accx[j] = f4v{0.f, 0.f, 0.f, 0.f};
    request_operands(a.T - 1);
  }
  // These multiplications are off the chain the next step waits for; the other workgroup of the CU may be on its chain, so
  // they run at the lower of two wavefront priorities.
  auto weight_gradient_step = [&]() {  // += [x_t | h_{t-1}]^T (16 rows) * dz_t (the tile in LDS)
    const float* dzr = Dzs + g * DZP + row16;
    __builtin_amdgcn_s_setprio(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float bx = dzr[4 * i * DZP + 16 * wave];
#pragma unroll
      for (int j = 0; j < XW; ++j) accx[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(x_lane ? ax[i][j] : 0.f, bx, accx[j], 0, 0, 0);
#pragma unroll
      for (int n = 0; n < S; ++n) {
        const float bh = dzr[4 * i * DZP + 16 * (nt0 + n)];
#pragma unroll
        for (int j = 0; j < 4; ++j) acch[j][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[i][j], bh, acch[j][n], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_setprio(1);
  };
  if constexpr (WG) __builtin_amdgcn_s_setprio(1);
  for (int t = a.T - 1;; --t) {
    // (opaque per step: otherwise the compiler folds each offset into a 64-bit per-lane pointer of its own that it carries
    // through the loop, two registers per access instead of one for all)
    asm volatile("" : "+v"(ci), "+v"(zi), "+v"(a_off), "+v"(hoff), "+v"(xoff));
    // ---- gate gradients of step t
    if constexpr (WG) {
      if (!live) {
#pragma unroll
        for (int q = 0; q < 4; ++q) Dzs[crow * DZP + 16 * q + cu] = 0.f;
      }
    }
    if (live) {
      const float tc = tanhf(cc);
      float d = dh;
      if (a.dy_seq) d = d + dyv;
      const float d_o = d * tc;
      const float dc = dcv + (1.0f - tc * tc) * (d * o);
      const float df = dc * cp, di = dc * gg, dg = dc * in;
      const float dzf = (f * (1.0f - f)) * df;
      const float dzi = (in * (1.0f - in)) * di;
      const float dzg = (1.0f - gg * gg) * dg;
      const float dzo = (o * (1.0f - o)) * d_o;
      dcv = dc * f;
      float* zt = a.dz + (int64_t)t * 4 * a.slice;
      if (spread) {
        __hip_atomic_store(at_bytes(zt, zi), dzf, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(at_bytes(zt + H, zi), dzi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(at_bytes(zt + 2 * H, zi), dzg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(at_bytes(zt + 3 * H, zi), dzo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        *at_bytes(zt, zi) = dzf;
        *at_bytes(zt + H, zi) = dzi;
        *at_bytes(zt + 2 * H, zi) = dzg;
        *at_bytes(zt + 3 * H, zi) = dzo;
      }
      if constexpr (WG) {
        float* dl = Dzs + crow * DZP + cu;
        dl[0] = dzf;
        dl[16] = dzi;
        dl[32] = dzg;
        dl[48] = dzo;
        bsum[0] += dzf;
        bsum[1] += dzi;
        bsum[2] += dzg;
        bsum[3] += dzo;
      }
    }
    if (!WG && t == 0) break;
    // ---- hand dz_t over: stores acknowledged in every wavefront, then one thread counts the workgroup in
    //      (with the weight gradient the last step comes this far too: the barrier publishes its dz tile)
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));  // vmcnt(0)
    __syncthreads();
    if (tid == 0 && t > 0) __hip_atomic_fetch_add(my_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // ---- what step t - 1 needs from the forward pass is requested while the others arrive
    if (t > 0) {
      const float* gt = a.gates + (int64_t)(t - 1) * 4 * a.slice;
      f = *at_bytes(gt, zi);
      in = *at_bytes(gt + H, zi);
      gg = *at_bytes(gt + 2 * H, zi);
      o = *at_bytes(gt + 3 * H, zi);
      cc = cp;
      cp = t > 1 ? *at_bytes(a.c + (int64_t)(t - 2) * a.slice, ci) : (a.c0 ? *at_bytes(a.c0, ci) : 0.f);
      dyv = a.dy_seq ? a.dy_seq[yi + (int64_t)(t - 1) * H] : 0.f;
    }
    // ---- this step's share of the weight gradient while the others arrive (the tile was published by the barrier above),
    //      then the operand rows of step t - 1, which have a whole step to land
    if constexpr (WG) {
      weight_gradient_step();
      if (t == 0) break;
    }
    const int done = a.T - 1 - t;  // hand-overs before this one
    if (wait_arrivals(my_count, (unsigned)a.unit_groups * (unsigned)(done + 2), abort_word, a.spin_limit, a.gave_up, a.failed, &stop)) return;
    if (done == 0) spread = __hip_atomic_load(my_spread, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
    // ---- dh_{t-1} of this workgroup's cells = dz_t (16 complete rows) * the weight slab
    {
      // Block kb lies 64 kb bytes further along the row and 1024 kb bytes further in LDS.  The instruction's immediate offset
      // moves both addresses, so one per-lane address serves all blocks: the LDS base handed over is 64 kb bytes short.
      const global_ptr_t ap = (global_ptr_t)at_bytes(a.dz + (int64_t)t * 4 * a.slice + wave * H, a_off);
      if (spread) load_row_blocks<0, NKB, 16>(ap, aw);  // sc1: coherent at device scope
      else load_row_blocks<0, NKB, 0>(ap, aw);
      // The weight gradient's operand rows of step t - 1 are requested behind these loads (8 load instructions): in front
      // of them they would have to land before the first block could be multiplied, in front of the wait before the poll
      // could return.  They have a whole step to land.
      constexpr int YOUNGER = WG ? 8 : 0;
      if constexpr (WG) request_operands(t - 1);
      // The blocks are this wavefront's own, so no barrier: block kb is multiplied as soon as all but the NKB - 1 - kb loads
      // behind it (and the YOUNGER ones behind those) have landed (loads return in order; the compiler does not order LDS
      // reads behind these loads by itself).
      f4v acc[2] = {f4v{0.f, 0.f, 0.f, 0.f}, f4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKB - 1 - kb + YOUNGER) : "memory");
        const f4v av = *(const f4v*)(ar + kb * 256);
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[kb & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[v], bw[kb][v], acc[kb & 1], 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) Ps[(wave * SRB + 4 * g + v) * ZP + row16] = acc[0][v] + acc[1][v];
    }
    if constexpr (WG) {  // (not __syncthreads: its fence would wait for the operand rows requested above)
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the partial sums are in LDS
      __builtin_amdgcn_s_barrier();
    } else {
      __syncthreads();
    }
    dh = (Ps[crow * ZP + cu] + Ps[(SRB + crow) * ZP + cu]) + (Ps[(2 * SRB + crow) * ZP + cu] + Ps[(3 * SRB + crow) * ZP + cu]);
  }
  if constexpr (WG) {
    // ---- this row group's partial: rows 0..F-1 (x), F..F+H-1 (h), F+H (column sums of dz)
    const int N = 4 * H;
    float* out = a.wpartial + (int64_t)rg * (a.F + H + 1) * N + u0 + row16;
#pragma unroll
    for (int j = 0; j < XW; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = XW * (4 * g + v) + j;
        if (m < a.F) out[(int64_t)m * N + wave * H] = accx[j][v];
      }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int n = 0; n < S; ++n)
#pragma unroll
        for (int v = 0; v < 4; ++v) out[(int64_t)(a.F + 64 * sw + 4 * (4 * g + v) + j) * N + (nt0 + n) * H] = acch[j][n][v];
    __syncthreads();  // every wavefront has read the tile: it now carries the per-thread column sums
#pragma unroll
    for (int q = 0; q < 4; ++q) Dzs[crow * DZP + 16 * q + cu] = bsum[q];
    __syncthreads();
    if (tid < 64) {
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < SRB; ++r) sum += Dzs[r * DZP + tid];
      a.wpartial[((int64_t)rg * (a.F + H + 1) + a.F + H) * N + (tid >> 4) * H + u0 + (tid & 15)] = sum;
    }
  }
}

template <int NKB>
__global__ __launch_bounds__(256) void lstm_sequence_bwd_kernel(SeqBwdArgs a) {
  lstm_sequence_bwd_body<NKB, 0>(a);
}

// two workgroups per CU = two wavefronts per SIMD: 256 registers each
template <int NKB, int XW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void lstm_sequence_bwd_wgrad_kernel(SeqBwdArgs a) {
  lstm_sequence_bwd_body<NKB, XW>(a);
}

size_t sequence_bwd_lds_bytes(int H, bool with_wgrad = false) {
  return ((size_t)4 * SRB * ZP + (size_t)SRB * 4 * H + (with_wgrad ? (size_t)SRB * DZP : 0)) * sizeof(float);
}

size_t lds_bytes(int K, int cols) {  // cols: output columns per workgroup (64 or 32)
  const int K16 = round16(K);
  const size_t slabs = (size_t)RB * (K16 + 4) + (size_t)cols * K16, exchange = 4 * RB * ZP;
  return (slabs > exchange ? slabs : exchange) * sizeof(float);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

bool lstm_step_fused_ok(int F, int H, const float* x, const LstmWeights& w, int gates) {
  if (F % 4 != 0 || H % 16 != 0 || F + H > MAX_K || !aligned16(x)) return false;
  for (int g = 0; g < gates; ++g)
    if (!aligned16(w.wk[g]) || !aligned16(w.wr[g])) return false;
  return true;
}

int64_t lstm_pack_elems(int F, int H) { return (int64_t)4 * H * round16(F + H); }

int launch_lstm_pack(sn_ctx* ctx, const LstmWeights& w, int F, int H, float* pack_fwd, float* pack_dh, int gates) {
  if (pack_fwd) {
    const int64_t cells = (int64_t)gates * (H / 4) * round16(F + H);
    LaunchScope scope(ctx, "lstm_pack_weights");
    hipLaunchKernelGGL(pack_fwd_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(cells, 256), 2048)), dim3(256), 0, ctx->stream, w, F, H, gates,
                       pack_fwd);
  }
  if (pack_dh) {
    const int64_t cells = (int64_t)gates * (H / 4) * round16(H);
    LaunchScope scope(ctx, "lstm_pack_weights");
    hipLaunchKernelGGL(pack_dh_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(cells, 256), 2048)), dim3(256), 0, ctx->stream, w, H, gates,
                       pack_dh);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}

namespace {
// 32 units per workgroup (two workgroups per CU) when 64 would leave fewer than two per CU: 10.8 vs 11.4 us per LSTM step
int launch_step_product(sn_ctx* ctx, const StepMulArgs& a, int zs) {
  const int K = a.k0 + (a.a1 ? a.k1 : 0);
  const bool narrow = ceil_div(a.cols, 64) * ceil_div(a.rows, RB) * zs < (int64_t)2 * ctx->compute_units;
  if (narrow) {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)step_product_kernel<32>, lds_bytes(MAX_K, 32)));
    hipLaunchKernelGGL(step_product_kernel<32>, dim3((unsigned)ceil_div(a.cols, 32), (unsigned)ceil_div(a.rows, RB), (unsigned)zs), dim3(256),
                       lds_bytes(K, 32), ctx->stream, a);
  } else {
    SN_TRY(allow_dynamic_lds(ctx, (const void*)step_product_kernel<64>, lds_bytes(MAX_K, 64)));
    hipLaunchKernelGGL(step_product_kernel<64>, dim3((unsigned)ceil_div(a.cols, 64), (unsigned)ceil_div(a.rows, RB), (unsigned)zs), dim3(256),
                       lds_bytes(K, 64), ctx->stream, a);
  }
  SN_HIP(hipGetLastError());
  return SN_OK;
}
}  // namespace

int launch_lstm_step_fwd(sn_ctx* ctx, const float* x, int t, int T, int F, const float* h_prev, const float* c_prev, int rows, int H,
                         const LstmWeights& w, const float* wpack, float* gates, float* c, float* h) {
  if (rows <= 0) return SN_OK;
  SN_REQUIRE(lstm_step_fused_ok(F, H, x, w), "lstm_step_forward: F=%d H=%d outside what the fused kernel handles", F, H);
  StepFwdArgs a{x, h_prev, c_prev, w, wpack, gates, c, h, rows, T, F, H, t};
  const int K = h_prev ? F + H : F;
  // 16 units per workgroup.  The 8-unit form (two workgroups per CU) was measured slower here (13.0 vs 12.0 us per
  // step at 512 x 1024 x 288): it re-reads the [x_t, h] slab twice as often, and the step is bound by that traffic.
  LaunchScope scope(ctx, "lstm_step_forward", rows, 4 * H, K);
  SN_TRY(allow_dynamic_lds(ctx, (const void*)lstm_step_fwd_kernel, lds_bytes(MAX_K, 64)));
  hipLaunchKernelGGL(lstm_step_fwd_kernel, dim3((unsigned)(H / 16), (unsigned)ceil_div(rows, RB)), dim3(256), lds_bytes(K, 64), ctx->stream, a);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

namespace {
size_t sequence_lds_bytes(int nkb) { return (size_t)(nkb * 256 + 4 * SRB * ZP) * sizeof(float); }  // operand blocks + exchange area

// calls f(kernel, blocks of 16 k) for the smallest instantiation that covers K, or returns false
template <typename F>
bool with_sequence_fwd_kernel(int K, F&& f) {
  const int need = (K + 15) / 16;
  if (need <= 2) f(lstm_sequence_fwd_kernel<2>, 2);
  else if (need <= 3) f(lstm_sequence_fwd_kernel<3>, 3);
  else if (need <= 5) f(lstm_sequence_fwd_kernel<5>, 5);
  else if (need <= 8) f(lstm_sequence_fwd_kernel<8>, 8);
  else if (need <= 12) f(lstm_sequence_fwd_kernel<12>, 12);
  else if (need <= 18) f(lstm_sequence_fwd_kernel<18>, 18);
  else if (need <= 25) f(lstm_sequence_fwd_kernel<25>, 25);
  else return false;
  return true;
}
}  // namespace

// true once a one-launch kernel of this context has given up waiting, reported to the caller or not yet (the flag sits
// in pinned host memory, so looking needs no synchronisation): from then on the per-step kernels run
static bool sequence_kernels_off(const sn_ctx* ctx) {
  return ctx->seq_disabled || (ctx->seq_gave_up && *(volatile int*)ctx->seq_gave_up != 0);
}
static bool lstm_sequence_fwd_fits(sn_ctx* ctx, int rows, int F, int H, const float* x, const LstmWeights& w) {
  if (rows <= 0 || !lstm_step_fused_ok(F, H, x, w)) return false;
  const int64_t groups = ceil_div(rows, SRB), blocks = 8 * ceil_div(groups, 8) * (H / 16);
  if (groups > SEQ_MAX_GROUPS) return false;
  bool fits = false;
  const bool known = with_sequence_fwd_kernel(F + H, [&](auto kernel, int nkb) {
    if (allow_dynamic_lds(ctx, (const void*)kernel, sequence_lds_bytes(nkb)) != SN_OK) return;
    int per_cu = 0;  // the hand-over between workgroups needs the whole grid resident at once
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, sequence_lds_bytes(nkb)) != hipSuccess) return;
    fits = blocks <= (int64_t)per_cu * ctx->compute_units;
  });
  return known && fits;
}
bool lstm_sequence_fwd_ok(sn_ctx* ctx, int rows, int F, int H, const float* x, const LstmWeights& w) { return !sequence_kernels_off(ctx) && lstm_sequence_fwd_fits(ctx, rows, F, H, x, w); }

int launch_lstm_sequence_fwd(sn_ctx* ctx, const float* x, int T, int F, int h0_valid, const float* c0, int rows, int H, const LstmWeights& w,
                             float* gates, float* c, float* h, int64_t slice) {
  if (rows <= 0 || T <= 0) return SN_OK;
  SN_REQUIRE(lstm_sequence_fwd_fits(ctx, rows, F, H, x, w), "lstm_sequence_forward: rows=%d F=%d H=%d do not fit the device in one launch", rows, F, H);
  SN_REQUIRE(aligned16(h), "lstm_sequence_forward: operands must start on 16-byte boundaries");
  const int groups = (int)ceil_div(rows, SRB);
  unsigned* sync = nullptr;
  SN_TRY(seq_sync_take(ctx, groups, &sync));
  SeqFwdArgs a{x, c0, {w.wk[0], w.wk[1], w.wk[2], w.wk[3]}, {w.wr[0], w.wr[1], w.wr[2], w.wr[3]}, {w.b[0], w.b[1], w.b[2], w.b[3]}, gates, c, h, slice, h0_valid, rows, T, F, H, groups, H / 16,
               sync, ctx->seq_spin_limit, ctx->seq_gave_up_dev, ctx->seq_failed_dev, ctx->seq_force_coherent};
  LaunchScope scope(ctx, "lstm_sequence_forward", rows * T, 4 * H, F + H);  // T steps of rows x 4H x (F + H)
  with_sequence_fwd_kernel(F + H, [&](auto kernel, int nkb) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * ceil_div(groups, 8) * (H / 16))), dim3(256), sequence_lds_bytes(nkb), ctx->stream, a);
  });
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_lstm_step_dh(sn_ctx* ctx, const float* dz, int rows, int H, const float* wpack, float* dh_parts, int64_t part_stride, int gates) {
  if (rows <= 0) return SN_OK;
  SN_REQUIRE(H % 16 == 0 && H <= MAX_K && aligned16(dz) && aligned16(wpack), "lstm_step_hidden_gradient: H=%d outside what the fused kernel handles", H);
  const int kq = round16(H) / 4;
  StepMulArgs a{dz, (int64_t)gates * H, H, nullptr, 0, 0, H, wpack, kq, (int64_t)(H / 16) * kq * 64, dh_parts, H, part_stride, rows, H};
  LaunchScope scope(ctx, "lstm_step_hidden_gradient", rows, H, gates * H);
  return launch_step_product(ctx, a, gates);
}

bool lstm_step_bwd_fused_ok(int H, const LstmWeights& w) {
  if (H % BU != 0) return false;
  for (int g = 0; g < 4; ++g)
    if (!aligned16(w.wr[g])) return false;
  return true;
}

int lstm_bwd_parts(int H) { return H / BU; }

int launch_lstm_pack_bwd(sn_ctx* ctx, const LstmWeights& w, int H, float* pack) {
  const int64_t cells = (int64_t)(H / BU) * (H / 16) * (BK4 / 4) * 16;
  LaunchScope scope(ctx, "lstm_pack_weights");
  hipLaunchKernelGGL(pack_bwd_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(cells, 256), 2048)), dim3(256), 0, ctx->stream, w, H, pack);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

int launch_lstm_step_bwd(sn_ctx* ctx, const LstmGateBwdArgs& g, const float* dc_in, float* dc_out, const float* wpack, float* dh_out,
                         int64_t out_part_stride, int rows, int H) {
  if (rows <= 0) return SN_OK;
  SN_REQUIRE(H % BU == 0 && (!wpack || aligned16(wpack)), "lstm_step_backward: H=%d outside what the fused kernel handles", H);
  SN_REQUIRE(dc_in != dc_out, "lstm_step_backward: the cell gradient needs two buffers");
  StepBwdArgs a{g.gates, g.c, g.c_prev, g.dh, g.dh_parts, g.dh_part_stride, g.dy_seq, g.dy_seq_ld, dc_in, dc_out, g.dz, wpack, dh_out,
                out_part_stride, rows, H};
  const int chunks = wpack ? (int)ceil_div(H, BN_MAX) : 1;
  const size_t smem = ((size_t)BR * BKP + (size_t)std::min(H, BN_MAX) * BK4) * sizeof(float);
  LaunchScope scope(ctx, "lstm_step_backward", rows, H, 4 * H);
  SN_TRY(allow_dynamic_lds(ctx, (const void*)lstm_step_bwd_kernel, ((size_t)BR * BKP + (size_t)BN_MAX * BK4) * sizeof(float)));
  hipLaunchKernelGGL(lstm_step_bwd_kernel, dim3((unsigned)(H / BU), (unsigned)ceil_div(rows, BR), (unsigned)chunks), dim3(256), smem, ctx->stream, a);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

namespace {
// calls f(kernel) for the instantiation that handles H, or returns false
template <typename F>
bool with_sequence_bwd_kernel(int H, F&& f) {
  switch (H) {
    case 16: f(lstm_sequence_bwd_kernel<1>); return true;
    case 32: f(lstm_sequence_bwd_kernel<2>); return true;
    case 64: f(lstm_sequence_bwd_kernel<4>); return true;
    case 128: f(lstm_sequence_bwd_kernel<8>); return true;
    case 256: f(lstm_sequence_bwd_kernel<16>); return true;
    default: return false;
  }
}
}  // namespace

static bool lstm_sequence_bwd_fits(sn_ctx* ctx, int rows, int H, const LstmWeights& w) {
  if (rows <= 0) return false;
  for (int g = 0; g < 4; ++g)
    if (!aligned16(w.wr[g])) return false;
  const int64_t groups = ceil_div(rows, SRB), blocks = 8 * ceil_div(groups, 8) * (H / 16);
  if (groups > SEQ_MAX_GROUPS || (int64_t)rows * 4 * H >= ((int64_t)1 << 30)) return false;  // (the kernel's per-lane byte offsets are 32-bit)
  bool fits = false;
  const bool known = with_sequence_bwd_kernel(H, [&](auto kernel) {
    if (allow_dynamic_lds(ctx, (const void*)kernel, sequence_bwd_lds_bytes(H)) != SN_OK) return;
    int per_cu = 0;  // the hand-over between workgroups needs the whole grid resident at once
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, sequence_bwd_lds_bytes(H)) != hipSuccess) return;
    fits = blocks <= (int64_t)per_cu * ctx->compute_units;
  });
  return known && fits;
}
bool lstm_sequence_bwd_ok(sn_ctx* ctx, int rows, int H, const LstmWeights& w) { return !sequence_kernels_off(ctx) && lstm_sequence_bwd_fits(ctx, rows, H, w); }

namespace {
// calls f(kernel) for the instantiation that also accumulates the weight gradient, or returns false
template <typename Fn>
bool with_sequence_bwd_wgrad_kernel(int H, int F, Fn&& f) {
  const int xw = F % 2 == 0 && F <= 32 ? 2 : (F % 4 == 0 && F <= 64 ? 4 : 0);
  if (xw == 0) return false;
  switch (H * 8 + xw) {
    case 64 * 8 + 2: f(lstm_sequence_bwd_wgrad_kernel<4, 2>); return true;
    case 64 * 8 + 4: f(lstm_sequence_bwd_wgrad_kernel<4, 4>); return true;
    case 128 * 8 + 2: f(lstm_sequence_bwd_wgrad_kernel<8, 2>); return true;
    case 128 * 8 + 4: f(lstm_sequence_bwd_wgrad_kernel<8, 4>); return true;
    case 256 * 8 + 2: f(lstm_sequence_bwd_wgrad_kernel<16, 2>); return true;
    case 256 * 8 + 4: f(lstm_sequence_bwd_wgrad_kernel<16, 4>); return true;
    default: return false;
  }
}

bool sequence_wgrad_wanted() {  // SCANET_SEQUENCE_WGRAD=0 keeps the weight gradient in its own launch
  const char* e = getenv("SCANET_SEQUENCE_WGRAD");
  return !(e && e[0] == '0');
}
}  // namespace

// Floats of workspace the backward launch needs to carry the weight gradient along (one partial per 16-row group), or 0
// where it cannot (shape).
int64_t lstm_sequence_bwd_wgrad_workspace(int rows, int T, int F, int H) {
  if (rows <= 0 || rows % SRB != 0 || T <= 0 || (int64_t)rows * T * F >= ((int64_t)1 << 30)) return 0;
  if (!with_sequence_bwd_wgrad_kernel(H, F, [](auto) {})) return 0;
  return ceil_div(rows, SRB) * (int64_t)(F + H + 1) * 4 * H;
}

static bool lstm_sequence_bwd_wgrad_fits(sn_ctx* ctx, int rows, int T, int F, int H, const float* x, const float* h, const float* ws, int64_t ws_elems) {
  const int64_t need = lstm_sequence_bwd_wgrad_workspace(rows, T, F, H);
  if (!sequence_wgrad_wanted() || need == 0 || !ws || need > ws_elems || !aligned16(x) || !aligned16(h)) return false;
  const int64_t groups = ceil_div(rows, SRB), blocks = 8 * ceil_div(groups, 8) * (H / 16);
  bool fits = false;
  with_sequence_bwd_wgrad_kernel(H, F, [&](auto kernel) {
    if (allow_dynamic_lds(ctx, (const void*)kernel, sequence_bwd_lds_bytes(H, true)) != SN_OK) return;
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, sequence_bwd_lds_bytes(H, true)) != hipSuccess) return;
    fits = blocks <= (int64_t)per_cu * ctx->compute_units;
  });
  return fits;
}

// With x, h (T + 1 slices, slice t = h_{t-1}) and a workspace the launch also leaves the weight gradient's partial sums
// [*wgrad_parts][F + H + 1][4H] in ws where the shape allows it (*wgrad_parts = 0 otherwise: the caller runs the product).
int launch_lstm_sequence_bwd(sn_ctx* ctx, const float* gates, const float* c, const float* c0, const float* dh_last, const float* dy_seq, int T,
                             int rows, int H, const LstmWeights& w, float* dz, int64_t slice, const float* x, const float* h, int F, float* ws,
                             int64_t ws_elems, int* wgrad_parts) {
  if (wgrad_parts) *wgrad_parts = 0;
  if (rows <= 0 || T <= 0) return SN_OK;
  SN_REQUIRE(lstm_sequence_bwd_fits(ctx, rows, H, w), "lstm_sequence_backward: rows=%d H=%d do not fit the device in one launch", rows, H);
  SN_REQUIRE(aligned16(dz), "lstm_sequence_backward: operands must start on 16-byte boundaries");
  const int groups = (int)ceil_div(rows, SRB);
  const bool with_wgrad = wgrad_parts && x && h && lstm_sequence_bwd_wgrad_fits(ctx, rows, T, F, H, x, h, ws, ws_elems);
  unsigned* sync = nullptr;
  SN_TRY(seq_sync_take(ctx, groups, &sync));
  SeqBwdArgs a{gates, c, c0, dh_last, dy_seq, {w.wr[0], w.wr[1], w.wr[2], w.wr[3]}, dz, slice, rows, T, H, groups, H / 16,
               sync, ctx->seq_spin_limit, ctx->seq_gave_up_dev, ctx->seq_failed_dev, ctx->seq_force_coherent, x, h, ws, F};
  const dim3 grid((unsigned)(8 * ceil_div(groups, 8) * (H / 16)));
  if (with_wgrad) {
    // T - 1 products of rows x H x 4H and T of (F + H) x 4H x rows: as one shape, rows x 4H x ((T - 1) H + T (F + H)) / T per step
    LaunchScope scope(ctx, "lstm_sequence_backward_and_weight_gradient", rows, 4 * H, (T - 1) * H + T * (F + H));
    with_sequence_bwd_wgrad_kernel(H, F, [&](auto kernel) {
      hipLaunchKernelGGL(kernel, grid, dim3(256), sequence_bwd_lds_bytes(H, true), ctx->stream, a);
    });
    SN_HIP(hipGetLastError());
    *wgrad_parts = groups;
    return SN_OK;
  }
  LaunchScope scope(ctx, "lstm_sequence_backward", rows * (T - 1), H, 4 * H);  // T - 1 products of rows x H x 4H
  with_sequence_bwd_kernel(H, [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), sequence_bwd_lds_bytes(H), ctx->stream, a);
  });
  SN_HIP(hipGetLastError());
  return SN_OK;
}

// r_t[rows, H] = [x_t, r_prev] * [Wk; Wr]: the simple cell's step (pack from launch_lstm_pack(.., gates = 1))
int launch_rnn_step_fwd(sn_ctx* ctx, const float* x, int t, int T, int F, const float* r_prev, int rows, int H, const float* wpack, float* out) {
  if (rows <= 0) return SN_OK;
  SN_REQUIRE(F % 4 == 0 && H % 16 == 0 && F + H <= MAX_K && aligned16(x) && aligned16(wpack) && (!r_prev || aligned16(r_prev)),
             "rnn_step_forward: F=%d H=%d outside what the fused kernel handles", F, H);
  StepMulArgs a{x + (int64_t)t * F, (int64_t)T * F, F, r_prev, H, H, 0, wpack, round16(F + H) / 4, 0, out, H, 0, rows, H};
  LaunchScope scope(ctx, "rnn_step_forward", rows, H, r_prev ? F + H : F);
  return launch_step_product(ctx, a, 1);
}

namespace {
size_t rnn_sequence_lds_bytes(int nkbw, bool with_wgrad = false) {
  return ((size_t)4 * SRB * ZP + (size_t)4 * nkbw * 256 + (with_wgrad ? SRB * 16 : 0)) * sizeof(float);
}

// calls f(kernel, blocks per wavefront) for the backward instantiation that also accumulates the weight gradient, or returns false
template <typename Fn>
bool with_rnn_sequence_wgrad_kernel(int H, int F, Fn&& f) {
  if (F % 4 != 0 || F > 64) return false;
  const bool two = F <= 32;
  switch (H) {
    case 64: two ? f(rnn_sequence_kernel<true, 1, 2>, 1) : f(rnn_sequence_kernel<true, 1, 4>, 1); return true;
    case 128: two ? f(rnn_sequence_kernel<true, 2, 2>, 2) : f(rnn_sequence_kernel<true, 2, 4>, 2); return true;
    case 192: two ? f(rnn_sequence_kernel<true, 3, 2>, 3) : f(rnn_sequence_kernel<true, 3, 4>, 3); return true;
    case 256: two ? f(rnn_sequence_kernel<true, 4, 2>, 4) : f(rnn_sequence_kernel<true, 4, 4>, 4); return true;
    default: return false;
  }
}

// calls f(kernel, blocks per wavefront) for the smallest instantiation that covers K, or returns false
template <bool BACKWARD, typename F>
bool with_rnn_sequence_kernel(int K, F&& f) {
  const int need = (int)ceil_div(ceil_div(K, 16), 4);
  if (need <= 1) f(rnn_sequence_kernel<BACKWARD, 1>, 1);
  else if (need <= 2) f(rnn_sequence_kernel<BACKWARD, 2>, 2);
  else if (need <= 3) f(rnn_sequence_kernel<BACKWARD, 3>, 3);
  else if (need <= 4) f(rnn_sequence_kernel<BACKWARD, 4>, 4);
  else if (need <= 5) f(rnn_sequence_kernel<BACKWARD, 5>, 5);
  else if (need <= 7) f(rnn_sequence_kernel<BACKWARD, 7>, 7);
  else return false;
  return true;
}
template <bool BACKWARD>
bool rnn_sequence_fits(sn_ctx* ctx, int rows, int K, int H) {
  const int64_t groups = ceil_div(rows, SRB), blocks = 8 * ceil_div(groups, 8) * (H / 16);
  if (groups > SEQ_MAX_GROUPS) return false;
  bool fits = false;
  const bool known = with_rnn_sequence_kernel<BACKWARD>(K, [&](auto kernel, int nkbw) {
    if (allow_dynamic_lds(ctx, (const void*)kernel, rnn_sequence_lds_bytes(nkbw)) != SN_OK) return;
    int per_cu = 0;  // the hand-over between workgroups needs the whole grid resident at once
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, rnn_sequence_lds_bytes(nkbw)) != hipSuccess) return;
    fits = blocks <= (int64_t)per_cu * ctx->compute_units;
  });
  return known && fits;
}
template <bool BACKWARD>
int launch_rnn_sequence(sn_ctx* ctx, SeqMulArgs a, const char* name, int K) {
  a.row_groups = (int)ceil_div(a.rows, SRB);
  a.unit_groups = a.H / 16;
  SN_TRY(seq_sync_take(ctx, a.row_groups, &a.sync));
  a.spin_limit = ctx->seq_spin_limit;
  a.gave_up = ctx->seq_gave_up_dev;
  a.failed = ctx->seq_failed_dev;
  a.force_coherent = ctx->seq_force_coherent;
  const int steps = BACKWARD ? a.T - 1 : a.T;
  LaunchScope scope(ctx, name, a.rows * steps, a.H, K);  // `steps` products of rows x H x K
  with_rnn_sequence_kernel<BACKWARD>(K, [&](auto kernel, int nkbw) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * ceil_div(a.row_groups, 8) * a.unit_groups)), dim3(256), rnn_sequence_lds_bytes(nkbw),
                       ctx->stream, a);
  });
  SN_HIP(hipGetLastError());
  return SN_OK;
}
}  // namespace

static bool rnn_sequence_fwd_fits(sn_ctx* ctx, int rows, int F, int H, const float* x) {
  return rows > 0 && F % 4 == 0 && H % 16 == 0 && F + H <= MAX_K && aligned16(x) && rnn_sequence_fits<false>(ctx, rows, F + H, H);
}
bool rnn_sequence_fwd_ok(sn_ctx* ctx, int rows, int F, int H, const float* x) { return !sequence_kernels_off(ctx) && rnn_sequence_fwd_fits(ctx, rows, F, H, x); }

int launch_rnn_sequence_fwd(sn_ctx* ctx, const float* x, int T, int F, int first_valid, int rows, int H, const float* wk, const float* wr,
                            float* r_slices, int64_t slice) {
  if (rows <= 0 || T <= 0) return SN_OK;
  SN_REQUIRE(rnn_sequence_fwd_fits(ctx, rows, F, H, x), "rnn_sequence_forward: rows=%d F=%d H=%d do not fit the device in one launch", rows, F, H);
  SeqMulArgs a{};
  a.x = x; a.rec = r_slices; a.wk = wk; a.wr = wr; a.slice = slice; a.first_valid = first_valid;
  a.rows = rows; a.T = T; a.F = F; a.H = H;
  return launch_rnn_sequence<false>(ctx, a, "rnn_sequence_forward", F + H);
}

static bool rnn_sequence_bwd_fits(sn_ctx* ctx, int rows, int H, const float* wr) {
  return rows > 0 && H % 16 == 0 && H <= MAX_K && aligned16(wr) && rnn_sequence_fits<true>(ctx, rows, H, H);
}
bool rnn_sequence_bwd_ok(sn_ctx* ctx, int rows, int H, const float* wr) { return !sequence_kernels_off(ctx) && rnn_sequence_bwd_fits(ctx, rows, H, wr); }

// Floats of workspace the backward launch needs to carry the weight gradient along (one partial per 16-row group), or 0
// where it cannot (shape).
int64_t rnn_sequence_bwd_wgrad_workspace(int rows, int T, int F, int H) {
  if (rows <= 0 || rows % SRB != 0 || T <= 1 || (int64_t)rows * T * F >= ((int64_t)1 << 30) || (int64_t)rows * H >= ((int64_t)1 << 30)) return 0;
  if (!with_rnn_sequence_wgrad_kernel(H, F, [](auto, int) {})) return 0;
  return ceil_div(rows, SRB) * (int64_t)(F + H + 1) * H;
}

// With x [rows, T, F], the forward pass's slices r (slice t = r_{t-1}) and a workspace the launch also leaves the weight
// gradient's partial sums [*wgrad_parts][F + H + 1][H] in ws where the shape allows it (*wgrad_parts = 0 otherwise).
int launch_rnn_sequence_bwd(sn_ctx* ctx, float* dr_slices, const float* dy_seq, int T, int rows, int H, const float* wr, int64_t slice,
                            const float* x, const float* r_slices, int F, float* ws, int64_t ws_elems, int* wgrad_parts) {
  if (wgrad_parts) *wgrad_parts = 0;
  if (rows <= 0 || T <= 1) return SN_OK;
  SN_REQUIRE(rnn_sequence_bwd_fits(ctx, rows, H, wr), "rnn_sequence_backward: rows=%d H=%d do not fit the device in one launch", rows, H);
  SeqMulArgs a{};
  a.rec = dr_slices; a.dy_seq = dy_seq; a.wr = wr; a.slice = slice;
  a.rows = rows; a.T = T; a.F = 0; a.H = H;
  const int64_t need = rnn_sequence_bwd_wgrad_workspace(rows, T, F, H);
  bool with_wgrad = wgrad_parts && x && r_slices && sequence_wgrad_wanted() && need > 0 && ws && need <= ws_elems && aligned16(x) && aligned16(r_slices);
  if (with_wgrad) {  // the grid must still be resident at once with this instantiation's registers and LDS
    const int64_t groups = ceil_div(rows, SRB), blocks = 8 * ceil_div(groups, 8) * (H / 16);
    bool fits = false;
    with_rnn_sequence_wgrad_kernel(H, F, [&](auto kernel, int nkbw) {
      if (allow_dynamic_lds(ctx, (const void*)kernel, rnn_sequence_lds_bytes(nkbw, true)) != SN_OK) return;
      int per_cu = 0;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, rnn_sequence_lds_bytes(nkbw, true)) != hipSuccess) return;
      fits = blocks <= (int64_t)per_cu * ctx->compute_units;
    });
    with_wgrad = fits;
  }
  if (!with_wgrad) return launch_rnn_sequence<true>(ctx, a, "rnn_sequence_backward", H);
  a.wg_x = x; a.wg_r = r_slices; a.wpartial = ws; a.wg_F = F;
  a.row_groups = (int)ceil_div(a.rows, SRB);
  a.unit_groups = a.H / 16;
  SN_TRY(seq_sync_take(ctx, a.row_groups, &a.sync));
  a.spin_limit = ctx->seq_spin_limit;
  a.gave_up = ctx->seq_gave_up_dev;
  a.failed = ctx->seq_failed_dev;
  a.force_coherent = ctx->seq_force_coherent;
  // T - 1 products of rows x H x H and T of (F + H) x H x rows: as one shape, rows x H x ((T - 1) H + T (F + H))
  LaunchScope scope(ctx, "rnn_sequence_backward_and_weight_gradient", rows, H, (T - 1) * H + T * (F + H));
  with_rnn_sequence_wgrad_kernel(H, F, [&](auto kernel, int nkbw) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)(8 * ceil_div(a.row_groups, 8) * a.unit_groups)), dim3(256), rnn_sequence_lds_bytes(nkbw, true), ctx->stream, a);
  });
  SN_HIP(hipGetLastError());
  *wgrad_parts = a.row_groups;
  return SN_OK;
}

}  // namespace sn
