// Seeded random tensors, bit-compatible with the TensorFlow ops the reference's initializers lower to
// (math/rand/AllKernels.scala:12-43: RandomUniform, RandomStandardNormal, TruncatedNormal with a `seed` attribute).
//
// TensorFlow's CPU kernels draw from Philox4x32-10 keyed by the op seed (seed2 = 0): output group g (four consecutive
// outputs) is the generator's block at counter g, a uint32 becomes a float in [0,1) through its low 23 bits, normals
// come from Box-Muller on pairs, and the truncated normal keeps |f| < 2 from a stream of single samples that starts
// at counter 256 g for group g.  A counter-based generator needs no state: every thread computes its own group, so
// a tensor of any size is one pass that writes 16 bytes per thread.
#include "common.hpp"

namespace sn {
namespace {

typedef float rn_f4 __attribute__((ext_vector_type(4)));

struct Block {
  uint32_t v[4];
};

__device__ __forceinline__ Block philox(uint64_t counter, uint32_t k0, uint32_t k1) {
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0u, c3 = 0u;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    if (round) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
  }
  return Block{{c0, c1, c2, c3}};
}

__device__ __forceinline__ float to_unit(uint32_t x) { return __uint_as_float((x & 0x7fffffu) | (127u << 23)) - 1.0f; }

__device__ __forceinline__ void box_muller(uint32_t x0, uint32_t x1, float& f0, float& f1) {
  float u1 = to_unit(x0);
  if (u1 < 1.0e-7f) u1 = 1.0e-7f;
  const float v1 = (float)(6.283185307179586 * (double)to_unit(x1));  // `2.0f * M_PI * u` is a double product
  const float u2 = sqrtf(-2.0f * logf(u1));
  f0 = sinf(v1) * u2;
  f1 = cosf(v1) * u2;
}

__device__ __forceinline__ float finish(float x, int has_scale, float scale, int has_shift, float shift) {
  if (has_scale) x = x * scale;   // `rand`: multiply, then add, each only when asked for (math/rand/AllKernels.scala:76-80)
  if (has_shift) x = x + shift;
  return x;
}

// one thread per group of four outputs
__global__ __launch_bounds__(256) void random_fill_kernel(float* __restrict__ out, int64_t n, int dist, uint32_t k0, uint32_t k1,
                                                           int has_scale, float scale, int has_shift, float shift, int vec) {
  const int64_t groups = (n + 3) / 4;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += (int64_t)gridDim.x * blockDim.x) {
    float f[4];
    if (dist == SN_RANDOM_UNIFORM) {
      const Block b = philox((uint64_t)g, k0, k1);
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = to_unit(b.v[i]);
    } else if (dist == SN_RANDOM_NORMAL) {
      const Block b = philox((uint64_t)g, k0, k1);
      box_muller(b.v[0], b.v[1], f[0], f[1]);
      box_muller(b.v[2], b.v[3], f[2], f[3]);
    } else {
      // 256 generator blocks are reserved per group; a group that has not filled up by then (probability far below
      // 1e-300) keeps zeros, so the loop ends whatever the stream holds
      int got = 0;
      f[0] = f[1] = f[2] = f[3] = 0.f;
      for (int blk = 0; blk < 256 && got < 4; ++blk) {
        const Block b = philox((uint64_t)g * 256u + (uint64_t)blk, k0, k1);
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
          float a0, a1;
          box_muller(b.v[2 * pair], b.v[2 * pair + 1], a0, a1);
          if (got < 4 && fabsf(a0) < 2.0f) f[got++] = a0;
          if (got < 4 && fabsf(a1) < 2.0f) f[got++] = a1;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = finish(f[i], has_scale, scale, has_shift, shift);
    const int64_t e = g * 4;
    if (vec && e + 4 <= n) {
      *(rn_f4*)(out + e) = rn_f4{f[0], f[1], f[2], f[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (e + i < n) out[e + i] = f[i];
    }
  }
}

}  // namespace

int launch_random_fill(sn_ctx* ctx, float* out, int64_t n, int dist, uint64_t seed, const float* scale, const float* shift) {
  if (n <= 0) return SN_OK;
  SN_REQUIRE(dist >= SN_RANDOM_UNIFORM && dist <= SN_RANDOM_TRUNCATED_NORMAL, "unknown distribution %d", dist);
  // seed 0 (with seed2 = 0) makes TensorFlow pick seeds at random: there is no stream to reproduce
  SN_REQUIRE(seed != 0, "seed 0 means 'unseeded' to the reference's random ops; pass a non-zero seed");
  const int64_t groups = ceil_div(n, 4);
  int64_t blocks = ceil_div(groups, 256);
  const int64_t cap = (int64_t)ctx->compute_units * 32;
  if (blocks > cap) blocks = cap;
  const int vec = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
  LaunchScope scope(ctx, dist == SN_RANDOM_UNIFORM ? "random_uniform" : dist == SN_RANDOM_NORMAL ? "random_normal" : "random_truncated_normal");
  hipLaunchKernelGGL(random_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, out, n, dist, (uint32_t)seed, (uint32_t)(seed >> 32),
                     scale ? 1 : 0, scale ? *scale : 1.0f, shift ? 1 : 0, shift ? *shift : 0.0f, vec);
  SN_HIP(hipGetLastError());
  return SN_OK;
}

}  // namespace sn
