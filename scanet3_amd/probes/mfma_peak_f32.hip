// What the matrix cores alone sustain in float32: nothing but v_mfma_f32_32x32x2_f32 (or 16x16x4) on six accumulator
// tiles per wavefront (and, at the end, on 1 to 16 tiles and on operands that change from MFMA to MFMA), for launches as short as the convolution kernels' (87 iterations = the filter gradient's MFMA
// count per wavefront) and for long ones, on zeros and on random operands.  Build and run:
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/mfma_peak_f32 scanet3_amd/probes/mfma_peak_f32.hip && /tmp/mfma_peak_f32
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
template <int WAVES, int KIND>  // KIND 0: 32x32x2, 1: 16x16x4
__global__ __launch_bounds__(64 * WAVES) void peak(const float* __restrict__ src, float* out, int iters) {
  f16v acc[6];
  f4v acc4[6];
  for (int i = 0; i < 6; ++i) { for (int v = 0; v < 16; ++v) acc[i][v] = 0.f; for (int v = 0; v < 4; ++v) acc4[i][v] = 0.f; }
  float a[3], b[2];
  for (int i = 0; i < 3; ++i) a[i] = src[(threadIdx.x * 8 + i) % 4096];
  for (int i = 0; i < 2; ++i) b[i] = src[(threadIdx.x * 8 + 4 + i) % 4096];
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (KIND == 0) acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i * 2 + j], 0, 0, 0);
        else acc4[i * 2 + j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc4[i * 2 + j], 0, 0, 0);
      }
  }
  float s = 0.f;
  for (int i = 0; i < 6; ++i) { for (int v = 0; v < 16; ++v) s += acc[i][v]; for (int v = 0; v < 4; ++v) s += acc4[i][v]; }
  out[blockIdx.x * 64 * WAVES + threadIdx.x] = s;
}
template <int WAVES, int KIND> void run(const char* name, const float* src, float* out, int blocks, int iters) {
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL((peak<WAVES, KIND>), dim3(blocks), dim3(64 * WAVES), 0, 0, src, out, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  const int reps = 20;
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL((peak<WAVES, KIND>), dim3(blocks), dim3(64 * WAVES), 0, 0, src, out, iters);
  CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
  float ms; CK(hipEventElapsedTime(&ms, a, b)); ms /= reps;
  double per = KIND == 0 ? 4096.0 : 2048.0;
  double flops = (double)blocks * WAVES * iters * 6 * per;
  double cyc = ms * 1e-3 * 2.4e9 / ((double)iters * 6);
  printf("%-44s %8.1f us %8.1f TFLOP/s  (%.1f cycles@2.4GHz per MFMA per wave)\n", name, ms * 1e3, flops / ms / 1e9, cyc); fflush(stdout);
}
// More accumulator tiles per wavefront (MA x NB tiles of 32 x 32, the shape of a register-blocked GEMM) and operands that
// change from MFMA to MFMA (SETS register sets walked in turn), one wavefront per SIMD.
template <int MA, int NB, int SETS>
__global__ __launch_bounds__(256) void peak_tiles(const float* __restrict__ src, float* out, int iters) {
  f16v acc[MA * NB];
  for (int i = 0; i < MA * NB; ++i) for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  float a[SETS][MA], b[SETS][NB];
  for (int d = 0; d < SETS; ++d) {
    for (int i = 0; i < MA; ++i) a[d][i] = src[(threadIdx.x * 8 + i + 97 * d) % 4096];
    for (int i = 0; i < NB; ++i) b[d][i] = src[(threadIdx.x * 8 + 4 + i + 131 * d) % 4096];
  }
  for (int it = 0; it < iters; it += SETS) {
#pragma unroll
    for (int d = 0; d < SETS; ++d)
#pragma unroll
      for (int i = 0; i < MA; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[i * NB + j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[d][i], b[d][j], acc[i * NB + j], 0, 0, 0);
  }
  float s = 0.f;
  for (int i = 0; i < MA * NB; ++i) for (int v = 0; v < 16; ++v) s += acc[i][v];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
template <int MA, int NB, int SETS> void run_tiles(const char* name, const float* src, float* out, int blocks, int iters) {
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL((peak_tiles<MA, NB, SETS>), dim3(blocks), dim3(256), 0, 0, src, out, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  const int reps = 20;
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL((peak_tiles<MA, NB, SETS>), dim3(blocks), dim3(256), 0, 0, src, out, iters);
  CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
  float ms; CK(hipEventElapsedTime(&ms, a, b)); ms /= reps;
  double flops = (double)blocks * 4 * iters * MA * NB * 4096.0;
  double cyc = ms * 1e-3 * 2.4e9 / ((double)iters * MA * NB);
  printf("%-44s %8.1f us %8.1f TFLOP/s  (%.1f cycles@2.4GHz per MFMA per wave)\n", name, ms * 1e3, flops / ms / 1e9, cyc); fflush(stdout);
}
int main() {
  float* h = (float*)malloc(4096 * 4);
  float* src; float* out; CK(hipMalloc(&src, 4096 * 4)); CK(hipMalloc(&out, 4096 * 1024 * 4));
  for (int mode = 0; mode < 2; ++mode) {
    uint32_t st = 12345;
    for (int i = 0; i < 4096; ++i) { st = st * 1664525u + 1013904223u; h[i] = mode == 0 ? 0.f : ((st >> 8) / 8388608.0f - 1.0f); }
    CK(hipMemcpy(src, h, 4096 * 4, hipMemcpyHostToDevice));
    printf("data mode %d\n", mode);
    run<4, 0>("32x32x2: 256 WG x 4 waves x 87 it", src, out, 256, 87);
    run<4, 0>("32x32x2: 240 WG x 4 waves x 87 it", src, out, 240, 87);
    run<4, 0>("32x32x2: 256 WG x 4 waves x 870 it", src, out, 256, 870);
    run<4, 0>("32x32x2: 256 WG x 4 waves x 8700 it", src, out, 256, 8700);
    run<8, 0>("32x32x2: 256 WG x 8 waves x 435 it", src, out, 256, 435);
    run<4, 0>("32x32x2: 1024 WG x 4 waves x 218 it", src, out, 1024, 218);
    run<4, 1>("16x16x4: 256 WG x 4 waves x 870 it", src, out, 256, 870);
    run<4, 1>("16x16x4: 1024 WG x 4 waves x 435 it", src, out, 1024, 435);
    run_tiles<1, 1, 1>("32x32x2: 1 tile, 240 WG x 2600 it", src, out, 240, 2600);
    run_tiles<3, 2, 1>("32x32x2: 3x2 tiles, 240 WG x 432 it", src, out, 240, 432);
    run_tiles<3, 4, 1>("32x32x2: 3x4 tiles, 240 WG x 408 it", src, out, 240, 408);
    run_tiles<4, 4, 1>("32x32x2: 4x4 tiles, 240 WG x 408 it", src, out, 240, 408);
    run_tiles<3, 4, 8>("32x32x2: 3x4 tiles, 8 operand sets, 408 it", src, out, 240, 408);
  }
  return 0;
}
