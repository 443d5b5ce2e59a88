// What the matrix cores alone sustain on this part: nothing but v_mfma_f32_32x32x16_bf16 (4 x 4 accumulator tiles per
// wavefront, one wavefront per SIMD, the bf16 GEMM's MFMA stream without its loads, reads and stores), for operands that
// are all zero, that have random mantissas, and that are spread like N(0,1).  The rate depends on the data: the part is
// power limited.  Build and run:
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/mfma_peak_bf16 scanet3_amd/probes/mfma_peak_bf16.hip && /tmp/mfma_peak_bf16
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
// each wave: TI x TI accumulators of 32x32; operands from global once, then ITER rounds of TI*TI MFMAs x 4
template <int TI>
__global__ __launch_bounds__(256) void peak(const bf16x8* __restrict__ src, float* out, int iters) {
  f16v acc[TI][TI];
  for (int i = 0; i < TI; ++i) for (int j = 0; j < TI; ++j) for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  bf16x8 a[TI], b[TI];
  for (int i = 0; i < TI; ++i) { a[i] = src[(threadIdx.x * 8 + i) % 4096]; b[i] = src[(threadIdx.x * 8 + 4 + i) % 4096]; }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TI; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
  for (int i = 0; i < TI; ++i) for (int j = 0; j < TI; ++j) for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
template <int TI> void run(const char* name, const bf16x8* src, float* out, int blocks, int iters, int lds = 0) {
  if (lds) CK(hipFuncSetAttribute((const void*)peak<TI>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(peak<TI>, dim3(blocks), dim3(256), lds, 0, src, out, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(a));
  const int reps = 20;
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(peak<TI>, dim3(blocks), dim3(256), lds, 0, src, out, iters);
  CK(hipEventRecord(b)); CK(hipEventSynchronize(b));
  float ms; CK(hipEventElapsedTime(&ms, a, b)); ms /= reps;
  double flops = (double)blocks * 4 * iters * 4 * TI * TI * 32768.0;
  printf("%-40s %8.1f us %8.1f TFLOP/s\n", name, ms * 1e3, flops / ms / 1e9); fflush(stdout);
}
int main() {
  uint16_t* h = (uint16_t*)malloc(4096 * 16);
  bf16x8* src; float* out; CK(hipMalloc(&src, 4096 * 16)); CK(hipMalloc(&out, 4096 * 256 * 4));
  for (int mode = 0; mode < 3; mode += 2) {
    uint32_t st = 12345;
    for (int i = 0; i < 4096 * 8; ++i) {
      st = st * 1664525u + 1013904223u;
      // mode 0 zeros; mode 1 random mantissa around 1.0 with sign; mode 2 N(0,1)-like spread of exponents
      h[i] = mode == 0 ? 0 : mode == 1 ? (uint16_t)(0x3f80 + ((st >> 9) & 0x7f) + ((st >> 31) << 15)) : (uint16_t)(((st >> 8) & 0xffff & 0xbfff) | 0x3000);
    }
    CK(hipMemcpy(src, h, 4096 * 16, hipMemcpyHostToDevice));
    printf("data mode %d\n", mode);
    run<4>("256 blocks x 4096 it", src, out, 256, 4096);
    run<4>("512 blocks x 64 it", src, out, 512, 64);
    run<4>("512 blocks x 64 it, 128K LDS", src, out, 512, 64, 131072);
    run<4>("2048 blocks x 64 it, 128K LDS", src, out, 2048, 64, 131072);
    run<4>("2048 blocks x 64 it", src, out, 2048, 64);
    run<4>("256 blocks x 128 it", src, out, 256, 128);
    run<4>("256 blocks x 1024 it", src, out, 256, 1024);
  }
  return 0;
}
