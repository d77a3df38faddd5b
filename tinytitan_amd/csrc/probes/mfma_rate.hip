// Sustained v_mfma_f32_32x32x16_f16 rate on gfx950 as a function of the operand DATA.
//
// The matrix pipe issues one 32x32x16 MFMA per 32 shader clocks per SIMD whatever the data, but
// the shader clock it sustains depends on how much the operands toggle: constant operands
// hold ~2.1 GHz, random fp16 operands pull the card to its power limit and the clock falls
// to ~1.4-1.6 GHz.  This probe prints, for a few operand/accumulator patterns, the achieved
// TFLOP/s, the shader clocks per MFMA (s_memtime) and the clock implied by the two.
// It is the measured ceiling the prefill attention kernel is compared with: a kernel that
// computes on random data cannot reach the 2.5 PFLOP/s the clock-rate arithmetic gives.
//
// Build and run:  hipcc -O3 --offload-arch=gfx950 -o mfma_rate tinytitan_amd/csrc/probes/mfma_rate.hip && ./mfma_rate
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
template <int CHAINS, int NOPER>
__global__ __launch_bounds__(512) void k(int iters, float* out, const _Float16* data, long long* cycles) {
  h8 a[NOPER], b[NOPER];
  for (int i = 0; i < NOPER; ++i) {
    a[i] = *(const h8*)(data + ((threadIdx.x * NOPER + i) * 16 + 0));
    b[i] = *(const h8*)(data + ((threadIdx.x * NOPER + i) * 16 + 8));
  }
  f16v acc[CHAINS];
  for (int c = 0; c < CHAINS; ++c) acc[c] = (f16v)0.0f;
  long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 16 / CHAINS; ++r)
#pragma unroll
      for (int c = 0; c < CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(r * CHAINS + c) % NOPER], b[(r * CHAINS + c) % NOPER], acc[c], 0, 0, 0);
  }
  float s = 0; for (int c = 0; c < CHAINS; ++c) s += acc[c][0] + acc[c][7];
  long long t1 = clock64();
  if (threadIdx.x == 0 && blockIdx.x == 0) cycles[0] = t1 - t0;
  if (s == 12345.0f) out[0] = s;
}
template <int CHAINS, int NOPER> void run(int threads, const char* name, const _Float16* data) {
  float* out; CK(hipMalloc(&out, 64)); long long* cyc; CK(hipMalloc(&cyc, 64));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = 4000;
  k<CHAINS, NOPER><<<256, threads>>>(100, out, data, cyc); CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0)); k<CHAINS, NOPER><<<256, threads>>>(iters, out, data, cyc); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  long long c; CK(hipMemcpy(&c, cyc, 8, hipMemcpyDeviceToHost));
  double mfmas_per_wave = (double)iters * 16;
  double flops = mfmas_per_wave * 32768.0 * (threads / 64) * 256;
  printf("%s waves/SIMD %d: %.3f ms  %.1f TFLOP/s  %.1f shader clk per MFMA per SIMD, clock %.2f GHz\n", name, threads / 256, ms, flops / ms * 1e-9,
         (double)c / (mfmas_per_wave * (threads / 256.0)), (double)c / (ms * 1e6));
}
int main() {
  const int n = 512 * 16 * 16;
  _Float16* h = (_Float16*)malloc(n * 2); _Float16* hc = (_Float16*)malloc(n * 2);
  srand(1); for (int i = 0; i < n; ++i) { h[i] = (_Float16)((rand() / (float)RAND_MAX) * 2.0f - 1.0f); hc[i] = (_Float16)0.5f; }
  _Float16 *d, *dc; CK(hipMalloc(&d, n * 2)); CK(hipMalloc(&dc, n * 2));
  CK(hipMemcpy(d, h, n * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(dc, hc, n * 2, hipMemcpyHostToDevice));
  run<1, 1>(256, "const data, 1 operand pair, chain x1   ", dc);
  run<1, 1>(256, "random data, 1 operand pair, chain x1  ", d);
  run<1, 16>(256, "random data, 16 operand pairs, chain x1", d);
  run<8, 16>(256, "random data, 16 operand pairs, 8 chains", d);
  run<1, 16>(512, "random data, 16 operand pairs, chain x1", d);
  run<8, 8>(512, "random data, 8 operand pairs, 8 chains ", d);
  run<8, 16>(256, "const data, 16 operand pairs, 8 chains ", dc);
  return 0;
}
