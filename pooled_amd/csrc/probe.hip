// Device probe: what the f16 matrix pipe of this part sustains, and at which shader clock.
//
// Measurement infrastructure next to pa_timer_* (no counterpart in the reference).  One kernel, no memory traffic:
// every wavefront issues v_mfma_f32_32x32x16_f16 back to back on 8 independent accumulators, with either constant
// operands or 16 random f16 fragments rotated through the A / B ports.  The kernel reads the shader clock counter
// and the 100 MHz wall clock at entry and exit, so the caller gets the clock the power management allowed during the
// run together with the arithmetic rate: with constant operands an MI355X holds its nominal clock and 2.5 PFLOP/s,
// with operands that toggle it does not, and that second figure is the ceiling a real attention kernel meets.
#include "pa_internal.h"
#include <vector>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void pa_mfma_probe_kernel(const h8* frag, float* sink, unsigned long long* clk, uint32_t iters) {
  const long long c0 = clock64(), w0 = wall_clock64();
  h8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; i++) { a[i] = frag[i * 256 + threadIdx.x]; b[i] = frag[(8 + i) * 256 + threadIdx.x]; }
  f16v acc[8];
#pragma unroll
  for (int k = 0; k < 8; k++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[k][i] = 0.f;
  for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 8; u++)
#pragma unroll
      for (int k = 0; k < 8; k++) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(u + k) & 7], b[k], acc[k], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < 8; k++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[k][i];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) { clk[blockIdx.x * 2] = clock64() - c0; clk[blockIdx.x * 2 + 1] = wall_clock64() - w0; }
}

// blocks = 2 per CU (8 wavefronts per CU); 64 MFMAs of 32768 flops per wavefront and iteration
hipError_t pa_run_mfma_probe(int n_cu, bool random_operands, uint32_t iters, hipStream_t st, float* tflops, float* shader_mhz) {
  const uint32_t blocks = 2 * (uint32_t)n_cu;
  std::vector<_Float16> h(16 * 256 * 8);
  uint32_t lcg = 12345u;
  for (auto& x : h) { lcg = lcg * 1664525u + 1013904223u; x = random_operands ? (_Float16)(((int)(lcg >> 20) % 2001 - 1000) / 500.f) : (_Float16)0.5f; }
  h8* frag = nullptr; float* sink = nullptr; unsigned long long* clk = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e;
  auto done = [&](hipError_t r) { if (frag) (void)hipFree(frag); if (sink) (void)hipFree(sink); if (clk) (void)hipFree(clk); if (e0) (void)hipEventDestroy(e0); if (e1) (void)hipEventDestroy(e1); return r; };
  if ((e = hipMalloc((void**)&frag, h.size() * 2)) != hipSuccess) return done(e);
  if ((e = hipMalloc((void**)&sink, (size_t)blocks * 256 * 4)) != hipSuccess) return done(e);
  if ((e = hipMalloc((void**)&clk, (size_t)blocks * 16)) != hipSuccess) return done(e);
  if ((e = hipMemcpy(frag, h.data(), h.size() * 2, hipMemcpyHostToDevice)) != hipSuccess) return done(e);
  if ((e = hipEventCreate(&e0)) != hipSuccess || (e = hipEventCreate(&e1)) != hipSuccess) return done(e);
  hipExtLaunchKernelGGL(pa_mfma_probe_kernel, dim3(blocks), dim3(256), 0, st, e0, e1, 0, (const h8*)frag, sink, clk, iters);
  if ((e = hipGetLastError()) != hipSuccess) return done(e);
  if ((e = hipEventSynchronize(e1)) != hipSuccess) return done(e);
  float ms = 0.f;
  if ((e = hipEventElapsedTime(&ms, e0, e1)) != hipSuccess) return done(e);
  std::vector<unsigned long long> hc((size_t)blocks * 2);
  if ((e = hipMemcpy(hc.data(), clk, hc.size() * 8, hipMemcpyDeviceToHost)) != hipSuccess) return done(e);
  double mhz = 0.0;
  for (uint32_t b = 0; b < blocks; b++) mhz += hc[2 * b + 1] ? 100.0 * (double)hc[2 * b] / (double)hc[2 * b + 1] : 0.0;
  *shader_mhz = (float)(mhz / blocks);
  *tflops = (float)((double)blocks * 4.0 * iters * 64.0 * 32768.0 / ((double)ms * 1e-3) / 1e12);
  return done(hipSuccess);
}
