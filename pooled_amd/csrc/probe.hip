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

typedef unsigned int probe_u4 __attribute__((ext_vector_type(4)));
typedef __fp16 probe_hh4 __attribute__((__vector_size__(4 * sizeof(__fp16))));

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

typedef float probe_f4 __attribute__((ext_vector_type(4)));

// SMALL = false: v_mfma_f32_32x32x16_f16 on 8 accumulators; true: v_mfma_f32_16x16x32_f16 on 16 accumulators.  Both issue
// 64 x 32768 flops per wavefront and iteration.
template <bool SMALL>
__global__ __launch_bounds__(256) void pa_mfma_probe_kernel(const h8* frag, float* sink, unsigned long long* clk, uint32_t iters) {
  const long long c0 = clock64(), w0 = wall_clock64();
  h8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; i++) { a[i] = frag[i * 256 + threadIdx.x]; b[i] = frag[(8 + i) * 256 + threadIdx.x]; }
  float s = 0.f;
  if constexpr (!SMALL) {
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
#pragma unroll
    for (int k = 0; k < 8; k++)
#pragma unroll
      for (int i = 0; i < 16; i++) s += acc[k][i];
  } else {
    probe_f4 acc[16];
#pragma unroll
    for (int k = 0; k < 16; k++) acc[k] = (probe_f4){0.f, 0.f, 0.f, 0.f};
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
      for (int u = 0; u < 8; u++)
#pragma unroll
        for (int k = 0; k < 16; k++) acc[k] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(u + k) & 7], b[k & 7], acc[k], 0, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < 16; k++)
#pragma unroll
      for (int i = 0; i < 4; i++) s += acc[k][i];
  }
  sink[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) { clk[blockIdx.x * 2] = clock64() - c0; clk[blockIdx.x * 2 + 1] = wall_clock64() - w0; }
}

// blocks = 2 per CU (8 wavefronts per CU); 64 MFMAs of 32768 flops per wavefront and iteration
hipError_t pa_run_mfma_probe(int n_cu, bool random_operands, bool small_tiles, uint32_t iters, hipStream_t st, float* tflops, float* shader_mhz) {
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
  if (small_tiles) hipExtLaunchKernelGGL(pa_mfma_probe_kernel<true>, dim3(blocks), dim3(256), 0, st, e0, e1, 0, (const h8*)frag, sink, clk, iters);
  else hipExtLaunchKernelGGL(pa_mfma_probe_kernel<false>, dim3(blocks), dim3(256), 0, st, e0, e1, 0, (const h8*)frag, sink, clk, iters);
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

// Second probe: what the LDS of a CU delivers to fragment reads.  One workgroup per CU of `waves` wavefronts, every
// wavefront issues conflict-free ds_read_b128 (TR = false: 1 KB an instruction) or ds_read_b64_tr_b16 (TR = true:
// 512 bytes an instruction, the transpose read the V^T fragments use) back to back over a 64 KB buffer; the shader
// clock counter over the loop gives bytes per clock and CU.
template <bool TR>
__global__ __launch_bounds__(512) void pa_lds_probe_kernel(unsigned long long* clk, uint32_t* sink, uint32_t iters) {
  __shared__ __attribute__((aligned(1024))) unsigned char buf[65536];
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (uint32_t i = threadIdx.x; i < 65536 / 4; i += blockDim.x) ((uint32_t*)buf)[i] = i;
  __syncthreads();
  probe_u4 acc = {0u, 0u, 0u, 0u};
  const long long c0 = clock64();
  for (uint32_t it = 0; it < iters; it++) {
    const unsigned char* base = buf + (it & 3) * 8192 + (wave & 3) * 8192;        // 8 KB a wavefront and iteration
    if (!TR) {
#pragma unroll
      for (int j = 0; j < 8; j++) acc ^= *(const probe_u4*)(base + j * 1024 + lane * 16);
    } else {
#pragma unroll
      for (int j = 0; j < 16; j++) {
        probe_hh4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16((probe_hh4 __attribute__((address_space(3)))*)(base + j * 512 + lane * 8));
        uint2 w; __builtin_memcpy(&w, &t, 8); acc[0] ^= w.x; acc[1] ^= w.y;
      }
    }
  }
  const long long c1 = clock64();
  sink[blockIdx.x * blockDim.x + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (threadIdx.x == 0) clk[blockIdx.x] = (unsigned long long)(c1 - c0);
}

hipError_t pa_run_lds_probe(int n_cu, bool transpose_reads, uint32_t waves, uint32_t iters, hipStream_t st, float* bytes_per_clk) {
  unsigned long long* clk = nullptr; uint32_t* sink = nullptr;
  hipError_t e;
  auto done = [&](hipError_t r) { if (clk) (void)hipFree(clk); if (sink) (void)hipFree(sink); return r; };
  if ((e = hipMalloc((void**)&clk, (size_t)n_cu * 8)) != hipSuccess) return done(e);
  if ((e = hipMalloc((void**)&sink, (size_t)n_cu * waves * 64 * 4)) != hipSuccess) return done(e);
  for (int rep = 0; rep < 2; rep++) {
    if (transpose_reads) hipLaunchKernelGGL(pa_lds_probe_kernel<true>, dim3(n_cu), dim3(waves * 64), 0, st, clk, sink, iters);
    else hipLaunchKernelGGL(pa_lds_probe_kernel<false>, dim3(n_cu), dim3(waves * 64), 0, st, clk, sink, iters);
    if ((e = hipGetLastError()) != hipSuccess) return done(e);
  }
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return done(e);
  std::vector<unsigned long long> hc((size_t)n_cu);
  if ((e = hipMemcpy(hc.data(), clk, hc.size() * 8, hipMemcpyDeviceToHost)) != hipSuccess) return done(e);
  double clocks = 0.0;
  for (auto c : hc) clocks += (double)c;
  clocks /= (double)n_cu;
  *bytes_per_clk = clocks > 0.0 ? (float)((double)iters * 8192.0 * waves / clocks) : 0.f;
  return done(hipSuccess);
}
