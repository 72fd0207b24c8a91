// Measurement stand-ins for the one-column decode kernel's K/V stream (bench.py --stream-ceiling): kernels that do
// nothing but read 32 MiB of a K plane and 32 MiB of a V plane with a given launch shape -- optionally staged through
// LDS and followed by the stores of the split partials -- and an empty kernel of the same grid.  They say what a
// one-shot 64 MiB read can reach on this part with the decode kernel's launch shape, on the same clock (dispatch
// events, or a kernel trace) the decode kernel itself is timed with.  Not part of the attention path.
#include "pa_internal.h"

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

#define PROBE_CHUNKS 32768u          // 1 KB chunks per tensor: 32 MiB of K and 32 MiB of V per launch

// Every wave reads ROUNDS x NLOAD 1 KB chunks of each tensor, the NLOAD loads of a round issued before the first use.
// ILV: a wave's chunks are 4 KB pieces dealt round robin over all waves of the launch (the decode kernel's row order);
// else one contiguous run per wave.  NT: non-temporal loads.
// STAGE: 0 = values only xor-ed; 1 = K and V staged through a wave-private LDS region with the decode kernel's row
// strides and read back once (8 + 8 128-bit reads a lane); 2 = the decode kernel's full LDS read volume (24 + 16);
// STORE: every wave also writes 2 KB (4 MiB a launch: the split partials).
template <int WAVES, int NLOAD, int ROUNDS, bool NT, bool ILV, int MINB, int STAGE, bool STORE>
__global__ __launch_bounds__(WAVES * 64, MINB) void pa_probe_read_kernel(const unsigned char* K, const unsigned char* V, unsigned char* sink) {
  static_assert((NLOAD * ROUNDS) % 4 == 0, "whole 4 KB pieces");
  static_assert(STAGE == 0 || (NLOAD == 16 && ROUNDS == 1), "staging: one 32-row tile of 512-byte rows per wave");
  extern __shared__ __attribute__((aligned(16))) unsigned char probe_lds[];
  const uint32_t lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const uint32_t g = blockIdx.x * WAVES + w, nw = gridDim.x * WAVES;
  uint32_t s = 0;
#pragma unroll 1
  for (int r = 0; r < ROUNDS; r++) {
    u4 a[NLOAD], b[NLOAD];
#pragma unroll
    for (int j = 0; j < NLOAD; j++) {
      const uint32_t c = r * NLOAD + j;
      const size_t chunk = ILV ? (size_t)(c / 4) * nw * 4 + (size_t)g * 4 + (c & 3) : (size_t)g * (ROUNDS * NLOAD) + c;
      const u4* pk = (const u4*)(K + chunk * 1024 + lane * 16);
      const u4* pv = (const u4*)(V + chunk * 1024 + lane * 16);
      if (NT) { a[j] = __builtin_nontemporal_load(pk); b[j] = __builtin_nontemporal_load(pv); }
      else { a[j] = *pk; b[j] = *pv; }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (STAGE == 0) {
#pragma unroll
      for (int j = 0; j < NLOAD; j++) s ^= a[j].x ^ a[j].y ^ a[j].z ^ a[j].w ^ b[j].x ^ b[j].y ^ b[j].z ^ b[j].w;
    } else {
      unsigned char* st = probe_lds + w * 17408;
      constexpr int KRD = STAGE == 2 ? 24 : 8, VRD = STAGE == 2 ? 16 : 8;
#pragma unroll
      for (int j = 0; j < 16; j++) *(u4*)(st + (2 * j + (lane >> 5)) * 528 + (lane & 31) * 16) = a[j];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < KRD; j++) { const u4 t = *(const u4*)(st + (lane & 31) * 528 + (j & 7) * 64 + (lane >> 5) * 16 + ((j >> 3) & 1) * 32); s ^= t.x ^ t.y ^ t.z ^ t.w; }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < 16; j++) *(u4*)(st + (2 * j + (lane >> 5)) * 544 + (lane & 31) * 16) = b[j];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < VRD; j++) { const u4 t = *(const u4*)(st + (lane & 31) * 544 + (j & 7) * 64 + (lane >> 5) * 16 + ((j >> 3) & 1) * 32); s ^= t.x ^ t.y ^ t.z ^ t.w; }
      __syncthreads();
    }
  }
  if constexpr (STORE) {
    unsigned char* d = sink + 4096 + (size_t)g * 2048 + lane * 16;
    *(u4*)d = (u4){s, s, s, s};
    *(u4*)(d + 1024) = (u4){s, s, s, s};
  } else if (s == 0x12345678u) {
    *(uint32_t*)(sink + (size_t)(g & 15) * 256 + lane * 4) = s;       // keeps the loads alive; practically never taken
  }
}

__global__ __launch_bounds__(256, 2) void pa_probe_empty_kernel(unsigned char* sink) {
  if (sink == (unsigned char*)1) sink[0] = 0;
}

struct ProbeVariant {
  const char* name;
  void (*kern)(const unsigned char*, const unsigned char*, unsigned char*);
  uint32_t grid, block, lds;
};

static const ProbeVariant g_variants[] = {
  {"empty kernel, 512 workgroups x 256 threads", nullptr, 512, 256, 0},
  {"read: 512 wg x 4 waves x (16+16) loads, 4 KB pieces chip-wide [the decode kernel's shape]", pa_probe_read_kernel<4, 16, 1, false, true, 2, 0, false>, 512, 256, 0},
  {"read: same shape, non-temporal loads", pa_probe_read_kernel<4, 16, 1, true, true, 2, 0, false>, 512, 256, 0},
  {"read: same shape, one contiguous 16 KB run per wave", pa_probe_read_kernel<4, 16, 1, false, false, 2, 0, false>, 512, 256, 0},
  {"read: 256 wg x 8 waves x (16+16) loads, 4 KB pieces", pa_probe_read_kernel<8, 16, 1, false, true, 1, 0, false>, 256, 512, 0},
  {"read: 1024 wg x 4 waves x (8+8) loads, 4 KB pieces", pa_probe_read_kernel<4, 8, 1, false, true, 4, 0, false>, 1024, 256, 0},
  {"read: 2048 wg x 4 waves x (4+4) loads, 4 KB pieces", pa_probe_read_kernel<4, 4, 1, false, true, 8, 0, false>, 2048, 256, 0},
  {"read: 256 wg x 4 waves x (32+32) loads up front, 4 KB pieces [two tiles a wave]", pa_probe_read_kernel<4, 32, 1, false, true, 1, 0, false>, 256, 256, 0},
  {"read: 256 wg x 4 waves x 2 rounds of (16+16) loads, 4 KB pieces", pa_probe_read_kernel<4, 16, 2, false, true, 1, 0, false>, 256, 256, 0},
  {"read + tiles staged through LDS, read back once", pa_probe_read_kernel<4, 16, 1, false, true, 2, 1, false>, 512, 256, 4 * 17408},
  {"read + staged + 4 MiB of partial stores", pa_probe_read_kernel<4, 16, 1, false, true, 2, 1, true>, 512, 256, 4 * 17408},
  {"read + staged with the decode kernel's LDS read volume + 4 MiB of stores", pa_probe_read_kernel<4, 16, 1, false, true, 2, 2, true>, 512, 256, 4 * 17408},
  {"read (non-temporal) + staged with the decode kernel's LDS read volume + 4 MiB of stores", pa_probe_read_kernel<4, 16, 1, true, true, 2, 2, true>, 512, 256, 4 * 17408},
};
static constexpr int N_VARIANTS = (int)(sizeof(g_variants) / sizeof(g_variants[0]));

extern "C" int pa_probe_count(void) { return N_VARIANTS; }
extern "C" const char* pa_probe_name(int variant) { return variant >= 0 && variant < N_VARIANTS ? g_variants[variant].name : nullptr; }

// One launch of a stand-in on the context's stream over 32 MiB at d_k and 32 MiB at d_v (d_sink: 8 MiB of scratch).
// With pa_profile_enable on, the launch is timed like an attention call's main kernel (pa_profile_read_each).
extern "C" int pa_probe_stream(pa_ctx* ctx, int variant, const void* d_k, const void* d_v, void* d_sink) {
  if (!ctx || variant < 0 || variant >= N_VARIANTS || !d_k || !d_v || !d_sink) return PA_ERR_INVALID;
  const ProbeVariant& v = g_variants[variant];
  PaTiming tm;
  if (ctx->profiling) {
    if (ctx->prof_used + 2 > ctx->prof_events.size()) {
      for (int i = 0; i < 2; i++) { hipEvent_t ev; if (hipEventCreate(&ev) != hipSuccess) return PA_ERR_HIP; ctx->prof_events.push_back(ev); }
    }
    tm.start = ctx->prof_events[ctx->prof_used]; tm.stop = ctx->prof_events[ctx->prof_used + 1];
    ctx->prof_used += 2;
  }
  if (!v.kern) {
    PA_LAUNCH(pa_probe_empty_kernel, dim3(v.grid), dim3(v.block), 0, ctx->stream, &tm, (unsigned char*)d_sink);
  } else {
    if (v.lds > 48 * 1024 && hipFuncSetAttribute((const void*)v.kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)v.lds) != hipSuccess) return PA_ERR_HIP;
    // the launch covers PROBE_CHUNKS chunks per tensor: grid x waves x loads x rounds is fixed by the table above
    PA_LAUNCH(v.kern, dim3(v.grid), dim3(v.block), v.lds, ctx->stream, &tm, (const unsigned char*)d_k, (const unsigned char*)d_v, (unsigned char*)d_sink);
  }
  return hipGetLastError() == hipSuccess ? PA_OK : PA_ERR_HIP;
}
