// Pre-step kernel: q de-interleave + per-head RMSNorm + NeoX RoPE (+ f16 KV-cache write) for gfx950.
//
// One 64-lane wavefront per (head, column); heads [0, nH) are query heads, [nH, nH + nKV) are key heads,
// and a key head's workgroup also packs the matching value head.  This is the launch shape of the
// reference's fused glue kernels (engine/wgsl/qwen35.js:1082-1136 attn_glue, engine/wgsl/layer_fuse.js:87-146
// attn_glue_kv, engine/wgsl/dense.js:144-196 attn_glue_d), which it replaces.
//
// The per-head arithmetic lives in glue_math.h (shared with the fused decode-step kernel); cache elements are the
// f16 round-to-nearest-even of the f32 values (engine/wgsl/qwen35.js:889-906).
#include "pa_internal.h"
#include "glue_math.h"

#define GLUE_DO_MATH 0x100u

// int8 cache row (the reference's kv_store_q8, engine/wgsl/qwen35.js:908-946): per block of 32 values
// the arithmetic is quant4_q8 (glue_math.h).  One wavefront, 4 consecutive values a lane (8 lanes = one block);
// src holds the row's hd f32 values (LDS or global), dst the row's hd int8, sc_dst its hd / 32 scales.
static __device__ inline void store_row_q8(const float* src, uint32_t hd, uint32_t lane, unsigned char* dst, float* sc_dst) {
  const bool on = 4 * lane < hd;
  float x[4] = {0.f, 0.f, 0.f, 0.f};
  if (on) { x[0] = src[4 * lane]; x[1] = src[4 * lane + 1]; x[2] = src[4 * lane + 2]; x[3] = src[4 * lane + 3]; }
  uint32_t w; float sc;
  quant4_q8(x, w, sc);
  if (on) {
    *(uint32_t*)(dst + 4 * lane) = w;
    if ((lane & 7) == 0) sc_dst[lane >> 3] = sc;
  }
}

static __device__ inline uint32_t pack_f16x2(float lo, float hi) {
  return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
}

// The same values for every (position, pair), computed once per context: rope_tab[pos * half + i] = (cos, sin).
__global__ __launch_bounds__(256) void pa_rope_table_kernel(float2* tab, const float* inv_freq, uint32_t half, uint32_t n_pos) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= (size_t)n_pos * half) return;
  float c, s;
  rope_cos_sin((uint32_t)(e / half), inv_freq[e % half], c, s);
  tab[e] = make_float2(c, s);
}

hipError_t pa_launch_rope_table(float2* tab, const float* inv_freq, uint32_t half, uint32_t n_pos, hipStream_t st) {
  const size_t n = (size_t)n_pos * half;
  hipLaunchKernelGGL(pa_rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, tab, inv_freq, half, n_pos);
  return hipGetLastError();
}

__global__ __launch_bounds__(64) void pa_glue_kernel(GlueParams p) {
  // (every kernel argument in the first batch of scalar loads instead of a dependent round trip at each first use)
  asm volatile("" :: "s"(p.q_in), "s"(p.k_in), "s"(p.v_in), "s"(p.k_out), "s"(p.qw), "s"(p.kw), "s"(p.inv_freq), "s"(p.rope_tab), "s"(p.q_out),
               "s"(p.gate_out), "s"(p.k_cache), "s"(p.v_cache), "s"(p.ks_cache), "s"(p.vs_cache), "s"(p.head_rows), "s"(p.q_stride), "s"(p.k_stride),
               "s"(p.v_stride), "s"(p.n_heads), "s"(p.n_kv_heads), "s"(p.head_dim), "s"(p.n_rot), "s"(p.base_pos), "s"(p.n_cols), "s"(p.flags), "s"(p.eps));
  __shared__ float xs[256];
  const uint32_t hh = blockIdx.x, col = blockIdx.y, lane = threadIdx.x;
  const uint32_t nH = p.n_heads, hd = p.head_dim;
  const bool isQ = hh < nH;
  const uint32_t h = isQ ? hh : hh - nH;
  const bool gated = (p.flags & PA_FLAG_GATE) != 0;
  const bool math = (p.flags & GLUE_DO_MATH) != 0;
  const uint32_t pos = p.base_pos + col;
  const uint32_t qDim = nH * hd;
  const float* src = isQ ? p.q_in + (size_t)col * p.q_stride + (size_t)h * (gated ? 2 * hd : hd)
                         : p.k_in + (size_t)col * p.k_stride + (size_t)h * hd;
  // Everything the wave reads is requested before anything is stored or computed -- the head's values, the gate half
  // of a gated query head, the value row of a key head, the rotation's (cos, sin), the norm weights -- and every load
  // is unconditional: an element past head_dim re-reads the last one and is zeroed afterwards.  (A load and a
  // dependent store per element, or a register preset to zero and loaded under a branch, is one round trip each:
  // the kernel was seven of them.)
  float x[4], gt[4] = {0.f, 0.f, 0.f, 0.f}, w[4] = {0.f, 0.f, 0.f, 0.f};
  float2 vv[2] = { make_float2(0.f, 0.f), make_float2(0.f, 0.f) };
  float2 cs[2] = { make_float2(1.f, 0.f), make_float2(1.f, 0.f) };
  const bool gate_copy = isQ && gated;
  const bool v_copy = !isQ && p.k_cache && !p.ks_cache;
  const uint32_t half = math ? p.n_rot / 2 : 0;
  const bool norm = math && (p.flags & PA_FLAG_QK_NORM);
#pragma unroll
  for (int j = 0; j < 4; j++) x[j] = src[min(lane + 64 * j, hd - 1)];
  if (gate_copy) {
#pragma unroll
    for (int j = 0; j < 4; j++) gt[j] = src[hd + min(lane + 64 * j, hd - 1)];
  }
  if (v_copy) {
    const float2* vs2 = (const float2*)(p.v_in + (size_t)col * p.v_stride + (size_t)h * hd);
#pragma unroll
    for (int t = 0; t < 2; t++) vv[t] = vs2[min(lane + 64 * t, hd / 2 - 1)];
  }
  if (half) {
#pragma unroll
    for (int j = 0; j < 2; j++) cs[j] = rope_pair(p.rope_tab, p.inv_freq, pos, half, min(lane + 64 * j, half - 1));
  }
  if (norm) {
    const float* wp = isQ ? p.qw : p.kw;
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = wp[min(lane + 64 * j, hd - 1)];
  }
#pragma unroll
  for (int j = 0; j < 4; j++) if (lane + 64 * j >= hd) { x[j] = 0.f; w[j] = 0.f; }
  if (gate_copy) {
#pragma unroll
    for (int j = 0; j < 4; j++) if (lane + 64 * j < hd) p.gate_out[(size_t)col * qDim + h * hd + lane + 64 * j] = gt[j];
  }
  glue_head_wave(x, w, norm, p.eps, hd, half, cs, xs, lane);
  if (isQ) {
    for (uint32_t i = lane; i < hd; i += 64) p.q_out[(size_t)col * qDim + h * hd + i] = xs[i];
    return;
  }
  if (p.k_out) for (uint32_t i = lane; i < hd; i += 64) p.k_out[(size_t)col * p.k_stride + h * hd + i] = xs[i];
  if (p.k_cache && p.ks_cache) {                                     // int8 caches
    const size_t row = (size_t)h * p.head_rows + pos;
    store_row_q8(xs, hd, lane, (unsigned char*)p.k_cache + row * hd, p.ks_cache + row * (hd / 32));
    store_row_q8(p.v_in + (size_t)col * p.v_stride + (size_t)h * hd, hd, lane, (unsigned char*)p.v_cache + row * hd, p.vs_cache + row * (hd / 32));
  } else if (p.k_cache) {
    const size_t ro = ((size_t)h * p.head_rows + pos) * hd;           // head-major caches
    uint32_t* kc = (uint32_t*)(p.k_cache + ro);
    uint32_t* vc = (uint32_t*)(p.v_cache + ro);
    // (the empty statement pins the conversion of the value row here: hoisted to its load, it would make the wave wait for
    // that load before the rotation's and the norm's loads have gone out)
#pragma unroll
    for (int t = 0; t < 2; t++) asm volatile("" : "+v"(vv[t].x), "+v"(vv[t].y));
#pragma unroll
    for (int t = 0; t < 2; t++)
      if (lane + 64 * t < hd / 2) {
        const uint32_t w = lane + 64 * t;
        kc[w] = pack_f16x2(xs[2 * w], xs[2 * w + 1]);
        vc[w] = pack_f16x2(vv[t].x, vv[t].y);
      }
  }
}

hipError_t pa_launch_glue(const GlueParams& p, hipStream_t s) {
  const uint32_t heads = p.n_heads + p.n_kv_heads;
  if (heads == 0 || p.n_cols == 0) return hipSuccess;
  hipLaunchKernelGGL(pa_glue_kernel, dim3(heads, p.n_cols), dim3(64), 0, s, p);
  return hipGetLastError();
}

// int8 caches -> an f16 staging cache of the same head-major geometry, rows [0, n_rows) of every kv head; rows from
// n_live up to n_rows are written as zeros (their scales need not be numbers).  A value is widened as the split-K
// kernel widens it: exact integer times the f16-rounded scale, rounded once.  One thread = 16 values.
__global__ __launch_bounds__(256) void pa_widen_q8_kernel(const unsigned char* k8, const unsigned char* v8, const float* ks, const float* vs,
                                                          uint16_t* ko, uint16_t* vo, uint32_t hd, uint32_t head_rows, uint32_t n_live,
                                                          uint32_t n_rows) {
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  const uint32_t ppr = hd / 16;                                       // pieces per row
  const uint32_t idx = blockIdx.x * 256 + threadIdx.x, row = idx / ppr, pc = idx % ppr, h = blockIdx.y;
  if (row >= n_rows) return;
  const bool isV = blockIdx.z != 0;
  const size_t r = (size_t)h * head_rows + row;
  uint16_t* dst = (isV ? vo : ko) + r * hd + pc * 16;
  h8 lo = {0, 0, 0, 0, 0, 0, 0, 0}, hi = lo;
  if (row < n_live) {
    const uint4 q = *(const uint4*)((isV ? v8 : k8) + r * hd + pc * 16);
    const _Float16 sc = (_Float16)(isV ? vs : ks)[r * (hd / 32) + pc / 2];
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      lo[i] = (_Float16)(int)(signed char)(w[i / 4] >> (8 * (i & 3))) * sc;
      hi[i] = (_Float16)(int)(signed char)(w[2 + i / 4] >> (8 * (i & 3))) * sc;
    }
  }
  *(h8*)dst = lo;
  *(h8*)(dst + 8) = hi;
}

hipError_t pa_launch_widen_q8(const void* k8, const void* v8, const float* ks, const float* vs, uint16_t* ko, uint16_t* vo,
                              uint32_t n_kv_heads, uint32_t hd, uint32_t head_rows, uint32_t n_live, uint32_t n_rows, hipStream_t s) {
  if (n_rows == 0) return hipSuccess;
  if (hd % 32 || n_rows > head_rows || n_live > n_rows) return hipErrorInvalidValue;
  const uint32_t threads = n_rows * (hd / 16);
  hipLaunchKernelGGL(pa_widen_q8_kernel, dim3((threads + 255) / 256, n_kv_heads, 2), dim3(256), 0, s, (const unsigned char*)k8,
                     (const unsigned char*)v8, ks, vs, ko, vo, hd, head_rows, n_live, n_rows);
  return hipGetLastError();
}
