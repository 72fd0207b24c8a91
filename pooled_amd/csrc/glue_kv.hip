// Pre-step kernel: q de-interleave + per-head RMSNorm + NeoX RoPE (+ f16 KV-cache write) for gfx950.
//
// One 64-lane wavefront per (head, column); heads [0, nH) are query heads, [nH, nH + nKV) are key heads,
// and a key head's workgroup also packs the matching value head.  This is the launch shape of the
// reference's fused glue kernels (engine/wgsl/qwen35.js:1082-1136 attn_glue, engine/wgsl/layer_fuse.js:87-146
// attn_glue_kv, engine/wgsl/dense.js:144-196 attn_glue_d), which it replaces.
//
// Arithmetic (chosen so a CPU restatement can reproduce the bits):
//   ss   = sum v_i^2 in f64 (exact products), inv = f32(1 / sqrt(ss / hd + eps)) evaluated in f64
//   v_i  = v_i * (inv * w_i)                 two f32 multiplies (engine/wgsl/base.js:65-79)
//   ang  = f32(pos) * inv_freq[i]            f32 product; inv_freq is a host-built f32 table of
//                                            theta^(-2i/n_rot) (engine/wgsl/qwen35.js:397)
//   c, s = f32(cos(f64(ang))), f32(sin(f64(ang)))
//   a'   = a*c - b*s,  b' = b*c + a*s        separately rounded f32 products and sums (no FMA)
//   cache element = f16 round-to-nearest-even of the f32 value (engine/wgsl/qwen35.js:889-906)
#include "pa_internal.h"
#include <hip/hip_fp16.h>

// every product and sum below is rounded on its own: no fused multiply-add may be formed in this file
// (plain operators are used instead of the __fmul_rn family, whose header bodies are compiled with contraction on)
#pragma clang fp contract(off)

#define GLUE_DO_MATH 0x100u

static __device__ inline double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

static __device__ inline uint32_t pack_f16x2(float lo, float hi) {
  return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
}

// c, s of the f32 angle f32(pos) * inv_freq, evaluated in f64 and rounded once
static __device__ inline void rope_cos_sin(uint32_t pos, float inv_freq, float& c, float& s) {
  const float ang = (float)pos * inv_freq;
  double sd, cd;
  sincos((double)ang, &sd, &cd);
  c = (float)cd; s = (float)sd;
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
  __shared__ float xs[256];
  const uint32_t hh = blockIdx.x, col = blockIdx.y, lane = threadIdx.x;
  const uint32_t nH = p.n_heads, hd = p.head_dim;
  const bool isQ = hh < nH;
  const uint32_t h = isQ ? hh : hh - nH;
  const bool gated = (p.flags & PA_FLAG_GATE) != 0;
  const bool math = (p.flags & GLUE_DO_MATH) != 0;
  const uint32_t pos = p.base_pos + col;
  const uint32_t qDim = nH * hd, kvDim = p.n_kv_heads * hd;
  const float* src = isQ ? p.q_in + (size_t)col * p.q_stride + (size_t)h * (gated ? 2 * hd : hd)
                         : p.k_in + (size_t)col * p.k_stride + (size_t)h * hd;
  float x[4];
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint32_t i = lane + 64 * j;
    x[j] = 0.f;
    if (i < hd) {
      x[j] = src[i];
      ss += (double)x[j] * (double)x[j];
      if (isQ && gated) p.gate_out[(size_t)col * qDim + h * hd + i] = src[hd + i];
    }
  }
  if (math && (p.flags & PA_FLAG_QK_NORM)) {
    ss = wave_sum_f64(ss);
    const float inv = (float)(1.0 / sqrt(ss / (double)hd + (double)p.eps));
    const float* w = isQ ? p.qw : p.kw;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t i = lane + 64 * j;
      if (i < hd) { const float sw = inv * w[i]; x[j] = x[j] * sw; }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; j++) { const uint32_t i = lane + 64 * j; if (i < hd) xs[i] = x[j]; }
  __syncthreads();
  if (math) {
    const uint32_t half = p.n_rot / 2;
    float ra[2], rb[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t i = lane + 64 * j;
      if (i < half) {
        float c, s;
        if (p.rope_tab) { const float2 cs = p.rope_tab[(size_t)pos * half + i]; c = cs.x; s = cs.y; }
        else rope_cos_sin(pos, p.inv_freq[i], c, s);
        const float a = xs[i], b = xs[i + half];
        const float ac = a * c, bs = b * s, bc = b * c, as = a * s;   // rounded one by one (contract off above)
        ra[j] = ac - bs;
        rb[j] = bc + as;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t i = lane + 64 * j;
      if (i < half) { xs[i] = ra[j]; xs[i + half] = rb[j]; }
    }
    __syncthreads();
  }
  if (isQ) {
    for (uint32_t i = lane; i < hd; i += 64) p.q_out[(size_t)col * qDim + h * hd + i] = xs[i];
    return;
  }
  if (p.k_out) for (uint32_t i = lane; i < hd; i += 64) p.k_out[(size_t)col * p.k_stride + h * hd + i] = xs[i];
  if (p.k_cache) {
    uint32_t* kc = (uint32_t*)(p.k_cache + (size_t)pos * kvDim + h * hd);
    uint32_t* vc = (uint32_t*)(p.v_cache + (size_t)pos * kvDim + h * hd);
    const float* vs = p.v_in + (size_t)col * p.v_stride + (size_t)h * hd;
    for (uint32_t w = lane; w < hd / 2; w += 64) {
      kc[w] = pack_f16x2(xs[2 * w], xs[2 * w + 1]);
      vc[w] = pack_f16x2(vs[2 * w], vs[2 * w + 1]);
    }
  }
}

hipError_t pa_launch_glue(const GlueParams& p, hipStream_t s) {
  const uint32_t heads = p.n_heads + p.n_kv_heads;
  if (heads == 0 || p.n_cols == 0) return hipSuccess;
  hipLaunchKernelGGL(pa_glue_kernel, dim3(heads, p.n_cols), dim3(64), 0, s, p);
  return hipGetLastError();
}
