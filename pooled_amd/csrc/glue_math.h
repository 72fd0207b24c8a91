// Per-head arithmetic of the pre-step (RMSNorm + NeoX RoPE), shared by the stand-alone pre-step kernel and the
// fused decode-step kernel so that both produce the same bits.
//
// Arithmetic (chosen so a CPU restatement can reproduce the bits):
//   ss   = sum v_i^2 in f64 (exact products), inv = f32(1 / sqrt(ss / hd + eps)) evaluated in f64
//   v_i  = v_i * (inv * w_i)                 two f32 multiplies (engine/wgsl/base.js:65-79)
//   ang  = f32(pos) * inv_freq[i]            f32 product; inv_freq is a host-built f32 table of
//                                            theta^(-2i/n_rot) (engine/wgsl/qwen35.js:397)
//   c, s = f32(cos(f64(ang))), f32(sin(f64(ang)))
//   a'   = a*c - b*s,  b' = b*c + a*s        separately rounded f32 products and sums (no FMA)
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

// Compiler-level ordering of LDS accesses inside one wavefront (hardware executes a wave's LDS operations
// in order; lanes of one wave exchange data through a wave-private region without a workgroup barrier).
static __device__ inline void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

static __device__ inline double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// c, s of the f32 angle f32(pos) * inv_freq, evaluated in f64 and rounded once
static __device__ inline void rope_cos_sin(uint32_t pos, float inv_freq, float& c, float& s) {
  // every product below is rounded on its own (plain operators: the __fmul_rn family is compiled with contraction on)
#pragma clang fp contract(off)
  const float ang = (float)pos * inv_freq;
  double sd, cd;
  sincos((double)ang, &sd, &cd);
  c = (float)cd; s = (float)sd;
}

// (cos, sin) of rotation pair i at position pos: from the per-context table when there is one
static __device__ inline float2 rope_pair(const float2* rope_tab, const float* inv_freq, uint32_t pos, uint32_t half, uint32_t i) {
  if (rope_tab) return rope_tab[(size_t)pos * half + i];
  float c, s;
  rope_cos_sin(pos, inv_freq[i], c, s);
  return make_float2(c, s);
}

// One wavefront, one head of hd <= 256 values: x[j] is element lane + 64 j (0 past hd).  Optional RMSNorm with
// weights w[j] (of element lane + 64 j; norm == false: none), optional rotation of pairs (i, i + half), i < half,
// by cs[j] = (cos, sin) of pair lane + 64 j (half == 0: none).  xs is a wave-private LDS scratch of hd floats; on
// return xs[0, hd) holds the head and the wave's LDS accesses are fenced.
static __device__ inline void glue_head_wave(const float (&x_in)[4], const float (&w)[4], bool norm, float eps, uint32_t hd,
                                             uint32_t half, const float2 (&cs)[2], float* xs, uint32_t lane) {
#pragma clang fp contract(off)
  float x[4];
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < 4; j++) { x[j] = x_in[j]; ss += (double)x[j] * (double)x[j]; }
  if (norm) {
    ss = wave_sum_f64(ss);
    const float inv = (float)(1.0 / sqrt(ss / (double)hd + (double)eps));
#pragma unroll
    for (int j = 0; j < 4; j++) { const float sw = inv * w[j]; x[j] = x[j] * sw; }
  }
#pragma unroll
  for (int j = 0; j < 4; j++) { const uint32_t i = lane + 64 * j; if (i < hd) xs[i] = x[j]; }
  wave_lds_fence();
  if (half) {
    float ra[2], rb[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t i = lane + 64 * j;
      if (i < half) {
        const float c = cs[j].x, s = cs[j].y;
        const float a = xs[i], b = xs[i + half];
        const float ac = a * c, bs = b * s, bc = b * c, as = a * s;   // rounded one by one
        ra[j] = ac - bs;
        rb[j] = bc + as;
      }
    }
    wave_lds_fence();
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t i = lane + 64 * j;
      if (i < half) { xs[i] = ra[j]; xs[i + half] = rb[j]; }
    }
    wave_lds_fence();
  }
}
