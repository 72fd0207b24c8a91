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

// Sum over the 64 lanes, the same value in every lane, in a fixed order: quads, half rows and rows through DPP
// lane permutations (a lane adds its partner's value, so both partners end up with the same bits), then the four
// row sums as (r0 + r1) + (r2 + r3).  No LDS traffic: 8 moves + 4 adds + 8 lane reads, against 12 dependent
// ds_bpermute round trips for a shuffle butterfly.
template <int CTRL> static __device__ inline double dpp_f64(double v) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, 0xF, 0xF, false);
  hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, 0xF, 0xF, false);
  return __hiloint2double(hi, lo);
}
static __device__ inline double readlane_f64(double v, int l) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), l), __builtin_amdgcn_readlane(__double2loint(v), l));
}
static __device__ inline double wave_sum_f64(double v) {
  v += dpp_f64<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  v += dpp_f64<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  v += dpp_f64<0x141>(v);     // row_half_mirror: lane i <-> 7 - i of each 8
  v += dpp_f64<0x140>(v);     // row_mirror: lane i <-> 15 - i of each 16
  return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}

// the same for a float
template <int CTRL> static __device__ inline float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
static __device__ inline float readlane_f32(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
static __device__ inline float wave_sum_f32(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  return (readlane_f32(v, 0) + readlane_f32(v, 16)) + (readlane_f32(v, 32) + readlane_f32(v, 48));
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

// f32(1 / sqrt(ss / hd + eps)): the RMSNorm factor of a head from its f64 sum of squares.  The f64 value is good to a few
// units of its last place -- ss / hd by exponent arithmetic where hd is a power of two (exact), the reciprocal root from the
// hardware estimate and three Newton steps -- and is rounded once to f32: the same f32 as a correctly rounded f64 division
// and root give, except where their result lies within ~2^-50 of an f32 rounding boundary.  The library-call form
// (division, root, division) is ~40 dependent f64 instructions on the critical path of every wave of the fused decode
// step; this is ~12.
static __device__ inline float rms_inv(double ss, uint32_t hd, float eps) {
  const double mean = (hd & (hd - 1)) == 0 ? ldexp(ss, -(31 - (int)__builtin_clz(hd))) : ss / (double)hd;
  const double x = mean + (double)eps;
  const double h = 0.5 * x;
  double r = __builtin_amdgcn_rsq(x);
#pragma unroll
  for (int it = 0; it < 3; it++) {
    const double e = __builtin_fma(-h * r, r, 0.5);     // 0.5 - (x / 2) r^2
    r = __builtin_fma(r, e, r);                          // r (1.5 - (x / 2) r^2)
  }
  return (float)r;
}

// (cos, sin) of rotation pair i at position pos: from the per-context table when there is one
static __device__ inline float2 rope_pair(const float2* rope_tab, const float* inv_freq, uint32_t pos, uint32_t half, uint32_t i) {
  if (__builtin_expect(rope_tab != nullptr, 1)) return rope_tab[(size_t)pos * half + i];
  float c, s;
  rope_cos_sin(pos, inv_freq[i], c, s);
  return make_float2(c, s);
}

// One wavefront, N heads of hd <= 256 values side by side (their dependent chains -- reduction, 1 / sqrt, the LDS
// exchanges -- overlap): x[n][j] is element lane + 64 j of head n (0 past hd).  Optional RMSNorm with weights w[j]
// (of element lane + 64 j, shared by the heads; norm == false: none), optional rotation of pairs (i, i + half),
// i < half, by cs[j] = (cos, sin) of pair lane + 64 j (half == 0: none).  xs[n] = xs0 + n * xs_stride is a wave-private LDS
// scratch of hd floats; on return xs[n][0, hd) holds head n and the wave's LDS accesses are fenced.
template <int N>
static __device__ inline void glue_heads_wave(const float (&x_in)[N][4], const float (&w)[4], bool norm, float eps, uint32_t hd,
                                              uint32_t half, const float2 (&cs)[2], float* xs0, uint32_t xs_stride, uint32_t lane) {
#pragma clang fp contract(off)
  float* xs[N];
#pragma unroll
  for (int n = 0; n < N; n++) xs[n] = xs0 + n * xs_stride;
  float x[N][4];
  double ss[N];
#pragma unroll
  for (int n = 0; n < N; n++) {
    ss[n] = 0.0;
#pragma unroll
    for (int j = 0; j < 4; j++) { x[n][j] = x_in[n][j]; ss[n] += (double)x[n][j] * (double)x[n][j]; }
  }
  if (norm) {
#pragma unroll
    for (int n = 0; n < N; n++) ss[n] = wave_sum_f64(ss[n]);
    float inv[N];
#pragma unroll
    for (int n = 0; n < N; n++) inv[n] = rms_inv(ss[n], hd, eps);
#pragma unroll
    for (int n = 0; n < N; n++)
#pragma unroll
      for (int j = 0; j < 4; j++) { const float sw = inv[n] * w[j]; x[n][j] = x[n][j] * sw; }
  }
#pragma unroll
  for (int n = 0; n < N; n++)
#pragma unroll
    for (int j = 0; j < 4; j++) { const uint32_t i = lane + 64 * j; if (i < hd) xs[n][i] = x[n][j]; }
  wave_lds_fence();
  if (half) {
    float ra[N][2], rb[N][2];
#pragma unroll
    for (int n = 0; n < N; n++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const uint32_t i = lane + 64 * j;
        if (i < half) {
          const float c = cs[j].x, s = cs[j].y;
          const float a = xs[n][i], b = xs[n][i + half];
          const float ac = a * c, bs = b * s, bc = b * c, as = a * s;   // rounded one by one
          ra[n][j] = ac - bs;
          rb[n][j] = bc + as;
        }
      }
    wave_lds_fence();
#pragma unroll
    for (int n = 0; n < N; n++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const uint32_t i = lane + 64 * j;
        if (i < half) { xs[n][i] = ra[n][j]; xs[n][i + half] = rb[n][j]; }
      }
    wave_lds_fence();
  }
}

// The same arithmetic without LDS for the pair distances that the lane + 64 j layout keeps inside a register file: half a
// multiple of 64 (partners are registers j and j + half / 64 of one lane) and half == 32 (partners are lanes l and l ^ 32 of
// register 0, exchanged by a lane-swap instruction; cs[0] must then hold the (cos, sin) of pair lane & 31 in every lane).
// On return x holds the normed and rotated head, element lane + 64 j in x[n][j].  Same operations on the same values as
// glue_heads_wave, so the same bits; four dependent LDS round trips shorter.
static __device__ inline bool glue_regs_serves(uint32_t half) { return half == 0 || half == 32 || (half & 63) == 0; }
template <int N>
static __device__ inline void glue_heads_regs(float (&x)[N][4], const float (&w)[4], bool norm, float eps, uint32_t hd,
                                              uint32_t half, const float2 (&cs)[2], uint32_t lane) {
#pragma clang fp contract(off)
  if (norm) {
    double ss[N];
#pragma unroll
    for (int n = 0; n < N; n++) {
      ss[n] = 0.0;
#pragma unroll
      for (int j = 0; j < 4; j++) ss[n] += (double)x[n][j] * (double)x[n][j];
    }
#pragma unroll
    for (int n = 0; n < N; n++) ss[n] = wave_sum_f64(ss[n]);
#pragma unroll
    for (int n = 0; n < N; n++) {
      const float inv = rms_inv(ss[n], hd, eps);
#pragma unroll
      for (int j = 0; j < 4; j++) { const float sw = inv * w[j]; x[n][j] = x[n][j] * sw; }
    }
  }
  if (half == 32) {
    const float c = cs[0].x, s = cs[0].y;
#pragma unroll
    for (int n = 0; n < N; n++) {
      const float own = x[n][0];
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(own), __float_as_uint(own), false, false);
      const float other = __uint_as_float(lane < 32 ? sw[1] : sw[0]);      // element i + 32 for lanes i < 32, element i - 32 above
      const float pc = own * c, ps = other * s;                               // rounded one by one
      x[n][0] = lane < 32 ? pc - ps : pc + ps;                                // a' = a c - b s ; b' = b c + a s
    }
  } else if (half) {
    const uint32_t step = half >> 6;              // 1 or 2 at hd <= 256
#pragma unroll
    for (int n = 0; n < N; n++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        if ((uint32_t)j < step) {
          const float c = cs[j].x, s = cs[j].y;
          const float a = x[n][j], b = step == 1 ? x[n][j + 1] : x[n][j + 2];
          const float ac = a * c, bs = b * s, bc = b * c, as = a * s;
          x[n][j] = ac - bs;
          if (step == 1) x[n][j + 1] = bc + as; else x[n][j + 2] = bc + as;
        }
      }
  }
}

// one head
static __device__ inline void glue_head_wave(const float (&x_in)[4], const float (&w)[4], bool norm, float eps, uint32_t hd,
                                             uint32_t half, const float2 (&cs)[2], float* xs, uint32_t lane) {
  const float x1[1][4] = { { x_in[0], x_in[1], x_in[2], x_in[3] } };
  glue_heads_wave<1>(x1, w, norm, eps, hd, half, cs, xs, 0, lane);
}

// int8 cache row, the lane's 4 consecutive values of a 32-value block (8 lanes = one block; the reference's
// kv_store_q8, engine/wgsl/qwen35.js:908-946): scale = max|x| / 127 over the block, inv = 1 / scale (0 for an all-zero
// block), value = clamp(round-half-even(x * inv), -127, 127), every operation a separately rounded f32 one.  Returns
// the 4 values packed low byte first and the block's scale (the same in its 8 lanes).  All 64 lanes must call.
static __device__ inline void quant4_q8(const float (&x)[4], uint32_t& w, float& sc) {
#pragma clang fp contract(off)
  float a = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
  a = fmaxf(a, __shfl_xor(a, 1, 64)); a = fmaxf(a, __shfl_xor(a, 2, 64)); a = fmaxf(a, __shfl_xor(a, 4, 64));
  sc = a / 127.0f;
  const float inv = sc > 0.f ? 1.0f / sc : 0.f;
  w = 0;
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const float r = fminf(fmaxf(__builtin_rintf(x[b] * inv), -127.0f), 127.0f);
    w |= ((uint32_t)(int)r & 255u) << (8 * b);
  }
}
