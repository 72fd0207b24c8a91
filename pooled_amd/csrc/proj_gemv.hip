// One-token projections either side of the attention block on gfx950: y = W x for f32, Q8_0 and Q4_0 weights,
// optionally over rmsnorm(x) computed in the kernel, optionally accumulated into y.
//
// Replaces the reference's matvec / matvec_q8 / matvec_q4 and their cooperative forms (engine/wgsl/base.js:15-118,
// engine/wgsl/coop.js:236-345), the accumulate variants (_coop_acc, coop.js:347-349: y[row] += W x, the residual add
// folded in) and the normed variants (_coop_n, coop.js:371-420: rmsnorm of the raw residual inside the GEMV).
// Weight formats are the reference's split planes:
//   Q8_0: int8 [d_out][d_in] + one f16 scale per 32 values; y_r = sum_b sc_rb * sum_j q_rbj * x_bj
//   Q4_0: nibbles [d_out][d_in / 2], byte j of a 16-byte block = element j (low nibble) and j + 16 (high nibble),
//         value = nibble - 8; same scales.
//
// A one-token GEMV reads every weight once and the 8-32 KB activation many times: it is HBM- and latency-bound,
// not arithmetic.  Shape here: a 64-lane wavefront owns RW output rows; lane l owns the 32-value blocks l, l + 64,
// ... of the input (one Q4_0 block = one 16-byte load, so a wave-wide load is 1 KB of one row, fully coalesced),
// keeps its slices of x in registers for all its rows (x reaches them through LDS, loaded coalesced once per
// workgroup), issues every weight and scale load of its rows before the first use, and sums the 64 lanes with DPP
// permutations.  All arithmetic is f32 as in the reference; the order of
// the additions differs from the reference's workgroup tree (the parity tests use a tolerance, as the reference's do).
#include "pa_internal.h"
#include "glue_math.h"

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));

// 32 weights of one block times the lane's 32 activations, scale not applied
template <int KIND> struct BlockRegs;
template <> struct BlockRegs<PA_W_F32> { f4 w[8]; };
template <> struct BlockRegs<PA_W_Q8_0> { u4 w[2]; };
template <> struct BlockRegs<PA_W_Q4_0> { u4 w[1]; };

template <int KIND>
static __device__ inline void load_block(BlockRegs<KIND>& r, const unsigned char* base, size_t row, uint32_t nb, uint32_t b) {
  if constexpr (KIND == PA_W_F32) {
    const f4* s = (const f4*)(base + ((size_t)row * nb + b) * 128);
#pragma unroll
    for (int i = 0; i < 8; i++) r.w[i] = s[i];
  } else if constexpr (KIND == PA_W_Q8_0) {
    const u4* s = (const u4*)(base + ((size_t)row * nb + b) * 32);
    r.w[0] = s[0]; r.w[1] = s[1];
  } else {
    r.w[0] = *(const u4*)(base + ((size_t)row * nb + b) * 16);
  }
}

template <int KIND>
static __device__ inline float dot_block(const BlockRegs<KIND>& r, const float (&x)[32], float sx) {
  float a = 0.f;
  if constexpr (KIND == PA_W_F32) {
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) a = __builtin_fmaf(r.w[i][j], x[4 * i + j], a);
    return a;
  } else if constexpr (KIND == PA_W_Q8_0) {
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int word = (int)r.w[i][k];
#pragma unroll
        for (int j = 0; j < 4; j++) a = __builtin_fmaf((float)((word << (24 - 8 * j)) >> 24), x[16 * i + 4 * k + j], a);
      }
    return a;
  } else {
    // sum (n - 8) x = sum n x - 8 sum x.  A nibble n in the low bits of a 16-bit half IS the f16 subnormal n x 2^-24, and
    // the mixed-precision fma takes an f16 operand as it is: two nibbles of a word are isolated by one shift and one mask
    // (15 instructions for 8 weights instead of 23 with byte-to-float conversions), the products are the same bits scaled
    // by a power of two, and the sum is scaled back once.
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t word = r.w[0][k];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const uint32_t pr = (word >> (4 * t)) & 0x000F000Fu;          // nibble t of the word (low half) and nibble t + 4 (high half)
        h2v v; __builtin_memcpy(&v, &pr, 4);
        const int e = 4 * k + (t >> 1) + 16 * (t & 1);                 // nibble 2 j of a word is element j of its four bytes, nibble 2 j + 1 element j + 16
        a = __builtin_fmaf((float)v[0], x[e], a);
        a = __builtin_fmaf((float)v[1], x[e + 2], a);
      }
    }
    a *= 16777216.0f;
    return a - 8.0f * sx;
  }
}

// BPL: blocks per lane and pass; PASSES: passes over the input (d_in <= 2048 * BPL * PASSES; two for f32 weights past
// 4096 inputs, whose 32 registers a block leave no room for four blocks a lane: the second pass's weight rows are
// requested when the first pass's are consumed); RW: rows per wave
template <int KIND, int BPL, int RW, bool NORM, int PASSES = 1>
__global__ __launch_bounds__(256)
void pa_gemv_kernel(const float* a_x, const float* a_norm_w, const void* a_w, const uint16_t* a_scales, float* a_y, uint32_t a_d_out, uint32_t a_d_in, GemvParams p_in) {
  // The leading arguments repeat fields of p_in: the first twelve dwords of the arguments are preloaded into scalar
  // registers, so every load address of the kernel is there when the wave starts; the other arguments are fetched in one
  // batch of scalar loads (the compiler would fetch each where it is first used, a dependent round trip each).
  GemvParams p = p_in;
  p.x = a_x; p.norm_w = a_norm_w; p.w = a_w; p.scales = a_scales; p.y = a_y; p.d_out = a_d_out; p.d_in = a_d_in;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t nb = p.d_in / 32;
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * RW;
  const unsigned char* wbase = (const unsigned char*)p.w;
  // x (and the norm weights) are requested FIRST, the wave's weight rows right behind them: the loads of a wave complete
  // in order, x comes from L2 in a fraction of the time the weight stream takes from HBM, and everything that depends
  // on x alone -- the sum of squares, two barriers, the trip through LDS -- then runs under the latency of the weights
  // instead of after it.
  extern __shared__ __attribute__((aligned(16))) float xs[];
  __shared__ float red[4];
  constexpr int XPT = 2 * BPL * PASSES;                                // float4 of x per thread (d_in <= 2048 * BPL * PASSES)
  const uint32_t n4 = p.d_in / 4;
  f4 xv[XPT], wv[NORM ? XPT : 1];
  float ss = 0.f;
  // Loads past the end of x re-read its last float4 instead of being guarded (their values are never stored, and are
  // masked out of the sum of squares by a factor, not by a select on the loaded value): a guarded load is a branch,
  // and between guarded blocks the compiler placed a full wait.
#pragma unroll
  for (int k = 0; k < XPT; k++) xv[k] = ((const f4*)p.x)[min(threadIdx.x + 256 * k, n4 - 1)];
  if constexpr (NORM) {
#pragma unroll
    for (int k = 0; k < XPT; k++) wv[k] = ((const f4*)p.norm_w)[min(threadIdx.x + 256 * k, n4 - 1)];
  }
  __builtin_amdgcn_sched_barrier(0);
  BlockRegs<KIND> wr[RW][BPL];
  uint16_t sc[RW][BPL];
#pragma unroll
  for (int r = 0; r < RW; r++) {
    const size_t row = min(row0 + r, (size_t)p.d_out - 1);            // rows past the end repeat the last one (not stored)
#pragma unroll
    for (int i = 0; i < BPL; i++) {
      const uint32_t b = min(lane + 64 * i, nb - 1);                   // blocks past the end likewise (weighted by x = 0)
      load_block<KIND>(wr[r][i], wbase, row, nb, b);
      if constexpr (KIND != PA_W_F32) sc[r][i] = p.scales[row * nb + b];
    }
  }
  // accumulating calls: the old values of the wave's rows are requested here, with everything else, instead of in a
  // round trip of their own behind the reduction
  asm volatile("" :: "s"(p.xn_out), "s"(p.eps), "s"(p.acc));
  float yold[RW];
#pragma unroll
  for (int r = 0; r < RW; r++) yold[r] = p.acc ? p.y[min(row0 + r, (size_t)p.d_out - 1)] : 0.f;
  __builtin_amdgcn_sched_barrier(0);
  // x -> LDS (a lane's own slice is 32 consecutive floats: loaded directly, a wave-wide load would touch 64 cache lines
  // for 1 KB), normed on the way when asked; block b sits at xs[b * 36]: the 4-float pad makes the 8 lanes of a 128-bit
  // LDS read phase hit distinct banks
  if constexpr (NORM) {
#pragma unroll
    for (int k = 0; k < XPT; k++) {
      const float m = threadIdx.x + 256 * k < n4 ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++) ss = __builtin_fmaf(xv[k][j] * m, xv[k][j], ss);
    }
    ss = wave_sum_f32(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    // xn = (x * inv) * w with inv = 1 / sqrt(mean(x^2) + eps), as the reference's rmsnorm writes it
    // (engine/wgsl/base.js:119-152, coop.js:407-411); every workgroup recomputes it, as the reference's do
    const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)p.d_in + p.eps);
#pragma unroll
    for (int k = 0; k < XPT; k++)
#pragma unroll
      for (int j = 0; j < 4; j++) xv[k][j] = (xv[k][j] * inv) * wv[k][j];
    if (p.xn_out && blockIdx.x == 0) {
#pragma unroll
      for (int k = 0; k < XPT; k++) { const uint32_t e = threadIdx.x + 256 * k; if (e < n4) ((f4*)p.xn_out)[e] = xv[k]; }
    }
  }
#pragma unroll
  for (int k = 0; k < XPT; k++) {
    const uint32_t e = threadIdx.x + 256 * k;
    if (e < n4) *(f4*)(xs + (e / 8) * 36 + (e % 8) * 4) = xv[k];
  }
  __syncthreads();
  float part[RW];
#pragma unroll
  for (int r = 0; r < RW; r++) part[r] = 0.f;
#pragma unroll
  for (int pass = 0; pass < PASSES; pass++) {
  if (pass > 0) {                                                      // the next pass's weight rows
#pragma unroll
    for (int r = 0; r < RW; r++) {
      const size_t row = min(row0 + r, (size_t)p.d_out - 1);
#pragma unroll
      for (int i = 0; i < BPL; i++) {
        const uint32_t b = min(lane + 64 * (i + BPL * pass), nb - 1);
        load_block<KIND>(wr[r][i], wbase, row, nb, b);
        if constexpr (KIND != PA_W_F32) sc[r][i] = p.scales[row * nb + b];
      }
    }
  }
  float x[BPL][32], sx[BPL];
#pragma unroll
  for (int i = 0; i < BPL; i++) {
    const uint32_t b = lane + 64 * (i + BPL * pass);
    const bool on = b < nb;
    const f4* src = (const f4*)(xs + min(b, nb - 1) * 36);
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const f4 v = src[k];
#pragma unroll
      for (int j = 0; j < 4; j++) x[i][4 * k + j] = on ? v[j] : 0.f;
    }
  }
  if constexpr (KIND == PA_W_Q4_0) {
#pragma unroll
    for (int i = 0; i < BPL; i++) {
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < 32; j++) t += x[i][j];
      sx[i] = t;
    }
  } else {
#pragma unroll
    for (int i = 0; i < BPL; i++) sx[i] = 0.f;
  }
#pragma unroll
  for (int r = 0; r < RW; r++) {
    float a = part[r];
#pragma unroll
    for (int i = 0; i < BPL; i++) {
      const float d = dot_block<KIND>(wr[r][i], x[i], sx[i]);
      if constexpr (KIND == PA_W_F32) a += d;
      else a = __builtin_fmaf((float)__ushort_as_half(sc[r][i]), d, a);
    }
    part[r] = a;
  }
  }
#pragma unroll
  for (int r = 0; r < RW; r++) part[r] = wave_sum_f32(part[r]);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < RW; r++) {
      const size_t row = row0 + r;
      if (row < p.d_out) p.y[row] = p.acc ? yold[r] + part[r] : part[r];
    }
  }
}

template <int KIND, int BPL, int RW, bool NORM, int PASSES = 1>
static hipError_t launch_k(const GemvParams& p, hipStream_t s) {
  const uint32_t rows_wg = 4 * RW;
  const size_t lds = (size_t)(p.d_in / 32) * 36 * sizeof(float);
  hipLaunchKernelGGL((pa_gemv_kernel<KIND, BPL, RW, NORM, PASSES>), dim3((p.d_out + rows_wg - 1) / rows_wg), dim3(256), lds, s, p.x, p.norm_w, p.w, p.scales, p.y, p.d_out, p.d_in, p);
  return hipGetLastError();
}

template <int KIND, int BPL, bool NORM>
static hipError_t launch_rw(const GemvParams& p, int n_cu, hipStream_t s) {
  // rows per wave: as many as still leave about two 4-wave workgroups per CU, within the registers that RW x BPL
  // blocks of weights take (f32: 32 registers a block, Q8_0: 8, Q4_0: 4)
  constexpr int RWMAX = (KIND == PA_W_F32 ? 2 : 8) / BPL > 0 ? (KIND == PA_W_F32 ? 2 : 8) / BPL : 1;
  const uint32_t waves_wanted = 8u * (uint32_t)n_cu;
  uint32_t rw = p.d_out >= 8 * waves_wanted ? 8 : p.d_out >= 4 * waves_wanted ? 4 : p.d_out >= 2 * waves_wanted ? 2 : 1;
  if (rw > (uint32_t)RWMAX) rw = RWMAX;
  // Once the weights are there the kernel is VALU work, and the SIMD with the most rows sets the time: with four rows a
  // wave the MoE model's 9216 [q|k|v] rows are 2304 waves, 2.25 a SIMD -- some SIMDs work through three waves (12 rows),
  // most through two.  Three rows a wave are 3072 waves, three on every SIMD (9 rows).  Taken when it lowers the busiest
  // SIMD's rows.
  if constexpr (RWMAX >= 4) {
    const uint32_t simds = 4u * (uint32_t)n_cu;
    auto busiest = [&](uint32_t r) { const uint32_t waves = (p.d_out + r - 1) / r; return ((waves + simds - 1) / simds) * r; };
    if (rw == 4 && busiest(3) < busiest(4)) return launch_k<KIND, BPL, 3, NORM>(p, s);
  }
  if constexpr (RWMAX >= 8) { if (rw == 8) return launch_k<KIND, BPL, 8, NORM>(p, s); }
  if constexpr (RWMAX >= 4) { if (rw >= 4) return launch_k<KIND, BPL, 4, NORM>(p, s); }
  if constexpr (RWMAX >= 2) { if (rw >= 2) return launch_k<KIND, BPL, 2, NORM>(p, s); }
  return launch_k<KIND, BPL, 1, NORM>(p, s);
}

template <int KIND, bool NORM>
static hipError_t launch_bpl(const GemvParams& p, int n_cu, hipStream_t s) {
  const uint32_t nb = p.d_in / 32;
  if (nb <= 64) return launch_rw<KIND, 1, NORM>(p, n_cu, s);
  if (nb <= 128) return launch_rw<KIND, 2, NORM>(p, n_cu, s);
  if constexpr (KIND != PA_W_F32) {
    if (nb <= 192) return launch_rw<KIND, 3, NORM>(p, n_cu, s);
    if (nb <= 256) return launch_rw<KIND, 4, NORM>(p, n_cu, s);
  } else {
    if (nb <= 256) return launch_k<KIND, 2, 1, NORM, 2>(p, s);        // f32 weights past 4096 inputs: two passes of two blocks a lane
  }
  return hipErrorNotSupported;
}

hipError_t pa_launch_gemv(const GemvParams& p, int n_cu, hipStream_t s) {
  if (p.d_out == 0 || p.d_in == 0 || (p.d_in & 31)) return hipErrorInvalidValue;
  const bool norm = p.norm_w != nullptr;
  switch (p.kind) {
    case PA_W_F32: return norm ? launch_bpl<PA_W_F32, true>(p, n_cu, s) : launch_bpl<PA_W_F32, false>(p, n_cu, s);
    case PA_W_Q8_0: return norm ? launch_bpl<PA_W_Q8_0, true>(p, n_cu, s) : launch_bpl<PA_W_Q8_0, false>(p, n_cu, s);
    case PA_W_Q4_0: return norm ? launch_bpl<PA_W_Q4_0, true>(p, n_cu, s) : launch_bpl<PA_W_Q4_0, false>(p, n_cu, s);
    default: return hipErrorInvalidValue;
  }
}
