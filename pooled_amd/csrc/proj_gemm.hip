// Column-batched projections either side of the attention block on gfx950 (prefill chunks, verify blocks):
// Y[c][r] = sum_k W[r][k] X[c][k] for f32, Q8_0 and Q4_0 weights on the f16 matrix cores, and the input rmsnorm of a
// chunk written as the f16 operand the GEMM reads.
//
// Replaces the reference's batched GEMMs over the same weight planes (engine/wgsl/gemm.js:1-60 row-stationary ALU
// GEMM, engine/wgsl/gemm_sgm.js tensor-core path, dispatched by engine/qwen35.js:2142-2170 and :2600-2620) and the
// per-column rmsnorm in front of them.  Operand precision is the reference's "f16" prefill math (gemm.js:31-36, the
// r16 twins = what its tensor-core path computes): every dequantised weight (nibble - 8) * scale and every activation
// rounded to f16, products and sums in f32.
//
// Workgroup = 128 columns x 128 weight rows, 4 wavefronts of 64 x 64 (2 x 2 v_mfma_f32_32x32x16_f16 tiles), K in
// steps of one quantisation block (32): the 256 threads fetch the next step's 128 x 32 activations (f16) and 128 x 32
// weights (packed, one scale a row) into registers while the matrix cores work on the current step out of LDS,
// widen the weights to f16 on the way into LDS (0x6400 | nibble is the f16 1024 + nibble: one byte permute, a packed
// subtract and a packed multiply by the scale for two weights), and swap two LDS buffers with one barrier a step.
// Rows of the LDS tiles are 80 bytes apart so that the 128-bit fragment reads are bank-conflict free.  The activation
// is the MFMA A operand and the weight the B operand: a lane then owns one weight row and four consecutive columns per
// accumulator quad, and a wave-wide store covers 32 consecutive rows of a column (128 bytes).
#include "pa_internal.h"
#include "glue_math.h"

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));

#define GT 128          // tile edge (columns and rows per workgroup)
#define GK 32           // K per step = one quantisation block
#define GROW 80         // LDS row stride in bytes (64 of data + 16 of padding)

static __device__ inline h2 as_h2(uint32_t u) { h2 r; __builtin_memcpy(&r, &u, 4); return r; }

// two bytes of a word (byte indices by the selector) -> two f16 = (byte - bias) * scale
static __device__ inline h2 bytes_to_h2(uint32_t w, uint32_t sel, h2 bias, h2 sc) {
  return (as_h2(__builtin_amdgcn_perm(0x64646464u, w, sel)) - bias) * sc;
}

// 16 weights of one (row, block half) as two h8, from the packed registers of a kind
template <int KIND> struct WRegs;
template <> struct WRegs<PA_W_Q4_0> { u2 q; uint16_t sc; };      // bytes 8h .. 8h + 7: elements 8h + j (low), 16 + 8h + j (high)
template <> struct WRegs<PA_W_Q8_0> { u4 q; uint16_t sc; };      // elements 16h .. 16h + 15
template <> struct WRegs<PA_W_F32> { f4 q[4]; uint16_t sc; };    // elements 16h .. 16h + 15

template <int KIND>
static __device__ inline void w_load(WRegs<KIND>& r, const GemmParams& p, size_t row, uint32_t nb, uint32_t kb, uint32_t half) {
  const unsigned char* base = (const unsigned char*)p.w;
  if constexpr (KIND == PA_W_Q4_0) {
    r.q = *(const u2*)(base + (row * nb + kb) * 16 + 8 * half);
    r.sc = p.scales[row * nb + kb];
  } else if constexpr (KIND == PA_W_Q8_0) {
    r.q = *(const u4*)(base + (row * nb + kb) * 32 + 16 * half);
    r.sc = p.scales[row * nb + kb];
  } else {
    const f4* s = (const f4*)(base + ((row * nb + kb) * 32 + 16 * half) * 4);
#pragma unroll
    for (int i = 0; i < 4; i++) r.q[i] = s[i];
    r.sc = 0;
  }
}

// widen and store: dst = the row's 32 halves in LDS
template <int KIND>
static __device__ inline void w_store(const WRegs<KIND>& r, unsigned char* dst, uint32_t half) {
  if constexpr (KIND == PA_W_Q4_0) {
    const _Float16 s = __ushort_as_half(r.sc);
    const h2 sc = { s, s }, bias = { (_Float16)1032.f, (_Float16)1032.f };      // 0x6400 | n = 1024 + n; n - 8
    h2 lo[4], hi[4];
#pragma unroll
    for (int w = 0; w < 2; w++) {
      const uint32_t l = r.q[w] & 0x0F0F0F0Fu, h = (r.q[w] >> 4) & 0x0F0F0F0Fu;
      lo[2 * w] = bytes_to_h2(l, 0x04010400u, bias, sc); lo[2 * w + 1] = bytes_to_h2(l, 0x04030402u, bias, sc);
      hi[2 * w] = bytes_to_h2(h, 0x04010400u, bias, sc); hi[2 * w + 1] = bytes_to_h2(h, 0x04030402u, bias, sc);
    }
    *(h8*)(dst + (8 * half) * 2) = (h8){ lo[0][0], lo[0][1], lo[1][0], lo[1][1], lo[2][0], lo[2][1], lo[3][0], lo[3][1] };
    *(h8*)(dst + (16 + 8 * half) * 2) = (h8){ hi[0][0], hi[0][1], hi[1][0], hi[1][1], hi[2][0], hi[2][1], hi[3][0], hi[3][1] };
  } else if constexpr (KIND == PA_W_Q8_0) {
    const _Float16 s = __ushort_as_half(r.sc);
    const h2 sc = { s, s }, bias = { (_Float16)1152.f, (_Float16)1152.f };      // 0x6400 | (v + 128) = 1152 + v
    h2 o[8];
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const uint32_t x = r.q[w] ^ 0x80808080u;
      o[2 * w] = bytes_to_h2(x, 0x04010400u, bias, sc); o[2 * w + 1] = bytes_to_h2(x, 0x04030402u, bias, sc);
    }
    *(h8*)(dst + (16 * half) * 2) = (h8){ o[0][0], o[0][1], o[1][0], o[1][1], o[2][0], o[2][1], o[3][0], o[3][1] };
    *(h8*)(dst + (16 * half + 8) * 2) = (h8){ o[4][0], o[4][1], o[5][0], o[5][1], o[6][0], o[6][1], o[7][0], o[7][1] };
  } else {
    h8 a, b;
#pragma unroll
    for (int j = 0; j < 4; j++) { a[j] = (_Float16)r.q[0][j]; a[4 + j] = (_Float16)r.q[1][j]; b[j] = (_Float16)r.q[2][j]; b[4 + j] = (_Float16)r.q[3][j]; }
    *(h8*)(dst + (16 * half) * 2) = a;
    *(h8*)(dst + (16 * half + 8) * 2) = b;
  }
}

// lane <-> lane ^ 1
static __device__ inline uint32_t pair_swap(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false); }

// XT: the workgroup covers 128 XT columns (a wave 64 XT columns x 64 rows): with XT = 2 every weight fragment read from
// LDS feeds four MFMAs instead of two and the LDS traffic per flop drops by a quarter.
template <int KIND, int XT>
__global__ __launch_bounds__(256, XT == 2 ? 2 : 1) void pa_gemm_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char xs[2][GT * XT * GROW];
  __shared__ __attribute__((aligned(16))) unsigned char ws[2][GT * GROW];
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t wm = wave >> 1, wn = wave & 1;                       // the wave's 64 XT columns x 64 rows
  const uint32_t r0 = blockIdx.x * GT, c0 = blockIdx.y * GT * XT;
  const uint32_t nb = p.d_in / GK;
  // The memory pipeline takes a wave-wide load one cache line (128 bytes) at a time, so what a step's loads cost
  // is the number of lines they touch.  Activations: four lanes fetch the 64 bytes of a column's step (16 lines a
  // wave-wide load, two loads a step).  Weights: thread t widens half `t & 1` of row `t >> 1`; Q4_0 rows are fetched
  // as whole 16-byte blocks, two steps at a time -- the even lane of a pair holds the block of the even step, the odd
  // lane the next one (32 contiguous bytes a row) -- and each step the holder hands its partner the other half.
  const uint32_t xrow = tid >> 2, xch = tid & 3;
  const unsigned char* xsrc[2 * XT];
#pragma unroll
  for (int i = 0; i < 2 * XT; i++)
    xsrc[i] = (const unsigned char*)(p.x + min((size_t)c0 + xrow + 64 * i, (size_t)p.n_cols - 1) * p.x_stride) + 16 * xch;   // past the end: the last column again (never stored)
  const uint32_t lrow = tid >> 1, half = tid & 1;
  const size_t wrow = min((size_t)r0 + lrow, (size_t)p.d_out - 1);
  WRegs<KIND> wr;
  u4 wq4 = {0, 0, 0, 0}; uint16_t wsc4 = 0;                           // Q4_0: the pair's block and scale held by this lane
  u4 xr[2 * XT];
  auto fetch_x = [&](uint32_t kb) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2 * XT; i++) xr[i] = *(const u4*)(xsrc[i] + (size_t)kb * 64);
  };
  // Q4_0: blocks kb0 + half of the row (kb0 = the step the even lane's block belongs to)
  auto fetch_w4 = [&](uint32_t kb0) __attribute__((always_inline)) {
    const size_t b = wrow * nb + min(kb0 + half, nb - 1);
    wq4 = *(const u4*)((const unsigned char*)p.w + b * 16);
    wsc4 = p.scales[b];
  };
  auto stage = [&](int buf, uint32_t kb) __attribute__((always_inline)) {
    if constexpr (KIND == PA_W_Q4_0) {
      const bool holder = half == (kb & 1);
      const uint32_t m0 = half ? wq4[2] : wq4[0], m1 = half ? wq4[3] : wq4[1];        // my half of my own block
      const uint32_t g0 = pair_swap(half ? wq4[0] : wq4[2]), g1 = pair_swap(half ? wq4[1] : wq4[3]), gs = pair_swap((uint32_t)wsc4);   // my half of the partner's
      wr.q[0] = holder ? m0 : g0; wr.q[1] = holder ? m1 : g1; wr.sc = holder ? wsc4 : (uint16_t)gs;
    }
    w_store<KIND>(wr, ws[buf] + lrow * GROW, half);
#pragma unroll
    for (int i = 0; i < 2 * XT; i++) *(u4*)(xs[buf] + (xrow + 64 * i) * GROW + 16 * xch) = xr[i];
  };
  f16v acc[2 * XT][2];
#pragma unroll
  for (int a = 0; a < 2 * XT; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;
  fetch_x(0);
  if constexpr (KIND == PA_W_Q4_0) fetch_w4(0); else w_load<KIND>(wr, p, wrow, nb, 0, half);
  stage(0, 0);
  __syncthreads();
  const uint32_t fl = lane & 31, fk = lane >> 5;                      // fragment row and 8-wide k group of this lane
  auto mma = [&](int cur) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      h8 af[2 * XT], bf[2];
#pragma unroll
      for (int t = 0; t < 2 * XT; t++) af[t] = *(const h8*)(xs[cur] + (wm * 64 * XT + t * 32 + fl) * GROW + (ks * 16 + fk * 8) * 2);
#pragma unroll
      for (int t = 0; t < 2; t++) bf[t] = *(const h8*)(ws[cur] + (wn * 64 + t * 32 + fl) * GROW + (ks * 16 + fk * 8) * 2);
#pragma unroll
      for (int a = 0; a < 2 * XT; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
  };
  // Steps two at a time (buffer 0 then 1); every load is issued whatever the step -- past the last step the last block
  // again, staged into the buffer nobody reads -- so that the waits can count loads instead of draining them.
  // A compiler-level memory fence between a step's MFMAs and its staging code keeps the step's global loads above
  // the fence (left alone, the compiler sinks them next to the staging code that consumes them, and every step waits
  // out a full memory round trip) while the widening arithmetic may still be scheduled among the MFMAs; a full
  // scheduling barrier there costs 20 %.
  for (uint32_t kb = 0; kb < nb; kb += 2) {
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      if (kb + hh >= nb) break;
      fetch_x(min(kb + 1 + hh, nb - 1));
      if constexpr (KIND == PA_W_Q4_0) { if (hh == 1) fetch_w4(kb + 2); }     // block kb + 1 sits in the odd lanes since step kb - 1
      else w_load<KIND>(wr, p, wrow, nb, min(kb + 1 + hh, nb - 1), half);
      mma(hh);
      asm volatile("" ::: "memory");
      stage(hh ^ 1, kb + 1 + hh);
      __syncthreads();
    }
  }
  // accumulator i of a tile: column 8 (i / 4) + 4 (lane / 32) + i % 4, row lane % 32
#pragma unroll
  for (int a = 0; a < 2 * XT; a++)
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const uint32_t row = r0 + wn * 64 + b * 32 + fl;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const uint32_t col = c0 + wm * 64 * XT + a * 32 + 8 * (i / 4) + 4 * fk + (i % 4);
        if (row < p.d_out && col < p.n_cols) {
          float* y = p.y + (size_t)col * p.y_stride + row;
          *y = p.acc ? *y + acc[a][b][i] : acc[a][b][i];
        }
      }
    }
}

// ---- skinny chunks (a verify block, the reference's 16-column passes: engine/wgsl/coop.js batched matvec) ----
// With a handful of columns the tiled kernel leaves the chip empty (d_out / 128 workgroups, each walking all of K)
// while the work is one pass over the weights.  This kernel streams the weights GEMV-style -- a wave owns RW rows, a
// lane the 32-value blocks lane + 64 i of each -- widens them once into f16 pairs in registers, stages all the
// chunk's columns in LDS (80-byte block stride: conflict-free 128-bit reads) and runs one v_dot2_f32_f16 per two
// weights and column.  Same operand precision as the tiled kernel (weights and activations f16, sums f32), so a
// result does not depend on which kernel served the chunk beyond the order of the sums.  The lanes' partial sums go
// through LDS (the staging area, free by then): lane t of a wave adds up the 64 partials of its (row, column).
#define SK_NC 16        // columns a launch serves at most
template <int KIND, int BPL, int RW>
__global__ __launch_bounds__(256)
void pa_gemm_skinny_kernel(const uint16_t* a_x, const void* a_w, const uint16_t* a_scales, uint32_t a_x_stride, uint32_t a_d_out, uint32_t a_d_in, uint32_t a_n_cols,
                           GemmParams p_in) {
  static_assert(KIND == PA_W_Q4_0 || KIND == PA_W_Q8_0, "quantised weights");
  // (the leading arguments repeat fields of p_in: they are preloaded into scalar registers, so the loads below need no
  // scalar-load round trip; the other arguments are fetched in one batch behind them)
  GemmParams p = p_in;
  p.x = a_x; p.w = a_w; p.scales = a_scales; p.x_stride = a_x_stride; p.d_out = a_d_out; p.d_in = a_d_in; p.n_cols = a_n_cols;
  extern __shared__ __attribute__((aligned(16))) unsigned char sk_lds[];
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t nb = p.d_in / GK, ncol = p.n_cols;
  const uint32_t xcol = nb * GROW;                                    // bytes of a staged column
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * RW;
  // The first eight 16-byte pieces a thread stages of the chunk's columns (all of them for 8 columns of 2048) are
  // requested FIRST, the wave's weight rows right behind them: a wave's loads complete in order, the columns come from
  // L2 in a fraction of the time the weight stream takes from HBM, and their trip into LDS then runs under the latency
  // of the weights instead of after it.
  const uint32_t cpc = p.d_in / 8;                                    // 16-byte pieces of a column
  const uint32_t pieces = ncol * cpc;
  u4 xv0[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const uint32_t e = min(tid + 256 * j, pieces - 1), c = e / cpc, k8 = e % cpc;
    xv0[j] = *(const u4*)((const unsigned char*)(p.x + (size_t)c * p.x_stride) + k8 * 16);
  }
  __builtin_amdgcn_sched_barrier(0);
  constexpr int WQ = KIND == PA_W_Q4_0 ? 1 : 2;                       // 16-byte words of a packed block
  u4 wq[RW][BPL][WQ];
  uint16_t wsc[RW][BPL];
#pragma unroll
  for (int r = 0; r < RW; r++) {
    const size_t row = min(row0 + r, (size_t)p.d_out - 1);            // rows past the end repeat the last one (not stored)
#pragma unroll
    for (int i = 0; i < BPL; i++) {
      const uint32_t b = min(lane + 64 * i, nb - 1);                   // blocks past the end likewise (scale forced to 0)
      const u4* src = (const u4*)((const unsigned char*)p.w + (row * nb + b) * (16 * WQ));
#pragma unroll
      for (int w = 0; w < WQ; w++) wq[r][i][w] = src[w];
      wsc[r][i] = p.scales[row * nb + b];
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("" :: "s"(p.y), "s"(p.y_stride), "s"(p.acc));
  // the chunk's columns -> LDS, 16 bytes a thread and turn: the pieces requested above, ...
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const uint32_t e = tid + 256 * j, c = e / cpc, k8 = e % cpc;
    if (e < pieces) *(u4*)(sk_lds + c * xcol + (k8 >> 2) * GROW + (k8 & 3) * 16) = xv0[j];
  }
  // ... then any further turns (eight loads a thread go out before the first is stored -- unconditional, a turn past the
  // end re-reads the last piece: one load a loop turn is one round trip a turn)
  for (uint32_t e0 = tid + 256 * 8; e0 < pieces; e0 += 256 * 8) {
    u4 v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t e = min(e0 + 256 * j, pieces - 1), c = e / cpc, k8 = e % cpc;
      v[j] = *(const u4*)((const unsigned char*)(p.x + (size_t)c * p.x_stride) + k8 * 16);
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const uint32_t e = e0 + 256 * j, c = e / cpc, k8 = e % cpc;
      if (e < pieces) *(u4*)(sk_lds + c * xcol + (k8 >> 2) * GROW + (k8 & 3) * 16) = v[j];
    }
  }
  // widen: pair k of a block = elements 2k, 2k + 1
  h2 wv[RW][BPL][16];
#pragma unroll
  for (int r = 0; r < RW; r++)
#pragma unroll
    for (int i = 0; i < BPL; i++) {
      const _Float16 s1 = __ushort_as_half(lane + 64 * i < nb ? wsc[r][i] : (uint16_t)0);
      const h2 sc = { s1, s1 };
      if constexpr (KIND == PA_W_Q4_0) {
        const h2 bias = { (_Float16)1032.f, (_Float16)1032.f };
#pragma unroll
        for (int d = 0; d < 4; d++) {
          const uint32_t l = wq[r][i][0][d] & 0x0F0F0F0Fu, h = (wq[r][i][0][d] >> 4) & 0x0F0F0F0Fu;
          wv[r][i][2 * d] = bytes_to_h2(l, 0x04010400u, bias, sc); wv[r][i][2 * d + 1] = bytes_to_h2(l, 0x04030402u, bias, sc);
          wv[r][i][8 + 2 * d] = bytes_to_h2(h, 0x04010400u, bias, sc); wv[r][i][8 + 2 * d + 1] = bytes_to_h2(h, 0x04030402u, bias, sc);
        }
      } else {
        const h2 bias = { (_Float16)1152.f, (_Float16)1152.f };
#pragma unroll
        for (int w = 0; w < 2; w++)
#pragma unroll
          for (int d = 0; d < 4; d++) {
            const uint32_t x = wq[r][i][w][d] ^ 0x80808080u;
            wv[r][i][8 * w + 2 * d] = bytes_to_h2(x, 0x04010400u, bias, sc); wv[r][i][8 * w + 2 * d + 1] = bytes_to_h2(x, 0x04030402u, bias, sc);
          }
      }
    }
  __syncthreads();
  float part[SK_NC][RW];
#pragma unroll
  for (int c = 0; c < SK_NC; c++) {
#pragma unroll
    for (int r = 0; r < RW; r++) part[c][r] = 0.f;
    if ((uint32_t)c < ncol) {
#pragma unroll
      for (int i = 0; i < BPL; i++) {
        const unsigned char* xb = sk_lds + c * xcol + min(lane + 64 * i, nb - 1) * GROW;
        h2 xv[16];
#pragma unroll
        for (int q = 0; q < 4; q++) { const h8 v = *(const h8*)(xb + 16 * q); xv[4 * q] = (h2){ v[0], v[1] }; xv[4 * q + 1] = (h2){ v[2], v[3] }; xv[4 * q + 2] = (h2){ v[4], v[5] }; xv[4 * q + 3] = (h2){ v[6], v[7] }; }
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
          for (int k = 0; k < 16; k++) part[c][r] = __builtin_amdgcn_fdot2(wv[r][i][k], xv[k], part[c][r], false);
      }
    }
  }
  __syncthreads();                                                    // every wave is done with the staged columns
  // partials -> LDS [wave][lane][SK_NC * RW + 1], then lane t sums column t of its wave's 64 x (SK_NC * RW) table
  constexpr int PV = SK_NC * RW, PS = PV + 1;
  float* ps = (float*)sk_lds + (size_t)wave * 64 * PS;
#pragma unroll
  for (int c = 0; c < SK_NC; c++)
    if ((uint32_t)c < ncol)
#pragma unroll
      for (int r = 0; r < RW; r++) ps[lane * PS + c * RW + r] = part[c][r];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (uint32_t t = lane; t < ncol * RW; t += 64) {
    const uint32_t c = t / RW, r = t % RW;
    float* y = p.y + (size_t)c * p.y_stride + min(row0 + r, (size_t)p.d_out - 1);
    const float yo = p.acc ? *y : 0.f;                                // on its way while the partials are added up
    float a = 0.f;
    for (int l = 0; l < 64; l++) a += ps[l * PS + t];
    if (row0 + r < p.d_out) *y = p.acc ? yo + a : a;
  }
}

// LDS the skinny kernel needs: the staged columns, or the four waves' partial tables if those are larger
static size_t skinny_lds(const GemmParams& p, int rw) {
  const size_t x = (size_t)p.n_cols * (p.d_in / GK) * GROW, ps = (size_t)4 * 64 * (SK_NC * rw + 1) * sizeof(float);
  return x > ps ? x : ps;
}
template <int KIND, int BPL, int RW>
static hipError_t launch_skinny(const GemmParams& p, hipStream_t s) {
  const size_t lds = skinny_lds(p, RW);
  static size_t attr = 0;
  if (lds > attr) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_gemm_skinny_kernel<KIND, BPL, RW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr = lds;
  }
  hipLaunchKernelGGL((pa_gemm_skinny_kernel<KIND, BPL, RW>), dim3((p.d_out + 4 * RW - 1) / (4 * RW)), dim3(256), lds, s, p.x, p.w, p.scales, p.x_stride, p.d_out, p.d_in,
                     p.n_cols, p);
  return hipGetLastError();
}
template <int KIND>
static hipError_t launch_skinny_kind(const GemmParams& p, int n_cu, hipStream_t s) {
  if (p.d_in <= 2048) {
    // (three rows a wave where that lowers the rows of the busiest SIMD -- 9216 rows: 2304 waves at 2.25 a SIMD, or 3072
    // at three -- as the one-token GEMV chooses)
    const uint32_t simds = 4u * (uint32_t)(n_cu > 0 ? n_cu : 256);
    auto busiest = [&](uint32_t r) { const uint32_t waves = (p.d_out + r - 1) / r; return ((waves + simds - 1) / simds) * r; };
    if (busiest(3) < busiest(4)) return launch_skinny<KIND, 1, 3>(p, s);
    return launch_skinny<KIND, 1, 4>(p, s);
  }
  if (p.d_in <= 4096) return launch_skinny<KIND, 2, 2>(p, s);
  return launch_skinny<KIND, 4, 1>(p, s);
}

template <int XT>
static hipError_t launch_gemm_xt(const GemmParams& p, hipStream_t s) {
  const dim3 grid((p.d_out + GT - 1) / GT, (p.n_cols + GT * XT - 1) / (GT * XT)), block(256);
  switch (p.kind) {
    case PA_W_F32: hipLaunchKernelGGL((pa_gemm_kernel<PA_W_F32, 1>), dim3(grid.x, (p.n_cols + GT - 1) / GT), block, 0, s, p); break;
    case PA_W_Q8_0: hipLaunchKernelGGL((pa_gemm_kernel<PA_W_Q8_0, XT>), grid, block, 0, s, p); break;
    case PA_W_Q4_0: hipLaunchKernelGGL((pa_gemm_kernel<PA_W_Q4_0, XT>), grid, block, 0, s, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t pa_launch_gemm(const GemmParams& p, int n_cu, hipStream_t s) {
  if (p.d_out == 0 || p.d_in == 0 || (p.d_in & 31) || p.n_cols == 0) return hipErrorInvalidValue;
  // a handful of columns: a pass over the weights per launch of up to 16 columns (as many as fit the LDS staging),
  // up to 32 columns in all -- past that the tiled kernel wins
  if (p.kind != PA_W_F32 && p.n_cols <= 2 * SK_NC && p.d_in <= 8192 && (p.x_stride & 7) == 0) {
    const uint32_t fit = (uint32_t)((144 * 1024) / ((size_t)(p.d_in / GK) * GROW));
    const uint32_t per = fit < SK_NC ? fit : SK_NC;
    if (per >= 1) {
      for (uint32_t c0 = 0; c0 < p.n_cols; c0 += per) {
        GemmParams q = p;
        q.x = p.x + (size_t)c0 * p.x_stride; q.y = p.y + (size_t)c0 * p.y_stride;
        q.n_cols = p.n_cols - c0 < per ? p.n_cols - c0 : per;
        const hipError_t e = p.kind == PA_W_Q4_0 ? launch_skinny_kind<PA_W_Q4_0>(q, n_cu, s) : launch_skinny_kind<PA_W_Q8_0>(q, n_cu, s);
        if (e != hipSuccess) return e;
      }
      return hipSuccess;
    }
  }
  // 256-column workgroups (two fit a CU) when they still give every CU four: otherwise 128-column ones (three a CU)
  const size_t wgs2 = (size_t)((p.d_out + GT - 1) / GT) * ((p.n_cols + 2 * GT - 1) / (2 * GT));
  const bool xt2 = wgs2 >= (size_t)4 * (n_cu > 0 ? n_cu : 256);
  return xt2 ? launch_gemm_xt<2>(p, s) : launch_gemm_xt<1>(p, s);
}

// rmsnorm of n_cols columns, written as f16: one workgroup per column.  xn = f16((x * inv) * w),
// inv = 1 / sqrt(mean(x^2) + eps) (engine/wgsl/base.js:119-152); the sum of squares is a fixed-order tree.
__global__ __launch_bounds__(256) void pa_rmsnorm_f16_kernel(const float* x, uint32_t x_stride, const float* w, uint32_t dim, float eps,
                                                            uint16_t* out, uint32_t out_stride) {
  // (every kernel argument in the first batch of scalar loads instead of a dependent round trip at each first use)
  asm volatile("" :: "s"(x), "s"(x_stride), "s"(w), "s"(dim), "s"(eps), "s"(out), "s"(out_stride));
  __shared__ float red[4];
  const uint32_t col = blockIdx.x, tid = threadIdx.x;
  const f4* xs = (const f4*)(x + (size_t)col * x_stride);
  const uint32_t n4 = dim / 4;
  float ss = 0.f;
  // Columns of up to 8192 values: x and the norm weights are held in registers (2, 4 or 8 float4 a thread) and requested
  // together, unconditionally (a turn past the end re-reads the last float4 and is masked out of the sum by a factor):
  // one load a loop turn, twice over, was four round trips for 2048 values.
  auto in_regs = [&](auto XPC) __attribute__((always_inline)) {
    constexpr int XP = decltype(XPC)::value;
    f4 xv[XP], wv[XP];
#pragma unroll
    for (int k = 0; k < XP; k++) xv[k] = xs[min(tid + 256 * k, n4 - 1)];
#pragma unroll
    for (int k = 0; k < XP; k++) wv[k] = ((const f4*)w)[min(tid + 256 * k, n4 - 1)];
#pragma unroll
    for (int k = 0; k < XP; k++) {
      const float m = tid + 256 * k < n4 ? 1.f : 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++) ss = __builtin_fmaf(xv[k][j] * m, xv[k][j], ss);
    }
    ss = wave_sum_f32(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)dim + eps);
#pragma unroll
    for (int k = 0; k < XP; k++) {
      const uint32_t e = tid + 256 * k;
      const _Float16 o[4] = { (_Float16)((xv[k][0] * inv) * wv[k][0]), (_Float16)((xv[k][1] * inv) * wv[k][1]), (_Float16)((xv[k][2] * inv) * wv[k][2]), (_Float16)((xv[k][3] * inv) * wv[k][3]) };
      if (e < n4) __builtin_memcpy(out + (size_t)col * out_stride + 4 * e, o, 8);
    }
  };
  if (n4 <= 512) { in_regs(std::integral_constant<int, 2>{}); return; }
  if (n4 <= 1024) { in_regs(std::integral_constant<int, 4>{}); return; }
  if (n4 <= 2048) { in_regs(std::integral_constant<int, 8>{}); return; }
  for (uint32_t e = tid; e < n4; e += 256) { const f4 v = xs[e]; ss = __builtin_fmaf(v[0], v[0], ss); ss = __builtin_fmaf(v[1], v[1], ss); ss = __builtin_fmaf(v[2], v[2], ss); ss = __builtin_fmaf(v[3], v[3], ss); }
  ss = wave_sum_f32(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)dim + eps);
  for (uint32_t e = tid; e < n4; e += 256) {
    const f4 v = xs[e], wv = ((const f4*)w)[e];
    const _Float16 o[4] = { (_Float16)((v[0] * inv) * wv[0]), (_Float16)((v[1] * inv) * wv[1]), (_Float16)((v[2] * inv) * wv[2]), (_Float16)((v[3] * inv) * wv[3]) };
    __builtin_memcpy(out + (size_t)col * out_stride + 4 * e, o, 8);
  }
}

hipError_t pa_launch_rmsnorm_f16(const float* x, uint32_t x_stride, const float* w, uint32_t dim, float eps, uint32_t n_cols,
                                 uint16_t* out, uint32_t out_stride, hipStream_t s) {
  if (dim == 0 || (dim & 3) || n_cols == 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(pa_rmsnorm_f16_kernel, dim3(n_cols), dim3(256), 0, s, x, x_stride, w, dim, eps, out, out_stride);
  return hipGetLastError();
}
