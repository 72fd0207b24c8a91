// Column-batched projections for large chunks on gfx950: Y[c][r] = sum_k W[r][k] X[c][k] with the weights widened
// to f16 once per call and a matrix-core GEMM over two f16 operands.
//
// Same contract and the same operand precision as pa_gemm_kernel (proj_gemm.hip) -- the reference's "f16" prefill
// math, engine/wgsl/gemm.js:31-36: every dequantised weight and every activation rounded to f16, products and sums
// f32 -- for the chunks its batched GEMMs serve (engine/wgsl/gemm.js, gemm_sgm.js, gemm_wide.js; dispatched at
// engine/qwen35.js:2142-2170, :2600-2620).  What differs is where the widening happens.  The tiled kernel of
// proj_gemm.hip widens packed weights on their way into LDS inside its main loop; at 64 x 64 wave tiles that loop is
// bound by LDS traffic and by the widening arithmetic in front of every barrier.  For a chunk of hundreds of columns
// the weights are re-read by every column block anyway, so here they are widened once into a context-owned f16
// staging matrix [d_out][d_in] (pa_widen_w_kernel: one pass over the packed planes, HBM-bound), and the GEMM proper
// has nothing but loads and MFMAs in its loop:
//
//   * workgroup = 2 x 2 wavefronts, one per SIMD; a wavefront owns 128 columns x 32 TN rows (TN = 2, 3 or 4) as
//     4 x TN v_mfma_f32_32x32x16_f16 tiles whose accumulators (up to 256 registers) live in the accumulation
//     registers; every A (activation) fragment read from LDS feeds TN MFMAs and every B (weight) fragment four:
//     0.5 KB of LDS reads per MFMA at TN = 4 against 1 KB at 64 x 64 wave tiles;
//   * both operands go global -> LDS with global_load_lds_dwordx4 (no staging registers, no arithmetic), K in
//     stages of 64 (128-byte rows), two stages in LDS, one barrier a stage; rows cannot be padded (an LDS-direct
//     load writes 64 x 16 bytes contiguously), so the 16-byte chunk c of row r is fetched into slot
//     c ^ ((r >> 1) & 7): the ds_read_b128 fragment reads of any 16 consecutive rows then hit 64 distinct banks;
//   * one wave a SIMD means nothing hides an LDS round trip, so the fragments are double buffered in registers by
//     hand: the reads of k-step i + 1 (and, across the barrier, of the next stage's first k-step) are issued among
//     the MFMAs of k-step i;
//   * TN is picked per call so that the workgroups fill whole rounds of the chip.
#include "pf_common.h"

#ifndef GW_ABL
#define GW_ABL 0            // development ablations (wrong results, timing only): bit 0 no loads after the prologue, bit 1 no barriers
#endif
#define GW_COLS 256          // columns per workgroup (2 waves x 128)
#define GW_KS 64             // K per stage
#define GW_ROWB 128          // bytes of a staged row (64 halves)

struct Gemm16Params {
  const uint16_t* x; const uint16_t* w16; float* y;
  uint32_t x_stride, y_stride, d_out, d_in, n_cols;
  int acc;
};

template <int TN>
__global__ __launch_bounds__(256, 1) void pa_gemm16_kernel(Gemm16Params p) {
  constexpr int TM = 4;                                  // 32-column blocks per wave
  constexpr int ROWS = 64 * TN;                          // weight rows per workgroup
  constexpr int A_BYTES = GW_COLS * GW_ROWB, B_BYTES = ROWS * GW_ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LD = GW_COLS / 8 / 4, B_LD = ROWS / 8 / 4;     // 1 KB loads (8 rows) per wave and stage
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];   // [2][A | B]
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave >> 1, wn = wave & 1;
  const uint32_t c0 = blockIdx.y * GW_COLS, r0 = blockIdx.x * ROWS;
  const uint32_t n_stages = p.d_in / GW_KS;

  // ---- LDS-direct loads: a load covers 8 rows x 128 bytes; lane i lands at (row i / 8, slot i % 8) and fetches chunk
  //      slot ^ ((row >> 1) & 7) of that row.  Rows past the end of the operand repeat its last row (never stored). ----
  const uint32_t lrow = lane >> 3, lslot = lane & 7;
  const unsigned char* a_src[A_LD]; const unsigned char* b_src[B_LD];
#pragma unroll
  for (int i = 0; i < A_LD; i++) {
    const uint32_t row = (wave * A_LD + i) * 8 + lrow;                       // row of the A tile = column of the chunk
    const size_t col = min((size_t)c0 + row, (size_t)p.n_cols - 1);
    a_src[i] = (const unsigned char*)(p.x + col * p.x_stride) + ((lslot ^ ((row >> 1) & 7)) * 16);
  }
#pragma unroll
  for (int i = 0; i < B_LD; i++) {
    const uint32_t row = (wave * B_LD + i) * 8 + lrow;
    const size_t wr = min((size_t)r0 + row, (size_t)p.d_out - 1);
    b_src[i] = (const unsigned char*)(p.w16 + wr * p.d_in) + ((lslot ^ ((row >> 1) & 7)) * 16);
  }
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_addr_of(smem));
  auto issue = [&](uint32_t st) __attribute__((always_inline)) {
    const uint32_t base = lds0 + (st & 1) * STAGE;
    const size_t koff = (size_t)st * GW_ROWB;
#pragma unroll
    for (int i = 0; i < A_LD; i++) pf_gll(a_src[i] + koff, base + (wave * A_LD + i) * 1024);
#pragma unroll
    for (int i = 0; i < B_LD; i++) pf_gll(b_src[i] + koff, base + A_BYTES + (wave * B_LD + i) * 1024);
  };

  f16v acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

  // fragment addresses: row fl of a 32-row block, 8 halves at k = 16 ks + 8 fk -> chunk 2 ks + fk, swizzled by the row
  // (the swizzle is an XOR on the chunk index, and 2 ks has no bit in common with fk)
  const uint32_t fl = lane & 31, fk = lane >> 5;
  uint32_t a_rd[TM], b_rd[TN];
#pragma unroll
  for (int t = 0; t < TM; t++) { const uint32_t row = wm * 128 + t * 32 + fl; a_rd[t] = row * GW_ROWB + ((fk ^ ((row >> 1) & 7)) * 16); }
#pragma unroll
  for (int t = 0; t < TN; t++) { const uint32_t row = wn * 32 * TN + t * 32 + fl; b_rd[t] = A_BYTES + row * GW_ROWB + ((fk ^ ((row >> 1) & 7)) * 16); }
  struct Frag { h8 a[TM]; h8 b[TN]; };
  auto rd = [&](Frag& f, const unsigned char* sb, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TM; t++) f.a[t] = *(const h8*)(sb + (a_rd[t] ^ (ks * 32)));
#pragma unroll
    for (int t = 0; t < TN; t++) f.b[t] = *(const h8*)(sb + (b_rd[t] ^ (ks * 32)));
  };
  auto mma = [&](const Frag& f) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[a], f.b[b], acc[a][b], 0, 0, 0);
  };
  // the fragment reads of the next k-step are spread among this k-step's MFMAs (one wave a SIMD: nothing else hides
  // an LDS round trip)
  auto interleave = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM + TN; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, (TM * TN) / (TM + TN) > 0 ? (TM * TN) / (TM + TN) : 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN) * ((TM * TN) / (TM + TN)), 0);
  };

  Frag f0, f1;
  issue(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  rd(f0, smem, 0);
  for (uint32_t st = 0; st < n_stages; st++) {
    const bool more = st + 1 < n_stages;
    if (more && !((GW_ABL & 1) && st > 0)) issue(st + 1);     // into the buffer every wave left before the last barrier
    const unsigned char* sb = smem + (st & 1) * STAGE;
    rd(f1, sb, 1); mma(f0); interleave();
    rd(f0, sb, 2); mma(f1); interleave();
    rd(f1, sb, 3); mma(f0); interleave();
    // the stage's last fragments are on their way; behind the barrier the other buffer holds stage st + 1 (every wave
    // waited for its own loads) and nobody reads this one any more
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    if (!(GW_ABL & 2)) __syncthreads();
    if (more) rd(f0, smem + ((st + 1) & 1) * STAGE, 0);
    mma(f1);
    if (more) interleave();
  }

  // accumulator i of a tile: column 8 (i / 4) + 4 (lane / 32) + i % 4, row lane % 32
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) {
      const uint32_t row = r0 + wn * 32 * TN + b * 32 + fl;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const uint32_t col = c0 + wm * 128 + a * 32 + 8 * (i / 4) + 4 * fk + (i % 4);
        if (row < p.d_out && col < p.n_cols) {
          float* y = p.y + (size_t)col * p.y_stride + row;
          *y = p.acc ? *y + acc[a][b][i] : acc[a][b][i];
        }
      }
    }
}

// ---- weights -> f16 [d_out][d_in], the arithmetic of the tiled kernel's staging: (nibble - 8) * scale and
//      int8 * scale in f16 (exact integer, one rounding), f32 rounded to nearest even ----
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
static __device__ inline h2v gw_as_h2(uint32_t u) { h2v r; __builtin_memcpy(&r, &u, 4); return r; }
static __device__ inline h2v gw_bytes(uint32_t w, uint32_t sel, h2v bias, h2v sc) { return (gw_as_h2(__builtin_amdgcn_perm(0x64646464u, w, sel)) - bias) * sc; }

// one thread per quantisation block of 32 weights
template <int KIND>
__global__ __launch_bounds__(256) void pa_widen_w_kernel(const void* w, const uint16_t* scales, uint16_t* out, size_t n_blocks) {
  const size_t b = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= n_blocks) return;
  h8 o[4];
  if constexpr (KIND == PA_W_Q4_0) {
    const u4 q = *(const u4*)((const unsigned char*)w + b * 16);       // byte j: element j (low nibble), element 16 + j (high)
    const _Float16 s = __ushort_as_half(scales[b]);
    const h2v sc = { s, s }, bias = { (_Float16)1032.f, (_Float16)1032.f };
    h2v lo[8], hi[8];
#pragma unroll
    for (int d = 0; d < 4; d++) {
      const uint32_t l = q[d] & 0x0F0F0F0Fu, h = (q[d] >> 4) & 0x0F0F0F0Fu;
      lo[2 * d] = gw_bytes(l, 0x04010400u, bias, sc); lo[2 * d + 1] = gw_bytes(l, 0x04030402u, bias, sc);
      hi[2 * d] = gw_bytes(h, 0x04010400u, bias, sc); hi[2 * d + 1] = gw_bytes(h, 0x04030402u, bias, sc);
    }
#pragma unroll
    for (int v = 0; v < 2; v++)
#pragma unroll
      for (int j = 0; j < 4; j++) { o[v][2 * j] = lo[4 * v + j][0]; o[v][2 * j + 1] = lo[4 * v + j][1]; o[2 + v][2 * j] = hi[4 * v + j][0]; o[2 + v][2 * j + 1] = hi[4 * v + j][1]; }
  } else if constexpr (KIND == PA_W_Q8_0) {
    const u4* src = (const u4*)((const unsigned char*)w + b * 32);
    const _Float16 s = __ushort_as_half(scales[b]);
    const h2v sc = { s, s }, bias = { (_Float16)1152.f, (_Float16)1152.f };
#pragma unroll
    for (int v = 0; v < 2; v++) {
      const u4 q = src[v];
#pragma unroll
      for (int d = 0; d < 4; d++) {
        const uint32_t x = q[d] ^ 0x80808080u;
        const h2v e0 = gw_bytes(x, 0x04010400u, bias, sc), e1 = gw_bytes(x, 0x04030402u, bias, sc);
        o[2 * v + d / 2][4 * (d & 1)] = e0[0]; o[2 * v + d / 2][4 * (d & 1) + 1] = e0[1];
        o[2 * v + d / 2][4 * (d & 1) + 2] = e1[0]; o[2 * v + d / 2][4 * (d & 1) + 3] = e1[1];
      }
    }
  } else {
    const f4* src = (const f4*)((const float*)w + b * 32);
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const f4 x0 = src[2 * v], x1 = src[2 * v + 1];
      o[v] = (h8){ (_Float16)x0[0], (_Float16)x0[1], (_Float16)x0[2], (_Float16)x0[3], (_Float16)x1[0], (_Float16)x1[1], (_Float16)x1[2], (_Float16)x1[3] };
    }
  }
  h8* dst = (h8*)(out + b * 32);
#pragma unroll
  for (int v = 0; v < 4; v++) dst[v] = o[v];
}

template <int TN>
static hipError_t launch_gemm16(const Gemm16Params& q, hipStream_t s) {
  const size_t lds = 2 * (size_t)(GW_COLS * GW_ROWB + 64 * TN * GW_ROWB);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_gemm16_kernel<TN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const dim3 grid((q.d_out + 64 * TN - 1) / (64 * TN), (q.n_cols + GW_COLS - 1) / GW_COLS);
  hipLaunchKernelGGL((pa_gemm16_kernel<TN>), grid, dim3(256), lds, s, q);
  return hipGetLastError();
}

// large chunks only: at least 512 columns, and enough 256-column x 128-row workgroups to give every CU one (below that
// the tiled kernel's 128 x 128 workgroups fill the chip better)
bool pa_gemm_wide_serves(const GemmParams& p, int n_cu) {
  if (p.n_cols < 512 || p.d_in < 128 || (p.x_stride & 7) != 0 || ((uintptr_t)p.x & 15) != 0) return false;
  if (p.d_in % GW_KS != 0) return false;
  const uint64_t wgs = (uint64_t)((p.n_cols + GW_COLS - 1) / GW_COLS) * ((p.d_out + 127) / 128);
  return wgs >= (uint64_t)(n_cu > 0 ? n_cu : 256);
}

// w16: staging for d_out x d_in halves (the caller's, 16-byte aligned)
hipError_t pa_launch_gemm_wide(const GemmParams& p, uint16_t* w16, int n_cu, hipStream_t s) {
  const size_t n_blocks = (size_t)p.d_out * (p.d_in / 32);
  const dim3 wgrid((unsigned)((n_blocks + 255) / 256));
  switch (p.kind) {
    case PA_W_Q4_0: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_Q4_0>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, n_blocks); break;
    case PA_W_Q8_0: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_Q8_0>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, n_blocks); break;
    case PA_W_F32: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_F32>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, n_blocks); break;
    default: return hipErrorInvalidValue;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  Gemm16Params q;
  q.x = p.x; q.w16 = w16; q.y = p.y; q.x_stride = p.x_stride; q.y_stride = p.y_stride;
  q.d_out = p.d_out; q.d_in = p.d_in; q.n_cols = p.n_cols; q.acc = p.acc;
  // rows per workgroup (64 TN): the choice that wastes the least of the chip -- rounds of n_cu workgroups, each
  // round costing its workgroups' rows
  const uint32_t cb = (p.n_cols + GW_COLS - 1) / GW_COLS, cus = n_cu > 0 ? (uint32_t)n_cu : 256u;
  uint32_t best_tn = 4; uint64_t best = ~0ull;
  for (uint32_t tn = 4; tn >= 2; tn--) {
    const uint64_t wgs = (uint64_t)((p.d_out + 64 * tn - 1) / (64 * tn)) * cb;
    const uint64_t cost = ((wgs + cus - 1) / cus) * (64 * tn) * (tn == 4 ? 16 : tn == 3 ? 17 : 19);   // smaller tiles pay more LDS traffic per MFMA
    if (cost < best) { best = cost; best_tn = tn; }
  }
  return best_tn == 4 ? launch_gemm16<4>(q, s) : best_tn == 3 ? launch_gemm16<3>(q, s) : launch_gemm16<2>(q, s);
}
