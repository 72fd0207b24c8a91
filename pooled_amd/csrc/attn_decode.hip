// Split-K flash-decoding attention for decode and speculative-verify passes on gfx950 (MI355X).
//
// Replaces the reference's attn_dec + attn_dec_combine(_g) + sigmoid_mul
// (engine/wgsl/attn_dec.js:102-287, engine/wgsl/qwen35.js:406-416).  Same outer shape -- one workgroup per
// (split of the context, kv head, column group), per-split (m, l, O) partials, a second-pass log-sum-exp
// merge -- with a CDNA4 inside:
//
//   * Every wavefront streams its own 32-position K/V tiles: 128-bit coalesced global loads (a 64-lane load
//     covers two whole 512-byte f16 rows; the caches are head-major, so a tile is one contiguous 16 KB block) into registers, the next tile's loads issued as soon as the current
//     tile's registers have been staged, so a wave always has ~32 KB in flight.
//   * Tiles are staged in a wave-private LDS region (no workgroup barrier in the loop): K rows are read back
//     as MFMA A-operands (ds_read_b128), V rows through the gfx950 LDS transpose read (ds_read_b64_tr_b16),
//     which delivers 4 positions x 1 dim per lane -- the contraction-major layout PV needs.
//   * S^T = K Q^T and O^T = V^T P^T run on v_mfma_f32_16x16x32_f16.  The S^T accumulator layout (lane =
//     query row, 4+4 positions) is exactly the B-operand layout of the PV product, so probabilities never
//     leave registers.  All G heads of a kv head and all columns of a verify block are rows of one tile, so
//     K/V are read once for the whole block.
//   * Softmax state (m, l) and O are f32; q and P are rounded to f16 for the MFMA operands, and l is the sum of the
//     rounded P (an output is a convex combination of value rows whatever that rounding did).
//   * Every reduction has a fixed order (lane-group shuffles, wave order, split order): run-to-run deterministic,
//     no atomics.
//
// Row r of a workgroup's tile is (local column r / G, head r % G); column c (absolute position base_pos + c)
// sees cache rows [0, base_pos + c].
#include "pa_internal.h"
#include "glue_math.h"

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef __fp16 hh4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

#define TILE 32

#define NEG_INF (-__builtin_inff())
#ifndef PA_V_LATE_MIN_WGS
#define PA_V_LATE_MIN_WGS 384u   // single-round splits: workgroups from which the V loads wait for the K scores
#endif
#define DEC_RESCALE_TH 8.f   // tile loop: a row maximum may pass the reference maximum by this much before O is rescaled

static __device__ inline h4 lds_read_tr16(const unsigned char* p) {
  hh4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16((hh4 __attribute__((address_space(3)))*)p);
  h4 r; __builtin_memcpy(&r, &t, 8); return r;
}

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// Exchanges between the four 16-lane rows of a wavefront on the VALU (gfx950 lane-swap instructions) instead of the LDS
// crossbar (ds_bpermute: a dependent round trip of ~100 clocks each, four of them on the critical path of every tile's
// softmax).  xrow16(v): lane i's own value and the value of lane i ^ 16; xrow32(v): the same for i ^ 32.  Both partners see
// the same pair, so a commutative combine gives both the same bits.
static __device__ inline void xrow16(float v, float& a, float& b) {
  const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(sw[0]); b = __uint_as_float(sw[1]);
}
static __device__ inline void xrow32(float v, float& a, float& b) {
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(sw[0]); b = __uint_as_float(sw[1]);
}
// maximum / sum over the four lanes {i, i ^ 16, i ^ 32, i ^ 48} (the four position groups of a query row), the same bits in all four
static __device__ inline float rows_max(float v) {
  float a, b;
  xrow16(v, a, b); v = fmaxf(a, b);
  xrow32(v, a, b); return fmaxf(a, b);
}
static __device__ inline float rows_sum(float v) {
  float a, b;
  xrow16(v, a, b); v = a + b;
  xrow32(v, a, b); return a + b;
}
// acc + the sum of eight f16 probabilities, as the numbers the PV product really uses (v_dot2_f32_f16 with ones: products
// exact, sums in f32): the row total l is then the total of the weights that were applied, so a row's output is a convex
// combination of value rows whatever the rounding of P did -- one visible row gives that row's bits back, constant
// values give the constant
static __device__ inline float sum_f16(const h8 pf, float acc) {
  const h2 ones = { (_Float16)1.f, (_Float16)1.f };
#pragma unroll
  for (int j = 0; j < 8; j += 2) { const h2 pp = { pf[j], pf[j + 1] }; acc = __builtin_amdgcn_fdot2(pp, ones, acc, false); }
  return acc;
}
// lane i's copy of lane (i + N) % 16 of its row of 16 (DPP row rotation)
template <int N>
static __device__ inline float row_ror(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x120 + N, 0xf, 0xf, false));
}
// maximum / sum over the 16 lanes {(i & 3) + 4 k} (LPG == 4; LPG == 8: the 8 lanes {(i & 7) + 8 k}): rotations inside the row, then the four rows.  The sum's
// association differs from lane to lane (lane i starts at its own element); lanes 0 .. 3 are the ones that are read.
template <int LPG = 4>
static __device__ inline float quads_max(float v) {
  if constexpr (LPG == 4) v = fmaxf(v, row_ror<4>(v));
  v = fmaxf(v, row_ror<8>(v));
  return rows_max(v);
}
template <int LPG = 4>
static __device__ inline float quads_sum(float v) {
  if constexpr (LPG == 4) v += row_ror<4>(v);
  v += row_ror<8>(v);
  return rows_sum(v);
}

// 16 int8 values x scale -> 16 f16 (see the Q8 note at the kernel)
static __device__ inline void dq16(const u4 raw, const float sc, h8& lo, h8& hi) {
  const h2 s2 = { (_Float16)sc, (_Float16)sc };
  const h2 off = { (_Float16)1152.f, (_Float16)1152.f };
  h2 o[8];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const uint32_t w = raw[d] ^ 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, w, 0x04010400u), b = __builtin_amdgcn_perm(0x64646464u, w, 0x04030402u);
    h2 xa, xb;
    __builtin_memcpy(&xa, &a, 4); __builtin_memcpy(&xb, &b, 4);
    o[2 * d] = (xa - off) * s2;
    o[2 * d + 1] = (xb - off) * s2;
  }
  lo = (h8){ o[0][0], o[0][1], o[1][0], o[1][1], o[2][0], o[2][1], o[3][0], o[3][1] };
  hi = (h8){ o[4][0], o[4][1], o[5][0], o[5][1], o[6][0], o[6][1], o[7][0], o[7][1] };
}

// What the f16 rounding of four q values drops, as f16: q = hi + lo to 2^-22 of q.  With at most eight live query rows
// in a 16-row block, rows 8 .. 15 of the q tile carry the low halves of rows 0 .. 7: the same MFMAs then also produce
// K q_lo^T (in the lanes of rows 8 .. 15), one row rotation adds it to K q_hi^T, and the scores see q at f32 precision --
// the rounding of q to f16 is otherwise the largest error of a decode wherever a few rows share the weight (short
// contexts, peaked scores).
static __device__ inline h4 q_lo_row(const f4 v, const h4 hi) {
  return (h4){ (_Float16)(v[0] - (float)hi[0]), (_Float16)(v[1] - (float)hi[1]), (_Float16)(v[2] - (float)hi[2]), (_Float16)(v[3] - (float)hi[3]) };
}

// Fused pre-step of N query heads of one wave (heads wave, wave + W, ...): norm + rope side by side, then the heads
// as f16 rows of the q tile.  xs: wave-private LDS scratch of N x HD floats.
template <int N, int HD, int W, int QROW>
static __device__ inline void fused_q_rows(const float (&xq)[16 / W][4], const float (&wq)[4], bool norm, float eps, uint32_t half,
                                           const float2 (&cs)[2], float* xs, unsigned char* q_lds, uint32_t G, uint32_t wave, uint32_t lane,
                                           bool qsplit) {
  static_assert(N <= 16 / W, "at most 16 query heads per kv head");
  float x[N][4];
#pragma unroll
  for (int n = 0; n < N; n++)
#pragma unroll
    for (int j = 0; j < 4; j++) x[n][j] = xq[n][j];
  if (glue_regs_serves(half)) {
    // the usual pair distances: norm and rotation in registers, the heads written as f16 rows element by element
    glue_heads_regs<N>(x, wq, norm, eps, HD, half, cs, lane);
#pragma unroll
    for (int n = 0; n < N; n++) {
      const uint32_t r = wave + W * n;
      if (r < G) {
#pragma unroll
        for (int j = 0; j < HD / 64; j++) {
          const _Float16 hi = (_Float16)x[n][j];
          *(_Float16*)(q_lds + r * QROW + (lane + 64 * j) * 2) = hi;
          if (qsplit) *(_Float16*)(q_lds + (r + 8) * QROW + (lane + 64 * j) * 2) = (_Float16)(x[n][j] - (float)hi);     // (see q_lo_row)
        }
      }
    }
    wave_lds_fence();
    return;
  }
  glue_heads_wave<N>(x, wq, norm, eps, HD, half, cs, xs, HD, lane);
#pragma unroll
  for (int n = 0; n < N; n++) {
    const uint32_t r = wave + W * n;
    if (r < G && lane < HD / 4) {
      const f4 v = *(const f4*)(xs + n * HD + 4 * lane);
      const h4 hv = { (_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3] };
      *(h4*)(q_lds + r * QROW + lane * 8) = hv;
      if (qsplit) *(h4*)(q_lds + (r + 8) * QROW + lane * 8) = q_lo_row(v, hv);
    }
  }
  wave_lds_fence();
}

template <int HD> struct DecShape {
  static constexpr int LPR = HD / 8;            // lanes per f16 row at 16 bytes a lane
  static constexpr int RPL = 64 / LPR;          // rows per wave-wide load
  static constexpr int NLD = TILE / RPL;        // loads per tile and tensor
  static constexpr int KROW = HD * 2 + 16;      // staged K row stride (bytes): 16 rows x 16 B hit distinct banks
  static constexpr int VROW = HD * 2 + 32;      // staged V row stride (bytes)
  static constexpr int STAGE = TILE * VROW;     // wave-private staging bytes (>= 16 x (HD + 4) floats for the merge)
  static constexpr int QROW = HD * 2 + 16;      // staged q row stride (bytes)
  static constexpr int OROW = (HD + 4) * 4;     // merge row stride (bytes)
  // int8 caches: 16 values a lane
  static constexpr int LPR8 = HD / 16;          // lanes per int8 row
  static constexpr int RPL8 = 64 / LPR8;        // rows per wave-wide load
  static constexpr int NLD8 = TILE / RPL8;      // loads per tile and tensor
  static constexpr int SPR = HD / 32;           // scales per row
  static constexpr int LPS = SPR / 4;           // lanes per row of scales at 16 bytes a lane
  static constexpr int KS = HD / 32;            // k-steps of the QK product
  static constexpr int DB = HD / 16;            // 16-dim blocks of the output
};

// FUSED: the workgroup also runs the pre-step of its kv head for the one column at base_pos (n_cols == 1, NB == 1,
// self_row set): its G query heads are normed and roped from the raw projection on the way into LDS, and wave 0 of
// split 0 norms / ropes the new key row and writes it and the value row to the cache.
//
// self_row (every one-column decode, fused or not, f16 or int8 caches): the column's own row base_pos is not streamed with
// rows 0 .. base_pos - 1; wave 0 of split 0 holds it in registers (from the pre-step above, or loaded), scores it
// against the G query rows and writes it as one more split partial: an (m, l) pair under every head, the O row (the value
// row, the same for the G heads) once, under the kv head's first head, where the merge kernel reads it for all of them.
//
// GATHER (the reference's attn_dec_qsa, engine/wgsl/attn_dec.js:33-38, :105, :170-183): each column attends to a
// list of cache rows instead of rows 0 .. seqLen - 1.  Column col's list is sel[col * sel_stride] = n, then n row
// indices (ascending) at sel[col * sel_stride + 1 ..].  List position t stands where position t stands in the dense
// kernel: splits, tiles and masks are taken over list positions, only the K/V loads go through the list.  One
// column per workgroup (grid z = column, NB == 1), since the lists differ between columns.
//
// Q8 (the reference's kvQ8 caches read by attn_flash_q8, engine/wgsl/qwen35.js:99-139): K and V rows are int8 with one
// f32 scale per 32 values.  Only the way a tile gets into LDS differs: a lane loads 16 values (16 bytes) and the
// tile's scales (one 16-byte load), the scales make a round trip through the staging region so that every lane can
// pick the scale of each of its 16-value pieces, and the pieces are widened to f16 on their way into the staged
// tile -- int8 -> f16 through the 0x6400 | (v + 128) bit pattern (= 1152 + v exactly), a packed subtract and a
// packed multiply by the f16-rounded scale.  From there on (MFMA, softmax, merge) it is the f16 kernel.
//
// SR (single-round splits; one 16-row block, or two of a verify block): splits are one tile per wave (split_len = W x
// 32); the product O^T = V^T P^T of a split is divided over the waves by output dims, see the code.  Without SR every wave
// loops over its own tiles: contiguous splits of any length, or (AttnParams::tile_ilv) a kv head's tiles dealt round robin
// to the waves of all its splits.
template <int HD, int NB, int W, bool FUSED, bool GATHER, bool Q8, bool SR>
__global__ __launch_bounds__(W * 64, ((NB == 1 && !GATHER && W <= 4) || (SR && NB == 2 && HD == 128) ? 2 : 1))
void pa_decode_kernel(const uint16_t* a_k_cache, uint32_t a_base_pos, uint32_t a_max_seq, uint32_t a_n_splits, uint32_t a_self_row,
                      uint32_t a_grid_x, const float* a_f_q_in, uint32_t a_group, uint32_t a_f_q_head_stride, AttnParams p_in) {
  // The leading arguments repeat fields of p_in: the first twelve dwords of a kernel's arguments are preloaded into
  // scalar registers by the dispatcher (-amdgpu-kernarg-preload-count), so what the first tile loads' addresses are made
  // of is there when the wave starts instead of a scalar-load round trip later.
  AttnParams p = p_in;
  p.k_cache = a_k_cache; p.base_pos = a_base_pos; p.max_seq = a_max_seq; p.n_splits = a_n_splits; p.self_row = a_self_row & 1u;
  const bool cols_adjacent = (a_self_row & 2u) != 0;                 // (rides in a preloaded argument: see the workgroup mapping below)
  p.f_q_in = a_f_q_in; p.group = a_group; p.f_q_head_stride = a_f_q_head_stride;
  const uint32_t grid_x = a_grid_x;
  static_assert(!SR || NB == 1 || (NB == 2 && W == 4 && !FUSED && !GATHER), "single-round splits: one 16-row block, or two of a verify block");
  static_assert(!FUSED || NB == 1, "the fused pre-step serves one column");
  static_assert(!GATHER || (NB == 1 && !FUSED), "the gather mode serves one column per workgroup");
  static_assert(!Q8 || !GATHER, "int8 caches: no gather mode");
  typedef DecShape<HD> S;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* q_lds = smem;                                       // [16*NB][QROW]
  unsigned char* stage_all = smem + 16 * NB * S::QROW;               // [W][STAGE]
  float* mex = (float*)(stage_all + W * S::STAGE);                   // [W][16*NB]
  float* lex = mex + W * 16 * NB;                                    // [W][16*NB]
  float* sct = lex + W * 16 * NB;                                    // [W][16*NB]: the tile loop's merge, a wave's weight exp(m_w - M) per row
  uint32_t* rowcol = (uint32_t*)(sct + W * 16 * NB);                 // [16*NB]: the column of a stacked row ...
  uint32_t* rowhq = rowcol + 16 * NB;                                // [16*NB]: ... and its query head (same merge)
  unsigned char* p_lds = (unsigned char*)(rowhq + 16 * NB);          // [W][NB][64 x 16 B]: the tiles' P, single-round kernel with two row blocks

  uint32_t bx = blockIdx.x, by = blockIdx.y, cg = blockIdx.z;
  if constexpr (SR && !FUSED && !GATHER) {
    // A column-exact verify block in one launch (every column a column group of its own, all streaming the same rows):
    // dispatch id i runs on XCD i % 8, and XCD k takes the (split, kv head) items k, k + 8, ... with the columns of an
    // item on consecutive ids of that XCD, so that they run side by side and share the rows in its L2.  (The items past
    // the last multiple of eight come last, a column after the other.)
    if (__builtin_expect(cols_adjacent, 0)) {
      const uint32_t items = grid_x * gridDim.y, ncols = gridDim.z, items8 = items & ~7u;
      const uint32_t lin = bx + grid_x * (by + gridDim.y * cg);
      uint32_t item;
      if (lin < items8 * ncols) { const uint32_t k = lin % 8, j = lin / 8; item = (j / ncols) * 8 + k; cg = j % ncols; }
      else { const uint32_t e = lin - items8 * ncols; item = items8 + e / ncols; cg = e % ncols; }
      bx = item % grid_x; by = item / grid_x;
    }
  }
  uint32_t sp = bx, g = by;                                          // SR: the grid's own coordinates
  if constexpr (!SR) {
    // Tile loop: a one-dimensional grid over (kv head, split, column group) items, column group fastest.  Dispatch
    // id i runs on XCD i % 8 and XCD k owns the contiguous item range [k per, (k + 1) per): the column groups of a
    // (kv head, split) read the same K/V rows, so they sit on one XCD, side by side, and share the rows in its L2
    // whatever the number of splits.
    const uint32_t ncg = p.col_groups;
    const uint32_t total = p.n_splits * p.n_kv_heads * ncg, per = (total + 7) / 8;
    const uint32_t item = (blockIdx.x % 8) * per + blockIdx.x / 8;
    if (item >= total) return;
    // floor(n / d) = mulhi(n, ceil(2^32 / d)) while n d < 2^32 (the launcher checks): the first tile's addresses wait for these
    const uint32_t q1 = p.ncg_magic ? __umulhi(item, p.ncg_magic) : (ncg == 1 ? item : item / ncg);
    const uint32_t q2 = p.ns_magic ? __umulhi(q1, p.ns_magic) : (p.n_splits == 1 ? q1 : q1 / p.n_splits);
    cg = item - q1 * ncg; sp = q1 - q2 * p.n_splits; g = q2;
  }
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t ln = lane & 15, kg = lane >> 4;
  const uint32_t G = p.group, nH = p.n_heads;
  // row r of the stacked tile is (column r / G, head r % G): the quotient as a multiply and a shift (exact for r < 1024 and
  // G <= 64; a division by a run-time G is some thirty instructions, and the q loads' addresses wait for four of them a row block)
  const uint32_t g_magic = (65536u + G - 1u) / G;
  auto div_g = [&](uint32_t r) __attribute__((always_inline)) -> uint32_t { return (r * g_magic) >> 16; };
  const uint32_t c0 = FUSED ? 0u : cg * p.cols_per_group;            // (the fused step serves one column)
  const uint32_t ncl = FUSED ? 1u : min(p.cols_per_group, p.n_cols - c0);
  const uint32_t R = ncl * G;                                        // live rows (<= 16*NB)
  const uint32_t sel_base = GATHER ? c0 * p.sel_stride + 1 : 0;      // gather: first list entry of this column
  // rows visible to the group's last column (gather: the column's list length)
  // self_row (one-column decode): the column's own row base_pos is not streamed with the others -- see below
  const uint32_t seq_max = GATHER ? min(p.sel[c0 * p.sel_stride], p.sel_max) : p.base_pos + c0 + ncl - p.self_row;
  // rows 8 .. 15 of the q tile hold the low halves of rows 0 .. 7 (q_lo_row): every one-column decode with G <= 8, and
  // blocks of at most eight stacked rows
  const bool qsplit = NB == 1 && R <= 8;
  const uint32_t split_len = SR ? (uint32_t)(W * TILE) : p.split_len;   // single-round splits: one tile per wave
  // TILV (tile loop on a contiguous cache, p.tile_ilv): the tiles of a kv head are dealt round robin to the waves of
  // all its splits -- wave v of the n_splits x W takes tiles v, v + n_splits W, ... -- so the loads in flight on the chip
  // sweep one compact window of the cache per kv head instead of n_splits separate streams a split length apart, and
  // every split has the same number of tiles to within one.  Any partition of the rows is a valid set of splits.
  const bool tilv = !SR && !GATHER && p.tile_ilv;
  const uint32_t t_begin = sp * (tilv ? (uint32_t)(W * TILE) : split_len);
  // The workgroup of split 0 turns the column's own row into a partial of its own (wave 0, while the tile loads are
  // in flight), so it runs even when no other row exists (base_pos == 0).
  const bool self_wg = !GATHER && p.self_row && sp == 0;
  if (t_begin >= seq_max && !self_wg) return;
  const bool has_rows = t_begin < seq_max;
  // the last split of contiguous splits is open-ended: a splits override or a gather list may leave it a remainder
  const uint32_t t_end = (!SR && sp + 1 == p.n_splits) || tilv ? seq_max : min(t_begin + split_len, seq_max);
  const size_t head_rows = (size_t)p.max_seq + TILE;              // rows of one kv head's plane, padding included
  // SR: the whole splits of a kv head are interleaved.  With nw = (whole splits) x W waves, wave v of
  // them takes rows [(c nw + v) 8, + 8), c = 0 .. 3, instead of 32 consecutive ones: at any moment the loads in
  // flight on the chip then sweep a compact range of the cache (4 KB pieces, neighbouring waves on neighbouring
  // pieces) instead of 2048 separate 32 KB streams -- the memory controllers see open pages.  Measured on read-only
  // stand-ins of this launch shape: 11.9 -> 11.2 us for 64 MiB.  Any partition of the rows is a valid set of
  // splits; masks go by position.  A trailing partial split keeps consecutive rows.
  constexpr bool ILV = SR && !GATHER;
  uint32_t ilv_nw = 0, ilv_wv = 0;
  bool ilv = false;
  if constexpr (ILV) {
    const uint32_t nfull = min(p.n_splits, seq_max / split_len);
    ilv = sp < nfull;
    ilv_nw = nfull * W;
    ilv_wv = sp * W + (threadIdx.x >> 6);
  }
  // cache row of row r (0 .. 31) of the tile at tile_pos
  auto row_pos = [&](uint32_t tile_pos, uint32_t r) __attribute__((always_inline)) -> uint32_t {
    return ILV && ilv ? (((r >> 3) * ilv_nw + ilv_wv) << 3) + (r & 7) : tile_pos + r;
  };

  unsigned char* stage = stage_all + wave * S::STAGE;
  const size_t row_bytes = (size_t)HD * 2;                         // head-major caches: a kv head's rows are contiguous
  const uint32_t lrow = lane / S::LPR;
  // per-lane byte offset inside a wave-wide load; the tile base below is wave-uniform (scalar registers)
  const uint32_t voff = lrow * (uint32_t)row_bytes + (lane % S::LPR) * 16;
  const unsigned char* kbase = (const unsigned char*)(p.k_cache + (size_t)g * head_rows * HD);
  const unsigned char* vbase = (const unsigned char*)(p.v_cache + (size_t)g * head_rows * HD);
  // int8 caches: rows of HD bytes, scales of SPR floats per row
  const uint32_t lrow8 = lane / S::LPR8, voff8 = lrow8 * HD + (lane % S::LPR8) * 16;
  const uint32_t srow = min(lane / S::LPS, (uint32_t)TILE - 1), soff = srow * S::SPR * 4 + (lane % S::LPS) * 16;
  const unsigned char* kbase8 = (const unsigned char*)p.k_cache + (size_t)g * head_rows * HD;
  const unsigned char* vbase8 = (const unsigned char*)p.v_cache + (size_t)g * head_rows * HD;
  const unsigned char* ksbase = (const unsigned char*)(p.k_scale + (Q8 ? (size_t)g * head_rows * S::SPR : 0));
  const unsigned char* vsbase = (const unsigned char*)(p.v_scale + (Q8 ? (size_t)g * head_rows * S::SPR : 0));
  u4 ksr = {0u, 0u, 0u, 0u}, vsr = {0u, 0u, 0u, 0u};

  const uint32_t n_tiles = has_rows ? (t_end - t_begin + TILE - 1) / TILE : 0;      // (TILV: tiles from the split's first one to the end)
  const uint32_t tp_step = tilv ? p.n_splits * (uint32_t)(W * TILE) : (uint32_t)(W * TILE);   // from a wave's tile to its next one
  u4 kr[S::NLD], vr[S::NLD];
  const u4 zero4 = {0u, 0u, 0u, 0u};
  uint32_t tile = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t t0 = t_begin + min(tile, max(n_tiles, 1u) - 1) * TILE;
  // Fused single-round step: the first three eighths of the K tile loads go out ahead of the raw projection / weight
  // loads, as soon as the first kernel arguments are in: the K/V stream starts half a microsecond earlier.  The small
  // rows return behind them (loads of a wave complete in order), which is free as long as they are back before the
  // wave has pushed the rest of its K loads through the memory pipeline: measured on the 32K step, 6 of 16 loads ahead
  // 17.81 -> 17.63 us; 8 ahead 17.4 or 17.9 us from one process to the next; 10, 12, 16 ahead 18.1 - 18.8 us.
  constexpr int KF = SR && FUSED && !GATHER && !Q8 ? 3 * S::NLD / 8 : 0;
  if constexpr (KF > 0) {
#pragma unroll
    for (int i = 0; i < KF; i++) kr[i] = *(const u4*)(kbase + (size_t)row_pos(t0, i * S::RPL) * row_bytes + voff);
    __builtin_amdgcn_sched_barrier(0);
  }
  // Every other kernel argument the loads of the first microsecond need, fetched in one batch of scalar loads: left
  // alone, the compiler fetches arguments where they are first used, four dependent round trips before the first tile
  // load (measured on the 32K step: 17.62 -> 17.27 us).  (The arguments of the first tile loads are preloaded.)
  if constexpr (FUSED) {
    asm volatile("" :: "s"(p.v_cache), "s"(p.f_qw), "s"(p.rope_tab), "s"(p.n_rot));
  } else if constexpr (GATHER) {
    asm volatile("" :: "s"(p.q), "s"(p.v_cache), "s"(p.q_stride), "s"(p.n_heads), "s"(p.n_cols),
                 "s"(p.split_len), "s"(p.cols_per_group), "s"(p.sel), "s"(p.sel_stride), "s"(p.sel_max));
  } else {
    asm volatile("" :: "s"(p.q), "s"(p.v_cache), "s"(p.q_stride), "s"(p.n_heads), "s"(p.n_cols), "s"(p.split_len), "s"(p.cols_per_group));
    if constexpr (Q8) asm volatile("" :: "s"(p.k_scale), "s"(p.v_scale));
  }

  // the column's own K / V row, 4 dims a lane: loaded here (the pre-step wrote it), or made below by the fused pre-step
  const bool self_wave = self_wg && wave == 0;
  h4 kx = {0, 0, 0, 0}, vx = {0, 0, 0, 0};
  if constexpr (!FUSED && !GATHER && !Q8) {
    if (self_wave) {
      const size_t ro = (size_t)(p.base_pos + c0) * row_bytes + min(lane, (uint32_t)HD / 4 - 1) * 8;
      kx = *(const h4*)(kbase + ro);
      vx = *(const h4*)(vbase + ro);
    }
  }
  if constexpr (Q8 && !FUSED) {         // int8 row: widened as the tile path widens it (exact integer x f16-rounded scale, one rounding)
    if (self_wave) {
      const uint32_t l4 = min(lane, (uint32_t)HD / 4 - 1);
      const size_t ro = (size_t)(p.base_pos + c0) * HD + 4 * l4, so = ((size_t)(p.base_pos + c0) * S::SPR + l4 / 8) * 4;
      const uint32_t kq = *(const uint32_t*)(kbase8 + ro), vq = *(const uint32_t*)(vbase8 + ro);
      const _Float16 ksc = (_Float16)*(const float*)(ksbase + so), vsc = (_Float16)*(const float*)(vsbase + so);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        kx[i] = (_Float16)(int)(signed char)(kq >> (8 * i)) * ksc;
        vx[i] = (_Float16)(int)(signed char)(vq >> (8 * i)) * vsc;
      }
    }
  }
  // q loads first (they return first), then the first tile's K/V loads; staging q below overlaps the K/V latency.
  constexpr int QPT = 16 * NB * (HD / 4) / (W * 64);               // float4 of q per thread
  constexpr int HPW = 16 / W;                                      // fused: query heads per wave (G <= 16)
  f4 qv[FUSED ? 1 : QPT];
  float xq[FUSED ? HPW : 1][4], xk[4], wq[4], wk[4];
  f4 xv4 = {0.f, 0.f, 0.f, 0.f};
  float2 cs[2] = { make_float2(1.f, 0.f), make_float2(1.f, 0.f) };
  const uint32_t half = FUSED ? p.n_rot / 2 : 0;
  if constexpr (FUSED) {
    // Only what the wave uses is requested (wave-uniform conditions): its own query heads -- not the clamped duplicates of
    // head G - 1 --, and the new key / value row and the key weights in the one wave that makes the cache row.  Every wave
    // of the chip asks for these small rows in the same first microsecond, through the same L1s that then carry the K/V
    // stream; the K tile loads queue behind them.
#pragma unroll
    for (int t = 0; t < HPW; t++) {
#pragma unroll
      for (int j = 0; j < 4; j++) xq[t][j] = 0.f;
      if (wave + W * t < G) {
        const uint32_t h = g * G + wave + W * t;
#pragma unroll
        for (int j = 0; j < 4; j++) xq[t][j] = p.f_q_in[(size_t)h * p.f_q_head_stride + min(lane + 64 * j, (uint32_t)HD - 1)];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t i = min(lane + 64 * j, (uint32_t)HD - 1);
      wq[j] = p.f_qw ? p.f_qw[i] : 1.f;
      xk[j] = 0.f; wk[j] = 1.f;
    }
    if (self_wave) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t i = min(lane + 64 * j, (uint32_t)HD - 1);
        xk[j] = p.f_k_in[(size_t)g * HD + i];
        if (p.f_kw) wk[j] = p.f_kw[i];
      }
      xv4 = *(const f4*)(p.f_v_in + (size_t)g * HD + 4 * min(lane, (uint32_t)HD / 4 - 1));
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t i = lane + 64 * j;
      // (half == 32: every lane holds the pair lane & 31 -- the in-register rotation reads it in the upper lanes too;
      // pairs 64 .. 127 exist only with more than 64 pairs)
      if (half > 64u * j) cs[j] = rope_pair(p.rope_tab, p.inv_freq, p.base_pos, half, half == 32 ? i & 31 : min(i, half - 1));
    }
#pragma unroll
    for (int t = 0; t < HPW; t++)
#pragma unroll
      for (int j = 0; j < 4; j++) if (lane + 64 * j >= HD) xq[t][j] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) if (lane + 64 * j >= HD) xk[j] = 0.f;
  } else {
#pragma unroll
    for (int j = 0; j < QPT; j++) {
      const uint32_t e = tid + j * W * 64;
      const uint32_t r = e / (HD / 4), d4 = e % (HD / 4);
      const uint32_t rc = min(qsplit && r >= 8 ? r - 8 : r, R - 1);  // padding rows copy the last live row (masked out later)
      const uint32_t qc = div_g(rc);
      qv[j] = *(const f4*)(p.q + (size_t)(c0 + qc) * p.q_stride + (size_t)(g * G + rc - qc * G) * HD + 4 * d4);
    }
  }
  // Loads are unconditional: the caches carry TILE rows of padding past max_seq, so a tile that straddles the
  // end of the context reads valid memory; rows at or past t_end are zeroed (V) or masked (scores) below.
  // A wave with no tile of its own (short splits) loads the split's last tile and discards it: the prologue
  // stays branch-free, so the q staging below waits for the q loads only.
  // gather: byte offsets of this lane's rows of a tile, through the list (positions at or past the list's end take
  // its last row: valid memory, masked or zeroed like any row past t_end)
  uint32_t goff[GATHER ? S::NLD : 1];
  auto gather_offsets = [&](uint32_t tpos) {
    if constexpr (GATHER) {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) {
        const uint32_t li = min(tpos + i * S::RPL + lrow, seq_max - 1);
        goff[i] = min(p.sel[sel_base + li], p.max_seq - 1);      // a bad index must not leave the cache
      }
    }
  };
  if constexpr (GATHER) {
    gather_offsets(t0);
#pragma unroll
    for (int i = 0; i < S::NLD; i++) kr[i] = *(const u4*)(kbase + (size_t)goff[i] * row_bytes + (lane % S::LPR) * 16);
  } else if constexpr (Q8) {
#pragma unroll
    for (int i = 0; i < S::NLD8; i++) kr[i] = *(const u4*)(kbase8 + (size_t)row_pos(t0, i * S::RPL8) * HD + voff8);   // a load's rows share an 8-row piece
    ksr = *(const u4*)(ksbase + (size_t)row_pos(t0, srow) * S::SPR * 4 + (lane % S::LPS) * 16);
  } else {
#pragma unroll
    for (int i = KF; i < S::NLD; i++) kr[i] = *(const u4*)(kbase + (size_t)row_pos(t0, i * S::RPL) * row_bytes + voff);
  }
  auto first_v_loads = [&]() __attribute__((always_inline)) {
    if constexpr (GATHER) {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) vr[i] = *(const u4*)(vbase + (size_t)goff[i] * row_bytes + (lane % S::LPR) * 16);
    } else if constexpr (Q8) {
#pragma unroll
      for (int i = 0; i < S::NLD8; i++) vr[i] = *(const u4*)(vbase8 + (size_t)row_pos(t0, i * S::RPL8) * HD + voff8);
      vsr = *(const u4*)(vsbase + (size_t)row_pos(t0, srow) * S::SPR * 4 + (lane % S::LPS) * 16);
    } else {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) vr[i] = *(const u4*)(vbase + (size_t)row_pos(t0, i * S::RPL) * row_bytes + voff);
    }
  };
  // The fused pre-step computes between the K and the V loads: a wave sits in the issue of its tile loads for
  // microseconds (the memory pipeline is full), so arithmetic placed after all of them starts that much later, while
  // the K requests already queued keep the pipeline fed during the arithmetic.
  // V_LATE (single-round splits): the V loads go out only after the K tile has been scored.  A wave cannot compute while
  // it sits in the issue of its loads (the CU's memory pipeline accepts a load as an older one completes: 1 - 2 us for
  // 16 loads once the chip is streaming), so with K and V requested back to back the last waves' K tiles -- long since
  // arrived -- waited for the V issue to end, and staging, scores and softmax of K (1.1 us) came on top of the V work at
  // the very end of the kernel.  Scored first, that work runs while other waves keep the pipeline full, and what follows
  // the last V load is the V latency, the staging of V and the PV product.  Measured on the 32K decode step: 18.6 -> 18.15 us.
  constexpr bool V_LATE = SR && !GATHER;
  // ... when the chip is streaming.  With fewer workgroups than two a CU the memory pipeline is never full, the loads
  // of a wave are accepted at once, and V behind the scores is one more HBM round trip at the end: then V goes out with K.
  const bool v_late = V_LATE && gridDim.x * gridDim.y * gridDim.z >= PA_V_LATE_MIN_WGS;
  if (!FUSED && !v_late) first_v_loads();
  __builtin_amdgcn_sched_barrier(0);   // nothing below may be scheduled above the load issue
  // ---- q -> f16 rows in LDS; waits only for the q loads, which were issued first ----
  if constexpr (FUSED) {
    float* xs = (float*)stage;       // wave-private scratch (the staging region is not in use yet)
    // this wave's query heads wave, wave + W, ... side by side (ceil(G / W) of them; one past G is computed and dropped)
    switch ((G + W - 1) / W) {
      case 1: fused_q_rows<1, HD, W, S::QROW>(xq, wq, p.f_qw != nullptr, p.eps, half, cs, xs, q_lds, G, wave, lane, qsplit); break;
      case 2: fused_q_rows<2, HD, W, S::QROW>(xq, wq, p.f_qw != nullptr, p.eps, half, cs, xs, q_lds, G, wave, lane, qsplit); break;
      case 3: if constexpr (W <= 4) fused_q_rows<3, HD, W, S::QROW>(xq, wq, p.f_qw != nullptr, p.eps, half, cs, xs, q_lds, G, wave, lane, qsplit); break;
      default: if constexpr (W <= 4) fused_q_rows<4, HD, W, S::QROW>(xq, wq, p.f_qw != nullptr, p.eps, half, cs, xs, q_lds, G, wave, lane, qsplit); break;
    }
    for (uint32_t e = tid; e < (16 - G) * (HD / 4); e += W * 64) {   // padding rows (masked out later)
      const uint32_t row = G + e / (HD / 4);
      if (!(qsplit && row - 8 < G)) *(h4*)(q_lds + row * S::QROW + (e % (HD / 4)) * 8) = (h4){0, 0, 0, 0};    // (rows 8 .. 8 + G - 1: the low halves)
    }
    if (self_wave) {                 // the new key row: normed, roped, rounded; it and the value row go to the cache
      glue_head_wave(xk, wk, p.f_kw != nullptr, p.eps, HD, half, cs, xs, lane);
      if constexpr (Q8) {
        // int8 caches: both rows quantised as the stand-alone pre-step does (same bits), written with their scales,
        // and kept as the widened values the tile path would read back
        const bool on = lane < HD / 4;
        float kq[4] = {0.f, 0.f, 0.f, 0.f}, vq[4] = {0.f, 0.f, 0.f, 0.f};
        if (on) { const f4 v = *(const f4*)(xs + 4 * lane); kq[0] = v[0]; kq[1] = v[1]; kq[2] = v[2]; kq[3] = v[3]; vq[0] = xv4[0]; vq[1] = xv4[1]; vq[2] = xv4[2]; vq[3] = xv4[3]; }
        uint32_t kw8, vw8; float ksc, vsc;
        quant4_q8(kq, kw8, ksc);
        quant4_q8(vq, vw8, vsc);
        if (on) {
          const size_t row = (size_t)g * head_rows + p.base_pos;
          *(uint32_t*)((unsigned char*)const_cast<uint16_t*>(p.k_cache) + row * HD + 4 * lane) = kw8;
          *(uint32_t*)((unsigned char*)const_cast<uint16_t*>(p.v_cache) + row * HD + 4 * lane) = vw8;
          if ((lane & 7) == 0) {
            const_cast<float*>(p.k_scale)[row * S::SPR + (lane >> 3)] = ksc;
            const_cast<float*>(p.v_scale)[row * S::SPR + (lane >> 3)] = vsc;
          }
        }
        const _Float16 ks16 = (_Float16)ksc, vs16 = (_Float16)vsc;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          kx[i] = (_Float16)(int)(signed char)(kw8 >> (8 * i)) * ks16;
          vx[i] = (_Float16)(int)(signed char)(vw8 >> (8 * i)) * vs16;
        }
      } else if (lane < HD / 4) {
        const f4 v = *(const f4*)(xs + 4 * lane);
        kx = (h4){ (_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3] };
        vx = (h4){ (_Float16)xv4[0], (_Float16)xv4[1], (_Float16)xv4[2], (_Float16)xv4[3] };
        const size_t ro = ((size_t)g * head_rows + p.base_pos) * HD + 4 * lane;
        *(h4*)((_Float16*)const_cast<uint16_t*>(p.k_cache) + ro) = kx;
        *(h4*)((_Float16*)const_cast<uint16_t*>(p.v_cache) + ro) = vx;
      }
      wave_lds_fence();
    }
  } else {
#pragma unroll
    for (int j = 0; j < QPT; j++) {
      const uint32_t e = tid + j * W * 64;
      const uint32_t r = e / (HD / 4), d4 = e % (HD / 4);
      const h4 hv = { (_Float16)qv[j][0], (_Float16)qv[j][1], (_Float16)qv[j][2], (_Float16)qv[j][3] };
      *(h4*)(q_lds + r * S::QROW + d4 * 8) = qsplit && r >= 8 ? q_lo_row(qv[j], hv) : hv;
    }
  }
  if (FUSED && !v_late) {
    __builtin_amdgcn_sched_barrier(0);
    first_v_loads();
    __builtin_amdgcn_sched_barrier(0);
  }
  // per-lane row bookkeeping: row nb*16 + ln ends (exclusive) at end_pos[nb]; 0 for padding rows
  uint32_t end_pos[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const uint32_t r = nb * 16 + ln;
    end_pos[nb] = r < R ? (GATHER ? seq_max : p.base_pos + c0 + div_g(r) + 1 - p.self_row) : 0u;
  }
  __syncthreads();
  // ---- the column's own row as a partial of its own (slot = number of splits that hold rows): m = its score,
  // l = 1, O = its value row.  The scores run on the VALU over the f16 operands the MFMA path would see, f32 sums in a
  // fixed order; the work hides under the latency of the tile loads.  Decoding a token at a position that is a
  // multiple of the split length therefore streams whole tiles only.
  if (self_wave) {
    const uint32_t live_len = tilv ? (uint32_t)(W * TILE) : split_len;     // rows from one split's first row to the next one's
    const uint32_t self_slot = min((seq_max + live_len - 1) / live_len, p.n_splits);
    const bool on = lane < HD / 4;
    const f4 vxf = { (float)vx[0], (float)vx[1], (float)vx[2], (float)vx[3] };
    // No store inside the loop: while the chip streams, the memory pipeline accepts a store as slowly as a load, and
    // with a partial row and an (m, l) pair stored per head this one wave -- the last of the kernel to start on its tile
    // -- ran microseconds behind the rest and set the end of the kernel.  The G heads of a kv head share the value row, so
    // it is stored once, under the kv head's first head (the merge reads it there for every head), up front; lane r keeps
    // head r's score and the G (m, l) pairs leave in one store behind the loop.
    const size_t slot0 = ((size_t)c0 * nH + g * G) * p.slots + self_slot;
    if (on) {
      if (p.part_f16) *(h4*)((_Float16*)p.part_o + slot0 * HD + 4 * lane) = vx;
      else *(f4*)(p.part_o + slot0 * HD + 4 * lane) = vxf;
    }
    float dv = 0.f;
    for (uint32_t r = 0; r < G; r++) {                                 // one column: row r is head g * G + r
      const h4 qv = *(const h4*)(q_lds + r * S::QROW + min(lane, (uint32_t)HD / 4 - 1) * 8);
      h4 ql = {0, 0, 0, 0};
      if (qsplit) ql = *(const h4*)(q_lds + (r + 8) * S::QROW + min(lane, (uint32_t)HD / 4 - 1) * 8);
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < 4; i++) d = __builtin_fmaf((float)qv[i] + (float)ql[i], (float)kx[i], d);
      if (!on) d = 0.f;
      d = wave_sum_f32(d);
      if (lane == r) dv = d;
    }
    if (lane < G) *(float2*)(p.part_ml + (slot0 + (size_t)lane * p.slots) * 2) = make_float2(dv * p.scale, 1.f);
  }
  if (!has_rows) return;

  // The three staging / product steps of a tile, shared by the tile loop and the single-round path below.
  // stage_k: the K registers of the tile at position tp -> LDS (int8: widened), then the loads of the wave's next tile.
  auto stage_k = [&](const uint32_t tp, const bool more, const uint32_t tpn) __attribute__((always_inline)) {
    const size_t tnb = (size_t)tpn * row_bytes;               // next tile of this wave
    if constexpr (Q8) {
      if (lane / S::LPS < TILE) *(u4*)(stage + soff) = ksr;          // the tile's scales, [row][SPR] f32
      wave_lds_fence();
      float sc[S::NLD8];
#pragma unroll
      for (int i = 0; i < S::NLD8; i++) sc[i] = *(const float*)(stage + ((i * S::RPL8 + lrow8) * S::SPR + (lane % S::LPR8) / 2) * 4);
      wave_lds_fence();                                              // read before the tile overwrites the region
#pragma unroll
      for (int i = 0; i < S::NLD8; i++) {
        h8 lo, hi;
        dq16(kr[i], sc[i], lo, hi);
        unsigned char* d = stage + (i * S::RPL8 + lrow8) * S::KROW + (lane % S::LPR8) * 32;
        *(h8*)d = lo; *(h8*)(d + 16) = hi;
      }
      if (more) {
        const size_t tb = (size_t)tpn * HD;
#pragma unroll
        for (int i = 0; i < S::NLD8; i++) kr[i] = *(const u4*)(kbase8 + tb + (size_t)(i * S::RPL8) * HD + voff8);
        ksr = *(const u4*)(ksbase + (size_t)tpn * S::SPR * 4 + soff);
      }
    } else {
#pragma unroll
    for (int i = 0; i < S::NLD; i++) *(u4*)(stage + (i * S::RPL + lrow) * S::KROW + (lane % S::LPR) * 16) = kr[i];
    }
    if (!Q8 && more) {
      if constexpr (GATHER) {
        gather_offsets(tpn);
#pragma unroll
        for (int i = 0; i < S::NLD; i++) kr[i] = *(const u4*)(kbase + (size_t)goff[i] * row_bytes + (lane % S::LPR) * 16);
      } else {
#pragma unroll
        for (int i = 0; i < S::NLD; i++) kr[i] = *(const u4*)(kbase + tnb + (size_t)(i * S::RPL) * row_bytes + voff);
      }
    }
    wave_lds_fence();
  };
  // qk: S^T = K Q^T of the staged tile
  auto qk = [&](f4 (&s)[2][NB]) __attribute__((always_inline)) {
#pragma unroll
    for (int nb = 0; nb < NB; nb++) { s[0][nb] = (f4){0.f, 0.f, 0.f, 0.f}; s[1][nb] = (f4){0.f, 0.f, 0.f, 0.f}; }
    {
      // fragments are fetched FD k-steps ahead of the MFMAs that use them, and the issue order is pinned: left to
      // itself the compiler waits for each k-step's three LDS reads right before its MFMAs, one LDS latency a step
      constexpr int FD = HD == 256 ? (SR ? 4 : 1) : 3;     // the single-round kernel has the registers for four k-steps of fragments in flight
      h8 a0r[FD], a1r[FD], br[FD][NB];
      auto fetch = [&](int ks, int slot) __attribute__((always_inline)) {
        a0r[slot] = *(const h8*)(stage + ln * S::KROW + ks * 64 + kg * 16);
        a1r[slot] = *(const h8*)(stage + (16 + ln) * S::KROW + ks * 64 + kg * 16);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) br[slot][nb] = *(const h8*)(q_lds + (nb * 16 + ln) * S::QROW + ks * 64 + kg * 16);
      };
#pragma unroll
      for (int ks = 0; ks < FD; ks++) fetch(ks, ks);
#pragma unroll
      for (int ks = 0; ks < S::KS; ks++) {
        const h8 a0 = a0r[ks % FD], a1 = a1r[ks % FD];
        h8 b[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) b[nb] = br[ks % FD][nb];
        if (ks + FD < S::KS) fetch(ks + FD, ks % FD);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
          s[0][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b[nb], s[0][nb], 0, 0, 0);
          s[1][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b[nb], s[1][nb], 0, 0, 0);
        }
      }
#pragma unroll
      for (int ks = 0; ks < FD; ks++) __builtin_amdgcn_sched_group_barrier(0x100, 2 + NB, 0);
#pragma unroll
      for (int ks = 0; ks < S::KS; ks++) {
        if (ks + FD < S::KS) __builtin_amdgcn_sched_group_barrier(0x100, 2 + NB, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * NB, 0);
      }
    }
    if constexpr (NB == 1) {
      if (qsplit) {                      // K q_lo^T sits in the lanes of rows 8 .. 15: rows 0 .. 7 take it from there
#pragma unroll
        for (int pb = 0; pb < 2; pb++)
#pragma unroll
          for (int i = 0; i < 4; i++) s[pb][0][i] += row_ror<8>(s[pb][0][i]);
      }
    }
    wave_lds_fence();
  };
  // stage_v: the V registers -> LDS (rows at or past t_end as zeros: 0 x stale bits must not reach O), next V loads;
  // the caller fences
  auto stage_v = [&](const uint32_t tp, const bool more, const uint32_t tpn) __attribute__((always_inline)) {
    const size_t tnb = (size_t)tpn * row_bytes;
    if constexpr (Q8) {
      if (lane / S::LPS < TILE) *(u4*)(stage + soff) = vsr;
      wave_lds_fence();
      float sc[S::NLD8];
#pragma unroll
      for (int i = 0; i < S::NLD8; i++) sc[i] = *(const float*)(stage + ((i * S::RPL8 + lrow8) * S::SPR + (lane % S::LPR8) / 2) * 4);
      wave_lds_fence();
#pragma unroll
      for (int i = 0; i < S::NLD8; i++) {
        h8 lo, hi;
        dq16(vr[i], sc[i], lo, hi);
        if (tp + i * S::RPL8 + lrow8 >= t_end) { lo = (h8){0, 0, 0, 0, 0, 0, 0, 0}; hi = lo; }   // also rows whose scale is not a number
        unsigned char* d = stage + (i * S::RPL8 + lrow8) * S::VROW + (lane % S::LPR8) * 32;
        *(h8*)d = lo; *(h8*)(d + 16) = hi;
      }
      if (more) {
        const size_t tb = (size_t)tpn * HD;
#pragma unroll
        for (int i = 0; i < S::NLD8; i++) vr[i] = *(const u4*)(vbase8 + tb + (size_t)(i * S::RPL8) * HD + voff8);
        vsr = *(const u4*)(vsbase + (size_t)tpn * S::SPR * 4 + soff);
      }
    } else {
    if (tp + TILE > t_end) {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) if (tp + i * S::RPL + lrow >= t_end) vr[i] = zero4;
    }
#pragma unroll
    for (int i = 0; i < S::NLD; i++) *(u4*)(stage + (i * S::RPL + lrow) * S::VROW + (lane % S::LPR) * 16) = vr[i];
    }
    if (!Q8 && more) {
      if constexpr (GATHER) {                         // goff still holds the next tile's rows (set with the K loads above)
#pragma unroll
        for (int i = 0; i < S::NLD; i++) vr[i] = *(const u4*)(vbase + (size_t)goff[i] * row_bytes + (lane % S::LPR) * 16);
      } else {
#pragma unroll
        for (int i = 0; i < S::NLD; i++) vr[i] = *(const u4*)(vbase + tnb + (size_t)(i * S::RPL) * row_bytes + voff);
      }
    }
  };

  // ---- SR: the product O^T = V^T P^T of a split is divided over the waves by OUTPUT DIMS instead of by positions.
  // Every wave scores its own tile (own maximum m_w, probabilities P_w relative to it), publishes P_w -- in the 32
  // padding bytes of its staged V rows -- and (m_w, l_w); after one barrier wave w multiplies all tiles' V^T by their
  // P for dims [w * HD/W, (w + 1) * HD/W), re-weights the per-tile products by exp(m_w' - M) in registers and stores
  // its slice of the split's partial.  Nothing but P crosses waves, so the tail after the last V bytes is one barrier,
  // the MFMAs and a store (the tile loop further down merges the waves' O through LDS: two more LDS round trips).
  if constexpr (SR) {
    constexpr int DBW = S::DB / W;                                      // 16-dim output blocks per wave
    {
      const bool has_tile = wave < n_tiles;
      const uint32_t tp = t_begin + min(wave, n_tiles - 1) * TILE;      // the tile this wave holds in registers
      stage_k(tp, false, 0);
      f4 s[2][NB];
      qk(s);
      // (a wave without a tile contributes nothing: its rows end at 0)
      float mxs[NB], pss[NB];
      h8 pfs[NB];
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const uint32_t row_end = has_tile ? end_pos[nb] : 0u;
        float v[8], mx = NEG_INF;
#pragma unroll
        for (int pb = 0; pb < 2; pb++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const uint32_t pos = row_pos(tp, pb * 16 + 4 * kg + i);
            const float x = pos < row_end ? s[pb][nb][i] * p.scale : NEG_INF;
            v[pb * 4 + i] = x;
            mx = fmaxf(mx, x);
          }
        mx = rows_max(mx);
        const float mw_safe = mx == NEG_INF ? 0.f : mx;
        h8 pf;
#pragma unroll
        for (int j = 0; j < 8; j++) pf[j] = (_Float16)__expf(v[j] - mw_safe);
        mxs[nb] = mx; pss[nb] = rows_sum(sum_f16(pf, 0.f)); pfs[nb] = pf;
      }
      if (v_late) { __builtin_amdgcn_sched_barrier(0); first_v_loads(); __builtin_amdgcn_sched_barrier(0); }
      stage_v(ILV && ilv ? 0u : tp, false, 0);                          // interleaved splits are whole: no row past the end to zero
      // one row block: P rides in the padding of the staged V rows; two: in a region of its own
      if constexpr (NB == 1) *(h8*)(stage + (lane >> 1) * S::VROW + HD * 2 + (lane & 1) * 16) = pfs[0];
      else {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) *(h8*)(p_lds + ((wave * NB + nb) * 64 + lane) * 16) = pfs[nb];
      }
      if (kg == 0) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) { mex[wave * 16 * NB + nb * 16 + ln] = mxs[nb]; lex[wave * 16 * NB + nb * 16 + ln] = pss[nb]; }
      }
      __syncthreads();
      {
        // V^T fragments (two transpose reads each) and the tile's P are fetched VD steps ahead of their MFMA
        // (a tile's P is read once, not once per 16-dim block: the tail of the kernel is bound by the LDS port)
        constexpr int NS = W * DBW, VD = 4;
        h4 lor[VD], hir[VD];
        h8 pfr[W][NB];
        f4 pr[W][DBW][NB];
        auto fetch = [&](int st, int slot) __attribute__((always_inline)) {
          const int w2 = st / DBW, db = wave * DBW + st % DBW;
          const unsigned char* sw = stage_all + w2 * S::STAGE;
          const unsigned char* vp = sw + (4 * kg + (ln >> 2)) * S::VROW + (db * 16 + 4 * (ln & 3)) * 2;
          lor[slot] = lds_read_tr16(vp);
          hir[slot] = lds_read_tr16(vp + 16 * S::VROW);
        };
#pragma unroll
        for (int w2 = 0; w2 < W; w2++) {
          if constexpr (NB == 1) pfr[w2][0] = *(const h8*)(stage_all + w2 * S::STAGE + (lane >> 1) * S::VROW + HD * 2 + (lane & 1) * 16);
          else {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) pfr[w2][nb] = *(const h8*)(p_lds + ((w2 * NB + nb) * 64 + lane) * 16);
          }
        }
#pragma unroll
        for (int st = 0; st < VD; st++) fetch(st, st);
#pragma unroll
        for (int st = 0; st < NS; st++) {
          const h4 lo = lor[st % VD], hi = hir[st % VD];
          if (st + VD < NS) fetch(st + VD, st % VD);
          const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
#pragma unroll
          for (int nb = 0; nb < NB; nb++)
            pr[st / DBW][st % DBW][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pfr[st / DBW][nb], (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, W * NB, 1);
#pragma unroll
        for (int st = 0; st < VD; st++) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
#pragma unroll
        for (int st = 0; st < NS; st++) {
          if (st + VD < NS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
          __builtin_amdgcn_sched_group_barrier(0x008, NB, 1);
        }
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
          // a wave without a tile staged stale rows: its m is -inf, and its products must not reach O even as 0 x NaN
          float mw[W], lw[W], M = NEG_INF;
#pragma unroll
          for (int w2 = 0; w2 < W; w2++) { mw[w2] = mex[w2 * 16 * NB + nb * 16 + ln]; lw[w2] = lex[w2 * 16 * NB + nb * 16 + ln]; M = fmaxf(M, mw[w2]); }
          const float m_safe = M == NEG_INF ? 0.f : M;
          float Lr = 0.f;
          f4 o[DBW];
#pragma unroll
          for (int j = 0; j < DBW; j++) o[j] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int w2 = 0; w2 < W; w2++) {
            const bool dead = mw[w2] == NEG_INF;
            const float c = dead ? 0.f : __expf(mw[w2] - m_safe);
            Lr += lw[w2] * c;
#pragma unroll
            for (int j = 0; j < DBW; j++) o[j] += (dead ? (f4){0.f, 0.f, 0.f, 0.f} : pr[w2][j][nb]) * c;
          }
          const uint32_t r = nb * 16 + ln;
          if (r < R) {
            const uint32_t rc = div_g(r), col = c0 + rc, hq = g * G + r - rc * G;
            const size_t slot = ((size_t)col * nH + hq) * p.slots + sp;
            // f16 partials (|O| <= 128 rows x |v|: far inside the range; the merge adds them up in f32): half the bytes this
            // kernel writes at its very end and half of what the merge kernel waits for
            if (p.part_f16) {
#pragma unroll
              for (int j = 0; j < DBW; j++)
                *(h4*)((_Float16*)p.part_o + slot * HD + (wave * DBW + j) * 16 + 4 * kg) = (h4){ (_Float16)o[j][0], (_Float16)o[j][1], (_Float16)o[j][2], (_Float16)o[j][3] };
            } else {
#pragma unroll
              for (int j = 0; j < DBW; j++) *(f4*)(p.part_o + slot * HD + (wave * DBW + j) * 16 + 4 * kg) = o[j];
            }
            if (wave == 0 && kg == 0) *(float2*)(p.part_ml + slot * 2) = make_float2(M, Lr);
          }
        }
      }
    }
    return;
  }
  // ---- tile loop: every wave streams its own tiles and keeps its own (m, l, O) ----
  f4 acc[S::DB][NB];
#pragma unroll
  for (int db = 0; db < S::DB; db++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[db][nb] = (f4){0.f, 0.f, 0.f, 0.f};
  float m_run[NB], l_run[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) { m_run[nb] = NEG_INF; l_run[nb] = 0.f; }
  const uint32_t tp_lim = t_begin + n_tiles * TILE;
  for (uint32_t tp = t_begin + tile * TILE; tp < tp_lim; tp += tp_step) {
    const bool more = tp + tp_step < tp_lim;
    stage_k(tp, more, tp + tp_step);
    f4 s[2][NB];
    qk(s);
    // ---- online softmax; lane holds row nb*16 + ln, positions tp + pb*16 + 4*kg + i ----
    // m_run is a lazily updated reference maximum: O and l are rescaled only when some row's tile maximum passes it
    // by more than DEC_RESCALE_TH (natural-log units), so exp(x - m_run) <= e^TH stays far inside the f16 range and
    // the rescale of the whole accumulator tile is off the common path.
    h8 pfrag[NB];
    float v[NB][8], mxs[NB];
    bool grow = false;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      float mx = NEG_INF;
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint32_t pos = tp + pb * 16 + 4 * kg + i;
          const float x = pos < end_pos[nb] ? s[pb][nb][i] * p.scale : NEG_INF;
          v[nb][pb * 4 + i] = x;
          mx = fmaxf(mx, x);
        }
      mx = rows_max(mx);
      mxs[nb] = mx;
      grow |= mx > m_run[nb] + DEC_RESCALE_TH;
    }
    if (__builtin_expect(__any(grow), 0)) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const float m_new = fmaxf(m_run[nb], mxs[nb]);
        const float alpha = m_new == NEG_INF ? 1.f : __expf(m_run[nb] - m_new);
        l_run[nb] *= alpha;
        m_run[nb] = m_new;
        // With two or more row blocks the accumulators live in AGPRs.  The empty statements pin them there on both
        // sides of the multiply, so that the VGPR round trip stays inside this rare block instead of being hoisted
        // into the hot loop (128 register moves a tile).
#pragma unroll
        for (int db = 0; db < S::DB; db++) {
          if constexpr (NB > 1) asm volatile("" : "+a"(acc[db][nb]));
          acc[db][nb] *= alpha;
          if constexpr (NB > 1) asm volatile("" : "+a"(acc[db][nb]));
        }
      }
    }
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      const float m_safe = m_run[nb] == NEG_INF ? 0.f : m_run[nb];
      h8 pf;
#pragma unroll
      for (int j = 0; j < 8; j++) pf[j] = (_Float16)__expf(v[nb][j] - m_safe);
      pfrag[nb] = pf;
      l_run[nb] = sum_f16(pf, l_run[nb]);
    }
    // V after the softmax, so that the wait for the V loads comes as late as possible
    stage_v(tp, more, tp + tp_step);
    wave_lds_fence();
    // ---- O^T += V^T P^T ----
    {
      // the same for the V^T fragments (two transpose reads each), VD blocks ahead
      constexpr int VD = 4;
      h4 lor[VD], hir[VD];
      auto fetch = [&](int db, int slot) __attribute__((always_inline)) {
        const unsigned char* vp = stage + (4 * kg + (ln >> 2)) * S::VROW + (db * 16 + 4 * (ln & 3)) * 2;
        lor[slot] = lds_read_tr16(vp);
        hir[slot] = lds_read_tr16(vp + 16 * S::VROW);
      };
#pragma unroll
      for (int db = 0; db < VD; db++) fetch(db, db);
#pragma unroll
      for (int db = 0; db < S::DB; db++) {
        const h4 lo = lor[db % VD], hi = hir[db % VD];
        if (db + VD < S::DB) fetch(db + VD, db % VD);
        const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[db][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pfrag[nb], acc[db][nb], 0, 0, 0);
      }
#pragma unroll
      for (int db = 0; db < VD; db++) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
#pragma unroll
      for (int db = 0; db < S::DB; db++) {
        if (db + VD < S::DB) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
        __builtin_amdgcn_sched_group_barrier(0x008, NB, 1);
      }
    }
    wave_lds_fence();
  }

  // ---- merge the W waves of the workgroup ----
  // The waves' O rows meet in their staging regions UNSCALED (straight from the accumulators); a wave's weight per row,
  // exp(m_w - M), comes from a table one thread per (wave, row) fills, and is applied where the rows are summed.  So is the
  // (column, head) of a stacked row: a table filled once, instead of a division by the group size per element group.
  const bool direct = p.direct_out != 0;       // one split and no own-row partial: this workgroup holds the whole result
  if (tid < 16 * NB) { const uint32_t rc = div_g(tid); rowcol[tid] = c0 + rc; rowhq[tid] = g * G + tid - rc * G; }
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    l_run[nb] = rows_sum(l_run[nb]);
    if (kg == 0) { mex[wave * 16 * NB + nb * 16 + ln] = m_run[nb]; lex[wave * 16 * NB + nb * 16 + ln] = l_run[nb]; }
  }
  __syncthreads();
  static_assert(NB <= 4, "one thread per (wave, row) of the weight table");
  if (tid < W * 16 * NB) {                     // (read after the first barrier below)
    const uint32_t rw = tid % (16 * NB);
    float M = NEG_INF;
#pragma unroll
    for (int w = 0; w < W; w++) M = fmaxf(M, mex[w * 16 * NB + rw]);
    sct[tid] = __expf(mex[tid] - (M == NEG_INF ? 0.f : M));
  }
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    if (nb * 16 + ln < R) {                                            // padding rows are never read back
#pragma unroll
      for (int db = 0; db < S::DB; db++) *(f4*)(stage + ln * S::OROW + (db * 16 + 4 * kg) * 4) = acc[db][nb];
    }
    __syncthreads();
    // rows nb*16 .. nb*16+15, HD/4 float4 each, summed over waves in wave order.  Every thread first issues all
    // its LDS reads (the accumulators are dead, registers are free), then adds and stores: one LDS latency, not one
    // per element.  The (m, l) of a row is merged by one of the first 16 threads.
    constexpr int EPT = 16 * (HD / 4) / (W * 64);
    // direct output: the gate values of this thread's elements are requested before the LDS reads, unconditionally
    // (rows past the last live one re-read it) -- loaded where they are used, under the row guard, each was a round
    // trip of its own behind the sums
    f4 gtv[EPT];
    if (direct && p.gate) {
#pragma unroll
      for (int j = 0; j < EPT; j++) {
        const uint32_t e = tid + j * W * 64, r = min(nb * 16 + e / (HD / 4), R - 1), d4 = e % (HD / 4);
        gtv[j] = *(const f4*)(p.gate + (size_t)rowcol[r] * p.gate_stride + (size_t)rowhq[r] * p.gate_head_stride + 4 * d4);
      }
    }
    f4 part[EPT][W];
#pragma unroll
    for (int j = 0; j < EPT; j++) {
      const uint32_t e = tid + j * W * 64;
      const uint32_t rr = e / (HD / 4), d4 = e % (HD / 4);
      if (nb * 16 + rr < R) {
#pragma unroll
        for (int w = 0; w < W; w++) part[j][w] = *(const f4*)(stage_all + w * S::STAGE + rr * S::OROW + d4 * 16);
      }
    }
    float mw[W], lw[W];
    const bool ml_thread = tid < 16 && nb * 16 + tid < R;
    if (ml_thread) {
#pragma unroll
      for (int w = 0; w < W; w++) { mw[w] = mex[w * 16 * NB + nb * 16 + tid]; lw[w] = lex[w * 16 * NB + nb * 16 + tid]; }
    }
#pragma unroll
    for (int j = 0; j < EPT; j++) {
      const uint32_t e = tid + j * W * 64;
      const uint32_t rr = e / (HD / 4), d4 = e % (HD / 4);
      const uint32_t r = nb * 16 + rr;
      if (r < R) {
        f4 o = part[j][0] * sct[r];
#pragma unroll
        for (int w = 1; w < W; w++) o += part[j][w] * sct[w * 16 * NB + r];
        const uint32_t col = rowcol[r], hq = rowhq[r];
        if (direct) {
          // the only split of the pass: normalise, gate, convert and store here -- no partial, no merge launch
          float Mr = NEG_INF, L = 0.f;
#pragma unroll
          for (int w = 0; w < W; w++) Mr = fmaxf(Mr, mex[w * 16 * NB + r]);
          const float ms = Mr == NEG_INF ? 0.f : Mr;
#pragma unroll
          for (int w = 0; w < W; w++) L += lex[w * 16 * NB + r] * __expf(mex[w * 16 * NB + r] - ms);
          o = o * __builtin_amdgcn_rcpf(L);                              // (v_rcp_f32, 1 ulp, as in the merge kernels)
          if (p.gate) {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] *= __builtin_amdgcn_rcpf(1.f + __expf(-gtv[j][i]));
          }
          if (p.out_f16) {
            const h4 hv = { (_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3] };
            *(h4*)((_Float16*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + 4 * d4) = hv;
          } else {
            *(f4*)((float*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + 4 * d4) = o;
          }
        } else {
          const size_t slot = ((size_t)col * nH + hq) * p.slots + sp;
          *(f4*)(p.part_o + slot * HD + 4 * d4) = o;
        }
      }
    }
    if (ml_thread && !direct) {
      const uint32_t r = nb * 16 + tid;
      float Mr = NEG_INF;
#pragma unroll
      for (int w = 0; w < W; w++) Mr = fmaxf(Mr, mw[w]);
      const float ms = Mr == NEG_INF ? 0.f : Mr;
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < W; w++) L += lw[w] * __expf(mw[w] - ms);
      const size_t slot = ((size_t)rowcol[r] * nH + rowhq[r]) * p.slots + sp;
      *(float2*)(p.part_ml + slot * 2) = make_float2(Mr, L);
    }
    if (nb + 1 < NB) __syncthreads();                                  // the regions are rewritten by the next row block
  }
}

// ---- second pass: log-sum-exp merge over a column's splits, sigmoid gate, output conversion ----
// (the reference's attn_dec_combine(_g), engine/wgsl/attn_dec.js:215-287: M = max m_s, w_s = exp(m_s - M),
// out = sum O_s w_s / sum l_s w_s, times sigmoid(gate))
// The kernel is latency-bound (a few KB per output slice, read once from the memory side, after a dependent launch),
// so it has no barrier and no LDS: one wavefront per (head, 16-dim slice, column) -- nH x HD/16 single-wave
// workgroups, spread over the whole chip -- as 16 split groups x 4 float4 lanes.  A lane loads the (m, l) pairs and
// the output partials of its group's splits (group + 16 k) in one round trip, the maximum and the sums over the 16
// groups are xor-shuffle trees (fixed order), lanes 0 .. 3 finish and store.  The four lanes of a group hold the same
// (m, l), so each computes its splits' weights itself instead of fetching them from a neighbour.
template <int HD, int DS, bool PF16, int CH>
__global__ __launch_bounds__(64)
void pa_combine_wave_kernel(const float* a_part_o, const float* a_part_ml, uint32_t a_slots, uint32_t a_n_heads, uint32_t a_base_pos, uint32_t a_self_row,
                            uint32_t a_split_len, uint32_t a_n_splits, uint32_t a_grid_x, uint32_t a_has_sel, AttnParams p_in) {
  // The leading arguments repeat fields of p_in (a_has_sel: p_in.sel != nullptr): the first twelve dwords of the arguments
  // are preloaded into scalar registers, so the partial loads' addresses need no scalar-load round trip.  The other
  // arguments are fetched in one batch behind those loads (the compiler would fetch each where it is first used).
  AttnParams p = p_in;
  p.part_o = const_cast<float*>(a_part_o); p.part_ml = const_cast<float*>(a_part_ml); p.slots = a_slots; p.n_heads = a_n_heads;
  // a_self_row: 0, or G | ceil(65536 / G) << 8 for a pass whose columns' own rows are partials of their own
  p.base_pos = a_base_pos; p.self_row = a_self_row != 0; p.split_len = a_split_len; p.n_splits = a_n_splits;
  // CH splits per lane and chunk (a template argument: the launcher takes the smallest of 4 / 8 / 16 whose NG x CH covers the
  // pass's splits -- 256 at the most on the single-round kernel, 128 or 64 on the tile loop's plans; more go round the loop below)
  constexpr int SL = HD / DS, LPG = DS / 4, NG = 64 / LPG;
  // dispatch id i runs on XCD i % 8: XCD k takes the contiguous slice range [k n / 8, (k + 1) n / 8), so the slices that
  // share the 128-byte lines of a partial row (two 16-dim slices a line) read them through one L2
  uint32_t wg = blockIdx.x;
  if (a_grid_x % 8 == 0) wg = (blockIdx.x % 8) * (a_grid_x / 8) + blockIdx.x / 8;
  const uint32_t h = wg / SL, dq = wg % SL, col = blockIdx.y, lane = threadIdx.x;
  const uint32_t col_end = a_has_sel ? min(p.sel[col * p.sel_stride], p.sel_max) : p.base_pos + col + 1 - p.self_row;
  // ns_main splits hold streamed rows; the own row's partial, if there is one, is slot ns_main: its (m, l) under this head,
  // its O row under the kv head's first head (the G heads share the value row; the decode kernel stores it once)
  const uint32_t ns_main = min((col_end + p.split_len - 1) / p.split_len, p.n_splits), ns = ns_main + p.self_row;
  const size_t base = ((size_t)col * p.n_heads + h) * p.slots;
  const uint32_t G_ = a_self_row & 0xffu, h0 = ((h * (a_self_row >> 8)) >> 16) * G_;      // (h / G) G by multiply and shift
  const size_t own = (((size_t)col * p.n_heads + h0) * p.slots + ns_main) * HD;             // the own row's O, in elements
  const uint32_t grp = lane / LPG, l4 = lane % LPG;
  const float* po = p.part_o + base * HD + dq * DS + 4 * l4;
  const _Float16* po16 = (const _Float16*)p.part_o + base * HD + dq * DS + 4 * l4;       // PF16: f16 partial rows
  const float2* pml = (const float2*)p.part_ml + base;
  const f4 zero = {0.f, 0.f, 0.f, 0.f};
  // the partial rows stay as loaded (f16 rows as two dwords) until they are used: a conversion at the load would make
  // every load wait for its own data
  typedef typename std::conditional<PF16, h4, f4>::type orow;
  const orow zrow = {0, 0, 0, 0};
  auto load_o = [&](uint32_t s) __attribute__((always_inline)) -> orow {
    if constexpr (PF16) return *(const h4*)(po16 + (size_t)s * HD);
    else return *(const f4*)(po + (size_t)s * HD);
  };
  auto wide = [&](const orow v) __attribute__((always_inline)) -> f4 { return (f4){ (float)v[0], (float)v[1], (float)v[2], (float)v[3] }; };
  orow ov[CH], ov_own = zrow;
  float2 mlv[CH], ml_own = make_float2(NEG_INF, 0.f);
  if (p.self_row) {                             // every group loads the own row (a wave-uniform branch); group 0 counts it
    ml_own = pml[ns_main];
    if constexpr (PF16) ov_own = *(const h4*)((const _Float16*)p.part_o + own + dq * DS + 4 * l4);
    else ov_own = *(const f4*)(p.part_o + own + dq * DS + 4 * l4);
  }
#pragma unroll
  for (int k = 0; k < CH; k++) {
    const uint32_t s = grp + NG * k;
    mlv[k] = s < ns_main ? pml[s] : make_float2(NEG_INF, 0.f);
    ov[k] = s < ns_main ? load_o(s) : zrow;
  }
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("" :: "s"(p.gate), "s"(p.out), "s"(p.gate_stride), "s"(p.out_stride), "s"(p.out_f16), "s"(p.gate_head_stride));
  const uint32_t d_out = dq * DS + 4 * l4;
  f4 gt = zero;
  if (p.gate && lane < LPG) gt = *(const f4*)(p.gate + (size_t)col * p.gate_stride + (size_t)h * p.gate_head_stride + d_out);
  float M = NEG_INF;
#pragma unroll
  for (int k = 0; k < CH; k++) M = fmaxf(M, mlv[k].x);
  for (uint32_t s = grp + NG * CH; s < ns_main; s += NG) M = fmaxf(M, pml[s].x);   // more splits than NG x CH
  M = fmaxf(M, ml_own.x);
  // over the 16 split groups: on the VALU (row rotations + lane swaps) with four lanes a group, else through the LDS crossbar
  if constexpr (LPG == 4 || LPG == 8) M = quads_max<LPG>(M);
  else {
#pragma unroll
    for (int o = LPG; o < 64; o <<= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
  }
  float L = 0.f;
  f4 o = zero;
#pragma unroll
  for (int k = 0; k < CH; k++) {
    const float w = __expf(mlv[k].x - M);        // -inf for a split past the column's end: weight 0
    L += mlv[k].y * w;
    o += wide(ov[k]) * w;
  }
  for (uint32_t s0 = NG * CH; s0 < ns_main; s0 += NG * CH) {
#pragma unroll
    for (int k = 0; k < CH; k++) {
      const uint32_t s = s0 + grp + NG * k;
      mlv[k] = s < ns_main ? pml[s] : make_float2(NEG_INF, 0.f);
      ov[k] = s < ns_main ? load_o(s) : zrow;
    }
#pragma unroll
    for (int k = 0; k < CH; k++) {
      const float w = __expf(mlv[k].x - M);
      L += mlv[k].y * w;
      o += wide(ov[k]) * w;
    }
  }
  {
    const float w = grp == 0 ? __expf(ml_own.x - M) : 0.f;      // last in group 0's sums, as slot ns_main would be; (-inf, 0) and zeros where there is no own row
    L += ml_own.y * w;
    o += wide(ov_own) * w;
  }
  if constexpr (LPG == 4 || LPG == 8) {
    L = quads_sum<LPG>(L);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = quads_sum<LPG>(o[i]);
  } else {
#pragma unroll
    for (int x = LPG; x < 64; x <<= 1) {
      L += __shfl_xor(L, x, 64);
#pragma unroll
      for (int i = 0; i < 4; i++) o[i] += __shfl_xor(o[i], x, 64);
    }
  }
  if (lane < LPG) {
    // (reciprocals by v_rcp_f32, 1 ulp: eight IEEE divisions were some eighty instructions at the very end of the kernel)
    f4 r = ns ? o * __builtin_amdgcn_rcpf(L) : zero;   // an empty gather list: a column of zeros
    if (p.gate) {
#pragma unroll
      for (int i = 0; i < 4; i++) r[i] *= __builtin_amdgcn_rcpf(1.f + __expf(-gt[i]));
    }
    if (p.out_f16) {
      const h4 hv = { (_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3] };
      *(h4*)((_Float16*)p.out + (size_t)col * p.out_stride + (size_t)h * HD + d_out) = hv;
    } else {
      *(f4*)((float*)p.out + (size_t)col * p.out_stride + (size_t)h * HD + d_out) = r;
    }
  }
}

// The same merge for wide passes with few splits (a split prefill chunk: hundreds of columns, a handful of splits):
// one thread per (column, head, 4 dims) walks the splits in order, so a workgroup covers 256 / (HD / 4) (column,
// head) pairs instead of one 64-dim slice of one.  Same arithmetic, split order fixed.
template <int HD>
__global__ __launch_bounds__(256) void pa_combine_wide_kernel(AttnParams p) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  const uint32_t d4 = (uint32_t)(e % (HD / 4));
  const size_t ch = e / (HD / 4);
  if (ch >= (size_t)p.n_cols * p.n_heads) return;
  const uint32_t col = (uint32_t)(ch / p.n_heads), h = (uint32_t)(ch % p.n_heads);
  const uint32_t col_end = p.sel ? min(p.sel[col * p.sel_stride], p.sel_max) : p.base_pos + col + 1 - p.self_row;
  const uint32_t live_len = p.tile_ilv ? p.tile_ilv : p.split_len;      // rows from one split's first row to the next one's
  const uint32_t ns = min((col_end + live_len - 1) / live_len, p.n_splits) + p.self_row;
  const size_t base = ch * p.slots;
  const float* po = p.part_o + base * HD + 4 * d4;
  const float2* pml = (const float2*)p.part_ml + base;
  f4 gt = {0.f, 0.f, 0.f, 0.f};                   // requested with everything else, used last
  if (p.gate) gt = *(const f4*)(p.gate + (size_t)col * p.gate_stride + (size_t)h * p.gate_head_stride + 4 * d4);
  float L = 0.f;
  f4 o = {0.f, 0.f, 0.f, 0.f};
  if (ns) {
    // Eight splits a turn, every load of a turn unconditional and issued together (a turn past the last split re-reads
    // it: harmless for the maximum, weighted 0 in the sums): one load a loop turn was one round trip a split, twice
    // over.  Up to eight splits -- the usual case -- everything the thread reads is one round trip.
    constexpr int B = 8;
    float2 ml[B];
    f4 ov[B];
#pragma unroll
    for (int k = 0; k < B; k++) ml[k] = pml[min((uint32_t)k, ns - 1)];
#pragma unroll
    for (int k = 0; k < B; k++) ov[k] = *(const f4*)(po + (size_t)min((uint32_t)k, ns - 1) * HD);
    float M = NEG_INF;
#pragma unroll
    for (int k = 0; k < B; k++) M = fmaxf(M, ml[k].x);
    for (uint32_t s0 = B; s0 < ns; s0 += B) {
      float mx[B];
#pragma unroll
      for (int k = 0; k < B; k++) mx[k] = pml[min(s0 + k, ns - 1)].x;
#pragma unroll
      for (int k = 0; k < B; k++) M = fmaxf(M, mx[k]);
    }
#pragma unroll
    for (int k = 0; k < B; k++) {
      const float w = __expf(ml[k].x - M) * ((uint32_t)k < ns ? 1.f : 0.f);
      L += ml[k].y * w;
      o += ov[k] * w;
    }
    for (uint32_t s0 = B; s0 < ns; s0 += B) {
#pragma unroll
      for (int k = 0; k < B; k++) ml[k] = pml[min(s0 + k, ns - 1)];
#pragma unroll
      for (int k = 0; k < B; k++) ov[k] = *(const f4*)(po + (size_t)min(s0 + k, ns - 1) * HD);
#pragma unroll
      for (int k = 0; k < B; k++) {
        const float w = __expf(ml[k].x - M) * (s0 + k < ns ? 1.f : 0.f);
        L += ml[k].y * w;
        o += ov[k] * w;
      }
    }
  }
  f4 r = ns ? o * __builtin_amdgcn_rcpf(L) : (f4){0.f, 0.f, 0.f, 0.f};
  const uint32_t d = 4 * d4;
  if (p.gate) {
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] *= __builtin_amdgcn_rcpf(1.f + __expf(-gt[i]));
  }
  if (p.out_f16) {
    const h4 hv = { (_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3] };
    *(h4*)((_Float16*)p.out + (size_t)col * p.out_stride + (size_t)h * HD + d) = hv;
  } else {
    *(f4*)((float*)p.out + (size_t)col * p.out_stride + (size_t)h * HD + d) = r;
  }
}

template <int HD, int NB, int W>
static constexpr size_t decode_lds_bytes() {
  typedef DecShape<HD> S;
  // q rows, the waves' staging regions, the (m, l) exchange and the merge's weight table, its two row tables, and the
  // P region of the single-round kernel with two row blocks
  return 16 * NB * S::QROW + (size_t)W * S::STAGE + 3 * W * 16 * NB * sizeof(float) + 2 * 16 * NB * sizeof(uint32_t) + (NB == 2 && W == 4 ? (size_t)W * NB * 1024 : 0);
}
// the kernel's dynamic LDS limit, raised once per instantiation (at its first launch, or ahead of it by
// pa_prepare_decode_step)
template <int HD, int NB, int W, bool FUSED, bool GATHER, bool Q8, bool SR>
static hipError_t decode_lds_attr() {
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_decode_kernel<HD, NB, W, FUSED, GATHER, Q8, SR>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)decode_lds_bytes<HD, NB, W>());
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  return hipSuccess;
}

template <int HD, int NB, int W, bool FUSED, bool GATHER, bool Q8, bool SR>
static hipError_t launch_decode_k(const AttnParams& p, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  const size_t lds = decode_lds_bytes<HD, NB, W>();
  hipError_t e = decode_lds_attr<HD, NB, W, FUSED, GATHER, Q8, SR>();
  if (e != hipSuccess) return e;
  if (!SR && col_groups != (p.n_cols + p.cols_per_group - 1) / p.cols_per_group) return hipErrorInvalidValue;
  const dim3 grid = SR ? dim3(p.n_splits, p.n_kv_heads, col_groups) : dim3((p.n_splits * p.n_kv_heads * col_groups + 7) / 8 * 8);
  AttnParams pk = p;
  {
    const uint64_t total = (uint64_t)p.n_splits * p.n_kv_heads * col_groups;
    auto magic = [&](uint32_t d) -> uint32_t { return d > 1 && total * d < (1ull << 32) ? (uint32_t)(((1ull << 32) + d - 1) / d) : 0u; };
    pk.col_groups = col_groups; pk.ncg_magic = magic(col_groups); pk.ns_magic = magic(p.n_splits);
  }
  // (bit 1 of the self_row argument: the columns of a column-exact block on adjacent dispatch ids of an XCD)
  const uint32_t self_arg = p.self_row | (SR && p.exact_cols ? 2u : 0u);
  PA_LAUNCH((pa_decode_kernel<HD, NB, W, FUSED, GATHER, Q8, SR>), grid, dim3(W * 64), lds, s, t, p.k_cache, p.base_pos, p.max_seq, p.n_splits, self_arg,
            (uint32_t)grid.x, p.f_q_in, p.group, p.f_q_head_stride, pk);
  return hipGetLastError();
}

// one 16-row block with splits of one tile per wave: the single-round kernel; two blocks when the plan asks
// for it (AttnParams::single_round2: a pass of one split keeps the tile loop, which writes the output itself)
template <int HD, int NB, int W, bool FUSED, bool GATHER = false, bool Q8 = false>
static hipError_t launch_decode_t(const AttnParams& p, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  if constexpr (NB == 1) {
    if (p.split_len == W * TILE) return launch_decode_k<HD, NB, W, FUSED, GATHER, Q8, true>(p, col_groups, s, t);
  }
  if constexpr (NB == 2 && W == 4 && !FUSED && !GATHER) {
    if (p.single_round2 && p.split_len == W * TILE) return launch_decode_k<HD, NB, W, FUSED, GATHER, Q8, true>(p, col_groups, s, t);
  }
  return launch_decode_k<HD, NB, W, FUSED, GATHER, Q8, false>(p, col_groups, s, t);
}

template <int HD>
static hipError_t launch_decode_hd(const AttnParams& p, uint32_t nb, uint32_t waves, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  // eight waves: the one-launch path for small chunks at head_dim 128 with two row blocks (its 250 registers a wave
  // leave room for two waves a SIMD, and a tile's softmax and LDS work is what the loop waits for)
  if (waves == 8) {
    if constexpr (HD == 128) { if (nb == 2 && !p.k_scale) return launch_decode_t<HD, 2, 8, false>(p, col_groups, s, t); }
    return hipErrorInvalidValue;
  }
  if (waves != 4) return hipErrorInvalidValue;
  if (p.k_scale) {                                // int8 caches
    switch (nb) {
      case 1: return launch_decode_t<HD, 1, 4, false, false, true>(p, col_groups, s, t);
      case 2: return launch_decode_t<HD, 2, 4, false, false, true>(p, col_groups, s, t);
      case 3: return launch_decode_t<HD, 3, 4, false, false, true>(p, col_groups, s, t);
      case 4: return launch_decode_t<HD, 4, 4, false, false, true>(p, col_groups, s, t);
      default: return hipErrorInvalidValue;
    }
  }
  switch (nb) {
    case 1: return launch_decode_t<HD, 1, 4, false>(p, col_groups, s, t);
    case 2: return launch_decode_t<HD, 2, 4, false>(p, col_groups, s, t);
    case 3: return launch_decode_t<HD, 3, 4, false>(p, col_groups, s, t);
    case 4: return launch_decode_t<HD, 4, 4, false>(p, col_groups, s, t);
    default: return hipErrorInvalidValue;
  }
}

hipError_t pa_launch_decode(const AttnParams& p, uint32_t hd, uint32_t nb, uint32_t waves, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  if (hd == 256) return launch_decode_hd<256>(p, nb, waves, col_groups, s, t);
  if (hd == 128) return launch_decode_hd<128>(p, nb, waves, col_groups, s, t);
  return hipErrorInvalidValue;
}

hipError_t pa_launch_decode_step(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t) {
  if (!p.f_q_in || p.n_cols != 1 || p.group > 16 || !p.self_row) return hipErrorInvalidValue;
  if (p.k_scale) {                                // int8 caches
    if (hd == 256) return launch_decode_t<256, 1, 4, true, false, true>(p, 1, s, t);
    if (hd == 128) return launch_decode_t<128, 1, 4, true, false, true>(p, 1, s, t);
    return hipErrorInvalidValue;
  }
  if (hd == 256) return launch_decode_t<256, 1, 4, true>(p, 1, s, t);
  if (hd == 128) return launch_decode_t<128, 1, 4, true>(p, 1, s, t);
  return hipErrorInvalidValue;
}

// one-time set-up of the fused step's kernels (both split shapes), so that a later launch makes no other runtime call
hipError_t pa_prepare_decode_step(uint32_t hd, bool q8) {
  hipError_t e = hipErrorInvalidValue;
  if (hd == 256) {
    e = q8 ? decode_lds_attr<256, 1, 4, true, false, true, true>() : decode_lds_attr<256, 1, 4, true, false, false, true>();
    if (e == hipSuccess) e = q8 ? decode_lds_attr<256, 1, 4, true, false, true, false>() : decode_lds_attr<256, 1, 4, true, false, false, false>();
  } else if (hd == 128) {
    e = q8 ? decode_lds_attr<128, 1, 4, true, false, true, true>() : decode_lds_attr<128, 1, 4, true, false, false, true>();
    if (e == hipSuccess) e = q8 ? decode_lds_attr<128, 1, 4, true, false, true, false>() : decode_lds_attr<128, 1, 4, true, false, false, false>();
  }
  return e;
}

hipError_t pa_launch_decode_gather(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t) {
  if (!p.sel || p.cols_per_group != 1 || p.group > 16) return hipErrorInvalidValue;
  if (hd == 256) return launch_decode_t<256, 1, 4, false, true>(p, p.n_cols, s, t);
  if (hd == 128) return launch_decode_t<128, 1, 4, false, true>(p, p.n_cols, s, t);
  return hipErrorInvalidValue;
}

hipError_t pa_launch_combine(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t) {
  // many columns, few splits: one thread per (column, head, 4 dims)
  if (p.n_cols >= 16 && p.n_splits <= 32 && (hd == 256 || hd == 128) && !p.exact_cols && !p.self_row) {
    const size_t threads = (size_t)p.n_cols * p.n_heads * (hd / 4);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (hd == 256) hipLaunchKernelGGL(pa_combine_wide_kernel<256>, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(pa_combine_wide_kernel<128>, grid, dim3(256), 0, s, p);
    return hipGetLastError();
  }
  const uint32_t gx = p.n_heads * (hd / 16), has_sel = p.sel != nullptr;
  // own rows: the group size and ceil(65536 / G) ride in the self_row argument (the kernel finds a kv head's first head)
  const uint32_t self_arg = p.self_row ? (p.group | ((65536u + p.group - 1) / p.group) << 8) : 0u;
  // rows from one split's first row to the next one's (round-robin tiles: a workgroup's first tiles)
  const uint32_t live_len = p.tile_ilv ? p.tile_ilv : p.split_len;
  if (hd != 256 && hd != 128) return hipErrorInvalidValue;
#define PA_COMBINE_WAVE_(HD_, F16_, CH_) PA_LAUNCH((pa_combine_wave_kernel<HD_, 16, F16_, CH_>), dim3(gx, p.n_cols), dim3(64), 0, s, t, (const float*)p.part_o, \
    (const float*)p.part_ml, p.slots, p.n_heads, p.base_pos, self_arg, live_len, p.n_splits, gx, has_sel, p)
  // a lane's unrolled loads are guarded one by one: a pass with few slots takes the instantiation with few of them
  // (f16 partials come from 64 splits on, so their short form is never needed)
#define PA_COMBINE_WAVE(HD_, F16_) do { if (F16_ || p.n_splits > 128) PA_COMBINE_WAVE_(HD_, F16_, 16); \
    else if (p.n_splits > 64) PA_COMBINE_WAVE_(HD_, F16_, (F16_ ? 16 : 8)); else PA_COMBINE_WAVE_(HD_, F16_, (F16_ ? 16 : 4)); } while (0)
  if (hd == 256) { if (p.part_f16) PA_COMBINE_WAVE(256, true); else PA_COMBINE_WAVE(256, false); }
  else { if (p.part_f16) PA_COMBINE_WAVE(128, true); else PA_COMBINE_WAVE(128, false); }
#undef PA_COMBINE_WAVE
#undef PA_COMBINE_WAVE_
  return hipGetLastError();
}
