// Column-batched projections for large chunks on gfx950: Y[c][r] = sum_k W[r][k] X[c][k] with the weights widened
// to f16 once and a matrix-core GEMM over two f16 operands.
//
// Same contract and the same operand precision as pa_gemm_kernel (proj_gemm.hip) -- the reference's "f16" prefill
// math, engine/wgsl/gemm.js:31-36: every dequantised weight and every activation rounded to f16, products and sums
// f32 -- for the chunks its batched GEMMs serve (engine/wgsl/gemm.js, gemm_sgm.js, gemm_wide.js; dispatched at
// engine/qwen35.js:2142-2170, :2600-2620).  What differs is where the widening happens.  The tiled kernel of
// proj_gemm.hip widens packed weights on their way into LDS inside its main loop; at 64 x 64 wave tiles that loop is
// bound by LDS traffic and by the widening arithmetic in front of every barrier.  For a chunk of hundreds of columns
// the weights are re-read by every column block anyway, so here they are widened once into an f16 staging matrix
// (pa_widen_w_kernel: one pass over the packed planes, HBM-bound; the caller keeps the matrix with the weight or
// widens per call), and the GEMM proper has nothing but loads and MFMAs in its loop:
//
//   * a wavefront owns 128 columns x 32 TN weight rows (TN = 2, 3 or 4) as 4 x TN v_mfma_f32_32x32x16_f16 tiles whose
//     accumulators (up to 256 registers) live in the accumulation registers, one wave a SIMD; a workgroup is four
//     such waves side by side along the weight rows: 128 columns x 128 TN rows;
//   * the staging matrix is written in MFMA fragment order -- for every block of 32 rows and 16 k the 64 lanes' 16
//     bytes are contiguous (1 KB) -- so a weight (B) fragment is ONE coalesced wave-wide load straight into the
//     registers the MFMA reads: the weights never touch LDS.  (With both operands staged through LDS, the fragment
//     reads and the staging writes together kept the LDS port 75 % busy and the loop ran at 740 - 790 TFLOP/s.)  The
//     fragments of eight k-steps (four at TN = 4) are in flight per wave, a register ring refilled slot by slot
//     behind the MFMAs that used it;
//   * the activations (A), which all four waves share, go through LDS, K in stages of 64 (128-byte rows), two stages
//     in LDS, one bare barrier a stage; a stage is fetched into registers a stage ahead and written with ds_write
//     (16 registers), rows unpadded with the 16-byte chunk c of row r at slot c ^ ((r >> 1) & 7): the ds_read_b128
//     fragment reads of any 16 consecutive rows then hit 64 distinct banks.  One wave a SIMD means nothing hides an
//     LDS round trip, so the A fragments are double buffered in registers by hand: the reads of k-step i + 1 (across
//     the barrier: of the next stage's first k-step) are issued among the MFMAs of k-step i;
//   * every load is a plain load the compiler sees, and the issue order is pinned (scheduling barriers per k-step,
//     the prologue's ring loads in ring order): its vmcnt waits then let a whole ring of fragments stay in flight.
//     An LDS-direct load issued from inline assembly shares the in-order counter without the compiler knowing, and
//     a ring slot loaded late in the prologue makes the wait at the head of the loop drain the ring every iteration
//     (both measured: 0.21 ms instead of 0.18 on a 4096 x 9216 x 2048 chunk);
//   * workgroup ids are dealt so that the 32 workgroups an XCD runs side by side form a block of 8 column blocks x 4
//     row blocks, which share 8 activation tiles and 4 weight panels in that XCD's L2 (3 % over row-major order);
//   * TN is picked per call so that the workgroups fill whole rounds of the chip.
//
// Measured on a 4096 x 9216 x 2048 Q4_0 chunk: 0.160 - 0.168 ms (920 - 970 TFLOP/s) with the staging matrix kept.
// Ablations on an earlier build that ran 0.178 ms: without the output stores 0.163 ms, without the weight loads of
// the loop 0.163, with neither and no activation loads 0.134.
#include "pf_common.h"

#define GW_COLS 128          // columns per workgroup
#define GW_KS 64             // K per stage
#define GW_ROWB 128          // bytes of a staged activation row (64 halves)

struct Gemm16Params {
  const uint16_t* x; const uint16_t* w16; float* y;
  uint32_t x_stride, y_stride, d_out, d_in, n_cols;
  int acc;
};

template <int TN, bool ACC>
__global__ __launch_bounds__(256, 1) void pa_gemm16_kernel(Gemm16Params p) {
  constexpr int TM = 4;                                  // 32-column blocks per wave
  constexpr int ROWS = 128 * TN;                         // weight rows per workgroup (4 waves x 32 TN)
  constexpr int STAGE = GW_COLS * GW_ROWB;               // bytes of a staged A tile
  constexpr int A_LD = GW_COLS / 8 / 4;                  // 1 KB loads (8 rows) per wave and stage
  constexpr int RING = TN == 4 ? 4 : 8;                  // k-steps of weight fragments in flight per wave (what the register file holds next to 4 x TN accumulator tiles)
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * STAGE];
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // XCD-aware tile order: dispatch id i runs on XCD i % 8 as that XCD's (i / 8)-th workgroup, so XCD k walks the tiles
  // [k per, (k + 1) per) of a linear order in which 32 neighbours (what an XCD runs at a time) form a block of 8
  // column blocks x 4 row blocks: they share 8 activation tiles and 4 weight panels in that XCD's L2 instead of 32 + 1
  const uint32_t n_cb = (p.n_cols + GW_COLS - 1) / GW_COLS, n_rb = (p.d_out + ROWS - 1) / ROWS, total = n_cb * n_rb;
  const uint32_t per = (total + 7) / 8, tile = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (tile >= total) return;
  uint32_t cb = tile % n_cb, rb_ = tile / n_cb;
  if (n_cb % 8 == 0) {
    const uint32_t panel = tile / (4 * n_cb), r = tile % (4 * n_cb), h = min(4u, n_rb - panel * 4);
    cb = r / (8 * h) * 8 + r % 8; rb_ = panel * 4 + r % (8 * h) / 8;
  }
  const uint32_t c0 = cb * GW_COLS, r0 = rb_ * ROWS;
  const uint32_t n_stages = p.d_in / GW_KS, nk16 = p.d_in / 16;

  // ---- A: LDS-direct loads, 8 rows x 128 bytes each; lane i lands at (row i / 8, slot i % 8) and fetches chunk
  //      slot ^ ((row >> 1) & 7) of that row.  Columns past the end of the chunk repeat its last column (never stored).
  const uint32_t lrow = lane >> 3, lslot = lane & 7;
  const unsigned char* a_src[A_LD];
#pragma unroll
  for (int i = 0; i < A_LD; i++) {
    const uint32_t row = (wave * A_LD + i) * 8 + lrow;
    const size_t col = min((size_t)c0 + row, (size_t)p.n_cols - 1);
    a_src[i] = (const unsigned char*)(p.x + col * p.x_stride) + ((lslot ^ ((row >> 1) & 7)) * 16);
  }
  // the stage's 16 bytes per lane and load go through registers (fetched a stage ahead) and a ds_write: every load of
  // the loop is then visible to the compiler, whose vmcnt waits count the weight-fragment ring correctly (an LDS-direct
  // load issued from inline assembly sits in the same in-order counter without the compiler knowing, and its
  // conservative wait for a ring slot then also waits for the just-issued activation loads)
  u4 areg[A_LD];
  auto fetch_a = [&](uint32_t st) __attribute__((always_inline)) {
    const size_t koff = (size_t)st * GW_ROWB;
#pragma unroll
    for (int i = 0; i < A_LD; i++) areg[i] = *(const u4*)(a_src[i] + koff);
  };
  auto store_a = [&](uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < A_LD; i++) *(u4*)(smem + buf * STAGE + (wave * A_LD + i) * 1024 + lane * 16) = areg[i];
  };
  // ---- B: fragment (row block rb, k block kb) of the staging matrix = 1 KB at ((rb nk16 + kb) 64 + lane) 16; the
  //      staging matrix is padded to whole 32-row blocks, row blocks past d_out repeat the last one (never stored)
  const uint32_t n_rb32 = (p.d_out + 31) / 32;
  const unsigned char* b_src[TN];
#pragma unroll
  for (int t = 0; t < TN; t++) {
    const uint32_t rb = min(r0 / 32 + wave * TN + t, n_rb32 - 1);
    b_src[t] = (const unsigned char*)p.w16 + ((size_t)rb * nk16 * 64 + lane) * 16;
  }
  u4 ring[RING][TN];
  auto load_b = [&](int slot, uint32_t kb) __attribute__((always_inline)) {
    const size_t off = (size_t)min(kb, nk16 - 1) * 1024;         // past the last k block: the last one again, never used
#pragma unroll
    for (int t = 0; t < TN; t++) ring[slot][t] = *(const u4*)(b_src[t] + off);
  };

  const uint32_t fl = lane & 31, fk = lane >> 5;
  auto col_of = [&](int a, int i) { return c0 + a * 32 + 8 * (i / 4) + 4 * fk + (i % 4); };
  auto row_of = [&](int b) { return r0 + (wave * TN + b) * 32 + fl; };
  // Accumulating calls.  Loads and stores share one counter on this part, and with both kinds pending the compiler's
  // wait for a loaded value waits for every store in flight as well: old values fetched in the epilogue tile by tile,
  // between the stores, cost a memory round trip per tile (0.097 ms against 0.072 plain on a 4096 x 2048 x 4096 chunk,
  // however many tiles ahead they are fetched).  With 8 tiles a wave (TN = 2) the accumulators therefore START from
  // the old values -- requested first, they arrive under the prologue's loads -- and the epilogue is the plain store;
  // with 12 or 16 tiles there is no room to stage them all before the loop, and the epilogue works in phases of
  // several tiles: all of a phase's loads, then all of its stores.
  constexpr bool INIT = ACC && TN == 2;
  f16v acc[TM][TN];
  if constexpr (INIT) {
    // every load goes out before the first value is moved into an accumulation register (left alone, the compiler
    // stages them a few at a time: a round trip per batch)
    float old[TM * TN][16];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++)
#pragma unroll
        for (int i = 0; i < 16; i++)
          old[a * TN + b][i] = p.y[(size_t)min(col_of(a, i), p.n_cols - 1) * p.y_stride + min(row_of(b), p.d_out - 1)];   // unconditional (clamped): a guarded load is a branch, and one load a basic block is one round trip a load
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[a][b][i] = old[a * TN + b][i];
    __builtin_amdgcn_sched_barrier(0);
  } else {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;
  }

  // A fragment addresses: row fl of a 32-row block, 8 halves at k = 16 ks + 8 fk -> chunk 2 ks + fk, swizzled by the
  // row (the swizzle is an XOR on the chunk index, and 2 ks has no bit in common with fk)
  uint32_t a_rd[TM];
#pragma unroll
  for (int t = 0; t < TM; t++) { const uint32_t row = t * 32 + fl; a_rd[t] = row * GW_ROWB + ((fk ^ ((row >> 1) & 7)) * 16); }
  struct Frag { h8 a[TM]; };
  auto rd = [&](Frag& f, const unsigned char* sb, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TM; t++) f.a[t] = *(const h8*)(sb + (a_rd[t] ^ (ks * 32)));
  };
  auto mma = [&](const Frag& f, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int b = 0; b < TN; b++) {
      h8 bf; __builtin_memcpy(&bf, &ring[slot][b], 16);
#pragma unroll
      for (int a = 0; a < TM; a++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[a], bf, acc[a][b], 0, 0, 0);
    }
  };

#pragma unroll
  for (int j = 0; j < RING; j++) {
    // in ring order and not reordered: the wait the compiler places at the head of the loop counts the loads behind
    // slot 0 on both ways into it, and a slot loaded late here would make it drain the ring every iteration
    load_b(j, j);
    __builtin_amdgcn_sched_barrier(0);
  }
  fetch_a(0);
  store_a(0);
  __syncthreads();
  Frag f0, f1;
  rd(f0, smem, 0);
  // One stage = four k-steps; PAR = st & 1 picks the LDS buffer and (ring of 8) the half of the register ring, so that
  // every index into the ring is static.  The body has no branch: past the last stage the A loads fetch the last
  // stage again into the buffer nobody reads, the B loads the last k block, and the fragment reads a tile nobody uses
  // (d_in is a multiple of 128 here, so stages come in pairs).
  auto stage = [&](auto PAR, const uint32_t st) __attribute__((always_inline)) {
    constexpr int par = decltype(PAR)::value;
    fetch_a(min(st + 1, n_stages - 1));
    const unsigned char* sb = smem + par * STAGE;
    constexpr int s0 = RING == 8 ? par * 4 : 0;                  // this stage's slots of the ring
    const uint32_t kb_next = st * 4 + RING;                      // a slot is refilled RING k-steps ahead, right after its use
    // source order = issue order (pinned): the next k-step's four A fragment reads first, then this k-step's MFMAs,
    // then the refill of the ring slot they just used
    auto pin = [&]() __attribute__((always_inline)) {
      __builtin_amdgcn_sched_group_barrier(0x100, TM, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, TN, 0);
      __builtin_amdgcn_sched_barrier(0);
    };
    rd(f1, sb, 1); mma(f0, s0 + 0); load_b(s0 + 0, kb_next + 0); pin();
    rd(f0, sb, 2); mma(f1, s0 + 1); load_b(s0 + 1, kb_next + 1); pin();
    rd(f1, sb, 3); mma(f0, s0 + 2); load_b(s0 + 2, kb_next + 2); pin();
    // the stage's last A fragments are on their way; the next stage goes into the other buffer (every wave left it
    // before the last barrier), and behind this barrier nobody reads this one any more.  The barrier is bare (LDS
    // traffic only crosses it): a workgroup fence would also wait for the ring refills in flight.
    store_a(par ^ 1);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    rd(f0, smem + (par ^ 1) * STAGE, 0); mma(f1, s0 + 3); load_b(s0 + 3, kb_next + 3); pin();
  };
  for (uint32_t st = 0; st < n_stages; st += 2) {
    stage(std::integral_constant<int, 0>{}, st);
    stage(std::integral_constant<int, 1>{}, st + 1);
  }
  // accumulator i of a tile: column 8 (i / 4) + 4 (lane / 32) + i % 4, row lane % 32
  if constexpr (!ACC || INIT) {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++)
#pragma unroll
        for (int i = 0; i < 16; i++)
          if (row_of(b) < p.d_out && col_of(a, i) < p.n_cols) p.y[(size_t)col_of(a, i) * p.y_stride + row_of(b)] = acc[a][b][i];
  } else {
    constexpr int D = TN == 3 ? 6 : 4, NT = TM * TN;       // tiles per phase (the ring and the fragment registers are dead by now)
    static_assert(NT % D == 0, "whole phases");
#pragma unroll
    for (int t0 = 0; t0 < NT; t0 += D) {
      float old[D][16];
#pragma unroll
      for (int t = 0; t < D; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int a = (t0 + t) / TN, b = (t0 + t) % TN;
          old[t][i] = p.y[(size_t)min(col_of(a, i), p.n_cols - 1) * p.y_stride + min(row_of(b), p.d_out - 1)];      // unconditional (clamped), see above
        }
      __builtin_amdgcn_sched_barrier(0);                   // every load of the phase before its first store
#pragma unroll
      for (int t = 0; t < D; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int a = (t0 + t) / TN, b = (t0 + t) % TN;
          if (row_of(b) < p.d_out && col_of(a, i) < p.n_cols) p.y[(size_t)col_of(a, i) * p.y_stride + row_of(b)] = old[t][i] + acc[a][b][i];
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// ---- weights -> f16 in MFMA fragment order: for row block rb (32 rows, the last one padded with copies of the last
//      row) and k block kb (16 values) the 1 KB at ((rb nk16 + kb) 64 + lane) 16 holds, for lane = 32 fk + fl, the 8
//      values k = 16 kb + 8 fk .. + 7 of row 32 rb + fl.  The arithmetic is the tiled kernel's staging: (nibble - 8) *
//      scale and int8 * scale in f16 (exact integer, one rounding), f32 rounded to nearest even ----
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
static __device__ inline h2v gw_as_h2(uint32_t u) { h2v r; __builtin_memcpy(&r, &u, 4); return r; }
static __device__ inline h2v gw_bytes(uint32_t w, uint32_t sel, h2v bias, h2v sc) { return (gw_as_h2(__builtin_amdgcn_perm(0x64646464u, w, sel)) - bias) * sc; }

// one thread per (row, quantisation block of 32 weights), the 32 rows of a row block on consecutive threads
template <int KIND>
__global__ __launch_bounds__(256) void pa_widen_w_kernel(const void* w, const uint16_t* scales, uint16_t* out, uint32_t d_out, uint32_t nb, size_t n_threads) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_threads) return;
  const uint32_t fl = (uint32_t)(idx % 32), bq = (uint32_t)((idx / 32) % nb);
  const size_t rb = idx / ((size_t)32 * nb);
  const size_t b = (size_t)min((uint32_t)(rb * 32 + fl), d_out - 1) * nb + bq;          // the packed block this thread widens
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
  // o[v] = values 8 v .. 8 v + 7 of the block: k block 2 bq + v / 2, half fk = v & 1
  const size_t nk16 = (size_t)nb * 2;
#pragma unroll
  for (int v = 0; v < 4; v++) *(h8*)(out + (((rb * nk16 + 2 * bq + v / 2) * 64 + (v & 1) * 32 + fl) * 8)) = o[v];
}

// ---- chunks too small to give every CU one of the tiles above (a few dozen to a few hundred columns, or few weight
//      rows): 64 columns x 64 weight rows a workgroup, and the workgroup's four waves split K between them instead of
//      the tile -- of every K stage of 128 wave w takes the k-steps w and w + 4 -- so that all four share the staged
//      activations (one coalesced fetch per workgroup) while each loads only the weight fragments of its own
//      k-steps.  Every wave holds the whole 64 x 64 tile (4 MFMA tiles, 64 accumulators: two workgroups a CU); at the
//      end the four copies meet in LDS and wave w adds up MFMA tile w in a fixed order (((w0 + w1) + w2) + w3) and
//      stores it.  A workgroup walks all of K, so there are no partial sums in memory and no second launch; what
//      bounds it is the L2 -> CU traffic of 64 x 64 tiles (K (64 + 64) 2 bytes a tile), about twice its MFMA time.
#define GM_T 64              // columns per workgroup
#define GM_KS 128            // K per stage
#define GM_ROWB 256          // bytes of a staged activation row

template <int TN, int RING, bool ACC>
__global__ __launch_bounds__(256, 2) void pa_gemm16_mid_kernel(Gemm16Params p) {
  constexpr int STAGE = GM_T * GM_ROWB;                  // 16 KB
  constexpr int ROWS = 32 * TN;                          // weight rows per workgroup
  constexpr int NT = 2 * TN;                             // MFMA tiles per wave: 2 column blocks x TN row blocks
  __shared__ __attribute__((aligned(1024))) unsigned char smem[(4 * NT * 16 * 64 * 4 > 2 * STAGE) ? 4 * NT * 16 * 64 * 4 : 2 * STAGE];   // two stages; at the end the four waves' tiles
  const uint32_t tid = threadIdx.x, lane = tid & 63, fl = lane & 31, fk = lane >> 5;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // XCD k owns a contiguous range of tiles, column blocks fastest: neighbours stream the same weight rows through one L2
  const uint32_t n_cb = (p.n_cols + GM_T - 1) / GM_T, n_rb = (p.d_out + ROWS - 1) / ROWS, total = n_cb * n_rb;
  const uint32_t per = (total + 7) / 8, tile = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (tile >= total) return;
  const uint32_t c0 = (tile % n_cb) * GM_T, r0 = (tile / n_cb) * ROWS;
  const uint32_t n_stages = p.d_in / GM_KS, nk16 = p.d_in / 16;

  // A: a load covers 4 rows x 256 bytes; chunk c of row r is staged at slot c ^ (r & 15)
  const uint32_t lrow = lane >> 4, lchunk = lane & 15;
  const unsigned char* a_src[4];
  uint32_t a_dst[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t row = (wave * 4 + i) * 4 + lrow;
    const size_t col = min((size_t)c0 + row, (size_t)p.n_cols - 1);     // columns past the end repeat the last one (never stored)
    a_src[i] = (const unsigned char*)(p.x + col * p.x_stride) + lchunk * 16;
    a_dst[i] = row * GM_ROWB + ((lchunk ^ (row & 15)) * 16);
  }
  // a stage's activations are fetched two stages ahead (two register sets), its weight fragments RING stages ahead:
  // one stage of MFMAs is far less than a round trip to L2, let alone to HBM, and a workgroup's time is its number of
  // stages x that latency / the stages it keeps in flight
  u4 areg[2][4];
  auto fetch_a = [&](int set, uint32_t st) __attribute__((always_inline)) {
    const size_t off = (size_t)min(st, n_stages - 1) * GM_ROWB;       // past the last stage: the last one again, never used
#pragma unroll
    for (int i = 0; i < 4; i++) areg[set][i] = *(const u4*)(a_src[i] + off);
  };
  auto store_a = [&](int set, uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; i++) *(u4*)(smem + buf * STAGE + a_dst[i]) = areg[set][i];
  };
  // fragment of column block t at k-step j of the stage: row 32 t + fl, chunk 2 j + fk
  uint32_t a_rd[2][2];
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const uint32_t row = t * 32 + fl, chunk = 2 * (wave + 4 * u) + fk;
      a_rd[t][u] = row * GM_ROWB + ((chunk ^ (row & 15)) * 16);
    }
  // B: this wave's k blocks 8 st + wave and 8 st + wave + 4 of the TN 32-row blocks
  const uint32_t n_rb32 = (p.d_out + 31) / 32;
  const unsigned char* b_src[TN];
#pragma unroll
  for (int t = 0; t < TN; t++) b_src[t] = (const unsigned char*)p.w16 + ((size_t)min(r0 / 32 + t, n_rb32 - 1) * nk16 * 64 + lane) * 16;
  u4 bq[RING][2][TN];                                    // [stage % RING][u][row block]
  auto load_b = [&](int slot, uint32_t st) __attribute__((always_inline)) {
    const size_t off = (size_t)(min(st, n_stages - 1) * 8 + wave) * 1024;
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int t = 0; t < TN; t++) bq[slot][u][t] = *(const u4*)(b_src[t] + off + (size_t)u * 4096);
  };
  f16v acc[2][TN];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

#pragma unroll
  for (int j = 0; j < RING; j++) load_b(j, j);
  fetch_a(0, 0);
  fetch_a(1, 1);
  store_a(0, 0);
  fetch_a(0, 2);
  __syncthreads();
  // stage st reads LDS buffer st % 2 and ring slot st % RING; register set p holds the stages of parity p: at the
  // end of stage st the other set (stage st + 1, fetched two stages ago) goes to the other buffer and then receives
  // stage st + 3
  auto stage = [&](auto J, uint32_t st) __attribute__((always_inline)) {
    constexpr int j = decltype(J)::value, par = j & 1;
    const unsigned char* sb = smem + par * STAGE;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      h8 af[2], bf[TN];
#pragma unroll
      for (int t = 0; t < 2; t++) af[t] = *(const h8*)(sb + a_rd[t][u]);
#pragma unroll
      for (int t = 0; t < TN; t++) __builtin_memcpy(&bf[t], &bq[j][u][t], 16);
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < TN; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
    load_b(j, st + RING);
    store_a(par ^ 1, par ^ 1);          // stage st + 1 into the other buffer: every wave left it before the last barrier
    fetch_a(par ^ 1, st + 3);
    __syncthreads();
  };
  static_assert(RING == 4 || RING == 8, "the loop below is unrolled by the ring");
  for (uint32_t st = 0; st < n_stages; st += RING) {
    stage(std::integral_constant<int, 0>{}, st);
    if (st + 1 < n_stages) stage(std::integral_constant<int, 1>{}, st + 1);
    if (st + 2 < n_stages) stage(std::integral_constant<int, 2>{}, st + 2);
    if (st + 3 < n_stages) stage(std::integral_constant<int, 3>{}, st + 3);
    if constexpr (RING == 8) {
      if (st + 4 < n_stages) stage(std::integral_constant<int, 4>{}, st + 4);
      if (st + 5 < n_stages) stage(std::integral_constant<int, 5>{}, st + 5);
      if (st + 6 < n_stages) stage(std::integral_constant<int, 6>{}, st + 6);
      if (st + 7 < n_stages) stage(std::integral_constant<int, 7>{}, st + 7);
    }
  }
  // the four partial tiles meet in LDS (the stages are dead behind the loop's last barrier): [wave][slot][lane], slot =
  // 16 (TN a + b) + i for accumulator i of the MFMA tile of column block a and row block b
  float* red = (float*)smem;
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) red[((wave * NT + a * TN + b) * 16 + i) * 64 + lane] = acc[a][b][i];
  __syncthreads();
  // wave w finishes slots [w SPW, (w + 1) SPW); accumulator i of a tile = column 8 (i / 4) + 4 fk + i % 4, row fl
  constexpr int SPW = NT * 16 / 4;
  float sum[SPW];
#pragma unroll
  for (int k = 0; k < SPW; k++) {
    const uint32_t o = (wave * SPW + k) * 64 + lane;
    sum[k] = ((red[o] + red[o + NT * 16 * 64]) + red[o + 2 * NT * 16 * 64]) + red[o + 3 * NT * 16 * 64];
  }
  auto col_of = [&](int k) { const uint32_t sl = wave * SPW + k, a = sl / (16 * TN), i = sl % 16; return c0 + a * 32 + 8 * (i / 4) + 4 * fk + (i % 4); };
  auto row_of = [&](int k) { const uint32_t sl = wave * SPW + k, b = sl / 16 % TN; return r0 + b * 32 + fl; };
  float old[SPW];
  if constexpr (ACC) {
#pragma unroll
    for (int k = 0; k < SPW; k++) old[k] = p.y[(size_t)min(col_of(k), p.n_cols - 1) * p.y_stride + min(row_of(k), p.d_out - 1)];   // unconditional (clamped): guarded loads would go out one round trip at a time
  }
#pragma unroll
  for (int k = 0; k < SPW; k++)
    if (row_of(k) < p.d_out && col_of(k) < p.n_cols) p.y[(size_t)col_of(k) * p.y_stride + row_of(k)] = ACC ? old[k] + sum[k] : sum[k];
}

template <int TN, int RING>
static hipError_t launch_gemm16_mid(const Gemm16Params& q, hipStream_t s) {
  const uint32_t total = ((q.n_cols + GM_T - 1) / GM_T) * ((q.d_out + 32 * TN - 1) / (32 * TN));
  if (q.acc) hipLaunchKernelGGL((pa_gemm16_mid_kernel<TN, RING, true>), dim3((total + 7) / 8 * 8), dim3(256), 0, s, q);
  else hipLaunchKernelGGL((pa_gemm16_mid_kernel<TN, RING, false>), dim3((total + 7) / 8 * 8), dim3(256), 0, s, q);
  return hipGetLastError();
}

template <int TN>
static hipError_t launch_gemm16(const Gemm16Params& q, hipStream_t s) {
  const uint32_t total = ((q.n_cols + GW_COLS - 1) / GW_COLS) * ((q.d_out + 128 * TN - 1) / (128 * TN));
  if (q.acc) hipLaunchKernelGGL((pa_gemm16_kernel<TN, true>), dim3((total + 7) / 8 * 8), dim3(256), 0, s, q);
  else hipLaunchKernelGGL((pa_gemm16_kernel<TN, false>), dim3((total + 7) / 8 * 8), dim3(256), 0, s, q);
  return hipGetLastError();
}

// large chunks only: at least 512 columns, and enough 128-column x 256-row workgroups to give every CU one (below that
// the tiled kernel's 128 x 128 workgroups fill the chip better)
bool pa_gemm_wide_serves(const GemmParams& p, int n_cu) {
  if (p.n_cols < 512 || p.d_in % (2 * GW_KS) != 0 || (p.x_stride & 7) != 0 || ((uintptr_t)p.x & 15) != 0) return false;
  const uint64_t wgs = (uint64_t)((p.n_cols + GW_COLS - 1) / GW_COLS) * ((p.d_out + 255) / 256);
  return wgs >= (uint64_t)(n_cu > 0 ? n_cu : 256);
}

// chunks of more than 16 columns that the large-chunk kernel does not serve.  Measured with cold weights (Q4_0, 32 to
// 64 weights in rotation): [q|k|v] 9216 x 2048 13.0 - 13.5 us for 8 to 32 columns against 12.9 / 17.9 / 28 / 34 us at 8 /
// 16 / 24 / 32 columns on the skinny kernel (which reads the packed weights, a quarter of the bytes, but one launch
// per 16 columns); wo 2048 x 4096 16.7 us against 8.5 / 15.9 / 19.9 / 27.6
bool pa_gemm_mid_serves(const GemmParams& p) {
  return p.n_cols > 16 && p.d_in % GM_KS == 0 && (p.x_stride & 7) == 0 && ((uintptr_t)p.x & 15) == 0;
}

// bytes of the staging matrix of a weight: whole 32-row blocks
size_t pa_gemm_wide_staging_bytes(uint32_t d_out, uint32_t d_in) { return (size_t)((d_out + 31) / 32) * 32 * d_in * sizeof(uint16_t); }

// w16: staging of pa_gemm_wide_staging_bytes (the caller's, 16-byte aligned); widen = false: it already holds these weights
hipError_t pa_launch_gemm_wide(const GemmParams& p, uint16_t* w16, bool widen, bool mid, int n_cu, hipStream_t s) {
  if (widen) {
    const uint32_t nb = p.d_in / 32;
    const size_t n_threads = (size_t)((p.d_out + 31) / 32) * 32 * nb;
    const dim3 wgrid((unsigned)((n_threads + 255) / 256));
    switch (p.kind) {
      case PA_W_Q4_0: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_Q4_0>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, p.d_out, nb, n_threads); break;
      case PA_W_Q8_0: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_Q8_0>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, p.d_out, nb, n_threads); break;
      case PA_W_F32: hipLaunchKernelGGL(pa_widen_w_kernel<PA_W_F32>, wgrid, dim3(256), 0, s, p.w, p.scales, w16, p.d_out, nb, n_threads); break;
      default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  Gemm16Params q;
  q.x = p.x; q.w16 = w16; q.y = p.y; q.x_stride = p.x_stride; q.y_stride = p.y_stride;
  q.d_out = p.d_out; q.d_in = p.d_in; q.n_cols = p.n_cols; q.acc = p.acc;
  if (mid) {
    // fewer 64 x 64 tiles than half the CUs: 32-row tiles (twice the workgroups) with twice the stages in flight
    // (wo 2048 x 4096 on up to 64 columns, cold: 20 -> 16.7 us; with 144 tiles, [q|k|v], it is 2 us slower)
    const uint64_t tiles64 = (uint64_t)((p.n_cols + GM_T - 1) / GM_T) * ((p.d_out + 63) / 64);
    return tiles64 * 2 < (uint64_t)(n_cu > 0 ? n_cu : 256) ? launch_gemm16_mid<1, 8>(q, s) : launch_gemm16_mid<2, 4>(q, s);
  }
  // rows per workgroup (128 TN): the choice that wastes the least of the chip -- rounds of n_cu workgroups, each
  // round costing its workgroups' rows (smaller wave tiles pay a little more LDS traffic per MFMA)
  const uint32_t cb = (p.n_cols + GW_COLS - 1) / GW_COLS, cus = n_cu > 0 ? (uint32_t)n_cu : 256u;
  uint32_t best_tn = 4; uint64_t best = ~0ull;
  for (uint32_t tn = 4; tn >= 2; tn--) {
    const uint64_t wgs = (uint64_t)((p.d_out + 128 * tn - 1) / (128 * tn)) * cb;
    const uint64_t cost = ((wgs + cus - 1) / cus) * (128 * tn) * (tn == 4 ? 16 : tn == 3 ? 17 : 18);
    if (cost < best) { best = cost; best_tn = tn; }
  }
  return best_tn == 4 ? launch_gemm16<4>(q, s) : best_tn == 3 ? launch_gemm16<3>(q, s) : launch_gemm16<2>(q, s);
}
