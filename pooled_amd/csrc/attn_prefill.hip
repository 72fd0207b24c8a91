// Causal prefill attention on f16 MFMA for gfx950 (MI355X).
//
// Replaces the reference's attn_flash_tile + attn_combine_tile + sigmoid_mul_mc
// (engine/wgsl/attn_tile.js:108-193, engine/wgsl/qwen35.js:877-887): a chunk of n_cols query columns at absolute
// positions base_pos + c attends causally to the f16 KV cache rows [0, base_pos + c].  One launch covers what
// the reference runs as consecutive 16-column passes.
//
// Work decomposition
//   * A workgroup (4 wavefronts, one per SIMD) owns one kv head and a block of columns; its 4 x 64 = 256 query
//     rows are (column, head-in-group) pairs, so every K/V tile it stages serves all G heads of the group
//     (the reference's "up to 64 rows share a tile", scaled to the MFMA shape).
//   * K/V tiles of 32 positions go global -> registers -> LDS (double buffered, one barrier a step); the next
//     tile's loads are in flight while the current one is consumed.
//   * S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_f16.  Q fragments stay in registers for the whole
//     kernel; K fragments are ds_read_b128, V^T fragments come from the gfx950 LDS transpose read
//     (ds_read_b64_tr_b16).  The S^T accumulator layout (lane = query row, 16 positions) is the B-operand
//     layout of the PV product, so P never leaves registers.
//   * Online softmax in f32 in the exp2 domain with a lazily updated reference maximum: O and l are rescaled
//     only when some row's maximum grows by more than 2^8, which keeps exp2(x - m_ref) <= 256 (exact enough
//     in f16) and takes the 256-register O rescale off the common path.
//   * Workgroup ids are remapped so that each XCD (ids are dealt round-robin to the 8 XCDs) works on one
//     contiguous range of (kv head, column block): the K/V stream of a kv head is fetched into one L2.
//   * Optional split over the context (short chunks on long contexts would otherwise leave CUs idle): partial
//     (m, l, O) go to the same buffers the decode kernel uses and the same merge kernel finishes them.
#include "pa_internal.h"
#include <hip/hip_fp16.h>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef __fp16 hh4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

#define NEG_INF (-__builtin_inff())
#define PF_TN 32                 // positions per step
#define PF_RESCALE_TH 8.0f       // log2 units

static __device__ inline h4 lds_read_tr16(const unsigned char* p) {
  hh4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16((hh4 __attribute__((address_space(3)))*)p);
  h4 r; __builtin_memcpy(&r, &t, 8); return r;
}

template <int HD, int W> struct PfShape {
  static constexpr int KROW = HD * 2 + 16;        // staged K row stride (bytes): conflict-free b128 fragment reads
  static constexpr int VROW = HD * 2 + 32;        // staged V row stride (bytes): 2-way (optimal) transpose reads
  static constexpr int KBUF = PF_TN * KROW;
  static constexpr int VBUF = PF_TN * VROW;
  static constexpr int KS = HD / 16;              // k-steps of QK^T
  static constexpr int DB = HD / 32;              // 32-dim blocks of the output
  static constexpr int CPR = HD / 8;              // 16-byte chunks per row
  static constexpr int LD = PF_TN * CPR / (W * 64);   // 16-byte loads per thread, tensor and step
};

template <int HD, int QB, int W>
__global__ __launch_bounds__(W * 64, W / 4) void pa_prefill_kernel(AttnParams p, uint32_t n_col_blocks) {
  typedef PfShape<HD, W> S;
  constexpr int RW = W * QB * 32;                  // query rows per workgroup
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* kbuf = smem;                      // [2][KBUF]
  unsigned char* vbuf = smem + 2 * S::KBUF;        // [2][VBUF]

  // ---- XCD-aware id -> (kv head, column block) ----
  const uint32_t total = n_col_blocks * p.n_kv_heads;
  const uint32_t per_xcd = (total + 7) / 8;
  const uint32_t lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (lid >= total) return;
  const uint32_t g = lid / n_col_blocks, cb = lid % n_col_blocks, sp = blockIdx.y;

  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t ln = lane & 31, hb = lane >> 5;   // MFMA row / column index, k half
  const uint32_t G = p.group, nH = p.n_heads;
  const uint32_t c0 = cb * p.cols_per_group;
  const uint32_t ncl = min(p.cols_per_group, p.n_cols - c0);
  const uint32_t R = ncl * G;                      // live rows (<= RW)
  const uint32_t seq_max = p.base_pos + c0 + ncl;  // rows visible to the block's last column
  const uint32_t t_begin = sp * p.split_len;
  if (t_begin >= seq_max) return;
  const uint32_t t_end = min(t_begin + p.split_len, seq_max);
  const uint32_t n_steps = (t_end - t_begin + PF_TN - 1) / PF_TN;
  const size_t row_bytes = (size_t)p.n_kv_heads * HD * 2;
  const unsigned char* kg_base = (const unsigned char*)(p.k_cache + (size_t)g * HD);
  const unsigned char* vg_base = (const unsigned char*)(p.v_cache + (size_t)g * HD);

  // ---- first K/V tile: global -> registers ----
  u4 kr[S::LD], vr[S::LD];
  uint32_t ld_row[S::LD], ld_chunk[S::LD];
#pragma unroll
  for (int i = 0; i < S::LD; i++) {
    const uint32_t e = tid + i * W * 64;
    ld_row[i] = e / S::CPR; ld_chunk[i] = e % S::CPR;
    const size_t off = (size_t)(t_begin + ld_row[i]) * row_bytes + ld_chunk[i] * 16;
    kr[i] = *(const u4*)(kg_base + off);
    vr[i] = *(const u4*)(vg_base + off);
  }

  // ---- per-lane rows: query row of block qb is wave*QB*32 + qb*32 + ln = (column r / G, head r % G) ----
  uint32_t end_pos[QB], row_id[QB];
  uint32_t w_min_end = 0xffffffffu, w_max_end = 0;
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const uint32_t r = wave * QB * 32 + qb * 32 + ln;
    row_id[qb] = min(r, R - 1);
    end_pos[qb] = r < R ? p.base_pos + c0 + r / G + 1 : 0u;
  }
  {
    const uint32_t r_first = wave * QB * 32, r_last = min(r_first + QB * 32, R) - 1;
    if (r_first < R) { w_min_end = p.base_pos + c0 + r_first / G + 1; w_max_end = p.base_pos + c0 + r_last / G + 1; }
  }

  // ---- Q fragments (B operand of S^T = K Q^T): row ln of block qb, dims 16 ks + 8 hb .. + 7, as f16 ----
  h8 qf[QB][S::KS];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const float* qrow = p.q + (size_t)(c0 + row_id[qb] / G) * p.q_stride + (size_t)(g * G + row_id[qb] % G) * HD + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      const f4 a = *(const f4*)(qrow + 16 * ks), b = *(const f4*)(qrow + 16 * ks + 4);
      qf[qb][ks] = (h8){ (_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3],
                         (_Float16)b[0], (_Float16)b[1], (_Float16)b[2], (_Float16)b[3] };
    }
  }

  f16v acc[S::DB][QB];
#pragma unroll
  for (int db = 0; db < S::DB; db++)
#pragma unroll
    for (int qb = 0; qb < QB; qb++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[db][qb][i] = 0.f;
  float m_ref[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) { m_ref[qb] = NEG_INF; l_run[qb] = 0.f; }
  const float c1 = p.scale * 1.4426950408889634f;   // scores -> log2 domain

  // ---- stage tile 0 ----
#pragma unroll
  for (int i = 0; i < S::LD; i++) {
    *(u4*)(kbuf + ld_row[i] * S::KROW + ld_chunk[i] * 16) = kr[i];
    const u4 z = {0u, 0u, 0u, 0u};
    *(u4*)(vbuf + ld_row[i] * S::VROW + ld_chunk[i] * 16) = (t_begin + ld_row[i] < t_end) ? vr[i] : z;
  }
  __syncthreads();

  for (uint32_t step = 0; step < n_steps; step++) {
    const uint32_t tp = t_begin + step * PF_TN;
    const bool more = step + 1 < n_steps;
    const unsigned char* kb = kbuf + (step & 1) * S::KBUF;
    const unsigned char* vb = vbuf + (step & 1) * S::VBUF;
    // next tile's loads (the caches carry 32 rows of padding, so a straddling tile reads valid memory)
    if (more) {
#pragma unroll
      for (int i = 0; i < S::LD; i++) {
        const size_t off = (size_t)(tp + PF_TN + ld_row[i]) * row_bytes + ld_chunk[i] * 16;
        kr[i] = *(const u4*)(kg_base + off);
        vr[i] = *(const u4*)(vg_base + off);
      }
    }
    if (tp < w_max_end) {
      // ---- S^T = K Q^T : rows = 32 positions, columns = 32 query rows per block ----
      f16v s[QB];
#pragma unroll
      for (int qb = 0; qb < QB; qb++)
#pragma unroll
        for (int i = 0; i < 16; i++) s[qb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < S::KS; ks++) {
        const h8 a = *(const h8*)(kb + ln * S::KROW + ks * 32 + hb * 16);
#pragma unroll
        for (int qb = 0; qb < QB; qb++) s[qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[qb][ks], s[qb], 0, 0, 0);
      }
      // ---- online softmax; lane holds query row ln of each block, positions tp + 8 (i / 4) + 4 hb + i % 4 ----
      const bool diag = tp + PF_TN > w_min_end;      // some row of this wave ends inside the tile
      float mt[QB];
#pragma unroll
      for (int qb = 0; qb < QB; qb++) {
        float mx = NEG_INF;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          float x = s[qb][i] * c1;
          if (diag) { const uint32_t pos = tp + 8 * (i >> 2) + 4 * hb + (i & 3); x = pos < end_pos[qb] ? x : NEG_INF; }
          s[qb][i] = x;
          mx = fmaxf(mx, x);
        }
        mt[qb] = fmaxf(mx, __shfl_xor(mx, 32, 64));
      }
      bool grow = false;
#pragma unroll
      for (int qb = 0; qb < QB; qb++) grow |= mt[qb] > m_ref[qb] + PF_RESCALE_TH;
      if (__any(grow)) {
#pragma unroll
        for (int qb = 0; qb < QB; qb++) {
          const float m_new = fmaxf(m_ref[qb], mt[qb]);
          const float alpha = m_new == NEG_INF ? 1.f : __builtin_amdgcn_exp2f(m_ref[qb] - m_new);
          m_ref[qb] = m_new;
          l_run[qb] *= alpha;
#pragma unroll
          for (int db = 0; db < S::DB; db++) acc[db][qb] *= alpha;
        }
      }
      h8 pf[QB][2];
#pragma unroll
      for (int qb = 0; qb < QB; qb++) {
        const float mr = m_ref[qb] == NEG_INF ? 0.f : m_ref[qb];
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const float e = __builtin_amdgcn_exp2f(s[qb][i] - mr);
          ps += e;
          pf[qb][i >> 3][i & 7] = (_Float16)e;
        }
        l_run[qb] += ps;
      }
      // ---- O^T += V^T P^T : rows = 32 dims, contraction over 2 x 16 positions ----
      const uint32_t b4 = lane >> 4, sl = lane & 15;
#pragma unroll
      for (int db = 0; db < S::DB; db++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const unsigned char* vp = vb + (16 * j + 4 * (b4 >> 1) + (sl >> 2)) * S::VROW + (32 * db + 16 * (b4 & 1) + 4 * (sl & 3)) * 2;
          const h4 lo = lds_read_tr16(vp);
          const h4 hi = lds_read_tr16(vp + 8 * S::VROW);
          const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
#pragma unroll
          for (int qb = 0; qb < QB; qb++) acc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pf[qb][j], acc[db][qb], 0, 0, 0);
        }
      }
    }
    // ---- stage the next tile into the other buffer ----
    if (more) {
      unsigned char* kn = kbuf + ((step + 1) & 1) * S::KBUF;
      unsigned char* vn = vbuf + ((step + 1) & 1) * S::VBUF;
#pragma unroll
      for (int i = 0; i < S::LD; i++) {
        *(u4*)(kn + ld_row[i] * S::KROW + ld_chunk[i] * 16) = kr[i];
        const u4 z = {0u, 0u, 0u, 0u};
        *(u4*)(vn + ld_row[i] * S::VROW + ld_chunk[i] * 16) = (tp + PF_TN + ld_row[i] < t_end) ? vr[i] : z;
      }
    }
    __syncthreads();
  }

  // ---- epilogue ----
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    l_run[qb] += __shfl_xor(l_run[qb], 32, 64);
    const uint32_t r = wave * QB * 32 + qb * 32 + ln;
    if (r >= R) continue;
    const uint32_t col = c0 + r / G, hq = g * G + r % G;
    if (p.n_splits == 1) {
      // the whole context was seen: normalise, gate, convert, store
      const float inv_l = 1.f / l_run[qb];
      const float* gate = p.gate ? p.gate + (size_t)col * p.gate_stride + (size_t)hq * HD : nullptr;
#pragma unroll
      for (int db = 0; db < S::DB; db++) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const uint32_t d = 32 * db + 8 * q4 + 4 * hb;
          f4 o = { acc[db][qb][4 * q4] * inv_l, acc[db][qb][4 * q4 + 1] * inv_l, acc[db][qb][4 * q4 + 2] * inv_l, acc[db][qb][4 * q4 + 3] * inv_l };
          if (gate) {
            const f4 gt = *(const f4*)(gate + d);
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] *= 1.f / (1.f + __expf(-gt[i]));
          }
          if (p.out_f16) {
            const h4 hv = { (_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3] };
            *(h4*)((_Float16*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + d) = hv;
          } else {
            *(f4*)((float*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + d) = o;
          }
        }
      }
    } else {
      // split partial: un-normalised O, m in natural-log units of the scaled scores, l
      const size_t slot = ((size_t)col * nH + hq) * p.slots + sp;
#pragma unroll
      for (int db = 0; db < S::DB; db++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const uint32_t d = 32 * db + 8 * q4 + 4 * hb;
          const f4 o = { acc[db][qb][4 * q4], acc[db][qb][4 * q4 + 1], acc[db][qb][4 * q4 + 2], acc[db][qb][4 * q4 + 3] };
          *(f4*)(p.part_o + slot * HD + d) = o;
        }
      if (hb == 0) {
        p.part_ml[slot * 2] = m_ref[qb] * 0.6931471805599453f;
        p.part_ml[slot * 2 + 1] = l_run[qb];
      }
    }
  }
}

template <int HD, int QB, int W>
static hipError_t launch_prefill_t(const AttnParams& p, uint32_t col_groups, hipStream_t s) {
  typedef PfShape<HD, W> S;
  const size_t lds = 2 * (S::KBUF + S::VBUF);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_prefill_kernel<HD, QB, W>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const uint32_t total = col_groups * p.n_kv_heads;
  const uint32_t gx = ((total + 7) / 8) * 8;       // whole rounds of the 8 XCDs
  hipLaunchKernelGGL((pa_prefill_kernel<HD, QB, W>), dim3(gx, p.n_splits), dim3(W * 64), lds, s, p, col_groups);
  return hipGetLastError();
}

// row_blocks = 32-row query blocks per wavefront (2); the workgroup covers 4 * row_blocks * 32 rows
hipError_t pa_launch_prefill(const AttnParams& p, uint32_t hd, uint32_t row_blocks, uint32_t col_groups, hipStream_t s) {
  if (row_blocks != 2) return hipErrorNotSupported;
  if (hd == 256) return launch_prefill_t<256, 1, 8>(p, col_groups, s);
  if (hd == 128) return launch_prefill_t<128, 2, 4>(p, col_groups, s);
  return hipErrorNotSupported;
}
