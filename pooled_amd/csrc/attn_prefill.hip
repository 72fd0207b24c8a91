// Causal prefill attention on f16 MFMA for gfx950 (MI355X).
//
// Replaces the reference's attn_flash_tile + attn_combine_tile + sigmoid_mul_mc
// (engine/wgsl/attn_tile.js:108-193, engine/wgsl/qwen35.js:877-887): a chunk of n_cols query columns at absolute
// positions base_pos + c attends causally to the f16 KV cache rows [0, base_pos + c].  One launch covers what
// the reference runs as consecutive 16-column passes.
//
// Work decomposition
//   * A workgroup owns one kv head and a block of columns; its 256 query rows are (column, head-in-group) pairs,
//     so every K/V tile it stages serves all G heads of the group (the reference's "up to 64 rows share a tile",
//     scaled to the MFMA shape).  8 wavefronts x 32 rows, two per SIMD: while one wave of a SIMD does its softmax
//     on the VALU the other one's MFMAs keep the matrix pipe busy.
//   * K/V tiles of 32 positions go global -> LDS directly (global_load_lds_dwordx4: no staging registers),
//     double buffered, one barrier a step; the next tile's loads are in flight while the current one is consumed.
//     An LDS-direct load writes 64 lanes x 16 B contiguously, so rows cannot be padded; bank conflicts are
//     avoided by an XOR swizzle applied on the *global* side (lane i fetches the chunk that belongs at its LDS
//     slot): K chunk c of row r sits at slot c ^ (r & 15) (conflict-free ds_read_b128 fragments), V chunk c at
//     c ^ 4 (r & 3) (2-way = optimal ds_read_b64_tr_b16).  Rows at or past the end of the context are fetched
//     from the cache's zero padding row instead, so 0 x stale bits never reaches O.
//   * S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_f16.  Q fragments stay in registers for the whole
//     kernel (at hd 256 half of them, the other half is parked in LDS); K fragments are ds_read_b128, V^T fragments come from the gfx950 LDS transpose read
//     (ds_read_b64_tr_b16).  The S^T accumulator layout (lane = query row, 16 positions) is the B-operand
//     layout of the PV product, so P never leaves registers.
//   * Online softmax in f32 in the exp2 domain with a lazily updated reference maximum: O and l are rescaled
//     only when some row's maximum grows by more than 2^8, which keeps exp2(x - m_ref) <= 256 (exact enough
//     in f16) and takes the 128-register O rescale off the common path.
//   * Workgroup ids are remapped so that each XCD (ids are dealt round-robin to the 8 XCDs) works on one
//     contiguous range of (kv head, column block): the K/V stream of a kv head is fetched into one L2.
//   * Optional split over the context (short chunks on long contexts would otherwise leave CUs idle): partial
//     (m, l, O) go to the same buffers the decode kernel uses and the same merge kernel finishes them.
#include "pf_common.h"

template <int HD, int W> struct PfShape {
  static constexpr int ROWB = HD * 2;             // bytes of one kv head's row
  static constexpr int TILE = PF_TN * ROWB;       // bytes of one staged tile (K or V)
  static constexpr int KS = HD / 16;              // k-steps of QK^T
  static constexpr int DB = HD / 32;              // 32-dim blocks of the output
  static constexpr int QR = HD == 256 ? PF_QR : KS;   // k-steps whose Q fragments stay in registers
  static constexpr int CPR = HD / 8;              // 16-byte chunks per row
  static constexpr int RPB = 64 / CPR;            // rows per 1 KB LDS-direct load
  static constexpr int NLD = PF_TN / RPB / W;   // LDS-direct loads per wave, tensor and step
  static_assert(NLD >= 1 && NLD * W * RPB == PF_TN, "tile must divide evenly over the waves");
};

template <int HD, int QB, int W>
__global__ __launch_bounds__(W * 64, W / 4) void pa_prefill_kernel(AttnParams p, uint32_t n_col_blocks) {
  typedef PfShape<HD, W> S;
  // four separate LDS objects (two K, two V buffers): the compiler then orders an LDS read only after the
  // LDS-direct loads into the *same* buffer, and the prefetch into the other buffer stays in flight
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf1[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf1[S::TILE];

  // ---- XCD-aware id -> (kv head, split, column block) ----
  // Work items are (kv head, split, column block), column block fastest: the workgroups of one (kv head, split) read
  // the same K/V rows.  The grid is one-dimensional; dispatch id i runs on XCD i % 8, and XCD k owns the contiguous
  // item range [k per_xcd, (k + 1) per_xcd): every XCD gets the same number of workgroups whatever the split count,
  // and the workgroups that share a K/V stream share an L2.
  const uint32_t total = n_col_blocks * p.n_kv_heads * p.n_splits;
  const uint32_t per_xcd = (total + 7) / 8;
  const uint32_t lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (lid >= total) return;
  const uint32_t cb = lid % n_col_blocks, sp = (lid / n_col_blocks) % p.n_splits, g = lid / (n_col_blocks * p.n_splits);

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform (scalar) so per-wave branches are scalar branches
  const uint32_t ln = lane & 31, hb = lane >> 5;   // MFMA row / column index, k half
  const uint32_t G = p.group, nH = p.n_heads;
  const uint32_t c0 = cb * p.cols_per_group;
  const uint32_t ncl = min(p.cols_per_group, p.n_cols - c0);
  const uint32_t R = ncl * G;                      // live rows (<= W * QB * 32)
  const uint32_t seq_max = p.base_pos + c0 + ncl;  // rows visible to the block's last column
  const uint32_t t_begin = sp * p.split_len;
  if (t_begin >= seq_max) return;
  const uint32_t t_end = min(t_begin + p.split_len, seq_max);
  const uint32_t n_steps = (t_end - t_begin + PF_TN - 1) / PF_TN;
  const size_t row_bytes = (size_t)HD * 2;                       // head-major caches: a kv head's rows are contiguous
  const size_t head_rows = (size_t)p.max_seq + PF_TN;            // rows of one kv head's plane, padding included
  const unsigned char* kg_base = (const unsigned char*)(p.k_cache + (size_t)g * head_rows * HD);
  const unsigned char* vg_base = (const unsigned char*)(p.v_cache + (size_t)g * head_rows * HD);

  // ---- LDS-direct tile loads: load i of wave w fills the 1 KB block i W + w of a buffer, i.e. rows (i W + w) RPB ..;
  //      lane l of a block lands at (row l / CPR, slot l % CPR) and therefore fetches chunk slot ^ swizzle(row) of
  //      that row.  W RPB is a multiple of 16, so the swizzle -- and with it the lane's byte offset from the block's
  //      first row -- is the same for every i and every tile: one 32-bit offset per tensor, the rest of the address
  //      is wave-uniform (scalar registers) ----
  static_assert((W * S::RPB) % 16 == 0, "the swizzle must not depend on the load index");
  const uint32_t ld_row0 = wave * S::RPB + lane / S::CPR, ld_slot = lane % S::CPR;
  const uint32_t k_off = ld_row0 * (uint32_t)row_bytes + (ld_slot ^ (ld_row0 & 15)) * 16;
  const uint32_t v_off = ld_row0 * (uint32_t)row_bytes + (ld_slot ^ (4 * (ld_row0 & 3))) * 16;
  constexpr uint32_t LD_STRIDE = W * S::RPB * S::ROWB;           // bytes between the rows of consecutive loads
  // rows at or past t_end (only in the last tile of the context) come from the zero padding row max_seq
  auto issue_t = [&](const unsigned char* g_base, const uint32_t off, unsigned char* dst, uint32_t tpos) {
    const unsigned char* t0p = g_base + (size_t)tpos * row_bytes;
    if (tpos + PF_TN <= t_end) {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) PF_GLL_S(t0p + i * LD_STRIDE, off, dst + (i * W + wave) * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) {
        const uint32_t row = i * W * S::RPB + ld_row0;
        const unsigned char* src = tpos + row < t_end ? t0p + i * LD_STRIDE + off
                                                      : g_base + (size_t)p.max_seq * row_bytes + (off - ld_row0 * (uint32_t)row_bytes);
        PF_GLL(src, dst + (i * W + wave) * 1024);
      }
    }
  };
  auto issue_k = [&](unsigned char* kdst, uint32_t tpos) { issue_t(kg_base, k_off, kdst, tpos); };
  auto issue_v = [&](unsigned char* vdst, uint32_t tpos) { issue_t(vg_base, v_off, vdst, tpos); };
  issue_k(kbuf0, t_begin);
  issue_v(vbuf0, t_begin);

  // ---- per-lane rows: query row of block qb is wave*QB*32 + qb*32 + ln = (column r / G, head r % G) ----
  uint32_t end_pos[QB], row_id[QB];
  uint32_t w_min_end = 0xffffffffu;
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const uint32_t r = wave * QB * 32 + qb * 32 + ln;
    row_id[qb] = min(r, R - 1);
    end_pos[qb] = r < R ? p.base_pos + c0 + r / G + 1 : 0u;
  }
  {
    const uint32_t r_first = wave * QB * 32;
    if (r_first < R) w_min_end = p.base_pos + c0 + r_first / G + 1;
  }

  // ---- Q fragments (B operand of S^T = K Q^T): row ln of block qb, dims 16 ks + 8 hb .. + 7, as f16 ----
  // The first QR k-steps stay in registers for the whole kernel; the others are parked in LDS in fragment order
  // ([wave][qb][ks - QR][lane] x 16 B: conflict-free b128 reads of a wave's own region) and re-read every step.
  // At hd 256 all 16 in registers (64 VGPRs) leave too little room beside the 128 accumulators; a single spill
  // reload inside the loop would also force the in-order vmcnt to drain the LDS-direct loads in flight.
  constexpr int QR = S::QR;
  extern __shared__ __attribute__((aligned(16))) unsigned char q_lds_all[];
  unsigned char* q_lds = q_lds_all + (size_t)wave * QB * (S::KS - QR) * 1024 + lane * 16;
  h8 qf[QB][QR];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const float* qrow = p.q + (size_t)(c0 + row_id[qb] / G) * p.q_stride + (size_t)(g * G + row_id[qb] % G) * HD + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      const f4 a = *(const f4*)(qrow + 16 * ks), b = *(const f4*)(qrow + 16 * ks + 4);
      const h8 f = { (_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3],
                     (_Float16)b[0], (_Float16)b[1], (_Float16)b[2], (_Float16)b[3] };
      if (ks < QR) qf[qb][ks] = f;
      else *(h8*)(q_lds + (qb * (S::KS - QR) + (ks - QR)) * 1024) = f;
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

  // per-lane LDS read offsets with the swizzles folded in (buffer bases are 1 KB aligned, so XOR == add on the
  // swizzled bits): K fragment of k-step ks is at k_rd ^ (ks * 32); V fragment of dim block db at v_rd ^ (db * 64)
  const uint32_t k_rd = ln * S::ROWB + ((hb ^ (ln & 1)) * 16) + ((ln & 15) >> 1) * 32;
  const uint32_t b4 = lane >> 4, sl = lane & 15;
  const uint32_t v_rd = (4 * (b4 >> 1) + (sl >> 2)) * S::ROWB + (2 * (b4 & 1) + ((sl & 3) >> 1)) * 16 + (sl & 1) * 8 + ((sl >> 2) & 3) * 64;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // The three phases of a tile.  s (raw scores) lives from qk to sm, pf (f16 probabilities) from sm to pv.
  f16v s[QB];
  h8 pf[QB][2];
  // ---- S^T = K Q^T : rows = 32 positions, columns = 32 query rows per block ----
  auto qk = [&](const unsigned char* kb, const uint32_t tp) {
#pragma unroll
    for (int qb = 0; qb < QB; qb++)
#pragma unroll
      for (int i = 0; i < 16; i++) s[qb][i] = 0.f;
    // K fragments (and the Q fragments parked in LDS) are fetched KD k-steps ahead of the MFMA that consumes them
    constexpr int KD = PF_KD;
    h8 ka[KD], qa[QB][KD];
#pragma unroll
    for (int i = 0; i < KD; i++) {
      ka[i] = *(const h8*)(kb + (k_rd ^ (i * 32)));
      if (i >= QR) {
#pragma unroll
        for (int qb = 0; qb < QB; qb++) qa[qb][i] = *(const h8*)(q_lds + (qb * (S::KS - QR) + (i - QR)) * 1024);
      }
    }
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      const h8 a = ka[ks % KD];
      h8 b[QB];
#pragma unroll
      for (int qb = 0; qb < QB; qb++) b[qb] = ks < QR ? qf[qb][ks < QR ? ks : 0] : qa[qb][ks % KD];
      if (ks + KD < S::KS) {
        ka[ks % KD] = *(const h8*)(kb + (k_rd ^ ((ks + KD) * 32)));
        if (ks + KD >= QR) {
#pragma unroll
          for (int qb = 0; qb < QB; qb++) qa[qb][ks % KD] = *(const h8*)(q_lds + (qb * (S::KS - QR) + (ks + KD - QR)) * 1024);
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; qb++) s[qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[qb], s[qb], 0, 0, 0);
    }
    // pin the issue order the source states: the first KD fetches up front, then each k-step's fetches behind its MFMAs
#pragma unroll
    for (int i = 0; i < KD; i++) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); if (i >= QR) __builtin_amdgcn_sched_group_barrier(0x100, QB, 0); }
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      __builtin_amdgcn_sched_group_barrier(0x008, QB, 0);
      if (ks + KD < S::KS) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); if (ks + KD >= QR) __builtin_amdgcn_sched_group_barrier(0x100, QB, 0); }
    }
  };
  // ---- online softmax; lane holds query row ln of each block, positions tp + 8 (i / 4) + 4 hb + i % 4 ----
  // Raw scores stay unscaled: the scale rides in the exp2 argument (one fma per element), the row sum is a
  // v_dot2 over the f16-rounded probabilities (the values PV really uses), and the mask is a separate pass
  // that only tiles straddling a row end execute.
  auto sm = [&](const uint32_t tp) {
    if (tp + PF_TN > w_min_end) {
      asm volatile("; causal tile" ::: "memory");   // keeps this a branch: most tiles skip the 3 ops per element
#pragma unroll
      for (int qb = 0; qb < QB; qb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const uint32_t pos = tp + 8 * (i >> 2) + 4 * hb + (i & 3);
          s[qb][i] = pos < end_pos[qb] ? s[qb][i] : NEG_INF;
        }
    }
    float mt[QB];
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
      float mx = fmaxf(s[qb][0], s[qb][1]);
#pragma unroll
      for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[qb][i]), s[qb][i + 1]);
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mt[qb] = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * c1;      // both k halves of the row, log2 domain
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
    const h2 ones = { (_Float16)1.f, (_Float16)1.f };
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
      const float nmr = m_ref[qb] == NEG_INF ? 0.f : -m_ref[qb];
      float ps = l_run[qb];
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][i], c1, nmr));
        const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qb][i + 1], c1, nmr));
        const h2 pp = { (_Float16)e0, (_Float16)e1 };
        ps = __builtin_amdgcn_fdot2(pp, ones, ps, false);
        pf[qb][i >> 3][i & 7] = pp[0]; pf[qb][i >> 3][(i & 7) + 1] = pp[1];
      }
      l_run[qb] = ps;
    }
  };
  // ---- O^T += V^T P^T : rows = 32 dims, contraction over 2 x 16 positions ----
  auto pv = [&](const unsigned char* vb, const uint32_t tp) {
    // fragment f = j DB + db: positions 16 j .., dims 32 db .. (consecutive MFMAs hit different accumulators);
    // fetched VD fragments ahead
    constexpr int VD = PF_VD, NF = 2 * S::DB;
    h4 vlo[VD], vhi[VD];
#pragma unroll
    for (int f = 0; f < VD; f++) {
      const unsigned char* vp = vb + (v_rd ^ ((f % S::DB) * 64)) + (f / S::DB) * 16 * S::ROWB;
      vlo[f] = lds_read_tr16(vp);
      vhi[f] = lds_read_tr16(vp + 8 * S::ROWB);
    }
#pragma unroll
    for (int f = 0; f < NF; f++) {
      const h4 lo = vlo[f % VD], hi = vhi[f % VD];
      if (f + VD < NF) {
        const int fn = f + VD;
        const unsigned char* vp = vb + (v_rd ^ ((fn % S::DB) * 64)) + (fn / S::DB) * 16 * S::ROWB;
        vlo[f % VD] = lds_read_tr16(vp);
        vhi[f % VD] = lds_read_tr16(vp + 8 * S::ROWB);
      }
      const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
#pragma unroll
      for (int qb = 0; qb < QB; qb++) acc[f % S::DB][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pf[qb][f / S::DB], acc[f % S::DB][qb], 0, 0, 0);
    }
#pragma unroll
    for (int f = 0; f < VD; f++) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
#pragma unroll
    for (int f = 0; f < NF; f++) {
      __builtin_amdgcn_sched_group_barrier(0x008, QB, 1);
      if (f + VD < NF) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
    }
  };

  // ---- main loop ----
  const uint32_t n_even = n_steps & ~1u;
  {
    // all waves in phase: QK, softmax, PV of a tile between two barriers (tile i + 1 of both K and V in flight)
    auto step_s = [&](auto PAR, const uint32_t i) {
      constexpr int par = decltype(PAR)::value;
      const uint32_t tp = t_begin + i * PF_TN;
      if (i + 1 < n_steps) { issue_k(par ? kbuf0 : kbuf1, tp + PF_TN); issue_v(par ? vbuf0 : vbuf1, tp + PF_TN); }
      qk(par ? kbuf1 : kbuf0, tp);
      sm(tp);
      pv(par ? vbuf1 : vbuf0, tp);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    };
    for (uint32_t i = 0; i < n_even; i += 2) {
      step_s(std::integral_constant<int, 0>{}, i);
      step_s(std::integral_constant<int, 1>{}, i + 1);
    }
    if (n_steps & 1) step_s(std::integral_constant<int, 0>{}, n_even);
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
static hipError_t launch_prefill_t(const AttnParams& p, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  typedef PfShape<HD, W> S;
  const size_t lds = (size_t)W * QB * (S::KS - S::QR) * 1024;     // Q fragments parked in LDS (dynamic part)
  static bool attr_set = false;
  if (!attr_set && lds > 0) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_prefill_kernel<HD, QB, W>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const uint32_t total = col_groups * p.n_kv_heads * p.n_splits;
  const uint32_t gx = ((total + 7) / 8) * 8;       // whole rounds of the 8 XCDs
  PA_LAUNCH((pa_prefill_kernel<HD, QB, W>), dim3(gx), dim3(W * 64), lds, s, t, p, col_groups);
  return hipGetLastError();
}

// row_blocks = 32-row query blocks per workgroup (8: one per wavefront)
hipError_t pa_launch_prefill(const AttnParams& p, uint32_t hd, uint32_t row_blocks, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  if (row_blocks != 8) return hipErrorNotSupported;
  if (hd == 256) return launch_prefill_t<256, 1, 8>(p, col_groups, s, t);
  if (hd == 128) return launch_prefill_t<128, 1, 8>(p, col_groups, s, t);
  return hipErrorNotSupported;
}
