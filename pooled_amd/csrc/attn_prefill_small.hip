// Causal prefill attention, small-MFMA-tile variant for gfx950 (MI355X).
//
// Same contract, work decomposition, LDS-direct K/V staging, global-side swizzles, lazily updated reference maximum
// and outputs as pa_prefill_kernel (attn_prefill.hip; it replaces the same reference kernels:
// engine/wgsl/attn_tile.js:108-193, engine/wgsl/qwen35.js:877-887).  What differs is the matrix instruction: the
// products run on v_mfma_f32_16x16x32_f16 instead of v_mfma_f32_32x32x16_f16.  Under the power limit of the part the
// small shape sustains 7-8 % more flops in a kernel of nothing but MFMAs (see the device probe in probe.hip); in this
// kernel that does not show -- it runs level with pa_prefill_kernel on the MoE shape at 128K rows and behind it on
// the other shapes -- so it is a measured alternative, selected by POOLED_ATTN_PREFILL_SMALL=1, not a default.
//
// A wavefront still owns 32 query rows, now as two 16-row blocks, and a step still covers 32 positions, as two
// 16-position blocks:
//   * S^T = K Q^T: A operand = 16 positions x 32 dims of K (lane = position ln, dims 8 kg ..), one ds_read_b128 that
//     feeds the MFMAs of both row blocks; B operand = the Q fragment of a row block (lane = row ln, dims 8 kg ..).
//     The accumulator of (position block pb, row block rb) holds, in lane (ln, kg), positions 16 pb + 4 kg + i of
//     row 16 rb + ln.
//   * O^T = V^T P^T: one MFMA contracts all 32 positions of the tile.  Its B operand takes contraction index
//     8 kg + j from lane (ln, kg); the two S^T accumulators of a row block hold positions 4 kg + j (j < 4) and
//     16 + 4 kg + (j - 4) there, so the probabilities go into the product as they stand and the V^T fragment is read
//     in the same order: the gfx950 transpose read of rows 4 kg .. 4 kg + 3 and of rows 16 + 4 kg .. (two
//     ds_read_b64_tr_b16), 16 dims a fragment.
//   * The K swizzle (chunk c of row r at slot c ^ (r & 15)) and the V swizzle (c ^ 4 (r & 3)) of the LDS-direct loads
//     are conflict-free for these read patterns as well.
#include "pf_common.h"
#include <cstdlib>

// Q k-steps kept in registers at hd 256, K / Q fragment k-steps and V^T fragments fetched ahead of their MFMAs: what
// fits 256 registers next to the 128 accumulators without spilling
#ifndef PS_QR
#define PS_QR 2
#endif
#ifndef PS_KD
#define PS_KD 1
#endif
#ifndef PS_VD
#define PS_VD 2
#endif

template <int HD, int W> struct PsShape {
  static constexpr int ROWB = HD * 2;             // bytes of one kv head's row
  static constexpr int TILE = PF_TN * ROWB;       // bytes of one staged tile (K or V)
  static constexpr int KS = HD / 32;              // k-steps of QK^T
  static constexpr int DB = HD / 16;              // 16-dim blocks of the output
  static constexpr int QR = HD == 256 ? PS_QR : KS;   // k-steps whose Q fragments stay in registers
  static constexpr int CPR = HD / 8;              // 16-byte chunks per row
  static constexpr int RPB = 64 / CPR;            // rows per 1 KB LDS-direct load
  static constexpr int NLD = PF_TN / RPB / W;     // LDS-direct loads per wave, tensor and step
  static_assert(NLD >= 1 && NLD * W * RPB == PF_TN, "tile must divide evenly over the waves");
};

template <int HD, int W>
__global__ __launch_bounds__(W * 64, W / 4) void pa_prefill_small_kernel(AttnParams p, uint32_t n_col_blocks) {
  typedef PsShape<HD, W> S;
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf1[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf1[S::TILE];

  // ---- XCD-aware id -> (kv head, split, column block), as in pa_prefill_kernel ----
  const uint32_t total = n_col_blocks * p.n_kv_heads * p.n_splits;
  const uint32_t per_xcd = (total + 7) / 8;
  const uint32_t lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (lid >= total) return;
  const uint32_t cb = lid % n_col_blocks, sp = (lid / n_col_blocks) % p.n_splits, g = lid / (n_col_blocks * p.n_splits);

  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ln = lane & 15, kg = lane >> 4;   // MFMA row / column index, k group
  const uint32_t G = p.group, nH = p.n_heads;
  const uint32_t c0 = cb * p.cols_per_group;
  const uint32_t ncl = min(p.cols_per_group, p.n_cols - c0);
  const uint32_t R = ncl * G;                      // live rows (<= W * 32)
  const uint32_t seq_max = p.base_pos + c0 + ncl;  // rows visible to the block's last column
  const uint32_t t_begin = sp * p.split_len;
  if (t_begin >= seq_max) return;
  const uint32_t t_end = min(t_begin + p.split_len, seq_max);
  const uint32_t n_steps = (t_end - t_begin + PF_TN - 1) / PF_TN;
  const size_t row_bytes = (size_t)HD * 2;
  const size_t head_rows = (size_t)p.max_seq + PF_TN;
  const unsigned char* kg_base = (const unsigned char*)(p.k_cache + (size_t)g * head_rows * HD);
  const unsigned char* vg_base = (const unsigned char*)(p.v_cache + (size_t)g * head_rows * HD);

  // ---- LDS-direct tile loads (global-side swizzle as in pa_prefill_kernel) ----
  uint32_t k_src[S::NLD], v_src[S::NLD], ld_row[S::NLD];
#pragma unroll
  for (int i = 0; i < S::NLD; i++) {
    const uint32_t row = (wave * S::NLD + i) * S::RPB + lane / S::CPR, slot = lane % S::CPR;
    ld_row[i] = row;
    k_src[i] = row * (uint32_t)row_bytes + (slot ^ (row & 15)) * 16;
    v_src[i] = row * (uint32_t)row_bytes + (slot ^ (4 * (row & 3))) * 16;
  }
  auto issue = [&](const unsigned char* gbase, const uint32_t* src, unsigned char* dst, uint32_t tpos) __attribute__((always_inline)) {
    const unsigned char* gt = gbase + (size_t)tpos * row_bytes;
    if (tpos + PF_TN <= t_end) {
#pragma unroll
      for (int i = 0; i < S::NLD; i++) PF_GLL(gt + src[i], dst + (wave * S::NLD + i) * 1024);
    } else {   // last tile of the context: rows at or past t_end come from the zero padding row max_seq
#pragma unroll
      for (int i = 0; i < S::NLD; i++) {
        const size_t pad = (size_t)p.max_seq * row_bytes - (size_t)ld_row[i] * row_bytes;
        PF_GLL(tpos + ld_row[i] < t_end ? gt + src[i] : gbase + pad + src[i], dst + (wave * S::NLD + i) * 1024);
      }
    }
  };
  issue(kg_base, k_src, kbuf0, t_begin);
  issue(vg_base, v_src, vbuf0, t_begin);

  // ---- per-lane rows: query row of block rb is wave*32 + rb*16 + ln = (column r / G, head r % G) ----
  uint32_t end_pos[2], row_id[2];
  uint32_t w_min_end = 0xffffffffu;
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    const uint32_t r = wave * 32 + rb * 16 + ln;
    row_id[rb] = min(r, R - 1);
    end_pos[rb] = r < R ? p.base_pos + c0 + r / G + 1 : 0u;
  }
  if (wave * 32 < R) w_min_end = p.base_pos + c0 + (wave * 32) / G + 1;

  // ---- Q fragments (B operand): row ln of block rb, dims 32 ks + 8 kg .. + 7, as f16.  The first QR k-steps stay in
  //      registers; the others are parked in LDS in fragment order and re-read every step. ----
  constexpr int QR = S::QR;
  extern __shared__ __attribute__((aligned(16))) unsigned char q_lds_all[];
  unsigned char* q_lds = q_lds_all + (size_t)wave * 2 * (S::KS - QR) * 1024 + lane * 16;
  h8 qf[2][QR];
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    const float* qrow = p.q + (size_t)(c0 + row_id[rb] / G) * p.q_stride + (size_t)(g * G + row_id[rb] % G) * HD + 8 * kg;
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      const f4 a = *(const f4*)(qrow + 32 * ks), b = *(const f4*)(qrow + 32 * ks + 4);
      const h8 f = { (_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3],
                     (_Float16)b[0], (_Float16)b[1], (_Float16)b[2], (_Float16)b[3] };
      if (ks < QR) qf[rb][ks < QR ? ks : 0] = f;
      else *(h8*)(q_lds + (rb * (S::KS - QR) + (ks - QR)) * 1024) = f;
    }
  }

  f4 acc[S::DB][2];
#pragma unroll
  for (int db = 0; db < S::DB; db++)
#pragma unroll
    for (int rb = 0; rb < 2; rb++) acc[db][rb] = (f4){0.f, 0.f, 0.f, 0.f};
  float m_ref[2], l_run[2];
#pragma unroll
  for (int rb = 0; rb < 2; rb++) { m_ref[rb] = NEG_INF; l_run[rb] = 0.f; }
  const float c1 = p.scale * 1.4426950408889634f;   // scores -> log2 domain

  // per-lane LDS read offsets with the swizzles folded in (buffer bases are 1 KB aligned, so XOR == add on the
  // swizzled bits).  K fragment (position block pb, k-step ks): row 16 pb + ln, chunk 4 ks + kg at slot chunk ^ ln.
  // V^T fragment (dim block db): rows 4 kg + (ln >> 2) (and + 16), 8 bytes at dims 16 db + 4 (ln & 3): chunk
  // 2 db + ((ln & 3) >> 1) at slot chunk ^ 4 (row & 3), byte (ln & 1) * 8 of it.
  const uint32_t k_rd = ln * S::ROWB + ((kg ^ (ln & 3)) * 16) + (ln >> 2) * 64;       // K fragment of k-step ks: k_rd ^ ((ks & 3) * 64), + (ks >> 2) * 256
  // slot = (2 db + c1) ^ 4 r3 with c1 = (ln & 3) >> 1, r3 = row & 3 = (ln >> 2) & 3, i.e. bytes 16 c1 + 32 (db ^ 2 r3): the
  // bits of db that the swizzle flips (db & 6) select one of four lane offsets, the others are an immediate
  uint32_t v_rd[4];
  {
    const uint32_t r3 = (ln >> 2) & 3;
    const uint32_t v_lane = (4 * kg + (ln >> 2)) * S::ROWB + ((ln & 3) >> 1) * 16 + (ln & 1) * 8;
#pragma unroll
    for (int q = 0; q < 4; q++) v_rd[q] = v_lane + 32 * ((2 * q) ^ (2 * r3));
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  f4 s[2][2];                       // [position block][row block]
  h8 pf[2];                         // probabilities of a row block: positions 4 kg + j (j < 4), 16 + 4 kg + (j - 4)
  // ---- S^T = K Q^T ----
  auto qk = [&](const unsigned char* kb) __attribute__((always_inline)) {
#pragma unroll
    for (int pb = 0; pb < 2; pb++)
#pragma unroll
      for (int rb = 0; rb < 2; rb++) s[pb][rb] = (f4){0.f, 0.f, 0.f, 0.f};
    constexpr int KD = PS_KD;           // k-steps of fragments fetched ahead
    h8 ka[KD][2], qa[KD][2];
    auto fetch = [&](int ks, int slot) __attribute__((always_inline)) {
#pragma unroll
      for (int pb = 0; pb < 2; pb++) ka[slot][pb] = *(const h8*)(kb + pb * 16 * S::ROWB + (k_rd ^ ((ks & 3) * 64)) + (ks >> 2) * 256);
      if (ks >= QR) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++) qa[slot][rb] = *(const h8*)(q_lds + (rb * (S::KS - QR) + (ks - QR)) * 1024);
      }
    };
#pragma unroll
    for (int ks = 0; ks < KD; ks++) fetch(ks, ks);
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      h8 a[2], b[2];
#pragma unroll
      for (int pb = 0; pb < 2; pb++) a[pb] = ka[ks % KD][pb];
#pragma unroll
      for (int rb = 0; rb < 2; rb++) b[rb] = ks < QR ? qf[rb][ks < QR ? ks : 0] : qa[ks % KD][rb];
      if (ks + KD < S::KS) fetch(ks + KD, ks % KD);
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int rb = 0; rb < 2; rb++) s[pb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[pb], b[rb], s[pb][rb], 0, 0, 0);
    }
    // pin the issue order the source states (left alone, the compiler clusters all fragment reads of the tile up front
    // and runs out of registers): the first KD fetches, then each k-step's fetches ahead of its four MFMAs
#pragma unroll
    for (int ks = 0; ks < KD; ks++) { if (ks >= QR) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0); else __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); }
#pragma unroll
    for (int ks = 0; ks < S::KS; ks++) {
      if (ks + KD < S::KS) { if (ks + KD >= QR) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0); else __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); }
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
  };
  // ---- online softmax; lane holds row ln of each row block, positions tp + 16 pb + 4 kg + i ----
  auto sm = [&](const uint32_t tp) __attribute__((always_inline)) {
    if (tp + PF_TN > w_min_end) {
      asm volatile("; causal tile" ::: "memory");
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const uint32_t pos = tp + 16 * pb + 4 * kg + i;
            s[pb][rb][i] = pos < end_pos[rb] ? s[pb][rb][i] : NEG_INF;
          }
    }
    float mt[2];
    bool grow = false;
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      float mx = fmaxf(fmaxf(s[0][rb][0], s[0][rb][1]), fmaxf(s[0][rb][2], s[0][rb][3]));
      mx = fmaxf(mx, fmaxf(fmaxf(s[1][rb][0], s[1][rb][1]), fmaxf(s[1][rb][2], s[1][rb][3])));
      // the row's four k groups sit in lanes ln, ln + 16, ln + 32, ln + 48: two lane-swap instructions, no LDS round trip
      const auto s16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mx = fmaxf(__uint_as_float(s16[0]), __uint_as_float(s16[1]));
      const auto s32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mx = fmaxf(__uint_as_float(s32[0]), __uint_as_float(s32[1]));
      mt[rb] = mx * c1;
      grow |= mt[rb] > m_ref[rb] + PF_RESCALE_TH;
    }
    if (__any(grow)) {
#pragma unroll
      for (int rb = 0; rb < 2; rb++) {
        const float m_new = fmaxf(m_ref[rb], mt[rb]);
        const float alpha = m_new == NEG_INF ? 1.f : __builtin_amdgcn_exp2f(m_ref[rb] - m_new);
        m_ref[rb] = m_new;
        l_run[rb] *= alpha;
#pragma unroll
        for (int db = 0; db < S::DB; db++) acc[db][rb] *= alpha;
      }
    }
    const h2 ones = { (_Float16)1.f, (_Float16)1.f };
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      const float nmr = m_ref[rb] == NEG_INF ? 0.f : -m_ref[rb];
      float ps = l_run[rb];
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int i = 0; i < 4; i += 2) {
          const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[pb][rb][i], c1, nmr));
          const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[pb][rb][i + 1], c1, nmr));
          const h2 pp = { (_Float16)e0, (_Float16)e1 };
          ps = __builtin_amdgcn_fdot2(pp, ones, ps, false);
          pf[rb][4 * pb + i] = pp[0]; pf[rb][4 * pb + i + 1] = pp[1];
        }
      l_run[rb] = ps;
    }
  };
  // ---- O^T += V^T P^T ----
  auto pv = [&](const unsigned char* vb) __attribute__((always_inline)) {
    constexpr int VD = PS_VD;           // fragments fetched ahead
    h4 lor[VD], hir[VD];
    auto fetch = [&](int db, int slot) __attribute__((always_inline)) {
      const unsigned char* vp = vb + v_rd[(db & 6) >> 1] + 32 * (db & ~6);
      lor[slot] = lds_read_tr16(vp);
      hir[slot] = lds_read_tr16(vp + 16 * S::ROWB);
    };
#pragma unroll
    for (int db = 0; db < VD; db++) fetch(db, db);
#pragma unroll
    for (int db = 0; db < S::DB; db++) {
      const h4 lo = lor[db % VD], hi = hir[db % VD];
      if (db + VD < S::DB) fetch(db + VD, db % VD);
      const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
#pragma unroll
      for (int rb = 0; rb < 2; rb++) acc[db][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pf[rb], acc[db][rb], 0, 0, 0);
    }
#pragma unroll
    for (int db = 0; db < VD; db++) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
#pragma unroll
    for (int db = 0; db < S::DB; db++) {
      if (db + VD < S::DB) __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 1);
    }
  };

  // ---- main loop: all waves in phase; tile i + 1 of K and V in flight while tile i is consumed.  Unrolled twice so
  //      that the buffer of a step is a compile-time address. ----
  auto step = [&](auto PAR, const uint32_t i) __attribute__((always_inline)) {
    constexpr int par = decltype(PAR)::value;
    const uint32_t tp = t_begin + i * PF_TN;
    if (i + 1 < n_steps) { issue(kg_base, k_src, par ? kbuf0 : kbuf1, tp + PF_TN); issue(vg_base, v_src, par ? vbuf0 : vbuf1, tp + PF_TN); }
    qk(par ? kbuf1 : kbuf0);
    sm(tp);
    pv(par ? vbuf1 : vbuf0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  const uint32_t n_even = n_steps & ~1u;
  for (uint32_t i = 0; i < n_even; i += 2) {
    step(std::integral_constant<int, 0>{}, i);
    step(std::integral_constant<int, 1>{}, i + 1);
  }
  if (n_steps & 1) step(std::integral_constant<int, 0>{}, n_even);

  // ---- epilogue: lane (ln, kg) holds dims 16 db + 4 kg + i of row 16 rb + ln ----
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    l_run[rb] += __shfl_xor(l_run[rb], 16, 64);
    l_run[rb] += __shfl_xor(l_run[rb], 32, 64);
    const uint32_t r = wave * 32 + rb * 16 + ln;
    if (r >= R) continue;
    const uint32_t col = c0 + r / G, hq = g * G + r % G;
    if (p.n_splits == 1) {
      const float inv_l = 1.f / l_run[rb];
      const float* gate = p.gate ? p.gate + (size_t)col * p.gate_stride + (size_t)hq * HD : nullptr;
#pragma unroll
      for (int db = 0; db < S::DB; db++) {
        const uint32_t d = 16 * db + 4 * kg;
        f4 o = acc[db][rb] * inv_l;
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
    } else {
      const size_t slot = ((size_t)col * nH + hq) * p.slots + sp;
#pragma unroll
      for (int db = 0; db < S::DB; db++) *(f4*)(p.part_o + slot * HD + 16 * db + 4 * kg) = acc[db][rb];
      if (kg == 0) {
        p.part_ml[slot * 2] = m_ref[rb] * 0.6931471805599453f;
        p.part_ml[slot * 2 + 1] = l_run[rb];
      }
    }
  }
}

template <int HD>
static hipError_t launch_small_t(const AttnParams& p, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  typedef PsShape<HD, 8> S;
  const size_t lds = (size_t)8 * 2 * (S::KS - S::QR) * 1024;     // Q fragments parked in LDS (dynamic part)
  static bool attr_set = false;
  if (!attr_set && lds > 0) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_prefill_small_kernel<HD, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const uint32_t total = col_groups * p.n_kv_heads * p.n_splits;
  const uint32_t gx = ((total + 7) / 8) * 8;       // whole rounds of the 8 XCDs
  PA_LAUNCH((pa_prefill_small_kernel<HD, 8>), dim3(gx), dim3(8 * 64), lds, s, t, p, col_groups);
  return hipGetLastError();
}

hipError_t pa_launch_prefill_small(const AttnParams& p, uint32_t hd, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  if (hd == 256) return launch_small_t<256>(p, col_groups, s, t);
  if (hd == 128) return launch_small_t<128>(p, col_groups, s, t);
  return hipErrorNotSupported;
}
