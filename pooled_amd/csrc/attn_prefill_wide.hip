// Causal prefill attention, wide-tile variant for gfx950 (MI355X).
//
// Same contract, data layout, swizzles and epilogue as pa_prefill_kernel (attn_prefill.hip; it replaces the same
// reference kernels: engine/wgsl/attn_tile.js:108-193, engine/wgsl/qwen35.js:877-887).  What differs is the shape
// of the work inside a workgroup:
//
//   * 4 wavefronts, one per SIMD, each owning 64 query rows (two 32-row blocks) with the whole 512-register
//     budget.  Every K and V^T fragment read from LDS feeds two MFMAs, so LDS fragment traffic per MFMA is half of
//     the 8-wave kernel's -- the resource that kernel runs out of.
//   * Register allocation is split by hand.  The O accumulators (16 DB QB = 256 registers at hd 256) live in
//     AGPRs that the compiler never sees: every instruction touching them is inline assembly naming a[..]
//     directly (MFMA with AGPR C/D, v_accvgpr_read / write for the rare rescale and the epilogue).  The S^T
//     accumulators use the VGPR form of the MFMA, again through assembly, because the compiler picks one form per
//     kernel.  Everything else (Q, K, V fragments, softmax state) is ordinary compiler-allocated VGPR code that
//     has to fit 256 registers without spilling: a compiler-made spill could land in an AGPR it believes free.
//     The assembly statements are volatile, so LDS fragment reads keep their source order relative to the MFMAs:
//     the fetch-ahead distance written below is the one that executes.
//   * MFMA results need wait states before a VALU instruction may read them; the compiler inserts those for MFMAs
//     it knows, here they are explicit s_nop at the three places a VALU read follows (end of QK, rescale,
//     epilogue).
#include "pf_common.h"
#include <cstdlib>
#include <utility>

template <class F, int... I>
static __device__ __attribute__((always_inline)) void pw_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, class F> static __device__ __attribute__((always_inline)) void pw_for(F&& f) {
  pw_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Every assembly statement of the kernel names all 256 AGPRs as clobbered: the compiler may use a free AGPR as a
// cheap spill slot for a VGPR, and no such value can then stay there across any of these statements (the build
// additionally scans the generated code for AGPR accesses outside the assembly blocks).
#define PW_A10(t) "a" #t "0", "a" #t "1", "a" #t "2", "a" #t "3", "a" #t "4", "a" #t "5", "a" #t "6", "a" #t "7", "a" #t "8", "a" #t "9"
#define PW_ALL_AGPRS "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", PW_A10(1), PW_A10(2), PW_A10(3), PW_A10(4), PW_A10(5), \
  PW_A10(6), PW_A10(7), PW_A10(8), PW_A10(9), PW_A10(10), PW_A10(11), PW_A10(12), PW_A10(13), PW_A10(14), PW_A10(15), PW_A10(16), \
  PW_A10(17), PW_A10(18), PW_A10(19), PW_A10(20), PW_A10(21), PW_A10(22), PW_A10(23), PW_A10(24), "a250", "a251", "a252", "a253", "a254", "a255"

// ---- hand-allocated AGPR accumulators: tile t = a[16 t .. 16 t + 15] ----
template <int T> static __device__ __attribute__((always_inline)) void pw_acc_mfma(const h8 a, const h8 b) {
  asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" :: "v"(a), "v"(b), "n"(16 * T), "n"(16 * T + 15) : PW_ALL_AGPRS);
}
template <int R> static __device__ __attribute__((always_inline)) void pw_acc_zero() {
  asm volatile("v_accvgpr_write_b32 a[%0], 0" :: "n"(R) : PW_ALL_AGPRS);
}
template <int R> static __device__ __attribute__((always_inline)) float pw_acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(R) : PW_ALL_AGPRS);
  return x;
}
template <int R> static __device__ __attribute__((always_inline)) void pw_acc_scale(const float alpha) {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %1, %0\n\tv_accvgpr_write_b32 a[%2], %0" : "=&v"(t) : "v"(alpha), "n"(R) : PW_ALL_AGPRS);
}
// VGPR-form MFMA for the S^T accumulators.  FIRST: C = 0 (no read of s); LAST: followed by the wait states an
// 8-pass MFMA result needs before VALU reads it.
template <bool FIRST, bool LAST> static __device__ __attribute__((always_inline)) void pw_s_mfma(f16v& s, const h8 a, const h8 b) {
  if (FIRST) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s) : "v"(a), "v"(b) : PW_ALL_AGPRS);
  else if (!LAST) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "v"(a), "v"(b) : PW_ALL_AGPRS);
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 1" : "+v"(s) : "v"(a), "v"(b) : PW_ALL_AGPRS);
}

template <int HD, int QR_> struct PwShape {
  static constexpr int W = 4, QB = 2;
  static constexpr int ROWB = HD * 2;             // bytes of one kv head's row
  static constexpr int TILE = PF_TN * ROWB;       // bytes of one staged tile (K or V)
  static constexpr int KS = HD / 16;              // k-steps of QK^T
  static constexpr int DB = HD / 32;              // 32-dim blocks of the output
  static constexpr int QR = QR_ < KS ? QR_ : KS;  // k-steps whose Q fragments stay in registers
  static constexpr int CPR = HD / 8;              // 16-byte chunks per row
  static constexpr int RPB = 64 / CPR;            // rows per 1 KB LDS-direct load
  static constexpr int NLD = PF_TN / RPB / W;     // LDS-direct loads per wave, tensor and step
  static constexpr int NF = 2 * DB;               // V^T fragments per tile
  static constexpr int NACC = 16 * DB * QB;       // AGPRs holding O
};

template <int HD, int QR_>
__global__ __launch_bounds__(256, 1) void pa_prefill_wide_kernel(AttnParams p, uint32_t n_col_blocks) {
  typedef PwShape<HD, QR_> S;
  constexpr int QB = S::QB, QR = S::QR;
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char kbuf1[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf0[S::TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char vbuf1[S::TILE];
  extern __shared__ __attribute__((aligned(16))) unsigned char q_lds_all[];


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
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ln = lane & 31, hb = lane >> 5;
  const uint32_t G = p.group, nH = p.n_heads;
  const uint32_t c0 = cb * p.cols_per_group;
#ifdef PW_CLK   // development builds: shader clock vs 100 MHz wall clock over the kernel
  long long clk0 = clock64(), wc0 = wall_clock64();
#endif
  const uint32_t ncl = min(p.cols_per_group, p.n_cols - c0);
  const uint32_t R = ncl * G;
  const uint32_t seq_max = p.base_pos + c0 + ncl;
  const uint32_t t_begin = sp * p.split_len;
  if (t_begin >= seq_max) return;
  const uint32_t t_end = min(t_begin + p.split_len, seq_max);
  const uint32_t n_steps = (t_end - t_begin + PF_TN - 1) / PF_TN;
  const size_t row_bytes = (size_t)HD * 2;                       // head-major caches: a kv head's rows are contiguous
  const size_t head_rows = (size_t)p.max_seq + PF_TN;            // rows of one kv head's plane, padding included
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
  if (n_steps > 1) issue(kg_base, k_src, kbuf1, t_begin + PF_TN);
  // iteration 0 runs the PV product of a tile "-1": P = 0 times this zeroed buffer
  for (uint32_t o = tid * 16; o < (uint32_t)S::TILE; o += 256 * 16) *(u4*)(vbuf1 + o) = u4{0, 0, 0, 0};

  // ---- per-lane rows: query row of block qb is wave*64 + qb*32 + ln = (column r / G, head r % G) ----
  uint32_t end_pos[QB], row_id[QB];
  uint32_t w_min_end = 0xffffffffu;
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const uint32_t r = wave * QB * 32 + qb * 32 + ln;
    row_id[qb] = min(r, R - 1);
    end_pos[qb] = r < R ? p.base_pos + c0 + r / G + 1 : 0u;
  }
  if (wave * QB * 32 < R) w_min_end = p.base_pos + c0 + (wave * QB * 32) / G + 1;

  // ---- Q fragments: the first QR k-steps in registers, the rest parked in LDS in fragment order ----
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

  pw_for<S::NACC>([&](auto I) { pw_acc_zero<decltype(I)::value>(); });
  float m_ref[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) { m_ref[qb] = NEG_INF; l_run[qb] = 0.f; }
  const float c1 = p.scale * 1.4426950408889634f;   // scores -> log2 domain

  const uint32_t k_rd = ln * S::ROWB + ((hb ^ (ln & 1)) * 16) + ((ln & 15) >> 1) * 32;
  const uint32_t b4 = lane >> 4, sl = lane & 15;
  const uint32_t v_rd = (4 * (b4 >> 1) + (sl >> 2)) * S::ROWB + (2 * (b4 & 1) + ((sl & 3) >> 1)) * 16 + (sl & 1) * 8 + ((sl >> 2) & 3) * 64;

  // ---- software-pipelined main loop ----
  // A single wave per SIMD has nobody to fill the MFMA pipe during its softmax, so the loop is pipelined across
  // tiles.  Iteration i issues, in this order:
  //   phase A: the PV MFMAs of tile i-1, with the row maxima of tile i (VALU) slotted between them,
  //   the (rare) rescale of O, which in program order follows PV(i-1) and so scales it too,
  //   phase C: the QK MFMAs of tile i+1, with exp2 / f16 conversion / row sums of tile i slotted between them.
  // S^T is double buffered in registers (s[i & 1]); LDS holds K(i+1) and V(i-1) while the LDS-direct loads of
  // K(i+2) and V(i) are in flight; one barrier per iteration.  A scheduling barrier after every pair of MFMAs with
  // its fragment reads and softmax slice keeps the compiler from regrouping the two instruction streams.
  constexpr int KD = 4, QD = 2, VD = 4;
  f16v s[2][QB];
  h8 pf[QB][2];
#pragma unroll
  for (int qb = 0; qb < QB; qb++)
#pragma unroll
    for (int j = 0; j < 2; j++) pf[qb][j] = h8{0, 0, 0, 0, 0, 0, 0, 0};
  h8 ka[KD], qa[QB][QD];
  h4 vlo[VD], vhi[VD];
  auto k_preload = [&](const unsigned char* kb) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < KD; i++) ka[i] = *(const h8*)(kb + (k_rd ^ (i * 32)));
#pragma unroll
    for (int i = 0; i < QD; i++)
      if (i >= QR) {
#pragma unroll
        for (int qb = 0; qb < QB; qb++) qa[qb][i] = *(const h8*)(q_lds + (qb * (S::KS - QR) + (i - QR)) * 1024);
      }
  };
  auto v_preload = [&](const unsigned char* vb) __attribute__((always_inline)) {
#pragma unroll
    for (int f = 0; f < VD; f++) {
      const unsigned char* vp = vb + (v_rd ^ ((f % S::DB) * 64)) + (f / S::DB) * 16 * S::ROWB;
      vlo[f] = lds_read_tr16(vp);
      vhi[f] = lds_read_tr16(vp + 8 * S::ROWB);
    }
  };
  // k-step ks of S^T = K Q^T into sd (both query blocks share the K fragment), then the fetches KD / QD steps ahead
  auto qk_step = [&](auto KSI, f16v (&sd)[QB], const unsigned char* kb) __attribute__((always_inline)) {
    constexpr int ks = decltype(KSI)::value;
    const h8 a = ka[ks % KD];
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
      const h8 b = ks < QR ? qf[qb][ks < QR ? ks : 0] : qa[qb][ks % QD];
      pw_s_mfma<ks == 0, (ks == S::KS - 1)>(sd[qb], a, b);
    }
    if (ks + KD < S::KS) ka[ks % KD] = *(const h8*)(kb + (k_rd ^ ((ks + KD) * 32)));
    if (ks + QD < S::KS && ks + QD >= QR) {
#pragma unroll
      for (int qb = 0; qb < QB; qb++) qa[qb][ks % QD] = *(const h8*)(q_lds + (qb * (S::KS - QR) + (ks + QD - QR)) * 1024);
    }
  };
  // fragment f = j DB + db of O^T += V^T P^T (positions 16 j .., dims 32 db ..; both query blocks share it)
  auto pv_step = [&](auto FI, const unsigned char* vb) __attribute__((always_inline)) {
    constexpr int f = decltype(FI)::value;
    const h4 lo = vlo[f % VD], hi = vhi[f % VD];
    const h8 a = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    pw_acc_mfma<(f % S::DB) * QB + 0>(a, pf[0][f / S::DB]);
    pw_acc_mfma<(f % S::DB) * QB + 1>(a, pf[1][f / S::DB]);
    if (f + VD < S::NF) {
      constexpr int fn = f + VD;
      const unsigned char* vp = vb + (v_rd ^ ((fn % S::DB) * 64)) + (fn / S::DB) * 16 * S::ROWB;
      vlo[f % VD] = lds_read_tr16(vp);
      vhi[f % VD] = lds_read_tr16(vp + 8 * S::ROWB);
    }
  };

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  k_preload(kbuf0);
  pw_for<S::KS>([&](auto KSI) { qk_step(KSI, s[0], kbuf0); });

  const h2 ones = { (_Float16)1.f, (_Float16)1.f };
  auto iter = [&](auto PAR, const uint32_t i) __attribute__((always_inline)) {
    constexpr int par = decltype(PAR)::value;         // tile i lives in s[par], K(i+1) in kbuf[1-par], V(i-1) in vbuf[1-par]
    const uint32_t tp = t_begin + i * PF_TN;
    f16v (&sc)[QB] = s[par];
    const unsigned char* vb = par ? vbuf0 : vbuf1;
    const unsigned char* kb = par ? kbuf0 : kbuf1;
    v_preload(vb);
    if (i + 2 < n_steps) issue(kg_base, k_src, par ? kbuf1 : kbuf0, tp + 2 * PF_TN);
    issue(vg_base, v_src, par ? vbuf1 : vbuf0, tp);
    if (tp + PF_TN > w_min_end) {
      asm volatile("; causal tile" ::: "memory");
#pragma unroll
      for (int qb = 0; qb < QB; qb++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          const uint32_t pos = tp + 8 * (e >> 2) + 4 * hb + (e & 3);
          sc[qb][e] = pos < end_pos[qb] ? sc[qb][e] : NEG_INF;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase A: PV(i-1) || row maxima of tile i ----
    float mx[QB];
    constexpr int MPG = 16 / S::NF;                   // max slices per fragment
    pw_for<S::NF>([&](auto FI) {
      constexpr int f = decltype(FI)::value;
      pv_step(FI, vb);
      if (f == S::NF - 2) k_preload(kb);
#pragma unroll
      for (int t = 0; t < MPG; t++) {
        const int c = f * MPG + t, qb = c / 8, j = c % 8;
        if (j == 0) mx[qb] = fmaxf(sc[qb][0], sc[qb][1]);
        else mx[qb] = fmaxf(fmaxf(mx[qb], sc[qb][2 * j]), sc[qb][2 * j + 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    float mt[QB];
    bool grow = false;
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx[qb]), __float_as_uint(mx[qb]), false, false);
      mt[qb] = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * c1;
      grow |= mt[qb] > m_ref[qb] + PF_RESCALE_TH;
    }
    if (__any(grow)) {
      float alpha[QB];
#pragma unroll
      for (int qb = 0; qb < QB; qb++) {
        const float m_new = fmaxf(m_ref[qb], mt[qb]);
        alpha[qb] = m_new == NEG_INF ? 1.f : __builtin_amdgcn_exp2f(m_ref[qb] - m_new);
        m_ref[qb] = m_new;
        l_run[qb] *= alpha[qb];
      }
      asm volatile("s_nop 15" ::: "memory");          // last PV MFMA -> v_accvgpr_read
      pw_for<S::NACC>([&](auto I) {
        constexpr int r = decltype(I)::value;
        pw_acc_scale<r>(alpha[(r / 16) % QB]);
      });
      asm volatile("s_nop 3" ::: "memory");           // v_accvgpr_write -> next MFMA
    }
    float nmr[QB];
#pragma unroll
    for (int qb = 0; qb < QB; qb++) nmr[qb] = m_ref[qb] == NEG_INF ? 0.f : -m_ref[qb];
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase C: QK(i+1) || exp2, f16 conversion and row sums of tile i ----
    constexpr int EPG = 16 / S::KS;                   // exp pairs per k-step
    pw_for<S::KS>([&](auto KSI) {
      constexpr int ks = decltype(KSI)::value;
      qk_step(KSI, s[1 - par], kb);
#pragma unroll
      for (int t = 0; t < EPG; t++) {
        const int c = ks * EPG + t, qb = c / 8, e = 2 * (c % 8);
        const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[qb][e], c1, nmr[qb]));
        const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[qb][e + 1], c1, nmr[qb]));
        const h2 pp = { (_Float16)e0, (_Float16)e1 };
        l_run[qb] = __builtin_amdgcn_fdot2(pp, ones, l_run[qb], false);
        pf[qb][e >> 3][e & 7] = pp[0]; pf[qb][e >> 3][(e & 7) + 1] = pp[1];
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  const uint32_t n_even = n_steps & ~1u;
  for (uint32_t i = 0; i < n_even; i += 2) {
    iter(std::integral_constant<int, 0>{}, i);
    iter(std::integral_constant<int, 1>{}, i + 1);
  }
  if (n_steps & 1) iter(std::integral_constant<int, 0>{}, n_even);
  // drain: PV of the last tile (its V landed before the last barrier)
  {
    const unsigned char* vb = ((n_steps - 1) & 1) ? vbuf1 : vbuf0;
    v_preload(vb);
    pw_for<S::NF>([&](auto FI) { pv_step(FI, vb); });
  }

#ifdef PW_CLK
  if (p.trace && tid == 0) { p.trace[blockIdx.x * 2] = clock64() - clk0; p.trace[blockIdx.x * 2 + 1] = wall_clock64() - wc0; }
#endif
  // ---- epilogue (same outputs as pa_prefill_kernel) ----
  asm volatile("s_nop 15" ::: "memory");              // last PV MFMA -> v_accvgpr_read
  pw_for<QB>([&](auto QBI) {
    constexpr int qb = decltype(QBI)::value;
    l_run[qb] += __shfl_xor(l_run[qb], 32, 64);
    const uint32_t r = wave * QB * 32 + qb * 32 + ln;
    if (r < R) {
      const uint32_t col = c0 + r / G, hq = g * G + r % G;
      const bool whole = p.n_splits == 1;
      // whole context seen: normalise, gate, convert, store; else un-normalised partial for the merge kernel
      const float inv_l = whole ? 1.f / l_run[qb] : 1.f;
      const float* gate = whole && p.gate ? p.gate + (size_t)col * p.gate_stride + (size_t)hq * HD : nullptr;
      const size_t slot = ((size_t)col * nH + hq) * p.slots + sp;
      pw_for<S::DB * 4>([&](auto DI) {
        constexpr int db = decltype(DI)::value / 4, q4 = decltype(DI)::value % 4;
        constexpr int rb = 16 * (db * QB + qb) + 4 * q4;
        const uint32_t d = 32 * db + 8 * q4 + 4 * hb;
        f4 o = { pw_acc_read<rb>() * inv_l, pw_acc_read<rb + 1>() * inv_l, pw_acc_read<rb + 2>() * inv_l, pw_acc_read<rb + 3>() * inv_l };
        if (gate) {
          const f4 gt = *(const f4*)(gate + d);
#pragma unroll
          for (int i = 0; i < 4; i++) o[i] *= 1.f / (1.f + __expf(-gt[i]));
        }
        if (!whole) {
          *(f4*)(p.part_o + slot * HD + d) = o;
        } else if (p.out_f16) {
          const h4 hv = { (_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3] };
          *(h4*)((_Float16*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + d) = hv;
        } else {
          *(f4*)((float*)p.out + (size_t)col * p.out_stride + (size_t)hq * HD + d) = o;
        }
      });
      if (!whole && hb == 0) {
        p.part_ml[slot * 2] = m_ref[qb] * 0.6931471805599453f;
        p.part_ml[slot * 2 + 1] = l_run[qb];
      }
    }
  });
}

#ifndef PW_QR
#define PW_QR 10
#endif

template <int HD>
static hipError_t launch_wide_t(const AttnParams& p, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  typedef PwShape<HD, PW_QR> S;
  const size_t lds = (size_t)S::W * S::QB * (S::KS - S::QR) * 1024;     // Q fragments parked in LDS (dynamic part)
  static bool attr_set = false;
  if (!attr_set && lds > 0) {
    hipError_t e = hipFuncSetAttribute((const void*)pa_prefill_wide_kernel<HD, PW_QR>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  const uint32_t total = col_groups * p.n_kv_heads * p.n_splits;
  const uint32_t gx = ((total + 7) / 8) * 8;
  PA_LAUNCH((pa_prefill_wide_kernel<HD, PW_QR>), dim3(gx), dim3(256), lds, s, t, p, col_groups);
  return hipGetLastError();
}

hipError_t pa_launch_prefill_wide(const AttnParams& p, uint32_t hd, uint32_t col_groups, hipStream_t s, const PaTiming* t) {
  if (hd == 256) return launch_wide_t<256>(p, col_groups, s, t);
  if (hd == 128) return launch_wide_t<128>(p, col_groups, s, t);
  return hipErrorNotSupported;
}
