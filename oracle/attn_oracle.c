/* CPU oracle for pooled's attention hot path (plain C, f64).  TEST INFRASTRUCTURE ONLY.
 *
 * A restatement of the reference's CPU attention for shapes too large for the numpy oracle:
 *   tests/reference/ref_qwen.mjs:114-131, tests/reference/ref_q38.mjs:171-191,
 *   tests/test_attn_dec.js:72-82, tests/unit/attn_tile_test.js:63-78
 *     s_t = (q_h . k_t) / sqrt(hd);  p_t = exp(s_t - max);  out_h = sum_t p_t v_t / sum_t p_t;
 *     optional out *= 1 / (1 + exp(-gate));  kv head = floor(h / (nH / nKV));
 *     column c at absolute position base_pos + c attends to cache rows [0, base_pos + c].
 * K/V are f16 bits widened exactly; every product and sum is f64.  The context is processed in
 * chunks (one OpenMP task per (column, kv head, chunk)) whose (m, l, O) partials are merged in
 * chunk order with the log-sum-exp rule (engine/wgsl/attn_dec.js:215-287), so the result does not
 * depend on the thread count.
 *
 * Pinned by tests/test_oracle.py against the numpy oracle, brute-force loops and closed forms.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float h2f(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u, u;
  if (e == 0) {
    if (m == 0) u = s;
    else { int sh = 0; while (!(m & 1024u)) { m <<= 1; sh++; } u = s | ((uint32_t)(113 - sh) << 23) | ((m & 1023u) << 13); }
  } else if (e == 31) u = s | 0x7f800000u | (m << 13);
  else u = s | ((e + 112u) << 23) | (m << 13);
  float f; memcpy(&f, &u, 4); return f;
}

#define CHUNK 2048

/* q: [n_cols][q_stride] f32 (head-major [nH][hd] inside a column); k16, v16: [rows][nKV][hd] f16 bits;
 * gate: NULL or [n_cols][gate_stride] f32; sel: NULL (all columns) or n_sel column indices;
 * out: [n_out][nH][hd] f64 where n_out = n_sel (or n_cols), row i = column sel[i].
 * Returns 0, or -1 on a bad shape / allocation failure. */
int pa_oracle_attention(const float* q, long q_stride, const uint16_t* k16, const uint16_t* v16,
                        int n_cols, const int* sel, int n_sel, int nH, int nKV, int hd, long base_pos,
                        const float* gate, long gate_stride, double* out) {
  if (nH <= 0 || nKV <= 0 || hd <= 0 || nH % nKV || n_cols <= 0) return -1;
  const int G = nH / nKV, n_out = sel ? n_sel : n_cols;
  const long kvd = (long)nKV * hd;
  const double rs = sqrt((double)hd);
  long maxL = base_pos + n_cols, maxChunks = (maxL + CHUNK - 1) / CHUNK;
  const long psz = (long)G * (hd + 2);                 /* per-task partial: O[G][hd], m[G], l[G] */
  long ntask = (long)n_out * nKV * maxChunks;
  double* part = (double*)malloc(sizeof(double) * psz * ntask);
  if (!part) return -1;
  int fail = 0;
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * hd);
    double* sc = (double*)malloc(sizeof(double) * (size_t)G * CHUNK);
    if (!row || !sc) {
#pragma omp atomic write
      fail = 1;
    } else {
#pragma omp for schedule(dynamic, 1)
      for (long task = 0; task < ntask; task++) {
        long ch = task % maxChunks, g = (task / maxChunks) % nKV, oi = task / (maxChunks * nKV);
        int c = sel ? sel[oi] : (int)oi;
        long L = base_pos + c + 1, t0 = ch * CHUNK, t1 = t0 + CHUNK < L ? t0 + CHUNK : L;
        double* P = part + task * psz;
        double* O = P; double* m = P + (long)G * hd; double* l = m + G;
        for (long i = 0; i < (long)G * hd; i++) O[i] = 0.0;
        for (int h = 0; h < G; h++) { m[h] = -INFINITY; l[h] = 0.0; }
        if (t0 >= L) continue;
        const float* qc = q + (long)c * q_stride + g * G * hd;
        for (long t = t0; t < t1; t++) {
          const uint16_t* kr = k16 + t * kvd + g * hd;
          for (int i = 0; i < hd; i++) row[i] = h2f(kr[i]);
          for (int h = 0; h < G; h++) {
            const float* qh = qc + h * hd; double a = 0.0;
            for (int i = 0; i < hd; i++) a += (double)qh[i] * (double)row[i];
            a /= rs; sc[(long)h * CHUNK + (t - t0)] = a; if (a > m[h]) m[h] = a;
          }
        }
        for (int h = 0; h < G; h++) {
          double s = 0.0;
          for (long t = t0; t < t1; t++) { double e = exp(sc[(long)h * CHUNK + (t - t0)] - m[h]); sc[(long)h * CHUNK + (t - t0)] = e; s += e; }
          l[h] = s;
        }
        for (long t = t0; t < t1; t++) {
          const uint16_t* vr = v16 + t * kvd + g * hd;
          for (int i = 0; i < hd; i++) row[i] = h2f(vr[i]);
          for (int h = 0; h < G; h++) {
            double p = sc[(long)h * CHUNK + (t - t0)]; double* Oh = O + (long)h * hd;
            for (int i = 0; i < hd; i++) Oh[i] += p * (double)row[i];
          }
        }
      }
    }
    free(row); free(sc);
  }
  if (!fail) {
    for (long oi = 0; oi < n_out; oi++) for (long g = 0; g < nKV; g++) {
      int c = sel ? sel[oi] : (int)oi;
      long L = base_pos + c + 1, nch = (L + CHUNK - 1) / CHUNK;
      for (int h = 0; h < G; h++) {
        double M = -INFINITY;
        for (long ch = 0; ch < nch; ch++) { double v = part[((oi * nKV + g) * maxChunks + ch) * psz + (long)G * hd + h]; if (v > M) M = v; }
        double Lsum = 0.0; double* o = out + (oi * nH + g * G + h) * hd;
        for (int i = 0; i < hd; i++) o[i] = 0.0;
        for (long ch = 0; ch < nch; ch++) {
          const double* P = part + ((oi * nKV + g) * maxChunks + ch) * psz;
          double w = exp(P[(long)G * hd + h] - M);
          Lsum += P[(long)G * hd + G + h] * w;
          for (int i = 0; i < hd; i++) o[i] += P[(long)h * hd + i] * w;
        }
        for (int i = 0; i < hd; i++) o[i] /= Lsum;
        if (gate) {
          const float* gt = gate + (long)c * gate_stride + (g * G + h) * hd;
          for (int i = 0; i < hd; i++) o[i] *= 1.0 / (1.0 + exp(-(double)gt[i]));
        }
      }
    }
  }
  free(part);
  return fail ? -1 : 0;
}

/* Single-threaded f32-storage restatement with the reference's own loop order (one head at a time, scores
 * array, softmax, weighted sum of V rows), used to time "the reference CPU path" when Node is not available.
 * tests/reference/ref_qwen.mjs:114-131.  K/V given as f32 (already widened). out: [nH][hd] f32. */
int pa_oracle_attention_ref_loops(const float* q, const float* K, const float* V, long L, int nH, int nKV, int hd,
                                  const float* gate, float* out) {
  const int G = nH / nKV; const long kvd = (long)nKV * hd;
  double* sc = (double*)malloc(sizeof(double) * (size_t)L);
  if (!sc) return -1;
  for (int h = 0; h < nH; h++) {
    int kvH = h / G; double mx = -INFINITY;
    for (long t = 0; t < L; t++) {
      double a = 0.0; const float* kt = K + t * kvd + kvH * hd;
      for (int i = 0; i < hd; i++) a += (double)q[h * hd + i] * (double)kt[i];
      sc[t] = (double)(float)(a / sqrt((double)hd)); if (sc[t] > mx) mx = sc[t];
    }
    double sum = 0.0;
    for (long t = 0; t < L; t++) { sc[t] = (double)(float)exp(sc[t] - mx); sum += sc[t]; }
    float* o = out + h * hd;
    for (int i = 0; i < hd; i++) o[i] = 0.f;
    for (long t = 0; t < L; t++) {
      double wt = sc[t] / sum; const float* vt = V + t * kvd + kvH * hd;
      for (int i = 0; i < hd; i++) o[i] = (float)((double)o[i] + wt * (double)vt[i]);
    }
    if (gate) for (int i = 0; i < hd; i++) o[i] = (float)((double)o[i] * (1.0 / (1.0 + exp(-(double)gate[h * hd + i]))));
  }
  free(sc);
  return 0;
}
