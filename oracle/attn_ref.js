// CPU oracle, JavaScript leg: pooled's reference attention loops restated for Node.  TEST INFRASTRUCTURE ONLY
// (tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg are the only callers).
//
// The reference's CPU attention lives inside whole-model scripts that open model files at import time
// (tests/reference/ref_qwen.mjs:65-66, ref_q38.mjs:10-13), so the loops are restated here with the same
// storage types and loop order: Float32Array scores, JS-double arithmetic, one query head at a time
//   tests/reference/ref_qwen.mjs:114-131      (scores -> softmaxInPlace -> sum of s * v rows)
//   tests/reference/ref_q38.mjs:171-191       (same, with wt = sc[t] / sum and the sigmoid gate)
// and f16 widening as tests/test_attn_dec.js:26 (h2f).  Single-threaded, like the reference.
//
// usage: node attn_ref.js <in.bin> <out.bin|-> [reps]
//   in.bin : int32 header [nCols, nH, nKV, hd, basePos, rows, hasGate, selCount] then selCount int32 column
//            indices, then q f32 [nCols][nH*hd], K u16 [rows][nKV*hd], V u16 [rows][nKV*hd], gate f32 [nCols][nH*hd]
//   out.bin: f32 [selCount][nH*hd]; prints one JSON line {"ms": best, "reps": n, "node": version, "max_weight": largest
//            softmax weight of any (column, head) -- 1 / sum after the maximum is subtracted: a peaked row shows here --
//            "cpus": os.cpus().length, "cpu_model": ...}
"use strict";
const fs = require("fs");
const os = require("os");
let maxWeight = 0;

function h2f(h) {
  const s = h & 0x8000 ? -1 : 1, e = (h >> 10) & 31, m = h & 1023;
  if (e === 0) return s * m * Math.pow(2, -24);
  if (e === 31) return m ? NaN : s * Infinity;
  return s * (1 + m / 1024) * Math.pow(2, e - 15);
}

function attention(q, K, V, gate, nH, nKV, hd, seqLen, attn) {
  const group = nH / nKV, kvDim = nKV * hd;
  const sc = new Float32Array(seqLen);
  attn.fill(0);
  for (let h = 0; h < nH; h++) {
    const kvH = Math.floor(h / group);
    for (let t = 0; t < seqLen; t++) {
      let acc = 0;
      const ko = t * kvDim + kvH * hd;
      for (let i = 0; i < hd; i++) acc += q[h * hd + i] * K[ko + i];
      sc[t] = acc / Math.sqrt(hd);
    }
    let mx = -Infinity;
    for (let t = 0; t < seqLen; t++) if (sc[t] > mx) mx = sc[t];
    let sum = 0;
    for (let t = 0; t < seqLen; t++) { sc[t] = Math.exp(sc[t] - mx); sum += sc[t]; }
    if (1 / sum > maxWeight) maxWeight = 1 / sum;
    for (let t = 0; t < seqLen; t++) {
      const wt = sc[t] / sum, vo = t * kvDim + kvH * hd;
      for (let i = 0; i < hd; i++) attn[h * hd + i] += wt * V[vo + i];
    }
  }
  if (gate) for (let i = 0; i < attn.length; i++) attn[i] *= 1 / (1 + Math.exp(-gate[i]));
}

function main() {
  const inPath = process.argv[2], outPath = process.argv[3], reps = Math.max(1, parseInt(process.argv[4] || "1", 10));
  const buf = fs.readFileSync(inPath);
  const ab = buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
  const hdr = new Int32Array(ab, 0, 8);
  const nCols = hdr[0], nH = hdr[1], nKV = hdr[2], hd = hdr[3], basePos = hdr[4], rows = hdr[5], hasGate = hdr[6], selCount = hdr[7];
  let off = 32;
  const sel = new Int32Array(ab, off, selCount); off += 4 * selCount;
  const qDim = nH * hd, kvDim = nKV * hd;
  const q = new Float32Array(ab, off, nCols * qDim); off += 4 * nCols * qDim;
  const K16 = new Uint16Array(ab, off, rows * kvDim); off += 2 * rows * kvDim;
  const V16 = new Uint16Array(ab, off, rows * kvDim); off += 2 * rows * kvDim;
  const gate = hasGate ? new Float32Array(ab, off, nCols * qDim) : null;
  // the cache as the reference's CPU path holds it: f32 rows (exact widening of the f16 values)
  const K = new Float32Array(rows * kvDim), V = new Float32Array(rows * kvDim);
  for (let i = 0; i < K.length; i++) { K[i] = h2f(K16[i]); V[i] = h2f(V16[i]); }
  const out = new Float32Array(selCount * qDim);
  let best = Infinity;
  for (let r = 0; r < reps; r++) {
    const t0 = process.hrtime.bigint();
    for (let si = 0; si < selCount; si++) {
      const c = sel[si];
      attention(q.subarray(c * qDim, (c + 1) * qDim), K, V, gate ? gate.subarray(c * qDim, (c + 1) * qDim) : null,
        nH, nKV, hd, basePos + c + 1, out.subarray(si * qDim, (si + 1) * qDim));
    }
    const ms = Number(process.hrtime.bigint() - t0) / 1e6;
    if (ms < best) best = ms;
  }
  if (outPath && outPath !== "-") fs.writeFileSync(outPath, Buffer.from(out.buffer, out.byteOffset, out.byteLength));
  console.log(JSON.stringify({ ms: best, reps: reps, node: process.version, threads: 1, max_weight: maxWeight, cpus: os.cpus().length, cpu_model: (os.cpus()[0] || {}).model || "unknown", cols: selCount, nH: nH, nKV: nKV, hd: hd, basePos: basePos }));
}
main();
