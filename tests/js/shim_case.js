// Runs the JavaScript host shim (pooled_amd/js/hip_attention.js) on a case written by tests/test_gpu_js_shim.py:
// a cache prefix, per-column raw q / k / v, norm weights and the oracle's expected attention outputs, and checks
//   1. a full-width pass (prefill kernel)            _encAttnGlue + _encAttnCore
//   2. the same columns as a verify pass (decode kernel, snapshot set)
//   3. one token at a time                            encodeLayerAttn
//   4. session state                                  saveSlot / loadSlot / dropSlot / exportSlot / importState
// against the expected values (max-abs 2e-3, rel 1e-2) and the written KV rows bit for bit; and the verify pass
// against the token-by-token outputs: within 1e-3 by default, bit for bit on a context made with verifyExact
// (the reference's verify column == decode invariant, engine/wgsl/attn_dec.js:12-16, tests/test_attn_dec.js:89-97).
"use strict";
const fs = require("fs"), path = require("path");
const { HipAttention } = require(path.join(__dirname, "..", "..", "pooled_amd", "js", "hip_attention.js"));
const dir = process.argv[2];
const C = JSON.parse(fs.readFileSync(path.join(dir, "case.json"), "utf8"));
const f32 = (n) => { const b = fs.readFileSync(path.join(dir, n)); return new Float32Array(b.buffer.slice(b.byteOffset, b.byteOffset + b.byteLength)); };
const u16 = (n) => { const b = fs.readFileSync(path.join(dir, n)); return new Uint16Array(b.buffer.slice(b.byteOffset, b.byteOffset + b.byteLength)); };
let fails = 0;
const check = (what, got, ref) => {
  let md = 0, mr = 0;
  for (let i = 0; i < ref.length; i++) { md = Math.max(md, Math.abs(got[i] - ref[i])); mr = Math.max(mr, Math.abs(ref[i])); }
  const ok = md <= 2e-3 && md / mr <= 1e-2 && Number.isFinite(md);
  console.log(what + ": max-abs " + md.toExponential(2) + " rel " + (md / mr).toExponential(2) + (ok ? " ok" : " FAIL"));
  if (!ok) fails++;
};
const cfg = C.cfg, n = C.nCols, base = C.basePos;
const A = new HipAttention({ nH: cfg.n_heads, nKV: cfg.n_kv_heads, hd: cfg.head_dim, nRot: cfg.n_rot, ropeTheta: cfg.rope_theta, eps: cfg.eps,
  maxSeq: base + n, nLayers: 1, batchCols: n, qkNorm: true, gate: !!cfg.gate, attnPrefillTile: true, weightCacheBytes: 64 * 1024 * 1024 });   // the matrix-core kernel whatever the chunk's size
const D = A.dims, qIn = cfg.gate ? 2 * D.qDim : D.qDim;
A.setLayerNorms(0, f32("qw.bin"), f32("kw.bin"));
const K0 = u16("k16.bin"), V0 = u16("v16.bin"), qraw = f32("qraw.bin"), kraw = f32("kraw.bin"), vraw = f32("vraw.bin"), expect = f32("expect.bin");
const kNew = u16("knew16.bin"), vNew = u16("vnew16.bin");
const loadCols = (c0, cnt) => { for (let c = 0; c < cnt; c++) {
  A.writeColumn(A.B.qFull, c, qraw.subarray((c0 + c) * qIn, (c0 + c + 1) * qIn));
  A.writeColumn(A.B.k, c, kraw.subarray((c0 + c) * D.kvDim, (c0 + c + 1) * D.kvDim));
  A.writeColumn(A.B.v, c, vraw.subarray((c0 + c) * D.kvDim, (c0 + c + 1) * D.kvDim)); } };
const flat = (cols) => { const o = new Float32Array(cols.length * D.qDim); cols.forEach((c, i) => o.set(c, i * D.qDim)); return o; };
const eqBits = (a, b) => { if (a.length !== b.length) return false; for (let i = 0; i < a.length; i++) if (a[i] !== b[i]) return false; return true; };

A.kvWrite(0, 0, 0, K0); A.kvWrite(0, 1, 0, V0);
// 1. full-width pass
loadCols(0, n);
A.encodeLayerBatchAttn(null, 0, base, n, false);
A.sync();
if (A.plan("prefill", base, n).kernel !== 1) { console.log("full-width pass did not take the prefill kernel FAIL"); fails++; }
check("full-width pass (prefill kernel)", flat(A.readAttnOut(n)), expect);
if (!eqBits(A.kvRead(0, 0, base, n), kNew) || !eqBits(A.kvRead(0, 1, base, n), vNew)) { console.log("KV rows written by the pass differ FAIL"); fails++; }
// 2. verify pass (snapshot): decode kernel, same expected values
loadCols(0, n);
A.encodeLayerBatchAttn(null, 0, base, n, true);
A.sync();
const verifyOut = flat(A.readAttnOut(n));
check("verify pass (decode kernel)", verifyOut, expect);
// 3. token by token
const outs = [];
for (let c = 0; c < n; c++) { loadCols(c, 1); A.encodeLayerAttn(null, 0, base + c); A.sync(); outs.push(A.readAttnOut(1)[0]); }
const seqOut = flat(outs);
check("token by token (fused glue + decode)", seqOut, expect);
// verify block vs sequential decodes: to rounding by default ...
{
  let md = 0; for (let i = 0; i < seqOut.length; i++) md = Math.max(md, Math.abs(seqOut[i] - verifyOut[i]));
  console.log("verify block vs sequential decodes: max-abs " + md.toExponential(2) + (md <= 1e-3 ? " ok" : " FAIL"));
  if (!(md <= 1e-3)) fails++;
}
// ... and bit for bit on a context constructed with verifyExact
{
  const E = new HipAttention({ nH: cfg.n_heads, nKV: cfg.n_kv_heads, hd: cfg.head_dim, nRot: cfg.n_rot, ropeTheta: cfg.rope_theta, eps: cfg.eps,
    maxSeq: base + n, nLayers: 1, batchCols: n, qkNorm: true, gate: !!cfg.gate, verifyExact: true });
  E.setLayerNorms(0, f32("qw.bin"), f32("kw.bin"));
  E.kvWrite(0, 0, 0, K0); E.kvWrite(0, 1, 0, V0);
  const m = Math.min(n, 16);                                      // a verify block is a few columns wide
  for (let c = 0; c < m; c++) {
    E.writeColumn(E.B.qFull, c, qraw.subarray(c * qIn, (c + 1) * qIn));
    E.writeColumn(E.B.k, c, kraw.subarray(c * D.kvDim, (c + 1) * D.kvDim));
    E.writeColumn(E.B.v, c, vraw.subarray(c * D.kvDim, (c + 1) * D.kvDim));
  }
  E._snapNow = 1;
  E._encAttnGlue(null, { layer: 0, basePos: base }, m);
  E._encAttnCore(null, { layer: 0 }, { layer: 0, basePos: base }, base, m);
  E._snapNow = null;
  E.sync();
  const ex = flat(E.readAttnOut(m));
  const same = eqBits(new Uint32Array(ex.buffer), new Uint32Array(seqOut.buffer, 0, m * D.qDim));
  console.log("verifyExact block == sequential encodeLayerAttn bit for bit: " + (same ? "ok" : "FAIL"));
  if (!same) fails++;
  // a short array is refused before anything is copied (RangeError), and a destroyed context is a bad argument
  try { E.kvRead(0, 0, 0, 4).length; require(path.join(__dirname, "..", "..", "pooled_amd", "lib", "pooled_attn.node")).kvRead(E.ctx, 0, 0, 0, 4, new Uint16Array(8)); console.log("short kvRead array did not throw FAIL"); fails++; }
  catch (e) { if (!(e instanceof RangeError)) { console.log("short kvRead array: unexpected error " + e.message + " FAIL"); fails++; } }
  const stale = E.ctx;
  E.destroy();
  try { require(path.join(__dirname, "..", "..", "pooled_amd", "lib", "pooled_attn.node")).sync(stale); console.log("call on a destroyed context did not throw FAIL"); fails++; }
  catch (e) { if (!(e instanceof TypeError)) { console.log("destroyed context: unexpected error " + e.message + " FAIL"); fails++; } }
}
if (!eqBits(A.kvRead(0, 0, base, n), kNew)) { console.log("KV rows written token by token differ FAIL"); fails++; }
// error path: a readable throw, not an abort
try { A.encodeLayerAttn(null, 0, base + n); console.log("out-of-range position did not throw FAIL"); fails++; } catch (e) { if (!/max_seq/.test(e.message)) { console.log("unexpected error text: " + e.message + " FAIL"); fails++; } }
// 4. session state: slot save / overwrite / load, export / import (saveSlot, loadSlot, exportSlot, importState)
{
  const rowsK = A.kvRead(0, 0, 0, base + n), rowsV = A.kvRead(0, 1, 0, base + n);
  A.pos = base + n;
  A.saveSlot("turn1");
  const st = A.exportSlot("turn1");
  if (st.pos !== base + n || st.parts.length !== 2 || !eqBits(new Uint16Array(st.parts[0]), rowsK) || !eqBits(new Uint16Array(st.parts[1]), rowsV)) { console.log("exportSlot parts differ from the cache rows FAIL"); fails++; }
  A.kvWrite(0, 0, 0, new Uint16Array(rowsK.length).fill(0x7e00)); A.kvWrite(0, 1, 0, new Uint16Array(rowsV.length).fill(0x7e00));
  A.pos = 0;
  A.loadSlot("turn1");
  if (A.pos !== base + n || !eqBits(A.kvRead(0, 0, 0, base + n), rowsK) || !eqBits(A.kvRead(0, 1, 0, base + n), rowsV)) { console.log("loadSlot did not restore the rows FAIL"); fails++; }
  A.kvWrite(0, 0, 0, new Uint16Array(rowsK.length).fill(0x7e00));
  A.importState(st);
  if (A.pos !== base + n || !eqBits(A.kvRead(0, 0, 0, base + n), rowsK)) { console.log("importState did not restore the rows FAIL"); fails++; }
  A.dropSlot("turn1");
  try { A.loadSlot("turn1"); console.log("loadSlot of a dropped slot did not throw FAIL"); fails++; } catch (e) { if (!/no saved slot/.test(e.message)) { console.log("unexpected error text: " + e.message + " FAIL"); fails++; } }
  try { A.importState({ sig: { v: 0 }, pos: 0, parts: [] }); console.log("importState of a foreign signature did not throw FAIL"); fails++; } catch (e) { if (!/different model/.test(e.message)) { console.log("unexpected error text: " + e.message + " FAIL"); fails++; } }
  console.log("session state (slots, export, import) " + (fails ? "see above" : "ok"));
}
// 5. projections either side: up / fuse / mv / mvN and the whole attention half of a layer (encodeLayerR) against
//    the same stages called one by one through the shim, and the GEMV alone against a float64 product
{
  let seed = 12345;
  const rnd = () => { seed = (seed * 1664525 + 1013904223) >>> 0; return seed / 4294967296; };
  const dim = 256, kvd = D.kvDim;
  const f16bits = (x) => { const f = new Float32Array([x]), u = new Uint32Array(f.buffer)[0]; const s = (u >>> 16) & 0x8000, e = ((u >>> 23) & 255) - 112, m = u & 0x7fffff; return s | (e << 10) | (m >>> 13); };  // exact for the values below
  const mkQ8 = (dOut, dIn) => { const qs = new Int8Array(dOut * dIn), sc = new Uint16Array(dOut * dIn / 32);
    for (let i = 0; i < qs.length; i++) qs[i] = Math.floor(rnd() * 255) - 127;
    for (let i = 0; i < sc.length; i++) sc[i] = f16bits((1 + Math.floor(rnd() * 8)) / 4096);
    return { kind: "q8", qs: qs, scales: sc, dOut: dOut, dIn: dIn }; };
  const scaleOf = (bits) => (bits & 0x3ff | 0x400) * Math.pow(2, ((bits >> 10) & 31) - 25);
  const eq = mkQ8(qIn, dim), ek = mkQ8(kvd, dim), ev = mkQ8(kvd, dim), eo = mkQ8(dim, D.qDim);
  const wqkv = A.up(A.fuse([eq, ek, ev])), wo = A.up(eo);
  const nw = new Float32Array(dim).map(() => 0.9 + 0.2 * rnd()), x0 = new Float32Array(dim).map(() => 2 * rnd() - 1);
  A.setLayerProj(0, wqkv, wo, nw);
  const pos = base + n - 1;                                      // rewrite the last token's row
  // (a) stage by stage: normed [q | k | v] GEMV into one buffer, then the columns the attention step reads
  const addon = require(path.join(__dirname, "..", "..", "pooled_amd", "lib", "pooled_attn.node"));
  const malloc = (nf) => addon.malloc(A.ctx, nf * 4);
  const dQkv = malloc(qIn + 2 * kvd), dX = malloc(dim), dXn = malloc(dim);
  addon.upload(A.ctx, dX, x0);
  A.mvN(null, wqkv, dX, A.layers[0].attnNorm, dQkv, dXn);
  A.sync();
  const qkv = new Float32Array(qIn + 2 * kvd); addon.download(A.ctx, qkv, dQkv, 0);
  const xn = new Float32Array(dim); addon.download(A.ctx, xn, dXn, 0);
  // GEMV alone against float64 over the same normed vector
  const refRow = (e, r, xv) => { let acc = 0; for (let b = 0; b < e.dIn / 32; b++) { let t = 0; for (let j = 0; j < 32; j++) t += e.qs[r * e.dIn + b * 32 + j] * xv[b * 32 + j]; acc += scaleOf(e.scales[r * e.dIn / 32 + b]) * t; } return acc; };
  const want = new Float32Array(qkv.length);
  for (let r = 0; r < qIn; r++) want[r] = refRow(eq, r, xn);
  for (let r = 0; r < kvd; r++) { want[qIn + r] = refRow(ek, r, xn); want[qIn + kvd + r] = refRow(ev, r, xn); }
  check("mvN over fuse([q, k, v]) vs float64", qkv, want);
  A.writeColumn(A.B.qFull, 0, qkv.subarray(0, qIn)); A.writeColumn(A.B.k, 0, qkv.subarray(qIn, qIn + kvd)); A.writeColumn(A.B.v, 0, qkv.subarray(qIn + kvd));
  A.encodeLayerAttn(null, 0, pos);
  A.mv(null, wo, A.B.attnOut.ptr, dX, true);
  A.sync();
  const xSteps = new Float32Array(dim); addon.download(A.ctx, xSteps, dX, 0);
  // (b) the same token through encodeLayerR
  A.writeColumn(A.B.x, 0, x0);
  A.encodeLayerR(null, 0, pos);
  A.sync();
  const xLayer = A.readColumn(A.B.x, 0);
  if (!eqBits(new Uint32Array(xLayer.buffer), new Uint32Array(xSteps.buffer))) { console.log("encodeLayerR differs from its stages called one by one FAIL"); fails++; }
  let moved = 0; for (let i = 0; i < dim; i++) moved = Math.max(moved, Math.abs(xLayer[i] - x0[i]));
  if (!(moved > 1e-4)) { console.log("encodeLayerR left the residual unchanged FAIL"); fails++; }
  // (c) two columns through encodeLayerBatchR: column 0 at pos - 1, column 1 at pos; f16 operands on the GEMMs, so
  //     it equals the one-token path only to the f16 rounding of activations and weights
  {
    const X = A.residualCols(dim);
    A.writeColumn(X, 0, x0); A.writeColumn(X, 1, x0);
    A.encodeLayerBatchR(null, 0, pos - 1, 2);
    A.sync();
    const c1 = A.readColumn(X, 1);
    // the one-token reference for column 1: position pos after column 0's row (same x0) was written at pos - 1
    A.writeColumn(A.B.x, 0, x0); A.encodeLayerR(null, 0, pos - 1); A.writeColumn(A.B.x, 0, x0); A.encodeLayerR(null, 0, pos); A.sync();
    check("encodeLayerBatchR column vs encodeLayerR", c1, A.readColumn(A.B.x, 0));
  }
  for (const p of [dQkv, dX, dXn]) addon.free(A.ctx, p);
  console.log("projections (up, fuse, mv, mvN, encodeLayerR) " + (fails ? "see above" : "ok"));
}
A.destroy();
console.log(fails ? "SHIM FAIL" : "SHIM PASS");
process.exit(fails ? 1 : 0);
