// Host-side mirror of pooled's attention dispatch for the MI355X library (CommonJS, runs on Node >= 12).
//
// pooled's engines record attention as WebGPU compute passes from these methods:
//   Qwen35Engine._encAttnGlue(p, M, nCols)                      engine/qwen35.js:2473-2483
//   Qwen35Engine._encAttnCore(p, LB, M, basePos, nCols)         engine/qwen35.js:2485-2517
//   Qwen35Engine._encodeLayerR (attention part, one token)      engine/qwen35.js:1598-1640
//   DenseEngine._encodeAttn(pass, BG, seqLen)                   engine/dense.js:463-469
//   DenseEngine._encodeAttnBatch(pass, LB, basePos, n)          engine/dense.js:796-805
// HipAttention keeps those names, argument meanings and buffer conventions (column-batched f32 q / k / v with
// 256-byte aligned column strides, engine/qwen35.js:2054-2055; f16 KV cache [maxSeq][nKV][hd]; attnOut f32
// [nCols][stride]) and forwards each to the C ABI through the Node-API addon.  `p` (the compute pass in the
// reference) is accepted and ignored: work is enqueued in order on the context's HIP stream, which is the
// ordering the engine relies on ("the queue is ordered", engine/dense.js:899-901).
//
// There is no CPU path here: if the addon is missing, require() throws.
"use strict";
const path = require("path");
const addon = require(path.join(__dirname, "..", "lib", "pooled_attn.node"));

const PA_FLAG_QK_NORM = 1, PA_FLAG_GATE = 2, PA_FLAG_KV_Q8 = 4, PA_FLAG_VERIFY_EXACT = 8, PA_OUT_F32 = 0, PA_OUT_F16 = 1;
const PA_W_F32 = 0, PA_W_Q8_0 = 1, PA_W_Q4_0 = 2;             // weight kinds of the projections (include/pooled_attn.h)

class HipAttention {
  // opts: { nH, nKV, hd, nRot, ropeTheta, eps, maxSeq, nLayers, batchCols, qkNorm = true, gate = false, outF16 = false,
  //         kvQ8 = false, fusedStep = true, verifyExact = false, attnPrefillTile = "auto", weightCacheBytes = 8 GiB }
  constructor(opts) {
    const nH = opts.nH, nKV = opts.nKV, hd = opts.hd;
    if (!(nH > 0 && nKV > 0 && nH % nKV === 0)) throw new Error("HipAttention: nH must be a positive multiple of nKV");
    this.dims = { nH: nH, nKV: nKV, hd: hd, nRot: opts.nRot || hd, qDim: nH * hd, kvDim: nKV * hd };
    this.maxSeq = opts.maxSeq;
    this.NC = Math.max(1, opts.batchCols || 16);                 // full pass width (engine/qwen35.js batchCols)
    this.gate = !!opts.gate;
    this.qkNorm = opts.qkNorm !== false;
    this.outDtype = opts.outF16 ? PA_OUT_F16 : PA_OUT_F32;
    this.fusedStep = opts.fusedStep !== false;
    // engine fields the attention dispatch reads (engine/qwen35.js:366, :416-419): always the f16-KV split-K path here
    this.flash = true; this.attnDecode = "v2"; this.attnPrefillTile = opts.attnPrefillTile !== false;
    this._snapNow = null;                                          // set by a verify pass (engine/qwen35.js:2960-2965)
    this.pos = 0;
    this.kvQ8 = !!opts.kvQ8;                                       // int8 caches (engine option kvQ8)
    // verifyExact: every column of a verify block is run as the one-column decode at its position, so it has the bits
    // of a sequential decode (the reference's invariant, engine/wgsl/attn_dec.js:12-16); every column then does a
    // one-column decode's work (about 2.3x the default block's time).  Off by default: a block's columns then agree with sequential decodes to rounding only.
    this.verifyExact = !!opts.verifyExact;
    const flags = (this.qkNorm ? PA_FLAG_QK_NORM : 0) | (this.gate ? PA_FLAG_GATE : 0) | (this.kvQ8 ? PA_FLAG_KV_Q8 : 0) | (this.verifyExact ? PA_FLAG_VERIFY_EXACT : 0);
    // a readable throw at create, like the engine's KV binding check (engine/qwen35.js:378-383)
    this.ctx = addon.create({ nH: nH, nKV: nKV, hd: hd, nRot: this.dims.nRot, ropeTheta: opts.ropeTheta, eps: opts.eps,
      maxSeq: opts.maxSeq, nLayers: opts.nLayers || 1, maxCols: this.NC, flags: flags });
    // the engine's attnPrefillTile option (engine/qwen35.js:389-401): undefined / "auto" = the library's table picks the
    // kernel of a prefill chunk, true = always the matrix-core kernel, false = full-width passes go through the decode
    // entry point like every other pass
    if (opts.attnPrefillTile === true) addon.setPrefillTile(this.ctx, 1);
    // budget of the f16 weight copies that gemm() keeps with a weight from its first chunk of more than 16 columns on
    // (0: none, every such call widens into per-context staging)
    if (opts.weightCacheBytes !== undefined) addon.setWeightCache(this.ctx, opts.weightCacheBytes);
    this.kvBufBytes = opts.maxSeq * this.dims.kvDim * 2;
    this.layers = [];
    for (let i = 0; i < (opts.nLayers || 1); i++) { addon.layerAlloc(this.ctx, i); this.layers.push({ index: i, qNorm: null, kNorm: null }); }
    // column-batched activations, 256-byte aligned column strides (engine/qwen35.js:2054-2055 mkB)
    const al = (n) => Math.ceil(n * 4 / 256) * 256;
    const mkB = (n) => ({ ptr: addon.malloc(this.ctx, this.NC * al(n)), stride: al(n), n: n });
    const qIn = this.gate ? nH * hd * 2 : nH * hd;
    this.B = { qFull: mkB(qIn), k: mkB(this.dims.kvDim), v: mkB(this.dims.kvDim), attnOut: mkB(this.dims.qDim) };
    this._ones = addon.malloc(this.ctx, hd * 4);
    addon.upload(this.ctx, this._ones, new Float32Array(hd).fill(1));
  }

  destroy() {
    if (!this.ctx) return;
    for (const k of Object.keys(this.B)) addon.free(this.ctx, this.B[k].ptr);
    for (const L of this.layers) { if (L.qNorm) addon.free(this.ctx, L.qNorm); if (L.kNorm) addon.free(this.ctx, L.kNorm); if (L.attnNorm) addon.free(this.ctx, L.attnNorm); }
    for (const w of this._weights || []) addon.weightDestroy(this.ctx, w);
    addon.free(this.ctx, this._ones);
    addon.destroy(this.ctx);
    this.ctx = null;
  }

  // ---- uploads the engine does with queue.writeBuffer ----
  setLayerNorms(i, qNorm, kNorm) {
    const L = this.layers[i], hd = this.dims.hd;
    if (qNorm.length !== hd || kNorm.length !== hd) throw new Error("setLayerNorms: weights must have headDim elements");
    if (!L.qNorm) { L.qNorm = addon.malloc(this.ctx, hd * 4); L.kNorm = addon.malloc(this.ctx, hd * 4); }
    addon.upload(this.ctx, L.qNorm, Float32Array.from(qNorm));
    addon.upload(this.ctx, L.kNorm, Float32Array.from(kNorm));
  }
  // column c of buffer b <- Float32Array (b.n floats)
  writeColumn(b, c, data) {
    if (data.length !== b.n) throw new Error("writeColumn: expected " + b.n + " floats");
    if (c >= this.NC) throw new Error("writeColumn: column " + c + " >= batchCols " + this.NC);
    addon.upload(this.ctx, b.ptr, data, c * b.stride);
  }
  readColumn(b, c) {
    const out = new Float32Array(b.n);
    addon.download(this.ctx, out, b.ptr, c * b.stride);
    return out;
  }
  // attnOut as the engine reads it back (f32 columns; f16 when constructed with outF16)
  readAttnOut(nCols) {
    const D = this.dims, out = [];
    for (let c = 0; c < nCols; c++) {
      if (this.outDtype === PA_OUT_F32) out.push(this.readColumn(this.B.attnOut, c));
      else { const h = new Uint16Array(D.qDim); addon.download(this.ctx, h, this.B.attnOut.ptr, c * this.B.attnOut.stride); out.push(h); }
    }
    return out;
  }
  // which: 0 K, 1 V (f16 bits as Uint16Array; on int8 caches Int8Array), 2 / 3 their scales (int8 caches, Float32Array)
  _kvPart(which, nRows) {
    if (!this.kvQ8) return new Uint16Array(nRows * this.dims.kvDim);
    return which < 2 ? new Int8Array(nRows * this.dims.kvDim) : new Float32Array(nRows * this.dims.kvDim / 32);
  }
  kvRead(layer, which, row0, nRows) { const a = this._kvPart(which, nRows); addon.kvRead(this.ctx, layer, which, row0, nRows, a); return a; }
  kvWrite(layer, which, row0, rows) {
    const per = this._kvPart(which, 1).length;
    if (rows.length % per !== 0) throw new RangeError("kvWrite: " + rows.length + " elements is not a whole number of rows of " + per);
    addon.kvWrite(this.ctx, layer, which, row0, rows.length / per, rows);
  }
  sync() { addon.sync(this.ctx); }
  plan(kind, basePos, nCols) { return addon.planQuery(this.ctx, kind === "prefill" ? 1 : 0, basePos, nCols); }

  // ---- session state: the engines' saveSlot / loadSlot / dropSlot (engine/dense.js:20-47, engine/qwen35.js:190-230)
  //      and the attention layers' share of exportSlot / importState (engine/qwen35.js:121-131, :151-190) ----
  // this.pos is the number of rows written so far, as in the engines; the callers keep it (the shim's attention
  // methods take positions as arguments and do not advance it).
  _slotId(name, make) {
    this._slotIds = this._slotIds || new Map();
    if (!this._slotIds.has(name) && make) this._slotIds.set(name, this._slotNext = (this._slotNext || 0) + 1);
    return this._slotIds.get(name);
  }
  saveSlot(name) { addon.slotSave(this.ctx, this._slotId(name, true), this.pos); }
  loadSlot(name) {
    const id = this._slotId(name, false);
    if (id === undefined) throw new Error("no saved slot " + name);
    this.pos = addon.slotLoad(this.ctx, id);
  }
  dropSlot(name) { const id = this._slotId(name, false); if (id !== undefined) { addon.slotDrop(this.ctx, id); this._slotIds.delete(name); } }
  dropAllSlots() { for (const k of Array.from((this._slotIds || new Map()).keys())) this.dropSlot(k); }
  // what a saved state must match to be loaded here (the attention-relevant fields of engine/qwen35.js:133-143)
  stateSignature() { return { v: 1, layers: this.layers.length, flash: true, kvQ8: this.kvQ8, dims: [this.dims.kvDim] }; }
  // { sig, pos, parts: [ArrayBuffer] }: per layer a K part and a V part of pos * kvDim f16, position-major
  exportSlot(name) {
    const id = this._slotId(name, false);
    if (id === undefined) throw new Error("no saved slot " + name);
    const pos = addon.slotPos(this.ctx, id), parts = [];
    // per layer kCache, vCache (and, int8 caches, kScale, vScale): the order of the reference's _stateParts
    for (let l = 0; l < this.layers.length; l++) for (let w = 0; w < (this.kvQ8 ? 4 : 2); w++) {
      const a = this._kvPart(w, pos);
      if (pos) addon.slotExport(this.ctx, id, l, w, a);
      parts.push(a.buffer);
    }
    return { sig: this.stateSignature(), pos: pos, parts: parts };
  }
  exportState() { this.saveSlot("__export"); try { return this.exportSlot("__export"); } finally { this.dropSlot("__export"); } }
  importState(st) {
    if (JSON.stringify(st.sig) !== JSON.stringify(this.stateSignature())) throw new Error("saved state is for a different model, layer range or KV format");
    const nt = this.kvQ8 ? 4 : 2;
    if (st.parts.length !== nt * this.layers.length || st.parts.some((p, i) => p.byteLength !== this._kvPart(i % nt, st.pos).byteLength)) throw new Error("saved state has the wrong shape");
    const id = this._slotId("__import", true);
    addon.slotCreate(this.ctx, id, st.pos);
    try {
      if (st.pos) st.parts.forEach((p, i) => addon.slotImport(this.ctx, id, Math.floor(i / nt), i % nt, new Uint8Array(p)));
      this.pos = addon.slotLoad(this.ctx, id);
    } finally { this.dropSlot("__import"); }
  }

  _norms(L) { return [L.qNorm || this._ones, L.kNorm || this._ones]; }
  _strideF(b) { return b.stride / 4; }
  _outStride() { return this.outDtype === PA_OUT_F32 ? this.B.attnOut.stride / 4 : this.B.attnOut.stride / 2; }

  // ---- Qwen35Engine: batched pass ----
  // qsplit + q/k head-norm + (partial) rope for nCols columns; k is rewritten in place, like attn_glue.
  // M = { layer, basePos } stands where the reference passes the layer's bind-group table (LB.mc); the columns'
  // positions come from the frame uniform there (engine/qwen35.js:3846), from M.basePos here.
  _encAttnGlue(p, M, nCols) {
    const L = this.layers[M.layer], n = this._norms(L);
    addon.glue(this.ctx, this.B.qFull.ptr, this._strideF(this.B.qFull), this.B.k.ptr, this._strideF(this.B.k), n[0], n[1], M.basePos, nCols);
  }
  // kv_store + attention + sigmoid gate: B.q / B.k / B.v / gate -> B.attnOut.  Kernel selection as the reference's:
  // a full-width pass that is not a verify runs the tiled prefill kernel, everything else the split-K decode kernel.
  // Unlike the reference's pair (engine/wgsl/attn_dec.js:12-16) a verify column here equals the one-column decode at
  // the same position to rounding only (|difference| <= 1e-3 by test, 3e-4 measured): the block's columns share
  // matrix-core tiles and splits.  Constructing with { verifyExact: true } restores the bit identity at the cost of
  // a one-column decode's work per column.
  _encAttnCore(p, LB, M, basePos, nCols) {
    const B = this.B, layer = LB.layer;
    addon.kvStore(this.ctx, layer, B.k.ptr, this._strideF(B.k), B.v.ptr, this._strideF(B.v), basePos, nCols);
    const gate = this.gate ? addon.gateBuffer(this.ctx) : null;
    const kind = (this.attnPrefillTile && nCols === this.NC && nCols > 1 && !this._snapNow) ? 1 : 0;
    addon.attn(this.ctx, kind, layer, null, 0, gate, this.dims.qDim, basePos, nCols, B.attnOut.ptr, this._outStride(), this.outDtype);
  }
  // a whole batched attention block, as _encodeLayerBatch strings the two together (engine/qwen35.js:2416, :2425)
  encodeLayerBatchAttn(p, i, basePos, nCols, snapshot) {
    this._snapNow = snapshot ? 1 : null;
    this._encAttnGlue(p, { layer: i, basePos: basePos }, nCols);
    this._encAttnCore(p, { layer: i }, { layer: i, basePos: basePos }, basePos, nCols);
    this._snapNow = null;
  }
  // ---- Qwen35Engine: one token (fused glue + KV write, split-K decode, merge + gate in one go) ----
  // By default this is the single fused call; { fusedStep: false } in the constructor options keeps the three
  // dispatches of the reference (glue + KV write, split-K decode, merge + gate) as separate launches.
  encodeLayerAttn(p, i, pos) {
    const B = this.B, L = this.layers[i], n = this._norms(L);
    if (this.fusedStep) {
      addon.attnDecodeStep(this.ctx, i, B.qFull.ptr, B.k.ptr, B.v.ptr, n[0], n[1], pos, B.attnOut.ptr, this.outDtype);
      return;
    }
    addon.glueKv(this.ctx, i, B.qFull.ptr, this._strideF(B.qFull), B.k.ptr, this._strideF(B.k), B.v.ptr, this._strideF(B.v), n[0], n[1], pos, 1);
    const gate = this.gate ? addon.gateBuffer(this.ctx) : null;
    addon.attn(this.ctx, 0, i, null, 0, gate, this.dims.qDim, pos, 1, B.attnOut.ptr, this._outStride(), this.outDtype);
  }

  // ---- projections either side of the attention block, one token (engine/qwen35.js:894-922 up / mv / mvN) ----
  // e: a weight entry as the engine's loaders make them: { kind: "q4" | "q8", qs, scales, dOut, dIn } (qs: Uint8Array /
  // Int8Array / Uint32Array words, scales: Uint16Array of f16 bits) or { kind: "f32", data, dOut, dIn }
  up(e) {
    const kind = e.kind === "q4" ? PA_W_Q4_0 : e.kind === "q8" ? PA_W_Q8_0 : e.kind === "f32" ? PA_W_F32 : -1;
    if (kind < 0) throw new Error("up: unknown weight kind " + e.kind);
    const h = addon.weightCreate(this.ctx, kind, e.dOut, e.dIn, kind === PA_W_F32 ? e.data : e.qs, kind === PA_W_F32 ? null : e.scales);
    (this._weights = this._weights || []).push(h);
    return { kind: e.kind, handle: h, dOut: e.dOut, dIn: e.dIn };
  }
  // the engine's fuse() (engine/qwen35.js:1001-1019): several weights of one kind and width as one, rows concatenated
  fuse(parts) {
    const k = parts[0].kind, dIn = parts[0].dIn;
    if (!parts.every((p) => p.kind === k && p.dIn === dIn)) throw new Error("fuse: parts must share kind and dIn");
    const cat = (arrs) => { const out = new arrs[0].constructor(arrs.reduce((n, x) => n + x.length, 0)); let o = 0; for (const x of arrs) { out.set(x, o); o += x.length; } return out; };
    const dOut = parts.reduce((n, p) => n + p.dOut, 0);
    return k === "f32" ? { kind: k, data: cat(parts.map((p) => p.data)), dOut: dOut, dIn: dIn }
                       : { kind: k, qs: cat(parts.map((p) => p.qs)), scales: cat(parts.map((p) => p.scales)), dOut: dOut, dIn: dIn };
  }
  // mv: y = W x (acc: y += W x); mvN: y = W rmsnorm(x) with norm weight nw (xnOut: also keep the normed vector)
  mv(p, w, x, y, acc) { addon.gemv(this.ctx, w.handle, x, y, acc ? 1 : 0); }
  mvN(p, w, x, nw, y, xnOut) { addon.gemvNorm(this.ctx, w.handle, x, nw, xnOut || null, y); }
  // per-layer projection weights: wqkv = fuse([wq, wk, wv]) uploaded, wo, attnNorm (Float32Array [dim])
  setLayerProj(i, wqkv, wo, attnNorm) {
    const L = this.layers[i];
    L.wqkv = wqkv; L.wo = wo;
    if (!L.attnNorm) L.attnNorm = addon.malloc(this.ctx, attnNorm.length * 4);
    addon.upload(this.ctx, L.attnNorm, Float32Array.from(attnNorm));
    if (!this.B.x) this.B.x = { ptr: addon.malloc(this.ctx, attnNorm.length * 4), stride: attnNorm.length * 4, n: attnNorm.length };
  }
  // one token through the attention half of full-attention layer i, as _encodeLayerR records it
  // (engine/qwen35.js:1586-1641): B.x (the residual) is read and updated in place
  encodeLayerR(p, i, pos) {
    const L = this.layers[i], n = this._norms(L);
    if (!L.wqkv) throw new Error("encodeLayerR: layer " + i + " has no projection weights (setLayerProj)");
    addon.attnLayerDecode(this.ctx, i, L.wqkv.handle, L.wo.handle, L.attnNorm, n[0], n[1], this.B.x.ptr, pos);
  }

  // nCols tokens at basePos .. through the attention half of full-attention layer i, as _encodeLayerBatch /
  // _encodeLayerWide record it (engine/qwen35.js:2416-2425, :2827): B.xCols (residual columns, f32, 256-byte aligned
  // stride; allocated on first use for batchCols columns) in and out
  residualCols(dim) {
    if (!this.B.xCols) { const st = Math.ceil(dim * 4 / 256) * 256; this.B.xCols = { ptr: addon.malloc(this.ctx, this.NC * st), stride: st, n: dim }; }
    return this.B.xCols;
  }
  encodeLayerBatchR(p, i, basePos, nCols) {
    const L = this.layers[i], n = this._norms(L);
    if (!L.wqkv) throw new Error("encodeLayerBatchR: layer " + i + " has no projection weights (setLayerProj)");
    const X = this.residualCols(L.wqkv.dIn);
    addon.attnLayerPrefill(this.ctx, i, L.wqkv.handle, L.wo.handle, L.attnNorm, n[0], n[1], X.ptr, X.stride / 4, basePos, nCols);
  }

  // ---- sparse-attention layers: the attn step of a QSA pass (engine/qsa.js:8-14, dispatch :41-56) ----
  // sel: device address of the per-column row lists qsa_select wrote (u32 [nCols][selStride]: n, then n rows);
  // maxRows = qsaMaxRows(pos, nCols).  Reads B.q (the context's roped q) and the gate, writes B.attnOut.
  _encAttnQsa(p, LB, sel, selStride, maxRows, nCols) {
    const gate = this.gate ? addon.gateBuffer(this.ctx) : null;
    addon.attnGather(this.ctx, LB.layer, null, 0, gate, this.dims.qDim, sel, selStride, maxRows, nCols, this.B.attnOut.ptr, this._outStride(), this.outDtype);
  }

  // ---- DenseEngine shapes (full RoPE, no gate): the glue writes the cache, then attention ----
  // _encodeAttn(pass, BG, seqLen): BG = { layer }; attention of the token at position seqLen - 1
  _encodeAttn(pass, BG, seqLen) {
    addon.attn(this.ctx, 0, BG.layer, null, 0, null, 0, seqLen - 1, 1, this.B.attnOut.ptr, this._outStride(), this.outDtype);
  }
  // _encodeAttnBatch(pass, LB, basePos, n): n columns at basePos .. basePos + n - 1 (the reference runs 4)
  _encodeAttnBatch(pass, LB, basePos, n) {
    addon.attn(this.ctx, 0, LB.layer, null, 0, null, 0, basePos, n === undefined ? 4 : n, this.B.attnOut.ptr, this._outStride(), this.outDtype);
  }
  // the dense layer's glue (head_norm_dmc + rope_dmc + kv_store_d, engine/dense.js:394-399) for n columns
  encodeGlueDense(pass, i, basePos, n) {
    const B = this.B, L = this.layers[i], w = this._norms(L);
    addon.glueKv(this.ctx, i, B.qFull.ptr, this._strideF(B.qFull), B.k.ptr, this._strideF(B.k), B.v.ptr, this._strideF(B.v), w[0], w[1], basePos, n);
  }
}

module.exports = { HipAttention, addon, PA_FLAG_QK_NORM, PA_FLAG_GATE, PA_FLAG_KV_Q8, PA_FLAG_VERIFY_EXACT, PA_OUT_F32, PA_OUT_F16 };
