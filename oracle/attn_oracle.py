"""CPU oracle for pooled's attention hot path (numpy).  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU, the arithmetic that pooled's engines run for one attention layer:
the QK-RMSNorm + RoPE pre-step, the f16 KV-cache write, GQA softmax attention over the cache
(decode, causal prefill, speculative verify), the log-sum-exp merge of split partials and the
sigmoid output gate.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import it; the shipped library never does.

Every function cites the reference lines it follows (paths relative to the pooled repository).
How each function is pinned (tests/test_oracle.py):
  f16 pack            IEEE binary16 known answers incl. ties, subnormals, overflow
  head_rmsnorm        closed form on constant / one-hot heads, unit-RMS invariant
  rope_neox           pos 0 identity, pairwise norm preservation, additivity of angles, quarter turns,
                      dims >= n_rot untouched
  attention           seqLen 1 -> V row, constant V, one-hot softmax (huge score), uniform softmax,
                      row-permutation invariance, brute-force scalar loops on tiny shapes, C oracle
  lse_merge           merging split partials == unsplit attention; one split -> O / l
  split formulas      integer known answers quoted in the reference's own comments
  q8_quantize         zero block, exact-integer block (scale 1), ties to even, clamp at +-127, the block maximum maps
                      to +-127, |x - dequant| <= scale / 2, scale from the f32 quotient
  w_dequant / gemv    hand-made Q4_0 / Q8_0 blocks with known values (nibble order, sign, scale), the reference's scalar
                      matvec loops restated element by element on small shapes, linearity, unit vectors pick columns
  rmsnorm             closed form on a constant vector, unit-RMS invariant, eps = 0 scale invariance
"""
import numpy as np

# ---------------------------------------------------------------------------------------------
# f16 pack (KV-cache element format)
# ---------------------------------------------------------------------------------------------

def f16_bits(x):
    """f32 -> IEEE binary16 bits, round-to-nearest-even, as the KV write models it.

    Reference: engine/wgsl/qwen35.js:889-906 (kv_store packs with pack2x16float) and the CPU model of
    that rounding in tests/test_attn_dec.js:24-25 (ties to even).  Subnormal results are kept (IEEE);
    engine/gguf.js:17-37 is a different (ties-up) rounding used for the wire format, not for KV.
    """
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_round(x):
    """f32 -> f16 -> f32 (the value attention reads back from the cache); exact widening."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# pre-step: q de-interleave, per-head RMSNorm, NeoX RoPE, KV write
# ---------------------------------------------------------------------------------------------

def qsplit(qfull, n_heads, hd):
    """qfull [.., nH*2*hd] -> (q [.., nH, hd], gate [.., nH, hd]).

    Reference: engine/wgsl/qwen35.js:370-384 (qsplit), :827-842 (qsplit_mc);
    tests/reference/ref_q38.mjs:157-161: q[h][i] = qFull[h*2hd + i], gate[h][i] = qFull[h*2hd + hd + i].
    """
    a = np.asarray(qfull, dtype=np.float32).reshape(qfull.shape[:-1] + (n_heads, 2, hd))
    return a[..., 0, :].copy(), a[..., 1, :].copy()


def head_rmsnorm(x, w, eps):
    """Per-head RMSNorm with a weight [hd] shared by all heads: x [.., heads, hd] f32 -> f32.

    Reference: engine/wgsl/base.js:65-79 (head_norm), engine/wgsl/qwen35.js:844-856, :1112-1122:
    inv = inverseSqrt(ss / hd + eps); v = v * (inv * w).  CPU refs: tests/reference/ref_qwen.mjs:45-54,
    ref_q38.mjs:50-57.  Here the sum of squares is exact-product f64 and inv is rounded once to f32;
    the two multiplies are f32 (no fused operation is possible between two multiplies).
    """
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    hd = x.shape[-1]
    ss = np.sum(x.astype(np.float64) ** 2, axis=-1, keepdims=True)
    inv = (1.0 / np.sqrt(ss / hd + np.float64(np.float32(eps)))).astype(np.float32)
    return x * (inv * w)


def rope_inv_freq(n_rot, theta):
    """f32 table freq[i] = theta^(-2i/n_rot), i < n_rot/2, correctly rounded from f64.

    Reference: engine/wgsl/base.js:165 (full), engine/wgsl/qwen35.js:397 (partial):
    pow(theta, -f32(2i) / f32(nRot)).
    """
    i = np.arange(n_rot // 2, dtype=np.float64)
    return np.power(np.float64(np.float32(theta)), -(2.0 * i) / n_rot).astype(np.float32)


def rope_neox(x, pos, n_rot, theta):
    """NeoX RoPE on the first n_rot dims of every head: x [n, heads, hd] f32, pos [n] ints -> f32.

    Reference: engine/wgsl/base.js:154-172 (rope: n_rot = hd), engine/wgsl/qwen35.js:386-404, :858-875
    (rope_part): pairs (i, i + n_rot/2); ang = f32(pos) * freq_i (an f32 product);
    a' = a*c - b*s, b' = b*c + a*s; dims >= n_rot untouched.  CPU refs: ref_qwen.mjs:32-44,
    ref_q38.mjs:67-79.  cos/sin are taken of the *f32* angle (as the GPU kernels do, and as
    tests/reference/qsa_ref.mjs:96-110 models), evaluated in f64 and rounded to f32; the products and
    the add/sub are separate f32 roundings (no fused multiply-add).
    """
    x = np.asarray(x, dtype=np.float32)
    pos = np.asarray(pos).reshape(-1)
    out = x.copy()
    half = n_rot // 2
    freq = rope_inv_freq(n_rot, theta)                                  # [half] f32
    ang = pos.astype(np.float32)[:, None] * freq[None, :]               # f32 product, [n, half]
    c = np.cos(ang.astype(np.float64)).astype(np.float32)[:, None, :]
    s = np.sin(ang.astype(np.float64)).astype(np.float32)[:, None, :]
    a = x[..., :half]
    b = x[..., half:n_rot]
    out[..., :half] = a * c - b * s
    out[..., half:n_rot] = b * c + a * s
    return out


def glue_kv(q_in, k_in, v_in, qw, kw, base_pos, cfg):
    """The whole pre-step for n columns at positions base_pos + c.

    q_in: [n, nH*2*hd] (interleaved q|gate, cfg['gate'] true) or [n, nH*hd]; k_in, v_in: [n, nKV*hd].
    Returns dict(q [n,nH,hd] f32, gate [n,nH,hd] f32 or None, k16/v16 [n,nKV,hd] uint16 = the cache rows
    written at positions base_pos + c).

    Reference: engine/wgsl/qwen35.js:1082-1136 (attn_glue), engine/wgsl/layer_fuse.js:87-146
    (attn_glue_kv: + the f16 cache write), engine/wgsl/dense.js:144-196 (attn_glue_d, full rope);
    V is neither normed nor roped (ref_q38.mjs:171).
    """
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    n = q_in.shape[0]
    pos = base_pos + np.arange(n)
    if cfg.get("gate", False):
        q, gate = qsplit(q_in, nH, hd)
    else:
        q, gate = np.asarray(q_in, np.float32).reshape(n, nH, hd).copy(), None
    k = np.asarray(k_in, np.float32).reshape(n, nKV, hd)
    if cfg.get("qk_norm", True):
        q = head_rmsnorm(q, qw, cfg["eps"])
        k = head_rmsnorm(k, kw, cfg["eps"])
    q = rope_neox(q, pos, cfg["n_rot"], cfg["rope_theta"])
    k = rope_neox(k, pos, cfg["n_rot"], cfg["rope_theta"])
    v = np.asarray(v_in, np.float32).reshape(n, nKV, hd)
    return dict(q=q, gate=gate, k16=f16_bits(k), v16=f16_bits(v))


# ---------------------------------------------------------------------------------------------
# int8 KV (one f32 scale per 32 values)
# ---------------------------------------------------------------------------------------------

def q8_quantize(x):
    """x [..., n] f32, n % 32 == 0 -> (q int8 [..., n], scale f32 [..., n/32]).

    Reference: engine/wgsl/qwen35.js:908-946 (kv_store_q8): per block of 32 values scale = max|x| / 127,
    inv = 1 / scale (0 for an all-zero block), value = clamp(round(x * inv), -127, 127), every operation in f32;
    WGSL round() rounds half-way cases to even.
    """
    x = np.asarray(x, dtype=np.float32)
    b = x.reshape(x.shape[:-1] + (x.shape[-1] // 32, 32))
    a = np.abs(b).max(axis=-1)
    sc = (a / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(sc > 0, np.float32(1.0) / sc, np.float32(0.0)).astype(np.float32)
    q = np.clip(np.rint((b * inv[..., None]).astype(np.float32)), -127.0, 127.0).astype(np.int8)
    return q.reshape(x.shape), sc


def q8_dequantize(q, sc):
    """value * scale in f32, as the attention kernels read an int8 cache (engine/wgsl/qwen35.js:112-126)."""
    q = np.asarray(q, dtype=np.int8)
    b = q.reshape(q.shape[:-1] + (q.shape[-1] // 32, 32)).astype(np.float32)
    return (b * np.asarray(sc, np.float32)[..., None]).astype(np.float32).reshape(q.shape)


# ---------------------------------------------------------------------------------------------
# projections either side of the attention block (one-token GEMVs over the reference's weight planes)
# ---------------------------------------------------------------------------------------------

W_F32, W_Q8_0, W_Q4_0 = 0, 1, 2


def w_dequant(kind, w, scales=None):
    """Weight planes -> f64 matrix [d_out, d_in].

    Reference: engine/wgsl/base.js:15-30 (f32 row-major), :32-63 (Q8_0: int8 packed 4 a word, value index = byte
    index; one f16 scale per 32 values, unpack2x16float), :81-118 (Q4_0: "byte j holds elem j (low nibble) and elem
    j+16 (high)", value = nibble - 8).  kind W_F32: w f32 [d_out, d_in]; W_Q8_0: w int8 [d_out, d_in];
    W_Q4_0: w uint8 [d_out, d_in / 2]; scales: f16 bits (uint16) [d_out, d_in / 32].
    """
    if kind == W_F32:
        return np.asarray(w, dtype=np.float32).astype(np.float64)
    sc = np.asarray(scales, dtype=np.uint16).view(np.float16).astype(np.float64)          # [d_out, nb]
    if kind == W_Q8_0:
        q = np.asarray(w, dtype=np.int8).astype(np.float64)
        d_out, d_in = q.shape
        return (q.reshape(d_out, d_in // 32, 32) * sc[:, :, None]).reshape(d_out, d_in)
    if kind == W_Q4_0:
        b = np.asarray(w, dtype=np.uint8)
        d_out, half = b.shape
        blk = b.reshape(d_out, half // 16, 16)
        vals = np.concatenate([(blk & 15).astype(np.float64) - 8.0, (blk >> 4).astype(np.float64) - 8.0], axis=2)   # [.., 32]
        return (vals * sc[:, :, None]).reshape(d_out, half * 2)
    raise ValueError("unknown weight kind")


def gemv(kind, w, scales, x):
    """y = W x in f64 (the reference accumulates in f32 in an order of its own; tests use its tolerance).

    Reference: engine/wgsl/base.js:20-30, :40-63, :90-118; cooperative forms engine/wgsl/coop.js:236-345.
    """
    return w_dequant(kind, w, scales) @ np.asarray(x, dtype=np.float32).astype(np.float64)


def gemv_reference_loops(kind, w, scales, x):
    """The reference's scalar kernels restated loop for loop (small shapes only): pins w_dequant / gemv.

    Reference: engine/wgsl/base.js:40-63 (matvec_q8: sum over words of extractBits(word, 8k, 8) * x, times the block
    scale), :90-118 (matvec_q4: word w of a block, nibble pairs (4k, 4k + 4) -> elements (4w + k, 4w + k + 16)).
    """
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    if kind == W_F32:
        wf = np.asarray(w, dtype=np.float32)
        return np.array([sum(float(wf[r, c]) * x[c] for c in range(wf.shape[1])) for r in range(wf.shape[0])])
    sc = np.asarray(scales, dtype=np.uint16).view(np.float16).astype(np.float64)
    d_out = w.shape[0]
    y = np.zeros(d_out)
    if kind == W_Q8_0:
        words = np.ascontiguousarray(np.asarray(w, dtype=np.int8)).view(np.uint32)       # [d_out, d_in / 4]
        nb = words.shape[1] // 8
        for r in range(d_out):
            acc = 0.0
            for b in range(nb):
                s_ = 0.0
                for wi in range(8):
                    word = int(words[r, b * 8 + wi])
                    for k in range(4):
                        v = (word >> (8 * k)) & 255
                        v = v - 256 if v >= 128 else v                                   # extractBits on an i32: sign-extended
                        s_ += v * x[b * 32 + wi * 4 + k]
                acc += sc[r, b] * s_
            y[r] = acc
        return y
    words = np.ascontiguousarray(np.asarray(w, dtype=np.uint8)).view(np.uint32)          # [d_out, d_in / 8]
    nb = words.shape[1] // 4
    for r in range(d_out):
        acc = 0.0
        for b in range(nb):
            s_ = 0.0
            for wi in range(4):
                word = int(words[r, b * 4 + wi])
                j = b * 32 + wi * 4
                for k in range(4):
                    s_ += (((word >> (8 * k)) & 15) - 8.0) * x[j + k]
                    s_ += (((word >> (8 * k + 4)) & 15) - 8.0) * x[j + 16 + k]
            acc += sc[r, b] * s_
        y[r] = acc
    return y


def rmsnorm(x, w, eps):
    """xn = (x * inv) * w, inv = 1 / sqrt(mean(x^2) + eps): f32 in, f64 arithmetic, f32 out.

    Reference: engine/wgsl/base.js:119-152 (rmsnorm), engine/wgsl/coop.js:389-411 (the same inside a GEMV).
    """
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    inv = 1.0 / np.sqrt(np.mean(x * x) + eps)
    return ((x * inv) * np.asarray(w, dtype=np.float32).astype(np.float64)).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------

def sigmoid_gate(out, gate):
    """out * 1/(1+exp(-gate)), f32.  Reference: engine/wgsl/qwen35.js:406-416 (sigmoid_mul),
    engine/wgsl/layer_fuse.js:148-181, tests/reference/ref_q38.mjs:191."""
    g = np.asarray(gate, dtype=np.float64)
    return (np.asarray(out, np.float64) * (1.0 / (1.0 + np.exp(-g))))


def attention(q, k16, v16, base_pos, gate=None, rows=None):
    """Exact (f64) GQA softmax attention over an f16 cache.

    q [n, nH, hd] f32; k16, v16 [S, nKV, hd] uint16 (f16 bits), S >= base_pos + n; column c sits at
    absolute position base_pos + c and attends to cache rows [0, base_pos + c] (causal by absolute
    position).  kv head of query head h is floor(h / (nH/nKV)).  Returns [n, nH, hd] f64.
    rows: optional iterable of column indices to evaluate (others left 0).

    Reference: tests/reference/ref_qwen.mjs:114-131, ref_q38.mjs:171-190, tests/test_attn_dec.js:72-82,
    tests/unit/attn_tile_test.js:63-78: s_t = (q.k_t)/sqrt(hd); p = exp(s - max)/sum; out = sum p_t v_t.
    One decode token is n = 1; a verify block or a prefill chunk is n > 1 (engine/qwen35.js:2485-2517:
    every column sees seqLen + col rows).
    """
    return attention_values(q, k16.view(np.float16), v16.view(np.float16), base_pos, gate=gate, rows=rows)


def attention_values(q, kf, vf, base_pos, gate=None, rows=None):
    """attention() over cache rows given as numbers (any float dtype, [S, nKV, hd]) instead of f16 bits: the same
    arithmetic; used for caches whose stored form is not f16 (the int8 cache after de-quantisation)."""
    q = np.asarray(q, dtype=np.float32)
    n, nH, hd = q.shape
    nKV = kf.shape[1]
    G = nH // nKV
    out = np.zeros((n, nH, hd), dtype=np.float64)
    cols = range(n) if rows is None else rows
    for c in cols:
        L = base_pos + c + 1
        for g in range(nKV):
            K = kf[:L, g, :].astype(np.float64)                         # [L, hd]
            V = vf[:L, g, :].astype(np.float64)
            qq = q[c, g * G:(g + 1) * G, :].astype(np.float64)          # [G, hd]
            s = (qq @ K.T) / np.sqrt(np.float64(hd))                    # [G, L]
            s -= s.max(axis=1, keepdims=True)
            p = np.exp(s)
            out[c, g * G:(g + 1) * G, :] = (p @ V) / p.sum(axis=1, keepdims=True)
    if gate is not None:
        out = sigmoid_gate(out, gate)
    return out


def attention_partial(q, k16, v16, t0, t1):
    """Un-normalised split partial over cache rows [t0, t1): returns (m [nH], l [nH], O [nH, hd]), f64.

    Reference: engine/wgsl/attn_dec.js:102-200 (per-split m, l, O = sum exp(s - m) v)."""
    q = np.asarray(q, dtype=np.float32)
    nH, hd = q.shape
    nKV = k16.shape[1]
    G = nH // nKV
    m = np.zeros(nH); l = np.zeros(nH); O = np.zeros((nH, hd))
    for g in range(nKV):
        K = k16[t0:t1, g, :].view(np.float16).astype(np.float64)
        V = v16[t0:t1, g, :].view(np.float16).astype(np.float64)
        s = (q[g * G:(g + 1) * G].astype(np.float64) @ K.T) / np.sqrt(np.float64(hd))
        mm = s.max(axis=1)
        p = np.exp(s - mm[:, None])
        m[g * G:(g + 1) * G] = mm
        l[g * G:(g + 1) * G] = p.sum(axis=1)
        O[g * G:(g + 1) * G] = p @ V
    return m, l, O


def lse_merge(ms, ls, Os):
    """Merge split partials: M = max m_s; w_s = exp(m_s - M); out = sum O_s w_s / sum l_s w_s.

    ms, ls: [ns, nH]; Os: [ns, nH, hd].  Reference: engine/wgsl/attn_dec.js:215-287 (attn_dec_combine),
    engine/wgsl/qwen35.js:1059-1080 (attn_combine), engine/wgsl/attn_tile.js:177-193."""
    ms = np.asarray(ms, np.float64); ls = np.asarray(ls, np.float64); Os = np.asarray(Os, np.float64)
    M = ms.max(axis=0)
    w = np.exp(ms - M[None, :])
    L = (ls * w).sum(axis=0)
    return (Os * w[:, :, None]).sum(axis=0) / L[:, None]


# ---------------------------------------------------------------------------------------------
# the reference's split / tile sizing formulas (integer closed forms)
# ---------------------------------------------------------------------------------------------

def dec_split_len(s, S):
    """engine/wgsl/attn_dec.js:47 / :64 (fd_split): max(64, up64(ceil(s / S)))."""
    return max(64, -(-(-(-s // S)) // 64) * 64)


def dec_splits(s, S):
    """engine/wgsl/attn_dec.js:48: ceil(s / decSplitLen(s, S))."""
    return -(-s // dec_split_len(s, S))


def dec_default_S(n_kv):
    """engine/wgsl/attn_dec.js:42: S = max(16, floor(256 / nKV))."""
    return max(16, 256 // n_kv)


def fa_sizing(max_seq):
    """engine/qwen35.js:367-368: faSplit = max(256, up64(maxSeq / 128)); faSplits = ceil(maxSeq / faSplit)."""
    fa_split = max(256, -(-max_seq // (128 * 64)) * 64)
    return fa_split, -(-max_seq // fa_split)


def tile_split_len(seq_end, fa_split, fa_splits, target=32):
    """engine/wgsl/attn_tile.js:53-56 (tileSplitLen)."""
    up64 = lambda x: -(-x // 64) * 64
    return min(fa_split, max(64, up64(-(-seq_end // target)), up64(-(-seq_end // fa_splits))))


# ---------------------------------------------------------------------------------------------
# seeded synthetic inputs shared by tests, smoke and bench
# ---------------------------------------------------------------------------------------------

def make_inputs(cfg, ctx, n_cols, seed, with_cache_rows=True):
    """Seeded N(0,1) raw tensors for one layer.

    Returns dict: qraw [n_cols, nH*hd*(2 if gate)] (interleaved q|gate per head when cfg['gate']),
    kraw, vraw [ctx + n_cols, nKV*hd], qw, kw [hd] (ones + 0.1 N(0,1)).  Row t of kraw/vraw is the
    token at absolute position t; the last n_cols rows are the query columns' own k/v.
    """
    rng = np.random.default_rng(seed)
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd = nH * hd * (2 if cfg.get("gate", False) else 1)
    total = ctx + n_cols
    d = dict(
        qraw=rng.standard_normal((n_cols, qd), dtype=np.float32),
        kraw=rng.standard_normal((total, nKV * hd), dtype=np.float32) if with_cache_rows else None,
        vraw=rng.standard_normal((total, nKV * hd), dtype=np.float32) if with_cache_rows else None,
        qw=(1.0 + 0.1 * rng.standard_normal(hd)).astype(np.float32),
        kw=(1.0 + 0.1 * rng.standard_normal(hd)).astype(np.float32),
    )
    return d


def attn_layer_decode(x, kind_qkv, w_qkv, sc_qkv, kind_o, w_o, sc_o, attn_norm_w, qw, kw, k16, v16, pos, cfg):
    """One token through the attention half of a full-attention layer; returns (x_out f32 [dim], k16 row, v16 row).

    Reference: engine/qwen35.js:1586-1641 (_encodeLayerR, L.isFull): rmsnorm -> q / [k | v] GEMVs -> pre-step ->
    KV write -> attention over rows [0, pos] -> sigmoid gate -> wo GEMV -> residual add.  k16 / v16: cache rows
    [0, pos) as f16 bits [pos, nKV, hd].  f32 hand-offs between the stages, as the engine's buffers are.
    """
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    gated = cfg.get("gate", False)
    xn = rmsnorm(x, attn_norm_w, cfg["eps"])
    qkv = gemv(kind_qkv, w_qkv, sc_qkv, xn).astype(np.float32)
    q_rows = nH * hd * (2 if gated else 1)
    kvd = nKV * hd
    g = glue_kv(qkv[None, :q_rows], qkv[None, q_rows:q_rows + kvd], qkv[None, q_rows + kvd:], qw, kw, pos, cfg)
    kall = np.concatenate([np.asarray(k16).reshape(pos, nKV, hd), g["k16"].reshape(1, nKV, hd)])
    vall = np.concatenate([np.asarray(v16).reshape(pos, nKV, hd), g["v16"].reshape(1, nKV, hd)])
    out = attention(g["q"], kall, vall, pos, gate=g["gate"] if gated else None)            # [1, nH, hd]
    y = gemv(kind_o, w_o, sc_o, np.asarray(out, dtype=np.float32).reshape(-1))
    return (np.asarray(x, dtype=np.float32).astype(np.float64) + y).astype(np.float32), g["k16"], g["v16"]


def gemm_f16(kind, w, scales, x):
    """Y[c] = W x[c] with the reference's "f16" prefill math: every dequantised weight and every activation rounded
    to f16, products and sums exact (f64 here, f32 in the kernels).  x: [n, d_in] f32 (or f16-representable) -> [n, d_out].

    Reference: engine/wgsl/gemm.js:31-36 (the r16 twins: "every dequantized weight and every activation rounded to f16
    (pack2x16float), products and sums still f32 ... the operand precision of the tensor-core path"), gemm_sgm.js.
    """
    w16 = w_dequant(kind, w, scales).astype(np.float32).astype(np.float16).astype(np.float64)     # the product is exact in f32
    x16 = np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float64)
    return x16 @ w16.T


def attn_layer_prefill(x, kind_qkv, w_qkv, sc_qkv, kind_o, w_o, sc_o, attn_norm_w, qw, kw, k16, v16, base_pos, cfg):
    """n tokens at positions base_pos .. through the attention half of a full-attention layer; returns (x_out f32
    [n, dim], new k16 rows, new v16 rows).  k16 / v16: cache rows [0, base_pos).

    Reference: engine/qwen35.js:2416-2425 (_encodeLayerBatch), :2827 (_encodeLayerWide): per-column rmsnorm -> batched
    q / k / v GEMMs -> pre-step + KV write -> causal attention -> gate -> wo GEMM -> residual add, with the f16 operand
    rounding of gemm_f16 on both GEMMs (the attention output is handed over as f16).
    """
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    gated = cfg.get("gate", False)
    x = np.asarray(x, dtype=np.float32)
    n = x.shape[0]
    xn = np.stack([rmsnorm(x[c], attn_norm_w, cfg["eps"]) for c in range(n)])
    qkv = gemm_f16(kind_qkv, w_qkv, sc_qkv, xn).astype(np.float32)
    q_rows = nH * hd * (2 if gated else 1)
    kvd = nKV * hd
    g = glue_kv(qkv[:, :q_rows], qkv[:, q_rows:q_rows + kvd], qkv[:, q_rows + kvd:], qw, kw, base_pos, cfg)
    kall = np.concatenate([np.asarray(k16).reshape(base_pos, nKV, hd), g["k16"].reshape(n, nKV, hd)])
    vall = np.concatenate([np.asarray(v16).reshape(base_pos, nKV, hd), g["v16"].reshape(n, nKV, hd)])
    out = attention(g["q"], kall, vall, base_pos, gate=g["gate"] if gated else None)       # [n, nH, hd]
    y = gemm_f16(kind_o, w_o, sc_o, np.asarray(out, dtype=np.float32).reshape(n, -1))
    return (x.astype(np.float64) + y).astype(np.float32), g["k16"], g["v16"]
