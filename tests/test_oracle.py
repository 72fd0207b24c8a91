"""Pins the CPU oracle (oracle/) with checks that do not restate its formulas: IEEE known answers, closed
forms, invariants, brute force on tiny inputs, and agreement between the numpy, C and JavaScript legs.
The reference ships no golden vectors for attention in isolation (its tests generate inputs inline and
compare with an inline f64 closed form), so these are what fix the oracle."""
import json
import math
import os
import shutil
import struct
import subprocess
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from helpers import SHAPES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_f16_known_answers():
    # IEEE binary16, round to nearest even (values from the format definition)
    cases = [(0.0, 0x0000), (-0.0, 0x8000), (1.0, 0x3C00), (-2.0, 0xC000), (65504.0, 0x7BFF), (65520.0, 0x7C00),
             (1e-8, 0x0000), (2.0 ** -24, 0x0001), (2.0 ** -14, 0x0400), (0.333251953125, 0x3555),
             (1.0 + 2.0 ** -11, 0x3C00),            # tie -> even (down)
             (1.0 + 3 * 2.0 ** -11, 0x3C02),        # tie -> even (up)
             (1.0 + 2.0 ** -11 + 2.0 ** -20, 0x3C01),
             (2.0 ** -25, 0x0000), (2.0 ** -25 * 1.5, 0x0001), (float("inf"), 0x7C00)]
    for x, bits in cases:
        assert int(O.f16_bits(np.float32(x))) == bits, (x, hex(int(O.f16_bits(np.float32(x)))), hex(bits))
    # the reference test's own f16 (tests/test_attn_dec.js:24-25) agrees on normal numbers: spot values it would produce
    assert int(O.f16_bits(np.float32(0.3))) == 0x34CD and int(O.f16_bits(np.float32(-0.1))) == 0xAE66


def test_head_rmsnorm_closed_forms():
    hd = 64
    w = np.ones(hd, np.float32)
    x = np.full((1, 2, hd), 3.0, np.float32)
    y = O.head_rmsnorm(x, w, 0.0)
    assert np.allclose(y, 1.0, atol=1e-7)                       # constant head -> all ones
    e = np.zeros((1, 1, hd), np.float32); e[0, 0, 5] = 2.0
    y = O.head_rmsnorm(e, w, 0.0)
    assert abs(y[0, 0, 5] - math.sqrt(hd)) < 1e-5 and np.count_nonzero(y) == 1   # one-hot -> sqrt(hd)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 4, hd), dtype=np.float32)
    wv = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    eps = 1e-6
    y = O.head_rmsnorm(x, wv, eps)
    ss = (x.astype(np.float64) ** 2).sum(-1)
    # mean((y/w)^2) = 1 / (1 + eps*hd/ss)
    got = ((y / wv).astype(np.float64) ** 2).mean(-1)
    assert np.allclose(got, 1.0 / (1.0 + eps * hd / ss), rtol=1e-6)
    assert np.allclose(O.head_rmsnorm(2 * x, wv, 0.0), O.head_rmsnorm(x, wv, 0.0), rtol=1e-6)   # scale invariance at eps 0


def test_rope_invariants():
    rng = np.random.default_rng(1)
    hd, nrot, theta = 64, 32, 1e7
    x = rng.standard_normal((5, 3, hd), dtype=np.float32)
    assert np.array_equal(O.rope_neox(x, np.zeros(5, int), nrot, theta), x)              # pos 0 = identity
    pos = np.array([1, 7, 100, 4097, 131071])
    y = O.rope_neox(x, pos, nrot, theta)
    assert np.array_equal(y[..., nrot:], x[..., nrot:])                                  # dims >= n_rot untouched
    h = nrot // 2
    n0 = x[..., :h].astype(np.float64) ** 2 + x[..., h:nrot].astype(np.float64) ** 2
    n1 = y[..., :h].astype(np.float64) ** 2 + y[..., h:nrot].astype(np.float64) ** 2
    assert np.allclose(n0, n1, rtol=2e-6)                                                # pairwise norm preserved
    # pair 0 has frequency 1: at pos p the rotation angle is exactly p radians
    p = 3
    z = O.rope_neox(x[:1], np.array([p]), nrot, theta)
    a, b = x[0, :, 0].astype(np.float64), x[0, :, h].astype(np.float64)
    assert np.allclose(z[0, :, 0], a * math.cos(p) - b * math.sin(p), atol=1e-6)
    assert np.allclose(z[0, :, h], b * math.cos(p) + a * math.sin(p), atol=1e-6)
    # relative-position property: <rope(q,m), rope(k,n)> depends on m - n (small positions: f32 angles exact enough)
    q = rng.standard_normal((1, 1, hd), dtype=np.float32); k = rng.standard_normal((1, 1, hd), dtype=np.float32)
    d1 = (O.rope_neox(q, [10], nrot, theta).astype(np.float64) * O.rope_neox(k, [4], nrot, theta)).sum()
    d2 = (O.rope_neox(q, [16], nrot, theta).astype(np.float64) * O.rope_neox(k, [10], nrot, theta)).sum()
    assert abs(d1 - d2) < 1e-4
    # frequencies: full-rope table endpoints theta^0 = 1 and theta^(-(n-2)/n)
    f = O.rope_inv_freq(128, 1e6)
    assert f[0] == 1.0 and abs(f[-1] - 1e6 ** (-126 / 128)) < 1e-12 and f.dtype == np.float32


def test_qsplit_layout():
    nH, hd = 3, 4
    qf = np.arange(2 * nH * 2 * hd, dtype=np.float32).reshape(2, nH * 2 * hd)
    q, g = O.qsplit(qf, nH, hd)
    assert q[1, 2, 1] == qf[1, 2 * 2 * hd + 1] and g[1, 2, 1] == qf[1, 2 * 2 * hd + hd + 1]
    assert q[0, 0].tolist() == [0, 1, 2, 3] and g[0, 0].tolist() == [4, 5, 6, 7]


def _brute(q, k16, v16, base_pos, gate=None):
    """scalar-loop attention in Python floats (tiny shapes only)"""
    n, nH, hd = q.shape
    nKV = k16.shape[1]
    K = k16.view(np.float16).astype(np.float64); V = v16.view(np.float16).astype(np.float64)
    out = np.zeros((n, nH, hd))
    for c in range(n):
        for h in range(nH):
            g = h // (nH // nKV)
            sc = []
            for t in range(base_pos + c + 1):
                a = 0.0
                for i in range(hd):
                    a += float(q[c, h, i]) * K[t, g, i]
                sc.append(a / math.sqrt(hd))
            mx = max(sc)
            e = [math.exp(s - mx) for s in sc]
            tot = sum(e)
            for i in range(hd):
                out[c, h, i] = sum(e[t] * V[t, g, i] for t in range(len(e))) / tot
            if gate is not None:
                for i in range(hd):
                    out[c, h, i] *= 1.0 / (1.0 + math.exp(-float(gate[c, h, i])))
    return out


def test_attention_brute_force_and_legs_agree():
    rng = np.random.default_rng(2)
    nH, nKV, hd, base, n = 4, 2, 8, 5, 3
    q = rng.standard_normal((n, nH, hd), dtype=np.float32)
    gate = rng.standard_normal((n, nH, hd), dtype=np.float32)
    k16 = rng.standard_normal((base + n, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    v16 = rng.standard_normal((base + n, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    ref = _brute(q, k16, v16, base, gate)
    assert np.allclose(O.attention(q, k16, v16, base, gate=gate), ref, rtol=1e-12, atol=1e-14)
    assert np.allclose(C.attention(q, k16, v16, base, gate=gate), ref, rtol=1e-12, atol=1e-14)
    assert np.allclose(C.attention(q, k16, v16, base, gate=gate, rows=[2, 0]), ref[[2, 0]], rtol=1e-12, atol=1e-14)


def test_attention_invariants():
    rng = np.random.default_rng(3)
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    L = 300
    q = rng.standard_normal((1, nH, hd), dtype=np.float32)
    k16 = rng.standard_normal((L, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    v = rng.standard_normal((L, nKV, hd), dtype=np.float32).astype(np.float16)
    v16 = v.view(np.uint16)
    for att in (O.attention, C.attention):
        # one visible row -> that V row for every head of the group (tests/reference/ref_q38_layer.mjs:179-184)
        o = att(q, k16, v16, 0)
        for h in range(nH):
            assert np.array_equal(o[0, h], v[0, h // (nH // nKV)].astype(np.float64))
        # constant V -> that constant
        cv = np.full((L, nKV, hd), 0.75, np.float16).view(np.uint16)
        assert np.allclose(att(q, k16, cv, L - 1), 0.75, rtol=1e-12)
        # permuting the cache rows leaves a decode output unchanged
        perm = rng.permutation(L)
        a, b = att(q, k16, v16, L - 1), att(q, k16[perm], v16[perm], L - 1)
        assert np.allclose(a, b, rtol=1e-10, atol=1e-12)
        # q = 0 -> uniform softmax -> mean of V rows
        o = att(np.zeros_like(q), k16, v16, L - 1)
        assert np.allclose(o[0, 0], v[:, 0].astype(np.float64).mean(0), rtol=1e-12)
        # a huge score on one row -> that V row
        kk = k16.copy().view(np.float16); kk[17, 0] = (q[0, 0] * 40).astype(np.float16)
        o = att(q, kk.view(np.uint16), v16, L - 1)
        assert np.allclose(o[0, 0], v[17, 0].astype(np.float64), atol=1e-9)
        # NaN rows past the causal end never leak (tests/unit/attn_tile_test.js:43-50)
        kn, vn = k16.copy(), v16.copy(); kn[200:] = 0x7E00; vn[200:] = 0x7E00
        assert np.array_equal(att(q, kn, vn, 199), att(q, k16, v16, 199))
    # multi-column == single columns
    qq = rng.standard_normal((4, nH, hd), dtype=np.float32)
    multi = C.attention(qq, k16, v16, 100)
    for c in range(4):
        assert np.array_equal(multi[c], C.attention(qq[c:c + 1], k16, v16, 100 + c)[0])


def test_lse_merge_equals_unsplit():
    rng = np.random.default_rng(4)
    nH, nKV, hd, L = 6, 2, 16, 257
    q = rng.standard_normal((nH, hd), dtype=np.float32) * 3
    k16 = rng.standard_normal((L, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    v16 = rng.standard_normal((L, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    full = O.attention(q[None], k16, v16, L - 1)[0]
    for sl in (64, 100, 256, 1000):
        parts = [O.attention_partial(q, k16, v16, t0, min(L, t0 + sl)) for t0 in range(0, L, sl)]
        ms, ls, Os = (np.stack(x) for x in zip(*parts))
        assert np.allclose(O.lse_merge(ms, ls, Os), full, rtol=1e-12, atol=1e-14)
    m, l, Ov = O.attention_partial(q, k16, v16, 0, L)          # one split -> O / l
    assert np.allclose(O.lse_merge(m[None], l[None], Ov[None]), Ov / l[:, None], rtol=1e-15)


def test_split_formulas_known_answers():
    # values the reference's own comments and logs state: S = 128 for the MoE (2 kv heads), 64 for the 27B
    # (engine/wgsl/attn_dec.js:40-48), faSplit "<= 128 splits per head" (engine/qwen35.js:367)
    assert O.dec_default_S(2) == 128 and O.dec_default_S(4) == 64 and O.dec_default_S(32) == 16
    assert O.dec_split_len(1, 128) == 64 and O.dec_splits(1, 128) == 1
    assert O.dec_split_len(8192, 128) == 64 and O.dec_splits(8192, 128) == 128
    assert O.dec_split_len(8193, 128) == 128 and O.dec_splits(8193, 128) == 65
    assert O.dec_split_len(32769, 128) == 320 and O.dec_splits(32769, 128) == 103
    assert O.dec_split_len(65537, 64) == 1088 and O.dec_splits(65537, 64) == 61
    for s in (1, 63, 64, 65, 4097, 69999):
        for S in (16, 64, 128):
            sl = O.dec_split_len(s, S)
            assert sl % 64 == 0 and sl >= 64 and O.dec_splits(s, S) <= S
    assert O.fa_sizing(131072) == (1024, 128) and O.fa_sizing(2048) == (256, 8) and O.fa_sizing(65536) == (512, 128)
    for max_seq in (256, 4096, 32768, 262144):
        fs, fn = O.fa_sizing(max_seq)
        for seq_end in range(1, max_seq + 1, max(1, max_seq // 97)):
            tl = O.tile_split_len(seq_end, fs, fn)
            assert tl % 64 == 0 and 64 <= tl <= fs and -(-seq_end // tl) <= fn      # tests/unit/attn_tile_test.js:84-100


@pytest.mark.skipif(shutil.which("node") is None, reason="node not installed")
def test_js_leg_matches_numpy_leg(tmp_path):
    rng = np.random.default_rng(5)
    nH, nKV, hd, base, n = 6, 2, 32, 70, 3
    q = rng.standard_normal((n, nH, hd), dtype=np.float32)
    gate = rng.standard_normal((n, nH, hd), dtype=np.float32)
    k16 = rng.standard_normal((base + n, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    v16 = rng.standard_normal((base + n, nKV, hd), dtype=np.float32).astype(np.float16).view(np.uint16)
    sel = np.array([0, 2], np.int32)
    inp = tmp_path / "in.bin"; outp = tmp_path / "out.bin"
    with open(inp, "wb") as f:
        f.write(struct.pack("8i", n, nH, nKV, hd, base, base + n, 1, len(sel)))
        f.write(sel.tobytes()); f.write(q.tobytes()); f.write(k16.tobytes()); f.write(v16.tobytes()); f.write(gate.tobytes())
    r = subprocess.run(["node", os.path.join(ROOT, "oracle", "attn_ref.js"), str(inp), str(outp), "1"], capture_output=True, text=True, check=True)
    info = json.loads(r.stdout.strip().splitlines()[-1])
    assert info["threads"] == 1 and info["cols"] == 2
    got = np.fromfile(outp, dtype=np.float32).reshape(2, nH, hd)
    ref = O.attention(q, k16, v16, base, gate=gate)[sel]
    assert np.abs(got - ref).max() < 2e-6           # the JS leg stores scores and sums in Float32Array


def test_glue_kv_composition():
    cfg = SHAPES["qwen36_moe"]
    d = O.make_inputs(cfg, 0, 3, seed=6)
    g = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], 1000, cfg)
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    assert g["q"].shape == (3, nH, hd) and g["gate"].shape == (3, nH, hd) and g["k16"].shape == (3, nKV, hd)
    assert np.array_equal(g["v16"], O.f16_bits(d["vraw"].reshape(3, nKV, hd)))                  # V untouched
    assert np.array_equal(g["gate"][2, 5], d["qraw"][2, 5 * 2 * hd + hd: 5 * 2 * hd + 2 * hd])
    qn = O.head_rmsnorm(O.qsplit(d["qraw"], nH, hd)[0], d["qw"], cfg["eps"])
    assert np.array_equal(g["q"][..., cfg["n_rot"]:], qn[..., cfg["n_rot"]:])                   # un-rotated dims = normed q


def test_q8_quantize_known_answers():
    """int8 KV blocks (engine/wgsl/qwen35.js:908-946): answers fixed by the definition, not by the oracle's code."""
    z = np.zeros(32, np.float32)
    q, sc = O.q8_quantize(z)
    assert sc.shape == (1,) and sc[0] == 0 and not q.any()                       # all-zero block: scale 0, inv 0
    x = np.zeros(32, np.float32); x[0] = 127.0; x[1:8] = [0.5, 1.5, 2.5, -0.5, -1.5, 3.49, -126.6]
    q, sc = O.q8_quantize(x)
    assert sc[0] == 1.0                                                           # max 127 -> scale exactly 1
    assert q[:8].tolist() == [127, 0, 2, 2, 0, -2, 3, -127]                       # ties to even; -126.6 -> -127
    x = np.linspace(-3, 3, 64, dtype=np.float32); x[40] = 9.0                     # two blocks with their own scales
    q, sc = O.q8_quantize(x)
    assert sc[0] == np.float32(3.0) / np.float32(127.0) and sc[1] == np.float32(9.0) / np.float32(127.0)
    assert q[0] == -127 and q[40] == 127 and np.abs(q).max() == 127
    d = O.q8_dequantize(q, sc)
    assert np.all(np.abs(d - x) <= np.repeat(sc, 32) * 0.5000001)                 # rounding error at most half a step
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 3, 256), dtype=np.float32)
    q, sc = O.q8_quantize(x)
    assert q.shape == x.shape and sc.shape == (5, 3, 8)
    blocks = x.reshape(5, 3, 8, 32)
    assert np.array_equal(np.abs(q.reshape(5, 3, 8, 32)).max(-1), np.full((5, 3, 8), 127))     # the block maximum maps to +-127


# ---- projections: weight planes, GEMV, rmsnorm ------------------------------------------------------------------

def _f16b(x):
    return np.asarray(x, np.float16).view(np.uint16)


def test_w_dequant_known_blocks():
    """Hand-made blocks: nibble order and sign of Q4_0 (engine/wgsl/base.js:81-83), byte order and sign of Q8_0."""
    # Q4_0, one row of one block, scale 0.5: byte j = (low nibble -> element j, high nibble -> element j + 16)
    b = np.zeros((1, 16), np.uint8)
    b[0, 0] = 0xF0          # element 0: nibble 0 -> -8;  element 16: nibble 15 -> +7
    b[0, 3] = 0x89          # element 3: nibble 9 -> +1;  element 19: nibble 8 -> 0
    b[0, 15] = 0x08         # element 15: nibble 8 -> 0;  element 31: nibble 0 -> -8
    w = O.w_dequant(O.W_Q4_0, b, _f16b([[0.5]]))
    want = np.full(32, -8.0 * 0.5)            # untouched bytes are 0x00: both nibbles 0 -> -8
    want[0], want[16], want[3], want[19], want[15], want[31] = -4.0, 3.5, 0.5, 0.0, 0.0, -4.0
    assert np.array_equal(w[0], want)
    # Q8_0: two blocks with different scales, negative values
    q = np.zeros((1, 64), np.int8); q[0, 0], q[0, 31], q[0, 32], q[0, 63] = -128, 127, 5, -1
    w = O.w_dequant(O.W_Q8_0, q, _f16b([[0.25, 2.0]]))
    assert w[0, 0] == -32.0 and w[0, 31] == 31.75 and w[0, 32] == 10.0 and w[0, 63] == -2.0 and np.count_nonzero(w) == 4


def test_gemv_matches_the_reference_loops_and_is_linear():
    rng = np.random.default_rng(3)
    d_out, d_in = 5, 96
    x = rng.standard_normal(d_in).astype(np.float32)
    sc = _f16b(rng.uniform(0.01, 0.2, (d_out, d_in // 32)))
    cases = [(O.W_F32, rng.standard_normal((d_out, d_in)).astype(np.float32), None),
             (O.W_Q8_0, rng.integers(-128, 128, (d_out, d_in)).astype(np.int8), sc),
             (O.W_Q4_0, rng.integers(0, 256, (d_out, d_in // 2)).astype(np.uint8), sc)]
    for kind, w, s in cases:
        y = O.gemv(kind, w, s, x)
        assert np.allclose(y, O.gemv_reference_loops(kind, w, s, x), rtol=1e-12, atol=1e-12)
        # unit vectors pick columns of the dequantised matrix; linearity
        e = np.zeros(d_in, np.float32); e[37] = 1.0
        assert np.array_equal(O.gemv(kind, w, s, e), O.w_dequant(kind, w, s)[:, 37])
        x2 = rng.standard_normal(d_in).astype(np.float32)
        lhs = O.gemv(kind, w, s, x) * 2.0 + O.gemv(kind, w, s, x2)
        assert np.allclose(lhs, O.w_dequant(kind, w, s) @ (2.0 * x.astype(np.float64) + x2), rtol=1e-12)


def test_rmsnorm_closed_forms():
    n, eps = 64, 1e-6
    w = np.linspace(0.5, 1.5, n).astype(np.float32)
    x = np.full(n, 3.0, np.float32)
    assert np.allclose(O.rmsnorm(x, w, eps), w * 3.0 / np.sqrt(9.0 + eps), rtol=1e-6)
    rng = np.random.default_rng(1)
    x = rng.standard_normal(n).astype(np.float32)
    y = O.rmsnorm(x, np.ones(n, np.float32), 0.0)
    assert abs(np.mean(y.astype(np.float64) ** 2) - 1.0) < 1e-6                      # unit RMS
    assert np.allclose(O.rmsnorm(4.0 * x, w, 0.0), O.rmsnorm(x, w, 0.0), rtol=1e-6)  # scale invariance at eps = 0


def test_gemm_f16_pins():
    """gemm_f16 (the reference's "f16" prefill math, engine/wgsl/gemm.js:31-36) pinned without restating it:
    unit-vector columns pick the f16-rounded columns of w_dequant (known answers for hand-made blocks whose scales
    make the products inexact in f16); f16-representable inputs over weights whose dequantised values are already
    f16 reproduce gemv exactly; the result is linear in x over f16-representable inputs; and an activation that is
    not f16-representable is rounded before the product (closed form on a one-hot weight row)."""
    rng = np.random.default_rng(31)
    d_out, d_in = 5, 64
    for kind in (O.W_Q8_0, O.W_Q4_0):
        w = rng.integers(-127, 128, (d_out, d_in)).astype(np.int8) if kind == O.W_Q8_0 else rng.integers(0, 256, (d_out, d_in // 2), dtype=np.uint8)
        sc = rng.uniform(0.01, 0.3, (d_out, d_in // 32)).astype(np.float16).view(np.uint16)
        W = O.w_dequant(kind, w, sc)                                   # exact products int x f16 scale (f64)
        W16 = W.astype(np.float32).astype(np.float16).astype(np.float64)
        assert np.any(W16 != W), "the case is meant to include weights that f16 rounds"
        # unit vectors pick the rounded columns
        Y = O.gemm_f16(kind, w, sc, np.eye(d_in, dtype=np.float32))    # [d_in, d_out]
        assert np.array_equal(Y, W16.T)
        # linearity over f16-representable inputs (small integers: every product and sum is exact in f64)
        xa = rng.integers(-8, 9, (3, d_in)).astype(np.float32); xb = rng.integers(-8, 9, (3, d_in)).astype(np.float32)
        assert np.array_equal(O.gemm_f16(kind, w, sc, xa + xb), O.gemm_f16(kind, w, sc, xa) + O.gemm_f16(kind, w, sc, xb))
    # weights whose dequantised values are f16-representable (power-of-two scales): gemm_f16 == gemv on f16 inputs
    w8 = rng.integers(-127, 128, (d_out, d_in)).astype(np.int8)
    sc2 = np.full((d_out, d_in // 32), 0.125, np.float16).view(np.uint16)
    x16 = rng.standard_normal((4, d_in)).astype(np.float16).astype(np.float32)
    want = np.stack([O.gemv(O.W_Q8_0, w8, sc2, x16[c]) for c in range(4)])
    assert np.array_equal(O.gemm_f16(O.W_Q8_0, w8, sc2, x16), want)
    # f32 weights: a one-hot row times x returns f16(w) * f16(x)
    wf = np.zeros((2, 32), np.float32); wf[0, 3] = 1.0 + 2.0 ** -12; wf[1, 7] = 3.0       # 1 + 2^-12 rounds to 1 in f16
    x = np.zeros((1, 32), np.float32); x[0, 3] = 1.0 + 2.0 ** -11 + 2.0 ** -12; x[0, 7] = 0.1   # rounds up to 1 + 2^-10
    y = O.gemm_f16(O.W_F32, wf, None, x)
    assert y[0, 0] == 1.0 + 2.0 ** -10
    assert y[0, 1] == 3.0 * float(np.float16(0.1))
