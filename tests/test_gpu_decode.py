"""GPU parity of decode / speculative-verify attention through the C ABI against the CPU oracle.
Tolerance (floating point): max-abs <= 2e-3 and max|d|/max|ref| <= 1e-2 of the f32/f64 reference."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PA_OUT_F16
from helpers import SHAPES, assert_parity, random_cache, oracle_cache

pytestmark = pytest.mark.gpu

NAN16 = 0x7E00


def _ctx_with_cache(cfg, k16, v16, max_seq, max_cols=16, poison_from=None):
    pa = PooledAttn(cfg, max_seq, n_layers=1, max_cols=max_cols)
    pa.layer_alloc(0)
    K, V = k16.copy(), v16.copy()
    if poison_from is not None:
        K[poison_from:] = NAN16; V[poison_from:] = NAN16
    pa.kv_write(0, 0, 0, K); pa.kv_write(0, 1, 0, V)
    return pa


SEQ_LENS = [1, 2, 5, 31, 32, 33, 63, 64, 65, 127, 128, 129, 300, 1000, 2049, 4097]


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_decode_seq_lens(shape):
    """The context lengths of tests/test_attn_dec.js:106-107 (split-length steps), K in +-0.3-like spread."""
    cfg = SHAPES[shape]
    rng = np.random.default_rng(7)
    max_seq = max(SEQ_LENS) + 40
    k16, v16 = random_cache(cfg, max_seq, seed=8)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32) * 2
    with _ctx_with_cache(cfg, k16, v16, max_seq) as pa:
        for L in SEQ_LENS:
            # rows at or past L are NaN: any causal leak poisons the output (tests/unit/attn_tile_test.js:43-50)
            pa.kv_write(0, 0, 0, np.where(np.arange(max_seq)[:, None, None] < L, k16, NAN16).astype(np.uint16))
            pa.kv_write(0, 1, 0, np.where(np.arange(max_seq)[:, None, None] < L, v16, NAN16).astype(np.uint16))
            got = pa.run_attn("decode", 0, q, L - 1)
            ref = C.attention(q, k16, v16, L - 1)
            assert_parity(got, ref, "%s seqLen %d" % (shape, L))


def test_decode_closed_forms():
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rng = np.random.default_rng(9)
    L = 1500
    k16, v16 = random_cache(cfg, L, seed=10)
    q = rng.standard_normal((1, nH, hd), dtype=np.float32)
    v = v16.view(np.float16)
    with _ctx_with_cache(cfg, k16, v16, L) as pa:
        o = pa.run_attn("decode", 0, q, 0)                                 # one row -> that V row
        for h in range(nH):
            assert np.allclose(o[0, h], v[0, h // (nH // nKV)].astype(np.float32), atol=1e-6)
        o = pa.run_attn("decode", 0, np.zeros_like(q), L - 1)               # q = 0 -> mean of V rows
        assert np.abs(o[0, 3] - v[:, 0].astype(np.float64).mean(0)).max() < 2e-4
        pa.kv_write(0, 1, 0, np.full((L, nKV, hd), 0x3A00, np.uint16))      # constant V = 0.75
        assert np.abs(pa.run_attn("decode", 0, q, L - 1) - 0.75).max() < 1e-3


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_outputs_are_convex_combinations_of_value_rows(shape):
    """Every value row the same vector => the output is that vector, whatever the scores: the row total l is summed
    from the f16-rounded probabilities the PV product uses, so the weights that are applied add up to exactly the
    divisor and the rounding of P cancels (with l summed from the unrounded exponentials the outputs were off by up to
    3e-4 of the value on short contexts).  What is left is f32 accumulation: a few 1e-7.  One-column decodes and verify
    blocks on the single-round kernel and on the tile loop, chunks on the split-K kernel with direct output and on the
    matrix-core kernel, with and without a split over the context."""
    cfg = SHAPES[shape]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rng = np.random.default_rng(5)
    L = 40000
    k16, _ = random_cache(cfg, L, seed=3, k_scale=2.0)
    vrow = rng.standard_normal((nKV, hd)).astype(np.float16)
    v16 = np.broadcast_to(vrow.view(np.uint16), (L, nKV, hd)).copy()
    want = np.repeat(vrow.astype(np.float64), nH // nKV, axis=0)
    with _ctx_with_cache(cfg, k16, v16, L, max_cols=400) as pa:
        kernels = set()
        for kind, n, lens in (("decode", 1, (1, 2, 3, 17, 40, 129, 1500, 33000, 39999)), ("decode", 5, (6, 40, 1500, 33000)),
                              ("prefill", 12, (12, 300)), ("prefill", 300, (300, 5000))):
            for Lc in lens:
                q = rng.standard_normal((n, nH, hd), dtype=np.float32)
                pl = pa.plan(kind, Lc - n, n)
                kernels.add((pl["kernel"], pl["n_splits"] > 1, pl["split_len"] == 128))
                o = pa.run_attn(kind, 0, q, Lc - n).astype(np.float64)
                err = np.abs(o - want[None]).max() / np.abs(want).max()
                assert err < 2e-6, "%s %s %d columns over %d rows: %.2e of the value (%s)" % (shape, kind, n, Lc, err, pl)
        assert {k[0] for k in kernels} == {0, 1} and any(k[1] and k[2] for k in kernels) and any(k[1] and not k[2] for k in kernels), kernels


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_short_context_decode_sees_q_at_f32_precision(shape):
    """A block of at most eight stacked rows carries the f16 rounding error of q in rows 8 .. 15 of its q tile, so its
    scores see q at f32 precision.  Inputs that make the rounding of q visible (q of twice, keys of twice the
    benchmark's spread: scores of a spread of 4, a few rows share the weight whatever the length) come out within 6e-4 of
    the f64 oracle (measured: up to 4.1e-4, what the f16 rounding of P leaves); with q rounded to f16 the same inputs are
    off by 1.6e-3 to 4.7e-3."""
    cfg = SHAPES[shape]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rng = np.random.default_rng(11)
    Lmax = 4100
    k16, v16 = random_cache(cfg, Lmax, seed=13, k_scale=2.0)
    with _ctx_with_cache(cfg, k16, v16, Lmax) as pa:
        for n in sorted({1, 8 // (nH // nKV)}):
            for L in (2, 3, 5, 17, 33, 129, 300, 1000, 2047, 2049, 4097):
                if L <= n:
                    continue
                for rep in range(3):
                    q = rng.standard_normal((n, nH, hd), dtype=np.float32) * 2
                    got = pa.run_attn("decode", 0, q, L - n)
                    ref = C.attention(q, k16[:L], v16[:L], L - n)
                    d = float(np.abs(got - ref).max())
                    assert d < 6e-4, "%s %d columns over %d rows: max-abs %.3e" % (shape, n, L, d)


def test_decode_split_invariance_and_plan():
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(11)
    L = 5000
    k16, v16 = random_cache(cfg, L, seed=12)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32) * 1.5
    ref = C.attention(q, k16, v16, L - 1)
    with _ctx_with_cache(cfg, k16, v16, L) as pa:
        outs = []
        for s in (0, 1, 3, 16, 40):
            pa.set_decode_splits(s)
            pl = pa.plan("decode", L - 1, 1)
            # a one-column decode streams rows 0 .. L - 2; its own row L - 1 is one more partial (slots = splits + 1)
            assert pl["n_splits"] * pl["split_len"] >= L - 1 and pl["split_len"] % 32 == 0 and pl["slots"] == pl["n_splits"] + 1
            if s:
                assert pl["n_splits"] <= s
            outs.append(pa.run_attn("decode", 0, q, L - 1))
            assert_parity(outs[-1], ref, "splits %d" % s)
        assert max(np.abs(o - outs[0]).max() for o in outs) < 2e-4
        # deterministic run to run
        pa.set_decode_splits(0)
        assert np.array_equal(pa.run_attn("decode", 0, q, L - 1), pa.run_attn("decode", 0, q, L - 1))


@pytest.mark.parametrize("pos", [63 * 128, 64 * 128, 64 * 128 + 77, 12000])
def test_decode_either_side_of_the_f16_partials_threshold(pos):
    """A one-column decode writes f16 O partials from 64 single-round splits on (f32 below): both sides of the threshold,
    a remainder split, and a longer context against the f64 oracle, with the margin the five configurations are held to."""
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(pos)
    k16, v16 = random_cache(cfg, pos + 1, seed=pos + 1)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = C.attention(q, k16, v16, pos, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, pos + 1) as pa:
        pl = pa.plan("decode", pos, 1)
        assert pl["split_len"] == 128 and (pl["n_splits"] >= 64) == (pos >= 64 * 128)
        for out_dtype in (0, PA_OUT_F16):
            assert_parity(pa.run_attn("decode", 0, q, pos, gate=gate, out_dtype=out_dtype), ref, "decode at %d, %d splits" % (pos, pl["n_splits"]), tight=True)


@pytest.mark.parametrize("shape,n_cols,base", [("qwen36_moe", 4, 996), ("qwen36_moe", 16, 3000), ("qwen38_27b", 8, 2040),
                                               ("qwen3_1p7b", 4, 510), ("qwen38_27b", 16, 17), ("qwen36_moe", 7, 0),
                                               ("qwen36_moe", 16, 20000), ("qwen38_27b", 12, 30000), ("qwen3_1p7b", 16, 9000)])
def test_verify_equals_sequential_decodes(shape, n_cols, base):
    """A verify block must equal n sequential single-token decodes (engine/wgsl/attn_dec.js:12-16;
    tests/test_attn_dec.js:89-97) -- here within tolerance -- and the oracle."""
    cfg = SHAPES[shape]
    rng = np.random.default_rng(base + n_cols)
    L = base + n_cols
    k16, v16 = random_cache(cfg, L + 5, seed=13)
    q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32) if cfg["gate"] else None
    ref = C.attention(q, k16, v16, base, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, L + 5, poison_from=L) as pa:
        multi = pa.run_attn("decode", 0, q, base, gate=gate)
        assert_parity(multi, ref, "verify block")
        for c in range(n_cols):
            single = pa.run_attn("decode", 0, q[c:c + 1], base + c, gate=None if gate is None else gate[c:c + 1])
            assert_parity(single, ref[c:c + 1], "single decode col %d" % c)
            assert np.abs(single[0] - multi[c]).max() <= 1e-3


@pytest.mark.parametrize("shape,n_cols,base", [("qwen36_moe", 4, 8000), ("qwen38_27b", 5, 5000), ("qwen3_1p7b", 12, 3000), ("qwen36_moe", 3, 16200),
                                               ("qwen36_moe", 8, 4090)])
def test_verify_block_on_the_single_round_kernel_with_two_row_blocks(shape, n_cols, base):
    """A verify block of 17 .. 32 stacked rows a workgroup over a context that fits one round of one-tile-per-wave splits
    at one workgroup a CU: the single-round kernel with two row blocks (f16 caches).  Causal ends differ by column, the
    last split is partial, rows past the context are poisoned; f32 and f16 out, with a gate where the shape has one."""
    cfg = SHAPES[shape]
    rng = np.random.default_rng(base + n_cols)
    L = base + n_cols
    k16, v16 = random_cache(cfg, L + 40, seed=base)
    q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
    ref = C.attention(q, k16, v16, base, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, L + 40, max_cols=n_cols, poison_from=L) as pa:
        pl = pa.plan("decode", base, n_cols)
        assert pl["row_blocks"] == 2 and pl["split_len"] == 128 and pl["n_splits"] == -(-L // 128) and pl["slots"] == pl["n_splits"], pl
        for out_dtype in (0, PA_OUT_F16):
            assert_parity(pa.run_attn("decode", 0, q, base, gate=gate, out_dtype=out_dtype), ref, "two row blocks, single round, %d columns at %d" % (n_cols, base), tight=True)
        pa.set_decode_splits(max(2, pl["n_splits"] // 3))            # the same block on the tile loop's contiguous splits
        assert pa.plan("decode", base, n_cols)["split_len"] > 128
        assert np.abs(pa.run_attn("decode", 0, q, base, gate=gate) - pa_first(pa, q, base, gate)).max() <= 2e-4


def pa_first(pa, q, base, gate):
    """The table's plan again (after a splits override)."""
    pa.set_decode_splits(0)
    return pa.run_attn("decode", 0, q, base, gate=gate)


@pytest.mark.parametrize("shape,n_cols,base", [("qwen36_moe", 4, 996), ("qwen38_27b", 8, 2040), ("qwen3_1p7b", 5, 510), ("qwen36_moe", 3, 32767),
                                               ("qwen36_moe", 8, 9000), ("qwen36_moe", 16, 20000), ("qwen38_27b", 6, 8190), ("qwen3_1p7b", 13, 119),
                                               ("qwen36_moe", 5, 40000), ("qwen38_27b", 4, 33000), ("qwen38_27b", 8, 65533)])
def test_verify_exact_flag_gives_the_sequential_decodes_bits(shape, n_cols, base):
    """PA_FLAG_VERIFY_EXACT: every column of a verify block has the bits of the one-column decode at its position
    (the reference's invariant, engine/wgsl/attn_dec.js:12-16; tests/test_attn_dec.js:89-97 checks it with Object.is);
    the plan a plan query reports is unchanged.  Blocks whose columns share a one-column plan run as one pass (the first
    three cases and the 9000- and 20000-row ones, with f16 partials on the last two; the 40000- and 33000-row ones on the
    tile loop's longer splits); blocks that straddle a change of plan (32767 .. 32769, 8190 .. 8195, 119 .. 131, and
    65536 .. 65543 of the 27B shape, where the tile loop goes from eight to nine tiles a wave) run as one pass per run of
    columns with the same plan, a lone column as the one-column decode itself."""
    cfg = dict(SHAPES[shape], verify_exact=True)
    rng = np.random.default_rng(base + n_cols)
    L = base + n_cols
    k16, v16 = random_cache(cfg, L + 5, seed=14)
    q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
    ref = C.attention(q, k16, v16, base, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, L + 5, poison_from=L) as pa:
        multi = pa.run_attn("decode", 0, q, base, gate=gate)
        assert_parity(multi, ref, "column-exact verify block")
        for c in range(n_cols):
            single = pa.run_attn("decode", 0, q[c:c + 1], base + c, gate=None if gate is None else gate[c:c + 1])
            assert np.array_equal(single[0].view(np.uint32), multi[c].view(np.uint32)), "column %d differs from its decode" % c


def test_decode_f16_output_and_strides():
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(14)
    L, n = 700, 3
    k16, v16 = random_cache(cfg, L + n, seed=15)
    q = rng.standard_normal((n, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = C.attention(q, k16, v16, L, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, L + n) as pa:
        got = pa.run_attn("decode", 0, q, L, gate=gate, out_dtype=PA_OUT_F16)
        assert got.dtype == np.float16
        assert_parity(got.astype(np.float32), ref, "f16 out")
        # padded column strides (the engine aligns columns to 256 bytes, engine/qwen35.js:2054-2055)
        qd, pad = pa.q_dim, 64
        qp = np.full((n, qd + pad), np.nan, np.float32); qp[:, :qd] = q.reshape(n, -1)
        gp = np.full((n, qd + pad), np.nan, np.float32); gp[:, :qd] = gate.reshape(n, -1)
        dq, dg = pa.to_device(qp), pa.to_device(gp)
        dout = pa.to_device(np.full((n, qd + pad), -7.0, np.float32))
        pa.attn("decode", 0, dq, qd + pad, dg, qd + pad, L, n, dout, qd + pad)
        pa.sync()
        o = dout.download(np.float32, n * (qd + pad)).reshape(n, qd + pad)
        assert_parity(o[:, :qd].reshape(ref.shape), ref, "padded strides")
        assert np.all(o[:, qd:] == -7.0), "wrote into the padding between columns"


def test_c1_decode_full_pipeline():
    """Config 1: Qwen3-1.7B shape, ctx 2048, pre-step (QK-RMSNorm + full RoPE theta 1e6) on the GPU for the
    query column, cache rows built by the oracle's pre-step; f32 softmax; f16 output."""
    cfg = SHAPES["qwen3_1p7b"]
    ctx = 2048
    d = O.make_inputs(cfg, ctx, 1, seed=0x5EED0001)
    k16, v16 = oracle_cache(cfg, d["kraw"][:ctx], d["vraw"][:ctx], d["kw"])
    g = O.glue_kv(d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx, cfg)
    kall = np.concatenate([k16, g["k16"]]); vall = np.concatenate([v16, g["v16"]])
    ref = C.attention(g["q"], kall, vall, ctx)
    with PooledAttn(cfg, ctx + 1, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        pa.run_glue_kv(0, d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx)
        assert np.array_equal(pa.kv_read(0, 0, ctx, 1), g["k16"])
        dout = pa.alloc(pa.q_dim * 2)
        pa.attn("decode", 0, None, 0, None, 0, ctx, 1, dout, pa.q_dim, PA_OUT_F16)    # q from the context's buffer
        pa.sync()
        got = dout.download(np.float16, pa.q_dim).reshape(ref.shape).astype(np.float32)
    assert_parity(got, ref, "C1 decode, f16 out", tight=True)


def test_c3_gated_decode_32k():
    """Config 3: Qwen3.6-35B-MoE attention shape, ctx 32768, partial RoPE (64 dims, theta 1e7), sigmoid gate."""
    cfg = SHAPES["qwen36_moe"]
    ctx = 32768
    d = O.make_inputs(cfg, ctx, 1, seed=0x5EED0003)
    k16, v16 = oracle_cache(cfg, d["kraw"][:ctx], d["vraw"][:ctx], d["kw"])
    g = O.glue_kv(d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx, cfg)
    kall = np.concatenate([k16, g["k16"]]); vall = np.concatenate([v16, g["v16"]])
    ref = C.attention(g["q"], kall, vall, ctx, gate=g["gate"])
    with PooledAttn(cfg, ctx + 1, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        pa.run_glue_kv(0, d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx)
        dout = pa.alloc(pa.q_dim * 4)
        pa.attn("decode", 0, None, 0, pa.gate_buffer_ptr(), pa.q_dim, ctx, 1, dout, pa.q_dim)
        pa.sync()
        got = dout.download(np.float32, pa.q_dim).reshape(ref.shape)
        # 32768 streamed rows over 256 workgroup slots per kv head = whole 128-row splits; the token's own row is
        # the 257th partial
        pl = pa.plan("decode", ctx, 1)
        assert pl["n_splits"] * pl["split_len"] == ctx and pl["split_len"] % 32 == 0 and pl["slots"] == pl["n_splits"] + 1
    assert_parity(got, ref, "C3 gated decode 32K", tight=True)


@pytest.mark.parametrize("extra", [1, 2, 3, 32, 33, 34, 128, 2000, 5000])
def test_decode_past_the_single_round_capacity(extra):
    """Contexts a little past what the single-round kernel holds in one round (256 one-tile-per-wave splits a kv head
    at this shape): the tile loop with one workgroup a CU, its tiles dealt round robin to the waves of all splits, the
    last tile partial (poisoned rows past the context must stay unused)."""
    cfg = SHAPES["qwen36_moe"]
    L = 32768 + extra
    rng = np.random.default_rng(40 + extra)
    k16, v16 = random_cache(cfg, L + 40, seed=41)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    ref = C.attention(q, k16, v16, L - 1)
    with _ctx_with_cache(cfg, k16, v16, L + 40, poison_from=L) as pa:
        pl = pa.plan("decode", L - 1, 1)
        if extra == 1:
            assert pl["n_splits"] * pl["split_len"] == L - 1 and pl["split_len"] == 128      # whole splits + the token's own row
        else:
            assert pl["n_splits"] <= 128 and pl["split_len"] > 128 and pl["n_splits"] * pl["split_len"] >= L - 1, pl
        got = pa.run_attn("decode", 0, q, L - 1)
    assert_parity(got, ref, "open-ended last split, +%d rows" % extra)


def test_decode_one_column_at_128k():
    """A one-column decode over 131072 cached rows (MoE shape): the tile loop with one workgroup a CU, a kv head's 4096
    tiles dealt round robin to the 512 waves of its 128 splits, eight a wave; with a gate, f32 and f16 out."""
    cfg = SHAPES["qwen36_moe"]
    pos = 131072
    rng = np.random.default_rng(131)
    k16, v16 = random_cache(cfg, pos + 1, seed=132)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = C.attention(q, k16, v16, pos, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, pos + 1, max_cols=1) as pa:
        pl = pa.plan("decode", pos, 1)
        assert pl["n_splits"] == 128 and pl["split_len"] == 1024 and pl["slots"] == 129 and pl["row_blocks"] == 1, pl
        for out_dtype in (0, PA_OUT_F16):
            assert_parity(pa.run_attn("decode", 0, q, pos, gate=gate, out_dtype=out_dtype), ref, "decode at 128K", tight=True)


def test_c4_verify_64k():
    """Config 4: 8-token draft block over a 65536-token cache, Qwen3.8-27B attention shape, gate; equals 8
    sequential decodes (checked on columns 0 and 7) and the oracle."""
    cfg = SHAPES["qwen38_27b"]
    ctx, n = 65536, 8
    rng = np.random.default_rng(0x5EED0004)
    k16, v16 = random_cache(cfg, ctx + n, seed=0x5EED0004)
    q = O.rope_neox(O.head_rmsnorm(rng.standard_normal((n, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32),
                                   np.ones(cfg["head_dim"], np.float32), cfg["eps"]), ctx + np.arange(n), cfg["n_rot"], cfg["rope_theta"])
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = C.attention(q, k16, v16, ctx, gate=gate)
    with _ctx_with_cache(cfg, k16, v16, ctx + n, max_cols=n) as pa:
        multi = pa.run_attn("decode", 0, q, ctx, gate=gate)
        assert_parity(multi, ref, "C4 verify block 64K", tight=True)
        for c in (0, 7):
            single = pa.run_attn("decode", 0, q[c:c + 1], ctx + c, gate=gate[c:c + 1])
            assert_parity(single, ref[c:c + 1], "C4 decode col %d" % c)
            assert np.abs(single[0] - multi[c]).max() <= 1e-3


@pytest.mark.parametrize("shape,n_cols,base,blocks", [("qwen36_moe", 1, 40000, 1), ("qwen36_moe", 4, 40000, 2),
                                                       ("qwen38_27b", 8, 50000, 3)])
def test_decode_growing_maximum(shape, n_cols, base, blocks):
    """Scores that jump along the context: K rows alternate between a scale of 0.1 and a scale of 4 every eighth of the
    context, so every wave of the tile loop (its tiles are spread over the whole context, three or more a wave) meets low
    tiles first and then row maxima far beyond the threshold of its lazily updated reference maximum, and has to take the
    rescale path -- with one, two and three row blocks per workgroup."""
    cfg = SHAPES[shape]
    rng = np.random.default_rng(base + n_cols)
    rows = base + n_cols
    shp = (rows, cfg["n_kv_heads"], cfg["head_dim"])
    scale = np.where((np.arange(rows) // (rows // 8)) % 2 == 0, 0.1, 4.0).astype(np.float32)[:, None, None]
    k16 = (rng.standard_normal(shp, dtype=np.float32) * scale).astype(np.float16).view(np.uint16)
    v16 = rng.standard_normal(shp, dtype=np.float32).astype(np.float16).view(np.uint16)
    q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    ref = C.attention(q, k16, v16, base)
    with _ctx_with_cache(cfg, k16, v16, rows, max_cols=n_cols) as pa:
        plan = pa.plan("decode", base, n_cols)
        assert plan["row_blocks"] == blocks and plan["split_len"] >= 3 * 128, plan     # the tile loop, three tiles a wave or more
        assert_parity(pa.run_attn("decode", 0, q, base), ref, "jumping maximum, %d row blocks" % blocks)
