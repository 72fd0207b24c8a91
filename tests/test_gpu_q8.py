"""GPU tests of the int8 KV mode (the reference's kvQ8: kv_store_q8 / attn_flash_q8, engine/wgsl/qwen35.js:908-946,
:99-139) through the C ABI.  The cache write is integer work: int8 values and scale bits equal the oracle's.
Attention over an int8 cache is compared with the oracle's attention over the de-quantised values (value * scale):
max-abs <= 2e-3 and max|d|/max|ref| <= 1e-2."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from pooled_amd.capi import PooledAttn, PaError, PA_ERR_UNSUPPORTED, PA_OUT_F16
from helpers import SHAPES, assert_parity

pytestmark = pytest.mark.gpu


def _q8cfg(shape):
    return dict(SHAPES[shape], kv_q8=True)


def _quantised_cache(cfg, rows, seed):
    """Random K / V rows, quantised by the oracle: (kq, ks, vq, vs, kf, vf) with kf / vf the de-quantised values."""
    rng = np.random.default_rng(seed)
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    k = (rng.standard_normal((rows, nKV, hd)) * 0.6).astype(np.float32); v = rng.standard_normal((rows, nKV, hd)).astype(np.float32)
    kq, ks = O.q8_quantize(k); vq, vs = O.q8_quantize(v)
    return kq, ks, vq, vs, O.q8_dequantize(kq, ks), O.q8_dequantize(vq, vs)


@pytest.mark.parametrize("shape,base_pos,n_cols", [("qwen36_moe", 0, 1), ("qwen36_moe", 777, 16), ("qwen3_1p7b", 2048, 5), ("qwen38_27b", 65000, 3)])
def test_q8_store_is_bit_exact(shape, base_pos, n_cols):
    cfg = _q8cfg(shape)
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    max_seq = base_pos + n_cols + 3
    d = O.make_inputs(cfg, 0, n_cols, seed=base_pos + n_cols)
    d["kraw"][0, :32] = 0.0; d["vraw"][0, 32:64] = 0.0                     # an all-zero block on each side
    g = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base_pos, dict(cfg))
    kf = g["k16"]                                                           # the oracle's roped K as f16 bits is not what is quantised:
    # the kernel quantises the f32 roped K, so restate that: rope / norm in f32, then q8
    nH = cfg["n_heads"]
    k = np.asarray(d["kraw"], np.float32).reshape(n_cols, nKV, hd)
    if cfg.get("qk_norm", True):
        k = O.head_rmsnorm(k, d["kw"], cfg["eps"])
    k = O.rope_neox(k, base_pos + np.arange(n_cols), cfg["n_rot"], cfg["rope_theta"])
    kq, ks = O.q8_quantize(k); vq, vs = O.q8_quantize(d["vraw"].reshape(n_cols, nKV, hd))
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=max(n_cols, 1)) as pa:
        pa.layer_alloc(0)
        pa.run_glue_kv(0, d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base_pos)
        K = pa.kv_read(0, 0, 0, max_seq); V = pa.kv_read(0, 1, 0, max_seq); KS = pa.kv_read(0, 2, 0, max_seq); VS = pa.kv_read(0, 3, 0, max_seq)
    rows = slice(base_pos, base_pos + n_cols)
    assert np.array_equal(K[rows], kq) and np.array_equal(V[rows], vq), "int8 values differ from the oracle's"
    assert np.array_equal(KS[rows].view(np.uint32), ks.view(np.uint32)) and np.array_equal(VS[rows].view(np.uint32), vs.view(np.uint32)), "scale bits differ"
    mask = np.ones(max_seq, bool); mask[rows] = False
    assert not K[mask].any() and not V[mask].any() and not KS[mask].any() and not VS[mask].any(), "rows outside the pass were written"


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_q8_decode_lengths(shape):
    cfg = _q8cfg(shape)
    rng = np.random.default_rng(3)
    max_seq = 4200
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, max_seq, seed=4)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=16) as pa:
        pa.layer_alloc(0)
        for L in (1, 2, 31, 32, 33, 127, 128, 129, 1000, 4097):
            # rows at or past L: garbage values with scales that are not numbers -- must never be used
            live = np.arange(max_seq)[:, None, None] < L
            pa.kv_write(0, 0, 0, np.where(live, kq, 77).astype(np.int8)); pa.kv_write(0, 1, 0, np.where(live, vq, -99).astype(np.int8))
            pa.kv_write(0, 2, 0, np.where(live, ks, np.nan).astype(np.float32)); pa.kv_write(0, 3, 0, np.where(live, vs, np.nan).astype(np.float32))
            got = pa.run_attn("decode", 0, q, L - 1, gate=gate)
            assert_parity(got, O.attention_values(q, kf, vf, L - 1, gate=gate), "%s q8 seqLen %d" % (shape, L))


def test_q8_verify_block_prefill_chunk_and_slots():
    cfg = _q8cfg("qwen36_moe")
    rng = np.random.default_rng(9)
    base, n = 3000, 40
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, base + n, seed=10)
    q = rng.standard_normal((n, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = O.attention_values(q, kf, vf, base, gate=gate)
    with PooledAttn(cfg, base + n, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        for w, a in enumerate((kq, vq, ks, vs)):
            pa.kv_write(0, w, 0, a)
        pl = pa.plan("decode", base, 8)      # two column groups of 32 stacked rows: the single-round kernel with two row blocks
        assert pl["row_blocks"] == 2 and pl["split_len"] == 128 and pl["n_splits"] == -(-(base + 8) // 128) and pl["col_groups"] == 2, pl
        assert_parity(pa.run_attn("decode", 0, q[:8], base, gate=gate[:8]), ref[:8], "q8 verify block")
        pa.set_decode_splits(4)              # the same block on the tile loop
        assert pa.plan("decode", base, 8)["split_len"] > 128
        assert_parity(pa.run_attn("decode", 0, q[:8], base, gate=gate[:8]), ref[:8], "q8 verify block, tile loop")
        pa.set_decode_splits(0)
        # a narrow chunk runs on the split-K kernel, a wide one on the MFMA prefill kernel over rows widened to f16 (forced:
        # the table would serve a chunk this small on the split-K kernel too)
        pa.set_prefill_tile(1)
        assert pa.plan("prefill", base, 4)["kernel"] == 0 and pa.plan("prefill", base, n)["kernel"] == 1
        assert_parity(pa.run_attn("prefill", 0, q[:4], base, gate=gate[:4]), ref[:4], "q8 narrow prefill chunk")
        assert_parity(pa.run_attn("prefill", 0, q, base, gate=gate, out_dtype=PA_OUT_F16).astype(np.float32), ref, "q8 prefill chunk")
        # slots carry the four tensors
        pa.slot_save(1, base + n)
        for w in range(4):
            pa.kv_write(0, w, 0, np.zeros_like((kq, vq, ks, vs)[w]))
        assert pa.slot_load(1) == base + n
        for w, a in enumerate((kq, vq, ks, vs)):
            assert np.array_equal(pa.kv_read(0, w, 0, base + n), a)
            assert np.array_equal(pa.slot_export(1, 0, w).reshape(a.shape), a)
        # the gather mode is an f16-cache path
        with pytest.raises(PaError) as e:
            pa.run_attn_gather(0, q[:1], [np.arange(10)])
        assert e.value.code == PA_ERR_UNSUPPORTED


@pytest.mark.parametrize("shape,pos", [("qwen36_moe", 0), ("qwen36_moe", 1), ("qwen36_moe", 777), ("qwen36_moe", 4096), ("qwen3_1p7b", 300), ("qwen38_27b", 129),
                                       ("qwen3_1p7b", 9001), ("qwen38_27b", 17000)])
def test_q8_fused_decode_step(shape, pos):
    """pa_attn_decode_step on int8 caches: the row it writes (values and scales) and its output equal pa_glue_kv +
    pa_attn_decode bit for bit, neighbouring rows stay untouched, and the output matches the oracle over the
    dequantised cache."""
    cfg = _q8cfg(shape)
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    d = O.make_inputs(cfg, pos, 1, seed=pos + 3)
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, pos + 2, seed=pos + 4)
    with PooledAttn(cfg, pos + 2, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        if pos > 8192:          # past what the single-round kernel holds at these shapes: the tile loop, three tiles a wave or more
            assert pa.plan("decode", pos, 1)["split_len"] >= 3 * 128
        for w, a in enumerate((kq, vq, ks, vs)):
            pa.kv_write(0, w, 0, a)
        pa.run_glue_kv(0, d["qraw"], d["kraw"][pos:], d["vraw"][pos:], d["qw"], d["kw"], pos)
        rows = [pa.kv_read(0, w, pos, 1).copy() for w in range(4)]
        dout = pa.alloc(pa.q_dim * 4)
        pa.attn("decode", 0, None, 0, pa.gate_buffer_ptr() if cfg["gate"] else None, pa.q_dim, pos, 1, dout, pa.q_dim); pa.sync()
        unfused = dout.download(np.float32, pa.q_dim)
        for w, a in enumerate((kq, vq, ks, vs)):                         # the cache as it was, row pos included
            pa.kv_write(0, w, 0, a)
        fused = pa.run_decode_step(0, d["qraw"][0], d["kraw"][pos], d["vraw"][pos], d["qw"], d["kw"], pos)
        for w in range(4):
            assert np.array_equal(pa.kv_read(0, w, pos, 1), rows[w]), "tensor %d of the written row" % w
            assert np.array_equal(pa.kv_read(0, w, pos + 1, 1), (kq, vq, ks, vs)[w][pos + 1:pos + 2]), "row after the written one"
            if pos:
                assert np.array_equal(pa.kv_read(0, w, pos - 1, 1), (kq, vq, ks, vs)[w][pos - 1:pos]), "row before the written one"
    assert np.array_equal(fused.reshape(-1).view(np.uint32), unfused.view(np.uint32))
    # oracle: attention over the dequantised rows, the new row dequantised from what the pre-step wrote
    g = O.glue_kv(d["qraw"], d["kraw"][pos:], d["vraw"][pos:], d["qw"], d["kw"], pos, cfg)
    knew = O.q8_dequantize(rows[0].reshape(1, nKV, hd), rows[2].reshape(1, nKV, hd // 32)); vnew = O.q8_dequantize(rows[1].reshape(1, nKV, hd), rows[3].reshape(1, nKV, hd // 32))
    ref = O.attention_values(g["q"], np.concatenate([kf[:pos], knew]), np.concatenate([vf[:pos], vnew]), pos, gate=g["gate"] if cfg["gate"] else None)
    assert_parity(fused.reshape(ref.shape), ref, "q8 fused step %s pos %d" % (shape, pos))


@pytest.mark.parametrize("shape,base,n", [("qwen36_moe", 0, 33), ("qwen36_moe", 1, 100), ("qwen36_moe", 2017, 300), ("qwen3_1p7b", 500, 257), ("qwen38_27b", 95, 64)])
def test_q8_prefill_on_the_matrix_cores(shape, base, n):
    """Wide chunks on int8 caches: rows [0, base + n) widened into the context's f16 staging cache, then the f16
    prefill kernel.  Rows past the chunk hold NaN scales (they must not leak); a second, shorter chunk on the same
    context is not disturbed by the rows the first one staged."""
    cfg = _q8cfg(shape)
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rng = np.random.default_rng(base * 7 + n)
    L = base + n
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, L, seed=base + n)
    q = rng.standard_normal((n, nH, hd), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg.get("gate") else None
    with PooledAttn(cfg, L + 64, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        for w, a in enumerate((kq, vq, ks, vs)):
            pa.kv_write(0, w, 0, a)
        bad = np.full((64, nKV, hd // 32), np.nan, np.float32)
        pa.kv_write(0, 2, L, bad); pa.kv_write(0, 3, L, bad)
        pa.set_prefill_tile(1)                       # the matrix-core kernel, whatever the table would pick for the size
        assert pa.plan("prefill", base, n)["kernel"] == 1
        ref = O.attention_values(q, kf, vf, base, gate=gate)
        assert_parity(pa.run_attn("prefill", 0, q, base, gate=gate), ref, "q8 wide prefill %s base %d n %d" % (shape, base, n))
        m = n // 2
        if pa.plan("prefill", base, m)["kernel"] == 1:
            got = pa.run_attn("prefill", 0, q[:m], base, gate=None if gate is None else gate[:m])
            assert_parity(got, ref[:m], "q8 wide prefill, shorter chunk after a longer one")


@pytest.mark.parametrize("base,n,rows", [(0, 256, 16), (0, 512, 32), (77, 129, 16)])
def test_q8_small_chunk_in_one_launch_writes_the_output_itself(base, n, rows):
    """The table's one-launch path for small chunks (one split per workgroup, the tile loop's epilogue normalises, gates,
    converts and stores; no partials, no merge) on an int8 cache: MoE shape, f32 and f16 output, and everything past
    the chunk -- values and scales -- poisoned (garbage under NaN scales), so a row past a column's end that reached
    the output would show."""
    cfg = _q8cfg("qwen36_moe")
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    G = cfg["n_heads"] // nKV
    rng = np.random.default_rng(100 + base + n)
    total, tail = base + n, 40
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, total, seed=200 + n)
    q = rng.standard_normal((n, cfg["n_heads"], hd), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = O.attention_values(q, kf, vf, base, gate=gate)
    with PooledAttn(cfg, total + tail, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        for w, a in enumerate((kq, vq, ks, vs)):
            pa.kv_write(0, w, 0, a)
        pa.kv_write(0, 0, total, np.full((tail, nKV, hd), 77, np.int8)); pa.kv_write(0, 1, total, np.full((tail, nKV, hd), -99, np.int8))
        pa.kv_write(0, 2, total, np.full((tail, nKV, hd // 32), np.nan, np.float32)); pa.kv_write(0, 3, total, np.full((tail, nKV, hd // 32), np.nan, np.float32))
        plan = pa.plan("prefill", base, n)
        assert plan["kernel"] == 0 and plan["n_splits"] == 1 and plan["slots"] == 1 and plan["cols_per_group"] * G == rows, plan
        for out_dtype in (0, PA_OUT_F16):
            got = pa.run_attn("prefill", 0, q, base, gate=gate, out_dtype=out_dtype).astype(np.float32)
            assert_parity(got, ref, "q8 small chunk base %d n %d out %d" % (base, n, out_dtype))


def test_q8_short_verify_block_is_one_split_with_two_row_blocks():
    """A verify block over a few tiles on an int8 cache: one split, two row blocks (4 columns x 8 heads), output written
    by the split-K kernel's own epilogue."""
    cfg = _q8cfg("qwen36_moe")
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    rng = np.random.default_rng(31)
    base, n, tail = 100, 4, 40
    kq, ks, vq, vs, kf, vf = _quantised_cache(cfg, base + n, seed=32)
    q = rng.standard_normal((n, cfg["n_heads"], hd), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    ref = O.attention_values(q, kf, vf, base, gate=gate)
    with PooledAttn(cfg, base + n + tail, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        for w, a in enumerate((kq, vq, ks, vs)):
            pa.kv_write(0, w, 0, a)
        pa.kv_write(0, 2, base + n, np.full((tail, nKV, hd // 32), np.nan, np.float32)); pa.kv_write(0, 3, base + n, np.full((tail, nKV, hd // 32), np.nan, np.float32))
        plan = pa.plan("decode", base, n)
        assert plan["kernel"] == 0 and plan["n_splits"] == 1 and plan["row_blocks"] == 2 and plan["slots"] == 1, plan
        for out_dtype in (0, PA_OUT_F16):
            got = pa.run_attn("decode", 0, q, base, gate=gate, out_dtype=out_dtype).astype(np.float32)
            assert_parity(got, ref, "q8 short verify block out %d" % out_dtype)
