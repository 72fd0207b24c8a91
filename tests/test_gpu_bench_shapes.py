"""GPU parity of the entry points the benchmark times, at the sizes it times them, through the C ABI.

* pa_attn_decode_step (pre-step fused into the single-round split-K kernel, interleaved rows, own-row partial) at
  configuration 3's position 32768 and a little past it (remainder splits dispatched last), f16 and int8 caches:
  written cache row = oracle bits, output = oracle within max-abs 2e-3 / relative 1e-2 and = pa_glue_kv followed by
  pa_attn_decode bit for bit (the reference states this for its own pair: engine/wgsl/attn_dec.js:12-16,
  tests/test_attn_dec.js:89-107).
* configurations 4 and 5 end to end: cache prefix from the oracle's pre-step, the block's / chunk's own pre-step and
  cache write on the GPU (bit-exact), then attention; configuration 5 is checked on one column of every one of its
  128 column blocks (tests/unit/attn_tile_test.js:43-50 checks every column of its small cases)."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PA_OUT_F16
from helpers import SHAPES, assert_parity, oracle_cache

pytestmark = pytest.mark.gpu

C3_POS = 32768
EXTRAS = [0, 1, 33, 128, 2000, 5000]
NAN16 = np.uint16(0x7E00)


@pytest.fixture(scope="module")
def c3_rows():
    """Raw tensors and oracle pre-step cache rows of the MoE shape for positions 0 .. 32768 + 5000."""
    cfg = SHAPES["qwen36_moe"]
    total = C3_POS + max(EXTRAS) + 1
    d = O.make_inputs(cfg, total, 0, seed=0x5EED0003)
    k16, v16 = oracle_cache(cfg, d["kraw"], d["vraw"], d["kw"])
    return d, k16, v16


def _token(cfg, pos):
    """The raw q (| gate) of the token at pos (its k / v are rows pos of the shared raw tensors)."""
    return np.random.default_rng(77000 + pos).standard_normal((1, cfg["n_heads"] * cfg["head_dim"] * 2), dtype=np.float32)


def test_decode_step_f16_at_c3_and_past_the_workgroup_slots(c3_rows):
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    d, k16, v16 = c3_rows
    max_seq = k16.shape[0] + 3
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        for extra in EXTRAS:
            pos = C3_POS + extra
            pl = pa.plan("decode", pos, 1)
            assert pl["slots"] == pl["n_splits"] + 1, pl
            if extra == 0:
                assert pl["n_splits"] == 256 and pl["split_len"] == 128      # the single-round kernel, every slot taken
            else:
                # one row past what two workgroups a CU hold in one round: the tile loop, one workgroup a CU
                assert pl["n_splits"] <= 128 and pl["split_len"] > 128 and pl["n_splits"] * pl["split_len"] >= pos, pl
            qraw = _token(cfg, pos)
            kraw, vraw = d["kraw"][pos:pos + 1], d["vraw"][pos:pos + 1]
            g = O.glue_kv(qraw, kraw, vraw, d["qw"], d["kw"], pos, cfg)
            assert np.array_equal(g["k16"][0], k16[pos]) and np.array_equal(g["v16"][0], v16[pos])
            ref = C.attention(g["q"], k16, v16, pos, gate=g["gate"])
            # rows from pos on are NaN before the call: the call must write row pos and never use the rows after it
            tail = np.full((max_seq - pos, nKV, hd), NAN16, np.uint16)
            pa.kv_write(0, 0, pos, tail); pa.kv_write(0, 1, pos, tail)
            fused = pa.run_decode_step(0, qraw[0], kraw[0], vraw[0], d["qw"], d["kw"], pos)
            for which, a in ((0, k16), (1, v16)):
                got = pa.kv_read(0, which, pos - 1, 3)
                assert np.array_equal(got[0], a[pos - 1]) and np.array_equal(got[1], a[pos]) and np.all(got[2] == NAN16), \
                    "cache rows around position %d (tensor %d)" % (pos, which)
            assert_parity(fused[None], ref, "C3 fused step at %d" % pos, tight=True)
            # the three-launch sequence on the same cache state
            pa.kv_write(0, 0, pos, tail); pa.kv_write(0, 1, pos, tail)
            pa.run_glue_kv(0, qraw, kraw, vraw, d["qw"], d["kw"], pos)
            unf = pa.run_attn("decode", 0, pa.read_q_buffer(1), pos, gate=pa.read_gate_buffer(1))
            assert np.array_equal(fused.view(np.uint32), unf[0].view(np.uint32)), "fused != pa_glue_kv + pa_attn_decode at %d" % pos
            pa.kv_write(0, 0, pos, k16[pos:]); pa.kv_write(0, 1, pos, v16[pos:])     # the real rows back for the next position


def test_decode_step_int8_at_c3_and_past_the_workgroup_slots(c3_rows):
    cfg = dict(SHAPES["qwen36_moe"], kv_q8=True)
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    d, _, _ = c3_rows
    total = C3_POS + max(EXTRAS) + 1
    # the f32 normed + roped K rows and raw V rows, quantised by the oracle's quantiser
    k = O.rope_neox(O.head_rmsnorm(d["kraw"].reshape(total, nKV, hd), d["kw"], cfg["eps"]), np.arange(total), cfg["n_rot"], cfg["rope_theta"])
    kq, ks = O.q8_quantize(k); vq, vs = O.q8_quantize(d["vraw"].reshape(total, nKV, hd))
    kf, vf = O.q8_dequantize(kq, ks), O.q8_dequantize(vq, vs)
    parts = (kq, vq, ks, vs)
    max_seq = total + 3
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        for w, a in enumerate(parts):
            pa.kv_write(0, w, 0, a)
        for extra in EXTRAS:
            pos = C3_POS + extra
            qraw = _token(cfg, pos)
            kraw, vraw = d["kraw"][pos:pos + 1], d["vraw"][pos:pos + 1]
            g = O.glue_kv(qraw, kraw, vraw, d["qw"], d["kw"], pos, cfg)
            ref = O.attention_values(g["q"], kf, vf, pos, gate=g["gate"])
            # rows from pos on: garbage values under scales that are not numbers
            n_tail = max_seq - pos
            junk = (np.full((n_tail, nKV, hd), 77, np.int8), np.full((n_tail, nKV, hd), -99, np.int8),
                    np.full((n_tail, nKV, hd // 32), np.nan, np.float32), np.full((n_tail, nKV, hd // 32), np.nan, np.float32))
            for w in range(4):
                pa.kv_write(0, w, pos, junk[w])
            fused = pa.run_decode_step(0, qraw[0], kraw[0], vraw[0], d["qw"], d["kw"], pos)
            for w, a in enumerate(parts):
                got = pa.kv_read(0, w, pos - 1, 3)
                same = lambda x, y: np.array_equal(x.view(np.uint32), y.view(np.uint32)) if x.dtype == np.float32 else np.array_equal(x, y)
                assert same(got[0], a[pos - 1]) and same(got[1], a[pos]), "int8 cache rows around position %d (tensor %d)" % (pos, w)
                assert same(got[2], junk[w][0]), "row after position %d was written (tensor %d)" % (pos, w)
            assert_parity(fused[None], ref, "int8 fused step at %d" % pos)
            for w in range(4):
                pa.kv_write(0, w, pos, junk[w])
            pa.run_glue_kv(0, qraw, kraw, vraw, d["qw"], d["kw"], pos)
            unf = pa.run_attn("decode", 0, pa.read_q_buffer(1), pos, gate=pa.read_gate_buffer(1))
            assert np.array_equal(fused.view(np.uint32), unf[0].view(np.uint32)), "int8: fused != three launches at %d" % pos
            for w, a in enumerate(parts):
                pa.kv_write(0, w, pos, a[pos:])


def test_c4_verify_64k_end_to_end():
    """Configuration 4 with the pre-step in the loop: 65536 cache rows from the oracle's pre-step, the 8-token block's
    QK-RMSNorm + partial RoPE + cache write by pa_glue_kv (bit-exact), then the verify pass on the context's own q and
    gate buffers."""
    cfg = SHAPES["qwen38_27b"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    ctx, n = 65536, 8
    d = O.make_inputs(cfg, ctx, n, seed=0x5EED0004)
    k16, v16 = oracle_cache(cfg, d["kraw"], d["vraw"], d["kw"])
    g = O.glue_kv(d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx, cfg)
    assert np.array_equal(g["k16"], k16[ctx:])
    ref = C.attention(g["q"], k16, v16, ctx, gate=g["gate"])
    with PooledAttn(cfg, ctx + n, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16[:ctx]); pa.kv_write(0, 1, 0, v16[:ctx])
        pa.run_glue_kv(0, d["qraw"], d["kraw"][ctx:], d["vraw"][ctx:], d["qw"], d["kw"], ctx)
        assert np.array_equal(pa.kv_read(0, 0, ctx, n), k16[ctx:]) and np.array_equal(pa.kv_read(0, 1, ctx, n), v16[ctx:])
        assert np.array_equal(pa.read_q_buffer(n).view(np.uint32), g["q"].view(np.uint32))
        dout = pa.alloc(n * pa.q_dim * 4)
        pa.attn("decode", 0, None, 0, pa.gate_buffer_ptr(), pa.q_dim, ctx, n, dout, pa.q_dim)
        pa.sync()
        got = dout.download(np.float32, n * pa.q_dim).reshape(ref.shape)
    assert_parity(got, ref, "C4 end to end", tight=True)


def test_c5_prefill_128k_end_to_end_every_column_block():
    """Configuration 5 with the pre-step in the loop: 126976 prefix rows from the oracle's pre-step, the 4096-token
    chunk's pre-step + cache write by pa_glue_kv (bit-exact), causal prefill with gate and f16 output.  A workgroup of
    the prefill kernel owns 32 consecutive columns of a kv head (256 stacked rows at 8 heads a kv head), so the chunk
    is 128 column blocks per kv head; one column of every block (all 16 heads, the offset inside the block walking
    through the block's 8 wavefronts) plus the first and the last column are checked against the f64 oracle."""
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    base, n = 126976, 4096
    d = O.make_inputs(cfg, base, n, seed=0x5EED0005)
    k16, v16 = oracle_cache(cfg, d["kraw"], d["vraw"], d["kw"])
    g = O.glue_kv(d["qraw"], d["kraw"][base:], d["vraw"][base:], d["qw"], d["kw"], base, cfg)
    cols = sorted(set([0, n - 1] + [b * 32 + (b * 13) % 32 for b in range(n // 32)]))
    assert len(set(c // 32 for c in cols)) == n // 32
    ref = C.attention(g["q"], k16, v16, base, gate=g["gate"], rows=cols)
    with PooledAttn(cfg, base + n, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16[:base]); pa.kv_write(0, 1, 0, v16[:base])
        pa.run_glue_kv(0, d["qraw"], d["kraw"][base:], d["vraw"][base:], d["qw"], d["kw"], base)
        assert np.array_equal(pa.kv_read(0, 0, base, n), k16[base:]) and np.array_equal(pa.kv_read(0, 1, base, n), v16[base:])
        plan = pa.plan("prefill", base, n)
        assert plan["kernel"] == 1 and plan["n_splits"] == 1 and plan["cols_per_group"] == 32 and plan["col_groups"] == n // 32, plan
        dout = pa.alloc(n * pa.q_dim * 2)
        pa.attn("prefill", 0, None, 0, pa.gate_buffer_ptr(), pa.q_dim, base, n, dout, pa.q_dim, PA_OUT_F16)
        pa.sync()
        got = dout.download(np.float16, n * pa.q_dim).reshape(n, nH, hd)[cols].astype(np.float32)
    assert np.all(np.isfinite(got))
    assert_parity(got, ref, "C5 end to end, every column block, f16 out", tight=True)
