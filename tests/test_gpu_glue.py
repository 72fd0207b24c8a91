"""GPU parity of the pre-step (q de-interleave + QK-RMSNorm + RoPE + f16 KV write) through the C ABI.
Integer / index work is bit-exact: the written cache rows, the rows left untouched, and the q / gate
buffers all equal the oracle's bits."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from pooled_amd.capi import PooledAttn, PaError, PA_ERR_INVALID
from helpers import SHAPES

pytestmark = pytest.mark.gpu


def _run(cfg, base_pos, n_cols, max_seq, seed, pad=0):
    d = O.make_inputs(cfg, 0, n_cols, seed)
    ref = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base_pos, cfg)
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    with PooledAttn(cfg, max_seq, n_layers=2, max_cols=max(n_cols, 1)) as pa:
        pa.layer_alloc(1)
        # pre-fill the cache with a pattern so untouched rows are detectable
        pat = (np.arange(max_seq * nKV * hd, dtype=np.uint32) * 2654435761 >> 7).astype(np.uint16).reshape(max_seq, nKV * hd)
        pa.kv_write(1, 0, 0, pat); pa.kv_write(1, 1, 0, pat ^ 0x5555)
        pad_cols = lambda a: np.concatenate([a, np.full((a.shape[0], pad), np.nan, np.float32)], axis=1) if pad else a
        pa.run_glue_kv(1, pad_cols(d["qraw"]), pad_cols(d["kraw"]), pad_cols(d["vraw"]), d["qw"], d["kw"], base_pos)
        q = pa.read_q_buffer(n_cols)
        K = pa.kv_read(1, 0, 0, max_seq); V = pa.kv_read(1, 1, 0, max_seq)
        gate = pa.read_gate_buffer(n_cols) if cfg.get("gate") else None
    assert np.array_equal(q.view(np.uint32), ref["q"].view(np.uint32)), "roped q differs from the oracle's bits"
    if gate is not None:
        assert np.array_equal(gate.view(np.uint32), ref["gate"].view(np.uint32))
    rows = slice(base_pos, base_pos + n_cols)
    assert np.array_equal(K[rows], ref["k16"]) and np.array_equal(V[rows], ref["v16"]), "cache rows differ"
    mask = np.ones(max_seq, bool); mask[rows] = False
    assert np.array_equal(K[mask].reshape(-1, nKV * hd), pat[mask]), "K rows outside [base_pos, base_pos + n_cols) were written"
    assert np.array_equal(V[mask].reshape(-1, nKV * hd), (pat ^ 0x5555)[mask]), "V rows outside the pass were written"


@pytest.mark.parametrize("shape,base_pos,n_cols,pad", [
    ("qwen3_1p7b", 0, 1, 0), ("qwen3_1p7b", 2048, 1, 0), ("qwen3_1p7b", 1536, 16, 64),
    ("qwen36_moe", 0, 1, 0), ("qwen36_moe", 32768, 1, 0), ("qwen36_moe", 131055, 16, 64),
    ("qwen38_27b", 65536, 8, 0), ("qwen38_27b", 7, 5, 64),
])
def test_glue_kv_bit_exact(shape, base_pos, n_cols, pad):
    _run(SHAPES[shape], base_pos, n_cols, base_pos + n_cols + 3, seed=base_pos + n_cols, pad=pad)


def test_glue_kv_no_norm_full_rope():
    cfg = dict(SHAPES["qwen3_1p7b"], qk_norm=False)
    _run(cfg, 77, 4, 90, seed=3)


def test_glue_then_kv_store_equals_fused():
    """pa_glue (k written back in place) + pa_kv_store == pa_glue_kv, as attn_glue + kv_store == attn_glue_kv."""
    cfg = SHAPES["qwen36_moe"]
    n, base = 6, 100
    d = O.make_inputs(cfg, 0, n, 11)
    ref = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base, cfg)
    with PooledAttn(cfg, 128, n_layers=1, max_cols=8) as pa:
        pa.layer_alloc(0)
        dq, dk, dv = pa.to_device(d["qraw"]), pa.to_device(d["kraw"]), pa.to_device(d["vraw"])
        dqw, dkw = pa.to_device(d["qw"]), pa.to_device(d["kw"])
        pa.glue(dq, d["qraw"].shape[1], dk, d["kraw"].shape[1], dqw, dkw, base, n)
        pa.kv_store(0, dk, d["kraw"].shape[1], dv, d["vraw"].shape[1], base, n)
        pa.sync()
        assert np.array_equal(pa.kv_read(0, 0, base, n), ref["k16"]) and np.array_equal(pa.kv_read(0, 1, base, n), ref["v16"])
        assert np.array_equal(pa.read_q_buffer(n).view(np.uint32), ref["q"].view(np.uint32))


def test_argument_errors():
    cfg = SHAPES["qwen36_moe"]
    with pytest.raises(PaError) as e:
        PooledAttn(dict(cfg, head_dim=96), 64)
    assert e.value.code == 2
    with PooledAttn(cfg, 64, n_layers=1, max_cols=4) as pa:
        d = O.make_inputs(cfg, 0, 4, 1)
        with pytest.raises(PaError) as e:          # no cache yet
            pa.run_glue_kv(0, d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], 0)
        assert e.value.code == PA_ERR_INVALID and "pa_layer_alloc" in str(e.value)
        pa.layer_alloc(0)
        with pytest.raises(PaError):               # past max_seq
            pa.run_glue_kv(0, d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], 62)
        with pytest.raises(PaError):               # more columns than max_cols
            d8 = O.make_inputs(cfg, 0, 8, 1)
            pa.run_glue_kv(0, d8["qraw"], d8["kraw"], d8["vraw"], d8["qw"], d8["kw"], 0)
