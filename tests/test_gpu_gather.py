"""GPU parity of the gather mode of the split-K kernel (each column attends to its own list of cache rows: the
reference's attn_dec_qsa, engine/wgsl/attn_dec.js:33-38) through the C ABI.  Oracle: the pinned attention oracle
applied to the gathered rows (a list is an index into the cache; list position t takes the place of position t).
Tolerance: max-abs <= 2e-3 and max|d|/max|ref| <= 1e-2; with the identity list the output equals pa_attn_decode's bits."""
import numpy as np
import pytest
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PaError, PA_ERR_INVALID, PA_OUT_F16
from helpers import SHAPES, assert_parity, random_cache

pytestmark = pytest.mark.gpu
NAN16 = 0x7E00


def _oracle(q, k16, v16, lists, gate):
    outs = []
    for c, l in enumerate(lists):
        idx = np.asarray(l)
        outs.append(C.attention(q[c:c + 1], k16[idx], v16[idx], len(l) - 1, gate=None if gate is None else gate[c:c + 1])[0])
    return np.stack(outs)


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_gather_lists_of_many_lengths(shape):
    """List lengths around the tile and split boundaries up to the reference's 2051-row maximum (QSA_MAXSEL),
    different per column; rows outside the lists are NaN."""
    cfg = SHAPES[shape]
    rows_total = 9000
    rng = np.random.default_rng(17)
    k16, v16 = random_cache(cfg, rows_total, seed=18)
    lens = [1, 2, 31, 32, 33, 127, 129, 700, 2051]
    lists = [np.sort(rng.choice(rows_total, size=n, replace=False)) for n in lens]
    q = rng.standard_normal((len(lens), cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
    used = np.zeros(rows_total, bool)
    for l in lists:
        used[l] = True
    K = np.where(used[:, None, None], k16, NAN16).astype(np.uint16); V = np.where(used[:, None, None], v16, NAN16).astype(np.uint16)
    with PooledAttn(cfg, rows_total, n_layers=1, max_cols=16) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, K); pa.kv_write(0, 1, 0, V)
        got = pa.run_attn_gather(0, q, lists, gate=gate)
        one = pa.run_attn_gather(0, q[4:5], lists[4:5], gate=None if gate is None else gate[4:5])     # a pass of one column
    ref = _oracle(q, k16, v16, lists, gate)
    assert_parity(got, ref, "gather %s" % shape)
    assert_parity(one, ref[4:5], "gather single column %s" % shape)


@pytest.mark.parametrize("pos", [0, 40, 2050, 6000, 9000])
def test_identity_list_equals_dense_decode(pos):
    """With the list 0 .. pos the gathered kernel computes what the dense kernel computes
    (engine/wgsl/attn_dec.js:35-37).  Not bit for bit: a dense one-column decode folds the column's own row in as a
    partial of its own (f32 products), the gathered kernel streams every listed row through the f16 MFMA path.  (9000
    rows are 71 splits: both passes then write f16 partials.)"""
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(pos + 1)
    k16, v16 = random_cache(cfg, pos + 1, seed=pos + 2)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    with PooledAttn(cfg, pos + 1, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        dense = pa.run_attn("decode", 0, q, pos, gate=gate)
        gath = pa.run_attn_gather(0, q, [np.arange(pos + 1)], gate=gate)
    assert np.abs(dense - gath).max() < 2e-5


def test_gather_f16_out_and_bad_arguments():
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(5)
    k16, v16 = random_cache(cfg, 500, seed=6)
    q = rng.standard_normal((2, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    lists = [np.arange(0, 500, 3), np.arange(1, 500, 7)]
    with PooledAttn(cfg, 500, n_layers=1, max_cols=2) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        got = pa.run_attn_gather(0, q, lists, out_dtype=PA_OUT_F16)
        assert_parity(got.astype(np.float32), _oracle(q, k16, v16, lists, None), "gather f16 out")
        dq = pa.to_device(q.reshape(2, -1)); dsel = pa.to_device(np.zeros((2, 8), np.uint32)); dout = pa.alloc(2 * pa.q_dim * 4)
        with pytest.raises(PaError) as e:                                    # stride shorter than max_rows + 1
            pa._chk(pa.L.pa_attn_decode_gather(pa.ctx, 0, dq.ptr, pa.q_dim, None, 0, dsel.ptr, 8, 8, 2, dout.ptr, pa.q_dim, 0))
        assert e.value.code == PA_ERR_INVALID
        with pytest.raises(PaError):                                         # more rows than the cache holds
            pa._chk(pa.L.pa_attn_decode_gather(pa.ctx, 0, dq.ptr, pa.q_dim, None, 0, dsel.ptr, 1000, 501, 2, dout.ptr, pa.q_dim, 0))


def test_gather_does_not_trust_the_length_word():
    """The length word of a list lives in device memory the caller's selection kernel wrote: a length past max_rows is
    read as max_rows (the list cannot run into the next column's), a length of 0 gives a column of zeros, and the
    other columns of the pass are unaffected."""
    cfg = SHAPES["qwen36_moe"]
    rng = np.random.default_rng(23)
    rows_total, max_rows = 3000, 300
    k16, v16 = random_cache(cfg, rows_total, seed=24)
    lists = [np.sort(rng.choice(rows_total, size=max_rows, replace=False)) for _ in range(3)]
    q = rng.standard_normal((3, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    ref = _oracle(q, k16, v16, lists, None)
    stride = max_rows + 1
    sel = np.zeros((3, stride), np.uint32)
    for c, l in enumerate(lists):
        sel[c, 0] = len(l); sel[c, 1:] = l
    sel[0, 0] = 100000                      # far past max_rows and the stride: must read as max_rows
    sel[1, 0] = 0                           # an empty list
    with PooledAttn(cfg, rows_total, n_layers=1, max_cols=4) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        dq = pa.to_device(q.reshape(3, -1)); dsel = pa.to_device(sel)
        dout = pa.to_device(np.full((3, pa.q_dim), np.nan, np.float32))
        pa._chk(pa.L.pa_attn_decode_gather(pa.ctx, 0, dq.ptr, pa.q_dim, None, 0, dsel.ptr, stride, max_rows, 3, dout.ptr, pa.q_dim, 0))
        pa.sync()
        got = dout.download(np.float32, 3 * pa.q_dim).reshape(ref.shape)
    assert_parity(got[0:1], ref[0:1], "over-long length word")
    assert np.all(got[1] == 0.0), "empty list must give zeros"
    assert_parity(got[2:3], ref[2:3], "neighbour of the bad lists")
