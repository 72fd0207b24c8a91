"""The allocation-free entry point pa_attn_decode_step_noalloc through the C ABI: its partials live in the library's
file-scope device array instead of a buffer of the context.  It runs the same kernels as pa_attn_decode_step, so the
bar is bit equality of the output and of the written cache row with that entry point -- on two calls in a row, the
second on a shorter context (fewer splits, so part of the array still holds the first call's partials) -- plus the
oracle within max-abs 2e-3 / relative 1e-2.  A shape whose partials exceed the array is refused with a clear error.
This file is collected last: the tests before it must not depend on it, and it must pass alone and after them."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PaError, PA_ERR_UNSUPPORTED
from helpers import SHAPES, assert_parity, random_cache

pytestmark = pytest.mark.gpu


def _step(pa, cfg, d, pos, noalloc):
    bufs = [pa.to_device(np.ascontiguousarray(a, dtype=np.float32)) for a in (d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"])]
    dout = pa.to_device(np.full(pa.q_dim, np.nan, np.float32))
    pa.attn_decode_step(0, bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], pos, dout, noalloc=noalloc)
    pa.sync()
    out = dout.download(np.float32, pa.q_dim).reshape(cfg["n_heads"], cfg["head_dim"])
    row = (pa.kv_read(0, 0, pos, 1).copy(), pa.kv_read(0, 1, pos, 1).copy())
    for b in bufs + [dout]:
        b.free(); pa._bufs.remove(b)
    return out, row


@pytest.mark.parametrize("shape,positions", [("qwen36_moe", (33000, 700)), ("qwen3_1p7b", (2048, 130)), ("qwen38_27b", (5000, 4999))])
def test_noalloc_step_equals_the_allocating_entry_point(shape, positions):
    cfg = SHAPES[shape]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    max_seq = max(positions) + 4
    k16, v16 = random_cache(cfg, max_seq, seed=sum(positions))
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        for pos in positions:                      # the second call is the shorter one
            d = O.make_inputs(cfg, 0, 1, seed=pos + 11)
            g = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], pos, cfg)
            K = k16.copy(); V = v16.copy()
            K[pos] = g["k16"][0]; V[pos] = g["v16"][0]
            ref = C.attention(g["q"], K, V, pos, gate=g["gate"])
            outs = {}
            for noalloc in (True, False):
                pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
                outs[noalloc] = _step(pa, cfg, d, pos, noalloc)
            got, row = outs[True]
            assert np.array_equal(row[0][0], g["k16"][0]) and np.array_equal(row[1][0], g["v16"][0]), "cache row differs from the oracle's bits"
            assert np.array_equal(got.view(np.uint32), outs[False][0].view(np.uint32)), "%s pos %d: differs from pa_attn_decode_step" % (shape, pos)
            assert_parity(got[None], ref, "%s pos %d (no-alloc step)" % (shape, pos))


def test_noalloc_step_on_int8_caches_and_over_the_limit():
    cfg = dict(SHAPES["qwen36_moe"], kv_q8=True)
    rng = np.random.default_rng(3)
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    positions = (9000, 64)
    max_seq = max(positions) + 2
    kq, ks = O.q8_quantize((rng.standard_normal((max_seq, nKV, hd)) * 0.6).astype(np.float32))
    vq, vs = O.q8_quantize(rng.standard_normal((max_seq, nKV, hd)).astype(np.float32))
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        for pos in positions:
            d = O.make_inputs(cfg, 0, 1, seed=pos)
            outs = []
            for noalloc in (True, False):
                for w, a in enumerate((kq, vq, ks, vs)):
                    pa.kv_write(0, w, 0, a)
                outs.append(_step(pa, cfg, d, pos, noalloc)[0])
            assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), "int8 pos %d" % pos
            assert np.all(np.isfinite(outs[0]))
    # 16 query heads on one kv head at 65536 rows, the most the single-round kernel takes at this shape: 512 splits + the
    # own row = 513 slots x 16 heads x 258 floats = 8.47 MB of partials > the 8 MiB array
    big = dict(n_heads=16, n_kv_heads=1, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=False)
    with PooledAttn(big, 65540, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        assert pa.plan("decode", 65536, 1)["slots"] == 513
        d = O.make_inputs(big, 0, 1, seed=1)
        with pytest.raises(PaError) as e:
            _step(pa, big, d, 65536, True)
        assert e.value.code == PA_ERR_UNSUPPORTED and "static scratch" in str(e.value)
        out, _ = _step(pa, big, d, 65536, False)          # the allocating entry point serves the shape
        assert np.all(np.isfinite(out))
