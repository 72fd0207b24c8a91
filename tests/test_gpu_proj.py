"""GPU tests of the one-token projections either side of the attention block (pa_gemv, pa_gemv_norm,
pa_attn_layer_decode) through the C ABI, against the oracle's dequantise-and-multiply in f64.

The reference checks its GEMVs against a CPU product of the dequantised weights with a tolerance relative to the
output scale (engine/selftest.js:120-139: max-abs / scale < 2e-3; tests/test_gemm.js:13-14, :105: ~1e-6 for
summation order alone).  Here: 2e-5 of the largest output for a GEMV alone, the path's 2e-3 / 1e-2 gate for the layer.
"""
import numpy as np
import pytest
from oracle import attn_oracle as O
from pooled_amd.capi import PooledAttn, PaError, PA_W_F32, PA_W_Q8_0, PA_W_Q4_0, PA_ERR_INVALID, PA_ERR_UNSUPPORTED
from helpers import SHAPES, assert_parity, oracle_cache

pytestmark = pytest.mark.gpu


def _weights(kind, d_out, d_in, rng, scale=0.02):
    """Random weight planes of a kind: (w, scales-or-None)."""
    if kind == PA_W_F32:
        return (rng.standard_normal((d_out, d_in)) * scale).astype(np.float32), None
    sc = np.asarray(rng.uniform(0.5, 1.5, (d_out, d_in // 32)) * scale / (127 if kind == PA_W_Q8_0 else 8) * 3, np.float16).view(np.uint16)
    if kind == PA_W_Q8_0:
        return rng.integers(-127, 128, (d_out, d_in)).astype(np.int8), sc
    return rng.integers(0, 256, (d_out, d_in // 2)).astype(np.uint8), sc


def _rel(got, ref):
    return np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30)


@pytest.mark.parametrize("kind", [PA_W_F32, PA_W_Q8_0, PA_W_Q4_0])
@pytest.mark.parametrize("d_out,d_in", [(9216, 2048), (2048, 4096), (1, 32), (37, 96), (5000, 6144), (130, 8192)])
def test_gemv_matches_oracle(kind, d_out, d_in):
    rng = np.random.default_rng(d_out * 7 + d_in + kind)
    w, sc = _weights(kind, d_out, d_in, rng)
    x = rng.standard_normal(d_in).astype(np.float32)
    y0 = rng.standard_normal(d_out).astype(np.float32)
    ref = O.gemv(kind, w, sc, x)
    with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
        wh = pa.weight(kind, w, sc)
        dx = pa.to_device(x); dy = pa.to_device(y0)
        pa.gemv(wh, dx, dy); pa.sync()
        got = dy.download(np.float32, d_out)
        assert _rel(got, ref) < 2e-5, "plain"
        pa.gemv(wh, dx, dy, acc=True); pa.sync()                      # y = W x, then y += W x
        assert _rel(dy.download(np.float32, d_out), 2.0 * ref) < 2e-5, "accumulate"
        # deterministic run to run
        pa.gemv(wh, dx, dy); pa.sync()
        assert np.array_equal(dy.download(np.float32, d_out), got)


@pytest.mark.parametrize("kind", [PA_W_F32, PA_W_Q4_0])
def test_gemv_norm_matches_rmsnorm_then_gemv(kind):
    cfg = SHAPES["qwen36_moe"]
    d_out, d_in = 1024 + 3, 2048
    rng = np.random.default_rng(11 + kind)
    w, sc = _weights(kind, d_out, d_in, rng)
    x = (rng.standard_normal(d_in) * 3.0).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(d_in)).astype(np.float32)
    xn_ref = O.rmsnorm(x, nw, cfg["eps"])
    ref = O.gemv(kind, w, sc, xn_ref)
    with PooledAttn(cfg, 64, n_layers=1, max_cols=1) as pa:
        wh = pa.weight(kind, w, sc)
        dx = pa.to_device(x); dnw = pa.to_device(nw); dy = pa.alloc(d_out * 4); dxn = pa.alloc(d_in * 4)
        pa.gemv_norm(wh, dx, dnw, dy, dxn); pa.sync()
        assert _rel(dxn.download(np.float32, d_in), xn_ref.astype(np.float64)) < 1e-6
        assert _rel(dy.download(np.float32, d_out), ref) < 2e-5
        pa.gemv_norm(wh, dx, dnw, dy); pa.sync()                      # without the xn copy
        assert _rel(dy.download(np.float32, d_out), ref) < 2e-5


def test_weight_and_gemv_errors():
    with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
        with pytest.raises(PaError) as e:
            pa.weight(PA_W_Q8_0, np.zeros((4, 48), np.int8), np.zeros((4, 1), np.uint16))       # d_in not a multiple of 32
        assert e.value.code == PA_ERR_INVALID
        with pytest.raises(PaError) as e:
            pa.weight(PA_W_Q4_0, np.zeros((4, 8192), np.uint8), np.zeros((4, 512), np.uint16))  # d_in 16384
        assert e.value.code == PA_ERR_UNSUPPORTED
        with pytest.raises(PaError) as e:
            pa.weight(7, np.zeros((4, 32), np.float32))
        assert e.value.code == PA_ERR_INVALID


@pytest.mark.parametrize("shape,dim,kind,pos", [("qwen36_moe", 2048, PA_W_Q4_0, 777), ("qwen36_moe", 2048, PA_W_Q8_0, 0),
                                                 ("qwen3_1p7b", 2048, PA_W_Q4_0, 300), ("qwen38_27b", 5120, PA_W_Q8_0, 1029)])
def test_attn_layer_decode_matches_oracle(shape, dim, kind, pos):
    """rmsnorm -> [q | k | v] -> pre-step -> attention over the cache -> gate -> wo, accumulated into x: the residual
    and the new cache rows against the oracle's composition of the same stages."""
    cfg = SHAPES[shape]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = nH * hd, nKV * hd
    q_rows = qd * (2 if cfg["gate"] else 1)
    rng = np.random.default_rng(pos + dim)
    w_qkv, s_qkv = _weights(kind, q_rows + 2 * kvd, dim, rng, scale=0.03)
    w_o, s_o = _weights(kind, dim, qd, rng, scale=0.03)
    x = rng.standard_normal(dim).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32); kw = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    k16, v16 = oracle_cache(cfg, rng.standard_normal((pos, kvd)).astype(np.float32), rng.standard_normal((pos, kvd)).astype(np.float32), kw)
    x_ref, k_row, v_row = O.attn_layer_decode(x, kind, w_qkv, s_qkv, kind, w_o, s_o, nw, qw, kw, k16, v16, pos, cfg)
    with PooledAttn(cfg, pos + 8, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        if pos:
            pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        wq = pa.weight(kind, w_qkv, s_qkv); wo = pa.weight(kind, w_o, s_o)
        dx = pa.to_device(x); dnw = pa.to_device(nw); dqw = pa.to_device(qw); dkw = pa.to_device(kw)
        pa.attn_layer_decode(0, wq, wo, dnw, dqw, dkw, dx, pos); pa.sync()
        got = dx.download(np.float32, dim)
        kc = pa.kv_read(0, 0, pos, 1).view(np.float16).astype(np.float64); vc = pa.kv_read(0, 1, pos, 1).view(np.float16).astype(np.float64)
    assert_parity(got, x_ref, "layer %s pos %d" % (shape, pos))
    # the new cache rows: f16 of GEMV outputs that differ from the oracle's f64 products in the last f32 bits, so a
    # value next to a rounding boundary may land one f16 step away
    for a, b in ((kc, k_row), (vc, v_row)):
        ref = np.asarray(b).reshape(a.shape).view(np.float16).astype(np.float64)
        assert np.abs(a - ref).max() <= np.abs(ref).max() * 2.0 ** -10


# ---- column-batched passes: rmsnorm -> f16, GEMM on the matrix cores, the whole attention half of a layer ----

@pytest.mark.parametrize("kind", [PA_W_F32, PA_W_Q8_0, PA_W_Q4_0])
@pytest.mark.parametrize("d_out,d_in,n", [(9216, 2048, 300), (2048, 4096, 129), (37, 96, 5), (130, 8192, 40), (256, 32, 128), (384, 96, 700),
                                          (100, 384, 65), (64, 128, 33), (4096, 2048, 512),      # the 64 x 64 kernel with an odd stage count, one stage, a C2-sized chunk (as are the first two and the fourth)
                                          (9216, 2048, 8), (2048, 4096, 16), (130, 8192, 3), (70, 64, 1), (2048, 4096, 31), (130, 8192, 17)])   # from (9216, 2048, 8) on: up to 16 columns the skinny-chunk kernel, one or more launches; the last two the 64 x 32 tiles of the mid-size kernel
def test_gemm_matches_oracle(kind, d_out, d_in, n):
    rng = np.random.default_rng(d_out + 3 * d_in + n + kind)
    w, sc = _weights(kind, d_out, d_in, rng)
    x16 = rng.standard_normal((n, d_in)).astype(np.float16)
    ref = O.gemm_f16(kind, w, sc, x16.astype(np.float32))
    xs, ys = d_in + 8, d_out + 5                                      # padded strides
    xpad = np.zeros((n, xs), np.float16); xpad[:, :d_in] = x16
    y0 = rng.standard_normal((n, ys)).astype(np.float32)
    with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
        wh = pa.weight(kind, w, sc)
        dx = pa.to_device(xpad.view(np.uint16)); dy = pa.to_device(y0)
        pa.gemm(wh, dx, xs, n, dy, ys); pa.sync()
        got = dy.download(np.float32, n * ys).reshape(n, ys)
        assert _rel(got[:, :d_out], ref) < 2e-5, "plain"
        assert np.array_equal(got[:, d_out:], y0[:, d_out:]), "the stride padding of y must stay untouched"
        pa.gemm(wh, dx, xs, n, dy, ys, acc=True); pa.sync()
        assert _rel(dy.download(np.float32, n * ys).reshape(n, ys)[:, :d_out], 2.0 * ref) < 2e-5, "accumulate"


@pytest.mark.parametrize("kind", [PA_W_F32, PA_W_Q8_0, PA_W_Q4_0])
@pytest.mark.parametrize("d_out,d_in,n", [(9216 - 40, 2048, 4096 - 3), (2048, 4096, 4000), (4090, 256, 4096), (600, 128, 11000),
                                          (2048, 4096, 600), (130, 8192, 513), (1000, 64, 1100)])
def test_gemm_large_chunks(kind, d_out, d_in, n):
    """Chunks of 512 columns and more over d_in a multiple of 128: the weights are widened to f16 in fragment order (a
    copy kept with the weight handle) and the GEMM runs over two f16 operands (128-column wave tiles, 256 to 512 weight
    rows a workgroup: the first four shapes take 384, 256, 512 and 384 on a 256-CU part; the last three stay on the
    tiled kernel, too few workgroups or d_in not a multiple of 128).  Ragged edges on both axes, padded strides that
    must stay untouched, the accumulating form (the second call on a handle, which finds the kept copy), and a second
    weight."""
    rng = np.random.default_rng(d_out + d_in + n + kind)
    w, sc = _weights(kind, d_out, d_in, rng)
    x16 = rng.standard_normal((n, d_in)).astype(np.float16)
    ref = O.gemm_f16(kind, w, sc, x16.astype(np.float32))
    xs, ys = d_in + 8, d_out + 5
    xpad = np.zeros((n, xs), np.float16); xpad[:, :d_in] = x16
    y0 = rng.standard_normal((n, ys)).astype(np.float32)
    with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
        wh = pa.weight(kind, w, sc)
        dx = pa.to_device(xpad.view(np.uint16)); dy = pa.to_device(y0)
        pa.gemm(wh, dx, xs, n, dy, ys); pa.sync()
        got = dy.download(np.float32, n * ys).reshape(n, ys)
        assert _rel(got[:, :d_out], ref) < 2e-5, "plain"
        assert np.array_equal(got[:, d_out:], y0[:, d_out:]), "the stride padding of y must stay untouched"
        pa.gemm(wh, dx, xs, n, dy, ys, acc=True); pa.sync()
        assert _rel(dy.download(np.float32, n * ys).reshape(n, ys)[:, :d_out], 2.0 * ref) < 2e-5, "accumulate"
        w2, sc2 = _weights(kind, d_out, d_in, rng)
        pa.gemm(pa.weight(kind, w2, sc2), dx, xs, n, dy, ys); pa.sync()
        assert _rel(dy.download(np.float32, n * ys).reshape(n, ys)[:, :d_out], O.gemm_f16(kind, w2, sc2, x16.astype(np.float32))) < 2e-5, "second weight"


@pytest.mark.parametrize("kind", [PA_W_Q8_0, PA_W_Q4_0])
def test_gemm_weight_cache_budget(kind):
    """The kept f16 copy and the per-call staging hold the same values: a context with no budget (every call widens into
    the context's staging), one whose budget holds the first weight only, and the default give the same bits, also
    when the weights alternate through the one staging matrix."""
    d_out, d_in, n = 2100, 256, 4000
    rng = np.random.default_rng(kind)
    ws = [_weights(kind, d_out, d_in, rng) for _ in range(2)]
    x16 = rng.standard_normal((n, d_in)).astype(np.float16)
    outs = []
    for budget in (None, 0, 2112 * 256 * 2 + 64):
        with PooledAttn(SHAPES["qwen36_moe"], 64, n_layers=1, max_cols=1) as pa:
            if budget is not None:
                pa.set_weight_cache(budget)
            whs = [pa.weight(kind, w, sc) for w, sc in ws]
            dx = pa.to_device(x16.view(np.uint16)); dy = pa.alloc(n * d_out * 4)
            got = []
            for i in (0, 1, 0, 1):
                pa.gemm(whs[i], dx, d_in, n, dy, d_out); pa.sync()
                got.append(dy.download(np.float32, n * d_out))
            assert np.array_equal(got[0], got[2]) and np.array_equal(got[1], got[3])
            outs.append(got[:2])
    for o in outs[1:]:
        assert np.array_equal(o[0], outs[0][0]) and np.array_equal(o[1], outs[0][1])
    assert _rel(outs[0][0].reshape(n, d_out), O.gemm_f16(kind, ws[0][0], ws[0][1], x16.astype(np.float32))) < 2e-5


def test_rmsnorm_f16_columns():
    cfg = SHAPES["qwen36_moe"]
    dim, n = 2048, 37
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((n, dim)) * rng.uniform(0.1, 10, (n, 1))).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    ref = np.stack([O.rmsnorm(x[c], nw, cfg["eps"]) for c in range(n)]).astype(np.float64)
    with PooledAttn(cfg, 64, n_layers=1, max_cols=1) as pa:
        dx = pa.to_device(x); dnw = pa.to_device(nw); do = pa.alloc(n * dim * 2)
        pa.rmsnorm_f16(dx, dim, dnw, dim, n, do, dim); pa.sync()
        got = do.download(np.uint16, n * dim).view(np.float16).astype(np.float64).reshape(n, dim)
    assert np.abs(got - ref).max() <= np.abs(ref).max() * 2.0 ** -10          # f16 rounding of an f32 result


@pytest.mark.parametrize("shape,dim,kind,base,n", [("qwen36_moe", 512, PA_W_Q4_0, 100, 64), ("qwen36_moe", 1024, PA_W_Q8_0, 0, 33),
                                                    ("qwen3_1p7b", 512, PA_W_Q4_0, 300, 160), ("qwen38_27b", 1024, PA_W_Q8_0, 77, 40)])
def test_attn_layer_prefill_matches_oracle(shape, dim, kind, base, n):
    cfg = SHAPES[shape]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = nH * hd, nKV * hd
    q_rows = qd * (2 if cfg["gate"] else 1)
    rng = np.random.default_rng(base + dim + n)
    w_qkv, s_qkv = _weights(kind, q_rows + 2 * kvd, dim, rng, scale=0.05)
    w_o, s_o = _weights(kind, dim, qd, rng, scale=0.005)              # keeps the residual O(1): the gate below is absolute
    x = rng.standard_normal((n, dim)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    qw = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32); kw = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    k16, v16 = oracle_cache(cfg, rng.standard_normal((base, kvd)).astype(np.float32), rng.standard_normal((base, kvd)).astype(np.float32), kw)
    x_ref, k_rows, v_rows = O.attn_layer_prefill(x, kind, w_qkv, s_qkv, kind, w_o, s_o, nw, qw, kw, k16, v16, base, cfg)
    xs = dim + 4
    xpad = np.zeros((n, xs), np.float32); xpad[:, :dim] = x
    with PooledAttn(cfg, base + n + 8, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        if base:
            pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        wq = pa.weight(kind, w_qkv, s_qkv); wo = pa.weight(kind, w_o, s_o)
        dx = pa.to_device(xpad); dnw = pa.to_device(nw); dqw = pa.to_device(qw); dkw = pa.to_device(kw)
        pa.attn_layer_prefill(0, wq, wo, dnw, dqw, dkw, dx, xs, base, n); pa.sync()
        got = dx.download(np.float32, n * xs).reshape(n, xs)[:, :dim]
        kc = pa.kv_read(0, 0, base, n).view(np.float16).astype(np.float64); vc = pa.kv_read(0, 1, base, n).view(np.float16).astype(np.float64)
    assert_parity(got, x_ref, "layer prefill %s base %d n %d" % (shape, base, n))
    for a, b in ((kc, k_rows), (vc, v_rows)):
        ref = np.asarray(b).reshape(a.shape).view(np.float16).astype(np.float64)
        assert np.abs(a - ref).max() <= np.abs(ref).max() * 2.0 ** -9


def test_layer_calls_on_int8_caches_equal_their_stages():
    """pa_attn_layer_decode / pa_attn_layer_prefill on int8 caches: the same bits as their stages called one by one
    (each stage has its own parity test)."""
    from pooled_amd.capi import PA_OUT_F16
    cfg = dict(SHAPES["qwen36_moe"], kv_q8=True)
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd, dim = nH * hd, nKV * hd, 512
    q_rows = 2 * qd
    rng = np.random.default_rng(21)
    w_qkv, s_qkv = _weights(PA_W_Q4_0, q_rows + 2 * kvd, dim, rng, scale=0.05)
    w_o, s_o = _weights(PA_W_Q4_0, dim, qd, rng, scale=0.005)
    nw = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    hw = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    base, n = 200, 24
    xs = rng.standard_normal((base + n + 1, dim)).astype(np.float32)
    with PooledAttn(cfg, base + n + 1, n_layers=2, max_cols=base) as pa:
        pa.layer_alloc(0); pa.layer_alloc(1)
        wq = pa.weight(PA_W_Q4_0, w_qkv, s_qkv); wo = pa.weight(PA_W_Q4_0, w_o, s_o)
        dnw = pa.to_device(nw); dhw = pa.to_device(hw)
        rows = q_rows + 2 * kvd
        for layer, staged in ((0, False), (1, True)):
            # a chunk of `base` tokens, then a chunk of n, then one token
            outs = []
            for b0, cnt in ((0, base), (base, n)):
                dx = pa.to_device(xs[b0:b0 + cnt])
                if not staged:
                    pa.attn_layer_prefill(layer, wq, wo, dnw, dhw, dhw, dx, dim, b0, cnt)
                else:
                    dxn = pa.alloc(cnt * dim * 2); dqkv = pa.alloc(cnt * rows * 4); dat = pa.alloc(cnt * qd * 2)
                    pa.rmsnorm_f16(dx, dim, dnw, dim, cnt, dxn, dim)
                    pa.gemm(wq, dxn, dim, cnt, dqkv, rows)
                    pa.L.pa_glue_kv(pa.ctx, layer, dqkv.ptr, rows, dqkv.ptr + q_rows * 4, rows, dqkv.ptr + (q_rows + kvd) * 4, rows, dhw.ptr, dhw.ptr, b0, cnt)
                    pa.attn("prefill", layer, None, 0, pa.gate_buffer_ptr(), qd, b0, cnt, dat, qd, PA_OUT_F16)
                    pa.gemm(wo, dat, qd, cnt, dx, dim, acc=True)
                pa.sync()
                outs.append(dx.download(np.float32, cnt * dim))
            dx = pa.to_device(xs[base + n])
            if not staged:
                pa.attn_layer_decode(layer, wq, wo, dnw, dhw, dhw, dx, base + n)
            else:
                dqkv = pa.alloc(rows * 4); dat = pa.alloc(qd * 4)
                pa.gemv_norm(wq, dx, dnw, dqkv)
                pa.L.pa_attn_decode_step(pa.ctx, layer, dqkv.ptr, dqkv.ptr + q_rows * 4, dqkv.ptr + (q_rows + kvd) * 4, dhw.ptr, dhw.ptr, base + n, dat.ptr, 0)
                pa.gemv(wo, dat, dx, acc=True)
            pa.sync()
            outs.append(dx.download(np.float32, dim))
            if not staged:
                first = outs
        for a, b in zip(first, outs):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
            assert np.all(np.isfinite(a))
        for w in range(4):
            assert np.array_equal(pa.kv_read(0, w, 0, base + n + 1), pa.kv_read(1, w, 0, base + n + 1))
