"""The decode entry points under HIP graph capture (callers that replay a recorded token step instead of launching
it): after one eager warm-up call (which sizes the context's partial buffers) the fused one-token call and the
layer call record nothing but kernel launches, so a captured sequence can be replayed.  Every replay -- with eager
work and synchronisations of the library's own between the replays -- must reproduce the eager results bit for bit."""
import ctypes
import numpy as np
import pytest
from pooled_amd.capi import PooledAttn, PA_OUT_F32, PA_W_Q4_0
from helpers import SHAPES

pytestmark = pytest.mark.gpu
vp = ctypes.c_void_p


def _hip():
    h = ctypes.CDLL("libamdhip64.so")
    for name, args in (("hipStreamCreate", [ctypes.POINTER(vp)]), ("hipStreamDestroy", [vp]), ("hipStreamSynchronize", [vp]),
                       ("hipStreamBeginCapture", [vp, ctypes.c_int]), ("hipStreamEndCapture", [vp, ctypes.POINTER(vp)]),
                       ("hipGraphInstantiate", [ctypes.POINTER(vp), vp, vp, vp, ctypes.c_size_t]), ("hipGraphLaunch", [vp, vp]),
                       ("hipGraphExecDestroy", [vp]), ("hipGraphDestroy", [vp])):
        f = getattr(h, name); f.restype = ctypes.c_int; f.argtypes = args
    return h


def _ok(rc, what):
    assert rc == 0, "%s failed with HIP error %d" % (what, rc)


def test_decode_steps_replayed_from_a_graph():
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd, dim = nH * hd, nKV * hd, 512
    base, steps = 3000, 4
    rng = np.random.default_rng(5)
    hip = _hip()
    stream = vp()
    _ok(hip.hipStreamCreate(ctypes.byref(stream)), "hipStreamCreate")
    with PooledAttn(cfg, base + steps + 1, n_layers=1, max_cols=1) as pa:
        pa._chk(pa.L.pa_set_stream(pa.ctx, stream))
        pa.layer_alloc(0)
        k0 = rng.standard_normal((base, kvd), dtype=np.float32).astype(np.float16).view(np.uint16)
        v0 = rng.standard_normal((base, kvd), dtype=np.float32).astype(np.float16).view(np.uint16)
        pa.kv_write(0, 0, 0, k0); pa.kv_write(0, 1, 0, v0)
        dq = [pa.to_device(rng.standard_normal(2 * qd, dtype=np.float32)) for _ in range(steps)]
        dk = [pa.to_device(rng.standard_normal(kvd, dtype=np.float32)) for _ in range(steps)]
        dv = [pa.to_device(rng.standard_normal(kvd, dtype=np.float32)) for _ in range(steps)]
        dw = pa.to_device((1 + 0.1 * rng.standard_normal(hd)).astype(np.float32))
        douts = [pa.alloc(qd * 4) for _ in range(steps)]
        # a layer call on top: residual in / out, Q4_0 projections
        sc = lambda r, c: np.asarray(rng.uniform(0.002, 0.004, (r, c // 32)), np.float16).view(np.uint16)
        wq = pa.weight(PA_W_Q4_0, rng.integers(0, 256, (2 * qd + 2 * kvd, dim // 2), dtype=np.uint8), sc(2 * qd + 2 * kvd, dim))
        wo = pa.weight(PA_W_Q4_0, rng.integers(0, 256, (dim, qd // 2), dtype=np.uint8), sc(dim, qd))
        x0 = rng.standard_normal(dim, dtype=np.float32)
        dx = pa.to_device(x0); dnw = pa.to_device(np.ones(dim, np.float32))

        def sequence():
            for i in range(steps):
                pa.attn_decode_step(0, dq[i], dk[i], dv[i], dw, dw, base + i, douts[i], PA_OUT_F32)
            pa.attn_layer_decode(0, wq, wo, dnw, dw, dw, dx, base + steps)

        def results():
            pa.sync()
            return [d.download(np.float32, qd).copy() for d in douts] + [dx.download(np.float32, dim).copy(),
                    pa.kv_read(0, 0, base, steps + 1).copy(), pa.kv_read(0, 1, base, steps + 1).copy()]

        sequence()                                        # eager: also the warm-up that sizes the context's buffers
        eager = results()
        assert all(np.all(np.isfinite(a)) for a in eager[:steps + 1])
        graph, gexec = vp(), vp()
        dx.upload(x0)
        _ok(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        sequence()
        _ok(hip.hipStreamEndCapture(stream, ctypes.byref(graph)), "hipStreamEndCapture")
        _ok(hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
        for rep in range(3):
            # eager work of the library's own between replays: wipe what the sequence writes, restore the residual
            pa.kv_write(0, 0, base, np.zeros((steps + 1, kvd), np.uint16)); pa.kv_write(0, 1, base, np.zeros((steps + 1, kvd), np.uint16))
            for d in douts:
                d.upload(np.zeros(qd, np.float32))
            dx.upload(x0)
            pa.sync()
            _ok(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            _ok(hip.hipStreamSynchronize(stream), "hipStreamSynchronize")
            for a, b in zip(results(), eager):
                assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), "replay %d differs from the eager run" % rep
        _ok(hip.hipGraphExecDestroy(gexec), "hipGraphExecDestroy"); _ok(hip.hipGraphDestroy(graph), "hipGraphDestroy")
        pa._chk(pa.L.pa_set_stream(pa.ctx, None))
    _ok(hip.hipStreamDestroy(stream), "hipStreamDestroy")
