"""The HIP path, through the C ABI, against the committed fixtures (tests/golden/attn_cases.npz): the pre-step's q,
gate and cache rows bit for bit, the attention outputs to the parity gate (max-abs 2e-3, relative 1e-2), for the
three-launch sequence, the fused one-token entry point, and both output types."""
import numpy as np
import pytest
from pooled_amd.capi import PooledAttn, PA_OUT_F16
from helpers import assert_parity
from test_golden import CASES, IDS

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("meta,d", CASES, ids=IDS)
def test_hip_path_matches_the_fixtures(meta, d):
    cfg, base, n, q8 = dict(meta["cfg"], kv_q8=meta["kv_q8"]), meta["base_pos"], meta["n_cols"], meta["kv_q8"]
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    gate = d.get("gate")
    kind = "decode" if n * (cfg["n_heads"] // nKV) <= (32 if hd == 256 else 64) else "prefill"
    with PooledAttn(cfg, base + n + 5, n_layers=1, max_cols=n) as pa:
        pa.layer_alloc(0)
        prior = (d["kq"], d["vq"], d["ks"], d["vs"]) if q8 else (d["k16"], d["v16"])
        if base:
            for w, a in enumerate(prior):
                pa.kv_write(0, w, 0, a[:base])
        # pre-step of the pass's columns: q, gate and the new cache rows
        pa.run_glue_kv(0, d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base)
        assert np.array_equal(pa.read_q_buffer(n).view(np.uint32).reshape(-1), d["q"].view(np.uint32).reshape(-1))
        if gate is not None:
            assert np.array_equal(pa.read_gate_buffer(n).view(np.uint32).reshape(-1), gate.view(np.uint32).reshape(-1))
        for w, a in enumerate(prior):
            assert np.array_equal(pa.kv_read(0, w, 0, base + n).reshape(a.shape), a), "cache tensor %d" % w
        # attention over the cache the library wrote
        out = pa.run_attn(kind, 0, d["q"], base, gate=gate)
        assert_parity(out, d["attn"], meta["name"])
        out16 = pa.run_attn(kind, 0, d["q"], base, gate=gate, out_dtype=PA_OUT_F16).astype(np.float32)
        assert_parity(out16, d["attn"], meta["name"] + " f16 out")
        if n == 1:
            # the fused one-token entry point rewrites row base with the same bits and gives the same output
            fused = pa.run_decode_step(0, d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"], base)
            assert_parity(fused.reshape(d["attn"].shape), d["attn"], meta["name"] + " fused step")
            for w, a in enumerate(prior):
                assert np.array_equal(pa.kv_read(0, w, 0, base + n).reshape(a.shape), a), "cache tensor %d after the fused step" % w
