"""GPU parity of the fused one-token entry point (pre-step + cache write + split-K attention + merge + gate in one
call) through the C ABI.  The written cache row equals the oracle's bits, the rows around it stay untouched, and
the output equals pa_glue_kv followed by pa_attn_decode bit for bit (same kernels' arithmetic) and the oracle
within the floating-point bar: max-abs <= 2e-3 and max|d|/max|ref| <= 1e-2."""
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PaError, PA_OUT_F16, PA_ERR_INVALID
from helpers import SHAPES, assert_parity, random_cache

pytestmark = pytest.mark.gpu


def _case(cfg, pos, seed):
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    max_seq = pos + 5
    k16, v16 = random_cache(cfg, max_seq, seed=seed)
    d = O.make_inputs(cfg, 0, 1, seed + 1)
    ref_g = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], pos, cfg)
    K = k16.copy(); V = v16.copy()
    K[pos] = ref_g["k16"].reshape(nKV, hd); V[pos] = ref_g["v16"].reshape(nKV, hd)
    gate = ref_g["gate"].reshape(1, nH, hd) if cfg.get("gate") else None
    ref = C.attention(ref_g["q"].reshape(1, nH, hd), K, V, pos, gate=gate)
    return d, k16, v16, K, V, ref, max_seq


@pytest.mark.parametrize("shape,pos", [
    ("qwen36_moe", 0), ("qwen36_moe", 1), ("qwen36_moe", 31), ("qwen36_moe", 32), ("qwen36_moe", 95), ("qwen36_moe", 777),
    ("qwen36_moe", 4096), ("qwen36_moe", 20001), ("qwen38_27b", 300), ("qwen38_27b", 5000), ("qwen3_1p7b", 129),
    ("qwen3_1p7b", 2500),
])
def test_decode_step_matches_oracle_and_unfused(shape, pos):
    cfg = SHAPES[shape]
    d, k16, v16, K, V, ref, max_seq = _case(cfg, pos, seed=pos + 3)
    poison = np.uint16(0x7E00)
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        for which, a in ((0, k16), (1, v16)):
            a = a.copy(); a[pos] = poison                        # the row the call must write is NaN before it
            pa.kv_write(0, which, 0, a)
        got = pa.run_decode_step(0, d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"], pos)
        Kg = pa.kv_read(0, 0, 0, max_seq); Vg = pa.kv_read(0, 1, 0, max_seq)
        # the unfused pair on a fresh copy of the same cache
        for which, a in ((0, k16), (1, v16)):
            pa.kv_write(0, which, 0, a)
        pa.run_glue_kv(0, d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], pos)
        gate = pa.read_gate_buffer(1) if cfg.get("gate") else None
        unf = pa.run_attn("decode", 0, pa.read_q_buffer(1), pos, gate=gate)
    assert np.array_equal(Kg.reshape(K.shape), K) and np.array_equal(Vg.reshape(V.shape), V), "cache differs from the oracle's bits"
    assert_parity(got[None], ref, "%s pos %d" % (shape, pos))
    assert np.array_equal(got.view(np.uint32), unf[0].view(np.uint32)), "fused output differs from pa_glue_kv + pa_attn_decode"


def test_decode_step_f16_out_and_no_norm():
    cfg = dict(SHAPES["qwen3_1p7b"], qk_norm=False)
    pos = 600
    d, k16, v16, K, V, ref, max_seq = _case(cfg, pos, seed=5)
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        got = pa.run_decode_step(0, d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"], pos, out_dtype=PA_OUT_F16)
        Kg = pa.kv_read(0, 0, 0, max_seq)
    assert np.array_equal(Kg.reshape(K.shape), K)
    assert_parity(got[None].astype(np.float32), ref, "f16 out, no norm")


def test_decode_step_sequence():
    """Twelve consecutive tokens through the fused call: every step sees the rows the earlier steps wrote."""
    cfg = SHAPES["qwen36_moe"]
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    base, n = 250, 12
    k16, v16 = random_cache(cfg, base + n, seed=31)
    d = O.make_inputs(cfg, 0, n, 32)
    ref_g = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base, cfg)
    K = k16.copy(); V = v16.copy()
    K[base:base + n] = ref_g["k16"].reshape(n, nKV, hd); V[base:base + n] = ref_g["v16"].reshape(n, nKV, hd)
    ref = C.attention(ref_g["q"].reshape(n, nH, hd), K, V, base, gate=ref_g["gate"].reshape(n, nH, hd))
    with PooledAttn(cfg, base + n, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        outs = [pa.run_decode_step(0, d["qraw"][c], d["kraw"][c], d["vraw"][c], d["qw"], d["kw"], base + c) for c in range(n)]
    assert_parity(np.stack(outs), ref, "sequence")


def test_decode_step_rejects_bad_arguments():
    cfg = SHAPES["qwen36_moe"]
    with PooledAttn(cfg, 64, n_layers=1, max_cols=1) as pa:
        pa.layer_alloc(0)
        d = O.make_inputs(cfg, 0, 1, 1)
        with pytest.raises(PaError) as e:
            pa.run_decode_step(0, d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"], 64)   # pos == max_seq
        assert e.value.code == PA_ERR_INVALID


@pytest.mark.parametrize("cfg", [
    dict(n_heads=32, n_kv_heads=2, head_dim=128, n_rot=128, rope_theta=1e6, eps=1e-6, qk_norm=True, gate=False),   # G = 16: a full MFMA row block
    dict(n_heads=32, n_kv_heads=2, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True),     # G = 16 at hd 256
    dict(n_heads=4, n_kv_heads=4, head_dim=256, n_rot=256, rope_theta=1e4, eps=1e-5, qk_norm=False, gate=True),    # G = 1, full RoPE, no norm
])
def test_group_sizes_one_and_sixteen(cfg):
    """Group sizes at both ends of what one 16-row block holds, through the fused step, the unfused pair, a verify
    block and a prefill chunk."""
    pos = 1234
    d, k16, v16, K, V, ref, max_seq = _case(cfg, pos, seed=77)
    nH, hd = cfg["n_heads"], cfg["head_dim"]
    with PooledAttn(cfg, max_seq, n_layers=1, max_cols=64) as pa:
        pa.layer_alloc(0); pa.kv_write(0, 0, 0, k16); pa.kv_write(0, 1, 0, v16)
        got = pa.run_decode_step(0, d["qraw"][0], d["kraw"][0], d["vraw"][0], d["qw"], d["kw"], pos)
        assert_parity(got[None], ref, "fused step G=%d" % (nH // cfg["n_kv_heads"]))
        rng = np.random.default_rng(1)
        q = rng.standard_normal((48, nH, hd), dtype=np.float32)
        gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
        base = pos - 47
        refb = C.attention(q, K, V, base, gate=gate)
        assert_parity(pa.run_attn("decode", 0, q[:5], base, gate=None if gate is None else gate[:5]), refb[:5], "verify block")
        assert_parity(pa.run_attn("prefill", 0, q, base, gate=gate), refb, "prefill chunk")
        # the unfused one-column decode: its own row's O partial sits under the kv head's first head, for G = 1 and 16 too
        assert_parity(pa.run_attn("decode", 0, q[47:], pos, gate=None if gate is None else gate[47:]), refb[47:], "one-column decode")
