"""Shared test helpers: the benchmark shapes, cache construction through the oracle, the parity gate."""
import numpy as np
from oracle import attn_oracle as O

# shapes of the five benchmark configurations
SHAPES = {
    "qwen3_1p7b": dict(n_heads=16, n_kv_heads=8, head_dim=128, n_rot=128, rope_theta=1e6, eps=1e-6, qk_norm=True, gate=False),
    "qwen36_moe": dict(n_heads=16, n_kv_heads=2, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True),
    "qwen38_27b": dict(n_heads=24, n_kv_heads=4, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True),
}

# the north star's tolerance: max-abs 2e-3 and relative 1e-2 of the f32 reference
MAX_ABS, MAX_REL = 2e-3, 1e-2


def assert_parity(got, ref, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.all(np.isfinite(got)), "%s: non-finite output" % what
    d = np.abs(got - ref).max()
    rel = d / max(np.abs(ref).max(), 1e-30)
    assert d <= MAX_ABS and rel <= MAX_REL, "%s: max-abs %.3e (limit %.0e), rel %.3e (limit %.0e)" % (what, d, MAX_ABS, rel, MAX_REL)
    return d, rel


def oracle_cache(cfg, kraw, vraw, kw):
    """f16 cache rows for tokens at positions 0..n-1 (K normed + roped, V raw), via the oracle's pre-step."""
    n = kraw.shape[0]
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    k = np.asarray(kraw, np.float32).reshape(n, nKV, hd)
    if cfg.get("qk_norm", True):
        k = O.head_rmsnorm(k, kw, cfg["eps"])
    k = O.rope_neox(k, np.arange(n), cfg["n_rot"], cfg["rope_theta"])
    return O.f16_bits(k), O.f16_bits(np.asarray(vraw, np.float32).reshape(n, nKV, hd))


def random_cache(cfg, rows, seed, k_scale=1.0):
    """Seeded N(0,1) f16 cache rows without the pre-step (for attention-only tests)."""
    rng = np.random.default_rng(seed)
    shape = (rows, cfg["n_kv_heads"], cfg["head_dim"])
    k = (rng.standard_normal(shape, dtype=np.float32) * k_scale).astype(np.float16).view(np.uint16)
    v = rng.standard_normal(shape, dtype=np.float32).astype(np.float16).view(np.uint16)
    return k, v
