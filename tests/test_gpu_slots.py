"""GPU tests of the checkpoint slots through the C ABI: byte-exact round trips (integer / byte work), the
reference's saveSlot / loadSlot / dropSlot semantics, and the host parts in the position-major layout."""
import numpy as np
import pytest
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn, PaError, PA_ERR_INVALID
from helpers import SHAPES, assert_parity, random_cache

pytestmark = pytest.mark.gpu


def _fill(pa, cfg, max_seq, layers, seed):
    caches = {}
    for l in layers:
        pa.layer_alloc(l)
        k16, v16 = random_cache(cfg, max_seq, seed=seed + l)
        pa.kv_write(l, 0, 0, k16); pa.kv_write(l, 1, 0, v16)
        caches[l] = (k16.reshape(max_seq, -1), v16.reshape(max_seq, -1))
    return caches


@pytest.mark.parametrize("shape,pos", [("qwen36_moe", 777), ("qwen3_1p7b", 1000), ("qwen38_27b", 1)])
def test_save_overwrite_load_is_byte_exact(shape, pos):
    cfg = SHAPES[shape]
    max_seq = pos + 50
    with PooledAttn(cfg, max_seq, n_layers=3, max_cols=1) as pa:
        caches = _fill(pa, cfg, max_seq, (0, 2), seed=5)           # layer 1 has no cache: slots skip it
        pa.slot_save(7, pos)
        assert pa.slot_pos(7) == pos
        junk = np.full((max_seq, cfg["n_kv_heads"] * cfg["head_dim"]), 0x7E00, np.uint16)
        for l in (0, 2):
            pa.kv_write(l, 0, 0, junk); pa.kv_write(l, 1, 0, junk)
        assert pa.slot_load(7) == pos
        for l in (0, 2):
            K = pa.kv_read(l, 0, 0, max_seq).reshape(max_seq, -1); V = pa.kv_read(l, 1, 0, max_seq).reshape(max_seq, -1)
            assert np.array_equal(K[:pos], caches[l][0][:pos]) and np.array_equal(V[:pos], caches[l][1][:pos])
            assert np.all(K[pos:] == 0x7E00) and np.all(V[pos:] == 0x7E00), "rows at or past the saved position were touched"
        # host parts: position-major, equal to what pa_kv_read gives for the same rows
        for l in (0, 2):
            assert np.array_equal(pa.slot_export(7, l, 0), caches[l][0][:pos])
            assert np.array_equal(pa.slot_export(7, l, 1), caches[l][1][:pos])


def test_slot_semantics():
    cfg = SHAPES["qwen36_moe"]
    with PooledAttn(cfg, 200, n_layers=1, max_cols=1) as pa:
        caches = _fill(pa, cfg, 200, (0,), seed=9)
        with pytest.raises(PaError) as e:
            pa.slot_load(3)                                          # "no saved slot"
        assert e.value.code == PA_ERR_INVALID and "no saved slot" in str(e.value)
        pa.slot_drop(3)                                              # dropping an unknown slot is fine
        pa.slot_save(3, 100); pa.slot_save(3, 40)                    # saving again replaces
        assert pa.slot_pos(3) == 40
        pa.slot_save(4, 0)                                           # an empty context is a valid checkpoint
        assert pa.slot_load(4) == 0
        pa.slot_drop(3)
        with pytest.raises(PaError):
            pa.slot_pos(3)
        with pytest.raises(PaError):
            pa.slot_save(5, 201)                                     # past max_seq


def test_import_parts_then_decode():
    """A state exported from one context loads into a fresh one (parts in the reference's layout) and attention over
    it equals the oracle."""
    cfg = SHAPES["qwen36_moe"]
    pos, max_seq = 1500, 1600
    rng = np.random.default_rng(3)
    q = rng.standard_normal((1, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
    gate = rng.standard_normal(q.shape, dtype=np.float32)
    with PooledAttn(cfg, max_seq, n_layers=2, max_cols=1) as a:
        caches = _fill(a, cfg, max_seq, (0, 1), seed=21)
        a.slot_save(1, pos)
        parts = [(l, w, a.slot_export(1, l, w)) for l in (0, 1) for w in (0, 1)]
    with PooledAttn(cfg, max_seq, n_layers=2, max_cols=1) as b:
        b.layer_alloc(0); b.layer_alloc(1)
        b.slot_create(9, pos)
        for l, w, part in parts:
            b.slot_import(9, l, w, part)
        assert b.slot_load(9) == pos
        got = b.run_attn("decode", 1, q, pos - 1, gate=gate)
    k16 = caches[1][0].reshape(max_seq, cfg["n_kv_heads"], cfg["head_dim"]); v16 = caches[1][1].reshape(k16.shape)
    assert_parity(got, C.attention(q, k16, v16, pos - 1, gate=gate), "decode over an imported state")
