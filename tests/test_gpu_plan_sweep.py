"""The gfx950 table over random (columns, position) pairs: what a plan query reports is consistent with the pass it
describes, and the pass it drives agrees with the oracle -- across the table's regimes (single-round splits with one and
two row blocks, the tile loop with tiles dealt round robin, several column groups, a single split that writes the
output itself) and at their edges (a context one row either side of a whole number of splits or of a regime's
capacity)."""
import numpy as np
import pytest
from oracle import c_oracle as C
from pooled_amd.capi import PooledAttn
from helpers import SHAPES, assert_parity, random_cache

pytestmark = pytest.mark.gpu

MAX_ROWS, MAX_COLS = 9000, 20


def _cases(shape, rng):
    cfg = SHAPES[shape]
    G = cfg["n_heads"] // cfg["n_kv_heads"]
    out = []
    # edges: contexts around multiples of 128 rows and around the two-row-block single-round kernel's capacity
    # (256 / kv heads splits at one column group, half of that at two), one row either side
    cap = 256 // cfg["n_kv_heads"] * 128
    for n_cols in (1, 2, 32 // G, 32 // G + 1, MAX_COLS):
        for L in (128, 129, 4096, cap, cap // 2):
            for d in (-1, 0, 1):
                if 0 < L + d - n_cols and L + d <= MAX_ROWS:
                    out.append((n_cols, L + d - n_cols))
    for _ in range(24):
        n_cols = int(rng.integers(1, MAX_COLS + 1))
        out.append((n_cols, int(rng.integers(0, MAX_ROWS - n_cols))))
    return sorted(set(out))


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_plans_and_passes_over_random_blocks(shape):
    cfg = SHAPES[shape]
    G = cfg["n_heads"] // cfg["n_kv_heads"]
    rng = np.random.default_rng(len(shape))
    k16, v16 = random_cache(cfg, MAX_ROWS + 40, seed=77)
    K, V = k16.copy(), v16.copy()
    with PooledAttn(cfg, MAX_ROWS + 40, n_layers=1, max_cols=MAX_COLS) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, K); pa.kv_write(0, 1, 0, V)
        seen = set()
        for n_cols, base in _cases(shape, rng):
            pl = pa.plan("decode", base, n_cols)
            L = base + n_cols
            streamed = max(L - (1 if n_cols == 1 else 0), 1)          # a one-column decode keeps its own row out of the stream
            assert pl["kernel"] == 0 and pl["waves"] in (4, 8) and 1 <= pl["row_blocks"] <= 4, pl
            assert pl["split_len"] % 32 == 0 and pl["n_splits"] * pl["split_len"] >= streamed, (n_cols, base, pl)
            assert (pl["n_splits"] - 1) * 128 < streamed, (n_cols, base, pl)      # no split without a row
            assert pl["slots"] == pl["n_splits"] + (1 if n_cols == 1 else 0), pl
            assert pl["col_groups"] * pl["cols_per_group"] >= n_cols > (pl["col_groups"] - 1) * pl["cols_per_group"], pl
            assert pl["cols_per_group"] * G <= 16 * pl["row_blocks"], pl
            seen.add((pl["row_blocks"], pl["split_len"] == 128, pl["n_splits"] > 1, pl["col_groups"] > 1))
            q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
            gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
            ref = C.attention(q, k16, v16, base, gate=gate)
            assert_parity(pa.run_attn("decode", 0, q, base, gate=gate), ref, "%s %d columns at %d: %s" % (shape, n_cols, base, pl))
        # the regimes the sweep is meant to cross: one and two row blocks on one-tile-per-wave splits, longer splits,
        # one split, several column groups
        assert any(s[0] == 1 and s[1] and s[2] for s in seen) and any(s[0] == 2 and s[1] and s[2] for s in seen), seen
        assert any(not s[1] and s[2] for s in seen) and any(not s[2] for s in seen), seen
        assert any(s[3] for s in seen) or cfg["head_dim"] == 128, seen      # (64 rows a workgroup at hd 128: 20 columns of G = 2 are one group)


@pytest.mark.parametrize("shape", ["qwen36_moe", "qwen38_27b", "qwen3_1p7b"])
def test_prefill_plans_and_passes_over_random_chunks(shape):
    """The same for prefill chunks: narrow chunks on the split-K kernel (column groups over a long context, one launch
    with direct output over a short one), wider ones on the matrix-core kernel, split over the context or not."""
    cfg = SHAPES[shape]
    rng = np.random.default_rng(7 + len(shape))
    rows, max_cols = 6000, 700
    k16, v16 = random_cache(cfg, rows + 40, seed=78)
    cases = [(1, 0), (33, 0), (256, 0), (512, 1536), (700, 5000), (16, 5900), (64, 4096), (100, 4095), (257, 255)]
    for _ in range(10):
        n = int(rng.integers(1, max_cols + 1))
        cases.append((n, int(rng.integers(0, rows - n))))
    with PooledAttn(cfg, rows + 40, n_layers=1, max_cols=max_cols) as pa:
        pa.layer_alloc(0)
        pa.kv_write(0, 0, 0, k16.copy()); pa.kv_write(0, 1, 0, v16.copy())
        kernels = set()
        for n_cols, base in cases:
            pl = pa.plan("prefill", base, n_cols)
            assert pl["kernel"] in (0, 1) and pl["n_splits"] >= 1 and pl["split_len"] % 32 == 0, pl
            assert pl["n_splits"] * pl["split_len"] >= base + n_cols, (n_cols, base, pl)
            assert pl["col_groups"] * pl["cols_per_group"] >= n_cols > (pl["col_groups"] - 1) * pl["cols_per_group"], pl
            kernels.add((pl["kernel"], pl["n_splits"] > 1))
            q = rng.standard_normal((n_cols, cfg["n_heads"], cfg["head_dim"]), dtype=np.float32)
            gate = rng.standard_normal(q.shape, dtype=np.float32) if cfg["gate"] else None
            ref = C.attention(q, k16, v16, base, gate=gate)
            assert_parity(pa.run_attn("prefill", 0, q, base, gate=gate), ref, "%s prefill %d columns at %d: %s" % (shape, n_cols, base, pl))
        # (chunks this narrow leave CUs idle on the matrix-core kernel, so it is always split over the context here)
        assert (0, False) in kernels and any(k[0] == 1 for k in kernels) and any(k[1] for k in kernels), kernels
