"""The committed fixtures (tests/golden/attn_cases.npz, written by tests/golden/make_fixtures.py from seeded inputs)
against the three CPU restatements: the numpy oracle must reproduce them (drift guard: cache bits and the roped q
exactly, attention to 1e-6), and the C oracle and the JavaScript restatement of the reference's loops, which share
no code with it, must agree with them to 2e-5 (the reference's own bar, tests/test_attn_dec.js:98)."""
import json
import os
import shutil
import struct
import subprocess
import numpy as np
import pytest
from oracle import attn_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIX = os.path.join(ROOT, "tests", "golden", "attn_cases.npz")


def load_cases():
    z = np.load(FIX)                                   # plain arrays only (allow_pickle stays off)
    meta = json.loads(bytes(z["meta"]).decode())
    return [(m, {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(m["name"] + ".")}) for m in meta]


CASES = load_cases()
IDS = [m["name"] for m, _ in CASES]


def _rel(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max()) / max(float(np.abs(b).max()), 1e-30)


@pytest.mark.parametrize("meta,d", CASES, ids=IDS)
def test_numpy_oracle_reproduces_the_fixtures(meta, d):
    cfg, base, n = meta["cfg"], meta["base_pos"], meta["n_cols"]
    step = O.glue_kv(d["qraw"], d["kraw"], d["vraw"], d["qw"], d["kw"], base, cfg)
    assert np.array_equal(step["q"].view(np.uint32), d["q"].view(np.uint32))
    assert np.array_equal(step["k16"], d["k16"][base:]) and np.array_equal(step["v16"], d["v16"][base:])
    if cfg["gate"]:
        assert np.array_equal(step["gate"].view(np.uint32), d["gate"].view(np.uint32))
    gate = d.get("gate")
    if meta["kv_q8"]:
        out = O.attention_values(d["q"], O.q8_dequantize(d["kq"], d["ks"]), O.q8_dequantize(d["vq"], d["vs"]), base, gate=gate)
    else:
        out = O.attention(d["q"], d["k16"], d["v16"], base, gate=gate)
    assert _rel(out, d["attn"]) < 1e-6


@pytest.mark.parametrize("meta,d", [c for c in CASES if not c[0]["kv_q8"]], ids=[i for i, c in zip(IDS, CASES) if not c[0]["kv_q8"]])
def test_c_oracle_agrees_with_the_fixtures(meta, d):
    from oracle import c_oracle
    out = c_oracle.attention(d["q"], d["k16"], d["v16"], meta["base_pos"], gate=d.get("gate"))
    assert _rel(out, d["attn"]) < 2e-5


@pytest.mark.skipif(shutil.which("node") is None, reason="node not installed")
@pytest.mark.parametrize("meta,d", [c for c in CASES if not c[0]["kv_q8"]], ids=[i for i, c in zip(IDS, CASES) if not c[0]["kv_q8"]])
def test_reference_loops_under_node_agree_with_the_fixtures(meta, d, tmp_path):
    cfg, base, n = meta["cfg"], meta["base_pos"], meta["n_cols"]
    gate = d.get("gate")
    inp, outp = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(inp, "wb") as f:
        f.write(struct.pack("8i", n, cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], base, d["k16"].shape[0], 1 if gate is not None else 0, n))
        f.write(np.arange(n, dtype=np.int32).tobytes())
        f.write(np.ascontiguousarray(d["q"], np.float32).tobytes())
        f.write(np.ascontiguousarray(d["k16"]).tobytes()); f.write(np.ascontiguousarray(d["v16"]).tobytes())
        if gate is not None:
            f.write(np.ascontiguousarray(gate, np.float32).tobytes())
    r = subprocess.run([shutil.which("node"), os.path.join(ROOT, "oracle", "attn_ref.js"), inp, outp, "1"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-400:]
    out = np.fromfile(outp, dtype=np.float32).reshape(d["attn"].shape)
    assert _rel(out, d["attn"]) < 2e-5
