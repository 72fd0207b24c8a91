"""The JavaScript host shim + Node-API addon on the GPU: one case through the engine-shaped methods
(_encAttnGlue / _encAttnCore / encodeLayerAttn), checked in tests/js/shim_case.js against the oracle."""
import json
import os
import shutil
import subprocess
import numpy as np
import pytest
from oracle import attn_oracle as O
from oracle import c_oracle as C
from helpers import SHAPES, oracle_cache

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("node") is None, reason="node not installed")
@pytest.mark.parametrize("shape,base,n", [("qwen36_moe", 1000, 32), ("qwen3_1p7b", 300, 128)])
def test_js_shim_case(tmp_path, shape, base, n):
    assert os.path.exists(os.path.join(ROOT, "pooled_amd", "lib", "pooled_attn.node")), "addon not built"
    cfg = SHAPES[shape]
    d = O.make_inputs(cfg, base, n, seed=77)
    k16, v16 = oracle_cache(cfg, d["kraw"], d["vraw"], d["kw"])
    g = O.glue_kv(d["qraw"], d["kraw"][base:], d["vraw"][base:], d["qw"], d["kw"], base, cfg)
    ref = C.attention(g["q"], k16, v16, base, gate=g["gate"])
    files = {"qw.bin": d["qw"], "kw.bin": d["kw"], "k16.bin": k16[:base], "v16.bin": v16[:base], "qraw.bin": d["qraw"],
             "kraw.bin": d["kraw"][base:], "vraw.bin": d["vraw"][base:], "expect.bin": ref.astype(np.float32),
             "knew16.bin": k16[base:], "vnew16.bin": v16[base:]}
    for name, arr in files.items():
        np.ascontiguousarray(arr).tofile(tmp_path / name)
    (tmp_path / "case.json").write_text(json.dumps({"cfg": cfg, "basePos": base, "nCols": n}))
    r = subprocess.run(["node", os.path.join(ROOT, "tests", "js", "shim_case.js"), str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr)
    assert r.returncode == 0 and "SHIM PASS" in r.stdout, r.stdout + r.stderr
