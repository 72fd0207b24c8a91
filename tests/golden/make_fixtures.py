#!/usr/bin/env python3
"""Writes tests/golden/attn_cases.npz: small input / expected-output vectors for the attention path.

The reference holds no attention vectors of its own (its tests generate inputs inline and compare against f64
loops computed on the spot: tests/test_attn_dec.js:72-98, tests/unit/attn_tile_test.js:63-129), so these fixtures
are produced here, from seeded inputs, by the CPU oracle (oracle/attn_oracle.py), and every attention output is
cross-checked at generation time against the JavaScript restatement of the reference's loops (oracle/attn_ref.js,
run under node) -- two independent implementations must agree to 2e-5 before a case is written.  The fixtures pin
the oracle against drift (tests/test_oracle.py) and give the GPU tests fixed vectors (tests/test_gpu_golden.py).

    python tests/golden/make_fixtures.py        # rewrites attn_cases.npz next to this file
"""
import json, os, shutil, struct, subprocess, sys, tempfile
import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import attn_oracle as O  # noqa: E402

DENSE = dict(n_heads=4, n_kv_heads=2, head_dim=128, n_rot=128, rope_theta=1e6, eps=1e-6, qk_norm=True, gate=False)
MOE = dict(n_heads=8, n_kv_heads=1, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True)
B27 = dict(n_heads=6, n_kv_heads=1, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True)

# name, config, base_pos, n_cols, int8 cache
CASES = [
    ("dense_decode", DENSE, 37, 1, False),
    ("moe_decode", MOE, 40, 1, False),
    ("moe_first_token", MOE, 0, 1, False),
    ("b27_verify4", B27, 29, 4, False),
    ("dense_prefill33", DENSE, 0, 33, False),
    ("moe_prefill_chunk", MOE, 21, 5, False),
    ("moe_decode_q8", MOE, 35, 1, True),
]


def js_attention(cfg, q, k16, v16, gate, base_pos):
    """The reference loops under node; None when node is absent."""
    node = shutil.which("node")
    if node is None:
        return None
    n, nH, hd = q.shape
    rows = k16.shape[0]
    with tempfile.TemporaryDirectory() as td:
        inp, outp = os.path.join(td, "in.bin"), os.path.join(td, "out.bin")
        with open(inp, "wb") as f:
            f.write(struct.pack("8i", n, nH, cfg["n_kv_heads"], hd, base_pos, rows, 1 if gate is not None else 0, n))
            f.write(np.arange(n, dtype=np.int32).tobytes())
            f.write(np.ascontiguousarray(q, np.float32).tobytes())
            f.write(np.ascontiguousarray(k16, np.uint16).tobytes()); f.write(np.ascontiguousarray(v16, np.uint16).tobytes())
            if gate is not None:
                f.write(np.ascontiguousarray(gate, np.float32).tobytes())
        r = subprocess.run([node, os.path.join(ROOT, "oracle", "attn_ref.js"), inp, outp, "1"], capture_output=True, text=True, timeout=120)
        if r.returncode != 0:
            raise RuntimeError("attn_ref.js failed: " + r.stderr[-400:])
        return np.fromfile(outp, dtype=np.float32).reshape(n, nH, hd)


def build_case(name, cfg, base, n, q8, seed):
    nKV, hd = cfg["n_kv_heads"], cfg["head_dim"]
    d = O.make_inputs(cfg, base, n, seed)
    # cache rows [0, base): the oracle's pre-step on the first `base` raw rows, one position each
    zq = np.zeros((base, d["qraw"].shape[1]), np.float32)
    prior = O.glue_kv(zq, d["kraw"][:base], d["vraw"][:base], d["qw"], d["kw"], 0, cfg) if base else None
    step = O.glue_kv(d["qraw"], d["kraw"][base:], d["vraw"][base:], d["qw"], d["kw"], base, cfg)
    k16 = np.concatenate([prior["k16"], step["k16"]]) if base else step["k16"]
    v16 = np.concatenate([prior["v16"], step["v16"]]) if base else step["v16"]
    # inputs of the pass: the raw rows of its columns and the cache rows before it; expected: q, gate, the cache
    # rows the pass writes (the last n of k16 / v16) and the attention output
    out = dict(qraw=d["qraw"], kraw=d["kraw"][base:], vraw=d["vraw"][base:], qw=d["qw"], kw=d["kw"],
               q=step["q"], k16=k16, v16=v16)
    if step["gate"] is not None:
        out["gate"] = step["gate"]
    if q8:
        # int8 caches hold the quantised f32 pre-step outputs (K normed + roped, V raw), not the f16 roundings
        kf = np.asarray(d["kraw"], np.float32).reshape(-1, nKV, hd)
        kf = O.rope_neox(O.head_rmsnorm(kf, d["kw"], cfg["eps"]), np.arange(base + n), cfg["n_rot"], cfg["rope_theta"])
        vf = np.asarray(d["vraw"], np.float32).reshape(-1, nKV, hd)
        kq, ks = O.q8_quantize(kf); vq, vs = O.q8_quantize(vf)
        out.update(kq=kq, ks=ks, vq=vq, vs=vs)
        ref = O.attention_values(step["q"], O.q8_dequantize(kq, ks), O.q8_dequantize(vq, vs), base, gate=step["gate"])
    else:
        ref = O.attention(step["q"], k16, v16, base, gate=step["gate"])
        js = js_attention(cfg, step["q"], k16, v16, step["gate"], base)
        if js is None:
            print("  %s: node not found, JavaScript cross-check skipped" % name)
        else:
            dmax = float(np.abs(js - ref).max()) / max(float(np.abs(ref).max()), 1e-30)
            assert dmax < 2e-5, "%s: the two oracles disagree (%.3e)" % (name, dmax)
            print("  %s: numpy f64 vs reference loops under node: rel %.2e" % (name, dmax))
    out["attn"] = ref.astype(np.float32)
    return out


def main():
    data, meta = {}, []
    for i, (name, cfg, base, n, q8) in enumerate(CASES):
        c = build_case(name, cfg, base, n, q8, seed=0x601D + i)
        for k, v in c.items():
            data["%s.%s" % (name, k)] = v
        meta.append(dict(name=name, cfg=cfg, base_pos=base, n_cols=n, kv_q8=q8))
    data["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "attn_cases.npz")
    np.savez_compressed(path, **data)
    print("wrote %s: %d cases, %.0f KB" % (path, len(meta), os.path.getsize(path) / 1024))


if __name__ == "__main__":
    main()
