#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (metric "decode attn KV-read GB/s @32K ctx"): configuration 3 --
single-token gated decode attention, Qwen3.6-35B-MoE attention shape (16 q heads, 2 kv heads, head_dim 256),
context 32768.  A step is one pass of the hot path for one token on one attention layer: pre-step (q
de-interleave + QK-RMSNorm + partial RoPE + f16 KV write at position 32768), split-K decode kernel, log-sum-exp
merge with the sigmoid gate -- by default through the fused entry point pa_attn_decode_step (--unfused: the three
separate launches).  Consecutive steps walk over distinct layers' caches (as a model does), so the 64 MiB of K/V a
step reads is not resident in the 256 MB last-level cache from the previous step; the step is timed with 6, 12 and 24
layers' caches in rotation and the headline is the smallest rotation past which the time no longer rises.
value = algorithmic KV bytes per step / wall time per step, all inputs resident in HBM.

Every tensor has a random stream of its own (numpy SeedSequence children of one root seed per configuration): cache
rows of each layer, the token's / chunk's q, k, v, the norm weights and the projection weights are independent
N(0,1) draws, and the CPU legs check that (an output far larger than a softmax average over independent rows can be
is an error).

One JSON line on stdout; progress on stderr.
"""
import argparse
import json
import os
import shutil
import struct
import subprocess
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0

C3 = dict(n_heads=16, n_kv_heads=2, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True)
C3_CTX = 32768
ROTATIONS = (6, 12, 24)   # layers' caches in rotation: 384 MiB, 768 MiB, 1.5 GiB of K/V against a 256 MB last-level cache
N_LAYERS = max(ROTATIONS)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def streams(root_seed, *names):
    """Independent random generators, one per named role, from one root seed (SeedSequence children)."""
    kids = np.random.SeedSequence(root_seed).spawn(len(names))
    return {n: np.random.default_rng(k) for n, k in zip(names, kids)}


def host_description():
    """The host CPU the baseline legs run on: model name, logical CPUs, CPUs this process may run on."""
    model = "unknown"
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.lower().startswith("model name"):
                model = ln.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        usable = os.cpu_count()
    return dict(cpu_model=model, logical_cpus=os.cpu_count(), usable_cpus=usable)


def check_independent(what, ref_out, diff):
    """The CPU legs' self-check: with independent N(0,1) rows the attention output is an average over tens of thousands
    of value rows (|out| of a few hundredths); an output of order 1 means the query collided with cache rows."""
    mx = float(np.abs(ref_out).max())
    rel = diff / max(mx, 1e-30)
    log("%s: max|ref| = %.4f, max|gpu - cpu| = %.3e, relative %.3e" % (what, mx, diff, rel))
    if not (mx <= 0.5):
        raise RuntimeError("%s: max|ref| = %.3f > 0.5 -- the benchmark inputs are not independent N(0,1) draws" % (what, mx))
    if not (diff <= 2e-3 and rel <= 1e-2):
        raise RuntimeError("%s: GPU and CPU reference differ: max-abs %.3e, relative %.3e" % (what, diff, rel))
    return mx, rel


def fill_cache(pa, cfg, layer, ctx, rng, chunk):
    """Write cache rows [0, ctx) of one layer by running the library's own pre-step on N(0,1) k / v drawn from rng."""
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    qin = cfg["n_heads"] * cfg["head_dim"] * (2 if cfg.get("gate") else 1)
    qw = pa.to_device(np.ones(cfg["head_dim"], np.float32)); kw = pa.to_device(np.ones(cfg["head_dim"], np.float32))
    dq = pa.to_device(np.zeros((chunk, qin), np.float32) + 0.5)
    dk = pa.alloc(chunk * kvd * 4); dv = pa.alloc(chunk * kvd * 4)
    for t0 in range(0, ctx, chunk):
        n = min(chunk, ctx - t0)
        dk.upload(rng.standard_normal((n, kvd), dtype=np.float32)); dv.upload(rng.standard_normal((n, kvd), dtype=np.float32))
        pa.glue_kv(layer, dq, qin, dk, kvd, dv, kvd, qw, kw, t0, n)
    pa.sync()
    for b in (qw, kw, dq, dk, dv):
        b.free(); pa._bufs.remove(b)


def run_reference_js(header, sel, q, k16, v16, gate, reps, timeout):
    """oracle/attn_ref.js (the reference's CPU loops, one thread) on the given tensors -> (out f32, info dict)."""
    node = shutil.which("node")
    if node is None:
        raise RuntimeError("node not found")
    with tempfile.TemporaryDirectory() as td:
        inp, outp = os.path.join(td, "in.bin"), os.path.join(td, "out.bin")
        with open(inp, "wb") as f:
            f.write(struct.pack("8i", *header))
            f.write(np.asarray(sel, np.int32).tobytes()); f.write(q.astype(np.float32).tobytes())
            f.write(k16.tobytes()); f.write(v16.tobytes()); f.write(gate.astype(np.float32).tobytes())
        r = subprocess.run([node, os.path.join(ROOT, "oracle", "attn_ref.js"), inp, outp, str(reps)], capture_output=True, text=True, timeout=timeout)
        if r.returncode != 0:
            raise RuntimeError("attn_ref.js failed: " + r.stderr[-500:])
        info = json.loads(r.stdout.strip().splitlines()[-1])
        out = np.fromfile(outp, dtype=np.float32)
    return out, info


def cpu_baseline_c3(pa, cfg, ctx, q, gate, gpu_out):
    """The reference's CPU attention loops (JavaScript restatement, one thread) on the same column: reads the
    layer-0 cache back from HBM, times node oracle/attn_ref.js, and compares its output with the GPU's."""
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rows = ctx + 1
    k16 = pa.kv_read(0, 0, 0, rows); v16 = pa.kv_read(0, 1, 0, rows)
    kv_bytes = 2 * rows * nKV * hd * 2
    host = host_description()
    if shutil.which("node") is None:
        from oracle import c_oracle
        K = k16.view(np.float16).astype(np.float32).reshape(rows, -1); V = v16.view(np.float16).astype(np.float32).reshape(rows, -1)
        out = np.zeros(nH * hd, np.float32)
        qf = np.ascontiguousarray(q.reshape(-1)); gf = np.ascontiguousarray(gate.reshape(-1))
        t0 = time.perf_counter()
        c_oracle.lib().pa_oracle_attention_ref_loops(qf.ctypes.data, K.ctypes.data, V.ctypes.data, rows, nH, nKV, hd, gf.ctypes.data, out.ctypes.data)
        ms = (time.perf_counter() - t0) * 1e3
        sample, extra = "full C3 column, 1 rep, C restatement of the reference loops (node not found), 1 thread", {}
    else:
        reps = 4
        out, info = run_reference_js((1, nH, nKV, hd, ctx, rows, 1, 1), [0], q, k16, v16, gate, reps, 300)
        ms = info["ms"]
        sample = "full C3 column (1 token over 32769 rows), best of %d reps, node %s, 1 thread" % (reps, info["node"])
        extra = dict(max_softmax_weight=info.get("max_weight"), node_os_cpus=info.get("cpus"), node_cpu_model=info.get("cpu_model"))
    diff = float(np.abs(out - gpu_out.reshape(-1)).max())
    mx, rel = check_independent("C3 cpu baseline", out, diff)
    return dict(value=kv_bytes / (ms / 1e3) / 1e9, unit="GB/s", cores=1, kind="port", sample=sample, ms=ms, host=host,
                max_abs_ref=mx, max_abs_diff_vs_gpu=diff, rel_diff_vs_gpu=rel, **extra)


C5 = dict(n_heads=16, n_kv_heads=2, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True)
C5_BASE, C5_COLS = 126976, 4096
PREFILL_WARMUP = 3


def causal_flops(cfg, base, n):
    """QK^T and PV multiply-adds of the causal chunk, masked-out work not counted: 4 nH hd sum_c (base + c + 1)."""
    return 4.0 * cfg["n_heads"] * cfg["head_dim"] * (n * base + n * (n + 1) // 2)


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def prefill_leg(steps, with_cpu, kv_q8=False):
    """Configuration 5: a 4096-token causal chunk at positions 126976-131071 over a 126976-token f16 prefix,
    Qwen3.6-35B-MoE attention shape, sigmoid gate, f16 output.  A step = pre-step for the 4096 columns
    (QK-RMSNorm + partial RoPE + KV write) + the MFMA prefill kernel.  PREFILL_WARMUP untimed steps (the first one's
    time is kept as cold_first_ms), then `steps` steps timed one by one; the MEDIAN step and kernel times are
    reported (the shader clock takes several launches to settle after idle, so a mean over the first few is a ramp)."""
    from pooled_amd.capi import PooledAttn, PA_OUT_F16
    cfg, base, n = dict(C5, kv_q8=True) if kv_q8 else C5, C5_BASE, C5_COLS
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = nH * hd, nKV * hd
    steps = max(steps, 10)
    rs = streams(0x5EED0005, "cache", "q", "k", "v", "norm", "weights", "x")
    pa = PooledAttn(cfg, base + n, n_layers=1, max_cols=n)
    pa.layer_alloc(0)
    fill_cache(pa, cfg, 0, base, rs["cache"], chunk=4096)
    d_qfull = pa.to_device(rs["q"].standard_normal((n, 2 * qd), dtype=np.float32))
    d_k = pa.to_device(rs["k"].standard_normal((n, kvd), dtype=np.float32)); d_v = pa.to_device(rs["v"].standard_normal((n, kvd), dtype=np.float32))
    d_qw = pa.to_device((1 + 0.1 * rs["norm"].standard_normal(hd)).astype(np.float32)); d_kw = pa.to_device((1 + 0.1 * rs["norm"].standard_normal(hd)).astype(np.float32))
    d_out = pa.alloc(n * qd * 2)
    gate_ptr = pa.gate_buffer_ptr()

    def step():
        pa.glue_kv(0, d_qfull, 2 * qd, d_k, kvd, d_v, kvd, d_qw, d_kw, base, n)
        pa.attn("prefill", 0, None, 0, gate_ptr, qd, base, n, d_out, qd, PA_OUT_F16)

    def timed_step():
        pa.timer_start(); step()
        return pa.timer_stop()                       # blocks until the step has finished

    pa.sync()
    cold_first_ms = timed_step()
    for _ in range(PREFILL_WARMUP - 1):
        timed_step()
    pa.profile_enable(True)
    step_ms = [timed_step() for _ in range(steps)]
    kern_ms = pa.profile_read_each()
    pa.profile_enable(False)
    ms_step, k_ms = median(step_ms), median(kern_ms)
    k_mean = sum(kern_ms) / max(len(kern_ms), 1)
    flops = causal_flops(cfg, base, n)
    tf_step, tf_kernel = flops / (ms_step * 1e-3) / 1e12, flops / (k_ms * 1e-3) / 1e12
    log("prefill C5: first launch %.3f ms; median of %d steps %.3f ms (min %.3f, max %.3f) -> %.1f TFLOP/s; kernel median %.3f ms (mean %.3f) -> %.1f TFLOP/s (%.1f%% of f16 MFMA peak)"
        % (cold_first_ms, steps, ms_step, min(step_ms), max(step_ms), tf_step, k_ms, k_mean, tf_kernel, 100 * tf_kernel / MFMA_F16_PEAK_TFLOPS))
    res = dict(workload="C5 causal chunked prefill: 4096 columns at positions 126976-131071 over a 126976-token %s prefix, 16q/2kv heads, head_dim 256, partial RoPE, sigmoid gate, f16 out; "
                        "every tensor an independent N(0,1) stream" % ("int8 (widened once per chunk into an f16 staging cache, inside the step)" if kv_q8 else "f16"),
               value=round(tf_step, 1), unit="TFLOP/s", ms_per_step=round(ms_step, 4), steps=steps, warmup=PREFILL_WARMUP, reported="median of the timed steps",
               min_ms_per_step=round(min(step_ms), 4), max_ms_per_step=round(max(step_ms), 4), cold_first_ms=round(cold_first_ms, 4),
               step_ms=[round(x, 3) for x in step_ms], flops_per_step=flops, plan=pa.plan("prefill", base, n),
               roofline=dict(bound="mfma", achieved=round(tf_kernel, 1), peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s", frac=round(tf_kernel / MFMA_F16_PEAK_TFLOPS, 4),
                             traffic=None, kernel="pa_prefill_kernel<256, 1, 8>", kernel_ms=round(k_ms, 4), kernel_ms_mean=round(k_mean, 4),
                             kernel_ms_min=round(min(kern_ms), 4), kernel_ms_max=round(max(kern_ms), 4), reported="median launch",
                             algorithmic_flops_per_launch=flops, launches=len(kern_ms)))
    if with_cpu:
        # CPU leg: the reference loops on a fixed subsample (all 16 heads of 4 evenly spaced columns), scaled by
        # columns; labelled extrapolated
        sel = np.array([0, n // 3, 2 * n // 3, n - 1], np.int32)
        rows = base + n
        q = pa.read_q_buffer(n); gate = pa.read_gate_buffer(n)
        gpu = d_out.download(np.float16, n * qd).reshape(n, qd)[sel].astype(np.float32)
        k16 = pa.kv_read(0, 0, 0, rows); v16 = pa.kv_read(0, 1, 0, rows)
        try:
            out, info = run_reference_js((n, nH, nKV, hd, base, rows, 1, len(sel)), sel, q, k16, v16, gate, 1, 600)
        except Exception as e:                       # the baseline is a reported figure; a missing node must not sink the GPU line
            res["cpu_baseline"] = dict(value=None, unit="TFLOP/s", cores=1, kind="port", sample="failed: %s" % e, host=host_description())
        else:
            out = out.reshape(len(sel), qd)
            sub_flops = 4.0 * nH * hd * sum(base + int(c) + 1 for c in sel)
            diff = float(np.abs(out - gpu).max())
            mx, rel = check_independent("C5 cpu baseline", out, diff)      # raises on collided inputs or a wrong result
            res["cpu_baseline"] = dict(value=sub_flops / (info["ms"] * 1e-3) / 1e12, unit="TFLOP/s", cores=1, kind="port",
                                       sample="4 of 4096 columns x 16 heads (%.2f GFLOP), 1 rep, node %s, 1 thread; whole chunk extrapolates to %.0f s" % (sub_flops / 1e9, info["node"], info["ms"] * 1e-3 * flops / sub_flops),
                                       ms=info["ms"], host=host_description(), node_os_cpus=info.get("cpus"), node_cpu_model=info.get("cpu_model"),
                                       max_softmax_weight=info.get("max_weight"), max_abs_ref=mx, max_abs_diff_vs_gpu=diff, rel_diff_vs_gpu=rel)
            log("prefill cpu baseline: %.0f ms for %.2f GFLOP -> %.5f TFLOP/s" % (info["ms"], sub_flops / 1e9, res["cpu_baseline"]["value"]))
    # the whole attention half of a layer for the same chunk: rmsnorm + [q|k|v] GEMM + pre-step + attention + wo GEMM
    try:
        from pooled_amd.capi import PA_W_Q4_0
        dim, rows_qkv = 2048, 2 * qd + 2 * kvd
        rng = rs["weights"]

        def mk(d_out, d_in):
            sc = np.asarray(rng.uniform(0.001, 0.003, (d_out, d_in // 32)), np.float16).view(np.uint16)
            return pa.weight(PA_W_Q4_0, rng.integers(0, 256, (d_out, d_in // 2), dtype=np.uint8), sc)
        wq, wo = mk(rows_qkv, dim), mk(dim, qd)
        d_x = pa.to_device(rs["x"].standard_normal((n, dim), dtype=np.float32))
        d_nw = pa.to_device((1 + 0.1 * rs["norm"].standard_normal(dim)).astype(np.float32))
        d_x16 = pa.to_device(rs["x"].standard_normal((n, dim)).astype(np.float16).view(np.uint16))
        d_y = pa.alloc(n * rows_qkv * 4)

        def timed(f, reps):
            f(); pa.sync()
            pa.timer_start()
            for _ in range(reps):
                f()
            return pa.timer_stop() / reps
        t_g1 = timed(lambda: pa.gemm(wq, d_x16, dim, n, d_y, rows_qkv), 10)
        t_g2 = timed(lambda: pa.gemm(wo, d_out, qd, n, d_x, dim, acc=True), 10)
        d_x.upload(rs["x"].standard_normal((n, dim), dtype=np.float32))
        t_layer = timed(lambda: pa.attn_layer_prefill(0, wq, wo, d_nw, d_qw, d_kw, d_x, dim, base, n), max(2, steps // 2))
        f1, f2 = 2.0 * n * rows_qkv * dim, 2.0 * n * dim * qd
        log("prefill layer: [q|k|v] GEMM %.3f ms (%.0f TFLOP/s), wo GEMM %.3f ms (%.0f TFLOP/s), whole attention half %.3f ms" % (t_g1, f1 / t_g1 / 1e9, t_g2, f2 / t_g2 / 1e9, t_layer))
        res["layer_prefill"] = dict(workload="the same chunk through the attention half of a layer (engine/qwen35.js:2416-2425): rmsnorm -> f16, [q|k|v] GEMM "
                                             "%dx%dx%d, pre-step, causal attention, wo GEMM %dx%dx%d accumulated into the residual; Q4_0 weights, f16 operands" % (n, rows_qkv, dim, n, dim, qd),
                                    ms_per_step=round(t_layer, 4), tflops=round((flops + f1 + f2) / (t_layer * 1e-3) / 1e12, 1),
                                    gemm_qkv=dict(ms=round(t_g1, 4), tflops=round(f1 / t_g1 / 1e9, 1)), gemm_o=dict(ms=round(t_g2, 4), tflops=round(f2 / t_g2 / 1e9, 1)))
    except Exception as e:                       # a reported extra; never let it sink the headline legs
        log("prefill layer leg failed:", e)
    pa.close()
    return res


def other_configs():
    """Configurations 1, 2 and 4 of the baseline (parity-test cases, not bench lines): steady-state time per call on
    caches in rotation, printed for the record."""
    from pooled_amd.capi import PooledAttn, PA_OUT_F16
    dense = dict(n_heads=16, n_kv_heads=8, head_dim=128, n_rot=128, rope_theta=1e6, eps=1e-6, qk_norm=True, gate=False)
    b27 = dict(n_heads=24, n_kv_heads=4, head_dim=256, n_rot=64, rope_theta=1e7, eps=1e-6, qk_norm=True, gate=True)
    out = {}
    for name, cfg, kind, base, n, layers in (("C1", dense, "decode", 2048, 1, 8), ("C2", dense, "prefill", 1536, 512, 8),
                                             ("C4", b27, "decode", 65536, 8, 3)):
        nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
        qd, kvd = nH * hd, nKV * hd
        pa = PooledAttn(cfg, base + n, n_layers=layers, max_cols=4096)
        rs = streams(0x5EED0100 + int(name[1]), "q", "gate", "weights", "x", *["cache%d" % l for l in range(layers)])
        for l in range(layers):
            pa.layer_alloc(l)
            fill_cache(pa, cfg, l, base + n, rs["cache%d" % l], chunk=4096)
        dq = pa.to_device(rs["q"].standard_normal((n, qd), dtype=np.float32))
        dg = pa.to_device(rs["gate"].standard_normal((n, qd), dtype=np.float32)) if cfg["gate"] else None
        dout = pa.alloc(n * qd * 2)
        call = lambda i: pa.attn(kind, i % layers, dq, qd, dg, qd if dg else 0, base, n, dout, qd, PA_OUT_F16)
        # the median of five windows after one discarded window: the first 10 - 20 ms after the cache fill run at a
        # lower clock (C4: 62 us in the first window, 58.7 - 59.1 us from the second on)
        reps, wins = 200, []
        for w in range(6):
            pa.sync()
            pa.timer_start()
            for i in range(reps):
                call(i)
            wins.append(pa.timer_stop() / reps)
        ms = sorted(wins[1:])[2]
        kv = 2 * (base + n) * kvd * 2
        fl = causal_flops(cfg, base, n)
        out[name] = dict(us_per_call=round(ms * 1e3, 2), windows_us=[round(w * 1e3, 2) for w in wins], kv_gb_s=round(kv / ms / 1e6, 1), tflops=round(fl / ms / 1e9, 2), plan=pa.plan(kind, base, n))
        log("%s: %.2f us/call, %.0f GB/s of KV, %.2f TFLOP/s" % (name, ms * 1e3, kv / ms / 1e6, fl / ms / 1e9))
        if name == "C2":
            # the same chunk through the attention half of a layer (projections either side), one weight set per layer
            from pooled_amd.capi import PA_W_Q4_0
            dim = 2048
            rng = rs["weights"]

            def mk(d_out, d_in):
                sc = np.asarray(rng.uniform(0.001, 0.003, (d_out, d_in // 32)), np.float16).view(np.uint16)
                return pa.weight(PA_W_Q4_0, rng.integers(0, 256, (d_out, d_in // 2), dtype=np.uint8), sc)
            ws = [(mk(qd + 2 * kvd, dim), mk(dim, qd)) for _ in range(layers)]
            d_x = pa.to_device(rs["x"].standard_normal((n, dim), dtype=np.float32) * 0.1)
            d_nw = pa.to_device(np.ones(dim, np.float32)); d_hw = pa.to_device(np.ones(hd, np.float32))
            lcall = lambda i: pa.attn_layer_prefill(i % layers, ws[i % layers][0], ws[i % layers][1], d_nw, d_hw, d_hw, d_x, dim, base, n)
            for i in range(layers + 2):
                lcall(i)
            pa.sync(); pa.timer_start()
            for i in range(100):
                lcall(i)
            lms = pa.timer_stop() / 100
            out[name]["layer_us_per_call"] = round(lms * 1e3, 2)
            log("C2 through the attention half of a layer (rmsnorm, [q|k|v] GEMM %dx%dx%d, pre-step, attention, wo GEMM %dx%dx%d): %.2f us/call" % (n, qd + 2 * kvd, dim, n, dim, qd, lms * 1e3))
        pa.close()
    return out


def layer_leg(pa, cfg, ctx, steps, warmup, attn_ms, n_rot, rng):
    """The attention half of a layer for one token, projections included (pa_attn_layer_decode: normed [q | k | v]
    GEMV, fused decode step, accumulating output GEMV; Q4_0 weights of the MoE model's shape, a set per layer and
    three sets in rotation so that weights and caches come from HBM), and the two GEMVs on their own."""
    from pooled_amd.capi import PA_W_Q4_0
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd, dim = nH * hd, nKV * hd, 2048
    rows_qkv = 2 * qd + 2 * kvd

    def mk(d_out, d_in):
        sc = np.asarray(rng.uniform(0.001, 0.003, (d_out, d_in // 32)), np.float16).view(np.uint16)
        return pa.weight(PA_W_Q4_0, rng.integers(0, 256, (d_out, d_in // 2), dtype=np.uint8), sc)
    n_sets = 18
    wq = [mk(rows_qkv, dim) for _ in range(n_sets)]
    wo = [mk(dim, qd) for _ in range(n_sets)]
    d_x = pa.to_device(rng.standard_normal(dim).astype(np.float32))
    d_nw = pa.to_device((1 + 0.1 * rng.standard_normal(dim)).astype(np.float32))
    d_hw = pa.to_device((1 + 0.1 * rng.standard_normal(hd)).astype(np.float32))
    d_y = pa.alloc(rows_qkv * 4)
    d_a = pa.to_device((rng.standard_normal(qd) * 0.01).astype(np.float32))
    steps, warmup = max(steps, 200), max(warmup, 20)

    def timed(f):
        for i in range(warmup):
            f(i)
        pa.sync()
        pa.timer_start()
        for i in range(steps):
            f(i)
        return pa.timer_stop() / steps
    t_qkv = timed(lambda i: pa.gemv_norm(wq[i % n_sets], d_x, d_nw, d_y))
    t_o = timed(lambda i: pa.gemv(wo[i % n_sets], d_a, d_x, acc=True))
    d_x.upload(rng.standard_normal(dim).astype(np.float32))
    t_layer = timed(lambda i: pa.attn_layer_decode(i % n_rot, wq[i % n_sets], wo[i % n_sets], d_nw, d_hw, d_hw, d_x, ctx))
    b_qkv = rows_qkv * dim // 2 + rows_qkv * (dim // 32) * 2
    b_o = dim * qd // 2 + dim * (qd // 32) * 2
    kv_bytes = 2 * (ctx + 1) * kvd * 2
    log("layer: [q|k|v] GEMV %.2f us, wo GEMV %.2f us, whole attention half %.2f us" % (t_qkv * 1e3, t_o * 1e3, t_layer * 1e3))
    # a speculative-verify block of 8 tokens through the same half of the layer (column-batched call, engine/qwen35.js:2416-2425)
    nv = 8
    d_xv = pa.to_device(rng.standard_normal((nv, dim)).astype(np.float32))
    t_verify = timed(lambda i: pa.attn_layer_prefill(i % n_rot, wq[i % n_sets], wo[i % n_sets], d_nw, d_hw, d_hw, d_xv, dim, ctx - nv + 1, nv))
    log("layer, verify block of %d tokens: %.2f us" % (nv, t_verify * 1e3))
    return dict(workload="one token through the attention half of a full-attention layer (engine/qwen35.js:1586-1641): rmsnorm + [q|k|v] "
                         "GEMV %dx%d, pre-step + split-K attention over %d rows + merge/gate, wo GEMV %dx%d accumulated into the residual; "
                         "Q4_0 weights, 4 launches; %d weight sets and %d layers' caches in rotation (cold HBM); %d timed steps" % (rows_qkv, dim, ctx, dim, qd, n_sets, n_rot, steps),
                us_per_step=round(t_layer * 1e3, 2), attention_us=round(attn_ms * 1e3, 2),
                gemv_qkv_norm=dict(us=round(t_qkv * 1e3, 2), weight_bytes=b_qkv, gbs=round(b_qkv / t_qkv / 1e6, 1)),
                gemv_o_acc=dict(us=round(t_o * 1e3, 2), weight_bytes=b_o, gbs=round(b_o / t_o / 1e6, 1)),
                bytes_per_step=kv_bytes + b_qkv + b_o, gbs=round((kv_bytes + b_qkv + b_o) / t_layer / 1e6, 1),
                pct_hbm_peak=round(100 * (kv_bytes + b_qkv + b_o) / t_layer / 1e6 / HBM_PEAK_GBS, 2),
                verify_block=dict(workload="%d tokens at positions %d .. %d through the same half of the layer (pa_attn_layer_prefill: rmsnorm, skinny-chunk "
                                           "projections, pre-step, split-K attention in column groups, merge/gate)" % (nv, ctx - nv + 1, ctx),
                                  us_per_step=round(t_verify * 1e3, 2), us_per_token=round(t_verify * 1e3 / nv, 2)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=600)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill (configuration 5) leg")
    ap.add_argument("--unfused", action="store_true", help="decode step as three launches (pa_glue_kv + pa_attn_decode) instead of the fused pa_attn_decode_step")
    ap.add_argument("--prefill-steps", type=int, default=12, help="timed prefill steps after %d warm-up steps (at least 10); the median is reported" % PREFILL_WARMUP)
    ap.add_argument("--kv-q8", action="store_true", help="run the C3 decode step on int8 caches (one f32 scale per 32 values) instead of f16")
    ap.add_argument("--no-layer", action="store_true", help="skip the whole-layer leg (projections + attention, pa_attn_layer_decode)")
    ap.add_argument("--other-configs", action="store_true", help="only time configurations 1, 2 and 4 (attention call alone, caches in rotation)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run 10 device-to-device copies of 256 MiB (the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--rotation", type=int, default=0, help="time the decode step with this many layers' caches in rotation only (default: sweep %s)" % (ROTATIONS,))
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from pooled_amd.capi import PooledAttn, PA_OUT_F16, load
    L = load()
    log("library:", L.pa_version().decode())
    if args.other_configs:
        print(json.dumps({"other_configs": other_configs()}))
        return
    if args.copy_calibration:
        pa = PooledAttn(C3, 64, n_layers=1, max_cols=1)
        nbytes = 256 << 20
        src, dst = pa.alloc(nbytes), pa.alloc(nbytes)
        src.upload(np.zeros(nbytes // 4, np.float32))
        for _ in range(10):
            pa.copy_d2d(dst, src, nbytes)
        pa.sync()
        pa.close()
        print(json.dumps({"copy_calibration": {"bytes_per_copy": nbytes, "copies": 10}}))
        return
    cfg, ctx = C3, C3_CTX
    if args.kv_q8:
        cfg = dict(C3, kv_q8=True); args.no_cpu = True
    nH, nKV, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    qd, kvd = nH * hd, nKV * hd
    rotations = (args.rotation,) if args.rotation else ROTATIONS
    n_layers = max(rotations)
    rs = streams(0x5EED0003, "q", "k", "v", "norm", "weights", *["cache%d" % l for l in range(n_layers)])
    pa = PooledAttn(cfg, ctx + 1, n_layers=n_layers, max_cols=4096)
    t_fill = time.time()
    for layer in range(n_layers):
        pa.layer_alloc(layer)
        fill_cache(pa, cfg, layer, ctx, rs["cache%d" % layer], chunk=4096)
    log("caches filled: %d layers x %.1f MiB in %.1fs" % (n_layers, 2 * ctx * kvd * 2 / 2**20, time.time() - t_fill))

    qfull = rs["q"].standard_normal((1, 2 * qd), dtype=np.float32)
    knew = rs["k"].standard_normal((1, kvd), dtype=np.float32); vnew = rs["v"].standard_normal((1, kvd), dtype=np.float32)
    qw = (1 + 0.1 * rs["norm"].standard_normal(hd)).astype(np.float32); kw = (1 + 0.1 * rs["norm"].standard_normal(hd)).astype(np.float32)
    d_qfull, d_k, d_v, d_qw, d_kw = (pa.to_device(a) for a in (qfull, knew, vnew, qw, kw))
    d_out = pa.alloc(qd * 2)
    gate_ptr = pa.gate_buffer_ptr()

    def step(i, n_rot):
        layer = i % n_rot
        if args.unfused:
            pa.glue_kv(layer, d_qfull, 2 * qd, d_k, kvd, d_v, kvd, d_qw, d_kw, ctx, 1)
            pa.attn("decode", layer, None, 0, gate_ptr, qd, ctx, 1, d_out, qd, PA_OUT_F16)
        else:
            pa.attn_decode_step(layer, d_qfull, d_k, d_v, d_qw, d_kw, ctx, d_out, PA_OUT_F16)

    kv_bytes = 2 * (ctx + 1) * kvd * 2            # K and V rows [0, 32768], f16
    if args.kv_q8:
        kv_bytes = 2 * (ctx + 1) * (kvd + kvd // 32 * 4)          # int8 values + one f32 scale per 32

    def window(n_rot):
        """EXACTLY args.steps steps between two synchronisations, on two clocks: a HIP event pair on the launch stream
        around the steps (what the GPU spent on them: the reported figure) and the host clock around the same region,
        which adds the host thread's wake-up after the closing synchronisation (about 10 us a window: half a
        microsecond a step at 20 steps, nothing at 500)."""
        pa.sync()
        t0 = time.perf_counter()
        pa.timer_start()
        for i in range(args.steps):
            step(i, n_rot)
        gpu_ms = pa.timer_stop()                       # blocks until the last step has finished
        wall_ms = (time.perf_counter() - t0) * 1e3
        host_windows.setdefault(n_rot, []).append(wall_ms / args.steps)
        return gpu_ms / args.steps

    # A window of a few hundred 20-microsecond steps is short against the box's noise (clock ramps, the host thread
    # being descheduled): the window is repeated and the median window is the reported ms_per_step.  The same is done
    # for every rotation size; the headline is the smallest rotation that no larger one exceeds by more than 1 %.
    n_windows = max(5, min(25, -(-3000 // max(args.steps, 1))))
    sweep, host_windows = {}, {}
    for n_rot in rotations:
        for i in range(max(args.warmup, 2 * n_rot)):
            step(i, n_rot)
        ws = sorted(window(n_rot) for _ in range(n_windows))
        sweep[n_rot] = ws
        log("%2d layers in rotation (%4.0f MiB of K/V): %d windows of %d steps: median %.2f us/step (min %.2f, max %.2f); host clock median %.2f"
            % (n_rot, n_rot * 2 * ctx * kvd * 2 / 2**20, n_windows, args.steps, ws[len(ws) // 2] * 1e3, ws[0] * 1e3, ws[-1] * 1e3, median(host_windows[n_rot]) * 1e3))
    med = {r: sweep[r][len(sweep[r]) // 2] for r in rotations}
    n_rot = next(r for r in rotations if all(med[r2] <= 1.01 * med[r] for r2 in rotations if r2 > r))
    windows = sweep[n_rot]
    ms_per_step = med[n_rot]
    value = kv_bytes / (ms_per_step * 1e-3) / 1e9
    log("headline: %d layers in rotation: %.2f us/step -> %.0f GB/s" % (n_rot, ms_per_step * 1e3, value))

    # the dominant kernel alone: one HIP event pair around every split-K launch, stamped by the dispatch on the launch stream
    n_k = max(args.steps, 240)
    for i in range(2 * n_rot):
        step(i, n_rot)
    pa.profile_enable(True)
    for i in range(n_k):
        step(i, n_rot)
    kern = pa.profile_read_each()
    pa.profile_enable(False)
    k_ms = sum(kern) / max(len(kern), 1)             # the average launch, as a kernel trace's statistics report it
    k_med = median(kern)
    achieved = kv_bytes / (k_ms * 1e-3) / 1e9
    # HBM bytes per launch are not measured in this run: they come from two rocprofv3 --pmc runs of this same command
    # (FETCH_SIZE, WRITE_SIZE) whose summary is committed; the line names the file and the commit it was taken at
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "decode_c3_traffic.json")
    if os.path.exists(tpath) and not args.kv_q8 and not args.unfused:      # measured for the default (fused, f16) kernel
        tj = json.load(open(tpath))
        traffic = tj.get("hbm_bytes_per_launch")
        traffic_source = "profiles/decode_c3_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, measured at commit %s; not re-measured by this run)" % tj.get("head", "unknown")
    plan = pa.plan("decode", ctx, 1)
    kname = pa_decode_kernel_name(plan, args)
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(achieved / HBM_PEAK_GBS, 4),
                    traffic=traffic, traffic_source=traffic_source, kernel=kname, kernel_us=round(k_ms * 1e3, 3), kernel_us_median=round(k_med * 1e3, 3),
                    kernel_us_min=round(min(kern) * 1e3, 3), reported="mean launch (dispatch-stamped HIP events; the step's merge launch is stamped too, as every dispatch is in a kernel trace)",
                    algorithmic_bytes_per_launch=kv_bytes, launches=len(kern), layers_in_rotation=n_rot)
    log("split-K kernel: mean %.2f us/launch (median %.2f) over %d launches -> %.0f GB/s (%.1f%% of 8 TB/s)" % (k_ms * 1e3, k_med * 1e3, len(kern), achieved, 100 * achieved / HBM_PEAK_GBS))

    # for the record, the same step on ONE layer's caches, which stay in the 256 MB last-level cache between steps:
    # what the kernel does when HBM is not in the way (never the reported value)
    for i in range(20):
        step(i, 1)
    pa.sync(); pa.timer_start()
    for i in range(200):
        step(i, 1)
    warm_ms = pa.timer_stop() / 200
    log("warm (one layer's caches, resident in the last-level cache): %.2f us/step -> %.0f GB/s" % (warm_ms * 1e3, kv_bytes / warm_ms / 1e6))

    cpu = None
    if not args.no_cpu:
        # GPU output of layer 0 for this token (f32), then the reference CPU loops on the same inputs
        d_o32 = pa.alloc(qd * 4)
        pa.glue_kv(0, d_qfull, 2 * qd, d_k, kvd, d_v, kvd, d_qw, d_kw, ctx, 1)
        pa.attn("decode", 0, None, 0, gate_ptr, qd, ctx, 1, d_o32, qd)
        pa.sync()
        gpu_out = d_o32.download(np.float32, qd)
        q = pa.read_q_buffer(1); gate = pa.read_gate_buffer(1)
        cpu = cpu_baseline_c3(pa, cfg, ctx, q, gate, gpu_out)        # raises on collided inputs or a wrong result
        log("cpu baseline: %.1f ms -> %.3f GB/s" % (cpu["ms"], cpu["value"]))

    line = dict(
        metric="decode attn KV-read GB/s (% HBM peak) @32K ctx; prefill attn TFLOP/s (% MFMA)",
        value=round(value, 1), unit="GB/s", n_gpus=1, steps=args.steps, warmup=args.warmup,
        ms_per_step=round(ms_per_step, 6), windows=dict(count=n_windows, steps_each=args.steps, reported="median", clock="HIP event pair on the launch stream around the steps of a window, synchronised on both sides",
                                                         min_ms_per_step=round(windows[0], 6), max_ms_per_step=round(windows[-1], 6),
                                                         host_clock_median_ms_per_step=round(median(host_windows[n_rot]), 6)),
        higher_is_better=True, scaling="weak", vs_baseline=None,
        dtype="f16 (int8 cache widened to f16)" if args.kv_q8 else "f16", data="synthetic",
        config=dict(workload="C3 gated decode: 16q/2kv heads, head_dim 256, ctx 32768, 1 token, %s KV," % ("int8 (f32 scale per 32)" if args.kv_q8 else "f16") + " partial RoPE 64 dims theta 1e7, sigmoid gate, f16 out; every tensor an independent N(0,1) stream",
                    step="%s on one layer; %d layers' caches in rotation (cold HBM: the smallest rotation of the sweep that no larger one exceeds by more than 1 %%)"
                         % ("pa_glue_kv + pa_attn_decode (pre-step, split-K decode, LSE merge/gate: 3 launches)" if args.unfused else "pa_attn_decode_step (pre-step fused into the split-K decode kernel + LSE merge/gate: 2 launches)", n_rot),
                    rotation_sweep={str(r): dict(kv_mib_in_rotation=round(r * 2 * ctx * kvd * 2 / 2**20), us_per_step=round(med[r] * 1e3, 3), min_us=round(sweep[r][0] * 1e3, 3),
                                                 max_us=round(sweep[r][-1] * 1e3, 3), gbs=round(kv_bytes / med[r] / 1e6, 1)) for r in rotations},
                    layers_in_rotation=n_rot, kv_bytes_per_step=kv_bytes, plan=plan, pct_hbm_peak=round(100 * value / HBM_PEAK_GBS, 2),
                    warm_cache=dict(note="one layer's caches repeated: served from the 256 MB last-level cache, not HBM; for the record only", us_per_step=round(warm_ms * 1e3, 2), gbs=round(kv_bytes / warm_ms / 1e6, 1))),
        roofline=roofline, cpu_baseline=cpu)
    if not args.no_layer and not args.kv_q8 and not args.unfused:
        line["layer_decode"] = layer_leg(pa, cfg, ctx, args.steps, args.warmup, ms_per_step, n_rot, rs["weights"])
    pa.close()
    if not args.no_prefill:
        line["prefill"] = prefill_leg(args.prefill_steps, not args.no_cpu, args.kv_q8)
    print(json.dumps(line), flush=True)


def pa_decode_kernel_name(plan, args):
    """Template arguments: head_dim, row blocks, waves, fused pre-step, gather, int8 caches, single-round splits."""
    return "pa_decode_kernel<256, 1, 4, %s, false, %s, %s>" % ("false" if args.unfused else "true", "true" if args.kv_q8 else "false",
                                                               "true" if plan["split_len"] == 128 and plan["row_blocks"] == 1 else "false")


if __name__ == "__main__":
    main()
