"""Builds the gfx950 shared library (C ABI of include/pooled_attn.h) and, optionally, the Node-API addon.

    python -m pooled_amd.build            # libpooled_attn.so (+ addon when node headers are present)
"""
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "pooled_amd", "csrc")
LIBDIR = os.path.join(ROOT, "pooled_amd", "lib")
LIB = os.path.join(LIBDIR, "libpooled_attn.so")
ADDON = os.path.join(LIBDIR, "pooled_attn.node")

HIP_SOURCES = ["pa_api.hip", "glue_kv.hip", "attn_decode.hip", "attn_prefill.hip", "proj_gemv.hip", "proj_gemm.hip", "proj_gemm_wide.hip", "stream_probe.hip"]
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
               # packed-FP32 VALU forms are kept off for all device code
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # the first twelve dwords of a kernel's leading scalar / pointer arguments arrive in scalar registers at wave start
               "-mllvm", "-amdgpu-kernarg-preload-count=12"]


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


TRACE_LIB = os.path.join(LIBDIR, "trace", "libpooled_attn.so")


def build_lib(verbose=False, extra=(), lib=LIB):
    objdir = os.path.dirname(lib)
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [_hipcc()] + HIPCC_FLAGS + list(extra) + ["-I", os.path.join(ROOT, "include"), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, pr in procs:
        out, _ = pr.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if pr.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if out.strip():
            print(out)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs
    subprocess.check_call(cmd)
    return lib


def build_trace_lib(verbose=False):
    """The development-timeline build of the same sources (-DPA_TRACE: the single-round decode kernel stamps its phases);
    used by bench.py --timeline only."""
    return build_lib(verbose, extra=("-DPA_TRACE",), lib=TRACE_LIB)


# timing-only ablations of the prefill step (attn_prefill.hip, PF_ABL): what is removed from every step
PREFILL_ABLATIONS = [(0, "nothing"), (1, "the 16 v_exp_f32 per lane (argument passed through)"), (2, "K fragment reads (one fragment reused)"),
                     (4, "V^T fragment reads"), (6, "K and V^T fragment reads"), (8, "the whole softmax (scores converted straight to f16)"),
                     (14, "fragment reads and softmax"), (16, "the LDS-direct tile loads (32 KB a step and CU from L2)"),
                     (30, "all of the above (MFMAs and the barrier remain)")]


def ablation_lib(mask):
    return os.path.join(LIBDIR, "abl%d" % mask, "libpooled_attn.so")


def build_prefill_ablations(verbose=False):
    """One library per ablation mask (results wrong on purpose; bench.py --prefill-ablation times them)."""
    out = []
    for mask, _ in PREFILL_ABLATIONS:
        lib = build_lib(verbose, extra=("-DPF_ABL=%d" % mask,), lib=ablation_lib(mask))
        for f in os.listdir(os.path.dirname(lib)):
            if f.endswith(".o"):
                os.remove(os.path.join(os.path.dirname(lib), f))
        out.append(lib)
    return out


def build_addon(verbose=False):
    """The thin Node-API layer over the C ABI (plain g++ against the system node headers; no node-gyp)."""
    src = os.path.join(CSRC, "pa_napi.cc")
    inc = "/usr/include/node"
    if not (os.path.exists(src) and os.path.exists(os.path.join(inc, "node_api.h"))):
        return None
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", inc, "-I", os.path.join(ROOT, "include"), src,
           "-o", ADDON, "-L", LIBDIR, "-lpooled_attn", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return ADDON


def build_all(verbose=False, extra=()):
    lib = build_lib(verbose, extra=extra)
    addon = build_addon(verbose)
    return lib, addon


if __name__ == "__main__":
    if "--trace" in sys.argv:
        print(build_trace_lib(verbose="-v" in sys.argv))
    elif "--prefill-ablation" in sys.argv:
        print(build_prefill_ablations(verbose="-v" in sys.argv))
    else:
        # -DNAME=VALUE arguments go to hipcc (the prefill kernel's PF_SUB / PF_QR / PF_KD / PF_VD experiments)
        print(build_all(verbose="-v" in sys.argv, extra=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
