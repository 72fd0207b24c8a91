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

HIP_SOURCES = ["pa_api.hip", "glue_kv.hip", "attn_decode.hip", "attn_prefill.hip", "proj_gemv.hip", "proj_gemm.hip", "proj_gemm_wide.hip"]
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
               # packed-FP32 VALU forms are kept off for all device code
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # the first twelve dwords of a kernel's leading scalar / pointer arguments arrive in scalar registers at wave start
               "-mllvm", "-amdgpu-kernarg-preload-count=12"]


def _hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


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


# timing-only ablations of the split-K kernel's tile loop (attn_decode.hip, PA_ABL): what is removed
TILE_LOOP_ABLATIONS = [(0, "nothing"), (1, "the tile loads after a wave's first tile"), (3, "those loads, the merge of the four waves and the partial stores"),
                       (5, "those loads and the loop (start-up, the waves' merge and the partial stores remain)"),
                       (7, "all three (launch, start-up and the merge kernel remain)")]


def ablation_lib(mask):
    return os.path.join(LIBDIR, "abl%d" % mask, "libpooled_attn.so")


def build_tile_loop_ablations(verbose=False):
    """One library per ablation mask (results wrong on purpose; bench.py --tile-loop-ablation times them)."""
    out = []
    for mask, _ in TILE_LOOP_ABLATIONS:
        lib = build_lib(verbose, extra=("-DPA_ABL=%d" % mask,), lib=ablation_lib(mask))
        for f in os.listdir(os.path.dirname(lib)):
            if f.endswith(".o"):
                os.remove(os.path.join(os.path.dirname(lib), f))
        out.append(lib)
    return out


def build_all(verbose=False, extra=()):
    lib = build_lib(verbose, extra=extra)
    addon = build_addon(verbose)
    return lib, addon


if __name__ == "__main__":
    # -DNAME=VALUE arguments go to hipcc (the prefill kernel's PF_QR / PF_KD / PF_VD constants)
    if "--tile-loop-ablation" in sys.argv:
        print(build_tile_loop_ablations(verbose="-v" in sys.argv))
    else:
        print(build_all(verbose="-v" in sys.argv, extra=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
