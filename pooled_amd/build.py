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


def build_all(verbose=False, extra=()):
    lib = build_lib(verbose, extra=extra)
    addon = build_addon(verbose)
    return lib, addon


if __name__ == "__main__":
    # -DNAME=VALUE arguments go to hipcc (the prefill kernel's PF_QR / PF_KD / PF_VD constants)
    print(build_all(verbose="-v" in sys.argv, extra=tuple(a for a in sys.argv[1:] if a.startswith("-D"))))
