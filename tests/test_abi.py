"""No-GPU checks of the boundary: the shared library loads and exports every symbol include/pooled_attn.h
declares, and the ctypes table covers the same set."""
import ctypes
import os
import re
from pooled_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "pooled_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    names = _declared()
    assert len(names) >= 25
    lib = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libpooled_attn.so does not export %s" % n
    assert sorted(capi.SYMBOLS) == names


def test_struct_layouts_match_header():
    assert ctypes.sizeof(capi.PaConfig) == 40 and ctypes.sizeof(capi.PaPlan) == 32
    assert capi.PaConfig.rope_theta.offset == 16 and capi.PaConfig.flags.offset == 36


def test_version_string_without_gpu():
    L = capi.load()
    assert L.pa_version().decode().startswith("pooled_attn")


def test_addon_exports_when_built():
    import shutil, subprocess
    addon = os.path.join(ROOT, "pooled_amd", "lib", "pooled_attn.node")
    if not (os.path.exists(addon) and shutil.which("node")):
        import pytest
        pytest.skip("addon or node missing")
    js = "const a=require(%r); const want=['create','destroy','layerAlloc','sync','malloc','free','upload','download','glueKv','glue','kvStore','attn','planQuery','kvRead','kvWrite','timerStart','timerStop','version']; for (const w of want) if (typeof a[w] !== 'function') { console.log('missing', w); process.exit(1); } console.log('ok', a.version());" % addon
    r = subprocess.run(["node", "-e", js], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.startswith("ok"), r.stdout + r.stderr
