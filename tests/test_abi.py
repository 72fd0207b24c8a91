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
