"""The C-ABI library loads and exports every symbol the header declares; the
ctypes structures have the layout of the C structs (no compute here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib_path():
    from metaattention_amd import hip_backend as hb
    if not os.path.exists(hb.LIB_PATH):
        from metaattention_amd.build import build_library
        build_library()
    return hb.LIB_PATH


def test_exports_match_header():
    from metaattention_amd import hip_backend as hb
    header = open(os.path.join(ROOT, "include", "metaattention_hip.h")).read()
    declared = set(re.findall(r"^\s*(?:int|size_t|const char\*)\s+(ma_\w+)\s*\(", header, re.M))
    assert declared == set(hb.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(_lib_path())
    for sym in declared:
        assert getattr(lib, sym) is not None


def test_version_and_error_string():
    lib = ctypes.CDLL(_lib_path())
    lib.ma_last_error.restype = ctypes.c_char_p
    assert lib.ma_version() == 1
    assert lib.ma_attn_fwd(None, None) == -1          # MA_ERR_INVALID_ARG, no GPU touched
    assert b"NULL" in lib.ma_last_error()


def test_struct_layout_matches_c():
    """Compile a tiny C program against the header and compare sizeof/offsetof."""
    import subprocess
    import tempfile
    from metaattention_amd import hip_backend as hb
    checks = [("ma_attn_params", hb.AttnParams), ("ma_attn_bwd_params", hb.AttnBwdParams), ("ma_linear_params", hb.LinearParams),
              ("ma_mla_params", hb.MlaParams)]
    src = ['#include <stdio.h>', '#include <stddef.h>', '#include "metaattention_hip.h"', 'int main(void){']
    for cname, cls in checks:
        src.append(f'printf("%zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            src.append(f'printf("%zu\\n", offsetof({cname}, {fname}));')
    src.append('return 0;}')
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write("\n".join(src))
        exe = os.path.join(d, "t")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        vals = [int(x) for x in subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split()]
    it = iter(vals)
    for cname, cls in checks:
        assert next(it) == ctypes.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert next(it) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_loader_fails_loudly_when_library_missing(tmp_path):
    from metaattention_amd import hip_backend as hb
    saved = hb._lib
    hb._lib = None
    try:
        with pytest.raises(hb.MetaAttentionError):
            hb.load_library(str(tmp_path / "nope.so"))
    finally:
        hb._lib = saved
