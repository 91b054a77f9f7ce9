"""CPU-only checks of the C-ABI library: it loads, exports every function the header
declares, and its argument checks answer without touching a GPU."""

import ctypes
import os
import re

import pytest

from come_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "come_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(come_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m come_amd.build`"


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 8
    for name in names:
        assert hasattr(lib, name), f"{name} declared in come_hip.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_error_string():
    lib = _lib.load()
    assert lib.come_version() >= 100
    # invalid arguments are rejected on the host, before any HIP call
    assert lib.come_merge_plan(None, 1, 1, -1, 2, 0, None, None, None) == 1
    assert b"start_index" in lib.come_last_error()
    assert lib.come_token_merge(None, 7, 1, 1, 1, 0, 1, 1, 1, 1, None, None, None, None, 0,
                                None, None, None, None, None) == 2
    assert b"dtype" in lib.come_last_error()
    assert lib.come_attn_varlen_fwd(None, None, None, _lib.COME_BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 128,
                                    None, 10, 0.125, None, 64, 64, None, None) == 2
    assert b"head_dim" in lib.come_last_error()
    assert lib.come_select_work_bytes(1, 16, 37, 37, 3, 3) >= 16 * 144 * 4


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libcome_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """The header compiles as C99 and a C caller that references every declared function links against the
    shared library (no C++ names, no torch types)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("gcc not available")
    names = _declared_functions()
    src = tmp_path / "caller.c"
    body = "\n".join(f"    table[{i}] = (fn)&{name};" for i, name in enumerate(names))
    src.write_text('#include "come_hip.h"\n#include <stdio.h>\ntypedef void (*fn)(void);\nint main(void) {\n'
                   f"    fn table[{len(names)}];\n{body}\n"
                   '    printf("%d %s|\\n", come_version(), come_last_error());\n'
                   f"    return table[0] == 0;\n}}\n")
    exe = tmp_path / "caller"
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    cmd = [gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", lib_dir, "-lcome_hip", f"-Wl,-rpath,{lib_dir}", "-Wl,--allow-shlib-undefined"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0, run.stderr
    assert run.stdout.startswith(str(_lib.load().come_version()))
