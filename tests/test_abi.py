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
    assert lib.come_attn_varlen_fwd(None, None, None, _lib.COME_BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 96,
                                    None, 10, 0.125, None, 64, 64, None, 0, None) == 2
    assert b"head_dim" in lib.come_last_error()
    assert lib.come_select_work_bytes(1, 16, 37, 37, 3, 3) >= 16 * 144 * 4


def test_q_prologue_entry_point_checks_its_descriptor_on_the_host():
    """come_attn_varlen_fwd_qp refuses what it cannot do before anything is launched (the pointers are never followed)."""
    lib = _lib.load()
    fake = 0x10000                                   # an aligned address that is not dereferenced

    def call(head_dim, desc, flags):
        row = 3 * 16 * head_dim
        return lib.come_attn_varlen_fwd_qp(fake, fake, fake, _lib.COME_BF16, row, head_dim, row, head_dim, row, head_dim,
                                           fake, 1, 10, 16, head_dim, None, 10, 0.125, fake, 16 * head_dim, head_dim, None,
                                           None, 0, desc, flags, None)

    norm = _lib.QPrologue(1, 1e-5, None, None, None, None, None, 0)
    assert call(128, ctypes.byref(norm), 0) == 2 and b"head_dim must be 64" in lib.come_last_error()
    assert call(64, ctypes.byref(norm), _lib.COME_ATTN_WORK_QUEUE) == 2 and b"COME_ATTN_WORK_QUEUE" in lib.come_last_error()
    assert call(64, ctypes.byref(_lib.QPrologue(1, -1.0, None, None, None, None, None, 0)), 0) == 1
    assert b"eps" in lib.come_last_error()
    assert call(64, ctypes.byref(_lib.QPrologue(0, 0.0, None, None, fake, None, None, 0)), 0) == 1
    assert b"tables" in lib.come_last_error()
    assert call(64, ctypes.byref(_lib.QPrologue(1, 1e-5, fake + 2, None, None, None, None, 0)), 0) == 1
    assert b"aligned" in lib.come_last_error()
    assert call(64, ctypes.byref(norm), 4) == 1 and b"flags" in lib.come_last_error()


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


def test_every_entry_point_rejects_bad_arguments_on_the_host():
    """Argument checks run before any HIP call, so they can be exercised without a GPU: every entry point
    returns a non-zero status and leaves a message that names the problem."""
    lib = _lib.load()
    BF16, F32 = _lib.COME_BF16, _lib.COME_F32

    def rejected(status, fragment):
        assert status != 0
        assert fragment.encode() in lib.come_last_error(), lib.come_last_error()

    rejected(lib.come_token_split(None, 9, 1, 8, None, None, 4, None, None), "dtype")
    rejected(lib.come_token_split(None, BF16, 1, 0, None, None, 4, None, None), "chans")
    rejected(lib.come_token_split(None, BF16, 1, 8, None, None, 4, None, None), "rev")            # no index given
    rejected(lib.come_token_split_pair(None, None, 9, 1, 8, None, None, 4, None, None), "dtype")
    rejected(lib.come_select_windows(None, _lib.COME_F16, 1, 1, 6, 6, 3, 3, 0, 0.5, None, None, None, 0, None),
             "come_select_windows")                                                                # fp16 confidence
    rejected(lib.come_select_windows(None, F32, 1, 1, 6, 6, 0, 3, 0, 0.5, None, None, None, 0, None), "group")
    rejected(lib.come_select_windows(None, F32, 1, 1, 6, 6, 3, 3, 7, 0.5, None, None, None, 0, None), "mode")
    rejected(lib.come_select_windows(None, F32, 1, 1, 6, 6, 3, 3, 0, 1.5, None, None, None, 0, None), "threshold")
    rejected(lib.come_attn_varlen_fwd(None, None, None, F32, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 64,
                                      None, 10, 0.125, None, 64, 64, None, 0, None), "fp16 and bf16")
    rejected(lib.come_attn_varlen_fwd(None, None, None, BF16, 64, 64, 64, 64, 64, 64, None, 0, 10, 1, 64,
                                      None, 10, 0.125, None, 64, 64, None, 0, None), "batch size")
    rejected(lib.come_attn_varlen_fwd(None, None, None, BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 64,
                                      None, 10, -1.0, None, 64, 64, None, 0, None), "softmax_scale")
    rejected(lib.come_attn_varlen_fwd(None, None, None, BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 64,
                                      None, 10, 0.125, None, 64, 64, None, 0, None), "NULL")
    rejected(lib.come_attn_varlen_fwd(None, None, None, BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 64,
                                      None, 10, 0.125, None, 64, 64, None, 12, None), "flags")
    rejected(lib.come_attn_varlen_fwd_ws(None, None, None, BF16, 64, 64, 64, 64, 64, 64, None, 1, 10, 1, 48,
                                         None, 10, 0.125, None, 64, 64, None, None, 0, 0, None), "head_dim")
    rejected(lib.come_qk_norm_rope(None, None, F32, 64, 64, 64, 64, 4, 1, 64, 1, None, None, None, None, 1e-5,
                                   None, None, None, 0, None), "bf16 or fp16")
    rejected(lib.come_qk_norm_rope(None, None, BF16, 64, 64, 64, 64, 4, 1, 32, 1, None, None, None, None, 1e-5,
                                   None, None, None, 0, None), "head_dim")
    rejected(lib.come_qk_norm_rope(None, None, BF16, 64, 64, 64, 64, 4, 1, 64, 1, None, None, None, None, 1e-5,
                                   None, None, None, 0, None), "null")
    rejected(lib.come_jagged_add_suffix(None, None, 9, 4, 8, None, 2, None, 1, None, None, None, None), "dtype")
    rejected(lib.come_jagged_add_suffix(None, None, BF16, 4, 8, None, 2, None, 1, None, None, None, None), "offsets")
    rejected(lib.come_jagged_split_suffix(None, None, BF16, 1, 8, None, 2, 1, None, None, None, None, None), "come_jagged_split_suffix")
    # sizes that need no work return success without touching the device
    assert lib.come_token_split(None, BF16, 0, 8, None, None, 0, None, None) == 0
    assert lib.come_attn_work_bytes(0, 0, 0, 0) == 0
