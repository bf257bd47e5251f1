"""CPU: the C ABI library loads, exports every function include/tsattn.h declares, and the ctypes
mirrors of its argument structs have the C compiler's size and field offsets.  No compute calls."""
import ctypes
import os
import re
import subprocess

import pytest

from tscale_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tsattn.h")
TEST_HOOKS = os.path.join(ROOT, "include", "tsattn_test_hooks.h")   # entry points for the library's own tests

STRUCTS = {
    "tsattn_config": capi.Config,
    "tsattn_prefill_args": capi.PrefillArgs,
    "tsattn_decode_args": capi.DecodeArgs,
    "tsattn_append_args": capi.AppendArgs,
    "tsattn_fill_args": capi.FillArgs,
    "tsattn_produce_args": capi.ProduceArgs,
    "tsattn_matmul_args": capi.MatmulArgs,
    "tsattn_merge_args": capi.MergeArgs,
}


def declared_functions():
    text = open(HEADER).read() + open(TEST_HOOKS).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tsattn_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_what_python_binds():
    assert declared_functions() == sorted(capi.EXPORTS)


def test_library_exports_every_declared_function():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail(f"{capi.LIB_PATH} has not been built (make -C tscale_amd/csrc)")
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.tsattn_version is not None


def test_ctypes_structs_match_the_c_layout(tmp_path):
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {"]
    for cname, cls in STRUCTS.items():
        lines.append(f'  printf("{cname} size %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'  printf("{cname} {fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    got = {}
    for ln in out:
        if ln:
            c, f, n = ln.split()
            got[(c, f)] = int(n)
    for cname, cls in STRUCTS.items():
        assert got[(cname, "size")] == ctypes.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert got[(cname, fname)] == getattr(cls, fname).offset, (cname, fname)


def test_scratch_bytes_is_a_pure_host_function():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail("library not built")
    lib = capi.load()
    cfg = capi.Config(0, 64, 16, 128, 32)
    n = lib.tsattn_scratch_bytes(ctypes.byref(cfg))
    assert n == 64 * 16 * 32 * (128 + 2) * 4 + 64 * 4   # split partials + per-sequence arrival counters
