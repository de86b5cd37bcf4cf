"""The public header is plain C: it compiles as C99 with pedantic warnings as errors, and imports as a
Clang module through include/module.modulemap -- the closest stand-in this image offers for importing it
from Swift (a SwiftPM C target exposes exactly this header and module map; no Swift toolchain is here)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")

C_USER = r"""
#include "nvmai_hip.h"
int main(void) {
    nvmai_expert_offsets off;
    uint64_t stride = 0;
    int rc = nvmai_expert_offsets_for(2048, 512, 4, &off, &stride);
    return (rc == NVMAI_OK && stride == 1769472u && sizeof(nvmai_prefill_pair) == 16 &&
            sizeof(nvmai_prefill_streamed_params) == 128) ? 0 : 1;
}
"""


def test_header_compiles_as_c99(tmp_path):
    src = tmp_path / "user.c"
    src.write_text(C_USER)
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", INC, str(src)],
                   check=True)


def _clang():
    for c in ("/opt/rocm/lib/llvm/bin/clang", "/opt/rocm/llvm/bin/clang", shutil.which("clang") or ""):
        if c and os.path.exists(c):
            return c
    return None


def test_header_imports_as_a_clang_module(tmp_path):
    clang = _clang()
    if clang is None:
        pytest.skip("no clang in this image")
    src = tmp_path / "user.m.c"
    src.write_text(C_USER)
    # -fmodules turns the #include into an import of the module the map declares
    subprocess.run([clang, "-std=c99", "-fmodules", "-fimplicit-module-maps", "-fmodules-cache-path=%s" % (tmp_path / "cache"),
                    "-Wall", "-Werror", "-Rmodule-import", "-fsyntax-only", "-I", INC, str(src)], check=True)
    with open(os.path.join(INC, "module.modulemap")) as f:
        text = f.read()
    assert "nvmai_hip.h" in text and "module" in text
