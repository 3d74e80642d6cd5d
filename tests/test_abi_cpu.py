"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/et.h declares,
and its host-only entry points (sizes, status strings, argument errors) behave.  No kernel runs."""
import ctypes as C
import os
import re

import pytest

from effective_transformer_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "et.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(et_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)


def test_status_strings_and_sizes():
    lib = _lib.load()
    assert lib.et_status_string(0) == b"ET_OK"
    assert lib.et_status_string(2) == b"ET_WORKSPACE_TOO_SMALL"
    assert lib.et_input_workspace_bytes(1000, 64) >= 4 * 63
    assert lib.et_input_workspace_bytes(0, 64) == 0
    # the layer workspace is sized by element type (the reference sizes in bytes and indexes in elements)
    h16 = lib.et_layer_workspace_bytes(_lib.ET_FP16, 500, 64, 12, 64)
    h32 = lib.et_layer_workspace_bytes(_lib.ET_FP32, 500, 64, 12, 64)
    assert h32 > 1.9 * h16 > 0
    rows, H = 500 * 64, 768
    assert h16 >= rows * 9 * H * 2
    assert lib.et_seq_workspace_bytes(256) >= 257 * 4


def test_null_handle_and_create_without_gpu():
    lib = _lib.load()
    assert lib.et_input(None, 0, None, None, None, None, None, None, 1, 1, 1, 1, None, 0, None, None) == 1
    assert b"null handle" in lib.et_last_error(None)
    import torch
    if not torch.cuda.is_available():
        h = C.c_void_p()
        st = lib.et_create(C.byref(h), 0)
        assert st != 0 and not h.value
        assert lib.et_last_error(None).startswith(b"[ET][ERROR]")
    assert lib.et_destroy(None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        _lib.load()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message instead of a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stderr + r.stdout)
    assert "{" not in r.stdout


def test_header_is_plain_c_and_links(tmp_path):
    """include/et.h is what a C (or cgo / JNI) caller includes: it must compile as strict C99, and a C program must link
    against the library and get sizes and status strings without a GPU."""
    import shutil
    import subprocess
    from effective_transformer_amd import _lib
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "caller.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "et.h"\n'
        "int main(void) {\n"
        "  et_layer_weights w; et_layer_prepared p; memset(&w, 0, sizeof w); memset(&p, 0, sizeof p);\n"
        "  if (et_layer_workspace_bytes(ET_FP16, 8, 32, 12, 64) == 0 || et_seq_workspace_bytes(8) < (2 * 8 + 1) * 4) return 1;\n"
        '  if (strcmp(et_status_string(ET_WORKSPACE_TOO_SMALL), "ET_WORKSPACE_TOO_SMALL") != 0) return 2;\n'
        "  if (et_output(NULL, ET_FP16, NULL, NULL, NULL, NULL, NULL, 1, 1, 1, 1, NULL) != ET_INVALID_ARGUMENT) return 3;\n"
        '  printf("%s\\n", et_last_error(NULL));\n'
        "  return 0;\n}\n")
    exe = tmp_path / "caller"
    libdir = os.path.dirname(_lib.LIB_PATH)
    inc = os.path.join(os.path.dirname(os.path.dirname(libdir)), "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, str(src), "-o", str(exe),
                    "-L", libdir, "-let_hip", "-Wl,-rpath," + libdir], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "null handle" in r.stdout
