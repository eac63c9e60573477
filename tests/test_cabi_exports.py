"""CPU-side checks of the C-ABI: every function declared under include/ is exported by the
built library with C linkage (no compute is called: there is no GPU here)."""
import ctypes
import glob
import os
import re

import __graft_entry__ as entry

INCLUDE = os.path.join(entry.ROOT, "include")


def _declared_functions():
    names = []
    for path in glob.glob(os.path.join(INCLUDE, "turboquant_c", "*.h")):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in re.finditer(r"\b(tq_[a-z0-9_]+)\s*\(", text):
            names.append(m.group(1))
    return sorted(set(names))


def test_headers_declare_the_hot_path_entry_points():
    names = _declared_functions()
    for required in ("tq_linear_create", "tq_linear_forward", "tq_linear_dequantize", "tq_linear_free",
                     "tq_wht_rotate", "tq_last_error"):
        assert required in names


def test_library_exports_every_declared_symbol():
    pkg = entry.load_package()
    assert os.path.exists(pkg.LIB_PATH), "build the library first (python __graft_entry__.py)"
    lib = ctypes.CDLL(pkg.LIB_PATH)
    missing = [n for n in _declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in include/ but not exported: {missing}"


def test_headers_compile_as_c():
    import subprocess
    import tempfile
    headers = sorted(glob.glob(os.path.join(INCLUDE, "turboquant_c", "*.h")))
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        with open(src, "w") as f:
            for h in headers:
                f.write(f'#include "{os.path.relpath(h, INCLUDE)}"\n')
            f.write("int main(void) { return 0; }\n")
        subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", INCLUDE, "-c", src, "-o", os.path.join(d, "t.o")])


def test_null_conventions_without_gpu():
    """Getters on NULL return 0, free(NULL) is a no-op, and calls with NULL handles fail cleanly
    (reference conventions, src/turboquant_c.cpp:56-69,311-314)."""
    pkg = entry.load_package()
    L = pkg.lib()
    assert L.tq_linear_in_features(None) == 0
    assert L.tq_linear_out_features(None) == 0
    assert L.tq_linear_mode(None) == 0
    L.tq_linear_free(None)
    assert L.tq_linear_forward(None, None, 0, 1, None, 0, None) != 0
    assert L.tq_linear_dequantize(None, None, None) != 0
    assert b"NULL" in L.tq_last_error()
