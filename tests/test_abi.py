"""The C-ABI library loads without a GPU and exports every function the headers declare."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = set()
    for h in ("moe_kernels.h", "moe_engine.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)          # comments
        text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)            # preprocessor lines
        text = re.sub(r"typedef\s+struct[^{;]*\{.*?\}[^;]*;", " ", text, flags=re.S)  # struct bodies
        for m in re.finditer(r"\b(moe_[a-z0-9_]+)\s*\(", text):
            names.add(m.group(1))
    return sorted(names)


def test_every_declared_function_is_exported():
    import torch  # noqa: F401  (the library shares torch's HIP runtime)
    from promoe_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH) if hasattr(_lib, "LIB_PATH") else _lib.lib
    names = declared_functions()
    assert len(names) > 50, names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_headers_compile_as_c():
    """include/*.h are plain C: compile them with gcc, no HIP or torch types in the signatures."""
    import subprocess
    import tempfile
    src = '#include "moe_kernels.h"\n#include "moe_engine.h"\nint main(void) { return 0; }\n'
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", c,
                            "-o", os.path.join(d, "t.o")], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
