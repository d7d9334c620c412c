"""CPU-only checks of the C-ABI boundary: the built library loads without a GPU and exports exactly
the entry points include/linmt_hip.h declares; the Python binding mirrors the same list."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", f) for f in sorted(os.listdir(os.path.join(ROOT, "include")))
           if f.endswith(".h")]


def declared_symbols(path):
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:lh|lnmt)_[a-z0-9_]+)\s*\(", text)))


def library_for(header):
    name = os.path.basename(header)
    return os.path.join(ROOT, "linmt_amd",
                        "liblinmt_hip.so" if name == "linmt_hip.h" else "liblinmt_host.so")


@pytest.mark.parametrize("header", HEADERS, ids=[os.path.basename(h) for h in HEADERS])
def test_library_exports_every_declared_symbol(header):
    syms = declared_symbols(header)
    assert syms, f"no entry points parsed from {header}"
    path = library_for(header)
    assert os.path.exists(path), f"{path} is not built (run __graft_entry__.build())"
    lib = ctypes.CDLL(path)
    missing = [s for s in syms if not hasattr(lib, s)]
    assert not missing, f"{os.path.basename(path)} does not export {missing}"


def test_python_binding_matches_header():
    from linmt_amd import lib
    hdr = declared_symbols(os.path.join(ROOT, "include", "linmt_hip.h"))
    assert sorted(lib.SIGNATURES) == hdr
    loaded = lib.load()
    assert loaded.lh_abi_version() == 1
    assert loaded.lh_last_error() == b""


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from linmt_amd import lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(lib.LinmtHipError):
        lib.load()


def test_c_headers_compile_as_plain_c(tmp_path):
    """The boundary is a C ABI: both headers that declare it are valid C99 on their own (no C++,
    no HIP or torch types), so a cgo / JNI / ctypes-style binding can include them as they are."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_headers.c"
    src.write_text('#include "linmt_hip.h"\n#include "linmt_host.h"\n'
                   "int main(void) { lh_error_term t = {0, 1, 0, 4}; lh_gemm_seg s = {0, 0, 0, 0, 0};\n"
                   "  return t.planes - 1 + s.K; }\n")
    r = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I",
                        os.path.join(ROOT, "include"), "-c", str(src), "-o", str(tmp_path / "use_headers.o")],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
