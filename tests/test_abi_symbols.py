"""The C-ABI library loads and exports every symbol include/saga_hip.h declares (no GPU needed)."""
import os
import re

from saga_amd import kernels as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "saga_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(saga_hip_\w+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    L = K.lib()
    names = declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(L, n), n
        assert n in K.SIGNATURES, f"{n} has no ctypes signature"
    assert set(K.SIGNATURES) == set(names)


def test_error_strings():
    assert K.lib().saga_hip_error_string(-2) == b"operand shapes do not agree"


def test_capi_symbols_exported():
    """libsaga.so (front end + hip engine) exports every function include/saga_capi.h declares."""
    import ctypes

    text = open(os.path.join(ROOT, "include", "saga_capi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(saga_[a-z_0-9]+)\s*\(", text)))
    assert len(names) >= 30
    K.lib()  # libsaga.so links against the kernel library
    L = ctypes.CDLL(os.path.join(ROOT, "saga_amd", "lib", "libsaga.so"))
    for n in names:
        assert hasattr(L, n), n


def test_headers_are_plain_c(tmp_path):
    """The drop-in boundary is a C ABI: both headers compile as strict C99 on their own."""
    import subprocess

    for h in ("saga_hip.h", "saga_capi.h"):
        src = tmp_path / (h + ".c")
        src.write_text(f'#include "{h}"\nint main(void) {{ return 0; }}\n')
        r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only",
                            "-I", os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
