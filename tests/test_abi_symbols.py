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
