"""The C-ABI libraries load and export every symbol their headers declare (no GPU needed)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(axhip_\w+)\s*\(", text)))


def test_axhip_exports_every_declared_symbol():
    from axiom_amd.hip import LIB_PATH, SIGNATURES
    names = declared_functions("axhip.h")
    assert len(names) >= 25
    lib = C.CDLL(LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/axhip.h but not exported"
    assert sorted(SIGNATURES) == names, "python binding and header disagree"


def test_axhip_fails_loudly_without_gpu():
    from axiom_amd import AxHip, AxHipError
    h = AxHip()
    if h.L.axhip_device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(AxHipError) as e:
        h.init()
    assert e.value.code == 9 and "no CPU fallback" in str(e.value)
    # compute entry points refuse too, rather than computing on the host
    assert h.L.axhip_sgemm(0, 0, 1, 1, 1, 1.0, 1, 1, 1, 1, 0.0, 1, 1, None, 0) == 9
    assert h.L.axhip_qgemm_w8a8(1, 1.0, 1, 1, None, 0, 1, None, 1, 1, 1) == 9
    assert h.L.axhip_malloc(16) is None
