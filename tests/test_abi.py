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


def test_tuning_variables_parse(monkeypatch):
    """AX_HIP_* tile-selection overrides: parsed without a GPU, unknown or out-of-range values mean automatic."""
    from axiom_amd import AxHip
    h = AxHip()
    names = ("AX_HIP_I8_TILE", "AX_HIP_I8_SPLITK", "AX_HIP_F32_TILE", "AX_HIP_F32_SPLITK", "AX_HIP_SKINNY_BLOCKS", "AX_HIP_W8A32_TILE",
             "AX_HIP_SKINNY_FORM", "AX_HIP_SKINNY_KPS", "AX_HIP_I8_MFMA", "AX_HIP_NT_WALK")
    for n in names:
        monkeypatch.delenv(n, raising=False)
    assert h.L.axhip_tuning_reload() == 0
    assert [h.L.axhip_tuning_get(n.encode()) for n in names] == [0] * len(names)
    cases = {"AX_HIP_I8_TILE": [("64x64", 64), ("64x64k2", 642), ("128x128", 128), ("128x64", 1264), ("256x256", 256), ("256", 256),
                                ("32x32", 0), ("", 0), ("tile", 0)],
             "AX_HIP_I8_SPLITK": [("1", 1), ("16", 16), ("17", 0), ("0", 0), ("-3", 0), ("4x", 0)],
             "AX_HIP_F32_TILE": [("64x64", 64), ("64x64k2", 642), ("128x128", 128), ("128x256", 128), ("256x256", 0)],
             "AX_HIP_F32_SPLITK": [("1", 1), ("4096", 4096), ("4097", 0)],
             "AX_HIP_SKINNY_BLOCKS": [("512", 512), ("65535", 65535), ("65536", 0), ("many", 0)],
             "AX_HIP_I8_MFMA": [("16", 16), ("32", 32), ("24", 0), ("64", 0), ("x", 0)],
             "AX_HIP_SKINNY_FORM": [("1", 1), ("3", 3), ("4", 0), ("0", 0), ("pre", 0)],
             "AX_HIP_NT_WALK": [("1", 1), ("2", 2), ("3", 0), ("0", 0), ("cols", 0)],
             "AX_HIP_SKINNY_KPS": [("512", 512), ("1000", 992), ("16", 16), ("15", 0), ("8193", 0)],
             "AX_HIP_W8A32_TILE": [("128x256", 1), ("128x128", 2), ("64x128", 3), ("32x128", 4), ("32x64", 5), ("64x64", 0), ("128", 0)]}
    for name, pairs in cases.items():
        for text, want in pairs:
            monkeypatch.setenv(name, text)
            assert h.L.axhip_tuning_reload() == (1 if want else 0), (name, text)
            assert h.L.axhip_tuning_get(name.encode()) == want, (name, text)
        monkeypatch.delenv(name)
    assert h.L.axhip_tuning_get(b"AX_HIP_NO_SUCH") == -1
    assert h.L.axhip_tuning_reload() == 0
