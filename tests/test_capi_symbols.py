"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and refuses work without a device instead of falling back."""
import ctypes as C
import re
from pathlib import Path

import pytest

from granite_amd import _capi

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "granite_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(granite_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _capi.load()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} declared in granite_hip.h but not exported"


def test_calibration_library_exports_its_header():
    """The measurement aid is a library of its own, beside the attention library."""
    cal_header = ROOT / "include" / "granite_hip_calibration.h"
    text = re.sub(r"/\*.*?\*/", "", cal_header.read_text(), flags=re.S)
    names = sorted(set(re.findall(r"\b(granite_hip_[a-z0-9_]+)\s*\(", text)))
    assert names == ["granite_hip_cal_mfma_mix", "granite_hip_cal_mfma_rate"]
    lib = C.CDLL(str(ROOT / "granite_amd" / "lib" / "libgranite_hip_calibration.so"))
    for name in names:
        assert hasattr(lib, name)
    for name in names:
        assert not hasattr(_capi.load(), name)   # and not in the product library


def test_binding_table_covers_the_header():
    assert sorted(_capi.SIGNATURES) == declared_symbols()


def test_struct_layouts_match_header_field_order():
    text = HEADER.read_text()
    for cname, cls in (("granite_hip_decode_args", _capi.DecodeArgs),
                       ("granite_hip_attention_args", _capi.AttentionArgs),
                       ("granite_hip_device_info", _capi.DeviceInfo)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), text, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                name = re.sub(r"\[.*\]", "", part.strip().split()[-1]).lstrip("*")
                fields.append(name)
        assert fields == [f[0] for f in cls._fields_], cname


def test_no_device_means_error_not_fallback():
    import subprocess, sys
    code = (
        "import ctypes as C\n"
        "from granite_amd import _capi\n"
        "lib = _capi.load()\n"
        "if lib.granite_hip_init(0) == 0:\n"
        "    print('HAS_GPU')\n"
        "else:\n"
        "    p = C.c_void_p()\n"
        "    assert lib.granite_hip_malloc(C.byref(p), 64, 0) == _capi.ENOTINIT\n"
        "    assert lib.granite_hip_sync() == _capi.ENOTINIT\n"
        "    a = _capi.DecodeArgs()\n"
        "    assert lib.granite_hip_decode_attention(C.byref(a)) == _capi.ENOTINIT\n"
        "    b = _capi.AttentionArgs()\n"
        "    assert lib.granite_hip_attention(C.byref(b)) == _capi.ENOTINIT\n"
        "    print('NO_GPU_OK')\n")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip() in ("HAS_GPU", "NO_GPU_OK")


def test_missing_library_raises(monkeypatch, tmp_path):
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", tmp_path / "libgranite_hip.so")
    with pytest.raises(_capi.GraniteHipError):
        _capi.load()
