"""CPU-only checks of the boundary: the shared library loads, exports every function the
header declares, and the host-side argument marshalling builds the reference's slot block."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "illatio_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ilt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from illatio_amd import hip
    assert os.path.exists(hip.LIB_PATH), "build the library first: make -C illatio_amd/csrc"
    lib = C.CDLL(hip.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 45
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_error_string_and_unknown_kernel_need_no_gpu():
    from illatio_amd import hip
    assert hip.lib().ilt_error_string(0) == b"no error"
    assert hip.lib().ilt_error_string(1)          # some text for an invalid-value error


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from illatio_amd import hip
    monkeypatch.setattr(hip, "_lib", None)
    monkeypatch.setattr(hip, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        hip.lib()


def test_launch_slot_block(monkeypatch):
    """LAUNCH writes pointer -> 64 bits, int -> low 32 bits, float -> 32 bits, (:i64 n) -> 64
    bits, NIL -> 0, (dbuf . offset) -> ptr + offset (cuda.lisp:328-338)."""
    from illatio_amd import hip
    seen = {}

    class FakeLib:
        def ilt_launch(self, name, gx, gy, gz, bx, by, bz, shared, stream, ptrs):
            seen["name"], seen["grid"], seen["block"] = name, (gx, gy, gz), (bx, by, bz)
            seen["slots"] = [C.cast(ptrs[i], C.POINTER(C.c_uint64))[0] for i in range(seen["n"])]
            return 0

        def ilt_error_string(self, code):
            return b""

    monkeypatch.setattr(hip, "_lib", FakeLib())
    dev = hip.Device(0, hip.DeviceInfo(), 0)
    b = hip.DBuf(0x7f0000001000, 4096, dev)
    args = [b, b.at(64), None, 7, -1, 1.5, hip.I64(1 << 40)]
    seen["n"] = len(args)
    hip.launch(dev, "mv_q8", (3, 2), 128, args)
    assert seen["name"] == b"mv_q8" and seen["grid"] == (3, 2, 1) and seen["block"] == (128, 1, 1)
    s = seen["slots"]
    assert s[0] == 0x7f0000001000 and s[1] == 0x7f0000001040 and s[2] == 0
    assert s[3] == 7 and s[4] == 0xFFFFFFFF
    assert s[5] == int(np.float32(1.5).view(np.uint32)) and s[6] == 1 << 40
    with pytest.raises(TypeError):
        hip.launch(dev, "mv_q8", 1, 1, ["a string"])
