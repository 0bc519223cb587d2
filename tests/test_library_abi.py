"""CPU-side checks of the boundary: the shared library loads and exports exactly the entry points that
include/lfm2_hip.h declares, and the Python binding table covers each of them.  No kernels are launched."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "lfm2_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lfm2_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    from climbing_gym_amd import _lib, build
    if not os.path.exists(_lib.LIBRARY_PATH):
        build.build()
    return ctypes.CDLL(_lib.LIBRARY_PATH)


def test_header_declares_the_expected_surface():
    names = _declared()
    assert len(names) >= 30
    for required in ("lfm2_fp8_gemm", "lfm2_decode_attention", "lfm2_prefill_attention", "lfm2_rms_norm_fp8",
                     "lfm2_conv_update", "lfm2_sample_filtered", "lfm2_record_sample"):
        assert required in names


def test_library_exports_every_declared_symbol(library):
    for name in _declared():
        assert hasattr(library, name), f"{name} is declared in include/lfm2_hip.h but not exported"
    library.lfm2_abi_version.restype = ctypes.c_int
    assert library.lfm2_abi_version() == 1


def test_python_binding_covers_the_header():
    from climbing_gym_amd import _lib
    assert _lib.exported_symbols() == _declared()


def test_argument_errors_are_reported_without_a_gpu(library):
    library.lfm2_last_error.restype = ctypes.c_char_p
    library.lfm2_swiglu.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert library.lfm2_swiglu(None, None, 0, 0, 0, None) == -1
    assert b"empty" in library.lfm2_last_error()
    assert library.lfm2_decode_attention_workspace is not None


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from climbing_gym_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIBRARY_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()
