"""The C-ABI library loads without a GPU, exports every declared symbol, and
fails loudly (never silently on a CPU path) when there is no device."""
import ctypes as C

import numpy as np
import pytest

import volvoxai_amd as vx
from volvoxai_amd._lib import declared_symbols, library


def test_library_exports_every_declared_symbol():
    lib = library()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/vxhip_w8a8.h but not exported"
    assert lib.vxhip_abi_version() == 1


def test_kernel_variant_table_shape():
    rows = vx.kernel_variants()
    ids = {r["id"] for r in rows}
    assert {"hip.qlinear.mfma-i8", "hip.qlinear.gemv-mfma", "hip.packed-linear.a8-mfma",
            "hip.packed-linear.a8-gemv-mfma", "hip.packed-linear.w4a8-mfma",
            "hip.packed-linear.w4a8-gemv-mfma"} <= ids
    for r in rows:
        assert r["backend"] == 0 and r["id"].startswith("hip.") and r["priority"] > 0
        assert r["operator_kind"] in (1002, 1005, 1007, 1036)
    # QLinear, QGemm and QMatMul share one kernel family, as upstream's cuda.qlinear.* rows do
    for fam in ("hip.qlinear.mfma-i8", "hip.qlinear.gemv-mfma"):
        assert {r["operator_kind"] for r in rows if r["id"] == fam} == {1002, 1005, 1007}


def _no_gpu():
    return library().vxhip_device_count() == 0


@pytest.mark.skipif(not _no_gpu(), reason="checks the no-device behaviour")
def test_without_device_entry_points_decline_and_say_why():
    lib = library()
    h = C.c_void_p()
    assert lib.vxhip_context_create(0, None, 0, C.byref(h)) == -6  # BACKEND_UNAVAILABLE
    assert not h and b"device" in lib.vxhip_last_error()
    x = np.zeros((2, 16), np.int8)
    w = np.zeros((4, 16), np.int8)
    ok, _ = vx.qlinear_i8u8(x, w, np.ones(4, np.float32), np.zeros(4, np.int32), np.zeros(4, np.int32),
                            2, 16, 4, 1.0, 0, 1.0, 0, vx.DTYPE_I8, vx.DTYPE_I8, vx.DTYPE_I8)
    assert ok == 0  # declined, not computed somewhere else
    st, _ = vx.packed_linear_f32(np.zeros((1, 32), np.float32), np.zeros((2, 8), np.uint32),
                                 np.ones((2, 1), np.float32), None, 32, 2, 32)
    assert st == -1


def test_argument_validation_happens_before_any_device_work():
    lib = library()
    h = C.c_void_p()
    # non-byte dtype, null tensors: INVALID_ARGUMENT regardless of hardware
    assert lib.vxhip_qlinear_create(None, None, None, None, 4, 4, vx.DTYPE_I8, C.byref(h)) == -1
    w = np.zeros((4, 4), np.int8)
    s = np.ones(4, np.float32)
    z = np.zeros(4, np.int32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    assert lib.vxhip_qlinear_create(p(w), p(s), p(z), None, 4, 4, 18, C.byref(h)) == -1
    bad = np.array([1, 1, 0, 1], np.float32)
    if _no_gpu():
        return
    assert lib.vxhip_qlinear_create(p(w), p(bad), p(z), None, 4, 4, vx.DTYPE_I8, C.byref(h)) == -1
    words = np.zeros((2, 8), np.uint32)
    assert lib.vxhip_packed_linear_create(p(words), p(s), None, 32, 2, 32, 4, C.byref(h)) == -7
    assert lib.vxhip_packed_linear_create(p(words), p(s), None, 32, 2, 48, 8, C.byref(h)) == -1
