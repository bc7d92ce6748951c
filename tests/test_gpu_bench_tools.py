"""The measurement aids that ship beside bench.py (not parity tests)."""
import pytest


@pytest.mark.gpu
def test_mfma_yardstick_reports_a_plausible_rate(hip):
    """The diagnostic that bench.py --workload mfma prints: register-fed bf16 MFMAs only."""
    import ctypes
    from openvino_contrib_amd import build as hip_build
    yard = ctypes.CDLL(hip_build.YARDSTICK_LIB_PATH)  # a bench-only library, not part of libhipattn
    tf, ghz = ctypes.c_double(), ctypes.c_double()
    assert yard.mfma_yardstick(1, 20, ctypes.byref(tf), ctypes.byref(ghz)) == 0
    assert 500.0 < tf.value < 2600.0   # never above the 2.5 PFLOP/s dense bf16 peak (plus timer slack)
    assert 1.0 < ghz.value < 2.6
    assert yard.mfma_yardstick(0, 0, ctypes.byref(tf), ctypes.byref(ghz)) != 0
