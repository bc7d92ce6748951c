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


@pytest.mark.gpu
def test_stream_yardstick_reads_what_it_says_at_a_plausible_rate(hip):
    """The reader that bench.py --workload stream times: every workgroup gets a whole number of 64 KB rounds of its share of
    the buffer; the rate of one launch over 1 GiB stays below the HBM peak; bad arguments are refused."""
    import ctypes
    from openvino_contrib_amd import build as hip_build
    yard = ctypes.CDLL(hip_build.YARDSTICK_LIB_PATH)
    yard.stream_yardstick_launch.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.POINTER(ctypes.c_longlong)]
    total = 1 << 30
    buf, sink = hip.DeviceBuffer(total), hip.DeviceBuffer(256)
    buf.fill(5)
    nread = ctypes.c_longlong()
    for workgroups in (256, 90, 7):
        e0, e1 = hip.Event(), hip.Event()
        assert yard.stream_yardstick_launch(buf.ptr, total, workgroups, sink.ptr, None, ctypes.byref(nread)) == 0  # (clock ramp, first touch)
        e0.record()
        assert yard.stream_yardstick_launch(buf.ptr, total, workgroups, sink.ptr, None, ctypes.byref(nread)) == 0
        e1.record()
        e1.synchronize()
        share = total // workgroups // 65536 * 65536
        assert nread.value == share * workgroups and total - nread.value < workgroups * 65536
        gbs = nread.value / (e0.elapsed_ms(e1) * 1e-3) / 1e9
        assert 20.0 * min(workgroups, 100) * 0.5 < gbs < 8000.0, (workgroups, gbs)
    assert yard.stream_yardstick_launch(buf.ptr, 1000, 4, sink.ptr, None, ctypes.byref(nread)) == 0 and nread.value == 0  # less than a round each
    assert yard.stream_yardstick_launch(None, total, 4, sink.ptr, None, ctypes.byref(nread)) != 0
    assert yard.stream_yardstick_launch(buf.ptr, total, 0, sink.ptr, None, ctypes.byref(nread)) != 0
    buf.free()
    sink.free()
