"""Paged-attention calls recorded into a HIP graph and replayed (gpu).

Callers with launch-bound decode steps capture the step once and replay it (the reference does the
same with CUDA graphs: src/cuda_graph_topology_runner.cpp).  The C ABI must therefore be
capturable: kernel launches and event fork/join only, no allocation, no host synchronisation, no
memset nodes.  A mixed batch is the interesting case: its call forks onto the library's side stream
and joins again, which a capture has to record as a fork and a join of the graph.

Every replay is checked against the eager result, with eager work and synchronisations between the
replays.
"""
import ctypes

import numpy as np
import pytest

import helpers as H
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu

CAPTURE_MODE_RELAXED = 2


def hip_runtime():
    """The HIP runtime library this process already has loaded (the one libhipattn.so links to)."""
    import os

    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64" in line})
    assert paths, "libhipattn.so is loaded, so the HIP runtime must be"
    # another copy may be mapped as well (a Python package that bundles its own): take the ROCm
    # installation's, which is the one libhipattn.so is linked against
    rocm = [q for q in paths if os.path.realpath(q).startswith(os.path.realpath("/opt/rocm"))]
    rt = ctypes.CDLL((rocm or paths)[0])
    vp = ctypes.c_void_p
    rt.hipStreamBeginCapture.argtypes = [vp, ctypes.c_int]
    rt.hipStreamEndCapture.argtypes = [vp, ctypes.POINTER(vp)]
    rt.hipGraphInstantiate.argtypes = [ctypes.POINTER(vp), vp, vp, vp, ctypes.c_size_t]
    rt.hipGraphLaunch.argtypes = [vp, vp]
    rt.hipGraphExecDestroy.argtypes = [vp]
    rt.hipGraphDestroy.argtypes = [vp]
    return rt


@pytest.mark.parametrize("batch", ["decode", "mixed"])
@pytest.mark.parametrize("cache_dtype,D,bs", [(W.F16, 128, 32), (W.U8, 128, 32), (W.F16, 64, 16), (W.F16, 96, 32), (W.F16, 256, 16), (W.F16, 192, 16),  # the stream-K kernels
                                              (W.F16, 96, 64), (W.F16, 192, 8)])                                                     # the query-tile kernel
def test_paged_attention_replays_from_a_graph(hip, oracle, batch, cache_dtype, D, bs):
    print("[case] graph capture", batch, cache_dtype, D, bs, flush=True)
    if batch == "decode":
        seqs = [(c - 1, 1) for c in (700, 64, 1500, 33, 2049, 5)]
    else:
        seqs = [(0, 130), (37, 1), (500, 1), (100, 257), (999, 1), (64, 1), (700, 128)]
    case = W.make_paged_case(95, seqs, 16, 4, D, bs, W.F16, W.F16, cache_dtype, sliding_window=0)
    ref, okc, ovc = H.oracle_paged(oracle, case)
    rt = hip_runtime()
    stream = hip.Stream()
    dev = H.PagedDeviceCase(hip, case)
    desc = H.pa_desc(hip, case)
    ws = hip.DeviceBuffer(hip.paged_attention_workspace_size(desc))
    shape = (case["T"], case["Hq"] * case["D"])

    def call():
        hip.paged_attention(desc, dev.q, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache, dev.past_lens,
                            dev.subsequence_begins, dev.block_indices, dev.block_indices_begins, dev.out, ws, stream)

    call()  # eager: also makes whatever the library sets up on a device's first call
    eager = dev.out.download(np.uint16, shape, stream)
    assert H.max_abs(H.storage_to_f32(eager, W.F16), ref) <= (1e-2 if cache_dtype == W.U8 else 2e-3)

    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.hipStreamBeginCapture(stream.handle, CAPTURE_MODE_RELAXED) == 0
    try:
        call()
    finally:
        status = rt.hipStreamEndCapture(stream.handle, ctypes.byref(graph))
    assert status == 0 and graph.value
    assert rt.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0
    try:
        for replay in range(3):
            dev.out.fill(0xFF, stream)  # eager work between the replays
            stream.synchronize()
            assert rt.hipGraphLaunch(graph_exec, stream.handle) == 0
            got = dev.out.download(np.uint16, shape, stream)
            np.testing.assert_array_equal(got, eager, err_msg="replay %d" % replay)
            if replay == 1:
                call()  # an eager call of the same work between two replays
                np.testing.assert_array_equal(dev.out.download(np.uint16, shape, stream), eager)
        kc, vc = dev.caches()
        np.testing.assert_array_equal(kc, okc)
        np.testing.assert_array_equal(vc, ovc)
    finally:
        rt.hipGraphExecDestroy(graph_exec)
        rt.hipGraphDestroy(graph)
        ws.free()
        dev.free()
        stream.close()
