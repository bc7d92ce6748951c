"""The attention operators through the plugin layer (Plugin -> CompiledModel -> InferRequest ->
SdpaOp / PagedAttentionOp -> C ABI -> HIP kernels), compared with the CPU oracle.  The SDPA cases
are the ones the reference's functional test instantiates for device "NVIDIA"
(modules/nvidia_plugin/tests/functional/shared_tests_instances/single_layer_tests/
scaled_dot_product_attention.cpp:76-137), with its f16 threshold tightened from 0.025 to 2e-3."""
import numpy as np
import pytest

import helpers as H
from openvino_contrib_amd import plugin_capi as P
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu


def _run_sdpa(plugin, case, causal, q_pshape, kv_pshape, compiled=None):
    compiled = compiled or plugin.compile_model(P.Model.sdpa(case["dtype"], q_pshape, kv_pshape, causal))
    req = compiled.create_infer_request()
    for i, name in enumerate(("q", "k", "v")):
        req.set_input(i, case[name + "_store"], case["dtype"])
    req.infer()
    out, dt = req.output(0)
    assert dt == case["dtype"]
    return H.storage_to_f32(out, case["dtype"]), compiled


@pytest.mark.parametrize("shape", [(1, 1, 4, 8), (1, 4, 16, 32), (1, 8, 32, 64)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [W.F32, W.F16])
def test_sdpa_reference_shapes_4d(hip, oracle, shape, causal, dtype):
    print("[plugin] sdpa 4d", shape, causal, dtype, flush=True)
    B, Hh, L, D = shape
    case = W.make_sdpa_case(91, B, Hh, Hh, L, L, D, dtype)
    out, _ = _run_sdpa(P.Plugin(), case, causal, list(shape), list(shape))
    ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=causal)
    assert out.shape == tuple(shape)
    assert H.max_abs(out, ref) <= (1e-4 if dtype == W.F32 else 2e-3)


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_reference_shape_3d(hip, oracle, causal):
    print("[plugin] sdpa 3d", causal, flush=True)
    case = W.make_sdpa_case(92, 1, 4, 4, 2, 2, 8, W.F32)
    c3 = dict(case)
    for n in ("q", "k", "v"):
        c3[n + "_store"] = case[n + "_store"].reshape(4, 2, 8)
    out, _ = _run_sdpa(P.Plugin(), c3, causal, [4, 2, 8], [4, 2, 8])
    ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=causal)
    assert H.max_abs(out.reshape(1, 4, 2, 8), ref) <= 1e-4


def test_sdpa_dynamic_shapes_one_compiled_model(hip, oracle):
    """One compiled model with dynamic sequence length serves requests of different lengths
    (tests/unit/dynamic_shape.cpp:165-283 does the same through Plugin::compile_model)."""
    plugin = P.Plugin()
    compiled = None
    for L in (5, 77, 300, 128):
        print("[plugin] sdpa dynamic L", L, flush=True)
        case = W.make_sdpa_case(93 + L, 2, 8, 2, L, L, 128, W.BF16, std=0.5)
        out, compiled = _run_sdpa(plugin, case, True, [-1, 8, -1, 128], [-1, 2, -1, 128], compiled)
        ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=True)
        assert out.shape == (2, 8, L, 128)
        assert H.max_abs(out, ref) <= 1e-2
    with pytest.raises(P.PluginError):  # wrong rank for the model's partial shape
        compiled.create_infer_request().set_input(0, np.zeros((8, 5, 128), np.uint16), W.BF16)
    with pytest.raises(P.PluginError):  # wrong precision
        compiled.create_infer_request().set_input(0, np.zeros((2, 8, 5, 128), np.float32), W.F32)
    with pytest.raises(P.PluginError):  # inputs not set
        compiled.create_infer_request().infer()


MIXED_BATCH = [(0, 130), (37, 1), (500, 1), (100, 257), (999, 1), (64, 1)]
LOOKS_LIKE_DECODE = [(1500, 1), (100, 2), (31, 0)]  # as many tokens as sequences, but not one each


@pytest.mark.parametrize("cache_dtype,q_dtype,window,seqs", [(W.F16, W.F16, 0, MIXED_BATCH), (W.U8, W.F16, 0, MIXED_BATCH),
                                                              (W.F16, W.BF16, 200, MIXED_BATCH),
                                                              (W.F16, W.F16, 64, LOOKS_LIKE_DECODE)])
def test_paged_attention_with_device_resident_cache(hip, oracle, cache_dtype, q_dtype, window, seqs):
    print("[plugin] paged attention", cache_dtype, q_dtype, window, seqs, flush=True)
    case = W.make_paged_case(94, seqs, 16, 4, 128, 32, q_dtype, q_dtype, cache_dtype, sliding_window=window)
    plugin = P.Plugin()
    plugin.set_property("PERF_COUNT", "YES")
    compiled = plugin.compile_model(P.Model.paged_attention(q_dtype, q_dtype, cache_dtype, 16, 4, 128, 32))
    assert compiled.input_names()[3:5] == ["key_cache", "value_cache"]
    assert compiled.get_property("EXECUTION_DEVICES") == "HIP.0"
    # the caches live on the device and are handed over as device tensors
    kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
    vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
    req = compiled.create_infer_request()
    req.set_input(0, case["q_store"], q_dtype)
    req.set_input(1, case["k_new_store"], q_dtype)
    req.set_input(2, case["v_new_store"], q_dtype)
    elem_shape = list(case["key_cache"].shape[:3]) + [case["key_cache"].shape[3] // hip.DTYPE_BYTES[cache_dtype]]
    req.set_device_input(3, kc.ptr, cache_dtype, elem_shape)
    req.set_device_input(4, vc.ptr, cache_dtype, elem_shape)
    req.set_input(5, case["past_lens"], P.I32)
    req.set_input(6, case["subsequence_begins"], P.I32)
    req.set_input(7, case["block_indices"], P.I32)
    req.set_input(8, case["block_indices_begins"], P.I32)
    req.set_input(9, np.zeros((0,), np.float32), W.F32)               # scale: default
    req.set_input(10, np.array([window], np.int32), P.I32)
    req.set_input(11, np.zeros((0,), np.float32), W.F32)              # no alibi slopes
    req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
    req.start_async()
    req.wait()
    out, _ = req.output(0)
    out = H.storage_to_f32(out, q_dtype)
    ref, okc, ovc = H.oracle_paged(oracle, case)
    tol = 1e-2 if (cache_dtype == W.U8 or q_dtype == W.BF16) else 2e-3
    assert H.max_abs(out, ref) <= tol
    # the operator updated the device-resident caches in place, bit for bit as the oracle does
    np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), okc)
    np.testing.assert_array_equal(vc.download(np.uint8, case["value_cache"].shape), ovc)
    prof = req.profiling()
    assert [t for _, t, _ in prof] == ["PagedAttentionExtension", "Result"]
    assert prof[0][2] > 0
    kc.free()
    vc.free()


def test_profiling_must_be_enabled(hip):
    plugin = P.Plugin()
    case = W.make_sdpa_case(95, 1, 1, 1, 4, 4, 8, W.F32)
    compiled = plugin.compile_model(P.Model.sdpa(W.F32, [1, 1, 4, 8], [1, 1, 4, 8], False))
    req = compiled.create_infer_request()
    for i, n in enumerate(("q", "k", "v")):
        req.set_input(i, case[n + "_store"], W.F32)
    req.infer()
    with pytest.raises(P.PluginError):
        req.profiling()
    with pytest.raises(P.PluginError):
        plugin.compile_model(P.Model.sdpa(W.F32, [1, 1, 4, 8], [1, 1, 4, 8], False), {"DEVICE_ID": 99})
