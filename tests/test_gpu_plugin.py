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


def test_set_tensors_puts_one_tensor_per_batch_entry_together(hip, oracle):
    """set_tensors on an input (several tensors, one batch entry each, src/cuda_infer_request.cpp:263-272):
    the request joins them along the batch axis when it runs; a single tensor set later replaces them;
    tensors that do not fit are refused with an error."""
    print("[plugin] set_tensors", flush=True)
    B, Hh, L, D = 3, 4, 40, 64
    case = W.make_sdpa_case(99, B, Hh, Hh, L, L, D, W.F16)
    plugin = P.Plugin()
    compiled = plugin.compile_model(P.Model.sdpa(W.F16, [-1, Hh, -1, D], [-1, Hh, -1, D], True))
    req = compiled.create_infer_request()
    req.set_input_batch(0, [case["q_store"][b:b + 1] for b in range(B)], W.F16)
    req.set_input(1, case["k_store"], W.F16)
    req.set_input_batch(2, [case["v_store"][b:b + 1] for b in range(B)], W.F16)
    req.infer()
    out, _ = req.output(0)
    ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=True)
    assert out.shape == (B, Hh, L, D) and H.max_abs(H.storage_to_f32(out, W.F16), ref) <= 2e-3
    # the tensors are read again by every infer: new values in the same memory, new result
    case2 = W.make_sdpa_case(100, B, Hh, Hh, L, L, D, W.F16)
    req.set_input_batch(0, [case2["q_store"][b:b + 1] for b in range(B)], W.F16)
    req.infer()
    out2, _ = req.output(0)
    assert H.max_abs(H.storage_to_f32(out2, W.F16), oracle.sdpa(case2["q"], case["k"], case["v"], causal=True)) <= 2e-3
    # one tensor for the whole input takes the place of the batch
    req.set_input(0, case["q_store"], W.F16)
    req.infer()
    out3, _ = req.output(0)
    np.testing.assert_array_equal(out3, out)
    with pytest.raises(P.PluginError):  # an entry that is more than one batch entry
        req.set_input_batch(0, [case["q_store"][0:2], case["q_store"][1:3]], W.F16)
    with pytest.raises(P.PluginError):  # the wrong precision
        req.set_input_batch(0, [np.zeros((1, Hh, L, D), np.float32)] * 2, W.F32)


def test_runtime_model_carries_execution_information(hip, oracle):
    """get_runtime_model (src/cuda_compiled_model.cpp:336-371): every node with its type, place in the execution
    order, precision and, with profiling on, the average time of its executions so far."""
    print("[plugin] runtime model", flush=True)
    case = W.make_sdpa_case(101, 1, 4, 4, 64, 64, 64, W.F16)
    plugin = P.Plugin()
    plugin.set_property("PERF_COUNT", "YES")
    compiled = plugin.compile_model(P.Model.sdpa(W.F16, [1, 4, 64, 64], [1, 4, 64, 64], True))
    before = compiled.runtime_info()
    assert [r[2] for r in before] == [str(i) for i in range(len(before))]
    assert "ScaledDotProductAttention" in [r[1] for r in before]
    assert all(r[3] == "not_executed" and r[5] == "HIP" for r in before)
    req = compiled.create_infer_request()
    for i, name in enumerate(("q", "k", "v")):
        req.set_input(i, case[name + "_store"], W.F16)
    for _ in range(3):
        req.infer()
    after = {r[1]: r for r in compiled.runtime_info()}
    sdpa = after["ScaledDotProductAttention"]
    assert sdpa[3] != "not_executed" and int(sdpa[3]) > 0 and sdpa[4] == "f16"
    # without profiling nothing is timed
    quiet = P.Plugin().compile_model(P.Model.sdpa(W.F16, [1, 4, 64, 64], [1, 4, 64, 64], True))
    r2 = quiet.create_infer_request()
    for i, name in enumerate(("q", "k", "v")):
        r2.set_input(i, case[name + "_store"], W.F16)
    r2.infer()
    assert all(r[3] == "not_executed" for r in quiet.runtime_info())


MIXED_BATCH = [(0, 130), (37, 1), (500, 1), (100, 257), (999, 1), (64, 1)]
LOOKS_LIKE_DECODE = [(1500, 1), (100, 2), (31, 0)]  # as many tokens as sequences, but not one each


@pytest.mark.parametrize("shape", [(16, 4, 128, 32), (8, 2, 256, 64), (12, 4, 96, 16)])
@pytest.mark.parametrize("cache_dtype,q_dtype,window,seqs", [(W.F16, W.F16, 0, MIXED_BATCH), (W.U8, W.F16, 0, MIXED_BATCH),
                                                              (W.F16, W.BF16, 200, MIXED_BATCH),
                                                              (W.F16, W.F16, 64, LOOKS_LIKE_DECODE)])
def test_paged_attention_with_device_resident_cache(hip, oracle, cache_dtype, q_dtype, window, seqs, shape):
    print("[plugin] paged attention", cache_dtype, q_dtype, window, seqs, shape, flush=True)
    Hq, Hkv, D, bs = shape  # (nothing in the operator is fixed to a head size or a cache block size)
    case = W.make_paged_case(94, seqs, Hq, Hkv, D, bs, q_dtype, q_dtype, cache_dtype, sliding_window=window)
    plugin = P.Plugin()
    plugin.set_property("PERF_COUNT", "YES")
    # the operator's full signature: four empty optional inputs behind max_context_len and the scores output
    compiled = plugin.compile_model(P.Model.paged_attention(q_dtype, q_dtype, cache_dtype, Hq, Hkv, D, bs,
                                                            extra_inputs=4, extra_len=0, scores_result=True))
    assert compiled.input_names()[3:5] == ["key_cache", "value_cache"]
    assert compiled.get_property("EXECUTION_DEVICES") == "HIP.0"
    assert compiled.num_outputs() == 2
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
    req.set_input(13, np.zeros((0,), np.int32), P.I32)                # score_aggregation_window: off
    req.set_input(14, np.zeros((0,), np.int32), P.I32)                # no cache rotation
    req.set_input(15, np.zeros((0,), np.int32), P.I32)
    req.set_input(16, np.zeros((0,), np.float32), W.F32)
    req.start_async()
    req.wait()
    out, _ = req.output(0)
    scores, _ = req.output(1)
    out = H.storage_to_f32(out, q_dtype)
    ref, okc, ovc = H.oracle_paged(oracle, case)
    # the scores Result is connected, so the second output is produced: every new token aggregated
    ref_scores = oracle.paged_attention_scores(case["q"], okc, cache_dtype, case["past_lens"], case["subsequence_begins"],
                                               case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs,
                                               sliding_window=window)
    assert scores.dtype == np.float32 and scores.shape == ref_scores.shape
    assert H.max_abs(scores, ref_scores) <= 2e-5 * max(1.0, float(ref_scores.max()))
    tol = 1e-2 if (cache_dtype == W.U8 or q_dtype == W.BF16) else 2e-3
    assert H.max_abs(out, ref) <= tol
    # the operator updated the device-resident caches in place, bit for bit as the oracle does
    np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), okc)
    np.testing.assert_array_equal(vc.download(np.uint8, case["value_cache"].shape), ovc)
    prof = req.profiling()
    assert [t for _, t, _ in prof] == ["PagedAttentionExtension", "Result", "Result"]
    assert prof[0][2] > 0
    kc.free()
    vc.free()


@pytest.mark.parametrize("cache_dtype,seqs", [(W.F16, MIXED_BATCH), (W.U8, [(700, 1), (31, 1), (1500, 1)])])
def test_paged_attention_with_alibi_slopes_through_the_plugin(hip, oracle, cache_dtype, seqs):
    """alibi_slopes with one value per query head: the model is supported, the slopes go to the device with the
    other inputs and the result is the oracle's with its distance term; an empty input is no bias."""
    print("[plugin] paged attention with alibi slopes", cache_dtype, flush=True)
    Hq, Hkv, D, bs = 16, 4, 128, 32
    case = W.make_paged_case(98, seqs, Hq, Hkv, D, bs, W.F16, W.F16, cache_dtype)
    slopes = (2.0 ** (-8.0 * np.arange(1, Hq + 1) / Hq)).astype(np.float32)
    plugin = P.Plugin()
    model = P.Model.paged_attention(W.F16, W.F16, cache_dtype, Hq, Hkv, D, bs, alibi_len=Hq)
    assert "paged_attention" in plugin.query_model(model)
    compiled = plugin.compile_model(model)
    kc_ref, vc_ref = case["key_cache"].copy(), case["value_cache"].copy()
    ref = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc_ref, vc_ref, cache_dtype, case["past_lens"],
                                 case["subsequence_begins"], case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs,
                                 alibi_slopes=slopes)
    kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
    vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
    req = compiled.create_infer_request()
    elem_shape = list(case["key_cache"].shape[:3]) + [case["key_cache"].shape[3] // hip.DTYPE_BYTES[cache_dtype]]
    for i, a in enumerate((case["q_store"], case["k_new_store"], case["v_new_store"])):
        req.set_input(i, a, W.F16)
    req.set_device_input(3, kc.ptr, cache_dtype, elem_shape)
    req.set_device_input(4, vc.ptr, cache_dtype, elem_shape)
    for i, n in enumerate(("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")):
        req.set_input(5 + i, case[n], P.I32)
    req.set_input(9, np.zeros((0,), np.float32), W.F32)
    req.set_input(10, np.array([0], np.int32), P.I32)
    req.set_input(11, slopes, W.F32)
    req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
    req.infer()
    out, _ = req.output(0)
    tol = 1e-2 if cache_dtype == W.U8 else 2e-3
    assert H.scaled_bound_error(H.storage_to_f32(out, W.F16), ref, "plugin alibi") <= tol
    np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), kc_ref)
    with pytest.raises(P.PluginError):  # one slope per query head, or none
        req.set_input(11, slopes[:3], W.F32)
        req.infer()
    kc.free()
    vc.free()


def test_decode_steps_replay_the_graph_while_the_context_bound_grows(hip, oracle):
    """A decode loop as a server runs it: every tensor device-resident, past_lens advanced in place, and
    max_context_len (a host scalar, advisory for the attention kernels) one larger every step.  The steps
    after the second replay the recorded graph all the same, and the last one still matches the oracle."""
    print("[plugin] decode loop under graph replay", flush=True)
    from openvino_contrib_amd import device_case as DC
    Hq, Hkv, D, bs = 16, 4, 128, 32
    past0 = [700, 64, 1500, 33]
    steps = 5
    # room in the block tables for the tokens of every step
    case = W.make_paged_case(102, [(p + steps, 1) for p in past0], Hq, Hkv, D, bs, W.F16, W.F16, W.F16)
    dev = DC.PagedDeviceCase(hip, case)
    plugin = P.Plugin()
    compiled = plugin.compile_model(P.Model.paged_attention(W.F16, W.F16, W.F16, Hq, Hkv, D, bs), {"HIP_GRAPH_MIN_OPERATORS": "1"})
    req = compiled.create_infer_request()
    T, S = case["T"], case["S"]
    cache_shape = list(case["key_cache"].shape[:3]) + [D]
    req.set_device_input(0, dev.q.ptr, W.F16, [T, Hq * D])
    req.set_device_input(1, dev.k_new.ptr, W.F16, [T, Hkv * D])
    req.set_device_input(2, dev.v_new.ptr, W.F16, [T, Hkv * D])
    req.set_device_input(3, dev.key_cache.ptr, W.F16, cache_shape)
    req.set_device_input(4, dev.value_cache.ptr, W.F16, cache_shape)
    req.set_device_input(5, dev.past_lens.ptr, P.I32, [S])
    req.set_device_input(6, dev.subsequence_begins.ptr, P.I32, [S + 1])
    req.set_device_input(7, dev.block_indices.ptr, P.I32, [len(case["block_indices"])])
    req.set_device_input(8, dev.block_indices_begins.ptr, P.I32, [S + 1])
    req.set_input(9, np.zeros((0,), np.float32), W.F32)
    req.set_input(10, np.array([0], np.int32), P.I32)
    req.set_input(11, np.zeros((0,), np.float32), W.F32)
    req.set_device_output(0, dev.out.ptr, W.F16, [T, Hq * D])
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    launches = []
    for step in range(steps):
        lens = np.array([p + step for p in past0], np.int32)
        dev.past_lens.upload(lens)
        req.set_input(12, np.array([int(lens.max()) + 1], np.int32), P.I32)  # grows with every step
        req.infer()
        launches.append(int(compiled.get_property("HIP_GRAPH_LAUNCHES")))
        ref = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, W.F16, lens, case["subsequence_begins"],
                                     case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs)
        out = H.storage_to_f32(dev.out.download(np.uint16, (T, Hq * D)), W.F16)
        assert H.max_abs(out, ref) <= 2e-3, step
    assert launches == [0, 1, 2, 3, 4], launches  # recorded at the second step, replayed from then on
    got_kc, got_vc = dev.caches()
    np.testing.assert_array_equal(got_kc, kc)
    np.testing.assert_array_equal(got_vc, vc)
    dev.free()


def test_paged_attention_scores_over_an_aggregation_window(hip, oracle):
    """score_aggregation_window holds one value per sequence: only that many of a sequence's last
    query tokens are aggregated.  Without a consumer of output 1 nothing is computed for it."""
    print("[plugin] paged attention scores with a window", flush=True)
    seqs = MIXED_BATCH
    window = [4, 1, 0, 300, 1, 1]
    case = W.make_paged_case(97, seqs, 16, 4, 128, 32, W.F16, W.F16, W.F16)
    plugin = P.Plugin()
    for with_scores in (True, False):
        compiled = plugin.compile_model(P.Model.paged_attention(W.F16, W.F16, W.F16, 16, 4, 128, 32, extra_inputs=1,
                                                                extra_len=len(seqs), scores_result=with_scores))
        kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
        vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
        req = compiled.create_infer_request()
        elem_shape = list(case["key_cache"].shape[:3]) + [128]
        for i, (a, dt) in enumerate([(case["q_store"], W.F16), (case["k_new_store"], W.F16), (case["v_new_store"], W.F16)]):
            req.set_input(i, a, dt)
        req.set_device_input(3, kc.ptr, W.F16, elem_shape)
        req.set_device_input(4, vc.ptr, W.F16, elem_shape)
        for i, n in enumerate(("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")):
            req.set_input(5 + i, case[n], P.I32)
        req.set_input(9, np.zeros((0,), np.float32), W.F32)
        req.set_input(10, np.array([0], np.int32), P.I32)
        req.set_input(11, np.zeros((0,), np.float32), W.F32)
        req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
        req.set_input(13, np.array(window, np.int32), P.I32)
        req.infer()
        out, _ = req.output(0)
        ref, okc, _ = H.oracle_paged(oracle, case)
        assert H.max_abs(H.storage_to_f32(out, W.F16), ref) <= 2e-3
        if with_scores:
            scores, _ = req.output(1)
            ref_scores = oracle.paged_attention_scores(case["q"], okc, W.F16, case["past_lens"], case["subsequence_begins"],
                                                       case["block_indices"], case["block_indices_begins"], 16, 4, 128, 32,
                                                       score_window=window)
            assert scores.shape == ref_scores.shape
            assert H.max_abs(scores, ref_scores) <= 2e-5 * max(1.0, float(ref_scores.max()))
            begin = sum(p + n for p, n in seqs[:2])
            assert not scores[begin:begin + sum(seqs[2])].any()  # a window of 0: nothing aggregated for that sequence
        else:
            assert compiled.num_outputs() == 1
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


@pytest.mark.parametrize("dtype,tol", [(W.F32, 1e-4), (W.F16, 2e-3)])
@pytest.mark.parametrize("mask_kind", ["bool_2d", "float_per_head", "none"])
@pytest.mark.parametrize("scale_kind", ["default", "constant", "parameter"])
def test_sdpa_with_mask_and_scale_inputs(hip, oracle, dtype, tol, mask_kind, scale_kind):
    """attention_mask and scale inputs of v13::ScaledDotProductAttention through the plugin; the
    reference executes them as Add / Select / Multiply nodes of the decomposed graph."""
    print("[plugin] sdpa mask/scale", dtype, mask_kind, scale_kind, flush=True)
    B, Hh, Lq, Lk, D = 2, 4, 33, 70, 64
    case = W.make_sdpa_case(96, B, Hh, Hh, Lq, Lk, D, dtype)
    rng = np.random.default_rng(97)
    mask, mask_dtype = None, None
    if mask_kind == "bool_2d":
        mask = rng.random((Lq, Lk)) < 0.6
        mask[:, 0] = True
        mask_dtype = P.BOOL
    elif mask_kind == "float_per_head":
        mask = (1.5 * rng.standard_normal((1, Hh, Lq, Lk))).astype(np.float32)
        mask_dtype = W.F32
    scale = {"default": 0.0, "constant": 0.21, "parameter": 0.07}[scale_kind]
    model = P.Model.sdpa(dtype, [-1, Hh, -1, D], [-1, Hh, -1, D], False, mask_dtype=mask_dtype,
                         mask_shape=[-1] * (mask.ndim if mask is not None else 0),
                         scale=(scale_kind == "parameter"), scale_constant=(scale if scale_kind == "constant" else None))
    compiled = P.Plugin().compile_model(model)
    req = compiled.create_infer_request()
    for i, name in enumerate(("q", "k", "v")):
        req.set_input(i, case[name + "_store"], dtype)
    nxt = 3
    if mask is not None or scale_kind != "default":
        if mask is not None:
            req.set_input(nxt, mask, mask_dtype)
        else:
            req.set_input(nxt, np.zeros((0,), W.np_storage_dtype(dtype)), dtype)  # the placeholder in front of scale
        nxt += 1
    if scale_kind == "parameter":
        req.set_input(nxt, np.array(scale, np.float32), W.F32)
    req.infer()
    out, _ = req.output(0)
    out = H.storage_to_f32(out, dtype)
    if mask is not None:
        ref = oracle.sdpa_masked(case["q"], case["k"], case["v"], mask, scale=scale)
    else:
        ref = oracle.sdpa(case["q"], case["k"], case["v"], scale=scale)
    assert H.max_abs(out, ref) <= tol


@pytest.mark.parametrize("dtype,shape,pshape", [(W.F32, (1, 4, 20, 20), None), (W.F16, (1, 4, 20, 20), None),
                                                (P.I32, (7, 4, 20, 20), None), (W.F32, (3, 4), (-1, 4)),
                                                (W.F32, (0, 4), (-1, 4))])
def test_read_value_assign_accumulator(hip, dtype, shape, pshape):
    """The stateful model of the reference's test (tests/functional/shared_tests_instances/
    single_layer_tests/read_value_assign.cpp:52-138, same shapes, precisions and input values,
    the empty initial state included): y = ReadValue(init = x) + x, Assign(y).  After a reset the
    variable reads as x, so the outputs run 2x, 3x, 4x; the state is device-resident."""
    print("[plugin] accumulator", dtype, shape, pshape, flush=True)
    n = int(np.prod(shape))
    x = (np.arange(n) % 10 + 1).astype(np.float32).reshape(shape)
    store = {W.F32: x, W.F16: W.to_storage(x, W.F16)[0], P.I32: x.astype(np.int32)}[dtype]
    value = (lambda a: W.f16_bits_to_f32(a)) if dtype == W.F16 else (lambda a: a.astype(np.float32))
    compiled = P.Plugin().compile_model(P.Model.accumulator(dtype, list(pshape or shape)))
    req = compiled.create_infer_request()
    assert req.states() == ["v0"]
    req.set_input(0, store, dtype)
    for k in (2, 3, 4):
        req.infer()
        out, _ = req.output(0)
        assert out.shape == tuple(shape)
        np.testing.assert_array_equal(value(out), k * x)
        np.testing.assert_array_equal(value(req.state_get()), k * x)  # the state is what was assigned
    req.state_reset()
    assert req.state_get().shape == tuple(0 if (pshape and pshape[i] < 0) else shape[i] for i in range(len(shape)))
    req.infer()
    np.testing.assert_array_equal(value(req.output(0)[0]), 2 * x)  # after reset the variable reads as the init value
    if n:
        req.state_set(store, dtype)  # set_state: the next ReadValue returns it
        req.infer()
        np.testing.assert_array_equal(value(req.output(0)[0]), 2 * x)
        req.infer()
        np.testing.assert_array_equal(value(req.output(0)[0]), 3 * x)
    # a second request of the same compiled model has a state of its own
    other = compiled.create_infer_request()
    other.set_input(0, store, dtype)
    other.infer()
    np.testing.assert_array_equal(value(other.output(0)[0]), 2 * x)


def test_state_grows_with_a_dynamic_shape(hip):
    """A variable with a dynamic extent takes the shape of what is assigned: grow-only capacity,
    logical shape per step (src/cuda_variable_state.hpp:135-183)."""
    compiled = P.Plugin().compile_model(P.Model.accumulator(W.F32, [-1, 4]))
    req = compiled.create_infer_request()
    for rows in (2, 5, 3):  # each new shape starts over from "state as large as the input"
        x = np.arange(rows * 4, dtype=np.float32).reshape(rows, 4)
        req.state_reset()
        req.set_input(0, x, W.F32)
        req.infer()
        req.infer()
        np.testing.assert_array_equal(req.output(0)[0], 3 * x)
        assert req.state_get().shape == (rows, 4)


def test_export_and_import_model(hip, oracle):
    """export_model writes [u64][model][u64][weights]; import_model compiles from it and says so
    (src/cuda_compiled_model.cpp:373-395, src/cuda_plugin.cpp:99-138)."""
    import struct
    plugin = P.Plugin()
    model = P.Model.sdpa(W.F16, [1, 8, -1, 64], [1, 8, -1, 64], False, mask_dtype=P.BOOL, mask_shape=[-1, -1],
                         scale_constant=0.2)
    compiled = plugin.compile_model(model)
    blob = compiled.export_model()
    n_model = struct.unpack_from("<Q", blob, 0)[0]
    n_weights = struct.unpack_from("<Q", blob, 8 + n_model)[0]
    assert len(blob) == 16 + n_model + n_weights and b"ScaledDotProductAttention" in blob[8:8 + n_model]
    assert compiled.get_property("LOADED_FROM_CACHE") == "NO"
    imported = plugin.import_model(blob, {"LOADED_FROM_CACHE": "YES"})
    assert imported.get_property("LOADED_FROM_CACHE") == "YES"
    assert imported.input_names() == compiled.input_names() == ["query", "key", "value", "attention_mask"]
    assert imported.export_model() == blob
    case = W.make_sdpa_case(98, 1, 8, 8, 19, 40, 64, W.F16)
    mask = np.random.default_rng(3).random((19, 40)) < 0.7
    mask[:, 1] = True
    outs = []
    for cm in (compiled, imported):
        req = cm.create_infer_request()
        for i, name in enumerate(("q", "k", "v")):
            req.set_input(i, case[name + "_store"], W.F16)
        req.set_input(3, mask, P.BOOL)
        req.infer()
        outs.append(req.output(0)[0])
    np.testing.assert_array_equal(outs[0], outs[1])
    ref = oracle.sdpa_masked(case["q"], case["k"], case["v"], mask, scale=0.2)
    assert H.max_abs(H.storage_to_f32(outs[1], W.F16), ref) <= 2e-3
    # a stateful model survives the round trip with its variable
    acc = plugin.import_model(plugin.compile_model(P.Model.accumulator(W.F32, [-1, 4])).export_model())
    req = acc.create_infer_request()
    x = np.ones((2, 4), np.float32)
    req.set_input(0, x, W.F32)
    req.infer()
    req.infer()
    np.testing.assert_array_equal(req.output(0)[0], 3 * x)


def test_async_pipeline_cancel_and_destruction(hip, oracle):
    """start_async / wait / cancel and the destructor's stop_and_wait
    (src/cuda_async_infer_request.cpp:26-61): a cancelled request ends with ov::Cancelled or, when
    it had already finished, normally; either way it can be used again; destroying a request that
    is still running waits for it."""
    case = W.make_sdpa_case(99, 2, 8, 2, 600, 600, 128, W.BF16, std=0.5)
    ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=True)
    compiled = P.Plugin().compile_model(P.Model.sdpa(W.BF16, [-1, 8, -1, 128], [-1, 2, -1, 128], True))
    req = compiled.create_infer_request()
    for i, name in enumerate(("q", "k", "v")):
        req.set_input(i, case[name + "_store"], W.BF16)
    cancelled = 0
    for _ in range(20):
        req.start_async()
        req.cancel()
        try:
            req.wait()
        except P.PluginError as e:
            assert e.code == P.CANCELLED
            cancelled += 1
    print("[plugin] cancelled", cancelled, "of 20", flush=True)
    req.infer()  # usable after cancellation
    assert H.max_abs(H.storage_to_f32(req.output(0)[0], W.BF16), ref) <= 1e-2
    req.cancel()  # idle: no effect
    req.start_async()
    req.wait()
    for _ in range(5):  # dropped while running: the destructor waits, nothing is left behind
        r2 = compiled.create_infer_request()
        for i, name in enumerate(("q", "k", "v")):
            r2.set_input(i, case[name + "_store"], W.BF16)
        r2.start_async()
        del r2
    # two requests in flight on the device's worker at once
    reqs = [compiled.create_infer_request() for _ in range(3)]
    for r in reqs:
        for i, name in enumerate(("q", "k", "v")):
            r.set_input(i, case[name + "_store"], W.BF16)
        r.start_async()
    for r in reqs:
        r.wait()
        assert H.max_abs(H.storage_to_f32(r.output(0)[0], W.BF16), ref) <= 1e-2


def test_output_left_on_the_device(hip, oracle):
    """An output port bound to a device tensor receives the result in place: nothing is downloaded."""
    case = W.make_sdpa_case(100, 1, 8, 2, 130, 130, 128, W.F16)
    compiled = P.Plugin().compile_model(P.Model.sdpa(W.F16, [-1, 8, -1, 128], [-1, 2, -1, 128], True))
    req = compiled.create_infer_request()
    bufs = [hip.DeviceBuffer.from_numpy(case[n + "_store"]) for n in ("q", "k", "v")]
    out = hip.DeviceBuffer(case["q_store"].nbytes)
    out.fill(0xFF)
    for i, (b, n) in enumerate(zip(bufs, ("q", "k", "v"))):
        req.set_device_input(i, b.ptr, W.F16, case[n + "_store"].shape)
    req.set_device_output(0, out.ptr, W.F16, case["q_store"].shape)
    req.infer()
    res = H.storage_to_f32(out.download(np.uint16, case["q_store"].shape), W.F16)
    assert H.max_abs(res, oracle.sdpa(case["q"], case["k"], case["v"], causal=True)) <= 2e-3
    for b in bufs + [out]:
        b.free()


def test_paged_attention_with_host_bound_caches_writes_them_back(hip, oracle):
    """KV caches bound as host tensors are uploaded, updated by the operator and copied back, so the
    caller's arrays hold the new rows (a device tensor avoids both copies; this is the slow, safe way)."""
    seqs = [(37, 1), (0, 70), (500, 1)]
    case = W.make_paged_case(101, seqs, 8, 2, 128, 32, W.F16, W.F16, W.F16)
    compiled = P.Plugin().compile_model(P.Model.paged_attention(W.F16, W.F16, W.F16, 8, 2, 128, 32))
    req = compiled.create_infer_request()
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    elem_shape = list(kc.shape[:3]) + [kc.shape[3] // 2]
    req.set_input(0, case["q_store"], W.F16)
    req.set_input(1, case["k_new_store"], W.F16)
    req.set_input(2, case["v_new_store"], W.F16)
    req.set_input(3, kc.view(np.uint16).reshape(elem_shape), W.F16)
    req.set_input(4, vc.view(np.uint16).reshape(elem_shape), W.F16)
    req.set_input(5, case["past_lens"], P.I32)
    req.set_input(6, case["subsequence_begins"], P.I32)
    req.set_input(7, case["block_indices"], P.I32)
    req.set_input(8, case["block_indices_begins"], P.I32)
    req.set_input(9, np.zeros((0,), np.float32), W.F32)
    req.set_input(10, np.array([0], np.int32), P.I32)
    req.set_input(11, np.zeros((0,), np.float32), W.F32)
    req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
    req.infer()
    ref, okc, ovc = H.oracle_paged(oracle, case)
    assert H.max_abs(H.storage_to_f32(req.output(0)[0], W.F16), ref) <= 2e-3
    np.testing.assert_array_equal(kc, okc)  # the caller's own arrays now hold the new rows
    np.testing.assert_array_equal(vc, ovc)


@pytest.mark.parametrize("cache_dtype,per_token", [(W.F16, False), (W.U8, True), (W.BF16, True)])
def test_paged_attention_with_cache_rotation_through_the_plugin(hip, oracle, cache_dtype, per_token):
    """rotated_block_indices, rotation_deltas and rotation_trig_lut with data: the listed key blocks are turned
    before the step's keys are stored and the attention runs on the turned cache; against the oracle's rotation
    followed by its attention, cache bytes bit-exact.  With the three inputs empty nothing is turned."""
    print("[plugin] paged attention with cache rotation", cache_dtype, per_token, flush=True)
    Hq, Hkv, D, bs = 8, 2, 128, 32
    seqs = [(200, 1), (70, 3), (0, 40), (500, 1)]
    qd = W.BF16 if cache_dtype == W.BF16 else W.F16
    case = W.make_paged_case(99, seqs, Hq, Hkv, D, bs, qd, qd, cache_dtype)
    begins, ids, nb = case["block_indices_begins"], case["block_indices"], case["num_blocks"]
    theta = 10000.0 ** (-np.arange(D // 2, dtype=np.float64) * 2.0 / D)
    ang = np.arange(64, dtype=np.float64)[:, None] * theta[None, :]
    lut = np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)
    rng = np.random.default_rng(3)
    rotated = np.array([ids[begins[0] + 1], ids[begins[0] + 2], ids[begins[3] + 7], nb + 1, ids[begins[1]]], np.int32)
    deltas = rng.integers(0, 64, (len(rotated), bs if per_token else 1)).astype(np.int32)
    g = P.GraphText("pa_rotation")
    el = {W.F16: "f16", W.BF16: "bf16", W.U8: "u8"}
    qp = g.parameter("q", qd, [-1, Hq * D])
    kp = g.parameter("k", qd, [-1, Hkv * D])
    vp = g.parameter("v", qd, [-1, Hkv * D])
    row = case["key_cache"].shape[3] // hip.DTYPE_BYTES[cache_dtype]
    kcp = g.parameter("key_cache", cache_dtype, [-1, Hkv, bs, row])
    vcp = g.parameter("value_cache", cache_dtype, [-1, Hkv, bs, row])
    idx = [g.parameter(n, P.I32, [-1]) for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")]
    rest = [g.parameter("scale", W.F32, [-1]), g.parameter("sliding_window", P.I32, [-1]), g.parameter("alibi_slopes", W.F32, [-1]),
            g.parameter("max_context_len", P.I32, [-1]), g.parameter("score_aggregation_window", P.I32, [-1]),
            g.parameter("rotated_block_indices", P.I32, [-1]), g.parameter("rotation_deltas", P.I32, [-1, -1]),
            g.parameter("rotation_trig_lut", W.F32, [-1, D])]
    pa = g.add("PagedAttentionExtension", "attention", [qp, kp, vp, kcp, vcp] + idx + rest)
    g.result("out", pa)
    plugin = P.Plugin()
    assert "attention" in plugin.query_model(g.model())
    compiled = plugin.compile_model(g.model())
    req = compiled.create_infer_request()
    cache_shape = list(case["key_cache"].shape[:3]) + [row]
    for use in (True, False):
        kc_ref, vc_ref = case["key_cache"].copy(), case["value_cache"].copy()
        if use:
            oracle.rotate_key_cache(kc_ref, cache_dtype, rotated, deltas, lut, Hkv, D, bs)
        ref = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc_ref, vc_ref, cache_dtype, case["past_lens"],
                                     case["subsequence_begins"], ids, begins, Hq, Hkv, D, bs)
        kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
        vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
        host = {"q": (case["q_store"], qd), "k": (case["k_new_store"], qd), "v": (case["v_new_store"], qd),
                "past_lens": (case["past_lens"], P.I32), "subsequence_begins": (case["subsequence_begins"], P.I32),
                "block_indices": (ids, P.I32), "block_indices_begins": (begins, P.I32),
                "scale": (np.zeros((0,), np.float32), W.F32), "sliding_window": (np.array([0], np.int32), P.I32),
                "alibi_slopes": (np.zeros((0,), np.float32), W.F32),
                "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32),
                "score_aggregation_window": (np.zeros((0,), np.int32), P.I32),
                "rotated_block_indices": (rotated if use else np.zeros((0,), np.int32), P.I32),
                "rotation_deltas": (deltas if use else np.zeros((0, 1), np.int32), P.I32),
                "rotation_trig_lut": (lut if use else np.zeros((0, D), np.float32), W.F32)}
        for i, n in enumerate(compiled.input_names()):
            if n in host:
                req.set_input(i, *host[n])
            else:
                req.set_device_input(i, (kc if n == "key_cache" else vc).ptr, cache_dtype, cache_shape)
        req.infer()
        out, _ = req.output(0)
        np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), kc_ref)
        np.testing.assert_array_equal(vc.download(np.uint8, case["value_cache"].shape), vc_ref)
        tol = 2e-3 if cache_dtype == W.F16 else 1e-2
        assert H.scaled_bound_error(H.storage_to_f32(out, qd), ref, "plugin cache rotation %s" % use) <= tol
        kc.free()
        vc.free()


@pytest.mark.parametrize("seqs", [[(300, 1), (70, 1), (1000, 1), (5, 1)], [(200, 1), (70, 3), (0, 140), (500, 1)]])
def test_paged_attention_with_sinks_through_the_plugin(hip, oracle, seqs):
    """The operator's last input, sinks, with one f32 logit per query head (as [1, heads, 1, 1]), on a shape of the
    models that carry it: head size 64, 64 query heads on 8 kv heads, a sliding window of 128, bf16.  Against the
    oracle; the sparse-attention inputs in front of it stay empty."""
    print("[plugin] paged attention with sinks", len(seqs), flush=True)
    Hq, Hkv, D, bs, window = 64, 8, 64, 32, 128
    case = W.make_paged_case(100, seqs, Hq, Hkv, D, bs, W.BF16, W.BF16, W.BF16, sliding_window=window)
    sinks = np.random.default_rng(8).uniform(-1.0, 3.0, Hq).astype(np.float32)
    g = P.GraphText("pa_sinks")
    qp = g.parameter("q", W.BF16, [-1, Hq * D])
    kp = g.parameter("k", W.BF16, [-1, Hkv * D])
    vp = g.parameter("v", W.BF16, [-1, Hkv * D])
    kcp = g.parameter("key_cache", W.BF16, [-1, Hkv, bs, D])
    vcp = g.parameter("value_cache", W.BF16, [-1, Hkv, bs, D])
    idx = [g.parameter(n, P.I32, [-1]) for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")]
    rest = [g.parameter("scale", W.F32, [-1]), g.parameter("sliding_window", P.I32, [-1]), g.parameter("alibi_slopes", W.F32, [-1]),
            g.parameter("max_context_len", P.I32, [-1]), g.parameter("score_aggregation_window", P.I32, [-1]),
            g.parameter("rotated_block_indices", P.I32, [-1]), g.parameter("rotation_deltas", P.I32, [-1, -1]),
            g.parameter("rotation_trig_lut", W.F32, [-1, D]), g.parameter("xattention_threshold", W.F32, [-1]),
            g.parameter("xattention_block_size", P.I32, [-1]), g.parameter("xattention_stride", P.I32, [-1]),
            g.parameter("sinks", W.F32, [1, -1, 1, 1])]
    g.result("out", g.add("PagedAttentionExtension", "attention", [qp, kp, vp, kcp, vcp] + idx + rest))
    plugin = P.Plugin()
    assert "attention" in plugin.query_model(g.model())
    compiled = plugin.compile_model(g.model())
    req = compiled.create_infer_request()
    kc_ref, vc_ref = case["key_cache"].copy(), case["value_cache"].copy()
    ref = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc_ref, vc_ref, W.BF16, case["past_lens"],
                                 case["subsequence_begins"], case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs,
                                 sliding_window=window, sinks=sinks)
    kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
    vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
    empty_i, empty_f = (np.zeros((0,), np.int32), P.I32), (np.zeros((0,), np.float32), W.F32)
    host = {"q": (case["q_store"], W.BF16), "k": (case["k_new_store"], W.BF16), "v": (case["v_new_store"], W.BF16),
            "past_lens": (case["past_lens"], P.I32), "subsequence_begins": (case["subsequence_begins"], P.I32),
            "block_indices": (case["block_indices"], P.I32), "block_indices_begins": (case["block_indices_begins"], P.I32),
            "scale": empty_f, "sliding_window": (np.array([window], np.int32), P.I32), "alibi_slopes": empty_f,
            "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32), "score_aggregation_window": empty_i,
            "rotated_block_indices": empty_i, "rotation_deltas": (np.zeros((0, 1), np.int32), P.I32),
            "rotation_trig_lut": (np.zeros((0, D), np.float32), W.F32), "xattention_threshold": empty_f,
            "xattention_block_size": empty_i, "xattention_stride": empty_i, "sinks": (sinks.reshape(1, Hq, 1, 1), W.F32)}
    cache_shape = list(case["key_cache"].shape[:3]) + [D]
    for i, n in enumerate(compiled.input_names()):
        if n in host:
            req.set_input(i, *host[n])
        else:
            req.set_device_input(i, (kc if n == "key_cache" else vc).ptr, W.BF16, cache_shape)
    req.infer()
    out, _ = req.output(0)
    np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), kc_ref)
    assert H.scaled_bound_error(H.storage_to_f32(out, W.BF16), ref, "plugin sinks") <= 2e-2
    plain, _, _ = H.oracle_paged(oracle, case)
    assert np.abs(plain - ref).max() > 1e-2
    kc.free()
    vc.free()
