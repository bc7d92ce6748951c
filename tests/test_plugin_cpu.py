"""Host logic of the plugin layer (libhip_plugin.so) that needs no GPU: registry, query_model,
properties, error behaviour.  Modelled on the reference's infrastructure unit tests
(modules/nvidia_plugin/tests/unit/operation_registry.cpp:46-87, tests/unit/plugin.cpp:42-53,
tests/unit/compile_model.cpp:86)."""
import ctypes
import os
import re

import pytest

from openvino_contrib_amd import plugin_capi as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_binding_and_exports_agree():
    text = open(os.path.join(ROOT, "include", "hip_plugin.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(hip_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(P.SYMBOLS)
    L = ctypes.CDLL(P.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name


def test_registry_holds_the_attention_operators():
    ops = P.registered_operations()
    for name in ("Parameter", "Result", "Constant", "ScaledDotProductAttention", "PagedAttentionExtension", "ReadValue",
                 "Assign", "Add", "RMS", "RoPE", "MatMul", "Gather", "Concat", "Swish", "Multiply", "GLU", "Reshape", "Squeeze",
                 "Unsqueeze", "Transpose", "Convert", "Subtract", "Divide", "Softmax"):
        assert name in ops


def test_query_model_on_the_operators_around_attention():
    """A text-form graph of RMS / MatMul / RoPE / Gather / Concat nodes: supported ones are listed,
    nodes an operator's constructor refuses are not (src/cuda_plugin.cpp:171-188)."""
    import numpy as np

    g = P.GraphText("layer")
    ids = g.parameter("ids", P.I32, [-1])
    table = g.constant("table", np.zeros((10, 64), np.uint16), "f16")
    axis = g.constant("axis", np.array(0, np.int64), "i64")
    emb = g.add("Gather", "embed", [table, ids, axis], batch_dims=0)
    gamma = g.constant("gamma", np.zeros(64, np.uint16), "f16")
    norm = g.add("RMS", "norm", [emb, gamma], epsilon=1e-6, output_type="dynamic")
    w = g.parameter("w", P.F16, [128, 64])
    proj = g.add("MatMul", "proj", [norm, w], transpose_a=False, transpose_b=True)
    cos = g.parameter("cos", P.F32, [-1, 64])
    sin = g.parameter("sin", P.F32, [-1, 64])
    rope = g.add("RoPE", "rope", [proj, cos, sin], head_cnt=2, head_size=64, rotary_ndims=64)
    glm = g.add("RoPE", "rope_glm", [proj, cos, sin], head_cnt=2, head_size=64, is_chatglm=True)
    w32 = g.parameter("w32", P.F32, [128, 64])
    mixed = g.add("MatMul", "mixed", [norm, w32], transpose_a=False, transpose_b=True)
    cat = g.add("Concat", "cat", [rope, glm], axis=1)
    g.result("out", cat)
    g.result("out2", mixed)
    supported = set(P.Plugin().query_model(g.model()))
    assert {"embed", "norm", "proj", "rope", "cat"} <= supported
    assert "rope_glm" not in supported and "mixed" not in supported


def test_plugin_object_comes_from_create_plugin_engine():
    """The facade asks the library's exported create_plugin_engine() for the plugin, as ov::Core would
    (src/cuda_create_plugin.cpp:11-12)."""
    L = ctypes.CDLL(P.LIB_PATH)
    assert hasattr(L, "create_plugin_engine")
    assert P.Plugin().device_name() == "HIP"


def test_query_model_reports_supported_nodes():
    plugin = P.Plugin()
    sdpa = P.Model.sdpa(P.F16, [1, 8, -1, 64], [1, 8, -1, 64], True)
    assert sorted(plugin.query_model(sdpa)) == ["key", "out", "query", "sdpa", "value"]
    unknown = P.Model.unsupported()
    assert sorted(plugin.query_model(unknown)) == ["out", "x"]
    stateful = P.Model.accumulator(P.F32, [-1, 4])
    assert sorted(plugin.query_model(stateful)) == ["add", "assign", "out", "read_value", "x"]


def test_sdpa_takes_the_operators_optional_inputs():
    """attention_mask (boolean or floating, any broadcastable rank) and scale (Parameter or Constant)
    are part of v13::ScaledDotProductAttention; the reference runs them through the decomposition."""
    plugin = P.Plugin()
    for kw in (dict(mask_dtype=P.BOOL, mask_shape=[-1, -1]), dict(mask_dtype=P.F16, mask_shape=[1, 8, -1, -1]),
               dict(scale=True), dict(scale_constant=0.125), dict(mask_dtype=P.F32, mask_shape=[-1, -1], scale=True)):
        model = P.Model.sdpa(P.F16, [1, 8, -1, 64], [1, 8, -1, 64], False, **kw)
        assert "sdpa" in plugin.query_model(model), kw
    # what stays unsupported: an integer mask, a mask of higher rank than the query
    assert "sdpa" not in plugin.query_model(P.Model.sdpa(P.F16, [1, 8, -1, 64], [1, 8, -1, 64], False, mask_dtype=P.I32,
                                                         mask_shape=[-1, -1]))
    assert "sdpa" not in plugin.query_model(P.Model.sdpa(P.F16, [8, -1, 64], [8, -1, 64], False, mask_dtype=P.F16,
                                                         mask_shape=[1, 8, -1, -1]))


def test_paged_attention_takes_the_operators_full_signature():
    """Exported models carry the inputs behind max_context_len (score aggregation, cache rotation,
    sparse attention, sinks) and the scores output even when the features are off: such a node is
    supported as long as the inputs of what is not built (sparse attention, sinks) are empty, and refused
    when they hold data; score aggregation and the three cache-rotation inputs may hold data."""
    plugin = P.Plugin()
    assert "paged_attention" in plugin.query_model(P.Model.paged_attention(P.F16, P.F16, P.U8, 32, 8, 128, 32))
    for extra in (1, 4, 8):
        pa = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=extra, extra_len=0,
                                     scores_result=True)
        names = plugin.query_model(pa)
        assert "paged_attention" in names and "scores" in names, extra
    windowed = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=1, extra_len=16, scores_result=True)
    assert "paged_attention" in plugin.query_model(windowed)  # score_aggregation_window may hold data
    rotated = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=4, extra_len=16)
    assert "paged_attention" in plugin.query_model(rotated)  # cache rotation: indices, deltas and the table together
    half_rotated = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=3, extra_len=16)
    assert "paged_attention" not in plugin.query_model(half_rotated)  # ... not two of the three
    sparse = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=5, extra_len=16)
    assert "paged_attention" not in plugin.query_model(sparse)  # xattention_threshold holds data
    unknown_inputs = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, extra_inputs=9, extra_len=0)
    assert "paged_attention" not in plugin.query_model(unknown_inputs)
    alibi = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, alibi_len=32)
    assert "paged_attention" in plugin.query_model(alibi)  # one slope per query head: ALiBi


def test_import_model_rejects_a_foreign_stream():
    plugin = P.Plugin()
    for blob in (b"", b"\x05\x00", b"\xff" * 32):
        with pytest.raises(P.PluginError):
            plugin.import_model(blob)


def test_properties():
    plugin = P.Plugin()
    assert "PERF_COUNT" in plugin.get_property("SUPPORTED_PROPERTIES")
    assert plugin.get_property("PERF_COUNT") == "NO"
    plugin.set_property("PERF_COUNT", "YES")
    assert plugin.get_property("PERF_COUNT") == "YES"
    plugin.set_property("INFERENCE_PRECISION_HINT", "bf16")
    assert plugin.get_property("INFERENCE_PRECISION_HINT") == "bf16"
    assert plugin.get_property("RANGE_FOR_ASYNC_INFER_REQUESTS") == "1 1 1"
    # graph replay of repeated infers is on unless switched off (the reference's NVIDIA_USE_CUDA_GRAPH)
    assert "HIP_USE_GRAPH" in plugin.get_property("SUPPORTED_PROPERTIES") and plugin.get_property("HIP_USE_GRAPH") == "YES"
    plugin.set_property("HIP_USE_GRAPH", "NO")
    assert plugin.get_property("HIP_USE_GRAPH") == "NO"
    with pytest.raises(P.PluginError) as e:
        plugin.set_property("INFERENCE_PRECISION_HINT", "f64")
    assert "INFERENCE_PRECISION_HINT" in str(e.value) and "hip_plugin.cpp" in str(e.value)  # file:line(function): text
    with pytest.raises(P.PluginError):
        plugin.set_property("NO_SUCH_PROPERTY", "1")
    with pytest.raises(P.PluginError):
        plugin.get_property("NO_SUCH_PROPERTY")
    with pytest.raises(P.PluginError):
        plugin.set_property("NUM_STREAMS", "0")


def test_compile_without_a_device_or_with_unknown_operator_fails():
    plugin = P.Plugin()
    with pytest.raises(P.PluginError) as e:
        plugin.compile_model(P.Model.unsupported())
    # either there is no device here, or the unknown operator is rejected: both are errors, never a fallback
    assert "SuperOperation" in str(e.value) or "no HIP device" in str(e.value)


def test_query_model_on_views_transpose_and_convert():
    """Static shapes of the stand-in nodes and the constructors' verdicts, without a device."""
    import numpy as np

    g = P.GraphText("formats")
    x = g.parameter("x", P.F32, [2, 5, 48])
    i64 = lambda name, values: g.constant(name, np.array(values, np.int64), "i64")
    split = g.add("Reshape", "split", [x, i64("p", [0, -1, 3, 16])], special_zero=True)
    moved = g.add("Transpose", "moved", [split, i64("o", [0, 2, 1, 3])])
    wide = g.add("Unsqueeze", "wide", [moved, i64("a", [0])])
    g.result("out", g.add("Convert", "half", [g.add("Squeeze", "narrow", [wide, i64("b", [0])])], destination_type="f16"))
    g.result("bad", g.add("Convert", "to_u16", [x], destination_type="u16"))
    supported = P.Plugin().query_model(g.model())
    assert {"split", "moved", "wide", "narrow", "half"} <= set(supported)
    assert "to_u16" not in supported


def test_memory_solver_packs_boxes_by_lifetime():
    """The offsets of the request's intermediate tensors (the reference packs its mutable blob with
    ov::MemorySolver, NP/src/memory_manager/model/cuda_memory_model_builder.cpp:11-25): boxes alive at the
    same step never share an address, a chain needs two buffers, and no packing beats the peak of live bytes."""
    import numpy as np

    def check(sizes, start, end):
        offsets, total = P.memory_solver_pack(sizes, start, end)
        n = len(sizes)
        up = [(b + 255) // 256 * 256 for b in sizes]
        assert all(o % 256 == 0 for o in offsets) and total == max([o + u for o, u in zip(offsets, up)] + [0])
        for i in range(n):
            for j in range(i + 1, n):
                if start[i] <= end[j] and start[j] <= end[i]:
                    assert offsets[i] + up[i] <= offsets[j] or offsets[j] + up[j] <= offsets[i], (i, j)
        peak = max([sum(up[i] for i in range(n) if start[i] <= t <= end[i]) for t in range(max(end) + 1)] + [0])
        assert peak <= total <= sum(up)
        return total, peak

    # a chain: tensor i is written by step i and read by step i + 1
    total, peak = check([1000] * 12, list(range(12)), list(range(1, 13)))
    assert total == peak == 2 * 1024
    # a residual stream: one tensor lives through, the others are a chain
    total, peak = check([4096] + [3000] * 8, [0] + list(range(1, 9)), [9] + list(range(2, 10)))
    assert total == peak
    # nothing overlaps in time: one buffer of the largest size
    total, _ = check([300, 70000, 5, 256], [0, 2, 4, 6], [1, 3, 5, 7])
    assert total == 70144
    # everything alive at once: the sum
    total, peak = check([100, 200, 300], [0, 0, 0], [5, 5, 5])
    assert total == peak == 256 * 4
    assert P.memory_solver_pack([], [], []) == ([], 0)
    rng = np.random.default_rng(3)
    worst = 1.0
    for _ in range(200):
        n = int(rng.integers(1, 40))
        start = [int(x) for x in rng.integers(0, 30, n)]
        end = [s + int(x) for s, x in zip(start, rng.integers(0, 8, n))]
        sizes = [int(x) for x in rng.integers(1, 100000, n)]
        total, peak = check(sizes, start, end)
        worst = max(worst, total / peak)
    assert worst <= 1.5, worst  # (greedy, largest first: close to the peak on such mixes)
