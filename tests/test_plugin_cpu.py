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
    for name in ("Parameter", "Result", "Constant", "ScaledDotProductAttention", "PagedAttentionExtension"):
        assert name in ops


def test_query_model_reports_supported_nodes():
    plugin = P.Plugin()
    sdpa = P.Model.sdpa(P.F16, [1, 8, -1, 64], [1, 8, -1, 64], True)
    assert sorted(plugin.query_model(sdpa)) == ["key", "out", "query", "sdpa", "value"]
    # attention_mask / scale inputs: the operator's constructor throws, the node is reported unsupported
    masked = P.Model.sdpa(P.F16, [1, 8, -1, 64], [1, 8, -1, 64], True, with_scale_input=True)
    assert "sdpa" not in plugin.query_model(masked)
    pa = P.Model.paged_attention(P.F16, P.F16, P.U8, 32, 8, 128, 32)
    assert "paged_attention" in plugin.query_model(pa)
    alibi = P.Model.paged_attention(P.F16, P.F16, P.F16, 32, 8, 128, 32, alibi_len=32)
    assert "paged_attention" not in plugin.query_model(alibi)
    unknown = P.Model.unsupported()
    assert sorted(plugin.query_model(unknown)) == ["out", "x"]


def test_properties():
    plugin = P.Plugin()
    assert "PERF_COUNT" in plugin.get_property("SUPPORTED_PROPERTIES")
    assert plugin.get_property("PERF_COUNT") == "NO"
    plugin.set_property("PERF_COUNT", "YES")
    assert plugin.get_property("PERF_COUNT") == "YES"
    plugin.set_property("INFERENCE_PRECISION_HINT", "bf16")
    assert plugin.get_property("INFERENCE_PRECISION_HINT") == "bf16"
    assert plugin.get_property("RANGE_FOR_ASYNC_INFER_REQUESTS") == "1 1 1"
    with pytest.raises(P.PluginError) as e:
        plugin.set_property("INFERENCE_PRECISION_HINT", "f64")
    assert "INFERENCE_PRECISION_HINT" in str(e.value) and "plugin.cpp" in str(e.value)  # file:line(function): text
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
