"""libhipops.so loads without a GPU and exports every symbol include/hipops.h declares.
Only argument validation is exercised here: no kernel is launched."""
import ctypes
import os
import re

from openvino_contrib_amd import capi, ops_capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "hipops.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipops_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert len(names) == 15
    assert sorted(ops_capi.SYMBOLS) == names


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(ops_capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(L, name), name


def test_struct_layout_matches_header():
    # two ints, int64, four ints, six int64
    assert ctypes.sizeof(ops_capi.RopeDesc) == 8 + 8 + 16 + 48
    assert ops_capi.RopeDesc.x_token_stride.offset == 32
    # two ints, four int64, two ints, two int64
    assert ctypes.sizeof(ops_capi.MatmulDesc) == 8 + 32 + 8 + 16


def test_validation_needs_no_device():
    L = ops_capi.lib()
    assert L.hipops_version() == 4
    n = ctypes.c_size_t(0)
    ok = ops_capi.MatmulDesc(capi.BF16, capi.BF16, 64, 6144, 4096, 1, 0, 1, 0, 0)
    assert L.hipops_matmul_workspace_size(ctypes.byref(ok), ctypes.byref(n)) == capi.OK and n.value == 32 << 20
    bad = ops_capi.MatmulDesc(capi.BF16, capi.F16, 64, 64, 64, 1, 0, 1, 0, 0)
    assert L.hipops_matmul_workspace_size(ctypes.byref(bad), ctypes.byref(n)) == capi.UNSUPPORTED
    assert b"result" in L.hipops_last_error_string()
    assert L.hipops_rms_norm(None, None, None, 4, -1, 1e-6, capi.F16, capi.F16, capi.F16, None) == capi.INVALID_ARGUMENT
    d = ops_capi.RopeDesc(capi.F16, capi.F16, 4, 2, 16, 7, 0, 32, 16, 32, 16, 8, 16)
    assert L.hipops_rope(ctypes.byref(d), None, None, None, None, None, None) == capi.INVALID_ARGUMENT
    assert b"rotary_ndims" in L.hipops_last_error_string()
    assert L.hipops_gather(None, None, None, 1, 1, 4, 8, 2, 5, None) == capi.UNSUPPORTED
    assert L.hipops_concat(None, None, 0, 1, None, None) == capi.INVALID_ARGUMENT
    order = (ctypes.c_int32 * 3)(0, 0, 1)
    dims = (ctypes.c_int64 * 3)(2, 3, 4)
    assert L.hipops_transpose(None, None, 3, dims, order, 2, None) == capi.INVALID_ARGUMENT
    assert b"permutation" in L.hipops_last_error_string()
    order = (ctypes.c_int32 * 3)(0, 2, 1)
    assert L.hipops_transpose(None, None, 3, dims, order, 3, None) == capi.UNSUPPORTED
    assert L.hipops_transpose(None, None, 9, dims, order, 2, None) == capi.INVALID_ARGUMENT
    assert L.hipops_convert(None, None, 8, capi.F32, 7, None) == capi.UNSUPPORTED
    assert L.hipops_convert(None, None, 0, capi.F32, ops_capi.I64, None) == capi.OK
    d3 = (ctypes.c_int64 * 2)(4, 8)
    d1 = (ctypes.c_int64 * 2)(4, 3)
    assert L.hipops_binary(0, None, None, None, 2, d3, d3, d1, capi.F32, None) == capi.INVALID_ARGUMENT
    assert b"broadcast" in L.hipops_last_error_string()
    assert L.hipops_binary(9, None, None, None, 2, d3, d3, d3, capi.F32, None) == capi.INVALID_ARGUMENT
    assert L.hipops_softmax(None, None, 4, 0, 1, capi.F16, None) == capi.OK
    assert L.hipops_softmax(None, None, 4, 8, 1, ops_capi.I64, None) == capi.UNSUPPORTED
