"""The C-ABI library loads without a GPU and exports every symbol include/hipattn.h declares.
No compute call is made here."""
import ctypes
import os
import re

from openvino_contrib_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "hipattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipattn_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert len(names) >= 30
    assert sorted(capi.SYMBOLS) == names


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(L, name), name


def test_struct_layout_matches_header():
    # 9 four-byte fields; 16 four-byte fields and two pointers, no padding
    assert ctypes.sizeof(capi.SdpaDesc) == 36
    assert ctypes.sizeof(capi.PaDesc) == 80 and capi.PaDesc.alibi_slopes.offset == 64 and capi.PaDesc.sinks.offset == 72
    # int + four int64, the int64s aligned to 8
    assert ctypes.sizeof(capi.MaskDesc) == 40 and capi.MaskDesc.stride.offset == 8


def test_non_compute_calls_work_without_a_device():
    L = capi.lib()
    assert L.hipattn_version() == 4  # (the paged descriptor grew by alibi_slopes and sinks; rotate_key_cache)
    assert L.hipattn_status_string(capi.UNSUPPORTED) == b"unsupported"
    assert capi.cache_row_bytes(capi.U8, 128) == 136
    assert capi.cache_row_bytes(capi.F16, 128) == 256
    assert capi.cache_row_bytes(capi.F32, 64) == 256
    # descriptor validation happens before any device work
    n = ctypes.c_size_t(7)
    bad = capi.SdpaDesc(capi.F16, 1, 3, 2, 4, 4, 128, 0, 0.0)
    assert L.hipattn_sdpa_workspace_size(ctypes.byref(bad), ctypes.byref(n)) == capi.INVALID_ARGUMENT
    assert b"num_heads_q" in L.hipattn_last_error_string()
    ok = capi.SdpaDesc(capi.F16, 1, 4, 2, 4, 4, 128, 0, 0.0)
    assert L.hipattn_sdpa_workspace_size(ctypes.byref(ok), ctypes.byref(n)) == capi.OK and n.value == 0
    pa = capi.PaDesc(capi.F16, capi.F16, capi.F16, capi.F16, 32, 8, 128, 32, 100, 64, 64, 8192, 0, 0.0, 0, 0)
    assert L.hipattn_paged_attention_workspace_size(ctypes.byref(pa), ctypes.byref(n)) == capi.OK
    assert n.value > 0
    pa.head_dim = 1024
    assert L.hipattn_paged_attention_workspace_size(ctypes.byref(pa), ctypes.byref(n)) == capi.UNSUPPORTED
    pa.head_dim = 128
    pa.cache_dtype = 9
    assert L.hipattn_paged_attention_workspace_size(ctypes.byref(pa), ctypes.byref(n)) == capi.INVALID_ARGUMENT
    # options are process-wide host state: no device needed
    assert L.hipattn_set_option(b"decode_switch_cost", 5) == capi.OK
    assert L.hipattn_set_option(b"decode_switch_cost", -1) == capi.OK
    assert L.hipattn_set_option(b"no_such_option", 1) == capi.INVALID_ARGUMENT
    assert b"no_such_option" in L.hipattn_last_error_string()
    # the entry point that allocates nothing refuses what its static scratch cannot hold before it
    # touches any device
    huge = capi.PaDesc(capi.F16, capi.F16, capi.F16, capi.F16, 128, 8, 128, 32, 8, 4096, 4096, 64, 0, 0.0, 0, 0)
    assert L.hipattn_paged_attention_workspace_size(ctypes.byref(huge), ctypes.byref(n)) == capi.OK
    assert n.value > capi.NOALLOC_SCRATCH_BYTES
    one = ctypes.c_void_p(16)
    assert L.hipattn_paged_attention_noalloc(ctypes.byref(huge), one, one, one, one, one, one, one, one, one, one,
                                             None) == capi.WORKSPACE_TOO_SMALL
