"""ctypes binding of libhipattn.so (include/hipattn.h).

This is how the tests and the benchmark reach the HIP kernels: straight through the C ABI,
with device memory owned by the library's own malloc/free wrappers.  There is no fallback:
if the shared library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libhipattn.so")

OK, INVALID_ARGUMENT, UNSUPPORTED, WORKSPACE_TOO_SMALL, HIP_ERROR, NO_DEVICE = range(6)
F32, F16, BF16, U8 = 0, 1, 2, 3
PA_SKIP_CACHE_WRITE = 1
PA_FORCE_GENERIC = 2
PA_ANY_LENGTHS = 8

DTYPE_BYTES = {F32: 4, F16: 2, BF16: 2, U8: 1}


class HipAttnError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("hipattn status %d: %s" % (status, message))
        self.status = status


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 32),
        ("compute_units", ctypes.c_int),
        ("wavefront_size", ctypes.c_int),
        ("lds_bytes_per_workgroup", ctypes.c_int),
        ("clock_mhz", ctypes.c_int),
        ("global_mem_bytes", ctypes.c_size_t),
    ]


class SdpaDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int),
        ("batch", ctypes.c_int),
        ("num_heads_q", ctypes.c_int),
        ("num_heads_kv", ctypes.c_int),
        ("len_q", ctypes.c_int),
        ("len_kv", ctypes.c_int),
        ("head_dim", ctypes.c_int),
        ("causal", ctypes.c_int),
        ("scale", ctypes.c_float),
    ]


class MaskDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int),
        ("stride", ctypes.c_int64 * 4),
    ]


class PaDesc(ctypes.Structure):
    _fields_ = [
        ("q_dtype", ctypes.c_int),
        ("kv_dtype", ctypes.c_int),
        ("cache_dtype", ctypes.c_int),
        ("out_dtype", ctypes.c_int),
        ("num_heads_q", ctypes.c_int),
        ("num_heads_kv", ctypes.c_int),
        ("head_dim", ctypes.c_int),
        ("block_size", ctypes.c_int),
        ("num_blocks", ctypes.c_int),
        ("num_tokens", ctypes.c_int),
        ("num_seqs", ctypes.c_int),
        ("max_context_len", ctypes.c_int),
        ("sliding_window", ctypes.c_int),
        ("scale", ctypes.c_float),
        ("flags", ctypes.c_int),
        ("decode_waves", ctypes.c_int),
        ("alibi_slopes", ctypes.c_void_p),  # device pointer to num_heads_q floats, or None
        ("sinks", ctypes.c_void_p),         # device pointer to num_heads_q floats, or None
    ]


# every symbol include/hipattn.h declares: name -> (restype, argtypes)
_vp, _i, _sz, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
_P = ctypes.POINTER
SYMBOLS = {
    "hipattn_last_error_string": (ctypes.c_char_p, []),
    "hipattn_status_string": (ctypes.c_char_p, [_i]),
    "hipattn_version": (_i, []),
    "hipattn_device_count": (_i, [_P(_i)]),
    "hipattn_set_device": (_i, [_i]),
    "hipattn_get_device_info": (_i, [_i, _P(DeviceInfo)]),
    "hipattn_stream_create": (_i, [_P(_vp)]),
    "hipattn_stream_destroy": (_i, [_vp]),
    "hipattn_stream_synchronize": (_i, [_vp]),
    "hipattn_malloc": (_i, [_P(_vp), _sz]),
    "hipattn_free": (_i, [_vp]),
    "hipattn_malloc_async": (_i, [_P(_vp), _sz, _vp]),
    "hipattn_free_async": (_i, [_vp, _vp]),
    "hipattn_host_malloc": (_i, [_P(_vp), _sz]),
    "hipattn_host_free": (_i, [_vp]),
    "hipattn_memcpy_h2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "hipattn_memcpy_d2h_async": (_i, [_vp, _vp, _sz, _vp]),
    "hipattn_memcpy_d2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "hipattn_fill_async": (_i, [_vp, _i, _sz, _vp]),
    "hipattn_add_async": (_i, [_vp, _vp, _vp, ctypes.c_int64, _i, _vp]),
    "hipattn_event_create": (_i, [_P(_vp)]),
    "hipattn_event_destroy": (_i, [_vp]),
    "hipattn_event_record": (_i, [_vp, _vp]),
    "hipattn_event_synchronize": (_i, [_vp]),
    "hipattn_event_elapsed_ms": (_i, [_vp, _vp, _P(_f)]),
    "hipattn_stream_begin_capture": (_i, [_vp]),
    "hipattn_stream_end_capture": (_i, [_vp, _P(_vp)]),
    "hipattn_graph_launch": (_i, [_vp, _vp]),
    "hipattn_graph_destroy": (_i, [_vp]),
    "hipattn_sdpa_workspace_size": (_i, [_P(SdpaDesc), _P(_sz)]),
    "hipattn_sdpa": (_i, [_P(SdpaDesc), _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "hipattn_sdpa_masked": (_i, [_P(SdpaDesc), _vp, _vp, _vp, _P(MaskDesc), _vp, _vp, _vp, _sz, _vp]),
    "hipattn_paged_attention_workspace_size": (_i, [_P(PaDesc), _P(_sz)]),
    "hipattn_paged_attention": (_i, [_P(PaDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "hipattn_paged_attention_noalloc": (_i, [_P(PaDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "hipattn_paged_attention_scores_workspace_size": (_i, [_P(PaDesc), _P(_sz)]),
    "hipattn_paged_attention_scores": (_i, [_P(PaDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int64, _vp, _sz, _vp]),
    "hipattn_set_option": (_i, [ctypes.c_char_p, _i]),
    "hipattn_kv_cache_write": (_i, [_P(PaDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "hipattn_rotate_key_cache": (_i, [_P(PaDesc), _vp, _vp, _i, _vp, _i, _vp, _i, _i, _vp]),
    "hipattn_cache_row_bytes": (_sz, [_i, _i]),
    "hipattn_last_kernel_path": (ctypes.c_char_p, []),
    "hipattn_profile_dominant_kernel": (_i, [_vp, _vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipAttnError(-1, "%s is missing: run __graft_entry__.build() or "
                                   "python -m openvino_contrib_amd.build" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status):
    if status != OK:
        raise HipAttnError(status, lib().hipattn_last_error_string().decode())


def device_count():
    n = _i(0)
    st = lib().hipattn_device_count(ctypes.byref(n))
    if st == NO_DEVICE:
        return 0
    check(st)
    return n.value


def device_info(device=0):
    info = DeviceInfo()
    check(lib().hipattn_get_device_info(device, ctypes.byref(info)))
    return info


def last_kernel_path():
    return lib().hipattn_last_kernel_path().decode()


class Stream:
    def __init__(self):
        h = _vp()
        check(lib().hipattn_stream_create(ctypes.byref(h)))
        self.handle = h

    def synchronize(self):
        check(lib().hipattn_stream_synchronize(self.handle))

    def close(self):
        if self.handle is not None:
            lib().hipattn_stream_destroy(self.handle)
            self.handle = None


class Event:
    def __init__(self):
        h = _vp()
        check(lib().hipattn_event_create(ctypes.byref(h)))
        self.handle = h

    def record(self, stream=None):
        check(lib().hipattn_event_record(self.handle, stream.handle if stream else None))

    def synchronize(self):
        check(lib().hipattn_event_synchronize(self.handle))

    def elapsed_ms(self, stop):
        ms = _f(0)
        check(lib().hipattn_event_elapsed_ms(self.handle, stop.handle, ctypes.byref(ms)))
        return ms.value

    def close(self):
        if self.handle is not None:
            lib().hipattn_event_destroy(self.handle)
            self.handle = None


class DeviceBuffer:
    """Device allocation owned through hipattn_malloc / hipattn_free."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = _vp()
        check(lib().hipattn_malloc(ctypes.byref(p), max(self.nbytes, 1)))
        self.ptr = p

    @classmethod
    def from_numpy(cls, arr, stream=None):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr, stream)
        return buf

    def upload(self, arr, stream=None):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        check(lib().hipattn_memcpy_h2d_async(self.ptr, arr.ctypes.data_as(_vp), arr.nbytes,
                                             stream.handle if stream else None))
        check(lib().hipattn_stream_synchronize(stream.handle if stream else None))

    def download(self, dtype, shape, stream=None):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib().hipattn_stream_synchronize(stream.handle if stream else None))
        check(lib().hipattn_memcpy_d2h_async(out.ctypes.data_as(_vp), self.ptr, out.nbytes,
                                             stream.handle if stream else None))
        check(lib().hipattn_stream_synchronize(stream.handle if stream else None))
        return out

    def fill(self, byte_value, stream=None):
        check(lib().hipattn_fill_async(self.ptr, byte_value, self.nbytes, stream.handle if stream else None))

    def free(self):
        if self.ptr is not None:
            lib().hipattn_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _h(stream):
    return stream.handle if stream else None


def sdpa_workspace_size(desc):
    n = _sz(0)
    check(lib().hipattn_sdpa_workspace_size(ctypes.byref(desc), ctypes.byref(n)))
    return n.value


def sdpa(desc, q, k, v, out, workspace=None, stream=None):
    """All tensor arguments are DeviceBuffers."""
    check(lib().hipattn_sdpa(ctypes.byref(desc), q.ptr, k.ptr, v.ptr, out.ptr,
                             workspace.ptr if workspace else None, workspace.nbytes if workspace else 0,
                             _h(stream)))


def sdpa_masked(desc, q, k, v, mask_dtype, mask_strides, mask, out, workspace=None, stream=None):
    """SDPA with an attention mask (DeviceBuffer) addressed as [batch, head, query, key] by strides in elements."""
    md = MaskDesc(mask_dtype, (ctypes.c_int64 * 4)(*mask_strides))
    check(lib().hipattn_sdpa_masked(ctypes.byref(desc), q.ptr, k.ptr, v.ptr, ctypes.byref(md), mask.ptr, out.ptr,
                                    workspace.ptr if workspace else None, workspace.nbytes if workspace else 0,
                                    _h(stream)))


def paged_attention_workspace_size(desc):
    n = _sz(0)
    check(lib().hipattn_paged_attention_workspace_size(ctypes.byref(desc), ctypes.byref(n)))
    return n.value


def paged_attention(desc, q, k_new, v_new, key_cache, value_cache, past_lens, subsequence_begins, block_indices,
                    block_indices_begins, out, workspace=None, stream=None):
    check(lib().hipattn_paged_attention(
        ctypes.byref(desc), q.ptr, k_new.ptr if k_new else None, v_new.ptr if v_new else None, key_cache.ptr,
        value_cache.ptr, past_lens.ptr, subsequence_begins.ptr, block_indices.ptr, block_indices_begins.ptr,
        out.ptr, workspace.ptr if workspace else None, workspace.nbytes if workspace else 0, _h(stream)))


def paged_attention_noalloc(desc, q, k_new, v_new, key_cache, value_cache, past_lens, subsequence_begins,
                            block_indices, block_indices_begins, out, stream=None):
    """The entry point that allocates nothing: scratch is the library's static device array."""
    check(lib().hipattn_paged_attention_noalloc(
        ctypes.byref(desc), q.ptr, k_new.ptr if k_new else None, v_new.ptr if v_new else None, key_cache.ptr,
        value_cache.ptr, past_lens.ptr, subsequence_begins.ptr, block_indices.ptr, block_indices_begins.ptr,
        out.ptr, _h(stream)))


def paged_attention_scores(desc, q, key_cache, past_lens, subsequence_begins, block_indices, block_indices_begins,
                           score_window, scores, capacity, stream=None, lse_only=False):
    """scores: DeviceBuffer of `capacity` floats.  The workspace is allocated here: what the size query asks for
    or, with lse_only, one float per token and head, which leaves the call to the fp32 kernels."""
    n = _sz(0)
    check(lib().hipattn_paged_attention_scores_workspace_size(ctypes.byref(desc), ctypes.byref(n)))
    ws = DeviceBuffer(desc.num_tokens * desc.num_heads_q * 4 if lse_only else n.value)
    check(lib().hipattn_paged_attention_scores(ctypes.byref(desc), q.ptr, key_cache.ptr, past_lens.ptr,
                                               subsequence_begins.ptr, block_indices.ptr, block_indices_begins.ptr,
                                               score_window.ptr if score_window is not None else None, scores.ptr,
                                               capacity, ws.ptr, ws.nbytes, _h(stream)))
    check(lib().hipattn_stream_synchronize(_h(stream)))
    ws.free()


def set_option(name, value):
    """Process-wide schedule option (see include/hipattn.h); value < 0 restores the default."""
    check(lib().hipattn_set_option(name.encode(), int(value)))


NOALLOC_SCRATCH_BYTES = 16 << 20


def rotate_key_cache(desc, key_cache, rotated_block_indices, rotation_deltas, deltas_per_block, trig_lut, lut_dtype, lut_rows,
                     stream=None):
    """DeviceBuffers: block ids [n] and deltas [n, deltas_per_block] int32, the table [lut_rows, head_dim] of lut_dtype."""
    n = rotated_block_indices.nbytes // 4
    check(lib().hipattn_rotate_key_cache(ctypes.byref(desc), key_cache.ptr, rotated_block_indices.ptr, n, rotation_deltas.ptr,
                                         deltas_per_block, trig_lut.ptr, lut_dtype, lut_rows, _h(stream)))


def kv_cache_write(desc, k_new, v_new, key_cache, value_cache, past_lens, subsequence_begins, block_indices,
                   block_indices_begins, stream=None):
    check(lib().hipattn_kv_cache_write(ctypes.byref(desc), k_new.ptr, v_new.ptr, key_cache.ptr, value_cache.ptr,
                                       past_lens.ptr, subsequence_begins.ptr, block_indices.ptr,
                                       block_indices_begins.ptr, _h(stream)))


def profile_dominant_kernel(before=None, after=None):
    check(lib().hipattn_profile_dominant_kernel(before.handle if before else None, after.handle if after else None))


def cache_row_bytes(cache_dtype, head_dim):
    return lib().hipattn_cache_row_bytes(cache_dtype, head_dim)
