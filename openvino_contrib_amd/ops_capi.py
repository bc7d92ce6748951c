"""ctypes binding of libhipops.so (include/hipops.h): RMS norm, RoPE, MatMul, Gather, Concat, Swish,
Multiply, GLU, Transpose, Convert, broadcasting arithmetic, Softmax.

Device memory, streams and events come from the hipattn binding (capi.DeviceBuffer & co.); this
module adds the operator calls.  No fallback: a missing library or a failed call raises.
"""
import ctypes
import os

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libhipops.so")

I32, I64, U8, I8, BOOL = 100, 101, 102, 103, 104
TRANSPOSE_MAX_RANK = 8

_i, _i64, _f, _vp, _sz = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
_P = ctypes.POINTER


class RopeDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", _i),
        ("table_dtype", _i),
        ("num_tokens", _i64),
        ("num_heads", _i),
        ("head_size", _i),
        ("rotary_ndims", _i),
        ("interleaved", _i),
        ("x_token_stride", _i64),
        ("x_head_stride", _i64),
        ("out_token_stride", _i64),
        ("out_head_stride", _i64),
        ("table_rows", _i64),
        ("table_row_stride", _i64),
    ]


class MatmulDesc(ctypes.Structure):
    _fields_ = [
        ("ab_dtype", _i),
        ("c_dtype", _i),
        ("m", _i64),
        ("n", _i64),
        ("k", _i64),
        ("batch", _i64),
        ("transpose_a", _i),
        ("transpose_b", _i),
        ("batch_stride_a", _i64),
        ("batch_stride_b", _i64),
    ]


SYMBOLS = {
    "hipops_last_error_string": (ctypes.c_char_p, []),
    "hipops_version": (_i, []),
    "hipops_rms_norm": (_i, [_vp, _vp, _vp, _i64, _i64, _f, _i, _i, _i, _vp]),
    "hipops_rope": (_i, [_P(RopeDesc), _vp, _vp, _vp, _vp, _vp, _vp]),
    "hipops_matmul_workspace_size": (_i, [_P(MatmulDesc), _P(_sz)]),
    "hipops_matmul": (_i, [_P(MatmulDesc), _vp, _vp, _vp, _vp, _sz, _vp]),
    "hipops_swish": (_i, [_vp, _vp, _i64, _f, _i, _vp]),
    "hipops_multiply": (_i, [_vp, _vp, _vp, _i64, _i, _vp]),
    "hipops_glu": (_i, [_vp, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "hipops_transpose": (_i, [_vp, _vp, _i, _P(_i64), _P(ctypes.c_int32), _i, _vp]),
    "hipops_convert": (_i, [_vp, _vp, _i64, _i, _i, _vp]),
    "hipops_binary": (_i, [_i, _vp, _vp, _vp, _i, _P(_i64), _P(_i64), _P(_i64), _i, _vp]),
    "hipops_softmax": (_i, [_vp, _vp, _i64, _i64, _i64, _i, _vp]),
    "hipops_gather": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _vp]),
    "hipops_concat": (_i, [_P(_vp), _P(_i64), _i, _i64, _vp, _vp]),
}

_lib = None


class HipOpsError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("hipops status %d: %s" % (status, message))
        self.status = status


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipOpsError(-1, "%s is missing: run __graft_entry__.build() or "
                                  "python -m openvino_contrib_amd.build" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status):
    if status != capi.OK:
        raise HipOpsError(status, lib().hipops_last_error_string().decode())


def _ptr(buf):
    return None if buf is None else buf.ptr


def _h(stream):
    return stream.handle if stream else None


def rms_norm(x, gamma, out, rows, hidden, eps, x_dtype, gamma_dtype, out_dtype, stream=None):
    check(lib().hipops_rms_norm(_ptr(x), _ptr(gamma), _ptr(out), rows, hidden, eps, x_dtype, gamma_dtype, out_dtype,
                                _h(stream)))


def rope(desc, x, cos, sin, positions, out, stream=None):
    check(lib().hipops_rope(ctypes.byref(desc), _ptr(x), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(out), _h(stream)))


def matmul_workspace_size(desc):
    n = _sz(0)
    check(lib().hipops_matmul_workspace_size(ctypes.byref(desc), ctypes.byref(n)))
    return n.value


def matmul(desc, a, b, c, workspace=None, stream=None):
    check(lib().hipops_matmul(ctypes.byref(desc), _ptr(a), _ptr(b), _ptr(c), _ptr(workspace),
                              workspace.nbytes if workspace is not None else 0, _h(stream)))


GLU_SWISH, GLU_GELU, GLU_GELU_TANH = 0, 1, 2


def swish(x, out, count, dtype, beta=1.0, stream=None):
    check(lib().hipops_swish(_ptr(x), _ptr(out), count, beta, dtype, _h(stream)))


def multiply(a, b, out, count, dtype, stream=None):
    check(lib().hipops_multiply(_ptr(a), _ptr(b), _ptr(out), count, dtype, _h(stream)))


def glu(x, out, rows, width, dtype, activation=GLU_SWISH, gate_first=True, stream=None):
    check(lib().hipops_glu(_ptr(x), _ptr(out), rows, width, activation, int(gate_first), dtype, _h(stream)))


def transpose(x, out, dims, order, element_bytes, stream=None):
    """out = x with output axis k taken from input axis order[k]; dims are x's extents."""
    n = len(dims)
    check(lib().hipops_transpose(_ptr(x), _ptr(out), n, (_i64 * n)(*dims), (ctypes.c_int32 * n)(*order), element_bytes, _h(stream)))


def convert(x, out, count, from_dtype, to_dtype, stream=None):
    check(lib().hipops_convert(_ptr(x), _ptr(out), count, from_dtype, to_dtype, _h(stream)))


ADD, SUBTRACT, MULTIPLY, DIVIDE = 0, 1, 2, 3


def binary(op, a, b, out, out_dims, a_dims, b_dims, dtype, stream=None):
    """out = a (op) b with numpy broadcasting; the three shapes are given at one rank (leading 1s added here)."""
    n = max(len(out_dims), len(a_dims), len(b_dims))
    pad = lambda d: (_i64 * n)(*([1] * (n - len(d)) + [int(x) for x in d]))
    check(lib().hipops_binary(op, _ptr(a), _ptr(b), _ptr(out), n, pad(out_dims), pad(a_dims), pad(b_dims), dtype, _h(stream)))


def softmax(x, out, outer, length, inner, dtype, stream=None):
    check(lib().hipops_softmax(_ptr(x), _ptr(out), outer, length, inner, dtype, _h(stream)))


def gather(data, indices, out, batch, outer, axis_dim, inner_bytes, num_indices, index_dtype, stream=None):
    check(lib().hipops_gather(_ptr(data), _ptr(indices), _ptr(out), batch, outer, axis_dim, inner_bytes, num_indices,
                              index_dtype, _h(stream)))


def concat(inputs, axis_bytes, outer, out, stream=None):
    n = len(inputs)
    ptrs = (_vp * n)(*[b.ptr.value if b is not None else None for b in inputs])
    widths = (_i64 * n)(*axis_bytes)
    check(lib().hipops_concat(ptrs, widths, n, outer, _ptr(out), _h(stream)))
