"""ctypes binding of libhip_plugin.so (include/hip_plugin.h): the C++ Plugin / CompiledModel /
InferRequest classes of the "HIP" device, driven from Python by the tests."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libhip_plugin.so")

F32, F16, BF16, U8, I32, BOOL, I64, I8 = 0, 1, 2, 3, 100, 101, 102, 103
_NP = {F32: np.float32, F16: np.uint16, BF16: np.uint16, U8: np.uint8, I32: np.int32, BOOL: np.bool_, I64: np.int64, I8: np.int8}
OK, ERROR, OTHER_ERROR, NOT_IMPLEMENTED, CANCELLED, BUSY = range(6)

_vp, _i, _sz, _cp = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_char_p
_P = ctypes.POINTER
_i64p = _P(ctypes.c_int64)
SYMBOLS = {
    "hip_plugin_last_error": (_cp, []),
    "hip_plugin_create": (_i, [_P(_vp)]),
    "hip_plugin_destroy": (None, [_vp]),
    "hip_plugin_device_name": (_i, [_vp, ctypes.c_char_p, _sz]),
    "hip_plugin_set_property": (_i, [_vp, _cp, _cp]),
    "hip_plugin_get_property": (_i, [_vp, _cp, ctypes.c_char_p, _sz]),
    "hip_plugin_compile_model": (_i, [_vp, _vp, _cp, _P(_vp)]),
    "hip_plugin_import_model": (_i, [_vp, _vp, _sz, _cp, _P(_vp)]),
    "hip_plugin_query_model": (_i, [_vp, _vp, ctypes.c_char_p, _sz]),
    "hip_plugin_registered_operations": (_i, [ctypes.c_char_p, _sz]),
    "hip_model_create_sdpa": (_i, [_i, _i, _i64p, _i64p, _i, _i, _i, _i64p, _i, ctypes.c_float, _P(_vp)]),
    "hip_model_create_paged_attention": (_i, [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _P(_vp)]),
    "hip_model_create_accumulator": (_i, [_i, _i, _i64p, _P(_vp)]),
    "hip_model_create_from_text": (_i, [_cp, _P(_vp)]),
    "hip_model_create_unsupported": (_i, [_P(_vp)]),
    "hip_model_destroy": (None, [_vp]),
    "hip_compiled_model_destroy": (None, [_vp]),
    "hip_compiled_model_num_inputs": (_i, [_vp]),
    "hip_compiled_model_num_outputs": (_i, [_vp]),
    "hip_compiled_model_input_name": (_i, [_vp, _i, ctypes.c_char_p, _sz]),
    "hip_compiled_model_get_property": (_i, [_vp, _cp, ctypes.c_char_p, _sz]),
    "hip_compiled_model_export": (_i, [_vp, _vp, _sz, _P(_sz)]),
    "hip_compiled_model_runtime_info": (_i, [_vp, ctypes.c_char_p, _sz]),
    "hip_compiled_model_create_infer_request": (_i, [_vp, _P(_vp)]),
    "hip_infer_request_destroy": (None, [_vp]),
    "hip_infer_request_set_input": (_i, [_vp, _i, _vp, _i, _i, _i, _i64p]),
    "hip_infer_request_set_input_batch": (_i, [_vp, _i, _P(_vp), _i, _i, _i, _i64p]),
    "hip_infer_request_set_output": (_i, [_vp, _i, _vp, _i, _i, _i, _i64p]),
    "hip_infer_request_infer": (_i, [_vp]),
    "hip_infer_request_start_async": (_i, [_vp]),
    "hip_infer_request_wait": (_i, [_vp]),
    "hip_infer_request_cancel": (_i, [_vp]),
    "hip_infer_request_output_info": (_i, [_vp, _i, _P(_i), _P(_i), _i64p, _P(_sz)]),
    "hip_infer_request_copy_output": (_i, [_vp, _i, _vp, _sz]),
    "hip_infer_request_profiling": (_i, [_vp, ctypes.c_char_p, _sz]),
    "hip_infer_request_intermediate_memory": (_i, [_vp, _P(_sz), _P(_sz)]),
    "hip_memory_solver_pack": (_sz, [_i, _P(_sz), _P(_i), _P(_i), _P(_sz)]),
    "hip_infer_request_num_states": (_i, [_vp]),
    "hip_infer_request_state_name": (_i, [_vp, _i, ctypes.c_char_p, _sz]),
    "hip_infer_request_state_reset": (_i, [_vp, _i]),
    "hip_infer_request_state_info": (_i, [_vp, _i, _P(_i), _P(_i), _i64p, _P(_sz)]),
    "hip_infer_request_state_get": (_i, [_vp, _i, _vp, _sz]),
    "hip_infer_request_state_set": (_i, [_vp, _i, _vp, _i, _i, _i64p]),
}

_lib = None


class PluginError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PluginError(-1, "%s is missing: run __graft_entry__.build()" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _check(code):
    if code != 0:
        raise PluginError(code, lib().hip_plugin_last_error().decode())


def _shape(s):
    return (ctypes.c_int64 * len(s))(*[int(x) for x in s])


def _text(fn, *args, size=1 << 16):
    buf = ctypes.create_string_buffer(size)
    _check(fn(*args, buf, size))
    return buf.value.decode()


def registered_operations():
    return _text(lib().hip_plugin_registered_operations).split(",")


_TYPE_NAMES = {F32: "f32", F16: "f16", BF16: "bf16", U8: "u8", I32: "i32", BOOL: "boolean", I64: "i64", I8: "i8"}


class GraphText:
    """Writes a graph in the stand-in text form, node by node: `add` returns the node's index, an
    input is an index (output 0) or an (index, port) pair.  Parameters and Results take part in the
    compiled model's inputs / outputs in the order they are added."""

    def __init__(self, name="model"):
        self.lines = ["standin-ir 1 " + name]

    def add(self, type_name, name, inputs=(), **attrs):
        idx = len(self.lines) - 1
        ins = ",".join("%d:%d" % (i if isinstance(i, tuple) else (i, 0)) for i in inputs)
        body = "".join("%s=%s;" % (k, ("true" if v else "false") if isinstance(v, bool) else v) for k, v in attrs.items())
        self.lines.append("%d %s %s inputs=%s {%s}" % (idx, type_name, name, ins, body))
        return idx

    @staticmethod
    def _shape(shape):
        return "[" + ",".join("?" if d < 0 else str(d) for d in shape) + "]"

    def parameter(self, name, dtype, shape):
        return self.add("Parameter", name, element_type=_TYPE_NAMES.get(dtype, dtype), shape=self._shape(shape))

    def constant(self, name, array, type_name):
        array = np.ascontiguousarray(array)
        return self.add("Constant", name, element_type=type_name, shape=self._shape(array.shape), data=array.tobytes().hex())

    def result(self, name, source):
        return self.add("Result", name, [source])

    def text(self):
        return "\n".join(self.lines) + "\n"

    def model(self):
        return Model.from_text(self.text())


class Model:
    def __init__(self, handle):
        self.handle = handle

    @classmethod
    def sdpa(cls, dtype, q_shape, kv_shape, causal, mask_dtype=None, mask_shape=(), scale=None, scale_constant=None):
        """mask_dtype / mask_shape: the attention_mask input (None: absent).  scale=True: a scalar f32
        Parameter named "scale"; scale_constant=x: a Constant holding x."""
        h = _vp()
        mode, value = (2, float(scale_constant)) if scale_constant is not None else ((1, 0.0) if scale else (0, 0.0))
        _check(lib().hip_model_create_sdpa(dtype, len(q_shape), _shape(q_shape), _shape(kv_shape), int(causal),
                                           -1 if mask_dtype is None else mask_dtype, len(mask_shape),
                                           _shape(mask_shape), mode, value, ctypes.byref(h)))
        return cls(h)

    @classmethod
    def paged_attention(cls, q_dtype, kv_dtype, cache_dtype, Hq, Hkv, D, block_size, alibi_len=0, extra_inputs=0,
                        extra_len=0, scores_result=False):
        h = _vp()
        _check(lib().hip_model_create_paged_attention(q_dtype, kv_dtype, cache_dtype, Hq, Hkv, D, block_size,
                                                      alibi_len, extra_inputs, extra_len, int(scores_result),
                                                      ctypes.byref(h)))
        return cls(h)

    @classmethod
    def accumulator(cls, dtype, shape):
        h = _vp()
        _check(lib().hip_model_create_accumulator(dtype, len(shape), _shape(shape), ctypes.byref(h)))
        return cls(h)

    @classmethod
    def from_text(cls, text):
        """A model in the stand-in text form; GraphText builds it."""
        h = _vp()
        _check(lib().hip_model_create_from_text(text.encode(), ctypes.byref(h)))
        return cls(h)

    @classmethod
    def unsupported(cls):
        h = _vp()
        _check(lib().hip_model_create_unsupported(ctypes.byref(h)))
        return cls(h)

    def __del__(self):
        if self.handle:
            lib().hip_model_destroy(self.handle)
            self.handle = None


class InferRequest:
    def __init__(self, handle):
        self.handle = handle
        self._keep = {}

    def set_input(self, index, array, dtype):
        """Host tensor: wrapped, not copied (kept alive here until replaced)."""
        array = np.asarray(array, dtype=_NP[dtype], order="C")  # (keeps a scalar's rank 0)
        self._keep[index] = array
        _check(lib().hip_infer_request_set_input(self.handle, index, array.ctypes.data_as(_vp), 0, dtype, array.ndim,
                                                 _shape(array.shape)))

    def intermediate_memory(self):
        """(bytes of the blob the last infer's intermediate tensors were packed into, bytes they take side by side)."""
        blob, apart = _sz(0), _sz(0)
        _check(lib().hip_infer_request_intermediate_memory(self.handle, ctypes.byref(blob), ctypes.byref(apart)))
        return blob.value, apart.value

    def set_input_batch(self, index, arrays, dtype):
        """set_tensors: one host tensor per batch entry (each of shape [1, ...]), wrapped, not copied."""
        arrays = [np.asarray(a, dtype=_NP[dtype], order="C") for a in arrays]
        self._keep[index] = arrays
        ptrs = (_vp * len(arrays))(*[a.ctypes.data_as(_vp) for a in arrays])
        shape = arrays[0].shape if arrays else (1,)
        _check(lib().hip_infer_request_set_input_batch(self.handle, index, ptrs, len(arrays), dtype, len(shape), _shape(shape)))

    def set_device_input(self, index, device_ptr, dtype, shape):
        _check(lib().hip_infer_request_set_input(self.handle, index, device_ptr, 1, dtype, len(shape), _shape(shape)))

    def set_device_output(self, index, device_ptr, dtype, shape):
        """The output is left in the caller's device memory instead of a host tensor."""
        _check(lib().hip_infer_request_set_output(self.handle, index, device_ptr, 1, dtype, len(shape), _shape(shape)))

    def infer(self):
        _check(lib().hip_infer_request_infer(self.handle))

    def cancel(self):
        _check(lib().hip_infer_request_cancel(self.handle))

    def states(self):
        n = lib().hip_infer_request_num_states(self.handle)
        return [_text(lib().hip_infer_request_state_name, self.handle, i, size=256) for i in range(n)]

    def state_reset(self, index=0):
        _check(lib().hip_infer_request_state_reset(self.handle, index))

    def state_get(self, index=0):
        dt, rank, nbytes = _i(0), _i(0), _sz(0)
        shape = (ctypes.c_int64 * 8)()
        _check(lib().hip_infer_request_state_info(self.handle, index, ctypes.byref(dt), ctypes.byref(rank), shape,
                                                  ctypes.byref(nbytes)))
        out = np.empty([shape[i] for i in range(rank.value)], _NP[dt.value])
        _check(lib().hip_infer_request_state_get(self.handle, index, out.ctypes.data_as(_vp), out.nbytes))
        return out

    def state_set(self, array, dtype, index=0):
        array = np.ascontiguousarray(array, _NP[dtype])
        _check(lib().hip_infer_request_state_set(self.handle, index, array.ctypes.data_as(_vp), dtype, array.ndim,
                                                 _shape(array.shape)))

    def start_async(self):
        _check(lib().hip_infer_request_start_async(self.handle))

    def wait(self):
        _check(lib().hip_infer_request_wait(self.handle))

    def output(self, index=0):
        dt, rank, nbytes = _i(0), _i(0), _sz(0)
        shape = (ctypes.c_int64 * 8)()
        _check(lib().hip_infer_request_output_info(self.handle, index, ctypes.byref(dt), ctypes.byref(rank), shape,
                                                   ctypes.byref(nbytes)))
        out = np.empty([shape[i] for i in range(rank.value)], _NP[dt.value])
        _check(lib().hip_infer_request_copy_output(self.handle, index, out.ctypes.data_as(_vp), out.nbytes))
        return out, dt.value

    def profiling(self):
        rows = []
        for line in _text(lib().hip_infer_request_profiling, self.handle).splitlines():
            name, typ, us = line.split("|")
            rows.append((name, typ, float(us)))
        return rows

    def __del__(self):
        if self.handle:
            lib().hip_infer_request_destroy(self.handle)
            self.handle = None


class CompiledModel:
    def __init__(self, handle):
        self.handle = handle

    def input_names(self):
        n = lib().hip_compiled_model_num_inputs(self.handle)
        return [_text(lib().hip_compiled_model_input_name, self.handle, i, size=256) for i in range(n)]

    def get_property(self, key):
        return _text(lib().hip_compiled_model_get_property, self.handle, key.encode(), size=4096)

    def num_outputs(self):
        return lib().hip_compiled_model_num_outputs(self.handle)

    def runtime_info(self):
        """get_runtime_model: (node name, layerType, execOrder, execTimeMcs, runtimePrecision, primitiveType) per node."""
        return [tuple(line.split("|")) for line in _text(lib().hip_compiled_model_runtime_info, self.handle, size=65536).splitlines()]

    def export_model(self):
        """The bytes CompiledModel::export_model writes."""
        n = _sz(0)
        _check(lib().hip_compiled_model_export(self.handle, None, 0, ctypes.byref(n)))
        buf = ctypes.create_string_buffer(max(n.value, 1))
        _check(lib().hip_compiled_model_export(self.handle, buf, n.value, ctypes.byref(n)))
        return buf.raw[:n.value]

    def create_infer_request(self):
        h = _vp()
        _check(lib().hip_compiled_model_create_infer_request(self.handle, ctypes.byref(h)))
        return InferRequest(h)

    def __del__(self):
        if self.handle:
            lib().hip_compiled_model_destroy(self.handle)
            self.handle = None


class Plugin:
    def __init__(self):
        h = _vp()
        _check(lib().hip_plugin_create(ctypes.byref(h)))
        self.handle = h

    def set_property(self, key, value):
        _check(lib().hip_plugin_set_property(self.handle, key.encode(), str(value).encode()))

    def get_property(self, key):
        return _text(lib().hip_plugin_get_property, self.handle, key.encode(), size=4096)

    def device_name(self):
        return _text(lib().hip_plugin_device_name, self.handle, size=64)

    def import_model(self, blob, properties=None):
        text = ";".join("%s=%s" % kv for kv in (properties or {}).items()).encode() if properties else None
        h = _vp()
        _check(lib().hip_plugin_import_model(self.handle, blob, len(blob), text, ctypes.byref(h)))
        return CompiledModel(h)

    def query_model(self, model):
        names = _text(lib().hip_plugin_query_model, self.handle, model.handle)
        return names.split(",") if names else []

    def compile_model(self, model, properties=None):
        text = ";".join("%s=%s" % kv for kv in (properties or {}).items()).encode() if properties else None
        h = _vp()
        _check(lib().hip_plugin_compile_model(self.handle, model.handle, text, ctypes.byref(h)))
        return CompiledModel(h)

    def __del__(self):
        if self.handle:
            lib().hip_plugin_destroy(self.handle)
            self.handle = None


def memory_solver_pack(bytes_, start, end):
    """hip_memory_solver_pack: (offsets, blob size) for boxes of bytes_[i] alive from step start[i] to end[i]."""
    n = len(bytes_)
    offsets = (_sz * n)()
    total = lib().hip_memory_solver_pack(n, (_sz * n)(*bytes_), (_i * n)(*start), (_i * n)(*end), offsets)
    return list(offsets), total
