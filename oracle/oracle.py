"""ctypes loader for the CPU oracle (oracle/hipattn_oracle.c, oracle/layer_ops_oracle.c).

Test infrastructure only: imported by tests/, the smoke check and the benchmark's
cpu_baseline leg.  The product package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhipattn_oracle.so")

F32, F16, BF16, U8 = 0, 1, 2, 3

_lib = None


def build(force=False):
    """Compile the oracle with the Makefile beside it."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
        L.oracle_num_threads.restype = i32
        L.oracle_set_num_threads.argtypes = [i32]
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = f32
        L.oracle_f32_to_f16.argtypes = [f32]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16.argtypes = [f32]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        for n in ("oracle_f32_to_f16_array", "oracle_f16_to_f32_array", "oracle_f32_to_bf16_array",
                  "oracle_bf16_to_f32_array"):
            getattr(L, n).argtypes = [vp, vp, i64]
            getattr(L, n).restype = None
        L.oracle_quant_u8_row.argtypes = [vp, i32, vp]
        L.oracle_quant_u8_row.restype = None
        L.oracle_dequant_u8_row.argtypes = [vp, i32, vp]
        L.oracle_dequant_u8_row.restype = None
        L.oracle_quant_u8_rows.argtypes = [vp, i64, i32, vp]
        L.oracle_quant_u8_rows.restype = None
        L.oracle_dequant_u8_rows.argtypes = [vp, i64, i32, vp]
        L.oracle_dequant_u8_rows.restype = None
        L.oracle_sdpa_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, f32]
        L.oracle_sdpa_f32.restype = i32
        L.oracle_sdpa_mask_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, f32, vp, vp]
        L.oracle_sdpa_mask_f32.restype = i32
        L.oracle_kv_cache_write.argtypes = [vp, vp, vp, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32]
        L.oracle_kv_cache_write.restype = i64
        L.oracle_gather_cache_rows.argtypes = [vp, i32, vp, i32, i32, i32, i32, i32, vp]
        L.oracle_gather_cache_rows.restype = None
        L.oracle_paged_attention.argtypes = [vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32,
                                             f32, i32, i32, vp, vp, vp]
        L.oracle_paged_attention.restype = i32
        L.oracle_paged_attention_scores.argtypes = [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, vp]
        L.oracle_paged_attention_scores.restype = i32
        L.oracle_rotate_key_cache.argtypes = [vp, i32, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32]
        L.oracle_rotate_key_cache.restype = i32
        L.oracle_rms_norm_f32.argtypes = [vp, vp, vp, i64, i64, f32]
        L.oracle_rms_norm_f32.restype = None
        L.oracle_rope_f32.argtypes = [vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i64]
        L.oracle_rope_f32.restype = None
        L.oracle_matmul_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i32, i32, i64, i64]
        L.oracle_matmul_f32.restype = None
        L.oracle_swish_f32.argtypes = [vp, vp, i64, f32]
        L.oracle_swish_f32.restype = None
        L.oracle_glu_f32.argtypes = [vp, vp, i64, i64, i32, i32]
        L.oracle_glu_f32.restype = None
        L.oracle_transpose_bytes.restype = i32
        L.oracle_transpose_bytes.argtypes = [vp, vp, i32, vp, vp, i64]
        L.oracle_convert.restype = i32
        L.oracle_convert.argtypes = [vp, vp, i64, i32, i32]
        L.oracle_binary_f32.restype = i32
        L.oracle_binary_f32.argtypes = [i32, vp, vp, vp, i32, vp, vp, vp]
        L.oracle_softmax_f32.restype = None
        L.oracle_softmax_f32.argtypes = [vp, vp, i64, i64, i64]
        L.oracle_gather_bytes.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64]
        L.oracle_gather_bytes.restype = None
        L.oracle_concat_bytes.argtypes = [vp, vp, i32, i64, vp]
        L.oracle_concat_bytes.restype = None
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def num_threads():
    return lib().oracle_num_threads()


def set_num_threads(n):
    lib().oracle_set_num_threads(int(n))


# ----------------------------------------------------------------------------- conversions
def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_f16_array(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_f16_to_f32_array(_p(h), _p(out), h.size)
    return out


def f32_to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_bf16_array(_p(x), _p(out), x.size)
    return out


def bf16_bits_to_f32(b):
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().oracle_bf16_to_f32_array(_p(b), _p(out), b.size)
    return out


def round_to(x, dtype):
    """fp32 array rounded to the storage type and expanded back to fp32."""
    if dtype == F32:
        return _c(x, np.float32).copy()
    if dtype == F16:
        return f16_bits_to_f32(f32_to_f16_bits(x))
    if dtype == BF16:
        return bf16_bits_to_f32(f32_to_bf16_bits(x))
    raise ValueError(dtype)


def cache_row_bytes(dtype, D):
    return {F32: 4 * D, F16: 2 * D, BF16: 2 * D, U8: D + 8}[dtype]


def quant_u8_rows(x):
    """x [..., D] fp32 -> uint8 [..., D + 8] rows of [scale][zp][D bytes]."""
    x = _c(x, np.float32)
    D = x.shape[-1]
    flat = x.reshape(-1, D)
    out = np.empty((flat.shape[0], D + 8), np.uint8)
    lib().oracle_quant_u8_rows(_p(flat), flat.shape[0], D, _p(out))
    return out.reshape(x.shape[:-1] + (D + 8,))


def dequant_u8_rows(rows):
    rows = _c(rows, np.uint8)
    D = rows.shape[-1] - 8
    flat = rows.reshape(-1, D + 8)
    out = np.empty((flat.shape[0], D), np.float32)
    lib().oracle_dequant_u8_rows(_p(flat), flat.shape[0], D, _p(out))
    return out.reshape(rows.shape[:-1] + (D,))


# ------------------------------------------------------------------------------ operators
def sdpa(q, k, v, causal=False, scale=0.0):
    """q [B,Hq,Lq,D], k/v [B,Hkv,Lk,D] fp32 -> out [B,Hq,Lq,D] fp32."""
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    B, Hq, Lq, D = q.shape
    _, Hkv, Lk, _ = k.shape
    out = np.empty_like(q)
    rc = lib().oracle_sdpa_f32(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, Lq, Lk, D, int(bool(causal)), float(scale))
    if rc:
        raise ValueError("oracle_sdpa_f32: bad arguments")
    return out


def sdpa_masked(q, k, v, mask, causal=False, scale=0.0):
    """SDPA with an attention mask broadcastable to [B,Hq,Lq,Lk]: float = added to the scaled scores,
    bool = True takes part (the operator's two mask forms)."""
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    B, Hq, Lq, D = q.shape
    _, Hkv, Lk, _ = k.shape
    mask = np.asarray(mask)
    if mask.dtype == np.bool_:
        mask = np.where(mask, np.float32(0.0), np.float32(-np.inf))
    mask = _c(mask, np.float32)
    while mask.ndim < 4:
        mask = mask[None]
    strides = np.zeros(4, np.int64)
    for ax, full in enumerate((B, Hq, Lq, Lk)):
        assert mask.shape[ax] in (1, full), "mask shape %s does not broadcast to %s" % (mask.shape, (B, Hq, Lq, Lk))
        strides[ax] = mask.strides[ax] // 4 if mask.shape[ax] == full and full > 1 else 0
    out = np.empty_like(q)
    rc = lib().oracle_sdpa_mask_f32(_p(q), _p(k), _p(v), _p(out), B, Hq, Hkv, Lq, Lk, D, int(bool(causal)),
                                    float(scale), _p(mask), _p(strides))
    if rc:
        raise ValueError("oracle_sdpa_mask_f32: bad arguments")
    return out


def kv_cache_write(k_new, v_new, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins, block_indices,
                   block_indices_begins, Hkv, D, block_size):
    """In-place scatter into uint8-viewed caches [num_blocks, Hkv, block_size, row_bytes]."""
    k_new, v_new = _c(k_new, np.float32), _c(v_new, np.float32)
    pl, sb = _c(past_lens, np.int32), _c(subsequence_begins, np.int32)
    bi, bb = _c(block_indices, np.int32), _c(block_indices_begins, np.int32)
    assert key_cache.dtype == np.uint8 and value_cache.dtype == np.uint8
    assert key_cache.flags.c_contiguous and value_cache.flags.c_contiguous
    num_blocks = key_cache.shape[0]
    return lib().oracle_kv_cache_write(_p(k_new), _p(v_new), _p(key_cache), _p(value_cache), cache_dtype, _p(pl),
                                       _p(sb), _p(bi), _p(bb), len(pl), Hkv, D, block_size, num_blocks)


def gather_cache_rows(cache, cache_dtype, seq_blocks, n, h, Hkv, D, block_size):
    seq_blocks = _c(seq_blocks, np.int32)
    out = np.empty((n, D), np.float32)
    lib().oracle_gather_cache_rows(_p(cache), cache_dtype, _p(seq_blocks), n, h, Hkv, D, block_size, _p(out))
    return out


def paged_attention(q, k_new, v_new, key_cache, value_cache, cache_dtype, past_lens, subsequence_begins,
                    block_indices, block_indices_begins, Hq, Hkv, D, block_size, scale=0.0, sliding_window=0,
                    do_write=True, alibi_slopes=None, sinks=None):
    """q [T, Hq*D] fp32; caches are uint8 views, updated in place when do_write; alibi_slopes, sinks: None or [Hq] f32.
    Returns out [T, Hq*D]."""
    q = _c(q, np.float32)
    k_new, v_new = _c(k_new, np.float32), _c(v_new, np.float32)
    pl, sb = _c(past_lens, np.int32), _c(subsequence_begins, np.int32)
    bi, bb = _c(block_indices, np.int32), _c(block_indices_begins, np.int32)
    assert key_cache.dtype == np.uint8 and value_cache.dtype == np.uint8
    out = np.zeros_like(q)
    al = None if alibi_slopes is None else _c(alibi_slopes, np.float32)
    assert al is None or al.shape == (Hq,)
    sk = None if sinks is None else _c(sinks, np.float32)
    assert sk is None or sk.shape == (Hq,)
    rc = lib().oracle_paged_attention(_p(q), _p(k_new), _p(v_new), _p(key_cache), _p(value_cache), cache_dtype,
                                      _p(pl), _p(sb), _p(bi), _p(bb), len(pl), Hq, Hkv, D, block_size,
                                      key_cache.shape[0], float(scale), int(sliding_window), int(bool(do_write)),
                                      _p(al) if al is not None else None, _p(sk) if sk is not None else None, _p(out))
    if rc:
        raise ValueError("oracle_paged_attention: bad arguments")
    return out


def paged_attention_scores(q, key_cache, cache_dtype, past_lens, subsequence_begins, block_indices, block_indices_begins,
                           Hq, Hkv, D, block_size, score_window=None, scale=0.0, sliding_window=0):
    """The operator's second output from the cache as it stands (after the step's write): f32
    [sum(past_lens) + tokens], sequence after sequence."""
    q = _c(q, np.float32)
    pl, sb = _c(past_lens, np.int32), _c(subsequence_begins, np.int32)
    bi, bb = _c(block_indices, np.int32), _c(block_indices_begins, np.int32)
    sw = None if score_window is None else _c(score_window, np.int32)
    total = int(pl.sum()) + int(sb[-1] - sb[0])
    out = np.zeros(total, np.float32)
    rc = lib().oracle_paged_attention_scores(_p(q), _p(key_cache), cache_dtype, _p(pl), _p(sb), _p(bi), _p(bb),
                                             _p(sw) if sw is not None else None, len(pl), Hq, Hkv, D, block_size,
                                             key_cache.shape[0], float(scale), int(sliding_window), _p(out))
    if rc:
        raise ValueError("oracle_paged_attention_scores: bad arguments")
    return out


def rotate_key_cache(key_cache, cache_dtype, rotated_block_indices, rotation_deltas, rotation_trig_lut, Hkv, D, block_size):
    """The operator's cache rotation, in place on key_cache (a uint8 view).  rotation_deltas: [n, 1] or
    [n, block_size] int32; rotation_trig_lut: [rows, D] fp32 (D/2 cosines, then D/2 sines per row)."""
    assert key_cache.dtype == np.uint8 and key_cache.flags.c_contiguous
    idx = _c(rotated_block_indices, np.int32)
    deltas = _c(rotation_deltas, np.int32).reshape(len(idx), -1)
    lut = _c(rotation_trig_lut, np.float32)
    assert lut.ndim == 2 and lut.shape[1] == D
    rc = lib().oracle_rotate_key_cache(_p(key_cache), cache_dtype, _p(idx), len(idx), _p(deltas), deltas.shape[1] if len(idx) else 1,
                                       _p(lut), lut.shape[0], Hkv, D, block_size, key_cache.shape[0])
    if rc:
        raise ValueError("oracle_rotate_key_cache: bad arguments")


# ---- the operators either side of attention (oracle/layer_ops_oracle.c) ------------------------
def rms_norm(x, gamma=None, eps=1e-6):
    """x [..., hidden] fp32, gamma [hidden] or None -> like x."""
    x = _c(x, np.float32)
    hidden = x.shape[-1]
    g = None if gamma is None else _c(gamma, np.float32)
    out = np.empty_like(x)
    lib().oracle_rms_norm_f32(_p(x), _p(g) if g is not None else None, _p(out), x.size // hidden, hidden, float(eps))
    return out


def rope(x, cos, sin, positions=None, rotary_ndims=0, interleaved=False):
    """x [tokens, heads, head_size] fp32; cos/sin [rows, rotary_ndims] (rotate-half) or
    [rows, rotary_ndims/2] (adjacent pairs); positions int32 [tokens] or None (row = token)."""
    x, cos, sin = _c(x, np.float32), _c(cos, np.float32), _c(sin, np.float32)
    T, H, S = x.shape
    rotary = rotary_ndims or S
    assert cos.shape == sin.shape and cos.shape[1] == (rotary // 2 if interleaved else rotary)
    pos = None if positions is None else _c(positions, np.int32)
    out = np.empty_like(x)
    lib().oracle_rope_f32(_p(x), _p(cos), _p(sin), _p(pos) if pos is not None else None, _p(out), T, H, S, rotary,
                          int(bool(interleaved)), cos.shape[1])
    return out


def matmul(a, b, transpose_a=False, transpose_b=False):
    """a [batch?, ., .], b [batch?, ., .] fp32 (2-D operands broadcast over the other's batch) -> [batch?, m, n]."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    batch = max(a.shape[0] if a.ndim == 3 else 1, b.shape[0] if b.ndim == 3 else 1)
    m, k = (a.shape[-1], a.shape[-2]) if transpose_a else (a.shape[-2], a.shape[-1])
    n = b.shape[-2] if transpose_b else b.shape[-1]
    assert (b.shape[-1] if transpose_b else b.shape[-2]) == k
    sa = m * k if a.ndim == 3 and a.shape[0] > 1 else 0
    sb = k * n if b.ndim == 3 and b.shape[0] > 1 else 0
    c = np.empty((batch, m, n), np.float32)
    lib().oracle_matmul_f32(_p(a), _p(b), _p(c), m, n, k, batch, int(transpose_a), int(transpose_b), sa, sb)
    return c if (a.ndim == 3 or b.ndim == 3) else c[0]


def gather(data, indices, axis=0, batch_dims=0):
    """Gather (opset 8 rules: negative indices wrap, rows out of range are zero) on any dtype."""
    data = np.ascontiguousarray(data)
    idx = _c(indices, np.int64)
    batch = int(np.prod(data.shape[:batch_dims], dtype=np.int64))
    outer = int(np.prod(data.shape[batch_dims:axis], dtype=np.int64))
    axis_dim = data.shape[axis]
    inner = int(np.prod(data.shape[axis + 1:], dtype=np.int64)) * data.dtype.itemsize
    n_idx = int(np.prod(idx.shape[batch_dims:], dtype=np.int64))
    out_shape = data.shape[:axis] + idx.shape[batch_dims:] + data.shape[axis + 1:]
    out = np.empty(out_shape, data.dtype)
    lib().oracle_gather_bytes(_p(data), _p(idx), _p(out), batch, outer, axis_dim, inner, n_idx)
    return out


def concat(arrays, axis):
    arrays = [np.ascontiguousarray(a) for a in arrays]
    first = arrays[0]
    axis = axis % first.ndim
    outer = int(np.prod(first.shape[:axis], dtype=np.int64))
    tail = int(np.prod(first.shape[axis + 1:], dtype=np.int64)) * first.dtype.itemsize
    widths = np.array([a.shape[axis] * tail for a in arrays], np.int64)
    shape = list(first.shape)
    shape[axis] = sum(a.shape[axis] for a in arrays)
    out = np.empty(shape, first.dtype)
    ptrs = (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    lib().oracle_concat_bytes(ptrs, _p(widths), len(arrays), outer, _p(out))
    return out


def transpose(x, order):
    """x with output axis k taken from input axis order[k] (numpy.transpose's rule), any dtype."""
    x = np.ascontiguousarray(x)
    order = [int(o) for o in order]
    out = np.empty([x.shape[o] for o in order], x.dtype)
    dims, od = np.array(x.shape, np.int64), np.array(order, np.int32)
    if lib().oracle_transpose_bytes(_p(x), _p(out), x.ndim, _p(dims), _p(od), x.dtype.itemsize):
        raise ValueError("oracle_transpose_bytes: bad arguments")
    return out


# element types of the Convert operator: code -> numpy storage type (f16 / bf16 travel as their bits)
CONVERT_STORAGE = {0: np.float32, 1: np.uint16, 2: np.uint16, 100: np.int32, 101: np.int64, 102: np.uint8, 103: np.int8, 104: np.uint8}


def convert(x, from_dtype, to_dtype):
    """Convert on storage arrays (CONVERT_STORAGE); returns the storage array of to_dtype."""
    x = _c(x, CONVERT_STORAGE[from_dtype])
    out = np.empty(x.shape, CONVERT_STORAGE[to_dtype])
    if lib().oracle_convert(_p(x), _p(out), x.size, from_dtype, to_dtype):
        raise ValueError("oracle_convert: unknown element type")
    return out


def binary(op, a, b):
    """a (op) b with numpy broadcasting, one fp32 operation per element; op: 0 add, 1 subtract, 2 multiply, 3 divide."""
    a, b = np.require(np.asarray(a, np.float32), requirements="C"), np.require(np.asarray(b, np.float32), requirements="C")
    out_shape = np.broadcast_shapes(a.shape, b.shape)
    n = len(out_shape)
    pad = lambda s: np.array([1] * (n - len(s)) + list(s), np.int64)
    out = np.empty(out_shape, np.float32)
    od, ad, bd = pad(out_shape), pad(a.shape), pad(b.shape)
    if lib().oracle_binary_f32(op, _p(a), _p(b), _p(out), n, _p(od), _p(ad), _p(bd)):
        raise ValueError("oracle_binary_f32: shapes do not broadcast")
    return out


def softmax(x, axis=-1):
    x = _c(x, np.float32)
    axis = axis % x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    out = np.empty_like(x)
    lib().oracle_softmax_f32(_p(x), _p(out), outer, x.shape[axis], inner)
    return out


def swish(x, beta=1.0):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().oracle_swish_f32(_p(x), _p(out), x.size, float(beta))
    return out


def glu(x, activation=0, gate_first=True):
    """x [..., 2 * width] -> act(gate half) * other half; activation 0 swish, 1 gelu (erf), 2 gelu (tanh)."""
    x = _c(x, np.float32)
    width = x.shape[-1] // 2
    out = np.empty(x.shape[:-1] + (width,), np.float32)
    lib().oracle_glu_f32(_p(x), _p(out), x.size // (2 * width), width, int(activation), int(bool(gate_first)))
    return out
