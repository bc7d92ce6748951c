"""Randomly drawn shapes, element types, operand layouts and address offsets for every operator of
libhipops.so, against the CPU oracle (gpu).  The hand-picked cases of test_gpu_layer_ops.py sit on
the boundaries that were thought of; these do not.  Seeds are fixed, so a failure names its case.

Byte movers, Convert and the broadcasting arithmetic are compared bit for bit; RMS norm, RoPE, GLU
and Softmax within one rounding of the output type (f32 Softmax: plus 1e-8 per element of the axis,
the growth of an fp32 sum that the oracle takes in fp64).
"""
import ctypes

import numpy as np
import pytest

from openvino_contrib_amd import device_case as H
from openvino_contrib_amd import workloads as W
from test_gpu_layer_ops import convert_input

pytestmark = pytest.mark.gpu

F32, F16, BF16 = W.F32, W.F16, W.BF16
ROUND = {F32: 2e-6, F16: 1e-3, BF16: 8e-3}
CONVERT_TYPES = [0, 1, 2, 100, 101, 102, 103, 104]
BYTES = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}


class Shifted:
    """A device address `nbytes` into an allocation."""

    def __init__(self, buf, nbytes):
        self.ptr = ctypes.c_void_p(buf.ptr.value + nbytes)


class Box:
    """The libraries and the oracle, with the upload / download helpers the cases share."""

    def __init__(self, hip, ops, oracle):
        self.hip, self.ops, self.oracle = hip, ops, oracle

    def up(self, x, dtype):
        st, exact = W.to_storage(np.asarray(x, np.float32), dtype)
        return self.hip.DeviceBuffer.from_numpy(st), exact

    def down(self, buf, dtype, shape):
        return np.asarray(H.storage_to_f32(buf.download(W.np_storage_dtype(dtype), shape), dtype)).reshape(shape)

    def buffer(self, nbytes, fill=0xEE):
        b = self.hip.DeviceBuffer(max(nbytes, 16))
        b.fill(fill)
        return b


@pytest.fixture(scope="module")
def box(hip, oracle):
    from openvino_contrib_amd import ops_capi

    ops_capi.lib()
    return Box(hip, ops_capi, oracle)


def dims(rng, rank, special=9, limit=1_000_000):
    shape = [int(rng.choice([1, 2, 3, 5, 8, 16, 24, special, 64, 72, int(rng.integers(1, 40))])) for _ in range(rank)]
    while np.prod(shape, dtype=np.int64) > limit:
        shape = [max(1, d // 2) for d in shape]
    return tuple(shape)


def scaled_error(got, ref):
    return float(np.max(np.abs(got - ref) / np.maximum(1.0, np.abs(ref)))) if got.size else 0.0


def case_transpose(box, rng):
    rank = int(rng.integers(1, 7))
    shape = dims(rng, rank, limit=2_000_000)
    order = tuple(int(v) for v in rng.permutation(rank))
    item = int(rng.choice([1, 2, 4, 8]))
    x = rng.integers(0, 250, shape).astype(BYTES[item])
    ref = box.oracle.transpose(x, order)
    off_in, off_out = int(rng.choice([0, 0, item, 16])), int(rng.choice([0, 0, item, 16]))
    raw = np.zeros(x.size + 32, BYTES[item])
    raw[off_in // item: off_in // item + x.size] = x.reshape(-1)
    dx = box.hip.DeviceBuffer.from_numpy(raw)
    do = box.buffer(ref.nbytes + 64)
    box.ops.transpose(Shifted(dx, off_in), Shifted(do, off_out), shape, order, item)
    got = do.download(np.uint8, (ref.nbytes + 64,))[off_out: off_out + ref.nbytes].view(BYTES[item]).reshape(ref.shape)
    assert np.array_equal(got, ref), (shape, order, item, off_in, off_out)


def case_binary(box, rng):
    out = dims(rng, int(rng.integers(0, 6)))

    def operand():  # the output's shape with some extents at 1 and, where they are 1, some leading axes dropped
        s = tuple(d if rng.random() < 0.6 else 1 for d in out)
        drop = int(rng.integers(0, len(s) + 1))
        while drop > 0 and any(d != 1 for d in s[:drop]):
            drop -= 1
        return s[drop:]

    a_shape, b_shape = operand(), operand()
    out = np.broadcast_shapes(a_shape, b_shape)
    dtype, op = int(rng.choice([F32, F16, BF16])), int(rng.integers(0, 4))
    da, a = box.up(rng.standard_normal(a_shape), dtype)
    db, b = box.up(rng.standard_normal(b_shape) + 3.0, dtype)
    n = int(np.prod(out, dtype=np.int64))
    do = box.buffer(n * box.hip.DTYPE_BYTES[dtype])
    box.ops.binary(op, da, db, do, out, a_shape, b_shape, dtype)
    if n:
        ref = np.asarray(box.oracle.round_to(box.oracle.binary(op, a, b), dtype)).reshape(out)
        assert np.array_equal(box.down(do, dtype, out), ref), (op, a_shape, b_shape, dtype)


def case_softmax(box, rng):
    rank = int(rng.integers(1, 5))
    shape = dims(rng, rank, special=int(rng.choice([9, 130, 520, 2048, 3000])))
    axis, dtype = int(rng.integers(0, rank)), int(rng.choice([F32, F16, BF16]))
    dx, x = box.up(rng.standard_normal(shape) * 4, dtype)
    do = box.buffer(int(np.prod(shape)) * box.hip.DTYPE_BYTES[dtype])
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    box.ops.softmax(dx, do, outer, shape[axis], inner, dtype)
    err = np.abs(box.down(do, dtype, shape) - box.oracle.softmax(x, axis)).max()
    assert err <= {F32: 2e-6 + 1e-8 * shape[axis], F16: 6e-4, BF16: 4.5e-3}[dtype], (shape, axis, dtype, err)


def case_convert(box, rng):
    src, dst = int(rng.choice(CONVERT_TYPES)), int(rng.choice(CONVERT_TYPES))
    n = int(rng.choice([24, 25, 31, 100, 4099, int(rng.integers(24, 20000))]))
    x = convert_input(rng, src, n)
    ref = box.oracle.convert(x, src, dst)
    off_in = int(rng.choice([0, 0, 1, 2])) * x.dtype.itemsize
    off_out = int(rng.choice([0, 0, 1, 2])) * ref.dtype.itemsize
    raw = np.zeros(x.nbytes + 64, np.uint8)
    raw[off_in: off_in + x.nbytes] = x.view(np.uint8)
    dx = box.hip.DeviceBuffer.from_numpy(raw)
    do = box.buffer(ref.nbytes + 64)
    box.ops.convert(Shifted(dx, off_in), Shifted(do, off_out), n, src, dst)
    got = do.download(np.uint8, (ref.nbytes + 64,))[off_out: off_out + ref.nbytes].view(ref.dtype)
    if dst in (0, 1, 2):  # NaN payloads are not part of the contract
        floats = lambda a: a if dst == 0 else (box.oracle.f16_bits_to_f32(a) if dst == 1 else box.oracle.bf16_bits_to_f32(a))
        assert np.array_equal(np.isnan(floats(got)), np.isnan(floats(ref)))
        keep = ~np.isnan(floats(ref))
        got, ref = got[keep], ref[keep]
        if dst == 0:
            got, ref = got.view(np.uint32), ref.view(np.uint32)
    assert np.array_equal(got, ref), (src, dst, n, off_in, off_out)


def case_gather(box, rng):
    rank = int(rng.integers(1, 5))
    shape = dims(rng, rank, limit=500_000)
    axis = int(rng.integers(0, rank))
    batch_dims = int(rng.integers(0, min(axis, 1) + 1))
    item = int(rng.choice([1, 2, 4]))
    data = rng.integers(0, 250, shape).astype(BYTES[item])
    idx_shape = shape[:batch_dims] + dims(rng, int(rng.integers(0, 3)), special=7)
    n = shape[axis]
    idx = rng.integers(-n - 1, n + 1, idx_shape)  # a few fall outside on either side
    ref = box.oracle.gather(data, idx, axis, batch_dims=batch_dims)
    wide = bool(rng.random() < 0.5)
    dd = box.hip.DeviceBuffer.from_numpy(data)
    flat = np.ascontiguousarray(idx).astype(np.int64 if wide else np.int32).reshape(-1)
    di = box.hip.DeviceBuffer.from_numpy(flat if flat.size else np.zeros(1, np.int64))
    do = box.buffer(ref.nbytes)
    batch = int(np.prod(shape[:batch_dims], dtype=np.int64))
    outer = int(np.prod(shape[batch_dims:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64)) * item
    count = int(np.prod(idx_shape[batch_dims:], dtype=np.int64))
    box.ops.gather(dd, di, do, batch, outer, n, inner, count, box.ops.I64 if wide else box.ops.I32)
    if ref.size:
        assert np.array_equal(do.download(BYTES[item], ref.shape), ref), (shape, axis, batch_dims, idx_shape, item)


def case_concat(box, rng):
    rank = int(rng.integers(1, 5))
    shape = list(dims(rng, rank, limit=200_000))
    axis, item = int(rng.integers(0, rank)), int(rng.choice([1, 2, 4]))
    widths = [int(rng.choice([0, 1, 2, 3, 8, 17])) for _ in range(int(rng.integers(1, 12)))]
    parts = []
    for w in widths:
        s = list(shape)
        s[axis] = w
        parts.append(rng.integers(0, 250, s).astype(BYTES[item]))
    ref = box.oracle.concat(parts, axis)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    tail = int(np.prod(shape[axis + 1:], dtype=np.int64)) * item
    bufs = [box.hip.DeviceBuffer.from_numpy(p) if p.size else None for p in parts]
    do = box.buffer(ref.nbytes)
    box.ops.concat(bufs, [w * tail for w in widths], outer, do)
    if ref.size:
        assert np.array_equal(do.download(BYTES[item], ref.shape), ref), (shape, axis, widths, item)


def case_rms_norm(box, rng):
    rows = int(rng.choice([1, 3, 4, 5, 64, 300]))
    hidden = int(rng.choice([8, 37, 64, 128, 1000, 4096, 4104, 8200, int(rng.integers(1, 3000))]))
    x_dtype, g_dtype, o_dtype = (int(rng.choice([F32, F16, BF16])) for _ in range(3))
    eps = float(rng.choice([1e-12, 1e-6, 1e-5, 1e-2]))
    dx, x = box.up(rng.standard_normal((rows, hidden)) * 2, x_dtype)
    dg, g = box.up(1 + 0.3 * rng.standard_normal(hidden), g_dtype)
    with_gamma = bool(rng.random() < 0.8)
    do = box.buffer(rows * hidden * box.hip.DTYPE_BYTES[o_dtype])
    box.ops.rms_norm(dx, dg if with_gamma else None, do, rows, hidden, eps, x_dtype, g_dtype, o_dtype)
    err = scaled_error(box.down(do, o_dtype, (rows, hidden)), box.oracle.rms_norm(x, g if with_gamma else None, eps))
    assert err <= ROUND[o_dtype], (rows, hidden, x_dtype, g_dtype, o_dtype, err)


def case_rope(box, rng):
    T, heads = int(rng.choice([1, 2, 7, 33, 200])), int(rng.choice([1, 2, 3, 8]))
    size = int(rng.choice([16, 32, 64, 80, 96, 128, 256]))
    rot = int(rng.choice([size, size // 2, size, 8]))
    interleaved = bool(rng.random() < 0.4)
    dtype, table_dtype = int(rng.choice([F32, F16, BF16])), int(rng.choice([F32, F16, BF16]))
    rows, width = 3 * T + 5, (rot // 2 if interleaved else rot)
    angle = rng.uniform(-3, 3, (rows, rot // 2))
    if not interleaved:
        angle = np.concatenate([angle, angle + 0.1], 1)  # the two halves of a row need not agree
    # heads and tokens with gaps between them, as inside a packed projection
    head_stride = size + int(rng.choice([0, 0, 8]))
    token_stride = heads * head_stride + int(rng.choice([0, 0, 8, 24]))
    dx, full = box.up(rng.standard_normal((T, token_stride)), dtype)
    x = np.ascontiguousarray(np.stack([full[:, h * head_stride: h * head_stride + size] for h in range(heads)], 1))
    dc, cos = box.up(np.cos(angle), table_dtype)
    ds, sin = box.up(np.sin(angle), table_dtype)
    positions = rng.integers(0, rows, T).astype(np.int32)
    with_positions = bool(rng.random() < 0.6)
    dp = box.hip.DeviceBuffer.from_numpy(positions)
    do = box.buffer(T * heads * size * box.hip.DTYPE_BYTES[dtype])
    desc = box.ops.RopeDesc(dtype, table_dtype, T, heads, size, rot, int(interleaved), token_stride, head_stride, heads * size, size,
                            rows, width)
    box.ops.rope(desc, dx, dc, ds, dp if with_positions else None, do)
    ref = box.oracle.rope(x, cos, sin, positions if with_positions else None, rot, interleaved)
    err = scaled_error(box.down(do, dtype, (T, heads, size)), ref)
    assert err <= 2 * ROUND[dtype], (T, heads, size, rot, interleaved, dtype, table_dtype, token_stride, head_stride, err)


def case_glu(box, rng):
    rows, width = int(rng.choice([1, 3, 64, 257])), int(rng.choice([8, 24, 37, 128, 1000, 4096]))
    dtype, activation, gate_first = int(rng.choice([F32, F16, BF16])), int(rng.integers(0, 3)), bool(rng.random() < 0.5)
    dx, x = box.up(rng.standard_normal((rows, 2 * width)) * 2, dtype)
    do = box.buffer(rows * width * box.hip.DTYPE_BYTES[dtype])
    box.ops.glu(dx, do, rows, width, dtype, activation, gate_first)
    err = scaled_error(box.down(do, dtype, (rows, width)), box.oracle.glu(x, activation, gate_first))
    assert err <= 2 * ROUND[dtype], (rows, width, dtype, activation, gate_first, err)


CASES = [case_transpose, case_binary, case_softmax, case_convert, case_gather, case_concat, case_rms_norm, case_rope, case_glu]


@pytest.mark.parametrize("case", CASES, ids=lambda f: f.__name__[5:])
def test_random_operator_cases(box, case):
    for seed in range(150):
        print("[case] random", case.__name__, seed, flush=True)
        case(box, np.random.default_rng(7000 + 100 * seed + CASES.index(case)))
