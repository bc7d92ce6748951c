"""GPU parity of libhipops.so (RMS norm, RoPE, MatMul, Gather, Concat, the gated MLP's element-wise
operators, Transpose, Convert) against the CPU oracle,
through the C ABI.  Byte movers are compared bit for bit; floating results against the oracle's
fp64-accumulated value, within one rounding of the output type plus the fp32 accumulation error
stated at each test.
"""
import ctypes

import numpy as np
import pytest

from openvino_contrib_amd import device_case as H
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu

F32, F16, BF16 = W.F32, W.F16, W.BF16
# half an ulp of the output type at magnitude 1, doubled for the kernel's fp32 arithmetic
ROUND = {F32: 2e-6, F16: 1e-3, BF16: 8e-3}


@pytest.fixture(scope="module")
def ops(hip):
    from openvino_contrib_amd import ops_capi

    ops_capi.lib()
    return ops_capi


def upload(hip, x, dtype):
    st, exact = W.to_storage(np.asarray(x, np.float32), dtype)
    return hip.DeviceBuffer.from_numpy(st), exact


def download(hip, buf, dtype, shape):
    return H.storage_to_f32(buf.download(W.np_storage_dtype(dtype), shape), dtype)


def scaled_error(got, ref):
    return float(np.max(np.abs(got - ref) / np.maximum(1.0, np.abs(ref))))


# ------------------------------------------------------------------------------ RMS norm
@pytest.mark.parametrize("rows,hidden", [(1, 8), (3, 37), (64, 4096), (5, 8192), (2, 20000), (4100, 128), (2500, 4096),
                                         (7, 4104)])
@pytest.mark.parametrize("x_dtype,g_dtype,o_dtype", [(F32, F32, F32), (F16, F16, F16), (BF16, BF16, BF16), (BF16, F32, BF16),
                                                     (F16, F32, F32)])
def test_rms_norm(hip, ops, oracle, rows, hidden, x_dtype, g_dtype, o_dtype):
    if rows * hidden > 6_000_000 and x_dtype != BF16:
        pytest.skip("the large shapes run once, in bf16")
    rng = np.random.default_rng(rows * 131 + hidden)
    print("[rms]", rows, hidden, x_dtype, g_dtype, o_dtype, flush=True)
    dx, x = upload(hip, rng.standard_normal((rows, hidden)) * 2.0, x_dtype)
    dg, g = upload(hip, 1.0 + 0.3 * rng.standard_normal(hidden), g_dtype)
    do = hip.DeviceBuffer(rows * hidden * hip.DTYPE_BYTES[o_dtype])
    ops.rms_norm(dx, dg, do, rows, hidden, 1e-5, x_dtype, g_dtype, o_dtype)
    got = download(hip, do, o_dtype, (rows, hidden))
    ref = oracle.rms_norm(x, g, 1e-5)
    assert scaled_error(got, ref) <= ROUND[o_dtype], scaled_error(got, ref)
    # without gamma, and in place
    ops.rms_norm(dx, None, dx if x_dtype == o_dtype else do, rows, hidden, 1e-5, x_dtype, g_dtype, o_dtype)
    got = download(hip, dx if x_dtype == o_dtype else do, o_dtype, (rows, hidden))
    assert scaled_error(got, oracle.rms_norm(x, None, 1e-5)) <= ROUND[o_dtype]


def test_rms_norm_unaligned_pointer_takes_the_scalar_path(hip, ops, oracle):
    rng = np.random.default_rng(7)
    rows, hidden = 6, 64
    st, exact = W.to_storage(rng.standard_normal((rows * hidden + 1,)).astype(np.float32), F16)
    dx = hip.DeviceBuffer.from_numpy(st)

    class Shifted:  # the same allocation, two bytes in
        ptr = ctypes.c_void_p(dx.ptr.value + 2)

    do = hip.DeviceBuffer(rows * hidden * 2)
    ops.rms_norm(Shifted, None, do, rows, hidden, 1e-6, F16, F16, F16)
    ref = oracle.rms_norm(exact[1:].reshape(rows, hidden), None, 1e-6)
    assert scaled_error(download(hip, do, F16, (rows, hidden)), ref) <= ROUND[F16]


def test_rms_norm_rejects_bad_arguments(hip, ops):
    buf = hip.DeviceBuffer(1024)
    with pytest.raises(ops.HipOpsError) as e:
        ops.rms_norm(buf, None, buf, 4, 0, 1e-6, F16, F16, F16)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.rms_norm(buf, None, buf, 4, 16, 1e-6, W.U8, F16, F16)
    assert e.value.status == hip.UNSUPPORTED
    ops.rms_norm(None, None, None, 0, 16, 1e-6, F16, F16, F16)  # no rows: nothing to do


# ------------------------------------------------------------------------------ RoPE
def rope_tables(rng, rows, width, interleaved, rot):
    theta = rng.uniform(0, 6.28, (rows, rot // 2))
    if interleaved:
        return np.cos(theta), np.sin(theta)
    theta2 = np.concatenate([theta, rng.uniform(0, 6.28, (rows, rot // 2))], axis=1)  # halves with angles of their own
    return np.cos(theta2), np.sin(theta2)


@pytest.mark.parametrize("T,Hh,S,rot", [(1, 1, 8, 8), (5, 3, 128, 128), (64, 32, 128, 128), (9, 2, 64, 32), (3, 5, 80, 16),
                                        (7, 2, 12, 6), (4000, 8, 128, 64)])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("dtype,tdtype", [(F32, F32), (F16, F32), (BF16, BF16), (F16, F16)])
def test_rope(hip, ops, oracle, T, Hh, S, rot, interleaved, dtype, tdtype):
    if T * Hh * S > 2_000_000 and dtype != BF16:
        pytest.skip("the large shape runs once, in bf16")
    rng = np.random.default_rng(T * 7 + S + rot)
    print("[rope]", T, Hh, S, rot, interleaved, dtype, tdtype, flush=True)
    rows = 3 * T + 5
    width = rot // 2 if interleaved else rot
    cos, sin = rope_tables(rng, rows, width, interleaved, rot)
    dx, x = upload(hip, rng.standard_normal((T, Hh, S)), dtype)
    dc, cos = upload(hip, cos, tdtype)
    ds, sin = upload(hip, sin, tdtype)
    positions = rng.integers(0, rows, T).astype(np.int32)
    dp = hip.DeviceBuffer.from_numpy(positions)
    do = hip.DeviceBuffer(T * Hh * S * hip.DTYPE_BYTES[dtype])
    d = ops.RopeDesc(dtype, tdtype, T, Hh, S, rot, int(interleaved), Hh * S, S, Hh * S, S, rows, width)
    ops.rope(d, dx, dc, ds, dp, do)
    ref = oracle.rope(x, cos, sin, positions, rot, interleaved)
    got = download(hip, do, dtype, (T, Hh, S))
    assert scaled_error(got, ref) <= 2 * ROUND[dtype], scaled_error(got, ref)
    assert np.array_equal(got[..., rot:], x[..., rot:])
    # token order as table row, in place
    ops.rope(d, dx, dc, ds, None, dx)
    got = download(hip, dx, dtype, (T, Hh, S))
    assert scaled_error(got, oracle.rope(x, cos, sin, None, rot, interleaved)) <= 2 * ROUND[dtype]


def test_rope_on_a_slice_of_a_packed_projection(hip, ops, oracle):
    """q, k and v of a token lie side by side; k is rotated where it lies and q into a buffer of its own."""
    rng = np.random.default_rng(11)
    T, Hq, Hkv, S = 33, 8, 2, 128
    width = (Hq + 2 * Hkv) * S
    dqkv, qkv = upload(hip, rng.standard_normal((T, width)), BF16)
    cos, sin = rope_tables(rng, T, S, False, S)
    dc, cos = upload(hip, cos, F32)
    ds, sin = upload(hip, sin, F32)
    dq = hip.DeviceBuffer(T * Hq * S * 2)
    ops.rope(ops.RopeDesc(BF16, F32, T, Hq, S, 0, 0, width, S, Hq * S, S, T, S), dqkv, dc, ds, None, dq)
    got_q = download(hip, dq, BF16, (T, Hq, S))
    assert scaled_error(got_q, oracle.rope(qkv[:, :Hq * S].reshape(T, Hq, S), cos, sin)) <= 2 * ROUND[BF16]

    class KSlice:
        ptr = ctypes.c_void_p(dqkv.ptr.value + Hq * S * 2)

    ops.rope(ops.RopeDesc(BF16, F32, T, Hkv, S, 0, 0, width, S, width, S, T, S), KSlice, dc, ds, None, KSlice)
    after = download(hip, dqkv, BF16, (T, width))
    ref_k = oracle.rope(qkv[:, Hq * S:(Hq + Hkv) * S].reshape(T, Hkv, S), cos, sin).reshape(T, Hkv * S)
    assert scaled_error(after[:, Hq * S:(Hq + Hkv) * S], ref_k) <= 2 * ROUND[BF16]
    assert np.array_equal(after[:, :Hq * S], qkv[:, :Hq * S]) and np.array_equal(after[:, (Hq + Hkv) * S:], qkv[:, (Hq + Hkv) * S:])


def test_rope_rejects_bad_descriptors(hip, ops):
    buf = hip.DeviceBuffer(4096)
    for d in (ops.RopeDesc(F16, F16, 4, 2, 16, 7, 0, 32, 16, 32, 16, 8, 16),   # odd rotary_ndims
              ops.RopeDesc(F16, F16, 4, 2, 16, 32, 0, 32, 16, 32, 16, 8, 32),  # rotary beyond the head
              ops.RopeDesc(F16, F16, 4, 2, 16, 16, 0, 32, 16, 32, 16, 8, 8),   # table rows too short
              ops.RopeDesc(F16, F16, 9, 2, 16, 16, 0, 32, 16, 32, 16, 8, 16),  # more tokens than rows, no positions
              ops.RopeDesc(F16, F16, 4, 2, 16, 16, 0, 32, 8, 32, 16, 8, 16)):  # head stride below the head size
        with pytest.raises(ops.HipOpsError) as e:
            ops.rope(d, buf, buf, buf, None, buf)
        assert e.value.status == hip.INVALID_ARGUMENT


# ------------------------------------------------------------------------------ MatMul
@pytest.mark.parametrize("m,n,k,batch", [(1, 16, 16, 1), (64, 6144, 4096, 1), (300, 200, 100, 1), (128, 128, 64, 6),
                                         (33, 17, 70, 3), (512, 4096, 4096, 1)])
@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_matmul(hip, ops, oracle, m, n, k, batch, ta, tb, dtype):
    if m * n * k > 5e8 and (dtype == F32 or ta):
        pytest.skip("the projection-sized shapes run in the 16-bit types, untransposed A")
    rng = np.random.default_rng(m + 3 * n + 7 * k + batch)
    print("[matmul]", m, n, k, batch, ta, tb, dtype, flush=True)
    a_shape = (batch, k, m) if ta else (batch, m, k)
    b_shape = (n, k) if tb else (k, n)  # one weight matrix for the whole batch
    da, a = upload(hip, rng.standard_normal(a_shape) * 0.5, dtype)
    db, b = upload(hip, rng.standard_normal(b_shape) * 0.5, dtype)
    dc = hip.DeviceBuffer(batch * m * n * hip.DTYPE_BYTES[dtype])
    d = ops.MatmulDesc(dtype, dtype, m, n, k, batch, int(ta), int(tb), m * k if batch > 1 else 0, 0)
    ws = hip.DeviceBuffer(ops.matmul_workspace_size(d))
    ops.matmul(d, da, db, dc, ws)
    got = download(hip, dc, dtype, (batch, m, n))
    if m * n * k > 5e8:  # the oracle on a sample of rows
        rows = rng.choice(m, 8, replace=False)
        a_s = a[:, :, rows] if ta else a[:, rows, :]
        ref, got = oracle.matmul(a_s, b, ta, tb), got[:, rows, :]
    else:
        ref = oracle.matmul(a, b, ta, tb)
    # fp32 accumulation of k products, then one rounding of the output (error relative to max(1, |ref|))
    bound = ROUND[dtype] + 1e-6 * np.sqrt(k)
    assert scaled_error(got, ref) <= bound, (scaled_error(got, ref), bound)
    # no workspace at all, f32 result
    if dtype != F32:
        dc32 = hip.DeviceBuffer(batch * m * n * 4)
        d32 = ops.MatmulDesc(dtype, F32, m, n, k, batch, int(ta), int(tb), m * k if batch > 1 else 0, 0)
        ops.matmul(d32, da, db, dc32, None)
        got32 = download(hip, dc32, F32, (batch, m, n))
        if m * n * k > 5e8:
            got32 = got32[:, rows, :]
        assert scaled_error(got32, ref) <= 1e-6 * np.sqrt(k) + 1e-6


def test_matmul_batched_b(hip, ops, oracle):
    rng = np.random.default_rng(21)
    batch, m, n, k = 5, 40, 24, 56
    da, a = upload(hip, rng.standard_normal((m, k)), F16)          # A broadcast
    db, b = upload(hip, rng.standard_normal((batch, k, n)), F16)   # B per batch
    dc = hip.DeviceBuffer(batch * m * n * 2)
    ops.matmul(ops.MatmulDesc(F16, F16, m, n, k, batch, 0, 0, 0, k * n), da, db, dc, None)
    got = download(hip, dc, F16, (batch, m, n))
    assert scaled_error(got, oracle.matmul(a, b)) <= ROUND[F16] + 1e-6 * np.sqrt(k)


def test_matmul_rejects_bad_descriptors(hip, ops):
    buf = hip.DeviceBuffer(1 << 16)
    for d, status in ((ops.MatmulDesc(F16, F16, 0, 8, 8, 1, 0, 0, 0, 0), hip.INVALID_ARGUMENT),
                      (ops.MatmulDesc(F16, F16, 8, 8, 8, 2, 0, 0, 10, 0), hip.INVALID_ARGUMENT),
                      (ops.MatmulDesc(F16, BF16, 8, 8, 8, 1, 0, 0, 0, 0), hip.UNSUPPORTED),
                      (ops.MatmulDesc(W.U8, W.U8, 8, 8, 8, 1, 0, 0, 0, 0), hip.UNSUPPORTED)):
        with pytest.raises(ops.HipOpsError) as e:
            ops.matmul(d, buf, buf, buf, None)
        assert e.value.status == status


# ------------------------------------------------------------------------------ Gather / Concat
@pytest.mark.parametrize("shape,axis,n_idx,itemsize", [((1000, 4096), 0, 64, 2), ((7, 5, 3), 1, 9, 4), ((3, 4, 6, 5), 2, 4, 1),
                                                      ((2, 3, 50), 2, 11, 2), ((32000, 128), 0, 8192, 2), ((5, 17), 0, 3, 1)])
@pytest.mark.parametrize("index_dtype", ["i32", "i64"])
def test_gather(hip, ops, oracle, shape, axis, n_idx, itemsize, index_dtype):
    rng = np.random.default_rng(sum(shape) + axis)
    print("[gather]", shape, axis, n_idx, itemsize, index_dtype, flush=True)
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[itemsize]
    data = rng.integers(0, 250, shape).astype(dt)
    n = shape[axis]
    idx = rng.integers(-n - 2, n + 2, n_idx)  # a few fall outside on either side
    ref = oracle.gather(data, idx, axis)
    dd = hip.DeviceBuffer.from_numpy(data)
    di = hip.DeviceBuffer.from_numpy(idx.astype(np.int32 if index_dtype == "i32" else np.int64))
    do = hip.DeviceBuffer(ref.nbytes)
    do.fill(0xEE)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64)) * itemsize
    ops.gather(dd, di, do, 1, outer, n, inner, n_idx, ops.I32 if index_dtype == "i32" else ops.I64)
    assert np.array_equal(do.download(dt, ref.shape), ref)


def test_gather_batch_dims_and_empty(hip, ops, oracle):
    rng = np.random.default_rng(31)
    data = rng.integers(0, 2 ** 16, (3, 4, 6, 5)).astype(np.uint16)
    idx = rng.integers(0, 6, (3, 7))
    ref = oracle.gather(data, idx, 2, batch_dims=1)
    dd, di = hip.DeviceBuffer.from_numpy(data), hip.DeviceBuffer.from_numpy(idx.astype(np.int64))
    do = hip.DeviceBuffer(ref.nbytes)
    ops.gather(dd, di, do, 3, 4, 6, 10, 7, ops.I64)
    assert np.array_equal(do.download(np.uint16, ref.shape), ref)
    ops.gather(dd, di, do, 3, 4, 6, 0, 7, ops.I64)   # a KV-cache gather at sequence length 0: no work
    ops.gather(dd, di, do, 3, 4, 6, 10, 0, ops.I64)
    with pytest.raises(ops.HipOpsError):
        ops.gather(dd, di, do, 3, 4, 6, 10, 7, 7)


@pytest.mark.parametrize("shape,axis,widths,itemsize", [((2, 4, 6), 1, (3, 0, 5, 1), 4), ((64, 1, 128), 1, (100, 1), 2),
                                                       ((5, 7), 0, (1, 2, 3), 1), ((3, 2, 9), 2, (9, 7, 1, 1, 2, 3, 4, 5, 6, 8, 10), 2),
                                                       ((1, 8, 1, 128), 2, (4095, 1), 2)])
def test_concat(hip, ops, oracle, shape, axis, widths, itemsize):
    rng = np.random.default_rng(len(widths) + axis)
    print("[concat]", shape, axis, widths, itemsize, flush=True)
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[itemsize]
    parts = []
    for w in widths:
        s = list(shape)
        s[axis] = w
        parts.append(rng.integers(0, 250, s).astype(dt))
    ref = oracle.concat(parts, axis)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    tail = int(np.prod(shape[axis + 1:], dtype=np.int64)) * itemsize
    bufs = [hip.DeviceBuffer.from_numpy(p) if p.size else None for p in parts]
    do = hip.DeviceBuffer(ref.nbytes)
    do.fill(0xEE)
    ops.concat(bufs, [w * tail for w in widths], outer, do)
    assert np.array_equal(do.download(dt, ref.shape), ref)


# ------------------------------------------------------------------------------ Swish, Multiply, GLU
@pytest.mark.parametrize("count", [1, 8, 37, 4096, 1_000_003])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_swish_and_multiply(hip, ops, oracle, count, dtype):
    rng = np.random.default_rng(count)
    print("[swish, multiply]", count, dtype, flush=True)
    da, a = upload(hip, rng.standard_normal(count) * 3, dtype)
    db, b = upload(hip, rng.standard_normal(count), dtype)
    do = hip.DeviceBuffer(count * hip.DTYPE_BYTES[dtype])
    ops.swish(da, do, count, dtype)
    assert scaled_error(download(hip, do, dtype, (count,)), oracle.swish(a)) <= ROUND[dtype]
    ops.swish(da, do, count, dtype, beta=1.7)
    assert scaled_error(download(hip, do, dtype, (count,)), oracle.swish(a, 1.7)) <= ROUND[dtype]
    ops.multiply(da, db, do, count, dtype)
    assert scaled_error(download(hip, do, dtype, (count,)), a * b) <= ROUND[dtype]
    ops.multiply(da, db, da, count, dtype)  # in place
    assert scaled_error(download(hip, da, dtype, (count,)), a * b) <= ROUND[dtype]


@pytest.mark.parametrize("rows,width", [(1, 8), (5, 37), (64, 14336), (3, 11008), (4100, 128)])
@pytest.mark.parametrize("activation", [0, 1, 2])
@pytest.mark.parametrize("gate_first", [True, False])
@pytest.mark.parametrize("dtype", [F32, BF16, F16])
def test_glu(hip, ops, oracle, rows, width, activation, gate_first, dtype):
    if rows * width > 500_000 and dtype != BF16:
        pytest.skip("the large shapes run once, in bf16")
    rng = np.random.default_rng(rows + width + activation)
    print("[glu]", rows, width, activation, gate_first, dtype, flush=True)
    dx, x = upload(hip, rng.standard_normal((rows, 2 * width)) * 2, dtype)
    do = hip.DeviceBuffer(rows * width * hip.DTYPE_BYTES[dtype])
    ops.glu(dx, do, rows, width, dtype, activation, gate_first)
    ref = oracle.glu(x, activation, gate_first)
    assert scaled_error(download(hip, do, dtype, (rows, width)), ref) <= ROUND[dtype]


def test_eltwise_rejects_bad_arguments(hip, ops):
    buf = hip.DeviceBuffer(256)
    for call in (lambda: ops.swish(buf, buf, -1, F16), lambda: ops.multiply(buf, None, buf, 8, F16),
                 lambda: ops.glu(buf, buf, 2, 0, F16), lambda: ops.glu(buf, buf, 2, 8, F16, activation=7)):
        with pytest.raises(ops.HipOpsError) as e:
            call()
        assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.swish(buf, buf, 8, W.U8)
    assert e.value.status == hip.UNSUPPORTED
    ops.swish(None, None, 0, F16)


# ------------------------------------------------------------------------------ Transpose, Convert
TRANSPOSE_CASES = [
    ((5,), (0,)), ((3, 4), (1, 0)), ((2, 3, 4), (0, 2, 1)), ((2, 3, 4), (2, 0, 1)), ((2, 1, 3, 4), (3, 1, 0, 2)),
    ((2, 3, 2, 3, 2, 3), (5, 3, 1, 4, 2, 0)), ((4, 1, 6), (1, 0, 2)), ((2, 3, 4, 5, 2, 3, 2, 2), (7, 0, 6, 1, 5, 2, 4, 3)),
    ((3, 77, 5, 64), (0, 2, 1, 3)),       # [b, l, h, d] -> [b, h, l, d]: rows of 64 elements move whole
    ((2, 300, 8, 128), (0, 2, 1, 3)),
    ((2, 8, 300, 128), (0, 2, 1, 3)),
    ((300, 8, 3, 128), (2, 0, 1, 3)),     # a packed q|k|v split into three tensors
    ((5, 130, 70), (0, 2, 1)),            # the innermost axis changes: tiles, with ragged edges
    ((1000, 3), (1, 0)), ((3, 1000), (1, 0)), ((65, 2, 67), (2, 1, 0)), ((4, 66, 3, 65), (3, 0, 2, 1)),
    ((3, 72, 200), (0, 2, 1)),            # tiles with 16-byte accesses on both sides and ragged edges
    ((2, 10, 3, 24), (0, 3, 2, 1)), ((2, 100, 4, 36), (0, 3, 2, 1)),  # wide reads, narrow writes; a row end inside a wide access
    ((2, 3, 4), (0, 1, 2)), ((6, 1, 1, 7), (0, 2, 1, 3)),  # nothing moves
]


@pytest.mark.parametrize("shape,order", TRANSPOSE_CASES)
@pytest.mark.parametrize("itemsize", [1, 2, 4, 8])
def test_transpose(hip, ops, oracle, shape, order, itemsize):
    rng = np.random.default_rng(sum(shape) * 7 + itemsize)
    print("[transpose]", shape, order, itemsize, flush=True)
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[itemsize]
    x = rng.integers(0, 2 ** (8 * min(itemsize, 4)) - 1, shape).astype(dt)
    ref = oracle.transpose(x, order)
    dx = hip.DeviceBuffer.from_numpy(x)
    do = hip.DeviceBuffer(max(ref.nbytes, 16))
    do.fill(0xEE)
    ops.transpose(dx, do, shape, order, itemsize)
    assert np.array_equal(do.download(dt, ref.shape), ref)


def test_transpose_odd_addresses_and_errors(hip, ops, oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(0, 65535, (1 + 6 * 10 * 24,)).astype(np.uint16)
    dx = hip.DeviceBuffer.from_numpy(x)
    do = hip.DeviceBuffer(x.nbytes + 16)

    class In:   # two bytes into the allocation: pieces of 2 bytes only
        ptr = ctypes.c_void_p(dx.ptr.value + 2)

    class Out:
        ptr = ctypes.c_void_p(do.ptr.value + 6)

    ops.transpose(In, Out, (6, 10, 24), (1, 0, 2), 2)
    got = do.download(np.uint16, (3 + 6 * 10 * 24,))[3:].reshape(10, 6, 24)
    assert np.array_equal(got, oracle.transpose(x[1:].reshape(6, 10, 24), (1, 0, 2)))
    ops.transpose(dx, do, (0, 4), (1, 0), 2)  # empty: nothing to do
    with pytest.raises(ops.HipOpsError) as e:
        ops.transpose(dx, do, (2, 3), (1, 1), 2)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.transpose(dx, dx, (2, 3), (1, 0), 2)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.transpose(dx, do, (2, 3), (1, 0), 3)
    assert e.value.status == hip.UNSUPPORTED


CONVERT_TYPES = [0, 1, 2, 100, 101, 102, 103, 104]


def convert_input(rng, src, n):
    """Storage array of element type `src`: ordinary values, ties, and everything the rules single out
    (NaN, infinities, values beyond every integer range, negative zero, bytes that are neither 0 nor 1)."""
    import torch
    if src in (0, 1, 2):
        v = np.concatenate([rng.uniform(-300, 300, n - 24), rng.uniform(-1, 1, 8) * 1e-3,
                            [np.nan, np.inf, -np.inf, 3e9, -3e9, 1e20, -1e20, 65504.0, 70000.0, 255.5, 127.5, -128.5, 0.0, -0.0, 0.5, -0.5]]).astype(np.float32)
        v[: n // 4] = np.round(v[: n // 4])
        v[n // 4: n // 2] = np.round(v[n // 4: n // 2]) + 0.5
        if src == 1:
            with np.errstate(over="ignore"):
                return v.astype(np.float16).view(np.uint16)
        if src == 2:
            return torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        return v
    storage = {100: np.int32, 101: np.int64, 102: np.uint8, 103: np.int8, 104: np.uint8}[src]
    info = np.iinfo(storage)
    v = rng.integers(info.min, info.max, n, dtype=np.int64, endpoint=True)
    v[: n // 2] = rng.integers(max(info.min, -300), min(info.max, 300), n // 2, endpoint=True)
    v[-4:] = [info.min, info.max, 0, 1]
    if src in (100, 101):
        v[-8:-4] = [2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 24) - 1, 65519]  # ties of the roundings to f32 and f16
    return v.astype(storage)


@pytest.mark.parametrize("src", CONVERT_TYPES)
@pytest.mark.parametrize("dst", CONVERT_TYPES)
def test_convert(hip, ops, oracle, src, dst):
    rng = np.random.default_rng(100 * src + dst)
    print("[convert]", src, dst, flush=True)
    for n in (24, 4099, 100_000):
        x = convert_input(rng, src, n)
        ref = oracle.convert(x, src, dst)
        dx = hip.DeviceBuffer.from_numpy(x)
        do = hip.DeviceBuffer(ref.nbytes)
        do.fill(0xEE)
        ops.convert(dx, do, n, src, dst)
        got = do.download(ref.dtype, ref.shape)
        if dst in (0, 1, 2):  # NaN payloads are not part of the contract; everything else is, -0.0 included
            floats = lambda a: a if dst == 0 else (oracle.f16_bits_to_f32(a) if dst == 1 else oracle.bf16_bits_to_f32(a))
            assert np.array_equal(np.isnan(floats(got)), np.isnan(floats(ref)))
            keep = ~np.isnan(floats(ref))
            got, ref = got[keep], ref[keep]
            if dst == 0:
                got, ref = got.view(np.uint32), ref.view(np.uint32)
        assert np.array_equal(got, ref), (src, dst, n, np.flatnonzero(got != ref)[:5])


def test_convert_odd_addresses_in_place_and_errors(hip, ops, oracle):
    rng = np.random.default_rng(9)
    x = rng.uniform(-100, 100, 1001).astype(np.float32)
    dx = hip.DeviceBuffer.from_numpy(x)
    do = hip.DeviceBuffer(4096)

    class In:   # four bytes in: no 16-byte loads
        ptr = ctypes.c_void_p(dx.ptr.value + 4)

    class Out:
        ptr = ctypes.c_void_p(do.ptr.value + 2)

    ops.convert(In, Out, 1000, 0, 1)
    got = do.download(np.uint16, (1001,))[1:]
    assert np.array_equal(got, oracle.convert(x[1:], 0, 1))
    ops.convert(dx, dx, 1001, 0, 0)  # equal types in place: nothing
    assert np.array_equal(dx.download(np.float32, (1001,)), x)
    ops.convert(dx, do, 0, 0, 1)
    with pytest.raises(ops.HipOpsError) as e:
        ops.convert(dx, do, 8, 0, 3)  # 3 names the quantised KV-cache rows, not an element type
    assert e.value.status == hip.UNSUPPORTED
    with pytest.raises(ops.HipOpsError) as e:
        ops.convert(dx, do, -1, 0, 1)
    assert e.value.status == hip.INVALID_ARGUMENT


# ------------------------------------------------------------------------------ broadcasting arithmetic, Softmax
BINARY_CASES = [((4, 8), (4, 8)), ((2, 3, 40, 64), (1, 1, 40, 64)), ((2, 3, 4, 5), (5,)), ((3, 1, 5), (1, 4, 1)), ((7,), ()), ((), ()),
                ((2, 1, 16), (2, 3, 1)), ((1, 8), (5, 1)), ((64, 4096), (4096,)), ((64, 4096), (64, 1)), ((3, 5, 24), (3, 1, 24)),
                ((2, 8, 130, 136), (2, 1, 1, 136)), ((2, 8, 130, 136), (1,)), ((0, 4), (1, 4))]


@pytest.mark.parametrize("a_shape,b_shape", BINARY_CASES)
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_binary_broadcasting(hip, ops, oracle, a_shape, b_shape, dtype):
    rng = np.random.default_rng(len(a_shape) * 7 + len(b_shape))
    print("[binary]", a_shape, b_shape, dtype, flush=True)
    da, a = upload(hip, rng.standard_normal(a_shape), dtype)
    db, b = upload(hip, rng.standard_normal(b_shape) + 3.0, dtype)  # away from zero: the divisor
    out_shape = np.broadcast_shapes(a_shape, b_shape)
    n = int(np.prod(out_shape, dtype=np.int64))
    do = hip.DeviceBuffer(max(n, 1) * hip.DTYPE_BYTES[dtype])
    for op in (ops.ADD, ops.SUBTRACT, ops.MULTIPLY, ops.DIVIDE):
        for swap in (False, True):
            x, y, dx, dy, xs, ys = (b, a, db, da, b_shape, a_shape) if swap else (a, b, da, db, a_shape, b_shape)
            if swap and op == ops.DIVIDE:
                continue  # a is not kept away from zero
            do.fill(0xEE)
            ops.binary(op, dx, dy, do, out_shape, xs, ys, dtype)
            if n == 0:
                continue
            ref = oracle.round_to(oracle.binary(op, x, y), dtype).reshape(out_shape)
            got = np.asarray(download(hip, do, dtype, out_shape)).reshape(out_shape)
            # one fp32 operation, one rounding: the same bits (the oracle rounds its fp32 result the same way)
            assert np.array_equal(got, ref), (op, swap, np.abs(got - ref).max())


def test_binary_in_place_unaligned_and_errors(hip, ops, oracle):
    rng = np.random.default_rng(4)
    st, x = W.to_storage(rng.standard_normal((1 + 6 * 24,)).astype(np.float32), F16)
    dx = hip.DeviceBuffer.from_numpy(st)
    db, b = upload(hip, rng.standard_normal((24,)), F16)

    class Shifted:  # two bytes in: the scalar path
        ptr = ctypes.c_void_p(dx.ptr.value + 2)

    ops.binary(ops.ADD, Shifted, db, Shifted, (6, 24), (6, 24), (24,), F16)  # in place on the full-shaped operand
    got = H.storage_to_f32(dx.download(np.uint16, (1 + 6 * 24,)), F16)[1:].reshape(6, 24)
    assert np.array_equal(got, oracle.round_to(oracle.binary(0, x[1:].reshape(6, 24), b), F16))
    with pytest.raises(ops.HipOpsError) as e:
        ops.binary(ops.ADD, dx, db, dx, (6, 24), (6, 24), (23,), F16)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.binary(7, dx, db, dx, (6, 24), (6, 24), (24,), F16)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.binary(ops.ADD, dx, db, dx, (6, 24), (6, 24), (24,), ops.I64)
    assert e.value.status == hip.UNSUPPORTED


@pytest.mark.parametrize("shape,axis", [((5, 9), 1), ((5, 9), 0), ((2, 3, 4, 5), 2), ((2, 8, 130, 136), 3), ((3, 1000), 1), ((7,), 0),
                                        ((64, 8192), 1), ((4, 33, 64), 1), ((2, 3, 0), 1), ((1, 1), 1)])
@pytest.mark.parametrize("dtype", [F32, F16, BF16])
def test_softmax(hip, ops, oracle, shape, axis, dtype):
    rng = np.random.default_rng(sum(shape) + axis)
    print("[softmax]", shape, axis, dtype, flush=True)
    dx, x = upload(hip, rng.standard_normal(shape) * 4, dtype)
    n = int(np.prod(shape, dtype=np.int64))
    do = hip.DeviceBuffer(max(n, 1) * hip.DTYPE_BYTES[dtype])
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    ops.softmax(dx, do, outer, shape[axis], inner, dtype)
    if n == 0:
        return
    got = download(hip, do, dtype, shape)
    ref = oracle.softmax(x, axis)
    # probabilities are at most 1: absolute error of one rounding plus the fast exponential's few ulps
    assert np.abs(got - ref).max() <= {F32: 2e-6, F16: 6e-4, BF16: 4.5e-3}[dtype]
    ops.softmax(dx, dx, outer, shape[axis], inner, dtype)  # in place
    assert np.array_equal(download(hip, dx, dtype, shape), got)


def test_softmax_masked_entries_and_errors(hip, ops, oracle):
    x = np.array([[0.0, -np.inf, 1.0, -np.inf, 0.5, -np.inf, -np.inf, -np.inf], [-np.inf] * 7 + [2.0], [-np.inf] * 8], np.float32)
    dx = hip.DeviceBuffer.from_numpy(x)
    do = hip.DeviceBuffer(x.nbytes)
    ops.softmax(dx, do, 3, 8, 1, F32)
    got = do.download(np.float32, x.shape)
    ref = oracle.softmax(x, 1)
    assert np.abs(got[:2] - ref[:2]).max() <= 2e-6 and np.isnan(got[2]).all() and np.isnan(ref[2]).all()
    with pytest.raises(ops.HipOpsError) as e:
        ops.softmax(dx, do, 3, -1, 1, F32)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(ops.HipOpsError) as e:
        ops.softmax(dx, do, 3, 8, 1, W.U8)
    assert e.value.status == hip.UNSUPPORTED
