"""Pins the CPU oracle of the operators around attention (oracle/layer_ops_oracle.c) without a GPU.

Each function is checked against a library routine or a formulation that does not share its code:
torch's rms_norm and the transformers library's rotary helpers (committed fixtures), complex
multiplication, numpy's matmul / take / concatenate, and invariants a wrong sign, index or
transposed operand breaks.
"""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layer_ops_golden.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


@pytest.mark.parametrize("name", ["rms_small", "rms_odd", "rms_wide"])
def test_rms_norm_matches_torch_fixture(oracle, golden, name):
    out = oracle.rms_norm(golden[name + "/x"], golden[name + "/gamma"], float(golden[name + "/eps"]))
    np.testing.assert_allclose(out, golden[name + "/out"], rtol=2e-6, atol=1e-7)


def test_rms_norm_invariants(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((7, 96)).astype(np.float32)
    out = oracle.rms_norm(x, None, 0.0)
    np.testing.assert_allclose((out.astype(np.float64) ** 2).mean(-1), 1.0, rtol=1e-6)  # unit mean square
    np.testing.assert_allclose(oracle.rms_norm(4.0 * x, None, 0.0), out, rtol=1e-6)       # scale invariance at eps 0
    g = rng.standard_normal(96).astype(np.float32)
    np.testing.assert_allclose(oracle.rms_norm(x, g, 1e-6), oracle.rms_norm(x, None, 1e-6) * g, rtol=1e-6)
    big_eps = oracle.rms_norm(x, None, 1e6)  # eps dominates: out ~ x / 1000
    np.testing.assert_allclose(big_eps, x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e6), rtol=1e-6)


@pytest.mark.parametrize("name,rot,interleaved", [("llama", 16, False), ("llama_partial", 8, False), ("gptj", 16, True),
                                                  ("gptj_partial", 8, True)])
def test_rope_matches_transformers_fixture(oracle, golden, name, rot, interleaved):
    out = oracle.rope(golden[name + "/x"], golden[name + "/cos"], golden[name + "/sin"], None, rot, interleaved)
    np.testing.assert_allclose(out, golden[name + "/out"], rtol=0, atol=2e-6)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_is_a_complex_rotation(oracle, interleaved):
    rng = np.random.default_rng(2)
    T, H, S, rot = 9, 3, 32, 24
    half = rot // 2
    x = rng.standard_normal((T, H, S)).astype(np.float32)
    theta = rng.uniform(0, 6.28, (50, half))
    positions = rng.integers(0, 50, T).astype(np.int32)
    if interleaved:
        cos, sin = np.cos(theta), np.sin(theta)
        z = x[..., 0:rot:2].astype(np.float64) + 1j * x[..., 1:rot:2]
    else:
        cos, sin = np.cos(np.tile(theta, 2)), np.sin(np.tile(theta, 2))
        z = x[..., :half].astype(np.float64) + 1j * x[..., half:rot]
    w = z * np.exp(1j * theta[positions])[:, None, :]
    out = oracle.rope(x, cos, sin, positions, rot, interleaved)
    if interleaved:
        np.testing.assert_allclose(out[..., 0:rot:2], w.real, atol=2e-6)
        np.testing.assert_allclose(out[..., 1:rot:2], w.imag, atol=2e-6)
    else:
        np.testing.assert_allclose(out[..., :half], w.real, atol=2e-6)
        np.testing.assert_allclose(out[..., half:rot], w.imag, atol=2e-6)
    assert np.array_equal(out[..., rot:], x[..., rot:])                     # the tail passes through
    np.testing.assert_allclose(np.linalg.norm(out, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-6)
    back = oracle.rope(out, cos, -sin, positions, rot, interleaved)          # rotate by -theta
    np.testing.assert_allclose(back, x, atol=3e-6)
    ident = oracle.rope(x, np.ones_like(cos), np.zeros_like(sin), positions, rot, interleaved)
    assert np.array_equal(ident, x)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_matches_numpy(oracle, ta, tb):
    rng = np.random.default_rng(3)
    m, n, k = 13, 7, 29
    a = rng.standard_normal((3, k, m) if ta else (3, m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)  # broadcast over the batch
    ref = (np.swapaxes(a, 1, 2) if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
    np.testing.assert_allclose(oracle.matmul(a, b, ta, tb), ref, rtol=1e-6, atol=1e-6)
    b3 = rng.standard_normal((3, n, k) if tb else (3, k, n)).astype(np.float32)
    ref = (np.swapaxes(a, 1, 2) if ta else a).astype(np.float64) @ (np.swapaxes(b3, 1, 2) if tb else b3).astype(np.float64)
    np.testing.assert_allclose(oracle.matmul(a, b3, ta, tb), ref, rtol=1e-6, atol=1e-6)
    a2 = a[0]
    ref = (a2.T if ta else a2).astype(np.float64) @ (np.swapaxes(b3, 1, 2) if tb else b3).astype(np.float64)
    np.testing.assert_allclose(oracle.matmul(a2, b3, ta, tb), ref, rtol=1e-6, atol=1e-6)


def test_gather_matches_numpy_take_and_zero_rule(oracle):
    rng = np.random.default_rng(4)
    data = rng.integers(0, 2 ** 16, (3, 4, 6, 5)).astype(np.uint16)
    for axis in range(4):
        n = data.shape[axis]
        idx = rng.integers(-n, n, (2, 3))
        assert np.array_equal(oracle.gather(data, idx, axis), np.take(data, idx, axis=axis))
    idx = np.array([0, 6, -7, 5, -6])  # 6 and -7 fall outside an axis of 6
    got = oracle.gather(data, idx, 2)
    assert np.array_equal(got[:, :, [0, 3, 4]], data[:, :, [0, 5, 0]])
    assert not got[:, :, [1, 2]].any()
    # batch_dims = 1: every batch entry has its own indices
    bidx = rng.integers(0, 6, (3, 4))
    got = oracle.gather(data, bidx, 2, batch_dims=1)
    ref = np.stack([np.take(data[b], bidx[b], axis=1) for b in range(3)])
    assert np.array_equal(got, ref)
    assert oracle.gather(data, np.zeros((0,), np.int64), 1).shape == (3, 0, 6, 5)


def test_concat_matches_numpy(oracle):
    rng = np.random.default_rng(5)
    for axis in (0, 1, 2, -1):
        parts = []
        for w in (3, 0, 5, 1):
            shape = [2, 4, 6]
            shape[axis] = w
            parts.append(rng.standard_normal(shape).astype(np.float32))
        assert np.array_equal(oracle.concat(parts, axis), np.concatenate(parts, axis))


def test_swish_and_glu_match_torch_fixtures(oracle, golden):
    x = golden["act/x"]
    np.testing.assert_allclose(oracle.swish(x), golden["act/silu"], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.swish(x, 1.7), golden["act/silu_beta1p7"], rtol=2e-6, atol=1e-7)
    up = np.linspace(-2, 3, x.size).astype(np.float32)
    for act, name in ((0, "silu"), (1, "gelu_erf"), (2, "gelu_tanh")):
        packed = np.stack([np.concatenate([x, up]), np.concatenate([x[::-1], up])])  # [gate | up]
        want = np.stack([golden["act/" + name].astype(np.float64) * up, golden["act/" + name][::-1].astype(np.float64) * up])
        np.testing.assert_allclose(oracle.glu(packed, act, True), want, rtol=3e-6, atol=1e-6)
        swapped = np.stack([np.concatenate([up, x]), np.concatenate([up, x[::-1]])])     # [up | gate]
        np.testing.assert_allclose(oracle.glu(swapped, act, False), want, rtol=3e-6, atol=1e-6)


TRANSPOSE_CASES = [((5,), (0,)), ((3, 4), (1, 0)), ((2, 3, 4), (0, 2, 1)), ((2, 3, 4), (2, 0, 1)), ((2, 5, 3, 8), (0, 2, 1, 3)),
                   ((2, 1, 3, 4), (3, 1, 0, 2)), ((2, 3, 2, 3, 2, 3), (5, 3, 1, 4, 2, 0)), ((4, 1, 6), (1, 0, 2)), ((0, 3), (1, 0))]


@pytest.mark.parametrize("shape,order", TRANSPOSE_CASES)
def test_transpose_matches_numpy(oracle, shape, order):
    rng = np.random.default_rng(3)
    for dt in (np.uint8, np.uint16, np.float32, np.int64):
        x = rng.integers(0, 200, shape).astype(dt)
        out = oracle.transpose(x, order)
        assert out.shape == tuple(shape[o] for o in order)
        np.testing.assert_array_equal(out, np.transpose(x, order))


def convert_with_numpy(x_storage, src, dst):
    """Convert restated with numpy / torch casts; valid for values inside the target's range."""
    import torch
    F32, F16, BF16, BOOL = 0, 1, 2, 104
    if src == F16:
        v = x_storage.view(np.float16).astype(np.float32)
    elif src == BF16:
        v = (x_storage.astype(np.uint32) << 16).view(np.float32)
    elif src == BOOL:
        v = (x_storage != 0).astype(np.int64)
    else:
        v = x_storage
    if dst == BOOL:
        return (v != 0).astype(np.uint8)
    if dst in (F16, BF16):
        v32 = v.astype(np.float32)  # the reference casts through float (kernels/convert.cuh:24-33)
        if dst == F16:
            with np.errstate(over="ignore"):
                return v32.astype(np.float16).view(np.uint16)
        return torch.from_numpy(v32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    target = {F32: np.float32, 100: np.int32, 101: np.int64, 102: np.uint8, 103: np.int8}[dst]
    return v.astype(target)


CONVERT_TYPES = [0, 1, 2, 100, 101, 102, 103, 104]


def convert_samples(rng, src, dst, n=4096):
    """Storage array of type `src` whose values lie inside the range of `dst` (fractions included)."""
    limit = {102: (0, 255), 103: (-128, 127), 104: (0, 1)}.get(dst, (-30000, 30000))
    if src in (0, 1, 2):
        v = rng.uniform(limit[0], limit[1], n).astype(np.float32)
        v[: n // 8] = np.round(v[: n // 8])          # exact integers and ties
        v[n // 8: n // 4] = np.round(v[n // 8: n // 4]) + 0.5 * (limit[1] > 1)
        v = np.clip(v, limit[0], limit[1])
        v[-3:] = [0.0, -0.0, limit[1]]
        if src == 1:
            return v.astype(np.float16).view(np.uint16)
        if src == 2:
            import torch
            return torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        return v
    storage = {100: np.int32, 101: np.int64, 102: np.uint8, 103: np.int8, 104: np.uint8}[src]
    lo, hi = {100: (-2**31, 2**31 - 1), 101: (-2**62, 2**62), 102: (0, 255), 103: (-128, 127), 104: (0, 2)}[src]
    v = rng.integers(lo, hi, n, dtype=np.int64, endpoint=True)
    v[: n // 2] = rng.integers(max(lo, -300), min(hi, 300), n // 2, endpoint=True)  # small values too
    return v.astype(storage)


@pytest.mark.parametrize("src", CONVERT_TYPES)
@pytest.mark.parametrize("dst", CONVERT_TYPES)
def test_convert_matches_numpy_casts(oracle, src, dst):
    rng = np.random.default_rng(100 * src + dst)
    x = convert_samples(rng, src, dst)
    got = oracle.convert(x, src, dst)
    want = convert_with_numpy(x, src, dst)
    assert got.dtype == want.dtype
    np.testing.assert_array_equal(got, want)


def test_convert_rules_c_leaves_open(oracle):
    f = np.array([np.nan, np.inf, -np.inf, 3e9, -3e9, 1e20, -1e20, 300.7, -300.7, 255.9, -0.9, 127.5, -128.9], np.float32)
    np.testing.assert_array_equal(oracle.convert(f, 0, 100), [0, 2**31 - 1, -2**31, 2**31 - 1, -2**31, 2**31 - 1, -2**31, 300, -300, 255, 0, 127, -128])
    np.testing.assert_array_equal(oracle.convert(f, 0, 101), [0, 2**63 - 1, -2**63, 3000000000, -3000000000, 2**63 - 1, -2**63, 300, -300, 255, 0, 127, -128])
    np.testing.assert_array_equal(oracle.convert(f, 0, 102), [0, 255, 0, 255, 0, 255, 0, 255, 0, 255, 0, 127, 0])
    np.testing.assert_array_equal(oracle.convert(f, 0, 103), [0, 127, -128, 127, -128, 127, -128, 127, -128, 127, 0, 127, -128])
    np.testing.assert_array_equal(oracle.convert(f, 0, 104), [1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1])
    np.testing.assert_array_equal(oracle.convert(np.array([0.0, -0.0, 1e-30], np.float32), 0, 104), [0, 0, 1])
    # integers narrow modulo 2^bits, booleans read any non-zero byte as 1
    np.testing.assert_array_equal(oracle.convert(np.array([2**32 + 5, -1, 2**31], np.int64), 101, 100), [5, -1, -2**31])
    np.testing.assert_array_equal(oracle.convert(np.array([256 + 7, -1, 128], np.int32), 100, 102), [7, 255, 128])
    np.testing.assert_array_equal(oracle.convert(np.array([0, 1, 2, 255], np.uint8), 104, 100), [0, 1, 1, 1])
    # 2^24 + 1 is not a float: to nearest even
    np.testing.assert_array_equal(oracle.convert(np.array([2**24 + 1, 2**24 + 3], np.int64), 101, 0), np.array([2**24, 2**24 + 4], np.float32))


BROADCAST_CASES = [((4, 8), (4, 8)), ((2, 3, 4, 5), (1, 1, 4, 5)), ((2, 3, 4, 5), (5,)), ((3, 1, 5), (1, 4, 1)), ((7,), ()), ((), ()),
                   ((2, 1, 6), (2, 3, 1)), ((1, 8), (5, 1)), ((0, 4), (1, 4))]


@pytest.mark.parametrize("a_shape,b_shape", BROADCAST_CASES)
@pytest.mark.parametrize("op", [0, 1, 2, 3])
def test_binary_matches_numpy_broadcasting(oracle, a_shape, b_shape, op):
    rng = np.random.default_rng(len(a_shape) * 10 + op)
    a = rng.standard_normal(a_shape).astype(np.float32)
    b = (rng.standard_normal(b_shape) + 3.0).astype(np.float32)
    want = [np.add, np.subtract, np.multiply, np.divide][op](a, b)
    got = oracle.binary(op, a, b)
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    got = oracle.binary(op, b, a + 5.0)  # operands the other way round
    np.testing.assert_array_equal(got, [np.add, np.subtract, np.multiply, np.divide][op](b, a + 5.0))


def test_binary_refuses_shapes_that_do_not_broadcast(oracle):
    with pytest.raises(ValueError):
        oracle.binary(0, np.zeros((2, 3), np.float32), np.zeros((2, 4), np.float32))


@pytest.mark.parametrize("shape,axis", [((5, 9), 1), ((5, 9), 0), ((2, 3, 4, 5), 2), ((2, 3, 4, 5), -1), ((3, 1000), 1), ((7,), 0)])
def test_softmax_matches_scipy_and_torch(oracle, shape, axis):
    import scipy.special
    import torch
    rng = np.random.default_rng(sum(shape) + axis)
    x = (rng.standard_normal(shape) * 6).astype(np.float32)
    got = oracle.softmax(x, axis)
    np.testing.assert_allclose(got, scipy.special.softmax(x.astype(np.float64), axis=axis), rtol=2e-7, atol=1e-12)
    np.testing.assert_allclose(got, torch.softmax(torch.from_numpy(x).double(), axis).numpy(), rtol=2e-7, atol=1e-12)
    np.testing.assert_allclose(got.astype(np.float64).sum(axis), 1.0, rtol=1e-6)
    np.testing.assert_allclose(oracle.softmax(x + 100.0, axis), got, rtol=2e-5, atol=1e-9)  # shift invariance (x + 100 rounds)
    np.testing.assert_allclose(oracle.softmax(np.full(shape, -3.5, np.float32), axis), 1.0 / shape[axis], rtol=1e-7)


def test_softmax_with_masked_entries(oracle):
    x = np.array([[0.0, -np.inf, 1.0, -np.inf], [-np.inf, -np.inf, -np.inf, 2.0]], np.float32)
    got = oracle.softmax(x, 1)
    e = np.exp(1.0)
    np.testing.assert_allclose(got, [[1 / (1 + e), 0, e / (1 + e), 0], [0, 0, 0, 1]], rtol=1e-7)
    assert np.isnan(oracle.softmax(np.full((1, 4), -np.inf, np.float32), 1)).all()
