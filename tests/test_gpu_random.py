"""Randomly drawn paged-attention batches against the oracle (gpu).

The hand-picked cases of test_gpu_parity.py sit on the boundaries that were thought of; these do
not: head counts (GQA ratios 1..16, kv head counts that are not multiples of four), cache and query
types, sliding windows, and batches that are all decode, all prefill or mixed, with sequence
lengths on and off the block and tile boundaries.  Seeds are fixed, so a failure names its case.

Bounds: cache bytes bit-exact; outputs within 2e-3 (fp16 operands) or 1e-2 (bf16 queries, u8
caches) of the oracle's fp32 result, relative to max(1, |value|) because N(0, 1) values give
outputs beyond 1 where the 16-bit output type alone rounds by more.  bf16 caches are held to 2e-2:
their probabilities enter the second product as bf16 (8 significant bits), and with N(0, 1) values
single elements of a few million reach 1.2e-2 (the 99.99th percentile is 3e-3).
"""
import numpy as np
import pytest

import helpers as H
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu


def draw_batch(rng):
    G = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
    Hkv = int(rng.choice([1, 2, 3, 4, 8]))
    cache = int(rng.choice([W.F16, W.BF16, W.U8]))
    q_dtype = int(rng.choice([W.F16, W.BF16]))
    window = int(rng.choice([0, 0, 1, 17, 64, 300, 1000]))
    kind = str(rng.choice(["decode", "mixed", "prefill"]))
    seqs = []
    for _ in range(int(rng.integers(1, 40))):
        past = int(rng.choice([0, 1, 31, 32, 33, 100, 500, 1500, int(rng.integers(0, 3000))]))
        if kind == "decode":
            q_len = 1
        elif kind == "prefill":
            q_len = int(rng.choice([2, 5, 64, 127, 128, 129, 300]))
        else:
            q_len = int(rng.choice([1, 1, 1, 0, 2, 64, 130, 257]))
        seqs.append((past, q_len))
    return kind, G * Hkv, Hkv, cache, q_dtype, window, seqs


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_paged_batches(hip, oracle, seed):
    rng = np.random.default_rng(seed)
    worst = 0.0
    for it in range(16):
        kind, Hq, Hkv, cache, q_dtype, window, seqs = draw_batch(rng)
        if sum(n for _, n in seqs) == 0:
            continue
        # the interface takes a batch with as many tokens as sequences to be one token per sequence
        # (the host cannot see the lengths); a draw like (2 tokens, 0 tokens) is outside that contract
        if sum(n for _, n in seqs) == len(seqs) and any(n != 1 for _, n in seqs):
            continue
        print("[case] random paged", seed, it, kind, "Hq", Hq, "Hkv", Hkv, "cache", cache, "q", q_dtype, "window", window,
              "seqs", seqs, flush=True)
        case = W.make_paged_case(seed * 100 + it, seqs, Hq, Hkv, 128, 32, q_dtype, q_dtype, cache, sliding_window=window)
        ref, okc, ovc = H.oracle_paged(oracle, case)
        dev = H.PagedDeviceCase(hip, case)
        out, path = dev.run()
        kc, vc = dev.caches()
        dev.free()
        assert path == "paged_mfma"
        np.testing.assert_array_equal(kc, okc)
        np.testing.assert_array_equal(vc, ovc)
        assert np.isfinite(out).all()
        tol = 2e-2 if cache == W.BF16 else (1e-2 if (cache == W.U8 or q_dtype == W.BF16) else 2e-3)
        err = H.scaled_bound_error(out, ref, "random paged %d/%d q %d cache %d" % (seed, it, q_dtype, cache))
        worst = max(worst, err / tol)
        assert err <= tol, (seed, it)
    print("worst error / bound: %.2f" % worst)


@pytest.mark.parametrize("seed", [31, 32, 33])
def test_random_paged_batches_of_every_shape(hip, oracle, seed):
    """The same draws over the shapes the matrix-core paths take besides head size 128 / blocks of 32:
    head sizes that are multiples of 8 up to 256, block sizes that are powers of two, up to 128 query
    heads per kv head, 16-bit and u8 caches.  Which kernel takes a call follows from the shape
    (the stream-K kernels on blocks of 16 tokens or more with at most 16 query heads per kv head; the query-tile
    kernel for the rest)."""
    rng = np.random.default_rng(seed)
    worst = 0.0
    for it in range(40):
        kind, _, _, cache, q_dtype, window, seqs = draw_batch(rng)
        seqs = [(min(past, 800), n) for past, n in seqs][:8]
        D = 8 * int(rng.integers(1, 33))
        if rng.random() < 0.3:
            D = int(rng.choice([64, 96, 128, 256]))
        bs = int(rng.choice([4, 8, 16, 16, 32, 32, 64, 128, 256]))
        Hkv = int(rng.choice([1, 2, 3]))
        G = int(rng.choice([1, 2, 4, 7, 8, 16, 17, 40]))
        if G * Hkv * D > 8192:
            G = max(1, 8192 // (Hkv * D))
        if sum(n for _, n in seqs) == 0:
            continue
        if sum(n for _, n in seqs) == len(seqs) and any(n != 1 for _, n in seqs):
            continue
        print("[case] random paged shapes", seed, it, kind, "D", D, "bs", bs, "G", G, "Hkv", Hkv, "cache", cache, "q", q_dtype,
              "window", window, "seqs", seqs, flush=True)
        case = W.make_paged_case(seed * 100 + it, seqs, G * Hkv, Hkv, D, bs, q_dtype, q_dtype, cache, sliding_window=window)
        ref, okc, ovc = H.oracle_paged(oracle, case)
        dev = H.PagedDeviceCase(hip, case)
        out, path = dev.run()
        kc, vc = dev.caches()
        dev.free()
        assert path == H.paged_matrix_core_path(G * Hkv, Hkv, D, bs, cache)
        np.testing.assert_array_equal(kc, okc)
        np.testing.assert_array_equal(vc, ovc)
        assert np.isfinite(out).all()
        tol = 2e-2 if cache == W.BF16 else (1e-2 if (cache == W.U8 or q_dtype == W.BF16) else 2e-3)
        err = H.scaled_bound_error(out, ref, "random paged shapes %d/%d q %d cache %d" % (seed, it, q_dtype, cache))
        worst = max(worst, err / tol)
        assert err <= tol, (seed, it)
    print("worst error / bound: %.2f" % worst)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_sdpa_shapes(hip, oracle, seed):
    """Dense SDPA: batch, GQA ratio, head size (16-bit types take the matrix-core kernels at every
    multiple of 8 up to 256, fp32 the shape-generic one), square and rectangular score matrices,
    causal or not."""
    rng = np.random.default_rng(seed)
    worst = {}
    for it in range(24):
        G = int(rng.choice([1, 2, 3, 4, 5, 8]))
        Hkv = int(rng.choice([1, 2, 3]))
        B = int(rng.choice([1, 2, 3]))
        D = int(rng.choice([128, 128, 128, 64, 32, 96, 256, 8 * int(rng.integers(1, 33))]))
        dtype = int(rng.choice([W.F16, W.BF16, W.F32]))
        Lq = int(rng.choice([1, 2, 31, 64, 127, 128, 129, 255, 256, 257, 300, 511, 700, int(rng.integers(1, 900))]))
        Lk = Lq if rng.random() < 0.5 else int(rng.choice([1, 63, 64, 65, 200, 513, 1000, int(rng.integers(1, 1200))]))
        causal = bool(rng.random() < 0.6)
        print("[case] random sdpa", seed, it, "B", B, "Hq", G * Hkv, "Hkv", Hkv, "Lq", Lq, "Lk", Lk, "D", D, "dtype", dtype,
              "causal", causal, flush=True)
        case = W.make_sdpa_case(seed * 100 + it, B, G * Hkv, Hkv, Lq, Lk, D, dtype, std=0.5 if dtype == W.BF16 else 1.0)
        out, path = H.run_sdpa(hip, case, causal)
        ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=causal)
        rows = np.isfinite(ref)  # a row that attends to no key at all is unspecified in the oracle as well
        tol = {W.F32: 1e-4, W.F16: 2e-3, W.BF16: 1e-2}[dtype]
        e = H.scaled_bound_error(out, ref, "random sdpa %d/%d dtype %d %s" % (seed, it, dtype, path))
        worst[path] = max(worst.get(path, 0.0), e / tol)
        assert e <= tol, (seed, it, path)
    print("worst error / bound by kernel path:", worst)
