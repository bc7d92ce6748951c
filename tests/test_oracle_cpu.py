"""Pins the CPU oracle (oracle/hipattn_oracle.c) without any GPU.

Checks are chosen so that a plausible mistake fails one of them: a wrong mask offset fails the
torch fixtures and the first-row identity, a transposed GQA mapping fails the repeated-KV
identity, a wrong block/row index in the scatter fails the brute-force map, a wrong window
bound fails the explicit-mask comparison, a wrong rounding fails the bit comparisons.
"""
import os

import numpy as np
import pytest

from openvino_contrib_amd import workloads as W

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sdpa_golden.npz")


def brute_sdpa_f64(q, k, v, causal, scale=None, mask=None):
    """Closed form softmax(scale q k^T + mask) v in fp64 with explicit Python loops over heads."""
    q, k, v = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    B, Hq, Lq, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    out = np.zeros_like(q)
    for b in range(B):
        for h in range(Hq):
            s = scale * q[b, h] @ k[b, h // G].T
            if causal:
                i = np.arange(Lq)[:, None]
                j = np.arange(Lk)[None, :]
                s = np.where(j <= i, s, -np.inf)
            if mask is not None:
                s = np.where(mask, s, -np.inf)
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[b, h] = p @ v[b, h // G]
    return out


# ------------------------------------------------------------------------------------ SDPA
@pytest.mark.parametrize("name", ["ref_small", "ref_medium", "ref_llm", "ref_3d", "gqa", "rect", "long_row"])
@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_matches_torch_fixture(oracle, name, causal):
    z = np.load(GOLDEN)
    out = oracle.sdpa(z[name + "/q"], z[name + "/k"], z[name + "/v"], causal=causal)
    np.testing.assert_allclose(out, z["%s/out_causal%d" % (name, int(causal))], atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("shape", [(1, 2, 2, 5, 9, 8), (2, 6, 3, 12, 12, 16), (1, 4, 1, 9, 4, 32)])
@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_matches_fp64_brute_force(oracle, shape, causal):
    B, Hq, Hkv, Lq, Lk, D = shape
    c = W.make_sdpa_case(7, B, Hq, Hkv, Lq, Lk, D, W.F32)
    out = oracle.sdpa(c["q"], c["k"], c["v"], causal=causal, scale=0.37)
    ref = brute_sdpa_f64(c["q"], c["k"], c["v"], causal, scale=0.37)
    np.testing.assert_allclose(out, ref, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("name", ["float_full", "float_2d", "float_per_batch", "bool_full", "bool_keys"])
def test_sdpa_mask_matches_torch_fixture(oracle, name):
    """attention_mask input: float masks are added to the scaled scores, boolean masks select keys;
    fixtures from torch's CPU routine with attn_mask, broadcast shapes included."""
    z = np.load(GOLDEN)
    p = "mask_" + name
    out = oracle.sdpa_masked(z[p + "/q"], z[p + "/k"], z[p + "/v"], z[p + "/mask"])
    np.testing.assert_allclose(out, z[p + "/out"], atol=2e-6, rtol=1e-5)


def test_sdpa_mask_reductions(oracle):
    c = W.make_sdpa_case(12, 2, 4, 2, 11, 11, 16, W.F32)
    q, k, v = c["q"], c["k"], c["v"]
    tril = np.tril(np.ones((11, 11), bool))
    # an explicit lower-triangular boolean mask is the causal flag
    np.testing.assert_allclose(oracle.sdpa_masked(q, k, v, tril), oracle.sdpa(q, k, v, causal=True), atol=1e-6)
    # ... and so is its additive form; a mask of zeros changes nothing; with causal set the mask is ignored
    add = np.where(tril, 0.0, -np.inf).astype(np.float32)
    np.testing.assert_array_equal(oracle.sdpa_masked(q, k, v, add), oracle.sdpa_masked(q, k, v, tril))
    np.testing.assert_array_equal(oracle.sdpa_masked(q, k, v, np.zeros((1, 1, 1, 11), np.float32)), oracle.sdpa(q, k, v))
    np.testing.assert_array_equal(oracle.sdpa_masked(q, k, v, np.full((11, 11), -3.0, np.float32), causal=True),
                                  oracle.sdpa(q, k, v, causal=True))
    # a per-row constant shifts every score of the row: no change (softmax shift invariance)
    rowc = np.arange(11, dtype=np.float32)[:, None] * np.ones((1, 11), np.float32)
    np.testing.assert_allclose(oracle.sdpa_masked(q, k, v, rowc), oracle.sdpa(q, k, v), atol=1e-5)
    # fp64 brute force with a random boolean mask over batch and heads
    rng = np.random.default_rng(5)
    m = rng.random((2, 4, 11, 11)) < 0.5
    m[..., 3] = True
    ref = np.stack([np.stack([brute_sdpa_f64(q[b:b + 1, h:h + 1], k[b:b + 1, h // 2:h // 2 + 1], v[b:b + 1, h // 2:h // 2 + 1],
                                             False, mask=m[b, h])[0, 0] for h in range(4)]) for b in range(2)])
    np.testing.assert_allclose(oracle.sdpa_masked(q, k, v, m), ref, atol=2e-6, rtol=1e-5)


def test_sdpa_invariants(oracle):
    c = W.make_sdpa_case(11, 2, 4, 2, 10, 10, 16, W.F32)
    q, k, v = c["q"], c["k"], c["v"]
    out = oracle.sdpa(q, k, v, causal=True)
    # causal row 0 sees only key 0
    G = 2
    for h in range(4):
        np.testing.assert_allclose(out[:, h, 0], v[:, h // G, 0], atol=1e-6)
    # GQA == MHA with K/V repeated along heads
    out_mha = oracle.sdpa(q, np.repeat(k, G, axis=1), np.repeat(v, G, axis=1), causal=True)
    np.testing.assert_array_equal(out, out_mha)
    # uniform V gives V back; adding a constant to every score of a row changes nothing
    vu = np.broadcast_to(v[:, :, :1], v.shape).copy()
    np.testing.assert_allclose(oracle.sdpa(q, k, vu, causal=False), np.repeat(vu[:, :, :1], G, axis=1).repeat(10, 2),
                               atol=1e-6)
    # batch permutation equivariance
    np.testing.assert_array_equal(oracle.sdpa(q[::-1], k[::-1], v[::-1], causal=True), out[::-1])
    # default scale is 1/sqrt(D)
    np.testing.assert_array_equal(oracle.sdpa(q, k, v, causal=True, scale=0.0),
                                  oracle.sdpa(q, k, v, causal=True, scale=np.float32(1 / np.sqrt(np.float32(16)))))


def test_sdpa_empty_and_bad_args(oracle):
    q = np.zeros((1, 2, 0, 8), np.float32)
    k = np.zeros((1, 2, 5, 8), np.float32)
    assert oracle.sdpa(q, k, k).shape == (1, 2, 0, 8)
    q = np.ones((1, 2, 3, 8), np.float32)
    k = np.zeros((1, 2, 0, 8), np.float32)
    assert np.all(oracle.sdpa(q, k, k) == 0)  # nothing to attend: zeros, not NaN
    with pytest.raises(ValueError):
        oracle.sdpa(np.ones((1, 3, 2, 8), np.float32), np.ones((1, 2, 2, 8), np.float32),
                    np.ones((1, 2, 2, 8), np.float32))


# ------------------------------------------------------------------------------ conversions
def test_f16_bf16_conversions_bit_exact(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32),
        (rng.standard_normal(4096) * 1e-6).astype(np.float32),   # fp16 subnormal range
        (rng.standard_normal(1024) * 3e4).astype(np.float32),    # near fp16 overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -26,
                  np.inf, -np.inf], np.float32),
    ])
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    finite = (h & 0x7C00) != 0x7C00
    np.testing.assert_array_equal(oracle.f16_bits_to_f32(h)[finite], h.view(np.float16).astype(np.float32)[finite])
    # every finite half survives the round trip
    np.testing.assert_array_equal(oracle.f32_to_f16_bits(oracle.f16_bits_to_f32(h[finite])), h[finite])
    import torch
    tb = torch.from_numpy(x[:-2]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_bf16_bits(x[:-2]), tb)
    np.testing.assert_array_equal(W.f32_to_bf16_bits(x[:-2]), tb)
    np.testing.assert_array_equal(W.f32_to_f16_bits(x[:9000]), oracle.f32_to_f16_bits(x[:9000]))


# ---------------------------------------------------------------------------- u8 rows
def test_u8_quant_invariants(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((500, 128)).astype(np.float32)
    x[7] = 1.25       # constant row
    x[8, :] = 0.0
    rows = oracle.quant_u8_rows(x)
    scale = rows[:, 0:4].copy().view(np.float32)[:, 0]
    zp = rows[:, 4:8].copy().view(np.float32)[:, 0]
    q = rows[:, 8:]
    xh = oracle.dequant_u8_rows(rows)
    # layout and formula, restated independently in fp64
    np.testing.assert_allclose(scale[:7], (x[:7].max(1).astype(np.float64) - x[:7].min(1)) / 255.0, rtol=1e-6)
    assert scale[7] == np.float32(0.0001) and scale[8] == np.float32(0.0001)
    np.testing.assert_allclose(zp, -x.min(1).astype(np.float64) / scale, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(xh, (q.astype(np.float64) - zp[:, None]) * scale[:, None], rtol=1e-6, atol=1e-7)
    # error bound and extreme values
    assert np.all(np.abs(xh - x) <= scale[:, None] * 0.5 * (1 + 1e-4) + 1e-6)
    rowsel = np.arange(500) != 7
    assert np.all(q[rowsel & (np.arange(500) != 8)].min(1) == 0)
    assert np.all(q[rowsel & (np.arange(500) != 8)].max(1) == 255)
    # the workload generator's numpy quantiser agrees (bytes within one step, scale/zp exactly)
    rows_np = W.quantize_u8_rows(x)
    np.testing.assert_array_equal(rows_np[:, :8], rows[:, :8])
    assert np.abs(rows_np[:, 8:].astype(np.int32) - q.astype(np.int32)).max() <= 1
    assert (rows_np[:, 8:] != q).mean() < 1e-3


# -------------------------------------------------------------------------- KV scatter
def _brute_scatter(case, cache_dtype):
    """Independent restatement of the slot map in plain Python."""
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    D, Hkv, bs = case["D"], case["Hkv"], case["block_size"]
    for s in range(case["S"]):
        t0, t1 = case["subsequence_begins"][s], case["subsequence_begins"][s + 1]
        for t in range(t0, t1):
            p = case["past_lens"][s] + (t - t0)
            blk = case["block_indices"][case["block_indices_begins"][s] + p // bs]
            for h in range(Hkv):
                kc[blk, h, p % bs] = W.cache_rows_from_f32(case["k_new"][t, h * D:(h + 1) * D][None], cache_dtype)[0]
                vc[blk, h, p % bs] = W.cache_rows_from_f32(case["v_new"][t, h * D:(h + 1) * D][None], cache_dtype)[0]
    return kc, vc


@pytest.mark.parametrize("cache_dtype", [W.F16, W.BF16, W.F32])
def test_kv_write_matches_brute_force(oracle, cache_dtype):
    case = W.make_paged_case(21, [(0, 5), (31, 1), (32, 1), (40, 30), (7, 0), (63, 2)], 4, 2, 16, 32, W.F16, W.F16,
                             cache_dtype)
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    skipped = oracle.kv_cache_write(case["k_new"], case["v_new"], kc, vc, cache_dtype, case["past_lens"],
                                    case["subsequence_begins"], case["block_indices"], case["block_indices_begins"],
                                    2, 16, 32)
    assert skipped == 0
    bk, bv = _brute_scatter(case, cache_dtype)
    np.testing.assert_array_equal(kc, bk)
    np.testing.assert_array_equal(vc, bv)
    # exactly T * Hkv rows changed in each cache (values are random, so a rewritten row differs)
    changed = (kc != case["key_cache"]).any(axis=-1).sum()
    assert changed == case["T"] * 2


def test_kv_write_then_gather_is_identity_and_skips_bad_blocks(oracle):
    case = W.make_paged_case(22, [(3, 40), (0, 33)], 2, 2, 8, 16, W.F32, W.F32, W.F32)
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    oracle.kv_cache_write(case["k_new"], case["v_new"], kc, vc, W.F32, case["past_lens"], case["subsequence_begins"],
                          case["block_indices"], case["block_indices_begins"], 2, 8, 16)
    for s, (past, n) in enumerate([(3, 40), (0, 33)]):
        blocks = case["block_indices"][case["block_indices_begins"][s]:case["block_indices_begins"][s + 1]]
        for h in range(2):
            rows = oracle.gather_cache_rows(kc, W.F32, blocks, past + n, h, 2, 8, 16)
            t0 = case["subsequence_begins"][s]
            np.testing.assert_array_equal(rows[past:], case["k_new"][t0:t0 + n, h * 8:(h + 1) * 8])
    # out-of-range physical ids and positions past the table are skipped, nothing is written
    # (expectation of modules/nvidia_plugin/tests/unit/kernels/scatter_update.cpp:59-86)
    bad = case["block_indices"].copy()
    bad[0] = case["num_blocks"] + 5
    bad[1] = -1
    kc2, vc2 = case["key_cache"].copy(), case["value_cache"].copy()
    skipped = oracle.kv_cache_write(case["k_new"], case["v_new"], kc2, vc2, W.F32, case["past_lens"],
                                    case["subsequence_begins"], bad, case["block_indices_begins"], 2, 8, 16)
    assert skipped == (16 - 3) + 16  # positions 3..15 -> block 0, 16..31 -> block 1
    short = case["block_indices_begins"].copy()
    short[1] -= 1  # hide sequence 0's last block
    short_idx = np.concatenate([case["block_indices"][:2], case["block_indices"][3:]])
    short[2] -= 1
    kc3, vc3 = case["key_cache"].copy(), case["value_cache"].copy()
    skipped = oracle.kv_cache_write(case["k_new"], case["v_new"], kc3, vc3, W.F32, case["past_lens"],
                                    case["subsequence_begins"], short_idx, short, 2, 8, 16)
    assert skipped == (3 + 40) - 32


# ---------------------------------------------------------------------- paged attention
def _dense_reference(oracle, case, s, scale=None):
    """Paged attention of sequence s via gather + dense SDPA with an explicit brute-force mask."""
    D, Hq, Hkv, bs, Wn = case["D"], case["Hq"], case["Hkv"], case["block_size"], case["sliding_window"]
    past = int(case["past_lens"][s])
    t0, t1 = int(case["subsequence_begins"][s]), int(case["subsequence_begins"][s + 1])
    n = t1 - t0
    ctx = past + n
    blocks = case["block_indices"][case["block_indices_begins"][s]:case["block_indices_begins"][s + 1]]
    k = np.stack([oracle.gather_cache_rows(case["kc_after"], case["cache_dtype"], blocks, ctx, h, Hkv, D, bs)
                  for h in range(Hkv)])[None]
    v = np.stack([oracle.gather_cache_rows(case["vc_after"], case["cache_dtype"], blocks, ctx, h, Hkv, D, bs)
                  for h in range(Hkv)])[None]
    q = case["q"][t0:t1].reshape(n, Hq, D).transpose(1, 0, 2)[None]
    i = past + np.arange(n)[:, None]
    j = np.arange(ctx)[None, :]
    mask = j <= i
    if Wn > 0:
        mask &= j > i - Wn
    out = brute_sdpa_f64(q, k, v, causal=False, scale=scale, mask=mask)
    return out[0].transpose(1, 0, 2).reshape(n, Hq * D)


@pytest.mark.parametrize("cache_dtype,window", [(W.F16, 0), (W.F32, 0), (W.U8, 0), (W.F16, 24), (W.BF16, 7)])
def test_paged_attention_reduces_to_dense(oracle, cache_dtype, window):
    seqs = [(0, 9), (37, 1), (31, 2), (5, 40), (64, 1)]
    case = W.make_paged_case(31, seqs, 4, 2, 16, 16, W.F32, W.F32, cache_dtype, sliding_window=window)
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    out = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, cache_dtype, case["past_lens"],
                                 case["subsequence_begins"], case["block_indices"], case["block_indices_begins"],
                                 4, 2, 16, 16, sliding_window=window)
    case["kc_after"], case["vc_after"] = kc, vc
    for s in range(len(seqs)):
        t0, t1 = case["subsequence_begins"][s], case["subsequence_begins"][s + 1]
        np.testing.assert_allclose(out[t0:t1], _dense_reference(oracle, case, s), atol=3e-6, rtol=1e-5)
    # the op's own write equals the stand-alone writer
    kc2, vc2 = case["key_cache"].copy(), case["value_cache"].copy()
    oracle.kv_cache_write(case["k_new"], case["v_new"], kc2, vc2, cache_dtype, case["past_lens"],
                          case["subsequence_begins"], case["block_indices"], case["block_indices_begins"], 2, 16, 16)
    np.testing.assert_array_equal(kc, kc2)
    np.testing.assert_array_equal(vc, vc2)


def test_paged_attention_block_permutation_invariance_and_window(oracle):
    seqs = [(20, 12), (50, 1), (0, 3)]
    case = W.make_paged_case(32, seqs, 4, 2, 16, 8, W.F32, W.F32, W.F16)
    args = lambda c, kc, vc, w: (c["q"], c["k_new"], c["v_new"], kc, vc, W.F16, c["past_lens"],
                                 c["subsequence_begins"], c["block_indices"], c["block_indices_begins"], 4, 2, 16, 8)
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    out = oracle.paged_attention(*args(case, kc, vc, 0))
    # move every physical block to a new place and permute the table accordingly: bit-identical
    rng = np.random.default_rng(1)
    perm = rng.permutation(case["num_blocks"])
    case2 = dict(case)
    case2["block_indices"] = perm[case["block_indices"]].astype(np.int32)
    kc2 = np.empty_like(case["key_cache"])
    vc2 = np.empty_like(case["value_cache"])
    kc2[perm] = case["key_cache"]
    vc2[perm] = case["value_cache"]
    out2 = oracle.paged_attention(*args(case2, kc2, vc2, 0))
    np.testing.assert_array_equal(out, out2)
    # a window at least as long as every context changes nothing; a short one does
    kc3, vc3 = case["key_cache"].copy(), case["value_cache"].copy()
    out3 = oracle.paged_attention(*args(case, kc3, vc3, 0), sliding_window=51)
    np.testing.assert_array_equal(out, out3)
    kc4, vc4 = case["key_cache"].copy(), case["value_cache"].copy()
    out4 = oracle.paged_attention(*args(case, kc4, vc4, 0), sliding_window=4)
    assert np.abs(out4 - out).max() > 1e-3
    # chunked prefill: sequence 0 fed as 5 + 7 tokens gives the same rows as 12 at once
    caseA = W.make_paged_case(33, [(20, 12)], 4, 2, 16, 8, W.F32, W.F32, W.F32)
    kcA, vcA = caseA["key_cache"].copy(), caseA["value_cache"].copy()
    full = oracle.paged_attention(*args(caseA, kcA, vcA, 0)[:5], W.F32, *args(caseA, kcA, vcA, 0)[6:])
    kcB, vcB = caseA["key_cache"].copy(), caseA["value_cache"].copy()
    parts = []
    for past, lo, hi in ((20, 0, 5), (25, 5, 12)):
        parts.append(oracle.paged_attention(caseA["q"][lo:hi], caseA["k_new"][lo:hi], caseA["v_new"][lo:hi], kcB, vcB,
                                            W.F32, np.array([past], np.int32), np.array([0, hi - lo], np.int32),
                                            caseA["block_indices"], caseA["block_indices_begins"], 4, 2, 16, 8))
    np.testing.assert_allclose(np.concatenate(parts), full, atol=1e-6)
    np.testing.assert_array_equal(kcA, kcB)


@pytest.mark.parametrize("cache_dtype,window", [(W.F16, 0), (W.U8, 0), (W.F32, 11)])
def test_paged_attention_takes_no_key_from_a_block_outside_the_pool(oracle, cache_dtype, window):
    """A table entry outside [0, num_blocks) names no block: its positions get probability zero.  Pinned by an
    independent reduction: the rows of the valid blocks, gathered densely from a table whose bad entries are
    pointed at a real block, through the fp64 closed form with the bad positions masked by hand; a row with
    nothing left to attend is zeros; a table without bad entries gives what it gave before the rule existed."""
    bs, Hq, Hkv, D = 8, 4, 2, 16
    seqs = [(20, 12), (50, 1), (0, 3), (9, 1), (16, 2)]
    case = W.make_paged_case(34, seqs, Hq, Hkv, D, bs, W.F32, W.F32, cache_dtype, sliding_window=window)
    nb = case["num_blocks"]
    ids, begins = case["block_indices"].copy(), case["block_indices_begins"]
    good = ids.copy()
    bad_at = [begins[0] + 1, begins[0] + 3, begins[1] + 0, begins[1] + 6, begins[2] + 0, begins[4] + 2]
    for n, at in enumerate(bad_at):
        ids[at] = [nb, -1, nb + 7, -(1 << 30), 1 << 30, nb][n]
    for lb in range(begins[3], begins[4]):  # every block of sequence 3
        ids[lb] = -5
    # the cache as the step leaves it, from the table without holes (the holes' tokens are simply not stored)
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    oracle.kv_cache_write(case["k_new"], case["v_new"], kc, vc, cache_dtype, case["past_lens"], case["subsequence_begins"],
                          good, begins, Hkv, D, bs)
    out = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc.copy(), vc.copy(), cache_dtype, case["past_lens"],
                                 case["subsequence_begins"], ids, begins, Hq, Hkv, D, bs, sliding_window=window, do_write=False)
    assert np.isfinite(out).all()
    scale = 1.0 / np.sqrt(D)
    for s, (past, n) in enumerate(seqs):
        t0 = case["subsequence_begins"][s]
        ctx = past + n
        table_bad = (ids[begins[s]:begins[s + 1]] < 0) | (ids[begins[s]:begins[s + 1]] >= nb)
        key_bad = np.repeat(table_bad, bs)[:ctx]
        k = np.stack([oracle.gather_cache_rows(kc, cache_dtype, good[begins[s]:begins[s + 1]], ctx, h, Hkv, D, bs) for h in range(Hkv)])
        v = np.stack([oracle.gather_cache_rows(vc, cache_dtype, good[begins[s]:begins[s + 1]], ctx, h, Hkv, D, bs) for h in range(Hkv)])
        for i in range(n):
            pos = past + i
            j = np.arange(ctx)
            keep = (j <= pos) & ~key_bad
            if window > 0:
                keep &= j > pos - window
            for h in range(Hq):
                got = out[t0 + i, h * D:(h + 1) * D]
                if not keep.any():
                    assert not got.any()
                    continue
                sc = scale * (k[h // (Hq // Hkv)][keep].astype(np.float64) @ case["q"][t0 + i, h * D:(h + 1) * D].astype(np.float64))
                pr = np.exp(sc - sc.max())
                ref = (pr / pr.sum()) @ v[h // (Hq // Hkv)][keep].astype(np.float64)
                np.testing.assert_allclose(got, ref, atol=3e-6, rtol=1e-5)
    assert not out[case["subsequence_begins"][3]].any()  # sequence 3 has no block at all
    # without holes nothing changed: the same call on the good table equals the dense reduction used above
    whole = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc.copy(), vc.copy(), cache_dtype, case["past_lens"],
                                   case["subsequence_begins"], good, begins, Hq, Hkv, D, bs, sliding_window=window, do_write=False)
    case["kc_after"], case["vc_after"] = kc, vc
    for s in range(len(seqs)):
        t0, t1 = case["subsequence_begins"][s], case["subsequence_begins"][s + 1]
        np.testing.assert_allclose(whole[t0:t1], _dense_reference(oracle, case, s), atol=3e-6, rtol=1e-5)


ALIBI_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "alibi_golden.npz")


@pytest.mark.parametrize("name", ["decode", "chunk", "prefill", "window"])
@pytest.mark.parametrize("block_size", [4, 16])
def test_paged_attention_alibi_matches_torch_fixture(oracle, name, block_size):
    """alibi_slopes: slope[h] * (j - p) added to the scaled scores.  The fixture is torch's fp64
    scaled_dot_product_attention with that bias as an explicit mask on dense K/V; here the same K/V rows sit in
    a paged f32 cache behind a shuffled block table (the new tokens come in through the operator's own write)."""
    z = np.load(ALIBI_GOLDEN)
    Hq, Hkv, D, past, n, window = (int(x) for x in z[name + "/meta"])
    q, k, v, slopes = z[name + "/q"][0], z[name + "/k"][0], z[name + "/v"][0], z[name + "/slopes"]
    ctx = past + n
    nblk = (ctx + block_size - 1) // block_size
    rng = np.random.default_rng(5)
    table = rng.permutation(nblk + 3)[:nblk].astype(np.int32)
    kc = np.zeros((nblk + 3, Hkv, block_size, D), np.float32)
    vc = np.zeros_like(kc)
    for j in range(past):  # the cached tokens; the new ones are written by the call
        kc[table[j // block_size], :, j % block_size] = k[:, j]
        vc[table[j // block_size], :, j % block_size] = v[:, j]
    kc8, vc8 = kc.view(np.uint8).reshape(nblk + 3, Hkv, block_size, D * 4), vc.view(np.uint8).reshape(nblk + 3, Hkv, block_size, D * 4)
    k_new = k[:, past:].transpose(1, 0, 2).reshape(n, Hkv * D)
    v_new = v[:, past:].transpose(1, 0, 2).reshape(n, Hkv * D)
    out = oracle.paged_attention(q.transpose(1, 0, 2).reshape(n, Hq * D), k_new, v_new, kc8, vc8, W.F32,
                                 np.array([past], np.int32), np.array([0, n], np.int32), table, np.array([0, nblk], np.int32),
                                 Hq, Hkv, D, block_size, sliding_window=window, alibi_slopes=slopes)
    ref = z[name + "/out"][0].transpose(1, 0, 2).reshape(n, Hq * D)
    np.testing.assert_allclose(out, ref, atol=3e-6, rtol=1e-5)
    # the bias matters (the fixture is not met without it), and slopes of zero are no bias
    kc8b, vc8b = kc8.copy(), vc8.copy()
    plain = oracle.paged_attention(q.transpose(1, 0, 2).reshape(n, Hq * D), k_new, v_new, kc8b, vc8b, W.F32,
                                   np.array([past], np.int32), np.array([0, n], np.int32), table, np.array([0, nblk], np.int32),
                                   Hq, Hkv, D, block_size, sliding_window=window)
    if ctx > 2:
        assert np.abs(plain - ref).max() > 1e-3
    zero = oracle.paged_attention(q.transpose(1, 0, 2).reshape(n, Hq * D), k_new, v_new, kc8b, vc8b, W.F32,
                                  np.array([past], np.int32), np.array([0, n], np.int32), table, np.array([0, nblk], np.int32),
                                  Hq, Hkv, D, block_size, sliding_window=window, alibi_slopes=np.zeros(Hq, np.float32), do_write=False)
    np.testing.assert_array_equal(zero, plain)


# ---- the operator's second output ("scores") ----------------------------------------------------
def _dense_keys(oracle, case, s, h):
    pl, bb = case["past_lens"], case["block_indices_begins"]
    qlen = case["subsequence_begins"][s + 1] - case["subsequence_begins"][s]
    return oracle.gather_cache_rows(case["key_cache"], case["cache_dtype"], case["block_indices"][bb[s]:bb[s + 1]],
                                    int(pl[s] + qlen), h, case["Hkv"], case["D"], case["block_size"])


@pytest.mark.parametrize("cache_dtype,window,score_window", [(W.F16, 0, None), (W.U8, 0, [1, 3, 0, 2]), (W.F32, 20, None),
                                                              (W.BF16, 7, [2, 1, 1, 40])])
def test_paged_scores_match_a_numpy_restatement(oracle, cache_dtype, window, score_window):
    seqs = [(30, 5), (0, 9), (65, 1), (12, 4)]
    Hq, Hkv, D, bs = 4, 2, 16, 8
    case = W.make_paged_case(71, seqs, Hq, Hkv, D, bs, W.F32, W.F32, cache_dtype, sliding_window=window)
    oracle.kv_cache_write(case["k_new"], case["v_new"], case["key_cache"], case["value_cache"], cache_dtype, case["past_lens"],
                          case["subsequence_begins"], case["block_indices"], case["block_indices_begins"], Hkv, D, bs)
    got = oracle.paged_attention_scores(case["q"], case["key_cache"], cache_dtype, case["past_lens"], case["subsequence_begins"],
                                        case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs,
                                        score_window=score_window, sliding_window=window)
    q = case["q"].reshape(-1, Hq, D).astype(np.float64)
    ref, start = np.zeros_like(got, dtype=np.float64), 0
    for s, (past, qlen) in enumerate(seqs):
        ctx = past + qlen
        t0 = case["subsequence_begins"][s]
        w = qlen if score_window is None else min(qlen, score_window[s])
        for h in range(Hq):
            K = _dense_keys(oracle, case, s, h // (Hq // Hkv)).astype(np.float64)
            for i in range(qlen - w, qlen):
                p = past + i
                j0 = max(0, p - window + 1) if window > 0 else 0
                sc = (K[j0:p + 1] @ q[t0 + i, h]) / np.sqrt(D)
                e = np.exp(sc - sc.max())
                ref[start + j0:start + p + 1] += e / e.sum()
        assert abs(got[start:start + ctx].sum() - Hq * w) < 1e-4  # every softmax sums to one
        start += ctx
    assert start == got.size
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_paged_scores_give_nothing_to_positions_without_a_block(oracle):
    """Table entries outside the pool: their positions get no probability and the others share a row's
    whole unit of it, as if those positions were not there (numpy over the remaining keys); a sequence with
    no valid entry scores zeros."""
    seqs = [(30, 5), (0, 9), (65, 1), (12, 4)]
    Hq, Hkv, D, bs = 4, 2, 16, 8
    case = W.make_paged_case(73, seqs, Hq, Hkv, D, bs, W.F32, W.F32, W.F16)
    ids, bb, nb = case["block_indices"], case["block_indices_begins"], case["num_blocks"]
    ids[bb[0] + 1] = nb + 2
    ids[bb[0] + 4] = -1  # the block of the new tokens
    ids[bb[2] + 3] = 1 << 30
    ids[bb[3]:bb[4]] = -5
    oracle.kv_cache_write(case["k_new"], case["v_new"], case["key_cache"], case["value_cache"], W.F16, case["past_lens"],
                          case["subsequence_begins"], ids, bb, Hkv, D, bs)
    got = oracle.paged_attention_scores(case["q"], case["key_cache"], W.F16, case["past_lens"], case["subsequence_begins"],
                                        ids, bb, Hq, Hkv, D, bs)
    q = case["q"].reshape(-1, Hq, D).astype(np.float64)
    ref, start = np.zeros_like(got, dtype=np.float64), 0
    for s, (past, qlen) in enumerate(seqs):
        ctx, t0 = past + qlen, case["subsequence_begins"][s]
        table = ids[bb[s]:bb[s + 1]]
        there = np.array([0 <= table[j // bs] < nb for j in range(ctx)])
        safe = np.where((table >= 0) & (table < nb), table, 0).astype(np.int32)
        for h in range(Hq):
            K = oracle.gather_cache_rows(case["key_cache"], W.F16, safe, ctx, h // (Hq // Hkv), Hkv, D, bs).astype(np.float64)
            for i in range(qlen):
                p = past + i
                keep = np.nonzero(there[:p + 1])[0]
                if keep.size == 0:
                    continue
                sc = (K[keep] @ q[t0 + i, h]) / np.sqrt(D)
                e = np.exp(sc - sc.max())
                ref[start + keep] += e / e.sum()
        assert not got[start:start + ctx][~there].any()
        start += ctx
    assert not got[-16:].any() and ref[:35].any()
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_paged_scores_are_the_probabilities_of_the_attention(oracle):
    """One head, one new token: out = sum_j scores[j] * v[j], with out from the attention oracle."""
    seqs = [(37, 1), (5, 1)]
    case = W.make_paged_case(72, seqs, 1, 1, 32, 16, W.F32, W.F32, W.F32)
    ref, kc, vc = None, case["key_cache"].copy(), case["value_cache"].copy()
    out = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, W.F32, case["past_lens"],
                                 case["subsequence_begins"], case["block_indices"], case["block_indices_begins"], 1, 1, 32, 16)
    sc = oracle.paged_attention_scores(case["q"], kc, W.F32, case["past_lens"], case["subsequence_begins"],
                                       case["block_indices"], case["block_indices_begins"], 1, 1, 32, 16)
    start = 0
    for s, (past, qlen) in enumerate(seqs):
        bb = case["block_indices_begins"]
        V = oracle.gather_cache_rows(vc, W.F32, case["block_indices"][bb[s]:bb[s + 1]], past + 1, 0, 1, 32, 16)
        np.testing.assert_allclose(sc[start:start + past + 1] @ V, out[s], rtol=1e-5, atol=1e-6)
        start += past + 1


# ---- attention sinks --------------------------------------------------------------------------------
@pytest.mark.parametrize("window,alibi", [(0, False), (9, False), (0, True)])
def test_paged_attention_sinks_match_the_closed_form(oracle, window, alibi):
    """sinks: a per-head logit in the denominator of every row's softmax, no value row.  Against numpy in fp64 over
    the gathered keys and values; sinks of -inf change nothing, to the bit; a large sink takes nearly all of the
    probability and the output goes to zero."""
    seqs = [(20, 3), (0, 6), (33, 1)]
    Hq, Hkv, D, bs = 4, 2, 16, 8
    case = W.make_paged_case(75, seqs, Hq, Hkv, D, bs, W.F32, W.F32, W.F32, sliding_window=window)
    sinks = np.array([0.3, -1.5, 2.0, 0.0], np.float32)
    slopes = np.array([0.5, 0.25, 0.125, 0.0625], np.float32) if alibi else None
    def run(sk):
        kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
        out = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, W.F32, case["past_lens"], case["subsequence_begins"],
                                     case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs, sliding_window=window,
                                     alibi_slopes=slopes, sinks=sk)
        return out, kc, vc
    got, kc, vc = run(sinks)
    plain, _, _ = run(None)
    none, _, _ = run(np.full(Hq, -np.inf, np.float32))
    assert np.array_equal(plain, none)
    assert np.abs(got - plain).max() > 1e-2
    q = case["q"].reshape(-1, Hq, D).astype(np.float64)
    bb = case["block_indices_begins"]
    for s, (past, qlen) in enumerate(seqs):
        t0 = case["subsequence_begins"][s]
        blocks = case["block_indices"][bb[s]:bb[s + 1]]
        for h in range(Hq):
            K = oracle.gather_cache_rows(kc, W.F32, blocks, past + qlen, h // (Hq // Hkv), Hkv, D, bs).astype(np.float64)
            V = oracle.gather_cache_rows(vc, W.F32, blocks, past + qlen, h // (Hq // Hkv), Hkv, D, bs).astype(np.float64)
            for i in range(qlen):
                p = past + i
                j0 = max(0, p - window + 1) if window > 0 else 0
                sc = (K[j0:p + 1] @ q[t0 + i, h]) / np.sqrt(D)
                if alibi:
                    sc = sc + float(slopes[h]) * (np.arange(j0, p + 1) - p)
                e = np.exp(sc - sc.max())
                want = (e @ V[j0:p + 1]) / (e.sum() + np.exp(float(sinks[h]) - sc.max()))
                np.testing.assert_allclose(got[t0 + i].reshape(Hq, D)[h], want, rtol=2e-5, atol=2e-6)
    big, _, _ = run(np.full(Hq, 60.0, np.float32))
    assert np.abs(big).max() < 1e-15 * 1e3


# ---- the operator's cache rotation ----------------------------------------------------------------
def _trig_lut(rows, D, base=10000.0, sign=1.0):
    """Row r: cos(r theta_i) for i < D/2, then sign * sin(r theta_i), with the rotary embedding's frequencies."""
    theta = base ** (-np.arange(D // 2, dtype=np.float64) * 2.0 / D)
    ang = np.arange(rows, dtype=np.float64)[:, None] * theta[None, :]
    return np.concatenate([np.cos(ang), sign * np.sin(ang)], axis=1).astype(np.float32)


def _f32_cache(rng, num_blocks, Hkv, bs, D):
    rows = rng.standard_normal((num_blocks, Hkv, bs, D)).astype(np.float32)
    return rows, np.ascontiguousarray(rows).view(np.uint8).reshape(num_blocks, Hkv, bs, D * 4)


def test_cache_rotation_composes_inverts_and_keeps_norms(oracle):
    rng = np.random.default_rng(5)
    nb, Hkv, bs, D = 9, 3, 8, 32
    rows, cache = _f32_cache(rng, nb, Hkv, bs, D)
    lut = _trig_lut(64, D)
    blocks = [4, 1, 7]
    one = cache.copy()
    oracle.rotate_key_cache(one, W.F32, blocks, [[5], [9], [0]], lut, Hkv, D, bs)
    oracle.rotate_key_cache(one, W.F32, blocks, [[12], [3], [40]], lut, Hkv, D, bs)
    both = cache.copy()
    oracle.rotate_key_cache(both, W.F32, blocks, [[17], [12], [40]], lut, Hkv, D, bs)
    a, b = one.view(np.float32).reshape(rows.shape), both.view(np.float32).reshape(rows.shape)
    np.testing.assert_allclose(a, b, rtol=0, atol=3e-6)
    # the blocks that are not listed keep their bytes; the listed ones moved (but for the rotation by row 0) and kept their norms
    for blk in range(nb):
        if blk not in blocks:
            assert np.array_equal(b[blk], rows[blk])
    assert np.abs(b[4] - rows[4]).max() > 0.1 and np.abs(b[1] - rows[1]).max() > 0.1
    np.testing.assert_allclose(np.linalg.norm(b, axis=-1), np.linalg.norm(rows, axis=-1), rtol=1e-5)
    # the table with the sines negated turns back
    back = both.copy()
    oracle.rotate_key_cache(back, W.F32, blocks, [[17], [12], [40]], _trig_lut(64, D, sign=-1.0), Hkv, D, bs)
    np.testing.assert_allclose(back.view(np.float32).reshape(rows.shape), rows, rtol=0, atol=3e-6)


def test_cache_rotation_moves_a_rotary_embedded_key_to_another_position(oracle):
    """Keys stored with the rotary embedding of their positions (rotate-half layout, the embedding oracle that
    transformers' apply_rotary_pos_emb pins), turned by delta, are the keys embedded at position + delta: per
    block and per token."""
    rng = np.random.default_rng(6)
    Hkv, bs, D, nb = 2, 4, 64, 5
    plain = rng.standard_normal((nb * bs, Hkv, D)).astype(np.float32)
    lut = _trig_lut(200, D)
    cos = np.concatenate([lut[:, :D // 2], lut[:, :D // 2]], axis=1)
    sin = np.concatenate([lut[:, D // 2:], lut[:, D // 2:]], axis=1)
    positions = rng.integers(0, 60, nb * bs).astype(np.int32)
    def cache_of(pos):
        e = oracle.rope(plain, cos, sin, pos.astype(np.int32))                        # [tokens, Hkv, D]
        return np.ascontiguousarray(e.reshape(nb, bs, Hkv, D).transpose(0, 2, 1, 3))  # [block, head, token, D]
    cache = cache_of(positions).view(np.uint8).reshape(nb, Hkv, bs, D * 4).copy()
    per_block = rng.integers(0, 100, (2, 1)).astype(np.int32)
    per_token = rng.integers(0, 100, (2, bs)).astype(np.int32)
    oracle.rotate_key_cache(cache, W.F32, [3, 0], per_block, lut, Hkv, D, bs)
    oracle.rotate_key_cache(cache, W.F32, [1, 4], per_token, lut, Hkv, D, bs)
    shift = np.zeros((nb, bs), np.int32)
    shift[3], shift[0] = per_block[0, 0], per_block[1, 0]
    shift[1], shift[4] = per_token[0], per_token[1]
    want = cache_of(positions + shift.reshape(-1))
    np.testing.assert_allclose(cache.view(np.float32).reshape(want.shape), want, rtol=0, atol=2e-5)


@pytest.mark.parametrize("cache_dtype", [W.F16, W.BF16, W.U8])
def test_cache_rotation_in_the_cache_types_and_what_it_skips(oracle, cache_dtype):
    """16-bit and u8 caches: the fp32 rotation of the stored values, rounded (u8: quantised again, within half a
    step of the row's new scale); block ids outside the pool and deltas outside the table leave their rows alone."""
    rng = np.random.default_rng(7)
    nb, Hkv, bs, D = 6, 2, 8, 32
    rows = rng.standard_normal((nb, Hkv, bs, D)).astype(np.float32)
    rb = {W.F16: 2 * D, W.BF16: 2 * D, W.U8: D + 8}[cache_dtype]
    cache = np.zeros((nb, Hkv, bs, rb), np.uint8)
    for blk in range(nb):
        for h in range(Hkv):
            cache[blk, h] = W.cache_rows_from_f32(rows[blk, h], cache_dtype)
    stored = np.stack([[oracle.gather_cache_rows(cache, cache_dtype, [blk], bs, h, Hkv, D, bs) for h in range(Hkv)] for blk in range(nb)])
    lut = _trig_lut(50, D)
    before = cache.copy()
    deltas = np.array([[7] * bs, [3] * bs, [49] + [50] * (bs - 1), [1] * bs], np.int32)  # block 5: only token 0 has a row of the table
    oracle.rotate_key_cache(cache, cache_dtype, [2, -1, 5, nb], deltas, lut, Hkv, D, bs)
    f32 = np.ascontiguousarray(stored).view(np.uint8).reshape(nb, Hkv, bs, D * 4).copy()
    oracle.rotate_key_cache(f32, W.F32, [2, -1, 5, nb], deltas, lut, Hkv, D, bs)
    want = f32.view(np.float32).reshape(stored.shape)
    got = np.stack([[oracle.gather_cache_rows(cache, cache_dtype, [blk], bs, h, Hkv, D, bs) for h in range(Hkv)] for blk in range(nb)])
    for blk in (0, 1, 3, 4):
        assert np.array_equal(cache[blk], before[blk])
    assert np.array_equal(cache[5, :, 1:], before[5, :, 1:]) and not np.array_equal(cache[5, :, 0], before[5, :, 0])
    if cache_dtype == W.U8:
        scale = cache[2].view(np.float32).reshape(Hkv, bs, -1)[:, :, 0]  # (scale, zero-point) lead a row
        assert np.all(np.abs(got[2] - want[2]) <= 0.5 * scale[:, :, None] + 1e-6)
    else:
        np.testing.assert_allclose(got[2], want[2], rtol=2 ** -8 if cache_dtype == W.BF16 else 2 ** -11, atol=1e-6)
