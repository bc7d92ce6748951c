"""Synthetic inputs for the attention hot path: the five benchmark configurations and the
building blocks the tests use for smaller cases.  numpy only; nothing here touches the GPU.

All randomness comes from numpy.random.Generator(PCG64(seed)).  Arrays that stand for fp16 /
bf16 tensors are returned as uint16 bit patterns (`*_bits`) next to their exact fp32 value.
"""
import math

import numpy as np

F32, F16, BF16, U8 = 0, 1, 2, 3


# ------------------------------------------------------------------------------ conversions
def f32_to_bf16_bits(x):
    """Round to nearest even; x finite."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, np.uint16).view(np.float16).astype(np.float32)


def to_storage(x, dtype):
    """fp32 array -> (storage array, exact fp32 value of what was stored)."""
    x = np.ascontiguousarray(x, np.float32)
    if dtype == F32:
        return x, x
    if dtype == F16:
        b = f32_to_f16_bits(x)
        return b, f16_bits_to_f32(b)
    if dtype == BF16:
        b = f32_to_bf16_bits(x)
        return b, bf16_bits_to_f32(b)
    raise ValueError("dtype %r" % (dtype,))


def np_storage_dtype(dtype):
    return {F32: np.float32, F16: np.uint16, BF16: np.uint16, U8: np.uint8}[dtype]


def cache_row_bytes(dtype, D):
    return {F32: 4 * D, F16: 2 * D, BF16: 2 * D, U8: D + 8}[dtype]


def quantize_u8_rows(x):
    """x [..., D] fp32 -> uint8 [..., D + 8]: rows of [scale f32][zero-point f32][D bytes].

    Asymmetric per-row quantisation: scale = (max - min) / 255 (1e-4 if the row is constant),
    zp = -min / scale, q = clamp(rint(x / scale + zp), 0, 255).
    """
    x = np.ascontiguousarray(x, np.float32)
    D = x.shape[-1]
    flat = x.reshape(-1, D)
    mn = flat.min(axis=1)
    mx = flat.max(axis=1)
    scale = ((mx - mn) / np.float32(255.0)).astype(np.float32)
    scale[scale == 0] = np.float32(0.0001)
    zp = (-mn / scale).astype(np.float32) + np.float32(0.0)
    inv = (np.float32(1.0) / scale).astype(np.float32)
    # fused multiply-add emulated in fp64 (the product of two fp32 values is exact there)
    t = (flat.astype(np.float64) * inv[:, None].astype(np.float64) + zp[:, None].astype(np.float64)).astype(np.float32)
    q = np.clip(np.rint(t), 0, 255).astype(np.uint8)
    out = np.empty((flat.shape[0], D + 8), np.uint8)
    out[:, 0:4] = scale.view(np.uint8).reshape(-1, 4)
    out[:, 4:8] = zp.view(np.uint8).reshape(-1, 4)
    out[:, 8:] = q
    return out.reshape(x.shape[:-1] + (D + 8,))


def cache_rows_from_f32(x, cache_dtype):
    """x [..., D] fp32 -> uint8 [..., row_bytes]."""
    if cache_dtype == U8:
        return quantize_u8_rows(x)
    st, _ = to_storage(x, cache_dtype)
    return st.view(np.uint8).reshape(x.shape[:-1] + (-1,))


# --------------------------------------------------------------------------------- SDPA
def make_sdpa_case(seed, B, Hq, Hkv, Lq, Lk, D, dtype, std=1.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    case = {"B": B, "Hq": Hq, "Hkv": Hkv, "Lq": Lq, "Lk": Lk, "D": D, "dtype": dtype}
    for name, shape in (("q", (B, Hq, Lq, D)), ("k", (B, Hkv, Lk, D)), ("v", (B, Hkv, Lk, D))):
        x = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        st, val = to_storage(x, dtype)
        case[name + "_store"] = st
        case[name] = val
    return case


def sdpa_flops(B, Hq, Lq, Lk, D, causal):
    """Algorithmic FLOPs: 4 * D per attended (query, key) pair."""
    if causal:
        pairs = sum(min(i + 1, Lk) for i in range(Lq))
    else:
        pairs = Lq * Lk
    return 4 * D * pairs * B * Hq


# --------------------------------------------------------------------- paged attention
def make_paged_case(seed, seqs, Hq, Hkv, D, block_size, q_dtype, kv_dtype, cache_dtype, spare_blocks=3,
                    sliding_window=0, distinct_blocks=4096):
    """Build one PagedAttentionExtension call.

    seqs: list of (past_len, q_len).  Every sequence gets ceil((past + q_len) / block_size)
    physical blocks; the block table is a seeded random permutation of the pool, sliced per
    sequence.  The whole pool (also rows no sequence uses) holds N(0,1) values stored in
    cache_dtype, so the op's own cache write is visible as a change of exactly the new rows.
    Pools larger than `distinct_blocks` repeat the first `distinct_blocks` random blocks (drawing
    gigabytes of normals would only cost time; the kernels never see the repetition as such
    because the block table is a random permutation).
    """
    rng = np.random.Generator(np.random.PCG64(seed))
    S = len(seqs)
    past = np.array([p for p, _ in seqs], np.int32)
    qlen = np.array([n for _, n in seqs], np.int32)
    begins = np.zeros(S + 1, np.int32)
    begins[1:] = np.cumsum(qlen)
    T = int(begins[-1])
    nblk = (past.astype(np.int64) + qlen + block_size - 1) // block_size
    bbegins = np.zeros(S + 1, np.int32)
    bbegins[1:] = np.cumsum(nblk)
    num_blocks = int(bbegins[-1]) + spare_blocks
    perm = rng.permutation(num_blocks).astype(np.int32)
    block_indices = perm[: int(bbegins[-1])].copy()

    rb = cache_row_bytes(cache_dtype, D)
    key_cache = np.empty((num_blocks, Hkv, block_size, rb), np.uint8)
    value_cache = np.empty((num_blocks, Hkv, block_size, rb), np.uint8)
    n_rand = min(num_blocks, distinct_blocks)
    for cache in (key_cache, value_cache):
        for b0 in range(0, n_rand, 512):
            b1 = min(n_rand, b0 + 512)
            x = rng.standard_normal((b1 - b0, Hkv, block_size, D), dtype=np.float32)
            cache[b0:b1] = cache_rows_from_f32(x, cache_dtype)
        for b0 in range(n_rand, num_blocks, n_rand):
            b1 = min(num_blocks, b0 + n_rand)
            cache[b0:b1] = cache[: b1 - b0]

    q_st, q = to_storage(rng.standard_normal((T, Hq * D), dtype=np.float32), q_dtype)
    k_st, k_new = to_storage(rng.standard_normal((T, Hkv * D), dtype=np.float32), kv_dtype)
    v_st, v_new = to_storage(rng.standard_normal((T, Hkv * D), dtype=np.float32), kv_dtype)
    return {
        "S": S, "T": T, "Hq": Hq, "Hkv": Hkv, "D": D, "block_size": block_size, "num_blocks": num_blocks,
        "q_dtype": q_dtype, "kv_dtype": kv_dtype, "cache_dtype": cache_dtype, "sliding_window": sliding_window,
        "past_lens": past, "subsequence_begins": begins, "block_indices": block_indices,
        "block_indices_begins": bbegins, "max_context_len": int((past + qlen).max()) if S else 0,
        "q": q, "q_store": q_st, "k_new": k_new, "k_new_store": k_st, "v_new": v_new, "v_new_store": v_st,
        "key_cache": key_cache, "value_cache": value_cache,
    }


def paged_kv_bytes(case, decode_only=False):
    """Algorithmic KV bytes of the call: every attended (position, kv head) row of K and of V once.
    decode_only restricts the sum to sequences with exactly one new token."""
    W = case["sliding_window"]
    rb = cache_row_bytes(case["cache_dtype"], case["D"])
    total = 0
    for s in range(case["S"]):
        past = int(case["past_lens"][s])
        qlen = int(case["subsequence_begins"][s + 1] - case["subsequence_begins"][s])
        if qlen <= 0 or (decode_only and qlen != 1):
            continue
        ctx = past + qlen
        lo = max(0, past - W + 1) if W > 0 else 0  # first position any token of the sequence attends
        total += (ctx - lo) * case["Hkv"] * 2 * rb
    return total


def paged_flops(case):
    """Algorithmic FLOPs: 4 * D per attended (query token, query head, key) triple."""
    W = case["sliding_window"]
    pairs = 0
    for s in range(case["S"]):
        past = int(case["past_lens"][s])
        qlen = int(case["subsequence_begins"][s + 1] - case["subsequence_begins"][s])
        for i in range(qlen):
            n = past + i + 1
            pairs += min(n, W) if W > 0 else n
    return 4 * case["D"] * pairs * case["Hq"]


# ------------------------------------------------------------ the five benchmark configs
def config1(seed=1001):
    """f32 SDPA, B=1 H=8 Lq=Lk=128 D=64, causal, default scale."""
    c = make_sdpa_case(seed, 1, 8, 8, 128, 128, 64, F32)
    c["causal"] = True
    return c


def config2(seed=1002, B=4, Hq=32, Hkv=8, L=2048, D=128):
    """bf16 prefill SDPA with GQA, causal, inputs 0.5 * N(0,1)."""
    c = make_sdpa_case(seed, B, Hq, Hkv, L, L, D, BF16, std=0.5)
    c["causal"] = True
    return c


def config3(seed=1003, S=64, lo=512, hi=8192, head_dim=128, block_size=32):
    """fp16 paged decode: S sequences x 1 new token, contexts uniform in [lo, hi]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = rng.integers(lo, hi + 1, size=S)
    seqs = [(int(c) - 1, 1) for c in ctx]
    return make_paged_case(seed + 100000, seqs, 32, 8, head_dim, block_size, F16, F16, F16)


def config4(seed=1004, S=128, lo=1024, hi=16384, head_dim=128, block_size=32):
    """u8-KV paged decode, per-token per-head asymmetric scale / zero-point, Hq=64."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = rng.integers(lo, hi + 1, size=S)
    seqs = [(int(c) - 1, 1) for c in ctx]
    return make_paged_case(seed + 100000, seqs, 64, 8, head_dim, block_size, F16, F16, U8)


def config5(seed=1005, n_prefill=8, chunk=512, past_hi=4096, n_decode=120, dec_lo=256, dec_hi=8192, window=4096,
            cache_dtype=F16, block_size=32, head_dim=128):
    """Mixed chunked prefill + decode, sliding window, bf16 activations, fp16 cache (or cache_dtype), Hq=64."""
    rng = np.random.Generator(np.random.PCG64(seed))
    seqs = [(int(p), chunk) for p in rng.integers(0, past_hi + 1, size=n_prefill)]
    seqs += [(int(c) - 1, 1) for c in rng.integers(dec_lo, dec_hi + 1, size=n_decode)]
    return make_paged_case(seed + 100000, seqs, 64, 8, head_dim, block_size, BF16, BF16, cache_dtype, sliding_window=window)
