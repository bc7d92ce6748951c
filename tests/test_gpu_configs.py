"""The five benchmark configurations at full size, through the C ABI, against the CPU oracle
(whole output for the paged configurations, head slices for the 137 GFLOP prefill) and through
size-independent properties."""
import numpy as np
import pytest

import helpers as H
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu


def announce(*args):
    print("[config]", *args, flush=True)


def test_config1_f32_sdpa(hip, oracle):
    announce("C1 f32 B1 H8 L128 D64 causal")
    case = W.config1()
    out, path = H.run_sdpa(hip, case, True)
    ref = oracle.sdpa(case["q"], case["k"], case["v"], causal=True)
    err = H.max_abs(out, ref)
    announce("C1 max abs err", err, path)
    assert err <= 1e-4  # contract 2e-3; the fp32 kernel is held to 1e-4


def test_config2_bf16_prefill(hip, oracle):
    announce("C2 bf16 B4 Hq32 Hkv8 L2048 D128 causal")
    case = W.config2()
    out, path = H.run_sdpa(hip, case, True)
    assert path == "sdpa_flash_mfma"
    assert np.isfinite(out).all()
    # every one of the 128 query heads against the oracle (the launch order that maps workgroups to
    # (batch, kv head, query tile, head pair) is exactly what a wrong index would break for some of them)
    worst, worst_at = 0.0, None
    for b in range(case["B"]):
        for hkv in range(case["Hkv"]):
            hs = slice(hkv * 4, hkv * 4 + 4)
            ref = oracle.sdpa(case["q"][b:b + 1, hs], case["k"][b:b + 1, hkv:hkv + 1], case["v"][b:b + 1, hkv:hkv + 1],
                              causal=True)
            err = H.max_abs(out[b:b + 1, hs], ref)
            if err > worst:
                worst, worst_at = err, (b, hkv)
    announce("C2 max abs err over all 128 heads", worst, "at (batch, kv head)", worst_at)
    assert worst <= 1e-2
    # row 0 of every head attends key 0 only: the output row is V[0] of its kv head, exactly
    v0 = np.repeat(case["v"][:, :, 0], 4, axis=1)
    np.testing.assert_array_equal(out[:, :, 0], v0)
    # all-ones V: every softmax row sums to one
    ones = dict(case)
    ones["v_store"] = np.full_like(case["v_store"], 0x3F80)
    out1, _ = H.run_sdpa(hip, ones, True)
    assert np.abs(out1 - 1.0).max() <= 1e-2


def _run_paged_config(hip, oracle, case, tol, name):
    dev = H.PagedDeviceCase(hip, case)
    out, path = dev.run()
    assert path == "paged_mfma"
    assert np.isfinite(out).all()
    ref, okc, ovc = H.oracle_paged(oracle, case)
    kc, vc = dev.caches()
    np.testing.assert_array_equal(kc, okc)
    np.testing.assert_array_equal(vc, ovc)
    err = H.max_abs(out, ref)
    announce(name, "max abs err", err)
    assert err <= tol
    # idempotence: the cache now holds the new rows, a second call without the write step agrees bit for bit
    out2, _ = dev.run(flags=hip.PA_SKIP_CACHE_WRITE)
    np.testing.assert_array_equal(out, out2)
    dev.free()


def test_config3_fp16_paged_decode(hip, oracle):
    announce("C3 64 seq decode, ctx U[512,8192], fp16 cache")
    _run_paged_config(hip, oracle, W.config3(), 2e-3, "C3")


def test_config4_u8_paged_decode(hip, oracle):
    announce("C4 128 seq decode, ctx U[1024,16384], u8 cache")
    _run_paged_config(hip, oracle, W.config4(), 1e-2, "C4")


def test_config5_mixed_batch(hip, oracle):
    announce("C5 8x512 prefill + 120 decode, window 4096, bf16 q, fp16 cache")
    _run_paged_config(hip, oracle, W.config5(), 1e-2, "C5")


def test_config5_mixed_batch_u8_cache(hip, oracle):
    """Configuration 5's batch on a u8 cache: the chunks go through the flash kernel's u8 loads."""
    announce("C5 with a u8 cache")
    _run_paged_config(hip, oracle, W.config5(cache_dtype=W.U8), 1e-2, "C5-u8")


@pytest.mark.parametrize("D,bs", [(64, 16), (64, 32), (128, 16)])
def test_config3_at_head_64_and_blocks_of_16(hip, oracle, D, bs):
    """Configuration 3's batch on the other cache shapes of the matrix-core decode kernel."""
    announce("C3's batch, head size", D, "blocks of", bs)
    _run_paged_config(hip, oracle, W.config3(head_dim=D, block_size=bs), 2e-3, "C3 %d/%d" % (D, bs))


def test_config5_mixed_batch_on_blocks_of_16(hip, oracle):
    """Configuration 5's batch on cache blocks of 16 tokens: the same two kernels side by side."""
    announce("C5 with blocks of 16")
    _run_paged_config(hip, oracle, W.config5(block_size=16), 1e-2, "C5 blocks of 16")


def test_config5_mixed_batch_at_head_64(hip, oracle):
    """Configuration 5's batch at head size 64 on blocks of 16: decode rows and the head-64 chunk kernel."""
    announce("C5 at head size 64, blocks of 16")
    _run_paged_config(hip, oracle, W.config5(block_size=16, head_dim=64), 1e-2, "C5 64/16")
