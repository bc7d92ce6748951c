"""hipattn_paged_attention_noalloc: the entry point whose scratch is the library's static device
array.  It must give what hipattn_paged_attention gives with a caller workspace, on calls that
follow each other (the array keeps the previous call's contents), and refuse what does not fit."""
import numpy as np
import pytest

import helpers as H
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu


def run_both(hip, case, flags=0):
    """(output of the workspace entry point, output of the no-alloc entry point, caches of each)."""
    res = []
    for noalloc in (False, True):
        dev = H.PagedDeviceCase(hip, case)
        desc = H.pa_desc(hip, case, flags=flags)
        dev.out.fill(0xFF)
        if noalloc:
            hip.paged_attention_noalloc(desc, dev.q, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache,
                                        dev.past_lens, dev.subsequence_begins, dev.block_indices,
                                        dev.block_indices_begins, dev.out)
        else:
            nbytes = hip.paged_attention_workspace_size(desc)
            ws = hip.DeviceBuffer(nbytes) if nbytes else None
            hip.paged_attention(desc, dev.q, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache, dev.past_lens,
                                dev.subsequence_begins, dev.block_indices, dev.block_indices_begins, dev.out, ws)
        path = hip.last_kernel_path()
        out = dev.out.download(np.uint16, (case["T"], case["Hq"] * case["D"]))
        kc, vc = dev.caches()
        dev.free()
        res.append((out, kc, vc, path))
    return res


@pytest.mark.parametrize("cache_dtype", [W.F16, W.U8])
def test_noalloc_matches_the_workspace_entry_point_on_two_calls_in_a_row(hip, oracle, cache_dtype):
    print("noalloc two calls", cache_dtype, flush=True)
    big = [(c - 1, 1) for c in (3001, 1500, 700, 2049, 33, 1, 900, 4000, 257, 64, 1023, 5)]
    small = [(c - 1, 1) for c in (300, 31, 1200)]
    for i, seqs in enumerate((big, small)):  # the second call is smaller: stale scratch beyond it must not matter
        case = W.make_paged_case(120 + i, seqs, 32, 8, 128, 32, W.F16, W.F16, cache_dtype, sliding_window=0)
        (o_ws, k_ws, v_ws, p_ws), (o_na, k_na, v_na, p_na) = run_both(hip, case)
        assert p_ws == p_na == "paged_mfma"
        np.testing.assert_array_equal(k_ws, k_na)
        np.testing.assert_array_equal(v_ws, v_na)
        # the same kernels on the same schedule: the same bits
        np.testing.assert_array_equal(o_ws, o_na)
        ref, okc, ovc = H.oracle_paged(oracle, case)
        np.testing.assert_array_equal(k_na, okc)
        out = H.storage_to_f32(o_na, W.F16)
        assert H.max_abs(out, ref) <= (1e-2 if cache_dtype == W.U8 else 2e-3)


def test_noalloc_mixed_batch_runs_without_the_side_stream(hip, oracle):
    print("noalloc mixed", flush=True)
    seqs = [(0, 130), (37, 1), (500, 1), (100, 257), (999, 1), (5, 0)]
    case = W.make_paged_case(123, seqs, 16, 4, 128, 32, W.BF16, W.BF16, W.F16, sliding_window=300)
    (o_ws, _, _, _), (o_na, k_na, _, path) = run_both(hip, case)
    assert path == "paged_mfma"
    ref, okc, _ = H.oracle_paged(oracle, case)
    np.testing.assert_array_equal(k_na, okc)
    out = H.storage_to_f32(o_na, W.BF16)
    assert H.scaled_bound_error(out, ref, "noalloc mixed") <= 1e-2
    # against the workspace entry point (which overlaps the two parts on two streams): same arithmetic
    # per row, possibly a different split of the decode work, so equal to rounding, not to the bit
    assert H.max_abs(out, H.storage_to_f32(o_ws, W.BF16)) <= 1e-2


@pytest.mark.parametrize("D,bs,path", [(96, 16, "paged_mfma"), (64, 32, "paged_mfma"), (96, 64, "paged_mfma"), (256, 16, "paged_mfma"), (192, 16, "paged_mfma"), (192, 8, "paged_mfma_tiles")])
def test_noalloc_on_the_other_shapes(hip, oracle, D, bs, path):
    """The other 16-bit shapes keep their scratch (partials of the stream-K kernel, the tile numbering of
    the query-tile kernel) in the static array as well: two calls in a row, the second smaller."""
    print("noalloc other shapes", D, bs, flush=True)
    batches = ([(c - 1, 1) for c in (3001, 1500, 700, 2049, 33, 1, 900, 257)] + [(10, 140), (0, 3)], [(299, 1), (5, 20)])
    for i, seqs in enumerate(batches):
        case = W.make_paged_case(125 + i, seqs, 16, 4, D, bs, W.F16, W.F16, W.F16, sliding_window=0)
        (o_ws, k_ws, _, _), (o_na, k_na, _, p_na) = run_both(hip, case)
        assert p_na == path
        ref, okc, _ = H.oracle_paged(oracle, case)
        np.testing.assert_array_equal(k_na, okc)
        np.testing.assert_array_equal(k_ws, okc)
        assert H.scaled_bound_error(H.storage_to_f32(o_na, W.F16), ref, "noalloc other shapes") <= 2e-3
        assert H.max_abs(H.storage_to_f32(o_na, W.F16), H.storage_to_f32(o_ws, W.F16)) <= 2e-3


def test_noalloc_refuses_a_batch_beyond_its_scratch(hip):
    print("noalloc too big", flush=True)
    # 16 query heads per kv head and 4,096 sequences need far more partial-result slots than 16 MiB hold
    desc = hip.PaDesc(W.F16, W.F16, W.F16, W.F16, 128, 8, 128, 32, 8, 4096, 4096, 64, 0, 0.0, 0, 0)
    assert hip.paged_attention_workspace_size(desc) > hip.NOALLOC_SCRATCH_BYTES
    one = hip.DeviceBuffer(16)
    st = hip.lib().hipattn_paged_attention_noalloc(desc, one.ptr, one.ptr, one.ptr, one.ptr, one.ptr, one.ptr, one.ptr,
                                                   one.ptr, one.ptr, one.ptr, None)
    assert st == hip.WORKSPACE_TOO_SMALL
    assert b"static scratch" in hip.lib().hipattn_last_error_string()
    one.free()
