"""Shared plumbing of the GPU parity tests: the device-side case runners of the package plus the
oracle call they are compared with."""
from openvino_contrib_amd.device_case import (PagedDeviceCase, max_abs, pa_desc, run_sdpa, run_sdpa_masked,  # noqa: F401
                                              storage_to_f32)


def oracle_paged(oracle, case, scale=0.0):
    kc, vc = case["key_cache"].copy(), case["value_cache"].copy()
    out = oracle.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, case["cache_dtype"],
                                 case["past_lens"], case["subsequence_begins"], case["block_indices"],
                                 case["block_indices_begins"], case["Hq"], case["Hkv"], case["D"], case["block_size"],
                                 scale=scale, sliding_window=case["sliding_window"])
    return out, kc, vc


