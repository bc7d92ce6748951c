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


def oracle_paged_no_write(oracle, case, scale=0.0):
    """The oracle on the cache as the case holds it (no new rows stored): what a call with
    HIPATTN_PA_SKIP_CACHE_WRITE on the uploaded cache has to give."""
    return oracle.paged_attention(case["q"], case["k_new"], case["v_new"], case["key_cache"].copy(), case["value_cache"].copy(),
                                  case["cache_dtype"], case["past_lens"], case["subsequence_begins"], case["block_indices"],
                                  case["block_indices_begins"], case["Hq"], case["Hkv"], case["D"], case["block_size"],
                                  scale=scale, sliding_window=case["sliding_window"], do_write=False)



def scaled_bound_error(out, ref, label=""):
    """Parity figure of tests whose reference values leave [-1, 1].

    Prints the plain max-abs error (the figure the tolerance contract is stated in) and returns
    max |out - ref| / max(1, |ref|), which is what such tests hold to their tolerance: a 16-bit
    output type alone rounds a value v by up to |v| * 2^-9 (bf16) or |v| * 2^-12 (fp16), so beyond
    |ref| = 1 a bound that does not grow with |ref| measures the output type, not the kernel.  Where
    every reference value lies in [-1, 1] the two figures are the same.  The five benchmark
    configurations are held to the plain figure."""
    import numpy as np

    err = np.abs(out.astype(np.float64) - ref.astype(np.float64))
    fin = np.isfinite(ref)
    if not fin.any():
        return 0.0
    plain = float(err[fin].max())
    scaled = float((err[fin] / np.maximum(1.0, np.abs(ref[fin]))).max())
    print("[parity] %s max-abs %.3g, scaled by max(1,|ref|) %.3g, max |ref| %.3g" % (label, plain, scaled, float(np.abs(ref[fin]).max())),
          flush=True)
    return scaled


def paged_matrix_core_path(Hq, Hkv, D, bs, cache_dtype):
    """Kernel path of a paged call with 16-bit queries and a 16-bit or u8 cache at a head size that is a
    multiple of 8 up to 256 and a power-of-two block size: the stream-K kernels on blocks of 16 tokens or more
    with at most 16 query heads per kv head, or a number of them that splits into equal groups of 8 to 16
    (each kv head is then entered once per group); the query-tile kernel the rest."""
    G = Hq // Hkv
    splits = G <= 16 or any(G % share == 0 and 8 <= G // share <= 16 for share in range(2, G + 1))
    return "paged_mfma" if bs >= 16 and splits else "paged_mfma_tiles"


def sdpa_matrix_core_path(D, masked):
    """Kernel path of a dense SDPA call with 16-bit operands and a head size that is a multiple of 8 up to 256
    (masked: with an attention mask the tuned kernel's mask tiles do not take, or at another head size than 128)."""
    if D <= 128 and not masked:
        return "sdpa_flash_mfma"  # (below 128: the tuned head-128 kernel on rows of fewer columns)
    return "sdpa_flash_mfma_d64" if D == 64 else "sdpa_flash_mfma_small"
