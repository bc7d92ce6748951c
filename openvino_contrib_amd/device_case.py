"""Host-side plumbing around the C ABI for synthetic workloads: upload a case made by workloads.py,
run it through libhipattn and bring the results back as fp32 numpy arrays.  Used by the benchmark,
the smoke check and the GPU tests.  `hip` is the capi module."""
import numpy as np

from . import workloads as W


def storage_to_f32(arr, dtype):
    if dtype == W.F32:
        return arr.astype(np.float32)
    if dtype == W.F16:
        return W.f16_bits_to_f32(arr)
    return W.bf16_bits_to_f32(arr)


def run_sdpa(hip, case, causal, scale=0.0):
    desc = hip.SdpaDesc(case["dtype"], case["B"], case["Hq"], case["Hkv"], case["Lq"], case["Lk"], case["D"],
                        int(causal), scale)
    q = hip.DeviceBuffer.from_numpy(case["q_store"])
    k = hip.DeviceBuffer.from_numpy(case["k_store"])
    v = hip.DeviceBuffer.from_numpy(case["v_store"])
    out = hip.DeviceBuffer(case["q_store"].nbytes)
    out.fill(0xFF)  # NaN pattern: rows the kernel fails to write show up
    ws_bytes = hip.sdpa_workspace_size(desc)
    ws = hip.DeviceBuffer(ws_bytes) if ws_bytes else None
    hip.sdpa(desc, q, k, v, out, ws)
    res = out.download(W.np_storage_dtype(case["dtype"]), case["q_store"].shape)
    path = hip.last_kernel_path()
    for b in (q, k, v, out):
        b.free()
    return storage_to_f32(res, case["dtype"]), path


def run_sdpa_masked(hip, case, mask, scale=0.0, mask_dtype=None):
    """mask: numpy array broadcastable to [B,Hq,Lq,Lk]; bool (True = take part) or float32 / float16 (additive).
    mask_dtype W.F16 / W.BF16 stores a float mask in that type (rounded to nearest)."""
    desc = hip.SdpaDesc(case["dtype"], case["B"], case["Hq"], case["Hkv"], case["Lq"], case["Lk"], case["D"], 0, scale)
    m = np.asarray(mask)
    while m.ndim < 4:
        m = m[None]
    if m.dtype != np.bool_ and mask_dtype in (W.F16, W.BF16):
        store, mdtype = np.ascontiguousarray(W.to_storage(np.asarray(m, np.float32), mask_dtype)[0]), mask_dtype
    elif m.dtype == np.bool_:
        store, mdtype = np.ascontiguousarray(m.astype(np.uint8)), W.U8
    elif m.dtype == np.float16:
        store, mdtype = np.ascontiguousarray(m).view(np.uint16), W.F16
    else:
        store, mdtype = np.ascontiguousarray(m, np.float32), W.F32
    full = (case["B"], case["Hq"], case["Lq"], case["Lk"])
    strides = [store.strides[ax] // store.itemsize if (store.shape[ax] == full[ax] and full[ax] > 1) else 0
               for ax in range(4)]
    bufs = [hip.DeviceBuffer.from_numpy(case[n]) for n in ("q_store", "k_store", "v_store")]
    mbuf = hip.DeviceBuffer.from_numpy(store)
    out = hip.DeviceBuffer(case["q_store"].nbytes)
    out.fill(0xFF)
    hip.sdpa_masked(desc, bufs[0], bufs[1], bufs[2], mdtype, strides, mbuf, out)
    res = out.download(W.np_storage_dtype(case["dtype"]), case["q_store"].shape)
    path = hip.last_kernel_path()
    for b in bufs + [mbuf, out]:
        b.free()
    return storage_to_f32(res, case["dtype"]), path


def pa_desc(hip, case, out_dtype=None, flags=0, decode_waves=0, scale=0.0, max_context_len=None, alibi=None, sinks=None):
    """alibi, sinks: None or a DeviceBuffer of Hq floats (the operator's alibi_slopes / sinks input)."""
    return hip.PaDesc(case["q_dtype"], case["kv_dtype"], case["cache_dtype"],
                      case["q_dtype"] if out_dtype is None else out_dtype, case["Hq"], case["Hkv"], case["D"],
                      case["block_size"], case["num_blocks"], case["T"], case["S"],
                      case["max_context_len"] if max_context_len is None else max_context_len,
                      case["sliding_window"], scale, flags, decode_waves, alibi.ptr if alibi is not None else None,
                      sinks.ptr if sinks is not None else None)


class PagedDeviceCase:
    """Device copies of one paged-attention call."""

    def __init__(self, hip, case, out_dtype=None):
        self.hip, self.case = hip, case
        self.out_dtype = case["q_dtype"] if out_dtype is None else out_dtype
        up = hip.DeviceBuffer.from_numpy
        self.q = up(case["q_store"])
        self.k_new = up(case["k_new_store"])
        self.v_new = up(case["v_new_store"])
        self.key_cache = up(case["key_cache"])
        self.value_cache = up(case["value_cache"])
        self.past_lens = up(case["past_lens"])
        self.subsequence_begins = up(case["subsequence_begins"])
        self.block_indices = up(case["block_indices"])
        self.block_indices_begins = up(case["block_indices_begins"])
        self.out_elems = case["T"] * case["Hq"] * case["D"]
        self.out = hip.DeviceBuffer(self.out_elems * hip.DTYPE_BYTES[self.out_dtype])

    def run(self, flags=0, decode_waves=0, scale=0.0, max_context_len=None, stream=None, alibi=None, sinks=None):
        hip = self.hip
        desc = pa_desc(hip, self.case, self.out_dtype, flags, decode_waves, scale, max_context_len, alibi, sinks)
        nbytes = hip.paged_attention_workspace_size(desc)
        ws = hip.DeviceBuffer(nbytes) if nbytes else None
        self.out.fill(0xFF)
        hip.paged_attention(desc, self.q, self.k_new, self.v_new, self.key_cache, self.value_cache, self.past_lens,
                            self.subsequence_begins, self.block_indices, self.block_indices_begins, self.out, ws,
                            stream)
        path = hip.last_kernel_path()
        res = self.out.download(W.np_storage_dtype(self.out_dtype), (self.case["T"], self.case["Hq"] * self.case["D"]),
                                stream)
        if ws:
            ws.free()
        return storage_to_f32(res, self.out_dtype), path

    def scores(self, score_window=None, scale=0.0, max_context_len=None, stream=None, lse_only=False):
        """The operator's second output for the cache as it stands (call run() first): f32
        [sum(past_lens) + tokens].  lse_only: the smallest workspace the call accepts (the fp32 kernels)."""
        hip, case = self.hip, self.case
        desc = pa_desc(hip, case, self.out_dtype, 0, 0, scale, max_context_len)
        total = int(np.sum(case["past_lens"])) + case["T"]
        out = hip.DeviceBuffer((total + 16) * 4)
        out.fill(0xEE)
        sw = None if score_window is None else hip.DeviceBuffer.from_numpy(np.asarray(score_window, np.int32))
        hip.paged_attention_scores(desc, self.q, self.key_cache, self.past_lens, self.subsequence_begins,
                                   self.block_indices, self.block_indices_begins, sw, out, total, stream, lse_only=lse_only)
        res = out.download(np.float32, (total + 16,), stream)
        out.free()
        if sw is not None:
            sw.free()
        canary = np.frombuffer(b"\xee" * 4, np.float32)[0]
        assert np.all(res[total:].view(np.uint32) == canary.view(np.uint32)), "scores written beyond the capacity"
        return res[:total]

    def caches(self):
        kc = self.key_cache.download(np.uint8, self.case["key_cache"].shape)
        vc = self.value_cache.download(np.uint8, self.case["value_cache"].shape)
        return kc, vc

    def free(self):
        for b in (self.q, self.k_new, self.v_new, self.key_cache, self.value_cache, self.past_lens,
                  self.subsequence_begins, self.block_indices, self.block_indices_begins, self.out):
            b.free()


def max_abs(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64)))) if a.size else 0.0
