#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|layer|shapes|mqa|decoder|scores|masked] [--no-cpu] [--no-extra] [--no-plugin]

The LAST stdout line is ONE compact JSON object (under 3 KB); the full per-workload records go to the
file --detail names, or to stderr.  The headline is the fp16
paged-attention decode step (configuration 3, the one the headline metric is quoted on): a "step" is
one hipattn_paged_attention call on the whole synthetic batch (KV-cache write of the new tokens +
split-context decode + merge), inputs resident in HBM.
`value` is algorithmic KV bytes / wall time of a step; `roofline` is the same byte count over
the average duration of the dominant kernel (the split-context decode kernel), measured with
HIP events recorded by the library around that launch.  Unless --no-extra is given, the other
configurations are measured the same way and reported under "workloads" in the same line
(c2: bf16 causal prefill SDPA in TFLOP/s against the dense bf16 MFMA peak; c4: u8-KV decode;
c5: mixed chunked prefill + decode), each with a `cpu_baseline` of its own.  `cpu_baseline` times
the CPU oracle (a restatement, not OpenVINO's CPU plugin: OpenVINO is not installed) on a bounded
sample of the same workload.  `plugin_ms_per_step` of the headline workload is the same step through
the plugin layer's InferRequest::infer with device-resident tensors.  Everything that is not one of
the four configurations runs only when asked for: --workload layer (the operators of libhipops.so),
shapes (other cache shapes), decoder (a decoder layer through the plugin), scores (the operator's
second output), masked (config 2's shape with the causality as an attention mask).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16


CLOCK_RAMP_MS = 100.0  # untimed load ahead of the warmup steps, see time_steps


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(hip, fn, steps, warmup):
    """fn(i) enqueues one step on the default stream.  Returns (ms per step, dominant-kernel ms).

    Before the `warmup` untimed steps the same step runs untimed for CLOCK_RAMP_MS of GPU time: the
    shader clock of an idle MI355X takes some tens of milliseconds of load to reach its sustained
    level (a sub-millisecond step measured from idle runs 15-20 % slower than the same step in a
    serving loop), and a handful of warmup steps is over long before that."""
    ramp0, ramp1 = hip.Event(), hip.Event()
    ramped = 0.0
    while ramped < CLOCK_RAMP_MS:
        ramp0.record()
        for i in range(32):
            fn(i)
        ramp1.record()
        ramp1.synchronize()
        ramped += ramp0.elapsed_ms(ramp1)
    ramp0.close()
    ramp1.close()
    for i in range(warmup):
        fn(i)
    hip.check(hip.lib().hipattn_stream_synchronize(None))
    # timed region: exactly `steps` steps, bracketed by a synchronize on both sides
    start, stop = hip.Event(), hip.Event()
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    stop.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = start.elapsed_ms(stop) / steps
    # second pass of the same steps with an event pair around the dominant kernel of every step
    # (the extra event records serialise the launches a little, so this pass is not the one timed above)
    befores = [hip.Event() for _ in range(steps)]
    afters = [hip.Event() for _ in range(steps)]
    for i in range(steps):
        hip.profile_dominant_kernel(befores[i], afters[i])
        fn(i)
    hip.profile_dominant_kernel(None, None)
    hip.check(hip.lib().hipattn_stream_synchronize(None))
    kern = [befores[i].elapsed_ms(afters[i]) for i in range(steps)]
    for e in befores + afters + [start, stop]:
        e.close()
    # An event pair brackets the kernel plus the two record packets, so on a step that is one launch
    # the probed figure can read a microsecond or two above the step itself; a kernel cannot take
    # longer than the step it is part of, so the step time of the timed pass bounds it.
    return ev_ms, wall_ms, min(sum(kern) / len(kern), ev_ms)


def bench_paged(hip, case, steps, warmup, name):
    from openvino_contrib_amd import device_case as H
    from openvino_contrib_amd import workloads as W

    dev = H.PagedDeviceCase(hip, case)
    desc = H.pa_desc(hip, case)
    ws_bytes = hip.paged_attention_workspace_size(desc)
    ws = hip.DeviceBuffer(ws_bytes) if ws_bytes else None

    def step(_):
        hip.paged_attention(desc, dev.q, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache, dev.past_lens,
                            dev.subsequence_begins, dev.block_indices, dev.block_indices_begins, dev.out, ws)

    ms, wall_ms, kern_ms = time_steps(hip, step, steps, warmup)
    path = hip.last_kernel_path()
    kv_bytes = W.paged_kv_bytes(case)
    flops = W.paged_flops(case)
    decode_only = W.paged_kv_bytes(case, decode_only=True)  # what the split-context decode kernel reads
    res = {
        "decode_kv_bytes": decode_only,
        "workload": name, "kernel_path": path, "ms_per_step": ms, "host_ms_per_step": wall_ms,
        "dominant_kernel_ms": kern_ms, "kv_bytes": kv_bytes, "flops": flops, "workspace_bytes": ws_bytes,
        "kv_gbs": kv_bytes / (ms * 1e-3) / 1e9, "tflops": flops / (ms * 1e-3) / 1e12,
    }
    dev.free()
    if ws:
        ws.free()
    return res


def bench_paged_scores(hip, case, steps, name):
    """The operator's second output for the same batch (every new token aggregated), timed between two events:
    with the workspace the size query asks for (the matrix-core kernels: one read of the K rows) and with the
    smallest one the call accepts (the fp32 kernels: two reads)."""
    from openvino_contrib_amd import device_case as H
    from openvino_contrib_amd import workloads as W
    import ctypes
    import numpy as np

    dev = H.PagedDeviceCase(hip, case)
    dev.run()
    desc = H.pa_desc(hip, case)
    total = int(np.sum(case["past_lens"])) + case["T"]
    out = hip.DeviceBuffer(total * 4)
    n = ctypes.c_size_t(0)
    hip.check(hip.lib().hipattn_paged_attention_scores_workspace_size(ctypes.byref(desc), ctypes.byref(n)))
    k_bytes = W.paged_kv_bytes(case) // 2
    steps = max(3, min(steps, 20))
    res = {}
    for label, nbytes in (("asked_workspace", n.value), ("smallest_workspace", case["T"] * case["Hq"] * 4)):
        ws = hip.DeviceBuffer(nbytes)

        def call():
            hip.check(hip.lib().hipattn_paged_attention_scores(
                ctypes.byref(desc), dev.q.ptr, dev.key_cache.ptr, dev.past_lens.ptr, dev.subsequence_begins.ptr,
                dev.block_indices.ptr, dev.block_indices_begins.ptr, None, out.ptr, total, ws.ptr, ws.nbytes, None))

        for _ in range(2):
            call()
        e0, e1 = hip.Event(), hip.Event()
        e0.record()
        for _ in range(steps):
            call()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / steps
        path = hip.last_kernel_path()
        passes = 1 if path == "scores_mfma" else 2
        a = (passes * k_bytes + total * 4) / (ms * 1e-3) / 1e9
        res[label] = {"ms_per_step": ms, "kernels": path, "workspace_bytes": nbytes, "k_row_passes": passes,
                      "roofline": {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
                                   "traffic": None}}
        ws.free()
    dev.free()
    out.free()
    first = res["asked_workspace"]
    return {"workload": name, "ms_per_step": first["ms_per_step"], "dominant_kernel_ms": first["ms_per_step"], "steps": steps,
            "bytes": first["k_row_passes"] * k_bytes + total * 4, "roofline": first["roofline"], "by_workspace": res,
            "note": "algorithmic bytes: the K half of the attended cache once per pass of the kernels that ran, plus the output"}


def bench_sdpa_masked(hip, steps):
    """Configuration 2's shape with the causality spelt as an attention mask (an additive bf16 triangle of
    -inf shared by all heads, causal flag off), as converted models carry it: the flash kernel with the
    mask tile staged through LDS.  FLOPs are those of the full score matrix, which the kernel works
    through (it cannot know that half of the mask is -inf)."""
    from openvino_contrib_amd import workloads as W
    import numpy as np

    B, Hq, Hkv, L, D = 4, 32, 8, 2048, 128
    case = W.make_sdpa_case(2, B, Hq, Hkv, L, L, D, W.BF16, std=0.5)
    bufs = [hip.DeviceBuffer.from_numpy(case[n]) for n in ("q_store", "k_store", "v_store")]
    out = hip.DeviceBuffer(case["q_store"].nbytes)
    mask = hip.DeviceBuffer.from_numpy(W.to_storage(np.triu(np.full((L, L), -np.inf, np.float32), 1), W.BF16)[0])
    desc = hip.SdpaDesc(W.BF16, B, Hq, Hkv, L, L, D, 0, 0.0)
    call = lambda: hip.sdpa_masked(desc, bufs[0], bufs[1], bufs[2], W.BF16, [0, 0, L, 1], mask, out)
    e0, e1 = hip.Event(), hip.Event()
    for _ in range(300):  # clock ramp
        call()
    e0.record()
    for _ in range(steps):
        call()
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_ms(e1) / steps
    path = hip.last_kernel_path()
    flops = 4.0 * B * Hq * L * L * D
    a = flops / (ms * 1e-3) / 1e12
    for b in bufs + [out, mask]:
        b.free()
    return {"workload": "SDPA bf16 B=4 Hq=32 Hkv=8 L=2048 D=128, causal flag off, additive bf16 mask [1,1,L,L]", "kernel_path": path,
            "ms_per_step": ms, "dominant_kernel_ms": ms, "flops": flops, "tflops": a,
            "roofline": {"bound": "mfma", "achieved": a, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": a / MFMA_BF16_PEAK_TFLOPS,
                         "traffic": None, "kernel": "sdpa_flash_masked_kernel"}}


def bench_paged_through_plugin(hip, case, steps, warmup):
    """The same step through the plugin layer: Plugin -> CompiledModel -> InferRequest::infer ->
    PagedAttentionOp -> C ABI, every tensor device-resident (remote tensors over the buffers of the raw
    measurement, the output included), the scalar inputs on the host.  Host wall time per infer():
    each call enqueues the operator on the worker's stream and waits for it, as OpenVINO's synchronous
    infer does, so this is launch + execution + synchronisation, not a pipelined rate."""
    from openvino_contrib_amd import device_case as H
    from openvino_contrib_amd import plugin_capi as P
    import numpy as np

    dev = H.PagedDeviceCase(hip, case)
    plugin = P.Plugin()
    compiled = plugin.compile_model(P.Model.paged_attention(case["q_dtype"], case["kv_dtype"], case["cache_dtype"],
                                                            case["Hq"], case["Hkv"], case["D"], case["block_size"]))
    req = compiled.create_infer_request()
    T, S = case["T"], case["S"]
    row = case["key_cache"].shape[3] // hip.DTYPE_BYTES[case["cache_dtype"]]
    cache_shape = list(case["key_cache"].shape[:3]) + [row]
    req.set_device_input(0, dev.q.ptr, case["q_dtype"], [T, case["Hq"] * case["D"]])
    req.set_device_input(1, dev.k_new.ptr, case["kv_dtype"], [T, case["Hkv"] * case["D"]])
    req.set_device_input(2, dev.v_new.ptr, case["kv_dtype"], [T, case["Hkv"] * case["D"]])
    req.set_device_input(3, dev.key_cache.ptr, case["cache_dtype"], cache_shape)
    req.set_device_input(4, dev.value_cache.ptr, case["cache_dtype"], cache_shape)
    req.set_device_input(5, dev.past_lens.ptr, P.I32, [S])
    req.set_device_input(6, dev.subsequence_begins.ptr, P.I32, [S + 1])
    req.set_device_input(7, dev.block_indices.ptr, P.I32, [len(case["block_indices"])])
    req.set_device_input(8, dev.block_indices_begins.ptr, P.I32, [S + 1])
    req.set_input(9, np.zeros((0,), np.float32), P.F32)
    req.set_input(10, np.array([case["sliding_window"]], np.int32), P.I32)
    req.set_input(11, np.zeros((0,), np.float32), P.F32)
    req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
    req.set_device_output(0, dev.out.ptr, case["q_dtype"], [T, case["Hq"] * case["D"]])
    for _ in range(max(warmup, 20)):
        req.infer()
    t0 = time.perf_counter()
    for _ in range(steps):
        req.infer()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    del req, compiled, plugin
    dev.free()
    return ms


def bench_sdpa(hip, case, steps, warmup, name):
    from openvino_contrib_amd import workloads as W

    desc = hip.SdpaDesc(case["dtype"], case["B"], case["Hq"], case["Hkv"], case["Lq"], case["Lk"], case["D"], 1, 0.0)
    q = hip.DeviceBuffer.from_numpy(case["q_store"])
    k = hip.DeviceBuffer.from_numpy(case["k_store"])
    v = hip.DeviceBuffer.from_numpy(case["v_store"])
    out = hip.DeviceBuffer(case["q_store"].nbytes)

    def step(_):
        hip.sdpa(desc, q, k, v, out)

    ms, wall_ms, kern_ms = time_steps(hip, step, steps, warmup)
    flops = W.sdpa_flops(case["B"], case["Hq"], case["Lq"], case["Lk"], case["D"], True)
    res = {"workload": name, "kernel_path": hip.last_kernel_path(), "ms_per_step": ms, "host_ms_per_step": wall_ms,
           "dominant_kernel_ms": kern_ms, "flops": flops, "tflops": flops / (ms * 1e-3) / 1e12}
    for b in (q, k, v, out):
        b.free()
    return res


# HBM bytes per launch of the dominant kernel.  Hardware counters cannot be read from inside this
# process, so these are RECORDED figures: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB per dispatch from
# rocprofv3 --pmc runs of this script on the default seeds (scale factors from a plain 1 GiB copy,
# profiles/copy_calibration.txt); the file each pair of numbers was read from is named beside it.
RECORDED_TRAFFIC = {
    "c3": ((563582.6 * 2.0 + 3258.4) * 1024, "profiles/paged_decode_kernel_config3_fp16.txt"),
    "c4": ((1225872.7 * 2.0 + 12671.2) * 1024, "profiles/paged_decode_kernel_config4_u8.txt"),
    "c2": ((49302.7 * 2.0 + 65536.0) * 1024, "profiles/sdpa_flash_kernel_config2_bf16.txt"),
    "c5": ((786147.1 * 2.0 + 6318.8) * 1024, "profiles/paged_attention_config5_mixed.txt"),  # the decode kernel of the mixed step
}


def recorded_traffic(w):
    t = RECORDED_TRAFFIC.get(w)
    return (t[0], "recorded, not measured in this run: " + t[1]) if t else (None, None)


def roofline_hbm(res, w):
    a = res["decode_kv_bytes"] / (res["dominant_kernel_ms"] * 1e-3) / 1e9
    traffic, source = recorded_traffic(w)
    return {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
            "traffic": traffic, "traffic_source": source, "kernel": "paged_decode_kernel"}


def roofline_mfma(res):
    a = res["flops"] / (res["dominant_kernel_ms"] * 1e-3) / 1e12
    traffic, source = recorded_traffic("c2")
    return {"bound": "mfma", "achieved": a, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": a / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic, "traffic_source": source,
            "kernel": "sdpa_flash_kernel"}


def oracle_kind():
    """Which CPU implementation stands beside the GPU figure.  The reference's natural one is
    OpenVINO's CPU plugin running the same single-operator model; it is used only where OpenVINO is
    installed, which is probed here and said in the record either way."""
    import importlib.util

    if importlib.util.find_spec("openvino") is None:
        return "restatement (openvino is not importable on this machine)"
    try:
        import openvino

        version = getattr(openvino, "__version__", "unknown version")
    except Exception as e:  # an installation that does not load is as good as none
        return "restatement (openvino found but failed to import: %s)" % type(e).__name__
    return "restatement (OpenVINO %s is importable; running the single-operator model on its CPU plugin is not wired up)" % version


def cpu_baseline_paged(case, budget_s=12.0):
    """Oracle (port, OpenMP over sequences x kv heads) on the whole batch, attention only,
    repeated until about budget_s seconds of CPU work have been spent."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    from openvino_contrib_amd import workloads as W

    kc, vc = case["key_cache"], case["value_cache"]
    times = []
    t_begin = time.perf_counter()
    while not times or (time.perf_counter() - t_begin < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        O.paged_attention(case["q"], case["k_new"], case["v_new"], kc, vc, case["cache_dtype"], case["past_lens"],
                          case["subsequence_begins"], case["block_indices"], case["block_indices_begins"],
                          case["Hq"], case["Hkv"], case["D"], case["block_size"],
                          sliding_window=case["sliding_window"], do_write=False)
        times.append(time.perf_counter() - t0)
    mean = sum(times) / len(times)
    return {"value": W.paged_kv_bytes(case) / mean / 1e9, "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
            "oracle": oracle_kind(),
            "sample": "all %d sequences, attention only, %d passes, %.1f s" % (case["S"], len(times), sum(times))}


def cpu_baseline_sdpa(case, budget_s=20.0):
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    from openvino_contrib_amd import workloads as W

    G = case["Hq"] // case["Hkv"]
    times = []
    t_begin = time.perf_counter()
    n = 0
    while not times or (time.perf_counter() - t_begin < budget_s and n < case["B"] * case["Hkv"]):
        b, hkv = divmod(n, case["Hkv"])
        t0 = time.perf_counter()
        O.sdpa(case["q"][b:b + 1, hkv * G:(hkv + 1) * G], case["k"][b:b + 1, hkv:hkv + 1],
               case["v"][b:b + 1, hkv:hkv + 1], causal=True)
        times.append(time.perf_counter() - t0)
        n += 1
    fl = W.sdpa_flops(1, G, case["Lq"], case["Lk"], case["D"], True) * len(times)
    return {"value": fl / sum(times) / 1e12, "unit": "TFLOP/s", "cores": O.num_threads(), "kind": "port",
            "oracle": oracle_kind(),
            "sample": "%d of %d (batch, kv head) groups, %.1f s" % (len(times), case["B"] * case["Hkv"], sum(times))}


def bench_layer_ops(hip, steps, warmup, with_cpu):
    """The operators around attention (libhipops.so) at the shapes of a decoder layer that feeds
    configuration 2 (8,192 tokens, hidden 4,096, 32 query and 8 kv heads of 128) and of a 64-token
    decode step.  Each operator is one kernel; its duration is the mean of `steps` back-to-back
    launches between two events.  Rooflines: algorithmic bytes (every input and output byte once)
    against 8 TB/s, or 2*m*n*k against the dense bf16 MFMA peak."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    from openvino_contrib_amd import ops_capi as ops
    from openvino_contrib_amd import workloads as W

    ops.lib()
    rng = np.random.default_rng(2024)
    T, hidden, Hq, Hkv, D, vocab = 8192, 4096, 32, 8, 128, 32000
    BF16 = W.BF16

    def dev(shape, scale=1.0):
        st, exact = W.to_storage((rng.standard_normal(shape) * scale).astype(np.float32), BF16)
        return hip.DeviceBuffer.from_numpy(st), exact

    def timed(fn):
        e0, e1 = hip.Event(), hip.Event()
        ramped = 0.0
        while ramped < CLOCK_RAMP_MS / 2:  # idle clocks, as in time_steps
            e0.record()
            for _ in range(64):
                fn()
            e1.record()
            e1.synchronize()
            ramped += e0.elapsed_ms(e1)
        for _ in range(max(warmup, 3)):
            fn()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / steps
        e0.close()
        e1.close()
        return ms

    def cpu_time(fn, budget_s=2.0):
        times, t_begin = [], time.perf_counter()
        while not times or (time.perf_counter() - t_begin < budget_s and len(times) < 50):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sum(times) / len(times), len(times)

    # HBM bytes per launch from rocprofv3 FETCH_SIZE x 2 KiB + WRITE_SIZE x 1 KiB (recorded, not measured in this run)
    source = "recorded, not measured in this run: profiles/layer_ops_bf16.txt"
    recorded = {"rms_norm_vec_kernel": (32888.8 * 2 + 65536.0) * 1024, "rope_vec_kernel": (36550.8 * 2 + 65536.0) * 1024,
                "gather_kernel": (32508.4 * 2 + 65536.0) * 1024, "concat_kernel": (32787.9 * 2 + 65536.0) * 1024,
                "transpose_rows_kernel": (32783.3 * 2 + 65536.0) * 1024, "transpose_tiles_kernel": (32796.0 * 2 + 65536.0) * 1024,
                "convert_kernel": (262155.5 * 2 + 262144.0) * 1024,
                "matmul_prefill": (320733.2 * 2 + 98347.4) * 1024, "matmul_decode": (29104.8 * 2 + 5385.0) * 1024}

    def hbm(name, ms, nbytes, kernel):
        a = nbytes / (ms * 1e-3) / 1e9
        return {"workload": name, "ms_per_step": ms, "dominant_kernel_ms": ms, "bytes": nbytes,
                "roofline": {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
                             "traffic": recorded.get(kernel), "traffic_source": source if kernel in recorded else None,
                             "kernel": kernel}}

    out = {}
    import oracle as O
    sample = 256  # rows of the CPU samples

    # RMS norm
    dx, x = dev((T, hidden))
    dg, g = dev((hidden,))
    do = hip.DeviceBuffer(T * hidden * 2)
    ms = timed(lambda: ops.rms_norm(dx, dg, do, T, hidden, 1e-5, BF16, BF16, BF16))
    out["rms"] = hbm("RMS norm, %d x %d bf16" % (T, hidden), ms, 2 * T * hidden * 2 + hidden * 2, "rms_norm_vec_kernel")
    if with_cpu:
        t, n = cpu_time(lambda: O.rms_norm(x[:sample], g, 1e-5))
        out["rms"]["cpu_baseline"] = {"value": (2 * sample * hidden * 4) / t / 1e9, "unit": "GB/s", "cores": O.num_threads(),
                                      "kind": "port", "sample": "oracle (fp32) on %d of %d rows, mean of %d passes" % (sample, T, n)}

    # RoPE on the query heads
    pos = hip.DeviceBuffer.from_numpy(np.arange(T, dtype=np.int32) % 2048)
    inv = 10000.0 ** (-np.arange(0, D, 2) / D)
    ang = np.arange(2048)[:, None] * inv[None, :]
    cos, sin = np.cos(np.tile(ang, 2)).astype(np.float32), np.sin(np.tile(ang, 2)).astype(np.float32)
    dc, ds = hip.DeviceBuffer.from_numpy(cos), hip.DeviceBuffer.from_numpy(sin)
    dq, q = dev((T, Hq, D))
    dqo = hip.DeviceBuffer(T * Hq * D * 2)
    rd = ops.RopeDesc(BF16, W.F32, T, Hq, D, D, 0, Hq * D, D, Hq * D, D, 2048, D)
    ms = timed(lambda: ops.rope(rd, dq, dc, ds, pos, dqo))
    out["rope"] = hbm("RoPE (rotate-half), %d tokens x %d heads x %d bf16, f32 tables" % (T, Hq, D), ms,
                      2 * T * Hq * D * 2 + 2 * 2048 * D * 4 + T * 4, "rope_vec_kernel")
    if with_cpu:
        p = (np.arange(sample) % 2048).astype(np.int32)
        t, n = cpu_time(lambda: O.rope(q[:sample], cos, sin, p))
        out["rope"]["cpu_baseline"] = {"value": (2 * sample * Hq * D * 4) / t / 1e9, "unit": "GB/s", "cores": O.num_threads(),
                                       "kind": "port", "sample": "oracle (fp32) on %d of %d tokens, mean of %d passes" % (sample, T, n)}

    # Gather: embedding lookup
    dt, table = dev((vocab, hidden))
    ids = rng.integers(0, vocab, T).astype(np.int32)
    dids = hip.DeviceBuffer.from_numpy(ids)
    ms = timed(lambda: ops.gather(dt, dids, do, 1, 1, vocab, hidden * 2, T, ops.I32))
    out["gather"] = hbm("Gather (embedding lookup), %d rows of %d bf16 from %d" % (T, hidden, vocab), ms,
                        2 * T * hidden * 2 + T * 4, "gather_kernel")
    if with_cpu:
        tb = np.ascontiguousarray(table[:, :]).astype(np.float32)
        t, n = cpu_time(lambda: O.gather(tb, ids[:sample], 0))
        out["gather"]["cpu_baseline"] = {"value": (2 * sample * hidden * 4) / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                         "sample": "oracle (fp32 rows, one thread) on %d of %d indices, mean of %d passes" % (sample, T, n)}
        del tb
    dt.free()

    # Concat of two halves along the last axis
    da, _ = dev((T, hidden // 2))
    db, _ = dev((T, hidden // 2))
    ms = timed(lambda: ops.concat([da, db], [hidden, hidden], T, do))
    out["concat"] = hbm("Concat of two [%d, %d] bf16 along the last axis" % (T, hidden // 2), ms, 2 * T * hidden * 2, "concat_kernel")

    # gated MLP: GLU over the fused gate|up projection (width 14,336) and the unfused Swish and Multiply
    ffn, Tm = 14336, 2048
    dgu, gu = dev((Tm, 2 * ffn))
    dmo = hip.DeviceBuffer(Tm * ffn * 2)
    ms = timed(lambda: ops.glu(dgu, dmo, Tm, ffn, BF16))
    out["glu"] = hbm("GLU (Swish), [%d, 2 x %d] bf16" % (Tm, ffn), ms, 3 * Tm * ffn * 2, "eltwise_vec_kernel(glu)")
    if with_cpu:
        t, n = cpu_time(lambda: O.glu(gu[:sample], 0, True))
        out["glu"]["cpu_baseline"] = {"value": (3 * sample * ffn * 4) / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                      "sample": "oracle (fp32, one thread) on %d of %d rows, mean of %d passes" % (sample, Tm, n)}
    ms = timed(lambda: ops.swish(dgu, dmo, Tm * ffn, BF16))
    out["swish"] = hbm("Swish, %d x %d bf16" % (Tm, ffn), ms, 2 * Tm * ffn * 2, "eltwise_vec_kernel(swish)")
    ms = timed(lambda: ops.multiply(dgu, dx, dmo, Tm * ffn, BF16))
    out["multiply"] = hbm("Multiply, %d x %d bf16" % (Tm, ffn), ms, 3 * Tm * ffn * 2, "eltwise_vec_kernel(multiply)")
    dgu.free()
    dmo.free()

    # Transpose [tokens, heads, size] -> [heads, tokens, size] (runs of 256 bytes move whole), the K^T form whose
    # innermost axis changes (tiles through LDS), and Convert f32 -> bf16
    dqt = hip.DeviceBuffer(T * Hq * D * 2)
    ms = timed(lambda: ops.transpose(dq, dqt, (T, Hq, D), (1, 0, 2), 2))
    out["transpose_rows"] = hbm("Transpose [%d, %d, %d] bf16 -> heads first" % (T, Hq, D), ms, 2 * T * Hq * D * 2, "transpose_rows_kernel")
    ms = timed(lambda: ops.transpose(dq, dqt, (Hq, T, D), (0, 2, 1), 2))
    out["transpose_tiles"] = hbm("Transpose [%d, %d, %d] bf16 -> [%d, %d, %d]" % (Hq, T, D, Hq, D, T), ms, 2 * T * Hq * D * 2, "transpose_tiles_kernel")
    if with_cpu:
        t, n = cpu_time(lambda: O.transpose(q[:sample], (1, 0, 2)))
        out["transpose_rows"]["cpu_baseline"] = {"value": (2 * sample * Hq * D * 4) / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                                 "sample": "oracle (fp32 elements, one thread) on %d of %d tokens, mean of %d passes" % (sample, T, n)}
    Tc = 4 * T  # 805 MB in and out: more than the 256 MB last-level cache holds from one launch to the next
    df32 = hip.DeviceBuffer(Tc * hidden * 4)
    dbf = hip.DeviceBuffer(Tc * hidden * 2)
    df32.fill(0)
    ms = timed(lambda: ops.convert(df32, dbf, Tc * hidden, 0, 2))
    out["convert"] = hbm("Convert f32 -> bf16, %d x %d" % (Tc, hidden), ms, Tc * hidden * 6, "convert_kernel")
    if with_cpu:
        xs = np.ascontiguousarray(x[:sample])
        t, n = cpu_time(lambda: O.convert(xs, 0, 2))
        out["convert"]["cpu_baseline"] = {"value": (sample * hidden * 6) / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                          "sample": "oracle (one thread) on %d of %d rows, mean of %d passes" % (sample, Tc, n)}
    dqt.free()
    df32.free()
    dbf.free()

    # the decomposed form of attention: mask added to the scores of 32 heads (broadcast over the heads), softmax over the keys
    Hs, Ls = 32, 2048
    dsc, _ = dev((Hs, Ls, Ls))
    dmask, _ = dev((1, Ls, Ls))
    dso = hip.DeviceBuffer(Hs * Ls * Ls * 2)
    ms = timed(lambda: ops.binary(ops.ADD, dsc, dmask, dso, (Hs, Ls, Ls), (Hs, Ls, Ls), (1, Ls, Ls), BF16))
    out["add_broadcast"] = hbm("Add [%d, %d, %d] + [1, %d, %d] bf16" % (Hs, Ls, Ls, Ls, Ls), ms, (2 * Hs + 1) * Ls * Ls * 2, "binary_kernel")
    ms = timed(lambda: ops.softmax(dsc, dso, Hs * Ls, Ls, 1, BF16))
    out["softmax"] = hbm("Softmax over the last axis of [%d, %d, %d] bf16" % (Hs, Ls, Ls), ms, 2 * Hs * Ls * Ls * 2, "softmax_rows_kernel")
    if with_cpu:
        xs = np.ascontiguousarray(x[:sample, :Ls])
        t, n = cpu_time(lambda: O.softmax(xs, -1))
        out["softmax"]["cpu_baseline"] = {"value": (2 * sample * Ls * 4) / t / 1e9, "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
                                          "sample": "oracle (fp32 in, fp64 arithmetic) on %d rows of %d, mean of %d passes" % (sample, Ls, n)}
    for b in (dsc, dmask, dso):
        b.free()

    # MatMul: fused q|k|v projection of a prefill batch (MFMA-bound) and of a decode step (HBM-bound)
    N = (Hq + 2 * Hkv) * D
    dw, w = dev((N, hidden), 1.0 / 64)
    for name, m in (("matmul_prefill", T), ("matmul_decode", 64)):
        dc_out = hip.DeviceBuffer(m * N * 2)
        md = ops.MatmulDesc(BF16, BF16, m, N, hidden, 1, 0, 1, 0, 0)
        ws = hip.DeviceBuffer(ops.matmul_workspace_size(md))
        ms = timed(lambda: ops.matmul(md, dx, dw, dc_out, ws))
        flops = 2.0 * m * N * hidden
        nbytes = (m * hidden + N * hidden + m * N) * 2
        r = {"workload": "MatMul x[%d,%d] w[%d,%d]^T bf16 (q|k|v projection), hipBLASLt" % (m, hidden, N, hidden),
             "ms_per_step": ms, "dominant_kernel_ms": ms, "flops": flops, "bytes": nbytes, "tflops": flops / (ms * 1e-3) / 1e12}
        t_mfma, t_hbm = flops / (MFMA_BF16_PEAK_TFLOPS * 1e12), nbytes / (HBM_PEAK_GBS * 1e9)
        if t_mfma >= t_hbm:
            a = flops / (ms * 1e-3) / 1e12
            r["roofline"] = {"bound": "mfma", "achieved": a, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": a / MFMA_BF16_PEAK_TFLOPS, "traffic": recorded[name], "traffic_source": source,
                             "kernel": "hipBLASLt GEMM"}
        else:
            a = nbytes / (ms * 1e-3) / 1e9
            r["roofline"] = {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
                             "traffic": recorded[name], "traffic_source": source, "kernel": "hipBLASLt GEMM"}
        if with_cpu:
            rows = min(m, 16)
            t, n = cpu_time(lambda: O.matmul(x[:rows], w, False, True), 3.0)
            r["cpu_baseline"] = {"value": 2.0 * rows * N * hidden / t / 1e12, "unit": "TFLOP/s", "cores": O.num_threads(),
                                 "kind": "port", "sample": "oracle (fp64 accumulation) on %d of %d rows, mean of %d passes" % (rows, m, n)}
        out[name] = r
        dc_out.free()
        ws.free()
    for k, r in out.items():
        log("%s: %.4f ms, roofline frac %.3f (%s)" % (k, r["ms_per_step"], r["roofline"]["frac"], r["roofline"]["bound"]))
    return out


def bench_other_shapes(hip, steps, warmup):
    """config 3's and config 5's batches at the other cache shapes of the matrix-core decode kernel and, at
    head size 96 on blocks of 8, through the query-tile kernel that takes every other 16-bit shape; config 2's
    shape at head size 96.  Not reference configurations; no byte counters recorded for them."""
    from openvino_contrib_amd import workloads as W

    results = {}
    for D, bs in ((64, 32), (64, 16), (128, 16), (128, 64), (96, 16), (96, 64), (96, 8), (256, 16), (256, 128)):
        key = "c3_d%d_blk%d" % (D, bs)
        case = W.config3(head_dim=D, block_size=bs)
        r = bench_paged(hip, case, steps, warmup, "config3's batch with head size %d and cache blocks of %d tokens" % (D, bs))
        r["roofline"] = roofline_hbm(r, key)
        if r["kernel_path"] == "paged_mfma_tiles":
            r["roofline"]["kernel"] = "paged_tiles_kernel"
        log("%s: %.3f ms/step, dominant kernel %.3f ms, roofline frac %.3f (%s)"
            % (key, r["ms_per_step"], r["dominant_kernel_ms"], r["roofline"]["frac"], r["kernel_path"]))
        results[key] = r
        del case
    for key, kw in (("c4_blk16", {"block_size": 16}), ("c4_d64_blk32", {"head_dim": 64}),
                    ("c4_d256_blk16_s64", {"head_dim": 256, "block_size": 16, "S": 64})):
        case = W.config4(**kw)
        r = bench_paged(hip, case, steps, warmup, "config4's batch (u8 cache%s) with head size %d and cache blocks of %d tokens"
                        % (", its first 64 sequences' lengths" if "S" in kw else "", case["D"], case["block_size"]))
        r["roofline"] = roofline_hbm(r, key)
        log("%s: %.3f ms/step, dominant kernel %.3f ms, roofline frac %.3f (%s)"
            % (key, r["ms_per_step"], r["dominant_kernel_ms"], r["roofline"]["frac"], r["kernel_path"]))
        results[key] = r
        del case
    for key, kw, what in (("c5_blk16", {"block_size": 16}, "on cache blocks of 16 tokens"),
                          ("c5_d64_blk16", {"block_size": 16, "head_dim": 64}, "with head size 64 on cache blocks of 16 tokens"),
                          ("c5_d96_blk16", {"block_size": 16, "head_dim": 96}, "with head size 96 on cache blocks of 16 tokens")):
        case = W.config5(**kw)
        r = bench_paged(hip, case, steps, warmup, "config5's batch " + what)
        log("%s: %.3f ms/step (%s)" % (key, r["ms_per_step"], r["kernel_path"]))
        results[key] = r
        del case
    case = W.config2(D=96)
    r = bench_sdpa(hip, case, steps, warmup, "config2's shape at head size 96 (the tuned head-128 kernel on rows of 96 columns)")
    r["roofline"] = roofline_mfma(r)
    r["roofline"]["traffic"], r["roofline"]["traffic_source"], r["roofline"]["kernel"] = None, None, "sdpa_flash_padded_kernel"
    log("c2_d96: %.3f ms/step, roofline frac %.3f (%s)" % (r["ms_per_step"], r["roofline"]["frac"], r["kernel_path"]))
    results["c2_d96"] = r
    return results


def bench_multi_query(hip, steps, warmup):
    """config 3's sequences (64 decode rows, contexts U[512,8192], head size 128, blocks of 32) with more than 16 query
    heads per kv head -- the stream-K kernel enters a kv head once per group of 8..16 heads, so its K/V rows are read
    once per group -- and with fp16 queries on a bf16 cache (fp16 operands, blocks converted in registers).  Bytes
    counted are the cache rows once, as everywhere."""
    import numpy as np
    from openvino_contrib_amd import workloads as W

    rng = np.random.Generator(np.random.PCG64(1003))
    seqs = [(int(c) - 1, 1) for c in rng.integers(512, 8193, size=64)]
    results = {}
    for key, Hq, Hkv, qd, cache in (("mq_48_1_f16", 48, 1, W.F16, W.F16), ("mq_32_1_f16", 32, 1, W.F16, W.F16),
                                    ("mq_64_2_u8", 64, 2, W.F16, W.U8), ("mq_40_2_f16", 40, 2, W.F16, W.F16),
                                    ("f16q_bf16cache_32_8", 32, 8, W.F16, W.BF16), ("bf16q_bf16cache_32_8", 32, 8, W.BF16, W.BF16)):
        case = W.make_paged_case(101003, seqs, Hq, Hkv, 128, 32, qd, qd, cache)
        r = bench_paged(hip, case, steps, warmup, "config3's sequences with %d query heads on %d kv heads, q dtype %d, cache dtype %d" % (Hq, Hkv, qd, cache))
        r["roofline"] = roofline_hbm(r, key)
        log("%s: %.3f ms/step, dominant kernel %.3f ms, roofline frac %.3f (%s)"
            % (key, r["ms_per_step"], r["dominant_kernel_ms"], r["roofline"]["frac"], r["kernel_path"]))
        results[key] = r
        del case
    return results


def bench_kv_cache_writer(hip, steps, warmup):
    """hipattn_kv_cache_write alone on a prefill-sized batch: 32 sequences x 4,096 new tokens, 8 kv heads x 128, fp16 rows
    into an fp16, a bf16 and a u8 cache (about 1 GB per call: several times the 256 MB of the last-level cache, so that a
    call does not find the previous call's lines there).  Bytes per call: the new K and V rows read once, their cache
    rows written once."""
    from openvino_contrib_amd import device_case as H
    from openvino_contrib_amd import workloads as W
    out = {}
    for cache_dtype, name in ((W.F16, "writer_f16_cache"), (W.BF16, "writer_bf16_cache"), (W.U8, "writer_u8_cache")):
        case = W.make_paged_case(77, [(0, 4096)] * 32, 8, 8, 128, 32, W.F16, W.F16, cache_dtype)
        dev = H.PagedDeviceCase(hip, case)
        desc = H.pa_desc(hip, case)

        def step(_):
            hip.kv_cache_write(desc, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache, dev.past_lens,
                               dev.subsequence_begins, dev.block_indices, dev.block_indices_begins)

        for i in range(warmup + 100):  # (the clock ramp as well)
            step(i)
        e0, e1 = hip.Event(), hip.Event()
        e0.record()
        for i in range(steps):
            step(i)
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / steps
        e0.close()
        e1.close()
        rows = case["T"] * case["Hkv"] * 2
        nbytes = rows * (128 * 2 + W.cache_row_bytes(cache_dtype, 128))
        gbs = nbytes / (ms * 1e-3) / 1e9
        out[name] = {"workload": name, "ms_per_step": ms, "bytes": nbytes, "gb_per_s": gbs,
                     "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                                  "traffic": None, "kernel": "kv_cache_write_kernel"}}
        log("%s: %.4f ms per call, %.0f MB, %.0f GB/s (%.2f of the HBM peak)" % (name, ms, nbytes / 1e6, gbs, gbs / HBM_PEAK_GBS))
        dev.free()
    return out


def bench_stream_reader(hip):
    """What N compute units stream when each runs one workgroup that only reads (stream_yardstick.hip): alone, and
    launched just ahead of config 5's chunk sequences (the flash kernel over the block table, which then has the
    other compute units), as the decode kernel of a mixed batch is."""
    import ctypes
    from openvino_contrib_amd import build as hip_build
    from openvino_contrib_amd import device_case as H
    from openvino_contrib_amd import workloads as W
    if not os.path.exists(hip_build.YARDSTICK_LIB_PATH):
        sys.exit("bench.py: %s is missing (python -m openvino_contrib_amd.build)" % hip_build.YARDSTICK_LIB_PATH)
    yard = ctypes.CDLL(hip_build.YARDSTICK_LIB_PATH)
    yard.stream_yardstick_launch.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.POINTER(ctypes.c_longlong)]
    total = 2 << 30
    buf, sink = hip.DeviceBuffer(total), hip.DeviceBuffer(256)
    buf.fill(3)
    side, main = hip.Stream(), hip.Stream()
    case = W.config5(n_decode=0)
    dev = H.PagedDeviceCase(hip, case)
    desc = H.pa_desc(hip, case, flags=hip.PA_SKIP_CACHE_WRITE)
    ws = hip.DeviceBuffer(hip.paged_attention_workspace_size(desc))

    def chunks():
        hip.paged_attention(desc, dev.q, dev.k_new, dev.v_new, dev.key_cache, dev.value_cache, dev.past_lens,
                            dev.subsequence_begins, dev.block_indices, dev.block_indices_begins, dev.out, ws, stream=main)

    def timed(workgroups, beside):
        best, chunk_ms = None, None
        for _ in range(5):
            r0, r1, c0, c1 = hip.Event(), hip.Event(), hip.Event(), hip.Event()
            nread = ctypes.c_longlong()
            r0.record(side)
            rc = yard.stream_yardstick_launch(buf.ptr, total, workgroups, sink.ptr, side.handle, ctypes.byref(nread))
            if rc != 0:
                sys.exit("bench.py: stream_yardstick_launch failed with HIP error %d" % rc)
            r1.record(side)
            if beside:
                c0.record(main)
                chunks()
                c1.record(main)
            r1.synchronize()
            main.synchronize()
            ms = r0.elapsed_ms(r1)
            if best is None or ms < best:
                best, chunk_ms = ms, (c0.elapsed_ms(c1) if beside else None)
            for e in (r0, r1, c0, c1):
                e.close()
        gbs = nread.value / (best * 1e-3) / 1e9
        return {"workgroups": workgroups, "reader_gb_per_s": _r(gbs), "per_cu_gb_per_s": _r(gbs / workgroups), "frac_of_hbm_peak": _r(gbs / HBM_PEAK_GBS),
                "chunks_ms_beside": None if chunk_ms is None else _r(chunk_ms)}

    for _ in range(40):  # clock ramp
        chunks()
    main.synchronize()
    c0, c1 = hip.Event(), hip.Event()
    c0.record(main)
    for _ in range(20):
        chunks()
    c1.record(main)
    c1.synchronize()
    cus = hip.device_info(0).compute_units
    out = {"workload": "stream", "reader": "512 threads and all LDS of a compute unit per workgroup, 64 KB in flight per workgroup, 2 GiB read once",
           "chunks_alone_ms": _r(c0.elapsed_ms(c1) / 20),
           "alone": [timed(n, False) for n in (cus, cus // 2, 90, 64, 32)],
           "ahead_of_config5_chunks": [timed(n, True) for n in (90, 64)]}
    for r in out["alone"] + out["ahead_of_config5_chunks"]:
        log("reader on %3d compute units%s: %.0f GB/s, %.1f per compute unit" %
            (r["workgroups"], "" if r["chunks_ms_beside"] is None else " ahead of the chunks (%.3f ms)" % r["chunks_ms_beside"],
             r["reader_gb_per_s"], r["per_cu_gb_per_s"]))
    return out


def bench_decoder_layer(hip, steps, warmup):
    """One decoder layer of LLaMA-3-8B's shape (hidden 4096, 32 query / 8 kv heads of 128, MLP 14336) on
    configuration 3's decode batch, as ONE compiled model through the plugin layer: RMS -> q/k/v MatMul ->
    RoPE -> PagedAttentionExtension -> o MatMul -> Add -> RMS -> gate|up MatMul -> GLU -> down MatMul ->
    Add, thirteen operators per infer() with every tensor device-resident (weights are bound as device
    inputs) and the recorded graph replayed.  The step has to read the layer's weights (bf16) and the batch's
    KV cache (fp16) once: that is the HBM roofline it is held against."""
    from openvino_contrib_amd import plugin_capi as P
    from openvino_contrib_amd import workloads as W
    import numpy as np

    hidden, Hq, Hkv, D, ffn, bs = 4096, 32, 8, 128, 14336, 32
    case = W.config3()
    T, S = case["T"], case["S"]
    rng = np.random.default_rng(7)
    g = P.GraphText("decoder_layer")
    names, arrays = [], {}

    def dev_param(name, dtype, array):
        arrays[name] = (hip.DeviceBuffer.from_numpy(np.ascontiguousarray(array)), dtype, list(array.shape))
        return g.parameter(name, dtype, list(array.shape))

    def weight(name, rows, cols):
        return dev_param(name, W.BF16, W.to_storage((rng.standard_normal((rows, cols), dtype=np.float32) / np.sqrt(cols)), W.BF16)[0])

    h = dev_param("hidden", W.BF16, W.to_storage(rng.standard_normal((T, hidden), dtype=np.float32), W.BF16)[0])
    positions = np.concatenate([np.arange(p, p + n) for p, n in zip(case["past_lens"], np.diff(case["subsequence_begins"]))]).astype(np.int32)
    half = np.arange(0, D, 2, dtype=np.float64) / D
    ang = np.arange(int(positions.max()) + 1, dtype=np.float64)[:, None] * (10000.0 ** -half)[None, :]
    cos_p = dev_param("cos", W.F32, np.concatenate([np.cos(ang), np.cos(ang)], 1).astype(np.float32))
    sin_p = dev_param("sin", W.F32, np.concatenate([np.sin(ang), np.sin(ang)], 1).astype(np.float32))
    pos_p = dev_param("positions", P.I32, positions)
    idx = [dev_param(n, P.I32, case[n]) for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")]
    scale_p = g.parameter("scale", W.F32, [-1])
    win_p = g.parameter("sliding_window", P.I32, [-1])
    alibi_p = g.parameter("alibi_slopes", W.F32, [0])
    mcl_p = g.parameter("max_context_len", P.I32, [-1])
    kc = dev_param("key_cache", W.F16, case["key_cache"].view(np.uint16))
    vc = dev_param("value_cache", W.F16, case["value_cache"].view(np.uint16))
    gamma = lambda name: g.constant(name, W.to_storage(1.0 + 0.1 * rng.standard_normal(hidden).astype(np.float32), W.BF16)[0], "bf16")
    mm = lambda name, x, wt: g.add("MatMul", name, [x, wt], transpose_a=False, transpose_b=True)
    n1 = g.add("RMS", "norm1", [h, gamma("g1")], epsilon=1e-5, output_type="dynamic")
    q = mm("q", n1, weight("wq", Hq * D, hidden))
    k = mm("k", n1, weight("wk", Hkv * D, hidden))
    v = mm("v", n1, weight("wv", Hkv * D, hidden))
    rope = dict(head_size=D, rotary_ndims=D, gather_position_arg_id=3)
    qr = g.add("RoPE", "q_rope", [q, cos_p, sin_p, pos_p], head_cnt=Hq, **rope)
    kr = g.add("RoPE", "k_rope", [k, cos_p, sin_p, pos_p], head_cnt=Hkv, **rope)
    pa = g.add("PagedAttentionExtension", "attention", [qr, kr, v, kc, vc] + idx + [scale_p, win_p, alibi_p, mcl_p])
    h1 = g.add("Add", "res1", [mm("o", pa, weight("wo", hidden, Hq * D)), h])
    n2 = g.add("RMS", "norm2", [h1, gamma("g2")], epsilon=1e-5, output_type="dynamic")
    gu = mm("gate_up", n2, weight("wgu", 2 * ffn, hidden))
    act = g.add("GLU", "glu", [gu], axis=-1, split_lengths=ffn, glu_type=0, split_to_glu_idx=0, output_type="dynamic")
    g.result("out", g.add("Add", "res2", [mm("down", act, weight("wd", hidden, ffn)), h1]))

    plugin = P.Plugin()
    compiled = plugin.compile_model(g.model())
    req = compiled.create_infer_request()
    host = {"scale": (np.zeros((0,), np.float32), W.F32), "sliding_window": (np.array([0], np.int32), P.I32),
            "alibi_slopes": (np.zeros((0,), np.float32), W.F32),
            "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32)}
    for i, n in enumerate(compiled.input_names()):
        if n in host:
            req.set_input(i, *host[n])
        else:
            buf, dtype, shape = arrays[n]
            req.set_device_input(i, buf.ptr, dtype, shape)
    out = hip.DeviceBuffer(T * hidden * 2)
    req.set_device_output(0, out.ptr, W.BF16, [T, hidden])
    for _ in range(max(warmup, 30)):
        req.infer()
    t0 = time.perf_counter()
    for _ in range(steps):
        req.infer()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    graphs, launches = int(compiled.get_property("HIP_NUMBER_OF_GRAPHS")), int(compiled.get_property("HIP_GRAPH_LAUNCHES"))
    weight_bytes = 2 * (hidden * (Hq + 2 * Hkv) * D + hidden * Hq * D + 3 * hidden * ffn)
    kv_bytes = W.paged_kv_bytes(case)
    res = {"workload": "decoder layer (hidden 4096, 32/8 heads of 128, MLP 14336, bf16 weights, fp16 cache) on config3's "
                       "decode batch through InferRequest::infer; the same inputs every infer, so every infer after the "
                       "second replays the recorded graph (a serving loop replays as long as shapes and pointers stay)",
           "ms_per_step": ms, "weight_bytes": weight_bytes, "kv_bytes": kv_bytes, "operators": 13,
           "graphs": graphs, "graph_launches": launches,
           "roofline": {"bound": "hbm", "achieved": (weight_bytes + kv_bytes) / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                        "unit": "GB/s", "frac": (weight_bytes + kv_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                        "note": "host wall time per synchronous infer() over the bytes one step must read (weights + KV)"}}
    del req, compiled, plugin
    for buf, _, _ in arrays.values():
        buf.free()
    out.free()
    return res


def _r(x, digits=5):
    """Floats to `digits` significant digits: the compact line is for a reader, the detail file keeps everything."""
    return float("%.*g" % (digits, x)) if isinstance(x, float) else x


def compact_roofline(r):
    return {k: _r(r[k]) for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel") if k in r}


def compact_cpu(c):
    return {k: _r(c[k]) for k in ("value", "unit", "cores", "kind", "sample") if k in c}


def compact_workload(r):
    """What the last stdout line carries per configuration (the whole record goes to stderr and the detail file)."""
    out = {k: _r(r[k]) for k in ("ms_per_step", "dominant_kernel_ms", "kv_gbs", "tflops", "kernel_path", "ideal_ms",
                                 "frac_of_ideal", "plugin_ms_per_step") if k in r}
    if r.get("kernel_path", "").startswith("sdpa"):
        out.pop("kv_gbs", None)
    else:
        out.pop("tflops", None)
    out["roofline"] = compact_roofline(r["roofline"])
    if "cpu_baseline" in r:
        out["cpu_baseline"] = compact_cpu(r["cpu_baseline"])
    return out


def main():
    global CLOCK_RAMP_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5", "c5u8", "layer", "shapes", "mqa", "decoder", "scores", "masked", "copy", "mfma", "stream", "writer"],
                    help="copy = plain 1 GiB device copy and fill, the yardstick for hardware byte counters; "
                         "mfma = register-fed bf16 MFMAs only, the yardstick for the MFMA-bound kernels; "
                         "stream = a plain reader on a share of the compute units, alone and beside config 5's chunks; "
                         "writer = hipattn_kv_cache_write alone on a prefill-sized batch")
    ap.add_argument("--ramp-ms", type=float, default=CLOCK_RAMP_MS,
                    help="untimed GPU time of the step run ahead of the warmup steps (0 for hardware-counter runs, "
                         "which only count bytes)")
    ap.add_argument("--detail", default="", help="file for the full per-workload records (default: one line on stderr)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-extra", action="store_true", help="measure the headline workload only")
    ap.add_argument("--no-plugin", action="store_true", help="skip the timing through the plugin layer")
    args = ap.parse_args()
    CLOCK_RAMP_MS = args.ramp_ms
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)")

    from openvino_contrib_amd import capi as hip
    from openvino_contrib_amd import workloads as W

    hip.lib()
    if hip.device_count() < 1:
        sys.exit("bench.py: no HIP device")
    hip.check(hip.lib().hipattn_set_device(0))
    info = hip.device_info(0)
    dev_name = info.name.decode() or ("AMD " + info.arch.decode())
    log("device:", dev_name, info.arch.decode(), info.compute_units, "CUs")

    if args.workload == "mfma":
        # What the device sustains on v_mfma_f32_32x32x16_bf16 alone, and at which shader clock, with
        # random and with all-zero operands (the power an MFMA draws follows the bits that toggle).
        import ctypes
        from openvino_contrib_amd import build as hip_build
        if not os.path.exists(hip_build.YARDSTICK_LIB_PATH):
            sys.exit("bench.py: %s is missing (python -m openvino_contrib_amd.build)" % hip_build.YARDSTICK_LIB_PATH)
        yard = ctypes.CDLL(hip_build.YARDSTICK_LIB_PATH)
        out = {"workload": "mfma", "peak_tflops": MFMA_BF16_PEAK_TFLOPS}
        for name, zero in (("random_operands", 0), ("zero_operands", 1)):
            tf, ghz = ctypes.c_double(), ctypes.c_double()
            rc = yard.mfma_yardstick(zero, max(args.steps, 50), ctypes.byref(tf), ctypes.byref(ghz))
            if rc != 0:
                sys.exit("bench.py: mfma_yardstick failed with HIP error %d" % rc)
            out[name] = {"tflops": tf.value, "shader_ghz": ghz.value, "frac_of_peak": tf.value / MFMA_BF16_PEAK_TFLOPS}
        print(json.dumps(out))
        return

    if args.workload == "stream":
        print(json.dumps(bench_stream_reader(hip)))
        return

    if args.workload == "writer":
        print(json.dumps({"workload": "writer", "steps": args.steps, "warmup": args.warmup,
                          "workloads": bench_kv_cache_writer(hip, args.steps, args.warmup)}))
        return

    if args.workload == "layer":
        print(json.dumps({"workload": "layer", "steps": args.steps, "warmup": args.warmup,
                          "workloads": bench_layer_ops(hip, args.steps, args.warmup, not args.no_cpu)}))
        return

    if args.workload == "decoder":
        print(json.dumps({"workload": "decoder", "steps": args.steps, "warmup": args.warmup,
                          "workloads": {"decoder_layer": bench_decoder_layer(hip, args.steps, args.warmup)}}))
        return

    if args.workload == "mqa":
        print(json.dumps({"workload": "mqa", "steps": args.steps, "warmup": args.warmup, "workloads": bench_multi_query(hip, args.steps, args.warmup)}))
        return
    if args.workload == "shapes":
        print(json.dumps({"workload": "shapes", "steps": args.steps, "warmup": args.warmup,
                          "workloads": bench_other_shapes(hip, args.steps, args.warmup)}))
        return

    if args.workload == "scores":
        r = bench_paged_scores(hip, W.config3(), args.steps, "config3's batch: the scores output (all heads, the new token of every sequence)")
        print(json.dumps({"workload": "scores", "steps": args.steps, "workloads": {"c3_scores": r}}))
        return

    if args.workload == "masked":
        print(json.dumps({"workload": "masked", "steps": args.steps, "workloads": {"c2_masked": bench_sdpa_masked(hip, args.steps)}}))
        return

    if args.workload == "copy":
        # Known-size traffic for scaling FETCH_SIZE / WRITE_SIZE: a device-to-device copy of 1 GiB
        # (1 GiB read + 1 GiB written per launch) and a 1 GiB fill kernel (1 GiB written).
        n = 1 << 30
        src, dst = hip.DeviceBuffer(n), hip.DeviceBuffer(n)
        src.fill(1)
        dst.fill(2)
        hip.check(hip.lib().hipattn_stream_synchronize(None))
        e0, e1, e2 = hip.Event(), hip.Event(), hip.Event()
        e0.record()
        for _ in range(args.steps):
            hip.check(hip.lib().hipattn_memcpy_d2d_async(dst.ptr, src.ptr, n, None))
        e1.record()
        for _ in range(args.steps):
            dst.fill(3)
        e2.record()
        e2.synchronize()
        print(json.dumps({"workload": "copy", "bytes_per_launch": n, "launches_each": args.steps,
                          "d2d_copy_ms": e0.elapsed_ms(e1) / args.steps, "fill_ms": e1.elapsed_ms(e2) / args.steps}))
        return

    names = {"c2": "config2: bf16 causal prefill SDPA B4 Hq32 Hkv8 L2048 D128",
             "c3": "config3: fp16 paged decode, 64 seq x 1 token, ctx U[512,8192], blk 32, Hq32 Hkv8 D128",
             "c4": "config4: u8-KV paged decode, 128 seq, ctx U[1024,16384], Hq64 Hkv8 D128",
             "c5": "config5: 8x512 prefill chunks + 120 decode, window 4096, bf16 q, fp16 cache, Hq64 Hkv8 D128"}
    names["c5u8"] = "config5's batch on a u8 cache (not one of the reference configurations: the u8 load path of the prefill kernel)"
    makers = {"c2": W.config2, "c3": W.config3, "c4": W.config4, "c5": W.config5,
              "c5u8": lambda: W.config5(cache_dtype=W.U8)}
    order = [args.workload] + ([w for w in ("c3", "c2", "c4", "c5") if w != args.workload] if not args.no_extra else [])
    results, cpu = {}, {}
    for w in order:
        t0 = time.perf_counter()
        case = makers[w]()
        log("%s: inputs generated in %.1f s" % (w, time.perf_counter() - t0))
        if w == "c2":
            r = bench_sdpa(hip, case, args.steps, args.warmup, names[w])
            r["roofline"] = roofline_mfma(r)
        else:
            r = bench_paged(hip, case, args.steps, args.warmup, names[w])
            r["roofline"] = roofline_hbm(r, w)
            if w in ("c5", "c5u8"):
                t_ideal = max(r["kv_bytes"] / (HBM_PEAK_GBS * 1e9), r["flops"] / (MFMA_BF16_PEAK_TFLOPS * 1e12))
                r["ideal_ms"] = t_ideal * 1e3
                r["frac_of_ideal"] = t_ideal * 1e3 / r["ms_per_step"]
                r["roofline"]["note"] = ("mixed batch: the decode kernel runs beside the chunks' flash kernel on a share "
                                         "of the compute units, so its duration is not a whole-chip figure; "
                                         "frac_of_ideal is the one for this step")
        log("%s: %.3f ms/step, dominant kernel %.3f ms, roofline frac %.3f"
            % (w, r["ms_per_step"], r["dominant_kernel_ms"], r["roofline"]["frac"]))
        if w == args.workload and w != "c2" and not args.no_plugin:
            r["plugin_ms_per_step"] = bench_paged_through_plugin(hip, case, args.steps, args.warmup)
            r["plugin_overhead_ms"] = r["plugin_ms_per_step"] - r["ms_per_step"]
            log("%s through InferRequest::infer: %.3f ms/step (raw C ABI, back to back: %.3f)"
                % (w, r["plugin_ms_per_step"], r["ms_per_step"]))
        if not args.no_cpu:
            # the headline gets the larger budget; every other workload a bounded sample beside its figure
            budget = 12.0 if w == args.workload else 6.0
            c = cpu_baseline_sdpa(case, budget) if w == "c2" else cpu_baseline_paged(case, budget)
            r["cpu_baseline"] = c
            if w == args.workload:
                cpu = c
            log("%s cpu baseline:" % w, c)
        results[w] = r
        del case

    head = results[args.workload]
    is_sdpa = args.workload == "c2"
    line = {
        "metric": "prefill SDPA TFLOPS" if is_sdpa else "paged-attn decode KV GB/s",
        "value": head["tflops"] if is_sdpa else head["kv_gbs"],
        "unit": "TFLOP/s" if is_sdpa else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if is_sdpa else ("u8" if args.workload in ("c4", "c5u8") else "f16"),
        "data": "synthetic",
        "config": {"workload": head["workload"], "kernel_path": head["kernel_path"],
                   "device": dev_name, "arch": info.arch.decode(), "compute_units": info.compute_units,
                   "clock_ramp_ms": CLOCK_RAMP_MS},
        "roofline": compact_roofline(head["roofline"]),
        "cpu_baseline": compact_cpu(cpu) if cpu else None,
        "workloads": {k: compact_workload(v) for k, v in results.items()},
    }
    detail = dict(line, roofline=head["roofline"], cpu_baseline=cpu if cpu else None, workloads=results)
    if args.detail:
        with open(args.detail, "w") as f:
            json.dump(detail, f)
    else:
        log("detail:", json.dumps(detail))
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
