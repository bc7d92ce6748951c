"""The operators around attention through the plugin (compile_model on device "HIP", infer), each
against the CPU oracle, and then chained into the attention half of a decoder layer:
RMS -> q/k/v MatMul -> RoPE -> PagedAttentionExtension -> output MatMul -> residual Add."""
import numpy as np
import pytest

from openvino_contrib_amd import device_case as H
from openvino_contrib_amd import plugin_capi as P
from openvino_contrib_amd import workloads as W

pytestmark = pytest.mark.gpu

F32, F16, BF16 = W.F32, W.F16, W.BF16
ROUND = {F32: 2e-6, F16: 1e-3, BF16: 8e-3}


def scaled_error(got, ref):
    return float(np.max(np.abs(got - ref) / np.maximum(1.0, np.abs(ref))))


def run(compiled, inputs):
    """inputs: list of (array in storage form, dtype code)."""
    req = compiled.create_infer_request()
    for i, (a, dt) in enumerate(inputs):
        req.set_input(i, a, dt)
    req.infer()
    return req


def storage(x, dtype):
    st, exact = W.to_storage(np.asarray(x, np.float32), dtype)
    return st, exact


@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_rms_through_the_plugin(hip, oracle, dtype):
    rng = np.random.default_rng(1)
    g = P.GraphText("rms")
    x = g.parameter("x", dtype, [-1, -1, 256])
    gamma_st, gamma = storage(1.0 + 0.2 * rng.standard_normal(256), dtype)
    gm = g.constant("gamma", gamma_st, P._TYPE_NAMES[dtype])
    g.result("out", g.add("RMS", "norm", [x, gm], epsilon=1e-5, output_type="dynamic"))
    compiled = P.Plugin().compile_model(g.model())
    for shape in ((2, 5, 256), (1, 1, 256), (3, 0, 256)):
        x_st, xv = storage(rng.standard_normal(shape) * 3, dtype)
        out, _ = run(compiled, [(x_st, dtype)]).output(0)
        assert out.shape == shape
        if out.size:
            assert scaled_error(H.storage_to_f32(out, dtype), oracle.rms_norm(xv, gamma, 1e-5)) <= ROUND[dtype]


def rope_tables(rows, rot, base=10000.0):
    inv = base ** (-np.arange(0, rot, 2) / rot)
    ang = np.arange(rows)[:, None] * inv[None, :]
    return np.cos(np.tile(ang, 2)).astype(np.float32), np.sin(np.tile(ang, 2)).astype(np.float32)


@pytest.mark.parametrize("in_t,out_t", [(False, False), (True, False), (True, True), (False, True)])
def test_rope_rank4_layouts(hip, oracle, in_t, out_t):
    rng = np.random.default_rng(2)
    B, Hh, L, S = 2, 3, 7, 64
    g = P.GraphText("rope4")
    x = g.parameter("x", F16, [-1, -1, -1, S])
    c = g.parameter("cos", F32, [-1, S])
    s = g.parameter("sin", F32, [-1, S])
    g.result("out", g.add("RoPE", "rope", [x, c, s], input_trans0213=in_t, output_trans0213=out_t, rotary_ndims=S))
    compiled = P.Plugin().compile_model(g.model())
    cos, sin = rope_tables(L, S)
    xv = rng.standard_normal((B, Hh, L, S)).astype(np.float32)           # logical [batch, heads, length, size]
    x_st, xv = storage(xv, F16)
    feed = np.ascontiguousarray(x_st.transpose(0, 2, 1, 3)) if in_t else x_st
    out, _ = run(compiled, [(feed, F16), (cos, F32), (sin, F32)]).output(0)
    got = H.storage_to_f32(out, F16)
    if out_t:
        assert got.shape == (B, L, Hh, S)
        got = got.transpose(0, 2, 1, 3)
    ref = np.stack([oracle.rope(np.ascontiguousarray(xv[b].transpose(1, 0, 2)), cos, sin).transpose(1, 0, 2) for b in range(B)])
    assert got.shape == ref.shape and scaled_error(got, ref) <= 2 * ROUND[F16]


def test_rope_on_packed_tokens_with_positions(hip, oracle):
    """The layout in front of PagedAttentionExtension: [tokens, packed q|k|v], the k heads rotated in a slice."""
    rng = np.random.default_rng(3)
    T, Hq, Hkv, S, rot = 19, 4, 2, 128, 64
    packed = (Hq + 2 * Hkv) * S
    g = P.GraphText("rope2")
    x = g.parameter("qkv", BF16, [-1, packed])
    c = g.parameter("cos", BF16, [-1, rot])
    s = g.parameter("sin", BF16, [-1, rot])
    pos = g.parameter("positions", P.I32, [-1])
    g.result("k_rot", g.add("RoPE", "rope_k", [x, c, s, pos], slice_start=Hq * S, slice_stop=(Hq + Hkv) * S, head_cnt=Hkv,
                            head_size=S, rotary_ndims=rot, gather_position_arg_id=3))
    compiled = P.Plugin().compile_model(g.model())
    cos, sin = rope_tables(500, rot)
    cos_st, cos = storage(cos, BF16)
    sin_st, sin = storage(sin, BF16)
    x_st, xv = storage(rng.standard_normal((T, packed)), BF16)
    positions = rng.integers(0, 500, T).astype(np.int32)
    out, _ = run(compiled, [(x_st, BF16), (cos_st, BF16), (sin_st, BF16), (positions, P.I32)]).output(0)
    assert out.shape == (T, Hkv * S)
    ref = oracle.rope(xv[:, Hq * S:(Hq + Hkv) * S].reshape(T, Hkv, S), cos, sin, positions, rot).reshape(T, Hkv * S)
    assert scaled_error(H.storage_to_f32(out, BF16), ref) <= 2 * ROUND[BF16]


def test_rope_variants_the_plugin_refuses(hip):
    plugin = P.Plugin()
    for attrs in (dict(is_chatglm=True), dict(is_qwen=True), dict(support_2d_rope=True), dict(use_rope_cache=True),
                  dict(gather_position_arg_id=2)):
        g = P.GraphText("r")
        x = g.parameter("x", F16, [-1, -1, -1, 64])
        c = g.parameter("cos", F32, [-1, 64])
        s = g.parameter("sin", F32, [-1, 64])
        g.result("out", g.add("RoPE", "rope", [x, c, s], **attrs))
        assert "rope" not in plugin.query_model(g.model())
        with pytest.raises(P.PluginError):
            plugin.compile_model(g.model())


@pytest.mark.parametrize("a_shape,b_shape,ta,tb", [((37, 96), (80, 96), False, True), ((2, 3, 20, 48), (48, 16), False, False),
                                                    ((4, 48, 20), (4, 48, 16), True, False), ((1, 64), (6, 24, 64), False, True)])
def test_matmul_through_the_plugin(hip, oracle, a_shape, b_shape, ta, tb):
    rng = np.random.default_rng(4)
    g = P.GraphText("mm")
    a = g.parameter("a", BF16, [-1] * (len(a_shape) - 1) + [a_shape[-1]])
    b = g.parameter("b", BF16, list(b_shape))
    g.result("out", g.add("MatMul", "mm", [a, b], transpose_a=ta, transpose_b=tb))
    compiled = P.Plugin().compile_model(g.model())
    a_st, av = storage(rng.standard_normal(a_shape), BF16)
    b_st, bv = storage(rng.standard_normal(b_shape), BF16)
    out, _ = run(compiled, [(a_st, BF16), (b_st, BF16)]).output(0)
    a3 = av.reshape((-1,) + a_shape[-2:])
    b3 = bv.reshape((-1,) + b_shape[-2:])
    ref = oracle.matmul(a3 if a3.shape[0] > 1 else a3[0], b3 if b3.shape[0] > 1 else b3[0], ta, tb)
    lead = a_shape[:-2] if len(a_shape) >= len(b_shape) and int(np.prod(a_shape[:-2])) >= int(np.prod(b_shape[:-2])) else b_shape[:-2]
    assert out.shape == tuple(lead) + ref.shape[-2:]
    assert scaled_error(H.storage_to_f32(out, BF16).reshape(ref.shape), ref) <= ROUND[BF16] + 1e-5


def test_gather_embedding_and_concat_through_the_plugin(hip, oracle):
    rng = np.random.default_rng(5)
    g = P.GraphText("embed")
    table_st, _ = storage(rng.standard_normal((300, 64)), F16)
    table = g.constant("table", table_st, "f16")
    ids = g.parameter("ids", P.I32, [-1])
    axis = g.constant("axis", np.array(0, np.int64), "i64")
    emb = g.add("Gather", "embed", [table, ids, axis], batch_dims=0)
    extra = g.parameter("extra", F16, [-1, 16])
    g.result("out", g.add("Concat", "cat", [emb, extra], axis=-1))
    plugin = P.Plugin()
    assert {"embed", "cat"} <= set(plugin.query_model(g.model()))
    compiled = plugin.compile_model(g.model())
    tokens = rng.integers(-300, 300, 23).astype(np.int32)
    extra_st, _ = storage(rng.standard_normal((23, 16)), F16)
    req = run(compiled, [(tokens, P.I32), (extra_st, F16)])
    out, _ = req.output(0)
    ref = oracle.concat([oracle.gather(table_st, tokens, 0), extra_st], 1)
    assert np.array_equal(out, ref)
    # the table is a Constant: a second infer on the same request reuses the device copy
    tokens2 = rng.integers(0, 300, 5).astype(np.int32)
    req.set_input(0, tokens2, P.I32)
    req.set_input(1, extra_st[:5], F16)
    req.infer()
    out, _ = req.output(0)
    assert np.array_equal(out, oracle.concat([oracle.gather(table_st, tokens2, 0), extra_st[:5]], 1))


def test_attention_half_of_a_decoder_layer(hip, oracle):
    """hidden -> RMS -> q, k, v projections -> RoPE(q), RoPE(k) -> PagedAttentionExtension (device-resident
    cache, mixed prefill + decode batch) -> output projection -> + hidden, all on device "HIP", against
    the chain of oracle functions with the same bf16 roundings between the operators."""
    rng = np.random.default_rng(6)
    Hq, Hkv, D, hidden, bs = 4, 2, 128, 512, 32
    seqs = [(0, 70), (300, 1), (41, 1), (96, 33)]
    case = W.make_paged_case(96, seqs, Hq, Hkv, D, bs, BF16, BF16, F16)
    T = case["q"].shape[0]
    g = P.GraphText("decoder_attention")
    hid = g.parameter("hidden", BF16, [-1, hidden])
    w = {n: g.parameter(n, BF16, [width, hidden if n != "wo" else Hq * D])
         for n, width in (("wq", Hq * D), ("wk", Hkv * D), ("wv", Hkv * D), ("wo", hidden))}
    cos_p = g.parameter("cos", F32, [-1, D])
    sin_p = g.parameter("sin", F32, [-1, D])
    pos_p = g.parameter("positions", P.I32, [-1])
    kc_p = g.parameter("key_cache", F16, [-1, Hkv, bs, D])
    vc_p = g.parameter("value_cache", F16, [-1, Hkv, bs, D])
    idx = [g.parameter(n, P.I32, [-1]) for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")]
    scale_p = g.parameter("scale", F32, [-1])
    win_p = g.parameter("sliding_window", P.I32, [-1])
    alibi_p = g.parameter("alibi_slopes", F32, [0])
    mcl_p = g.parameter("max_context_len", P.I32, [-1])
    gamma_st, gamma = storage(1.0 + 0.1 * rng.standard_normal(hidden), BF16)
    norm = g.add("RMS", "input_norm", [hid, g.constant("gamma", gamma_st, "bf16")], epsilon=1e-5, output_type="dynamic")
    q = g.add("MatMul", "q_proj", [norm, w["wq"]], transpose_a=False, transpose_b=True)
    k = g.add("MatMul", "k_proj", [norm, w["wk"]], transpose_a=False, transpose_b=True)
    v = g.add("MatMul", "v_proj", [norm, w["wv"]], transpose_a=False, transpose_b=True)
    qr = g.add("RoPE", "q_rope", [q, cos_p, sin_p, pos_p], head_cnt=Hq, head_size=D, rotary_ndims=D, gather_position_arg_id=3)
    kr = g.add("RoPE", "k_rope", [k, cos_p, sin_p, pos_p], head_cnt=Hkv, head_size=D, rotary_ndims=D, gather_position_arg_id=3)
    pa = g.add("PagedAttentionExtension", "attention", [qr, kr, v, kc_p, vc_p] + idx + [scale_p, win_p, alibi_p, mcl_p])
    o = g.add("MatMul", "o_proj", [pa, w["wo"]], transpose_a=False, transpose_b=True)
    g.result("out", g.add("Add", "residual", [o, hid]))
    plugin = P.Plugin()
    plugin.set_property("PERF_COUNT", "YES")
    supported = plugin.query_model(g.model())
    assert {"input_norm", "q_proj", "q_rope", "k_rope", "attention", "o_proj", "residual"} <= set(supported)
    compiled = plugin.compile_model(g.model())

    hid_st, hv = storage(rng.standard_normal((T, hidden)), BF16)
    weights = {n: storage(rng.standard_normal(shape) / np.sqrt(shape[1]), BF16)
               for n, shape in (("wq", (Hq * D, hidden)), ("wk", (Hkv * D, hidden)), ("wv", (Hkv * D, hidden)), ("wo", (hidden, Hq * D)))}
    positions = np.concatenate([np.arange(p, p + n) for p, n in seqs]).astype(np.int32)
    cos, sin = rope_tables(int(positions.max()) + 1, D)
    kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
    vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
    dev_w = {n: hip.DeviceBuffer.from_numpy(st) for n, (st, _) in weights.items()}   # weights stay on the device
    req = compiled.create_infer_request()
    names = compiled.input_names()
    host = {"hidden": (hid_st, BF16), "cos": (cos, F32), "sin": (sin, F32), "positions": (positions, P.I32),
            "past_lens": (case["past_lens"], P.I32), "subsequence_begins": (case["subsequence_begins"], P.I32),
            "block_indices": (case["block_indices"], P.I32), "block_indices_begins": (case["block_indices_begins"], P.I32),
            "scale": (np.zeros((0,), np.float32), F32), "sliding_window": (np.array([0], np.int32), P.I32),
            "alibi_slopes": (np.zeros((0,), np.float32), F32),
            "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32)}
    cache_shape = list(case["key_cache"].shape[:3]) + [D]
    for i, n in enumerate(names):
        if n in host:
            req.set_input(i, *host[n])
        elif n in dev_w:
            req.set_device_input(i, dev_w[n].ptr, BF16, list(weights[n][0].shape))
        elif n == "key_cache":
            req.set_device_input(i, kc.ptr, F16, cache_shape)
        elif n == "value_cache":
            req.set_device_input(i, vc.ptr, F16, cache_shape)
        else:
            raise AssertionError("unexpected input " + n)
    req.infer()
    out, _ = req.output(0)
    got = H.storage_to_f32(out, BF16)

    r = lambda x: oracle.round_to(x, BF16)
    n_ref = r(oracle.rms_norm(hv, gamma, 1e-5))
    q_ref, k_ref, v_ref = (r(oracle.matmul(n_ref, weights[n][1], False, True)) for n in ("wq", "wk", "wv"))
    qr_ref = r(oracle.rope(q_ref.reshape(T, Hq, D), cos, sin, positions)).reshape(T, Hq * D)
    kr_ref = r(oracle.rope(k_ref.reshape(T, Hkv, D), cos, sin, positions)).reshape(T, Hkv * D)
    okc, ovc = case["key_cache"].copy(), case["value_cache"].copy()
    att = r(oracle.paged_attention(qr_ref, kr_ref, v_ref, okc, ovc, F16, case["past_lens"], case["subsequence_begins"],
                                   case["block_indices"], case["block_indices_begins"], Hq, Hkv, D, bs))
    ref = r(r(oracle.matmul(att, weights["wo"][1], False, True)) + hv)
    err = scaled_error(got, ref)
    print("decoder attention block: scaled max error %.4g, plain %.4g" % (err, float(np.max(np.abs(got - ref)))), flush=True)
    # every operator rounds to bf16 once (2^-9 relative) and a one-ulp difference in an intermediate
    # spreads through the products that follow
    assert err <= 3e-2
    # the new tokens' keys went into the device-resident cache; a bf16 rounding difference in the
    # projection in front of it may flip the last bit of an fp16 cache entry
    kc_got = kc.download(np.uint8, case["key_cache"].shape).view(np.float16).astype(np.float32)
    assert float(np.max(np.abs(kc_got - okc.view(np.float16).astype(np.float32)))) <= 0.07
    types = [t for _, t, _ in req.profiling()]
    assert types.count("MatMul") == 4 and types.count("RoPE") == 2 and "PagedAttentionExtension" in types


def _small_chain(dtype=BF16):
    """RMS -> MatMul -> RoPE with a position input: enough operators for a graph to matter."""
    g = P.GraphText("chain")
    x = g.parameter("x", dtype, [-1, 256])
    w = g.parameter("w", dtype, [256, 256])
    c = g.parameter("cos", F32, [-1, 64])
    s = g.parameter("sin", F32, [-1, 64])
    pos = g.parameter("positions", P.I32, [-1])
    gamma_st, gamma = storage(np.linspace(0.5, 1.5, 256), dtype)
    n = g.add("RMS", "norm", [x, g.constant("gamma", gamma_st, P._TYPE_NAMES[dtype])], epsilon=1e-5, output_type="dynamic")
    m = g.add("MatMul", "proj", [n, w], transpose_a=False, transpose_b=True)
    g.result("out", g.add("RoPE", "rope", [m, c, s, pos], head_cnt=4, head_size=64, rotary_ndims=64, gather_position_arg_id=3))
    return g, gamma


def _chain_reference(oracle, xv, wv, gamma, cos, sin, positions, dtype=BF16):
    r = lambda a: oracle.round_to(a, dtype)
    n = r(oracle.rms_norm(xv, gamma, 1e-5))
    m = r(oracle.matmul(n, wv, False, True))
    return r(oracle.rope(m.reshape(-1, 4, 64), cos, sin, positions)).reshape(-1, 256)


def test_infer_request_replays_a_graph(hip, oracle):
    """The second infer in a row that hands the operators the same pointers, shapes and small host
    values is recorded into a graph and later ones replay it; host inputs are uploaded outside the
    graph, so new values in the same tensors flow through a replay; anything else that changes (a
    shape, a device pointer) sends the request back to operator-by-operator execution."""
    rng = np.random.default_rng(8)
    g, gamma = _small_chain()
    # (three operators: below the size from which a graph pays and is used unasked)
    compiled = P.Plugin().compile_model(g.model(), {"HIP_GRAPH_MIN_OPERATORS": "1"})
    assert compiled.get_property("HIP_USE_GRAPH") == "YES"
    T = 24
    w_st, wv = storage(rng.standard_normal((256, 256)) / 16, BF16)
    dw = hip.DeviceBuffer.from_numpy(w_st)
    cos, sin = rope_tables(100, 64)
    req = compiled.create_infer_request()
    req.set_device_input(1, dw.ptr, BF16, [256, 256])
    req.set_input(2, cos, F32)
    req.set_input(3, sin, F32)

    def step(x_st, positions):
        req.set_input(0, x_st, BF16)
        req.set_input(4, positions, P.I32)
        req.infer()
        out, _ = req.output(0)
        return H.storage_to_f32(out, BF16)

    counts = lambda: (int(compiled.get_property("HIP_NUMBER_OF_GRAPHS")), int(compiled.get_property("HIP_GRAPH_LAUNCHES")))
    x_st, xv = storage(rng.standard_normal((T, 256)), BF16)
    positions = rng.integers(0, 100, T).astype(np.int32)
    ref = _chain_reference(oracle, xv, wv, gamma, cos, sin, positions)
    first = step(x_st, positions)
    assert scaled_error(first, ref) <= 3e-2 and counts() == (0, 0)          # operator by operator
    assert np.array_equal(step(x_st, positions), first) and counts() == (1, 1)  # recorded, then launched
    assert np.array_equal(step(x_st, positions), first) and counts() == (1, 2)  # replayed
    # new values in the same host tensors: uploaded ahead of the replay
    x2_st, x2v = storage(rng.standard_normal((T, 256)), BF16)
    positions2 = rng.integers(0, 100, T).astype(np.int32)
    got = step(x2_st, positions2)
    assert counts() == (1, 3)
    assert scaled_error(got, _chain_reference(oracle, x2v, wv, gamma, cos, sin, positions2)) <= 3e-2
    assert not np.array_equal(got, first)
    # another number of tokens: no replay; twice more and the new shape has a graph of its own
    x3_st, x3v = storage(rng.standard_normal((T + 5, 256)), BF16)
    positions3 = rng.integers(0, 100, T + 5).astype(np.int32)
    ref3 = _chain_reference(oracle, x3v, wv, gamma, cos, sin, positions3)
    got3 = step(x3_st, positions3)
    assert counts() == (1, 3) and scaled_error(got3, ref3) <= 3e-2
    assert np.array_equal(step(x3_st, positions3), got3) and counts() == (2, 4)
    assert np.array_equal(step(x3_st, positions3), got3) and counts() == (2, 5)
    # a different weight tensor on the device: a new signature again
    dw2 = hip.DeviceBuffer.from_numpy(w_st)
    req.set_device_input(1, dw2.ptr, BF16, [256, 256])
    assert np.array_equal(step(x3_st, positions3), got3) and counts() == (2, 5)


@pytest.mark.gpu
@pytest.mark.parametrize("streams", [1, 2])
def test_requests_share_the_blobs_of_the_device_workers(hip, oracle, streams):
    """Intermediate tensors live in the blob of the worker thread that runs a request (one per stream), not in the
    request: three requests of one compiled model with inputs of three sizes, run in turn and in flight together,
    each get their own results, also when an infer replays a graph recorded before the other requests used the blob."""
    rng = np.random.default_rng(21)
    g, gamma = _small_chain()
    compiled = P.Plugin().compile_model(g.model(), {"HIP_GRAPH_MIN_OPERATORS": "1", "NUM_STREAMS": str(streams)})
    w_st, wv = storage(rng.standard_normal((256, 256)) / 16, BF16)
    dw = hip.DeviceBuffer.from_numpy(w_st)
    cos, sin = rope_tables(100, 64)
    requests, inputs, refs = [], [], []
    for T in (24, 56, 9):
        req = compiled.create_infer_request()
        req.set_device_input(1, dw.ptr, BF16, [256, 256])
        req.set_input(2, cos, F32)
        req.set_input(3, sin, F32)
        x_st, xv = storage(rng.standard_normal((T, 256)), BF16)
        positions = rng.integers(0, 100, T).astype(np.int32)
        req.set_input(0, x_st, BF16)
        req.set_input(4, positions, P.I32)
        requests.append(req)
        inputs.append((x_st, positions))
        refs.append(_chain_reference(oracle, xv, wv, gamma, cos, sin, positions))
    first = []
    for req, ref in zip(requests, refs):
        req.infer()
        first.append(H.storage_to_f32(req.output(0)[0], BF16))
        assert first[-1].shape == ref.shape and scaled_error(first[-1], ref) <= 3e-2
    for round_ in range(3):  # in turn: from the second round on every request replays its graph
        for req, want in zip(requests, first):
            req.infer()
            assert np.array_equal(H.storage_to_f32(req.output(0)[0], BF16), want), round_
    for round_ in range(3):  # in flight together
        for req in requests:
            req.start_async()
        for req, want in zip(requests, first):
            req.wait()
            assert np.array_equal(H.storage_to_f32(req.output(0)[0], BF16), want), round_
    sizes = [req.intermediate_memory()[0] for req in requests]
    assert sizes[1] > sizes[0] > sizes[2] > 0  # what each request's last infer took of its worker's blob
    dw.free()


def test_graph_replay_can_be_switched_off(hip, oracle):
    rng = np.random.default_rng(9)
    g, gamma = _small_chain()
    plugin = P.Plugin()
    compiled = plugin.compile_model(g.model(), {"HIP_USE_GRAPH": "NO", "HIP_GRAPH_MIN_OPERATORS": "1"})
    w_st, _ = storage(rng.standard_normal((256, 256)) / 16, BF16)
    cos, sin = rope_tables(50, 64)
    x_st, _ = storage(rng.standard_normal((8, 256)), BF16)
    positions = np.arange(8, dtype=np.int32)
    req = compiled.create_infer_request()
    outs = []
    for _ in range(3):
        for i, (a, dt) in enumerate([(x_st, BF16), (w_st, BF16), (cos, F32), (sin, F32), (positions, P.I32)]):
            req.set_input(i, a, dt)
        req.infer()
        outs.append(req.output(0)[0])
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
    assert int(compiled.get_property("HIP_NUMBER_OF_GRAPHS")) == 0
    # profiling needs the operators one by one: it keeps the graph off as well
    profiled = plugin.compile_model(g.model(), {"PERF_COUNT": "YES", "HIP_GRAPH_MIN_OPERATORS": "1"})
    # and so does a model of fewer operators than a graph pays for (three here, six by default)
    small = plugin.compile_model(g.model())
    req = small.create_infer_request()
    for _ in range(3):
        for i, (a, dt) in enumerate([(x_st, BF16), (w_st, BF16), (cos, F32), (sin, F32), (positions, P.I32)]):
            req.set_input(i, a, dt)
        req.infer()
    assert int(small.get_property("HIP_NUMBER_OF_GRAPHS")) == 0 and small.get_property("HIP_GRAPH_MIN_OPERATORS") == "6"
    req = profiled.create_infer_request()
    for _ in range(3):
        for i, (a, dt) in enumerate([(x_st, BF16), (w_st, BF16), (cos, F32), (sin, F32), (positions, P.I32)]):
            req.set_input(i, a, dt)
        req.infer()
    assert int(profiled.get_property("HIP_NUMBER_OF_GRAPHS")) == 0 and len(req.profiling()) > 0


def test_paged_attention_decode_steps_replay_a_graph(hip, oracle):
    """A decode-only PagedAttentionExtension step with device-resident tensors, replayed: the cache
    write and the attention of every replay must be those of the eager step (same lengths: the
    step is repeated, not advanced)."""
    seqs = [(c - 1, 1) for c in (700, 64, 1500, 33, 2049, 5)]
    case = W.make_paged_case(98, seqs, 16, 4, 128, 32, W.F16, W.F16, W.F16)
    compiled = P.Plugin().compile_model(P.Model.paged_attention(W.F16, W.F16, W.F16, 16, 4, 128, 32), {"HIP_GRAPH_MIN_OPERATORS": "1"})
    kc = hip.DeviceBuffer.from_numpy(case["key_cache"])
    vc = hip.DeviceBuffer.from_numpy(case["value_cache"])
    dev = {n: hip.DeviceBuffer.from_numpy(case[n]) for n in ("q_store", "k_new_store", "v_new_store", "past_lens",
                                                             "subsequence_begins", "block_indices", "block_indices_begins")}
    req = compiled.create_infer_request()
    T = case["q_store"].shape[0]
    req.set_device_input(0, dev["q_store"].ptr, W.F16, [T, 16 * 128])
    req.set_device_input(1, dev["k_new_store"].ptr, W.F16, [T, 4 * 128])
    req.set_device_input(2, dev["v_new_store"].ptr, W.F16, [T, 4 * 128])
    shape = list(case["key_cache"].shape[:3]) + [128]
    req.set_device_input(3, kc.ptr, W.F16, shape)
    req.set_device_input(4, vc.ptr, W.F16, shape)
    for i, n in enumerate(("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")):
        req.set_device_input(5 + i, dev[n].ptr, P.I32, list(case[n].shape))
    req.set_input(9, np.zeros((0,), np.float32), W.F32)
    req.set_input(10, np.array([0], np.int32), P.I32)
    req.set_input(11, np.zeros((0,), np.float32), W.F32)
    req.set_input(12, np.array([case["max_context_len"]], np.int32), P.I32)
    from helpers import oracle_paged

    ref, okc, ovc = oracle_paged(oracle, case)
    outs = []
    for _ in range(4):
        req.infer()
        outs.append(H.storage_to_f32(req.output(0)[0], W.F16))
    assert H.max_abs(outs[0], ref) <= 2e-3
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])
    assert int(compiled.get_property("HIP_NUMBER_OF_GRAPHS")) == 1 and int(compiled.get_property("HIP_GRAPH_LAUNCHES")) == 3
    np.testing.assert_array_equal(kc.download(np.uint8, case["key_cache"].shape), okc)


# ------------------------------------------------------------------------------ a whole small decoder
class TinyDecoder:
    """A LLaMA-shaped decoder of `layers` layers as one model in the text form: token ids -> Gather
    (embedding) -> per layer [RMS -> q/k/v MatMul -> RoPE -> PagedAttentionExtension -> o MatMul ->
    Add, RMS -> gate|up MatMul -> GLU -> down MatMul -> Add] -> RMS -> lm_head MatMul.  Weights are
    Constants (uploaded once per request); every layer has a paged KV cache of its own, bound as
    device tensors; the index tensors are shared by the layers."""

    def __init__(self, rng, layers=2, hidden=256, Hq=2, Hkv=1, D=128, ffn=512, vocab=300, bs=32):
        self.layers, self.hidden, self.Hq, self.Hkv, self.D, self.ffn, self.vocab, self.bs = layers, hidden, Hq, Hkv, D, ffn, vocab, bs
        w = lambda *shape: storage(rng.standard_normal(shape) / np.sqrt(shape[-1]), BF16)
        self.embed = storage(rng.standard_normal((vocab, hidden)), BF16)
        self.final_gamma = storage(1.0 + 0.1 * rng.standard_normal(hidden), BF16)
        self.lm_head = w(vocab, hidden)
        self.layer_w = [{"g1": storage(1.0 + 0.1 * rng.standard_normal(hidden), BF16), "wq": w(Hq * D, hidden),
                         "wk": w(Hkv * D, hidden), "wv": w(Hkv * D, hidden), "wo": w(hidden, Hq * D),
                         "g2": storage(1.0 + 0.1 * rng.standard_normal(hidden), BF16), "wgu": w(2 * ffn, hidden),
                         "wd": w(hidden, ffn)} for _ in range(layers)]

    def graph(self):
        g = P.GraphText("tiny_decoder")
        ids = g.parameter("ids", P.I32, [-1])
        cos_p = g.parameter("cos", F32, [-1, self.D])
        sin_p = g.parameter("sin", F32, [-1, self.D])
        pos_p = g.parameter("positions", P.I32, [-1])
        idx = [g.parameter(n, P.I32, [-1]) for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins")]
        scale_p = g.parameter("scale", F32, [-1])
        win_p = g.parameter("sliding_window", P.I32, [-1])
        alibi_p = g.parameter("alibi_slopes", F32, [0])
        mcl_p = g.parameter("max_context_len", P.I32, [-1])
        caches = [(g.parameter("key_cache.%d" % l, F16, [-1, self.Hkv, self.bs, self.D]),
                   g.parameter("value_cache.%d" % l, F16, [-1, self.Hkv, self.bs, self.D])) for l in range(self.layers)]
        c = lambda name, pair: g.constant(name, pair[0], "bf16")
        axis = g.constant("axis", np.array(0, np.int64), "i64")
        h = g.add("Gather", "embed", [c("embed_w", self.embed), ids, axis], batch_dims=0)
        mm = lambda name, x, wt: g.add("MatMul", name, [x, wt], transpose_a=False, transpose_b=True)
        for l, lw in enumerate(self.layer_w):
            n1 = g.add("RMS", "norm1.%d" % l, [h, c("g1.%d" % l, lw["g1"])], epsilon=1e-5, output_type="dynamic")
            q = mm("q.%d" % l, n1, c("wq.%d" % l, lw["wq"]))
            k = mm("k.%d" % l, n1, c("wk.%d" % l, lw["wk"]))
            v = mm("v.%d" % l, n1, c("wv.%d" % l, lw["wv"]))
            rope = dict(head_size=self.D, rotary_ndims=self.D, gather_position_arg_id=3)
            qr = g.add("RoPE", "q_rope.%d" % l, [q, cos_p, sin_p, pos_p], head_cnt=self.Hq, **rope)
            kr = g.add("RoPE", "k_rope.%d" % l, [k, cos_p, sin_p, pos_p], head_cnt=self.Hkv, **rope)
            pa = g.add("PagedAttentionExtension", "attention.%d" % l,
                       [qr, kr, v, caches[l][0], caches[l][1]] + idx + [scale_p, win_p, alibi_p, mcl_p])
            h = g.add("Add", "res1.%d" % l, [mm("o.%d" % l, pa, c("wo.%d" % l, lw["wo"])), h])
            n2 = g.add("RMS", "norm2.%d" % l, [h, c("g2.%d" % l, lw["g2"])], epsilon=1e-5, output_type="dynamic")
            gu = mm("gate_up.%d" % l, n2, c("wgu.%d" % l, lw["wgu"]))
            act = g.add("GLU", "glu.%d" % l, [gu], axis=-1, split_lengths=self.ffn, glu_type=0, split_to_glu_idx=0, output_type="dynamic")
            h = g.add("Add", "res2.%d" % l, [mm("down.%d" % l, act, c("wd.%d" % l, lw["wd"])), h])
        nf = g.add("RMS", "final_norm", [h, c("final_gamma", self.final_gamma)], epsilon=1e-5, output_type="dynamic")
        g.result("logits", mm("lm_head", nf, c("lm_head_w", self.lm_head)))
        return g

    def reference(self, oracle, ids, cos, sin, positions, cases):
        """The chain of oracle functions with a bf16 rounding behind every operator; cases[l] holds
        layer l's cache and tables (the caches are updated in place, as the operator does)."""
        r = lambda a: oracle.round_to(a, BF16)
        mm = lambda x, wt: r(oracle.matmul(x, wt[1], False, True))
        T = len(ids)
        h = self.embed[1][ids]
        for lw, case in zip(self.layer_w, cases):
            n1 = r(oracle.rms_norm(h, lw["g1"][1], 1e-5))
            q, k, v = mm(n1, lw["wq"]), mm(n1, lw["wk"]), mm(n1, lw["wv"])
            qr = r(oracle.rope(q.reshape(T, self.Hq, self.D), cos, sin, positions)).reshape(T, -1)
            kr = r(oracle.rope(k.reshape(T, self.Hkv, self.D), cos, sin, positions)).reshape(T, -1)
            att = r(oracle.paged_attention(qr, kr, v, case["key_cache"], case["value_cache"], F16, case["past_lens"],
                                           case["subsequence_begins"], case["block_indices"], case["block_indices_begins"],
                                           self.Hq, self.Hkv, self.D, self.bs))
            h = r(mm(att, lw["wo"]) + h)
            n2 = r(oracle.rms_norm(h, lw["g2"][1], 1e-5))
            h = r(mm(r(oracle.glu(mm(n2, lw["wgu"]), 0, True)), lw["wd"]) + h)
        return mm(r(oracle.rms_norm(h, self.final_gamma[1], 1e-5)), self.lm_head)


def test_a_whole_small_decoder_runs_on_the_device(hip, oracle):
    """Two decoder layers, embedding to logits, one mixed prefill + decode step on device "HIP": 35
    operators, one infer, against the oracle chain; then the same step twice more, which records and
    replays a graph (the caches are rewritten with the same rows, so the logits repeat)."""
    rng = np.random.default_rng(12)
    model = TinyDecoder(rng)
    seqs = [(0, 40), (70, 1), (33, 1), (5, 20)]
    cases = [W.make_paged_case(120 + l, seqs, model.Hq, model.Hkv, model.D, model.bs, BF16, BF16, F16) for l in range(model.layers)]
    for c in cases[1:]:  # one set of tables for all layers; every pool is random throughout, so any table fits it
        assert c["key_cache"].shape == cases[0]["key_cache"].shape
        for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins"):
            c[n] = cases[0][n]
    T = cases[0]["q"].shape[0]
    ids = rng.integers(0, model.vocab, T).astype(np.int32)
    positions = np.concatenate([np.arange(p, p + n) for p, n in seqs]).astype(np.int32)
    cos, sin = rope_tables(int(positions.max()) + 1, model.D)
    plugin = P.Plugin()
    g = model.graph()
    supported = set(plugin.query_model(g.model()))
    assert {"embed", "glu.0", "glu.1", "attention.1", "lm_head", "res2.1"} <= supported
    compiled = plugin.compile_model(g.model())
    req = compiled.create_infer_request()
    dev_caches = [(hip.DeviceBuffer.from_numpy(c["key_cache"]), hip.DeviceBuffer.from_numpy(c["value_cache"])) for c in cases]
    case = cases[0]
    host = {"ids": (ids, P.I32), "cos": (cos, F32), "sin": (sin, F32), "positions": (positions, P.I32),
            "past_lens": (case["past_lens"], P.I32), "subsequence_begins": (case["subsequence_begins"], P.I32),
            "block_indices": (case["block_indices"], P.I32), "block_indices_begins": (case["block_indices_begins"], P.I32),
            "scale": (np.zeros((0,), np.float32), F32), "sliding_window": (np.array([0], np.int32), P.I32),
            "alibi_slopes": (np.zeros((0,), np.float32), F32),
            "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32)}
    cache_shape = list(case["key_cache"].shape[:3]) + [model.D]
    for i, n in enumerate(compiled.input_names()):
        if n in host:
            req.set_input(i, *host[n])
        else:
            kind, l = n.split(".")
            req.set_device_input(i, dev_caches[int(l)][0 if kind == "key_cache" else 1].ptr, F16, cache_shape)
    req.infer()
    logits, _ = req.output(0)
    got = H.storage_to_f32(logits, BF16)
    ref = model.reference(oracle, ids, cos, sin, positions, cases)
    assert got.shape == ref.shape == (T, model.vocab)
    err = scaled_error(got, ref)
    print("tiny decoder: scaled max error of the logits %.4g" % err, flush=True)
    assert err <= 6e-2  # 35 bf16 roundings deep; a wrong operator anywhere is off by order one
    # the ranking of the logits is what a sampler sees: the top token agrees wherever the reference's
    # margin over the runner-up is larger than the error
    top_ref, top_got = ref.argmax(-1), got.argmax(-1)
    margin = np.sort(ref, -1)[:, -1] - np.sort(ref, -1)[:, -2]
    assert np.all((top_ref == top_got) | (margin <= 2 * err * np.maximum(1.0, np.abs(ref).max(-1))))
    for _ in range(2):
        req.infer()
        again, _ = req.output(0)
        assert np.array_equal(again, logits)
    assert int(compiled.get_property("HIP_NUMBER_OF_GRAPHS")) == 1 and int(compiled.get_property("HIP_GRAPH_LAUNCHES")) == 2
    # the intermediate tensors of the 35 operators share one blob by lifetime: a few tensors' worth, not all of them
    blob, apart = req.intermediate_memory()
    print("tiny decoder: intermediate tensors %d bytes packed, %d side by side" % (blob, apart), flush=True)
    assert 0 < blob <= apart // 3


def test_one_request_through_batches_of_changing_size(hip, oracle):
    """The blob of intermediate tensors (the running worker's) is laid out per infer: a decode step, a longer prefill (the blob
    grows and every offset moves), the decode step's size again (the blob is larger than needed), each against the
    oracle chain, on one request."""
    rng = np.random.default_rng(14)
    model = TinyDecoder(rng)
    plugin = P.Plugin()
    compiled = plugin.compile_model(model.graph().model())
    req = compiled.create_infer_request()
    blobs = []
    for step, seqs in enumerate([[(70, 1), (33, 1), (5, 1)], [(0, 150), (64, 1), (10, 70)], [(9, 1), (200, 1), (31, 1)]]):
        cases = [W.make_paged_case(140 + 10 * step + l, seqs, model.Hq, model.Hkv, model.D, model.bs, BF16, BF16, F16) for l in range(model.layers)]
        for c in cases[1:]:
            for n in ("past_lens", "subsequence_begins", "block_indices", "block_indices_begins"):
                c[n] = cases[0][n]
        case = cases[0]
        T = case["q"].shape[0]
        ids = rng.integers(0, model.vocab, T).astype(np.int32)
        positions = np.concatenate([np.arange(p, p + n) for p, n in seqs]).astype(np.int32)
        cos, sin = rope_tables(int(positions.max()) + 1, model.D)
        dev_caches = [(hip.DeviceBuffer.from_numpy(c["key_cache"]), hip.DeviceBuffer.from_numpy(c["value_cache"])) for c in cases]
        host = {"ids": (ids, P.I32), "cos": (cos, F32), "sin": (sin, F32), "positions": (positions, P.I32),
                "past_lens": (case["past_lens"], P.I32), "subsequence_begins": (case["subsequence_begins"], P.I32),
                "block_indices": (case["block_indices"], P.I32), "block_indices_begins": (case["block_indices_begins"], P.I32),
                "scale": (np.zeros((0,), np.float32), F32), "sliding_window": (np.array([0], np.int32), P.I32),
                "alibi_slopes": (np.zeros((0,), np.float32), F32),
                "max_context_len": (np.array([case["max_context_len"]], np.int32), P.I32)}
        cache_shape = list(case["key_cache"].shape[:3]) + [model.D]
        for i, n in enumerate(compiled.input_names()):
            if n in host:
                req.set_input(i, *host[n])
            else:
                kind, l = n.split(".")
                req.set_device_input(i, dev_caches[int(l)][0 if kind == "key_cache" else 1].ptr, F16, cache_shape)
        req.infer()
        logits, _ = req.output(0)
        got = H.storage_to_f32(logits, BF16)
        ref = model.reference(oracle, ids, cos, sin, positions, cases)
        assert got.shape == ref.shape == (T, model.vocab)
        err = scaled_error(got, ref)
        blobs.append(req.intermediate_memory())
        print("changing sizes, step %d: %d tokens, scaled max error %.4g, blob %d of %d bytes" % ((step, T, err) + blobs[-1]), flush=True)
        assert err <= 6e-2
        for kc, vc in dev_caches:
            kc.free()
            vc.free()
    assert blobs[1][0] > blobs[0][0] and blobs[2][0] < blobs[1][0]  # (the figure is what the infer needs, not the allocation)
    assert all(0 < b <= a // 3 for b, a in blobs)


# ------------------------------------------------------------------------------ views, Transpose, Convert
def test_reshape_transpose_convert_chain(hip, oracle):
    """[batch, length, heads * size] f32 -> Reshape (0, 0, heads, size) -> Transpose (0, 2, 1, 3) ->
    Convert to f16 -> Unsqueeze / Squeeze -> Reshape (-1, size): the views cost nothing, Transpose and
    Convert are compared with the oracle bit for bit; shapes change from infer to infer."""
    rng = np.random.default_rng(21)
    Hh, S = 3, 16
    g = P.GraphText("formats")
    x = g.parameter("x", F32, [-1, -1, Hh * S])
    i64 = lambda name, values: g.constant(name, np.array(values, np.int64), "i64")
    split = g.add("Reshape", "split_heads", [x, i64("p0", [0, 0, Hh, S])], special_zero=True)
    moved = g.add("Transpose", "heads_first", [split, i64("order", [0, 2, 1, 3])])
    half = g.add("Convert", "to_f16", [moved], destination_type="f16")
    up = g.add("Unsqueeze", "up", [half, i64("ax_up", [0, -1])])
    down = g.add("Squeeze", "down", [up, i64("ax_down", [0])])
    g.result("heads", g.add("Squeeze", "down_all", [down]))
    g.result("rows", g.add("Reshape", "rows", [half, i64("p1", [-1, S])], special_zero=False))
    plugin = P.Plugin()
    assert {"split_heads", "heads_first", "to_f16", "up", "down", "down_all", "rows"} <= set(plugin.query_model(g.model()))
    compiled = plugin.compile_model(g.model())
    req = compiled.create_infer_request()
    for B, L in ((2, 5), (1, 1), (3, 70), (2, 0)):
        xv = (rng.standard_normal((B, L, Hh * S)) * 4).astype(np.float32)
        req.set_input(0, xv, F32)
        req.infer()
        heads, dt = req.output(0)
        rows, _ = req.output(1)
        want = oracle.convert(oracle.transpose(xv.reshape(B, L, Hh, S), (0, 2, 1, 3)), 0, 1)
        assert dt == F16
        squeezed = tuple(d for d in (B, Hh, L, S) if d != 1)
        assert heads.shape == squeezed and rows.shape == (B * Hh * L, S)
        assert np.array_equal(heads.reshape(-1), want.reshape(-1)) and np.array_equal(rows.reshape(-1), want.reshape(-1))


def test_transpose_order_from_a_host_tensor_and_reversal(hip, oracle):
    """The order may arrive as a tensor at run time (the reference reads it from the input then too,
    src/ops/transpose.cpp:272-300); an empty order reverses the axes."""
    rng = np.random.default_rng(22)
    g = P.GraphText("orders")
    x = g.parameter("x", BF16, [-1, -1, -1])
    order = g.parameter("order", P.I32, [-1])
    g.result("out", g.add("Transpose", "t", [x, order]))
    compiled = P.Plugin().compile_model(g.model())
    xs = rng.integers(0, 65535, (4, 70, 9)).astype(np.uint16)
    for perm in ((2, 0, 1), (0, 2, 1), (1, 0, 2), ()):
        out, _ = run(compiled, [(xs, BF16), (np.array(perm, np.int32), P.I32)]).output(0)
        want = oracle.transpose(xs, perm if perm else (2, 1, 0))
        assert out.shape == want.shape and np.array_equal(out, want)
    req = compiled.create_infer_request()
    req.set_input(0, xs, BF16)
    req.set_input(1, np.array([0, 0, 1], np.int32), P.I32)
    with pytest.raises(P.PluginError):
        req.infer()


@pytest.mark.parametrize("src,dst", [(F32, BF16), (BF16, F32), (F16, P.I32), (P.I32, F16), (F32, P.I64), (P.I64, F32), (F32, P.BOOL),
                                     (P.BOOL, F16), (F32, P.I8), (P.I8, BF16)])
def test_convert_through_the_plugin(hip, oracle, src, dst):
    codes = {F32: 0, F16: 1, BF16: 2, P.I32: 100, P.I64: 101, P.I8: 103, P.BOOL: 104}
    rng = np.random.default_rng(23 + src + dst)
    g = P.GraphText("convert")
    x = g.parameter("x", src, [-1, 33])
    g.result("out", g.add("Convert", "c", [x], destination_type=P._TYPE_NAMES[dst]))
    compiled = P.Plugin().compile_model(g.model())
    v = rng.uniform(-100, 100, (7, 33)).astype(np.float32)
    v[0, :4] = [0.0, -0.0, 0.5, -0.5]
    if src in (F16, BF16):
        xs = W.to_storage(v, src)[0]
    elif src == P.BOOL:
        xs = (v > 0)
    else:
        xs = v.astype(P._NP[src])
    out, dt = run(compiled, [(xs, src)]).output(0)
    want = oracle.convert(xs.view(np.uint8) if src == P.BOOL else xs, codes[src], codes[dst])
    assert dt == dst and out.shape == (7, 33)
    assert np.array_equal(np.asarray(out).view(want.dtype) if dst == P.BOOL else out, want)


def test_format_operators_the_plugin_refuses(hip):
    plugin = P.Plugin()
    g = P.GraphText("bad")
    x = g.parameter("x", F32, [-1, 8])
    g.result("out", g.add("Convert", "to_f64", [x], destination_type="f64"))
    assert "to_f64" not in plugin.query_model(g.model())
    g = P.GraphText("bad2")
    x = g.parameter("x", F32, [-1, 8])
    pattern = g.parameter("pattern", F32, [2])
    g.result("out", g.add("Reshape", "float_pattern", [x, pattern], special_zero=False))
    assert "float_pattern" not in plugin.query_model(g.model())
    # a pattern that does not fit the data is reported at infer time, by name
    g = P.GraphText("bad3")
    x = g.parameter("x", F32, [-1, 8])
    g.result("out", g.add("Reshape", "misfit", [x, g.constant("p", np.array([-1, 3], np.int64), "i64")], special_zero=False))
    req = plugin.compile_model(g.model()).create_infer_request()
    req.set_input(0, np.zeros((2, 8), np.float32), F32)
    with pytest.raises(P.PluginError) as e:
        req.infer()
    assert "misfit" in str(e.value)


def test_sdpa_attention_block_with_split_heads(hip, oracle):
    """The prefill form of an attention block as a converted model carries it: q/k/v MatMul ->
    Reshape to [batch, length, heads, size] -> Transpose to heads first -> causal
    ScaledDotProductAttention -> Transpose back -> Reshape -> output MatMul -> residual Add."""
    rng = np.random.default_rng(24)
    hidden, Hh, S = 256, 2, 128
    w = lambda *shape: storage(rng.standard_normal(shape) / np.sqrt(shape[-1]), BF16)
    wq, wk, wv, wo = w(Hh * S, hidden), w(Hh * S, hidden), w(Hh * S, hidden), w(hidden, Hh * S)
    g = P.GraphText("sdpa_block")
    x = g.parameter("x", BF16, [-1, -1, hidden])
    i64 = lambda name, values: g.constant(name, np.array(values, np.int64), "i64")
    mm = lambda name, a, wt: g.add("MatMul", name, [a, g.constant(name + "_w", wt[0], "bf16")], transpose_a=False, transpose_b=True)
    heads = lambda name, t: g.add("Transpose", name + "_t", [g.add("Reshape", name + "_r", [t, i64(name + "_p", [0, 0, Hh, S])], special_zero=True),
                                                             i64(name + "_o", [0, 2, 1, 3])])
    att = g.add("ScaledDotProductAttention", "sdpa", [heads("q", mm("q", x, wq)), heads("k", mm("k", x, wk)), heads("v", mm("v", x, wv))], causal=True)
    back = g.add("Reshape", "merge", [g.add("Transpose", "back", [att, i64("back_o", [0, 2, 1, 3])]), i64("merge_p", [0, 0, Hh * S])], special_zero=True)
    g.result("out", g.add("Add", "residual", [mm("o", back, wo), x]))
    compiled = P.Plugin().compile_model(g.model())
    r = lambda a: oracle.round_to(a, BF16)
    for B, L in ((2, 200), (1, 37)):
        x_st, xv = storage(rng.standard_normal((B, L, hidden)), BF16)
        out, _ = run(compiled, [(x_st, BF16)]).output(0)
        proj = lambda wt: r(oracle.matmul(xv.reshape(B * L, hidden), wt[1], False, True)).reshape(B, L, Hh, S).transpose(0, 2, 1, 3)
        a = r(oracle.sdpa(np.ascontiguousarray(proj(wq)), np.ascontiguousarray(proj(wk)), np.ascontiguousarray(proj(wv)), causal=True))
        merged = np.ascontiguousarray(a.transpose(0, 2, 1, 3)).reshape(B * L, Hh * S)
        ref = r(r(oracle.matmul(merged, wo[1], False, True)) + xv.reshape(B * L, hidden)).reshape(B, L, hidden)
        got = H.storage_to_f32(out, BF16)
        assert got.shape == ref.shape
        err = scaled_error(got, ref)
        print("sdpa block %dx%d: scaled max error %.4g" % (B, L, err), flush=True)
        assert err <= 3e-2


# ------------------------------------------------------------------------------ arithmetic, Softmax, decomposed attention
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_broadcasting_arithmetic_through_the_plugin(hip, oracle, dtype):
    """(x * scale + bias - row) / column with numpy broadcasting, shapes changing from infer to infer."""
    rng = np.random.default_rng(31)
    g = P.GraphText("arith")
    x = g.parameter("x", dtype, [-1, -1, 24])
    row = g.parameter("row", dtype, [-1, 1, 24])
    col = g.parameter("col", dtype, [-1, 1])
    scale_st, scale = storage(np.array([0.25]), dtype)
    bias_st, bias = storage(rng.standard_normal(24), dtype)
    t = g.add("Multiply", "scaled", [x, g.constant("scale", scale_st, P._TYPE_NAMES[dtype])])
    t = g.add("Add", "biased", [t, g.constant("bias", bias_st, P._TYPE_NAMES[dtype])])
    t = g.add("Subtract", "centred", [t, row])
    g.result("out", g.add("Divide", "divided", [t, col]))
    plugin = P.Plugin()
    assert {"scaled", "biased", "centred", "divided"} <= set(plugin.query_model(g.model()))
    compiled = plugin.compile_model(g.model())
    r = lambda a: oracle.round_to(a, dtype)
    for B, L in ((2, 5), (1, 1), (3, 40)):
        x_st, xv = storage(rng.standard_normal((B, L, 24)), dtype)
        row_st, rv = storage(rng.standard_normal((B, 1, 24)), dtype)
        col_st, cv = storage(rng.standard_normal((L, 1)) + 3.0, dtype)
        out, _ = run(compiled, [(x_st, dtype), (row_st, dtype), (col_st, dtype)]).output(0)
        ref = r(oracle.binary(3, r(oracle.binary(1, r(oracle.binary(0, r(oracle.binary(2, xv, scale)), bias)), rv)), cv))
        assert out.shape == (B, L, 24) and np.array_equal(H.storage_to_f32(out, dtype), ref)
    req = compiled.create_infer_request()
    for i, a in enumerate((np.zeros((2, 5, 24)), np.zeros((3, 1, 24)), np.zeros((5, 1)))):
        req.set_input(i, storage(a, dtype)[0], dtype)
    with pytest.raises(P.PluginError) as e:  # batch 2 against batch 3
        req.infer()
    assert "centred" in str(e.value)


@pytest.mark.parametrize("opset,axis,shape", [(8, -1, (2, 3, 40)), (8, 1, (2, 3, 40)), (1, 0, (5, 7)), (8, -2, (4, 9, 16))])
def test_softmax_through_the_plugin(hip, oracle, opset, axis, shape):
    rng = np.random.default_rng(32)
    g = P.GraphText("softmax")
    x = g.parameter("x", F16, [-1] * len(shape))
    g.result("out", g.add("Softmax", "sm", [x], axis=axis, opset=opset))
    compiled = P.Plugin().compile_model(g.model())
    x_st, xv = storage(rng.standard_normal(shape) * 3, F16)
    out, _ = run(compiled, [(x_st, F16)]).output(0)
    assert out.shape == shape and np.abs(H.storage_to_f32(out, F16) - oracle.softmax(xv, axis)).max() <= 6e-4


def decomposed_attention_graph(dtype, Hh, D, L, scale):
    """Attention as the reference executes it once ScaledDotProductAttentionDecomposition has run
    (transformer/cuda_graph_transformer.cpp:151-156): Multiply by the scale, Transpose of the keys,
    MatMul, Add of the mask, Softmax, MatMul; beside it the fused operator on the same inputs."""
    g = P.GraphText("decomposed")
    q = g.parameter("q", dtype, [-1, Hh, -1, D])
    k = g.parameter("k", dtype, [-1, Hh, -1, D])
    v = g.parameter("v", dtype, [-1, Hh, -1, D])
    mask = g.parameter("mask", dtype, [1, 1, -1, -1])
    scale_st, _ = storage(np.array([scale]), dtype)
    qs = g.add("Multiply", "scale_q", [q, g.constant("scale", scale_st, P._TYPE_NAMES[dtype])])
    kt = g.add("Transpose", "k_t", [k, g.constant("order", np.array([0, 1, 3, 2], np.int64), "i64")])
    scores = g.add("Add", "masked", [g.add("MatMul", "qk", [qs, kt], transpose_a=False, transpose_b=False), mask])
    probs = g.add("Softmax", "softmax", [scores], axis=-1, opset=8)
    g.result("decomposed", g.add("MatMul", "pv", [probs, v], transpose_a=False, transpose_b=False))
    g.result("fused", g.add("ScaledDotProductAttention", "sdpa", [q, k, v], causal=True))
    return g


@pytest.mark.parametrize("dtype,B,Hh,L,D,tol", [(F32, 1, 8, 128, 64, 2e-5), (BF16, 2, 4, 200, 128, 1.5e-2), (F16, 1, 2, 77, 64, 3e-3)])
def test_decomposed_attention_matches_the_fused_operator(hip, oracle, dtype, B, Hh, L, D, tol):
    """The first case is the reference's own CPU-runnable configuration (fp32, 1 x 8 x 128 x 64, causal,
    scale 1/sqrt(64)); both forms run on device "HIP" in one infer and are held against the oracle."""
    rng = np.random.default_rng(33)
    scale = 1.0 / np.sqrt(D)
    g = decomposed_attention_graph(dtype, Hh, D, L, scale)
    compiled = P.Plugin().compile_model(g.model())
    q_st, q = storage(rng.standard_normal((B, Hh, L, D)), dtype)
    k_st, k = storage(rng.standard_normal((B, Hh, L, D)), dtype)
    v_st, v = storage(rng.standard_normal((B, Hh, L, D)), dtype)
    big = -np.inf if dtype == F32 else -60000.0  # f16 has no room for more; exp of it is 0 all the same
    mask_st, _ = storage(np.triu(np.full((L, L), big, np.float32), 1)[None, None], dtype)
    req = run(compiled, [(q_st, dtype), (k_st, dtype), (v_st, dtype), (mask_st, dtype)])
    outs = {name: H.storage_to_f32(req.output(i)[0], dtype) for i, name in enumerate(("decomposed", "fused"))}  # in the order of the results
    ref = oracle.sdpa(q, k, v, causal=True)
    for name in ("decomposed", "fused"):
        err = float(np.abs(outs[name] - ref).max())
        print("%s attention, dtype %d: max abs error %.3g" % (name, dtype, err), flush=True)
        assert outs[name].shape == ref.shape and err <= tol, (name, err)
