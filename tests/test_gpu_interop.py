"""GPU parity for the kernel-handle API: each kernel kind is compiled from program text, fed through its
input surface and compared with the CPU oracle's restatement of the reference generator it stands for."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

FMT = {"q8_0": orc.FMT_Q8_0, "q4_0": orc.FMT_Q4_0, "q4_k": orc.FMT_Q4_K, "f16": orc.FMT_F16}


@pytest.fixture(scope="module")
def io():
    import espresso_amd.interop as m
    import espresso_amd.ops as o
    o.init()
    return m


def _f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def _matrix(name, rows, cols, rng):
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    if name == "f16":
        return orc.blob_build(w), _f16(w)
    blocks = orc.quantize(FMT[name], w)
    return blocks.tobytes(), orc.dequantize(FMT[name], blocks, rows * cols).reshape(rows, cols)


def _fp16_close(got, want, extra=0.0):
    # one fp16 rounding of the result plus fp32 summation-order noise
    tol = np.abs(want) * 2.0 ** -10 + 1e-4 + extra
    assert np.all(np.abs(got - want) <= tol), float(np.abs(got - want).max())


@pytest.mark.parametrize("name,rows,cols,spatial,lanes", [("q8_0", 768, 768, 32, 1), ("q4_k", 512, 1024, 8, 4), ("q4_0", 96, 256, 1, 1), ("f16", 200, 320, 16, 16)])
def test_gemv_kernel_matches_oracle(io, name, rows, cols, spatial, lanes):
    rng = np.random.default_rng(rows + cols)
    blob, deq = _matrix(name, rows, cols, rng)
    before = io._L().esp_interop_compile_count()
    k = io.ANEKernel(io.program_text("gemv", name, spatial, lanes, rows=rows, cols=cols), [("@model_path/weights/w.bin", blob)],
                     [cols * spatial * 2], [rows * spatial * 2])
    assert io._L().esp_interop_compile_count() == before + 1 and io._L().esp_interop_live_handle_count() == 1
    x = rng.normal(0, 1, (cols, spatial)).astype(np.float32)
    xin, out = k.inputSurface(0), k.outputSurface(0)
    io.SurfaceIO.writeFP16(xin, x, cols, spatial)
    k.eval()
    got = io.SurfaceIO.readFP16(out, 0, rows, spatial)
    for lane in range(lanes):
        _fp16_close(got[:, lane], orc.matvec(deq, _f16(x[:, lane])))
    assert np.all(got[:, lanes:] == 0)                       # columns past `lanes` are never written
    assert k.lastHWExecutionTimeNS() > 0
    # a second eval after rewriting one column only changes that column
    col = rng.normal(0, 1, cols).astype(np.float32)
    io.SurfaceIO.writeFP16SpatialSlice(xin, 0, 0, spatial, col, cols)
    k.eval()
    got2 = io.SurfaceIO.readFP16(out, 0, rows, spatial)
    _fp16_close(got2[:, 0], orc.matvec(deq, _f16(col)))
    assert np.array_equal(got2[:, 1:], got[:, 1:])
    k.free()
    assert io._L().esp_interop_live_handle_count() == 0


def test_rmsnorm_classifier_kernel_matches_oracle(io):
    dim, vocab, spatial, lanes = 256, 4000, 8, 3
    rng = np.random.default_rng(1)
    blob, deq = _matrix("q8_0", vocab, dim, rng)
    gamma = (1.0 + rng.normal(0, 0.1, dim)).astype(np.float32)
    k = io.ANEKernel(io.program_text("rmsnorm_classifier", "q8_0", spatial, lanes, dim=dim, vocab=vocab),
                     [("@model_path/weights/rms_final.bin", orc.blob_build(gamma)), ("@model_path/weights/classifier.bin", blob)],
                     [dim * spatial * 2], [vocab * spatial * 2, spatial * 2])
    x = rng.normal(0, 1, (dim, spatial)).astype(np.float32)
    io.SurfaceIO.writeFP16(k.inputSurface(0), x, dim, spatial)
    k.eval()
    logits = io.SurfaceIO.readFP16(k.outputSurface(0), 0, vocab, spatial)
    mx = io.SurfaceIO.readFP16(k.outputSurface(1), 0, 1, spatial)
    for lane in range(lanes):
        n = _f16(orc.rmsnorm(_f16(x[:, lane]), _f16(gamma), 1e-5))
        want = orc.matvec(deq, n)
        _fp16_close(logits[:, lane], want, extra=2e-3)
        assert abs(mx[0, lane] - want.max()) <= abs(want.max()) * 2.0 ** -10 + 2e-3
        # the surface argmax agrees with the oracle's whenever the top-2 margin exceeds the fp16 step
        top = np.sort(want)[-2:]
        if top[1] - top[0] > 4e-3:
            assert io.SurfaceIO.argmaxFP16SpatialSlice(k.outputSurface(0), 0, lane, spatial, vocab)[0] == int(np.argmax(want))
    k.free()


@pytest.mark.parametrize("name,dim,hidden", [("q8_0", 768, 2048), ("q4_k", 512, 1024), ("q4_k", 2048, 8192), ("q4_k", 4096, 11008)])
def test_decode_ffn_kernel_matches_oracle(io, name, dim, hidden):
    spatial, lanes = 32, 2
    rng = np.random.default_rng(dim)
    b1, w1 = _matrix(name, hidden, dim, rng)
    b3, w3 = _matrix(name, hidden, dim, rng)
    b2, w2 = _matrix(name, dim, hidden, rng)
    gamma = (1.0 + rng.normal(0, 0.1, dim)).astype(np.float32)
    k = io.ANEKernel(io.program_text("decode_ffn", name, spatial, lanes, dim=dim, hidden=hidden),
                     [("@model_path/weights/rms_ffn.bin", orc.blob_build(gamma)), ("@model_path/weights/w1.bin", b1),
                      ("@model_path/weights/w3.bin", b3), ("@model_path/weights/w2.bin", b2)], [dim * spatial * 2], [dim * spatial * 2])
    x = rng.normal(0, 1, (dim, spatial)).astype(np.float32)
    io.SurfaceIO.writeFP16(k.inputSurface(0), x, dim, spatial)
    k.eval()
    got = io.SurfaceIO.readFP16(k.outputSurface(0), 0, dim, spatial)
    for lane in range(lanes):
        xl = _f16(x[:, lane])
        n = _f16(orc.rmsnorm(xl, _f16(gamma), 1e-5))
        g, u = orc.matvec(w1, n), orc.matvec(w3, n)
        act = _f16(np.array([orc.silu_tanh(float(v)) for v in g], dtype=np.float32) * u)
        want = xl + orc.matvec(w2, act)
        # the fp16 rounding of the hidden activations adds noise that grows with the number of terms of the down projection
        _fp16_close(got[:, lane], want, extra=1e-3 * max(1.0, hidden / 2048))
    k.free()


def test_compile_errors_eval_failure_hook_and_rebind(io):
    L = io._L()
    rng = np.random.default_rng(3)
    blob, deq = _matrix("q8_0", 64, 64, rng)
    before = L.esp_interop_compile_count()
    with pytest.raises(io.ANEError, match="compilationFailed"):      # not a program this library knows
        io.ANEKernel("this is not a program", [], [64], [64])
    with pytest.raises(io.ANEError, match="compilationFailed"):      # weight missing
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [], [128], [128])
    with pytest.raises(io.ANEError, match="compilationFailed"):      # weight bytes do not match rows x cols
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=128), [("w.bin", blob)], [256], [128])
    with pytest.raises(io.ANEError, match="invalidArguments"):       # surface size does not match the program
        io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [("w.bin", blob)], [64], [128])
    assert L.esp_interop_compile_count() == before and L.esp_interop_live_handle_count() == 0
    k = io.ANEKernel(io.program_text("gemv", "q8_0", rows=64, cols=64), [("w.bin", blob)], [128], [128])
    L.esp_interop_set_force_eval_failure(True)
    try:
        with pytest.raises(io.ANEError, match="evaluationFailed"):
            k.eval()
    finally:
        L.esp_interop_set_force_eval_failure(False)
    # rebinding the input to a caller-made surface
    mine = io.Surface.create(128)
    x = rng.normal(0, 1, 64).astype(np.float32)
    io.SurfaceIO.writeFP16(mine, x, 64, 1)
    k.rebindInput(0, mine)
    k.eval()
    _fp16_close(io.SurfaceIO.readFP16(k.outputSurface(0), 0, 64, 1)[:, 0], orc.matvec(deq, _f16(x)))
    with pytest.raises(io.ANEError):
        k.rebindInput(0, io.Surface.create(64))                      # wrong size
    k.free()


def test_decode_qkv_outputs_k_q_v_in_the_reference_order(io):
    """decodeQKVOnly's outputs are k @ 0, q @ 1, v @ 2 (DecodeForwardPass.swift:374-377); grouped-query shapes."""
    dim, q_dim, kv_dim, spatial, lanes = 512, 512, 128, 32, 2
    rng = np.random.default_rng(41)
    bq, wq = _matrix("q4_k", q_dim, dim, rng)
    bk, wk = _matrix("q4_k", kv_dim, dim, rng)
    bv, wv = _matrix("q4_k", kv_dim, dim, rng)
    gamma = (1.0 + rng.normal(0, 0.1, dim)).astype(np.float32)
    k = io.ANEKernel(io.program_text("decode_qkv", "q4_k", spatial, lanes, dim=dim, q_dim=q_dim, kv_dim=kv_dim),
                     [("@model_path/weights/rms_att.bin", orc.blob_build(gamma)), ("@model_path/weights/wq.bin", bq),
                      ("@model_path/weights/wk.bin", bk), ("@model_path/weights/wv.bin", bv)],
                     [dim * spatial * 2], [kv_dim * spatial * 2, q_dim * spatial * 2, kv_dim * spatial * 2])
    x = rng.normal(0, 1, (dim, spatial)).astype(np.float32)
    io.SurfaceIO.writeFP16(k.inputSurface(0), x, dim, spatial)
    k.eval()
    for out_index, w, rows in ((0, wk, kv_dim), (1, wq, q_dim), (2, wv, kv_dim)):
        got = io.SurfaceIO.readFP16(k.outputSurface(out_index), 0, rows, spatial)
        for lane in range(lanes):
            n = _f16(orc.rmsnorm(_f16(x[:, lane]), _f16(gamma), 1e-5))
            _fp16_close(got[:, lane], orc.matvec(w, n), extra=1e-3)
        assert np.all(got[:, lanes:] == 0)
    with pytest.raises(io.ANEError, match="invalidArguments"):      # the surfaces in q, k, v order are not what the kernel has
        io.ANEKernel(io.program_text("decode_qkv", "q4_k", spatial, lanes, dim=dim, q_dim=q_dim, kv_dim=kv_dim),
                     [("rms_att.bin", orc.blob_build(gamma)), ("wq.bin", bq), ("wk.bin", bk), ("wv.bin", bv)],
                     [dim * spatial * 2], [q_dim * spatial * 2, kv_dim * spatial * 2, kv_dim * spatial * 2])
    k.free()


def test_rope_scatter_and_sdpa_on_surfaces_match_the_oracle(io):
    """rope_decode, kv_cache_scatter and fused_decode_sdpa (MetalAttentionKernel.swift:1756-1886) on channel-first surfaces."""
    heads, kv_heads, hd, lane, stride = 8, 2, 64, 32, 48
    q_dim, kv_dim = heads * hd, kv_heads * hd
    rng = np.random.default_rng(42)
    q, kk = io.Surface.create(q_dim * lane * 2), io.Surface.create(kv_dim * lane * 2)
    v = io.Surface.create(kv_dim * lane * 2)
    kc, vc, ctx = io.Surface.create(kv_dim * stride * 2), io.Surface.create(kv_dim * stride * 2), io.Surface.create(q_dim * lane * 2)
    k_rows, v_rows = [], []
    for pos in range(37):
        qv, kv_, vv = (rng.normal(0, 1, n).astype(np.float32) for n in (q_dim, kv_dim, kv_dim))
        io.SurfaceIO.writeFP16SpatialSlice(q, 0, 0, lane, qv, q_dim)
        io.SurfaceIO.writeFP16SpatialSlice(kk, 0, 0, lane, kv_, kv_dim)
        io.SurfaceIO.writeFP16SpatialSlice(v, 0, 0, lane, vv, kv_dim)
        io.rope_decode(q, kk, heads, kv_heads, hd, pos, 10000.0, lane)
        q_rot = io.SurfaceIO.readFP16SpatialSlice(q, 0, 0, lane, q_dim)
        k_rot = io.SurfaceIO.readFP16SpatialSlice(kk, 0, 0, lane, kv_dim)
        _fp16_close(q_rot, orc.rope_half_split(_f16(qv), heads, hd, pos, 10000.0), extra=2e-3)
        _fp16_close(k_rot, orc.rope_half_split(_f16(kv_), kv_heads, hd, pos, 10000.0), extra=2e-3)
        io.kv_cache_scatter(kk, v, kc, vc, kv_dim, pos, stride, lane)
        k_rows.append(k_rot); v_rows.append(_f16(vv))
        assert np.array_equal(io.SurfaceIO.readFP16SpatialSlice(kc, 0, pos, stride, kv_dim), k_rot)
        assert np.array_equal(io.SurfaceIO.readFP16SpatialSlice(vc, 0, pos, stride, kv_dim), _f16(vv))
        if pos in (0, 1, 17, 36):
            io.decode_sdpa(q, kc, vc, ctx, heads, kv_heads, hd, pos + 1, 0, stride, lane)
            got = io.SurfaceIO.readFP16SpatialSlice(ctx, 0, 0, lane, q_dim)
            K, V = np.stack(k_rows), np.stack(v_rows)                     # [tokens, kv_dim]
            want = np.empty(q_dim, np.float32)
            for h in range(heads):
                g = h // (heads // kv_heads)
                sc = (K[:, g * hd:(g + 1) * hd] @ q_rot[h * hd:(h + 1) * hd]) / np.sqrt(np.float32(hd))
                p = np.exp(sc - sc.max()); p /= p.sum()
                want[h * hd:(h + 1) * hd] = p @ V[:, g * hd:(g + 1) * hd]
            _fp16_close(got, want, extra=1e-3)
    # a window that starts past column 0: tokens 30..36 only
    io.decode_sdpa(q, kc, vc, ctx, heads, kv_heads, hd, 7, 30, stride, lane)
    got = io.SurfaceIO.readFP16SpatialSlice(ctx, 0, 0, lane, q_dim)
    K, V = np.stack(k_rows[30:]), np.stack(v_rows[30:])
    sc = (K[:, :hd] @ q_rot[:hd]) / np.sqrt(np.float32(hd))
    p = np.exp(sc - sc.max()); p /= p.sum()
    _fp16_close(got[:hd], p @ V[:, :hd], extra=1e-3)
    with pytest.raises(io.ANEError):
        io.decode_sdpa(q, kc, vc, ctx, heads, kv_heads, hd, 20, 30, stride, lane)      # window runs past the cache
    with pytest.raises(io.ANEError):
        io.kv_cache_scatter(kk, v, kc, vc, kv_dim, stride, stride, lane)               # token index past the cache
    with pytest.raises(io.ANEError):
        io.rope_decode(q, kk, heads + 1, kv_heads, hd, 0, 10000.0, lane)               # more heads than the surface holds


@pytest.mark.parametrize("name,shape", [
    ("q8_0", dict(n_layer=1, n_head=12, n_kv_head=12, d_model=768, head_dim=64, hidden_dim=2048, vocab=2048, max_seq=64)),
    ("q4_k", dict(n_layer=1, n_head=8, n_kv_head=2, d_model=512, head_dim=64, hidden_dim=1024, vocab=1024, max_seq=64, rope_theta=500000.0)),
])
def test_one_layer_handle_by_handle_matches_the_runtime(io, name, shape):
    """The hybrid decode layer as the reference's DecodeForwardPass runs it (DecodeForwardPass.swift:360-400): decodeQKVOnly,
    rope_decode, kv_cache_scatter, fused_decode_sdpa, decodeProjection with the residual rebound to the layer input, decodeFFN;
    hidden state after every token against the runtime's own decode step.  The handles round q, k, v, the attention context
    and both residual sums to fp16 on their surfaces, the runtime keeps fp32: the tolerance is that rounding."""
    import espresso_amd.llama as ll
    import espresso_amd.synthetic as syn
    cfg = ll.MultiModelConfig(**shape)
    rt, packed = syn.build_runtime(cfg, FMT[name], seed=23, kv_format=orc.FMT_F16, keep_packed=True)
    lw = packed["layers"][0]
    dim, q_dim, kv_dim, hidden = cfg.d_model, cfg.n_head * cfg.head_dim, cfg.n_kv_head * cfg.head_dim, cfg.hidden_dim
    spatial, stride = 32, cfg.max_seq
    norm = lambda key: orc.blob_build(np.frombuffer(bytes(lw[key]), np.float16).astype(np.float32))
    path = lambda stem: f"@model_path/weights/{stem}.bin"
    qkv = io.ANEKernel(io.program_text("decode_qkv", name, spatial, 1, dim=dim, q_dim=q_dim, kv_dim=kv_dim),
                       [(path("rms_att"), norm("rms_att")), (path("wq"), bytes(lw["wq"])), (path("wk"), bytes(lw["wk"])), (path("wv"), bytes(lw["wv"]))],
                       [dim * spatial * 2], [kv_dim * spatial * 2, q_dim * spatial * 2, kv_dim * spatial * 2])
    proj = io.ANEKernel(io.program_text("decode_projection", name, spatial, 1, dim=dim, q_dim=q_dim), [(path("wo"), bytes(lw["wo"]))],
                        [q_dim * spatial * 2, dim * spatial * 2], [dim * spatial * 2])
    ffn = io.ANEKernel(io.program_text("decode_ffn", name, spatial, 1, dim=dim, hidden=hidden),
                       [(path("rms_ffn"), norm("rms_ffn")), (path("w1"), bytes(lw["w1"])), (path("w3"), bytes(lw["w3"])), (path("w2"), bytes(lw["w2"]))],
                       [dim * spatial * 2], [dim * spatial * 2])
    x_in = qkv.inputSurface(0)
    k_out, q_out, v_out = qkv.outputSurface(0), qkv.outputSurface(1), qkv.outputSurface(2)
    k_cache, v_cache = io.Surface.create(kv_dim * stride * 2), io.Surface.create(kv_dim * stride * 2)
    proj.rebindInput(1, x_in)                         # the residual is the layer's input surface
    ffn.rebindInput(0, proj.outputSurface(0))
    ctx, out = proj.inputSurface(0), ffn.outputSurface(0)
    emb = np.frombuffer(bytes(packed["embedding"]), np.float16).reshape(cfg.vocab, dim).astype(np.float32)
    rng = np.random.default_rng(7)
    worst = 0.0
    for pos, token in enumerate(rng.integers(0, cfg.vocab, 40).tolist()):
        io.SurfaceIO.writeFP16SpatialSlice(x_in, 0, 0, spatial, emb[token], dim)
        qkv.eval()
        io.rope_decode(q_out, k_out, cfg.n_head, cfg.n_kv_head, cfg.head_dim, pos, cfg.rope_theta, spatial)
        io.kv_cache_scatter(k_out, v_out, k_cache, v_cache, kv_dim, pos, stride, spatial)
        io.decode_sdpa(q_out, k_cache, v_cache, ctx, cfg.n_head, cfg.n_kv_head, cfg.head_dim, pos + 1, 0, stride, spatial)
        proj.eval()
        ffn.eval()
        got = io.SurfaceIO.readFP16SpatialSlice(out, 0, 0, spatial, dim)
        rt.advance(token)
        want = rt.last_hidden()
        scale = float(np.abs(want).max())
        worst = max(worst, float(np.abs(got - want).max()) / scale)
        assert np.all(np.abs(got - want) <= 2.0 ** -9 * scale + 1e-5), (pos, float(np.abs(got - want).max()), scale)
    print(f"\n  {name}: worst |handles - runtime| / max|hidden| over 40 tokens = {worst:.2e}")
    for kernel in (qkv, proj, ffn):
        kernel.free()
    rt.close()


@pytest.mark.parametrize("bottleneck,groups,vocab,spatial,streams", [(128, 1, 32000, 8, 3), (128, 4, 4096, 16, 16), (36, 3, 1002, 8, 1), (256, 1, 65535, 8, 2)])
def test_factored_head_resident_on_the_gpu(io, bottleneck, groups, vocab, spatial, streams):
    """The expansion + arg-max of the factored output head with its weights resident in HBM (MetalExpansionArgmax.swift:966-1186)
    against the host routine (surface_io.c:1438-1700 restated; itself held to exact fp16 arithmetic in test_interop_surfaces.py):
    bit-identical values and the same first maximum with fp16 sums; with fp32 sums against a sequential fp32 chain in numpy."""
    cpg, per = bottleneck // groups, vocab // groups
    rng = np.random.default_rng(vocab + bottleneck)
    proj = rng.normal(0, 1, (bottleneck, spatial)).astype(np.float16)
    w = rng.normal(0, 0.3, (vocab, cpg)).astype(np.float16)
    w[per // 2 + 1] = w[per // 2]                     # two rows of one group tie exactly
    s = io.Surface.create((bottleneck + 3) * spatial * 2)
    io.SurfaceIO.writeFP16At(s, 3, proj.astype(np.float32), bottleneck, spatial)
    head = io.FusedExpansionArgmax(w.view(np.uint16), bottleneck, vocab, spatial, groups)
    want_i, want_v = io.SurfaceIO.fusedExpansionArgmax(s, 3, spatial, bottleneck, groups, w.view(np.uint16), vocab, streams)
    got_i, got_v = head.run(s, streams, channelOffset=3, withValues=True)
    assert got_i == want_i and got_v == want_v
    assert head.run(s, streams, channelOffset=3) == want_i                       # a second call reuses the object's buffers
    # fp32 sums: one fused multiply-add per term in k order (the Metal shader's loop), first maximum
    got_i, got_v = head.run(s, streams, channelOffset=3, fp32Sums=True, withValues=True)
    wf = w.astype(np.float64)
    for lane in range(streams):
        acc = np.zeros(vocab, np.float32)
        pl = proj[:, lane].astype(np.float64).reshape(groups, cpg)
        for k in range(cpg):
            pk = np.repeat(pl[:, k], per)
            acc = (pk * wf[:, k] + acc.astype(np.float64)).astype(np.float32)    # exact product, one rounding: a fused multiply-add
        assert got_i[lane] == int(np.argmax(acc)) and got_v[lane] == float(acc.max())
    # the tie: a projection that is one-hot in the tied rows' group makes rows per/2 and per/2 + 1 lead when their weight is the column's largest
    col = int(np.argmax(w[per // 2].astype(np.float32)))
    onehot = np.zeros((bottleneck, spatial), np.float32); onehot[col, 0] = 1.0
    io.SurfaceIO.writeFP16At(s, 3, onehot, bottleneck, spatial)
    column = w[:per, col].astype(np.float32)
    i, v = head.run(s, 1, channelOffset=3, withValues=True)
    assert i == [int(np.argmax(column))] and v == [float(column.max())]
    if int(np.argmax(column)) == per // 2:
        assert column[per // 2 + 1] == column[per // 2]
    # argument checks of the host routine
    import ctypes as C
    idx, val = (C.c_int * 16)(), (C.c_float * 16)()
    L = io._L()
    assert not L.esp_interop_expansion_head_argmax(head.ref, s.ref, 3, 12, 1, 0, idx, val)                 # spatial not a multiple of 8
    assert not L.esp_interop_expansion_head_argmax(head.ref, s.ref, 3, spatial, spatial + 1, 0, idx, val)   # more streams than lanes
    assert not L.esp_interop_expansion_head_argmax(head.ref, s.ref, 4, spatial, 1, 0, idx, val)             # region past the surface
    assert not L.esp_interop_expansion_head_create(w.ctypes.data_as(C.c_void_p), bottleneck, groups, 65536 + groups)
    head.close()
