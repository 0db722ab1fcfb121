"""GPU parity of the seam's resident ops against the oracle, through the C ABI."""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPES = [(2304, 768), (768, 768), (3072, 768), (768, 3072)]   # the benchmark's int8 matvec sweep


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def test_backend_self_test(backend):
    """matmul / sgemm KATs (gpu/cuda/backend_cuda.cu:514-529) and resident-op KATs
    (gpu/metal/backend_metal_ops.m:1038-1107) inside the library."""
    _announce("self_test")
    rc, msg = backend.self_test()
    assert rc == 0, msg


def test_matmul_kat_through_function_pointer(backend):
    _announce("matmul KAT")
    x = np.array([[1.0, 2.0, 3.0], [-1.0, 0.5, 2.0]], np.float32)
    w = backend.keep(np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], np.float32))
    b = backend.keep(np.array([0.5, -0.5, 1.0, 2.0], np.float32))
    out = backend.matmul(x, w, b)
    assert np.allclose(out, [[1.5, 1.5, 4.0, 8.0], [-0.5, 0.0, 3.0, 3.5]], atol=1e-5)
    c = np.zeros((2, 4), np.float32)
    backend.sgemm(0, 1, 2, 4, 3, 1.0, x, 3, w, 3, 0.0, c, 4)
    assert np.allclose(c, [[1, 2, 3, 6], [-1, 0.5, 2, 1.5]], atol=1e-5)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("arith", [0, 1])
def test_int8_matvec_bit_exact_integers(backend, pkg, orc, nerr, shape, arith):
    """Packed weights, int8 activations, activation scale and int32 accumulators bit-exact; f32 output 1e-5."""
    n, k = shape
    _announce("int8 matvec %dx%d arith=%d" % (n, k, arith))
    rng = np.random.default_rng(100 + n + k)
    w = backend.keep((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal(k).astype(np.float32)
    bias = backend.keep((rng.standard_normal(n) * 0.1).astype(np.float32))
    # the library's own load-time quantiser == the oracle's == (tested on the CPU) the compiled reference's
    q, s = pkg.quantize_weight_int8(backend.lib, w, arith)
    oq, os_ = orc.quantize_weight_int8(w, arith)
    assert np.array_equal(q, oq) and np.array_equal(s.view(np.uint32), os_.view(np.uint32))
    backend.set_quant(pkg.INT8, arith)
    din, dout = backend.alloc(k).write(x), backend.alloc(n)
    dqx, dsx, dacc = backend.alloc(k // 4), backend.alloc(1), backend.alloc(n)
    backend.matmul_probe(din.ptr, dout.ptr, k, n, w, bias, dqx.ptr, dsx.ptr, dacc.ptr)
    got = dout.read()
    qx = dqx.read(dtype=np.int8)
    sx = dsx.read()[0]
    acc = dacc.read(dtype=np.int32)
    oqx, osx = orc.quantize_act_int8(x, arith)
    want, oacc = orc.matvec_q8(oqx, osx, oq, os_, bias)
    assert np.array_equal(qx, oqx), "int8 activations differ"
    assert np.float32(sx).view(np.uint32) == np.float32(osx).view(np.uint32), "activation scale differs"
    assert np.array_equal(acc, oacc), "int32 accumulators differ"
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "f32 epilogue differs bitwise"
    assert nerr(got, want) < 1e-5
    for b in (din, dout, dqx, dsx, dacc):
        b.free()
    backend.set_quant(pkg.F32)


@pytest.mark.parametrize("shape", SHAPES)
def test_int4_matvec_group_accumulators(backend, pkg, orc, nerr, shape):
    n, k = shape
    _announce("int4 matvec %dx%d" % (n, k))
    rng = np.random.default_rng(200 + n + k)
    w = backend.keep((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal(k).astype(np.float32)
    rc, q, s = pkg.quantize_weight_int4(backend.lib, w, 0)
    oq, os_ = orc.quantize_weight_int4(w, 0)
    assert rc == 0 and np.array_equal(q, oq) and np.array_equal(s.view(np.uint32), os_.view(np.uint32))
    backend.set_quant(pkg.INT4)
    din, dout = backend.alloc(k).write(x), backend.alloc(n)
    dqx, dsx, dacc = backend.alloc(k // 4), backend.alloc(1), backend.alloc(n * (k // 32))
    backend.matmul_probe(din.ptr, dout.ptr, k, n, w, None, dqx.ptr, dsx.ptr, dacc.ptr)
    got = dout.read()
    acc = dacc.read(dtype=np.int32).reshape(n, k // 32)
    oqx, osx = orc.quantize_act_int8(x)
    want, oacc = orc.matvec_q4(oqx, osx, oq, os_)
    assert np.array_equal(dqx.read(dtype=np.int8), oqx)
    assert np.array_equal(acc, oacc), "per-group int32 accumulators differ"
    # the group sum is a lane-local sequence followed by a butterfly, not the reference's single sequence
    assert nerr(got, want) < 1e-5
    for b in (din, dout, dqx, dsx, dacc):
        b.free()
    backend.set_quant(pkg.F32)


@pytest.mark.parametrize("qtype_name,tol", [("f32", 1e-5), ("f16", 1e-5)])
@pytest.mark.parametrize("shape", SHAPES)
def test_float_matvec(backend, pkg, orc, nerr, shape, qtype_name, tol):
    """f32 weights within 1e-5; f16 weights (exact widening, f32 FMA, f32 activations) within 1e-5 of the
    oracle's matvec_f16 and within 2e-3 of the f32-weight result."""
    n, k = shape
    _announce("%s matvec %dx%d" % (qtype_name, n, k))
    rng = np.random.default_rng(300 + n + k)
    w = backend.keep((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal(k).astype(np.float32)
    bias = backend.keep((rng.standard_normal(n) * 0.1).astype(np.float32))
    qtype = pkg.F32 if qtype_name == "f32" else pkg.F16
    backend.set_quant(qtype)
    din, dout = backend.alloc(k).write(x), backend.alloc(n)
    backend.matmul_d2d(din.ptr, dout.ptr, 1, k, n, w, bias)
    got = dout.read()
    if qtype == pkg.F32:
        want = orc.matvec_f32(x, w, bias)
    else:
        bits = pkg.convert_weight_f16(backend.lib, w)
        assert np.array_equal(bits, orc.f32_to_f16_bits(w)), "f16 weight bits differ"
        want = orc.matvec_f16(x, bits, bias)
        assert nerr(got, orc.matvec_f32(x, w, bias)) < 2e-3
    assert nerr(got, want) < tol
    din.free()
    dout.free()
    backend.set_quant(pkg.F32)


@pytest.mark.parametrize("qtype_name", ["int8", "int4", "f16", "f32"])
def test_batched_matvec_bit_identical_to_solo(backend, pkg, qtype_name):
    """self_test_batched (src/qmat.c:1107-1179) on the GPU: B=5 scattered rows, memcmp against one-at-a-time;
    then B = 8 and B = 13 (two weight passes)."""
    qtype = {"int8": pkg.INT8, "int4": pkg.INT4, "f16": pkg.F16, "f32": pkg.F32}[qtype_name]
    n, k = 768, 768
    _announce("batched matvec %s" % qtype_name)
    rng = np.random.default_rng(400)
    w = backend.keep((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    bias = backend.keep((rng.standard_normal(n) * 0.1).astype(np.float32))
    backend.set_quant(qtype)
    for B in (5, 8, 13):
        xs = rng.standard_normal((B, k)).astype(np.float32)
        xs[B // 2] = 0.0                                   # an all-zero activation row (sx == 0)
        dins = [backend.alloc(k).write(xs[b]) for b in range(B)]
        douts = [backend.alloc(n) for _ in range(B)]
        solo = []
        for b in range(B):
            backend.matmul_d2d(dins[b].ptr, douts[b].ptr, 1, k, n, w, bias)
            solo.append(douts[b].read())
        backend.matmul_d2d_batched([d.ptr for d in dins], [d.ptr for d in douts], k, n, w, bias)
        for b in range(B):
            got = douts[b].read()
            assert np.array_equal(got.view(np.uint32), solo[b].view(np.uint32)), "B=%d stream %d" % (B, b)
        assert np.array_equal(solo[B // 2], bias)          # zero activation -> exactly the bias
        for d in dins + douts:
            d.free()
    backend.set_quant(pkg.F32)


def test_matmul_rows_and_generic_shapes(backend, pkg, orc, nerr):
    """rows > 1 through matmul_d2d (prefill-like), shapes the fused matvec does not take, host-pointer matmul."""
    _announce("generic matmul shapes")
    rng = np.random.default_rng(500)
    for rows, k, n in ((1, 100, 37), (3, 48, 50), (40, 768, 96), (16, 768, 768), (17, 256, 64)):
        w = backend.keep((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        bias = backend.keep(rng.standard_normal(n).astype(np.float32))
        x = rng.standard_normal((rows, k)).astype(np.float32)
        want = np.stack([orc.matvec_f32(r, w, bias) for r in x])
        din, dout = backend.alloc(rows * k).write(x), backend.alloc(rows * n)
        backend.matmul_d2d(din.ptr, dout.ptr, rows, k, n, w, bias)
        assert nerr(dout.read().reshape(rows, n), want) < 1e-5, (rows, k, n)
        assert nerr(backend.matmul(x, w, bias), want) < 1e-5
        din.free()
        dout.free()
    # int4 request on a width that is not a multiple of 32 silently stays f32 (src/qmat.c:630)
    backend.set_quant(pkg.INT4)
    w = backend.keep((rng.standard_normal((64, 48)) * 0.05).astype(np.float32))
    x = rng.standard_normal((1, 48)).astype(np.float32)
    assert nerr(backend.matmul(x, w), orc.matvec_f32(x[0], w)[None]) < 1e-5
    backend.set_quant(pkg.F32)


def test_many_row_products_on_the_matrix_cores(backend, nerr):
    """Products of 24 rows and more take the f32 MFMA tile kernel: matmul (NT, bias) and sgemm with op(A) = A (NT and NN,
    padded leading dimensions, alpha / beta), at tile-aligned and ragged shapes, against float64.  1e-5 normalised."""
    _announce("many-row f32 products (MFMA)")
    rng = np.random.default_rng(510)
    for rows, k, n in ((24, 768, 2304), (64, 768, 768), (100, 3072, 768), (300, 70, 50), (33, 33, 65), (257, 129, 190), (512, 768, 3072)):
        w = backend.keep((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        bias = backend.keep(rng.standard_normal(n).astype(np.float32))
        x = rng.standard_normal((rows, k)).astype(np.float32)
        want = x.astype(np.float64) @ w.astype(np.float64).T + bias
        din, dout = backend.alloc(rows * k).write(x), backend.alloc(rows * n)
        backend.matmul_d2d(din.ptr, dout.ptr, rows, k, n, w, bias)
        assert nerr(dout.read().reshape(rows, n), want) < 1e-5, (rows, k, n)
        backend.matmul_d2d(din.ptr, dout.ptr, rows, k, n, w, None)
        assert nerr(dout.read().reshape(rows, n), want - bias) < 1e-5, (rows, k, n)
        din.free()
        dout.free()
    for tb in (1, 0):
        for m, n, k, pad in ((64, 64, 64, 0), (128, 200, 64, 0), (37, 130, 64, 3), (200, 64, 257, 4), (25, 31, 7, 1), (256, 256, 768, 8)):
            lda, ldb, ldc = k + pad, (k if tb else n) + pad, n + pad
            a = rng.standard_normal((m, lda)).astype(np.float32)
            b = rng.standard_normal(((n if tb else k), ldb)).astype(np.float32)
            c0 = rng.standard_normal((m, ldc)).astype(np.float32)
            a64, b64 = a[:, :k].astype(np.float64), (b[:, :k].T if tb else b[:, :n]).astype(np.float64)
            for alpha, beta in ((1.0, 0.0), (0.125, 0.5)):
                c = c0.copy()
                backend.sgemm(0, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)
                want = alpha * (a64 @ b64) + beta * c0[:, :n]
                assert nerr(c[:, :n], want) < 1e-5, (tb, m, n, k, pad, alpha, beta)
                assert np.array_equal(c[:, n:], c0[:, n:]), "columns beyond n were written"


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
def test_cross_kv_from_resident_memory(backend, pkg, orc, nerr, qtype_name):
    """decoder_cache_init's cross K/V (src/graph.c:3002-3028) from encoder memory on the device: per layer LayerNorm ->
    kv product -> K | V halves, for memories of 1, 9 (<= 16 rows: the current quantisation, checked against the oracle's
    quantised product of the whole kv matrix), 40 and 300 rows (f32, against float64)."""
    _announce("cross K/V precompute, %s" % qtype_name)
    qt = {"f32": pkg.F32, "int8": pkg.INT8, "int4": pkg.INT4}[qtype_name]
    rng = np.random.default_rng(520)
    layers, width, xw = 3, 768, 768
    gains = [backend.keep((1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)) for _ in range(layers)]
    biases = [backend.keep((0.02 * rng.standard_normal(width)).astype(np.float32)) for _ in range(layers)]
    kvw = [backend.keep((0.02 * rng.standard_normal((2 * xw, width))).astype(np.float32)) for _ in range(layers)]
    backend.set_quant(qt)
    try:
        for T, with_bias in ((1, False), (9, True), (40, False), (300, True)):
            memory = rng.standard_normal((T, width)).astype(np.float32)
            dmem = backend.alloc(T * width).write(memory)
            dck, dcv = backend.alloc(layers * T * xw), backend.alloc(layers * T * xw)
            backend.cross_kv_dev(dmem.ptr, T, width, gains, biases if with_bias else None, kvw, xw, dck.ptr, dcv.ptr)
            gk, gv = dck.read().reshape(layers, T, xw), dcv.read().reshape(layers, T, xw)
            for l in range(layers):
                normed = np.stack([orc.layernorm(r, gains[l], biases[l] if with_bias else None) for r in memory])
                if T <= 16 and qt != pkg.F32:
                    pw = orc.PackedWeight(kvw[l], {pkg.INT8: orc.INT8, pkg.INT4: orc.INT4}[qt])
                    want = np.stack([orc.linear(pw, r) for r in normed])
                    tol = 1e-5
                else:
                    want = normed.astype(np.float64) @ kvw[l].astype(np.float64).T
                    tol = 1e-5
                assert nerr(gk[l], want[:, :xw]) < tol, (T, l, "k")
                assert nerr(gv[l], want[:, xw:]) < tol, (T, l, "v")
            for d in (dmem, dck, dcv):
                d.free()
    finally:
        backend.set_quant(pkg.F32)


def test_decoder_head_argmax_for_all_slots_and_streams(backend, pkg, orc):
    """slot_advance's head (src/graph.c:3873-3905): per slot and stacked stream the constrained first maximum of
    final_proj's logits, stored codes and EOS bookkeeping, for five slots in one call -- against the oracle's f32 matvec +
    constrained argmax per stream.  EOS is forced into chosen streams through the bias; one of those slots forbids it.
    Runs under int8 quantisation too: the head stays f32 like the reference's loop."""
    _announce("decoder head: batched constrained argmax")
    rng = np.random.default_rng(530)
    width, streams, vocab, codebook, eos, per_frame = 768, 8, 1024, 1000, 1010, 4
    w = backend.keep((rng.standard_normal((streams * vocab, width)) * 0.05).astype(np.float32))
    bias = (rng.standard_normal(streams * vocab) * 0.1).astype(np.float32)
    bias[5 * vocab + eos] = 50.0        # stream 5 (frame 1) says EOS wherever it is allowed
    bias[2 * vocab + 1017] = 80.0       # a forbidden id with the largest logit of stream 2: never chosen
    bias = backend.keep(bias)
    hidden = rng.standard_normal((5, width)).astype(np.float32)
    forbid = [0, 1, 0, 0, 1]
    bufs = [backend.alloc(width).write(h) for h in hidden]
    for qt in (pkg.F32, pkg.INT8):
        backend.set_quant(qt)
        values, stored, saw, frame = backend.head_argmax([d.ptr for d in bufs], width, w, bias, streams, vocab, codebook, eos, per_frame, forbid)
        for b in range(5):
            logits = orc.matvec_f32(hidden[b], w, bias).reshape(streams, vocab)
            want_saw, want_frame = 0, None
            for s in range(streams):
                rc, want = orc.argmax_constrained(logits[s], codebook, eos, not forbid[b])
                assert rc == 0
                got = int(values[b, s])
                if got != want:      # only a tie within rounding may differ
                    assert abs(float(logits[s][got]) - float(logits[s][want])) <= 1e-5 * np.abs(logits[s]).max(), (b, s, got, want)
                assert got < codebook or (got == eos and not forbid[b])
                assert int(stored[b, s]) == (got if got < codebook else 0)
                if got == eos:
                    want_saw = 1
                    want_frame = s // per_frame if want_frame is None else min(want_frame, s // per_frame)
            assert int(saw[b]) == want_saw and frame[b] == want_frame, (b, saw[b], frame[b])
        assert saw[0] == 1 and frame[0] == 1 and saw[1] == 0 and values[0, 5] == eos
    backend.set_quant(pkg.F32)
    with pytest.raises(pkg.BackendError):
        backend.head_argmax([d.ptr for d in bufs], width, w, bias, streams, vocab, vocab + 1, eos, per_frame, forbid)   # more codes than vocabulary
    for d in bufs:
        d.free()


def test_layernorm_gelu_residual_softmax(backend, orc, nerr):
    _announce("layernorm/gelu/residual/softmax")
    rng = np.random.default_rng(600)
    x = (rng.standard_normal((5, 768)) * 3 + 0.5).astype(np.float32)
    gain = backend.keep((1 + 0.1 * rng.standard_normal(768)).astype(np.float32))
    beta = backend.keep((0.02 * rng.standard_normal(768)).astype(np.float32))
    din, dout = backend.alloc(x.size).write(x), backend.alloc(x.size)
    backend.layer_norm_inplace(din.ptr, dout.ptr, gain, 5, 768)
    assert nerr(dout.read().reshape(5, 768), orc.layernorm(x, gain)) < 1e-5
    backend.layer_norm_dev(din.ptr, dout.ptr, gain, beta, 5, 768)
    assert nerr(dout.read().reshape(5, 768), orc.layernorm(x, gain, beta)) < 1e-5
    # KAT: layernorm(1..4) = -+1.34164 (src/kernels.c:473-482; eps 1e-5 here)
    g4 = backend.keep(np.ones(4, np.float32))
    d4 = backend.alloc(4).write(np.array([1, 2, 3, 4], np.float32))
    backend.layer_norm_inplace(d4.ptr, d4.ptr, g4, 1, 4)
    r = d4.read()
    assert abs(r[0] + 1.34164) < 1e-4 and abs(r[3] - 1.34164) < 1e-4
    # GELU: gelu(0) = 0, gelu(1) = 0.8411920 (src/kernels.c:493-499) and 3072 values vs the scalar libm form
    v = np.concatenate([np.array([-1.0, 0.0, 1.0]), np.linspace(-9, 9, 3069)]).astype(np.float32)
    dv = backend.alloc(v.size).write(v)
    backend.gelu_inplace(dv.ptr, v.size)
    gv = dv.read()
    assert abs(gv[1]) < 1e-6 and abs(gv[2] - 0.8411920) < 1e-5
    assert np.max(np.abs(gv - orc.gelu_scalar(v))) < 1e-5 * np.max(np.abs(v))
    # residual
    a = rng.standard_normal(768).astype(np.float32)
    b = rng.standard_normal(768).astype(np.float32)
    da, db = backend.alloc(768).write(a), backend.alloc(768).write(b)
    backend.residual_inplace(da.ptr, db.ptr, 768)
    assert np.array_equal(da.read(), a + b)
    # a HOST row in the device slot (src/graph.c:1118-1120) resolves through the weight cache
    hostrow = backend.keep(rng.standard_normal(768).astype(np.float32))
    backend.residual_inplace(da.ptr, hostrow.ctypes.data, 768)
    assert np.array_equal(da.read(), (a + b) + hostrow)
    # masked softmax (src/backend.c:602-619) on 8 x 1024
    logits = (rng.standard_normal((8, 1024)) * 4).astype(np.float32)
    dl = backend.alloc(logits.size).write(logits)
    backend.softmax_dev(dl.ptr, 8, 1024, 700)
    got = dl.read().reshape(8, 1024)
    assert nerr(got, orc.softmax_masked(logits, 700)) < 1e-5 and not got[:, 700:].any()
    # copy / scale / clip
    dc = backend.alloc(768)
    backend.copy_dev(dc.ptr, da.ptr, 768)
    assert np.array_equal(dc.read(), da.read())
    backend.scale_dev(dc.ptr, 768, 0.25)
    assert np.array_equal(dc.read(), da.read() * np.float32(0.25))
    dclip = backend.alloc(4).write(np.array([-2.0, np.nan, 0.5, 7.0], np.float32))
    backend.clip_dev(dclip.ptr, 4)
    assert dclip.read().tolist() == [-1.0, 0.0, 0.5, 1.0]
    for d in (din, dout, d4, dv, da, db, dl, dc, dclip):
        d.free()


def test_upload_operator_download(backend, orc):
    """The engine's use of the upload buffer (src/graph.c:2263-2268): upload, one operator, download.  With argmax as
    the operator the buffer must come back untouched -- its result has a word of its own -- and with snake as the
    operator it must come back transformed."""
    _announce("upload -> operator -> download")
    rng = np.random.default_rng(701)
    logits = rng.standard_normal(1024).astype(np.float32)
    logits[0] = 3.25
    logits[77] = 8.5
    dev = backend.upload(logits)
    assert backend.argmax_dev(dev, 1024, 1024, 0, False) == 77
    assert backend.argmax_dev(dev, 1024, 50, 0, False) == orc.argmax_constrained(logits, 50, 0, False)[1]
    assert np.array_equal(backend.download(dev, 1024).view(np.uint32), logits.view(np.uint32))
    signal = rng.standard_normal(6 * 40).astype(np.float32)
    alpha = (rng.random(3) + 0.5).astype(np.float32)
    dev = backend.upload(signal)
    backend.snake_dev(dev, alpha, 6, 40, 3)
    got = backend.download(dev, signal.size)
    want = orc.snake(signal.reshape(6, 40), alpha, 3).reshape(-1)
    assert np.max(np.abs(got - want)) <= 1e-6 * max(1.0, float(np.max(np.abs(want))))
    with pytest.raises(Exception):
        backend.upload(np.zeros(0, np.float32))


def test_argmax(backend, orc):
    _announce("argmax")
    rng = np.random.default_rng(700)
    logits = rng.standard_normal(2048).astype(np.float32)
    logits[100] = logits[900] = 9.0        # tie: the first index wins
    logits[2030] = 11.0                    # above codebook: only counts when it is the eos id
    d = backend.alloc(2048).write(logits)
    for codebook, eos, allow in ((2016, 2030, False), (2016, 2030, True), (2016, 2040, True), (50, 2030, False), (2048, 0, False)):
        assert backend.argmax_dev(d.ptr, 2048, codebook, eos, allow) == orc.argmax_constrained(logits, codebook, eos, allow)[1]
    dinf = backend.alloc(8).write(np.full(8, -np.inf, np.float32))
    assert backend.argmax_dev(dinf.ptr, 8, 8, 0, False) == 0
    dnan = backend.alloc(2).write(np.array([np.nan, 1.0], np.float32))
    assert backend.argmax_dev(dnan.ptr, 2, 2, 0, False) == 1
    with pytest.raises(Exception):
        backend.argmax_dev(d.ptr, 2048, 4096, 0, False)     # codebook > vocab (src/backend.c:829-830)
    for x in (d, dinf, dnan):
        x.free()


@pytest.mark.parametrize("heads,hw,L", [(12, 64, 1), (12, 64, 63), (12, 64, 64), (12, 64, 65), (12, 64, 300),
                                        (12, 64, 1024), (1, 768, 200), (3, 20, 70), (1, 2, 5),
                                        (12, 64, 127), (12, 64, 128), (12, 64, 129), (12, 64, 257), (1, 768, 16), (1, 768, 17), (1, 768, 256), (1, 256, 100), (2, 512, 33), (1, 1024, 40)])
def test_self_and_cross_attention(backend, orc, nerr, heads, hw, L):
    """Split-L attention against the reference's two-pass order, incl. chunk edges (63/64/65), one wide head
    (what the engine passes for cross attention; its read-only form has a kernel of its own for head widths that are
    multiples of 256, sixteen rows per workgroup: chunk edges 16/17) and head widths that are not multiples of 4."""
    _announce("attention heads=%d hw=%d L=%d" % (heads, hw, L))
    rng = np.random.default_rng(800 + heads + hw + L)
    width = heads * hw
    scale = 1.0 / math.sqrt(hw)
    qkv = rng.standard_normal(3 * width).astype(np.float32)
    kc = np.zeros((L + 2, width), np.float32)
    vc = np.zeros((L + 2, width), np.float32)
    kc[:L - 1] = rng.standard_normal((L - 1, width))
    vc[:L - 1] = rng.standard_normal((L - 1, width))
    kc[L:] = 77.0     # rows beyond `valid` must be ignored and left alone
    vc[L:] = -77.0
    ok, ov = kc.copy(), vc.copy()
    want = orc.self_attention(qkv, ok, ov, L - 1, width, L, heads, hw, scale)
    dq, dk, dv, do = backend.alloc(qkv.size).write(qkv), backend.alloc(kc.size).write(kc), backend.alloc(vc.size).write(vc), backend.alloc(width)
    backend.self_attention_dev(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, scale, do.ptr)
    assert nerr(do.read(), want) < 1e-5
    assert np.array_equal(dk.read().reshape(kc.shape), ok), "KV append must write exactly row `position` of K"
    assert np.array_equal(dv.read().reshape(vc.shape), ov), "KV append must write exactly row `position` of V"
    # cross: read-only over the same caches
    wantx = orc.cross_attention(qkv[:width], ok, ov, L, width, heads, hw, scale)
    backend.cross_attention_dev(dq.ptr, dk.ptr, dv.ptr, L, width, heads, hw, scale, do.ptr)
    assert nerr(do.read(), wantx) < 1e-5
    assert np.array_equal(dk.read().reshape(kc.shape), ok)
    for d in (dq, dk, dv, do):
        d.free()


def test_batched_attention_bit_identical_to_solo(backend, orc, nerr):
    _announce("batched attention")
    rng = np.random.default_rng(900)
    heads, hw = 12, 64
    width = heads * hw
    scale = 0.125
    lengths = [64, 2048, 777, 65, 1, 300, 1999, 128]
    B = len(lengths)
    bufs = []
    for L in lengths:
        qkv = rng.standard_normal(3 * width).astype(np.float32)
        kc = rng.standard_normal((L, width)).astype(np.float32)
        vc = rng.standard_normal((L, width)).astype(np.float32)
        bufs.append((qkv, kc, vc, backend.alloc(qkv.size).write(qkv), backend.alloc(kc.size).write(kc),
                     backend.alloc(vc.size).write(vc), backend.alloc(width)))
    solo = []
    for (qkv, kc, vc, dq, dk, dv, do), L in zip(bufs, lengths):
        backend.self_attention_dev(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, scale, do.ptr)
        solo.append(do.read())
        ok, ov = kc.copy(), vc.copy()
        assert nerr(solo[-1], orc.self_attention(qkv, ok, ov, L - 1, width, L, heads, hw, scale)) < 1e-5
    backend.self_attention_dev_batched([b[3].ptr for b in bufs], [b[4].ptr for b in bufs], [b[5].ptr for b in bufs],
                                       [L - 1 for L in lengths], width, lengths, heads, hw, scale, [b[6].ptr for b in bufs])
    for b, buf in enumerate(bufs):
        assert np.array_equal(buf[6].read().view(np.uint32), solo[b].view(np.uint32)), "self stream %d" % b
    solo = []
    for (qkv, kc, vc, dq, dk, dv, do), L in zip(bufs, lengths):
        backend.cross_attention_dev(dq.ptr, dk.ptr, dv.ptr, L, width, heads, hw, scale, do.ptr)
        solo.append(do.read())
    backend.cross_attention_dev_batched([b[3].ptr for b in bufs], [b[4].ptr for b in bufs], [b[5].ptr for b in bufs],
                                        lengths, width, heads, hw, scale, [b[6].ptr for b in bufs])
    for b, buf in enumerate(bufs):
        assert np.array_equal(buf[6].read().view(np.uint32), solo[b].view(np.uint32)), "cross stream %d" % b
    for buf in bufs:
        for d in buf[3:]:
            d.free()


def test_embedding_gather_bit_exact(backend):
    """Text rows are a memcpy (src/graph.c:729-737); the audio frame is a sum of table rows / count (:764-804)."""
    _announce("gather")
    rng = np.random.default_rng(1000)
    table = backend.keep((rng.standard_normal((4096, 768)) * 0.02).astype(np.float32))
    pos = backend.keep((rng.standard_normal((512, 768)) * 0.02).astype(np.float32))
    ids = rng.integers(0, 4096, 256).astype(np.int32)
    dout = backend.alloc(256 * 768)
    backend.embed_gather([table], ids, 768, 1.0, None, 0, dout.ptr)
    assert np.array_equal(dout.read().reshape(256, 768).view(np.uint32), table[ids].view(np.uint32))
    backend.embed_gather([table], ids, 768, 1.0, pos, 3, dout.ptr)
    assert np.array_equal(dout.read().reshape(256, 768), table[ids] + pos[3:259])
    tables = [backend.keep((rng.standard_normal((2024, 768)) * 0.02).astype(np.float32)) for _ in range(16)]
    fid = rng.integers(0, 2024, (2, 16)).astype(np.int32)
    backend.embed_gather(tables, fid, 768, 1.0 / 16.0, None, 0, dout.ptr)
    want = np.zeros((2, 768), np.float32)
    for t in range(2):
        acc = tables[0][fid[t, 0]].copy()
        for j in range(1, 16):
            acc = acc + tables[j][fid[t, j]]
        want[t] = acc * np.float32(1.0 / 16.0)
    assert np.array_equal(dout.read(2 * 768).reshape(2, 768), want)
    with pytest.raises(Exception):
        backend.embed_gather([table], np.array([4096], np.int32), 768, 1.0, None, 0, dout.ptr)   # out of vocabulary
    dout.free()


def test_embedding_gather_decode_loop_positions(backend):
    """One token per call at a growing position (a decode loop), then a prefill range over rows already seen and beyond:
    every call adds the right position rows, from one device copy of the table that grows as rows are reached."""
    _announce("gather: positions of a decode loop")
    rng = np.random.default_rng(1001)
    table = backend.keep((rng.standard_normal((300, 768)) * 0.02).astype(np.float32))
    pos = backend.keep((rng.standard_normal((400, 768)) * 0.02).astype(np.float32))
    dout = backend.alloc(64 * 768)
    for step in range(130):
        ids = np.array([step % 300], np.int32)
        backend.embed_gather([table], ids, 768, 1.0, pos, step, dout.ptr)
        assert np.array_equal(dout.read(768), table[ids[0]] + pos[step]), "step %d" % step
    ids = rng.integers(0, 300, 64).astype(np.int32)
    for offset in (0, 100, 336):
        backend.embed_gather([table], ids, 768, 1.0, pos, offset, dout.ptr)
        assert np.array_equal(dout.read().reshape(64, 768), table[ids] + pos[offset:offset + 64]), "offset %d" % offset
    dout.free()


def test_freed_buffers_outlive_the_work_that_reads_them(backend):
    """mynah_hip_dev_free does not wait for the stream: a buffer freed right after a launch that reads it is still read
    correctly, and hundreds of allocate-use-free rounds neither stall nor run out of memory."""
    _announce("deferred frees")
    rng = np.random.default_rng(1002)
    n = 1 << 22
    want = rng.standard_normal(n).astype(np.float32)
    keep = backend.alloc(n)
    for _ in range(200):
        src = backend.alloc(n).write(want)
        backend.copy_dev(keep.ptr, src.ptr, n)
        src.free()
    assert np.array_equal(keep.read(), want)
    keep.free()


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4", "f16"])
def test_fused_seam_chains_match_separate_launches(backend, pkg, nerr, qtype_name):
    """Consecutive single-row seam calls that continue on each other's buffers run as one launch (LayerNorm + product
    (+ GELU), product + GELU, product + residual).  Every buffer the separate calls write must hold what they would have
    written: a synchronisation between two calls keeps them apart, which gives the reference values.  The product's own
    arithmetic is the same kernel code in both cases: bit-identical; the LayerNorm row comes from the matvec's prologue
    instead of the stand-alone kernel (other reduction tree): 1e-6 normalised, and what is computed from it 1e-5 (f32,
    f16) or, with quantised activations, within one quantisation step of a weight row's reach (2e-2)."""
    _announce("fused seam chains " + qtype_name)
    qt = {"f32": pkg.F32, "int8": pkg.INT8, "int4": pkg.INT4, "f16": pkg.F16}[qtype_name]
    tol = {"f32": 1e-5, "f16": 1e-5, "int8": 2e-2, "int4": 2e-2}[qtype_name]
    backend.set_quant(qt)
    rng = np.random.default_rng(77)
    w, f = 768, 3072
    gain = backend.keep((1 + 0.1 * rng.standard_normal(w)).astype(np.float32))
    up = backend.keep((0.02 * rng.standard_normal((f, w))).astype(np.float32))
    down = backend.keep((0.02 * rng.standard_normal((w, f))).astype(np.float32))
    x0 = rng.standard_normal(w).astype(np.float32)
    bufs = {n: backend.alloc(s) for n, s in (("x", w), ("nrm", w), ("hidden", f), ("proj", w))}

    def run(separate):
        gap = backend.sync if separate else (lambda: None)
        bufs["x"].write(x0)
        for b in ("nrm", "hidden", "proj"):
            bufs[b].write(np.zeros(bufs[b].n, np.float32))
        # the engine's feed-forward block (src/graph.c:3451-3476)
        backend.layer_norm_inplace(bufs["x"].ptr, bufs["nrm"].ptr, gain, 1, w)
        gap()
        backend.matmul_d2d(bufs["nrm"].ptr, bufs["hidden"].ptr, 1, w, f, up)
        gap()
        backend.gelu_inplace(bufs["hidden"].ptr, f)
        gap()
        backend.matmul_d2d(bufs["hidden"].ptr, bufs["proj"].ptr, 1, f, w, down)
        gap()
        backend.residual_inplace(bufs["x"].ptr, bufs["proj"].ptr, w)
        return {n: bufs[n].read() for n in bufs}

    want = run(True)
    got = run(False)
    assert nerr(got["nrm"], want["nrm"]) < 1e-6
    assert nerr(got["hidden"], want["hidden"]) < tol
    assert nerr(got["proj"], want["proj"]) < tol
    assert nerr(got["x"], want["x"]) < tol
    assert np.array_equal(got["x"], x0 + got["proj"]), "residual row and product row disagree"

    # product + GELU and product + residual on rows that are the same in both runs: bit-identical
    h0 = rng.standard_normal(f).astype(np.float32)

    def tail(separate):
        gap = backend.sync if separate else (lambda: None)
        bufs["x"].write(x0)
        bufs["hidden"].write(h0)
        backend.matmul_d2d(bufs["hidden"].ptr, bufs["proj"].ptr, 1, f, w, down)
        gap()
        backend.residual_inplace(bufs["x"].ptr, bufs["proj"].ptr, w)
        backend.matmul_d2d(bufs["x"].ptr, bufs["hidden"].ptr, 1, w, f, up)
        gap()
        backend.gelu_inplace(bufs["hidden"].ptr, f)
        return {n: bufs[n].read() for n in ("x", "proj", "hidden")}

    want, got = tail(True), tail(False)
    for n in want:
        assert np.array_equal(got[n], want[n]), n

    # chains that must NOT join: the residual add updates the row the product reads
    def aliased(separate):
        gap = backend.sync if separate else (lambda: None)
        bufs["x"].write(x0)
        backend.matmul_d2d(bufs["x"].ptr, bufs["proj"].ptr, 1, w, w, backend.keep(np.ascontiguousarray(down[:, :w])))
        gap()
        backend.residual_inplace(bufs["x"].ptr, bufs["proj"].ptr, w)
        # a LayerNorm whose row nobody multiplies, then an unrelated call
        backend.layer_norm_inplace(bufs["x"].ptr, bufs["nrm"].ptr, gain, 1, w)
        gap()
        backend.scale_dev(bufs["nrm"].ptr, w, 0.5)
        return {n: bufs[n].read() for n in ("x", "proj", "nrm")}

    want, got = aliased(True), aliased(False)
    for n in want:
        assert np.array_equal(got[n], want[n]), n
    for b in bufs.values():
        b.free()
    backend.set_quant(pkg.F32)


def test_batched_wide_head_cross_attention_bit_identical_to_solo(backend, orc, nerr):
    """Ragged memories behind one 768-wide head: each stream in the batch equals the same stream alone, bit for bit, and
    a stream without memory gets a zero context (src/graph.c:3237-3244)."""
    _announce("batched wide-head cross attention")
    rng = np.random.default_rng(901)
    hw = 768
    scale = 1.0 / math.sqrt(hw)
    lens = [256, 1, 40, 0, 17, 133]
    qs = [rng.standard_normal(hw).astype(np.float32) for _ in lens]
    ks = [rng.standard_normal((max(n, 1), hw)).astype(np.float32) for n in lens]
    vs = [rng.standard_normal((max(n, 1), hw)).astype(np.float32) for n in lens]
    dq = [backend.alloc(hw).write(q) for q in qs]
    dk = [backend.alloc(k.size).write(k) for k in ks]
    dv = [backend.alloc(v.size).write(v) for v in vs]
    do = [backend.alloc(hw) for _ in lens]
    backend.cross_attention_dev_batched([d.ptr for d in dq], [d.ptr for d in dk], [d.ptr for d in dv], lens, hw, 1, hw, scale,
                                        [d.ptr for d in do])
    together = [d.read() for d in do]
    for b, n in enumerate(lens):
        if n == 0:
            assert not together[b].any()
            continue
        assert nerr(together[b], orc.cross_attention(qs[b], ks[b], vs[b], n, hw, 1, hw, scale)) < 1e-5
        backend.cross_attention_dev(dq[b].ptr, dk[b].ptr, dv[b].ptr, n, hw, 1, hw, scale, do[b].ptr)
        assert np.array_equal(do[b].read(), together[b]), "stream %d" % b
    for d in dq + dk + dv + do:
        d.free()


@pytest.mark.parametrize("qtype_name", ["f32", "int8"])
@pytest.mark.parametrize("heads,hw,L,is_self", [(12, 64, 300, True), (12, 64, 1100, True), (1, 768, 200, False), (12, 64, 90, False)])
def test_fused_attention_fold_matches_separate_launches(backend, pkg, orc, nerr, qtype_name, heads, hw, L, is_self):
    """A single-stream attention call over more than one chunk leaves the fold of its chunks to the product that reads
    its output row (the engine's attention -> output projection -> residual add, src/graph.c:3416-3428).  The joined
    launch must leave in every buffer what the separate calls leave: the attention row (folded in another order: 1e-6
    against the separate call, 1e-5 against the oracle), the product and the updated residual row."""
    _announce("fused attention fold %s heads=%d hw=%d L=%d self=%s" % (qtype_name, heads, hw, L, is_self))
    qt = {"f32": pkg.F32, "int8": pkg.INT8}[qtype_name]
    tol = {"f32": 1e-5, "int8": 2e-2}[qtype_name]
    backend.set_quant(qt)
    rng = np.random.default_rng(1234 + L + hw)
    width = heads * hw
    scale = 1.0 / math.sqrt(hw)
    qkv = rng.standard_normal(3 * width).astype(np.float32)
    kc = rng.standard_normal((L + 1, width)).astype(np.float32)
    vc = rng.standard_normal((L + 1, width)).astype(np.float32)
    wo = backend.keep((0.02 * rng.standard_normal((width, width))).astype(np.float32))
    x0 = rng.standard_normal(width).astype(np.float32)
    dq, dk, dv = backend.alloc(qkv.size).write(qkv), backend.alloc(kc.size), backend.alloc(vc.size)
    dattn, dproj, dx = backend.alloc(width), backend.alloc(width), backend.alloc(width)

    def run(separate):
        gap = backend.sync if separate else (lambda: None)
        dk.write(kc)
        dv.write(vc)
        dx.write(x0)
        dattn.write(np.zeros(width, np.float32))
        if is_self:
            backend.self_attention_dev(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, scale, dattn.ptr)
        else:
            backend.cross_attention_dev(dq.ptr, dk.ptr, dv.ptr, L, width, heads, hw, scale, dattn.ptr)
        gap()
        backend.matmul_d2d(dattn.ptr, dproj.ptr, 1, width, width, wo)
        gap()
        backend.residual_inplace(dx.ptr, dproj.ptr, width)
        return dattn.read(), dproj.read(), dx.read(), dk.read().reshape(kc.shape)

    want = run(True)
    got = run(False)
    ok, ov = kc.copy(), vc.copy()
    ref = orc.self_attention(qkv, ok, ov, L - 1, width, L, heads, hw, scale) if is_self else \
        orc.cross_attention(qkv[:width], kc, vc, L, width, heads, hw, scale)
    assert nerr(got[0], ref) < 1e-5
    assert nerr(got[0], want[0]) < 1e-6
    assert nerr(got[1], want[1]) < tol and nerr(got[2], want[2]) < tol
    assert np.array_equal(got[2], x0 + got[1])
    assert np.array_equal(got[3], want[3]), "cache rows"
    for d in (dq, dk, dv, dattn, dproj, dx):
        d.free()
    backend.set_quant(pkg.F32)


def test_optional_seam_slots(pkg, backend, orc, nerr):
    """The four seam slots graph.c does not call (src/backend.h:59,62-64): causal im2col against its definition, the
    host-pointer GELU in f32 against the oracle's and in double against a float64 evaluation rounded once, and the
    "graph" matmul against the plain host-pointer matmul bit for bit."""
    _announce("optional seam slots")
    rng = np.random.default_rng(777)
    for in_ch, length, kernel, dilation in ((3, 17, 3, 1), (5, 64, 7, 3), (2, 9, 11, 5), (1, 1, 1, 1)):
        x = rng.standard_normal((in_ch, length)).astype(np.float32)
        want = np.zeros((in_ch, kernel, length), np.float32)
        for k in range(kernel):
            shift = (kernel - 1 - k) * dilation
            if shift < length:
                want[:, k, shift:] = x[:, :length - shift]
        din, dcol = backend.alloc(x.size).write(x), backend.alloc(want.size)
        backend.im2col(din.ptr, dcol.ptr, in_ch, length, kernel, dilation)
        got = dcol.read().reshape(want.shape)
        assert np.array_equal(got, want), (in_ch, length, kernel, dilation)
        din.free()
        dcol.free()
    v = (rng.standard_normal(5000) * 3).astype(np.float32)
    v[:4] = [0.0, 1.0, -1.0, 6.5]
    got32 = backend.gelu_host(v.copy())
    assert nerr(got32, orc.gelu_scalar(v.copy())) < 1e-6
    assert abs(float(got32[1]) - 0.8411920) < 1e-6 and got32[0] == 0.0            # src/kernels.c:493-499
    got64 = backend.gelu_host(v.copy(), in_double=True)
    x64 = v.astype(np.float64)
    want64 = (0.5 * x64 * (1.0 + np.tanh(0.7978845608028654 * (x64 + 0.044715 * x64 ** 3)))).astype(np.float32)
    # one rounding of a double result; where 1 + tanh cancels (x below about -5) the two double evaluations may differ in their
    # last bits, which is an absolute difference far below the smallest value compared here
    assert np.allclose(got64, want64, rtol=1.2e-7, atol=1e-12), "double-precision GELU differs from the float64 evaluation by more than a rounding"
    w = backend.keep((rng.standard_normal((40, 96)) * 0.1).astype(np.float32))
    b = backend.keep(rng.standard_normal(40).astype(np.float32))
    rows = rng.standard_normal((3, 96)).astype(np.float32)
    assert np.array_equal(backend.matmul_graph(rows, w, b).view(np.uint32), backend.matmul(rows, w, b).view(np.uint32))
