"""Pins the oracle's integer artefacts: quantisers, activation quantisation, int32 accumulators.

Evidence used, strongest first: the compiled reference (oracle/_ref, stock and strict flag sets),
brute-force tie cases, invariants, and a numpy int64 restatement of the integer dots.
"""
import ctypes as C

import numpy as np
import pytest

SHAPES = [(2304, 768), (768, 768), (3072, 768), (768, 3072)]   # the benchmark's int8 matvec sweep


def _w(shape, seed=0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)).astype(np.float32)


def _tie_matrix():
    """Rows built to provoke rounding ties and corner cases."""
    rng = np.random.default_rng(7)
    rows = []
    for amax in (127.0, 63.5, 1.0, 7.0, 3.5, 1e-3, 1e2):
        grid = np.arange(-127, 128, dtype=np.float32) + np.float32(0.5)   # exact .5 ties after scaling
        row = np.resize(grid * np.float32(amax / 127.0), 768).astype(np.float32)
        row[0] = amax
        rows.append(row)
    rows.append(np.zeros(768, np.float32))                          # all-zero row -> scale 1
    rows.append(np.full(768, 1e-30, np.float32))                    # near-denormal scale
    tiny = np.zeros(768, np.float32)
    tiny[5] = np.float32(1e-38)
    rows.append(tiny)
    rows.append((rng.standard_normal(768) * 10 ** rng.uniform(-4, 2)).astype(np.float32))
    return np.stack(rows)


@pytest.mark.parametrize("shape", SHAPES)
def test_int8_quantiser_matches_compiled_reference(orc, ref, ref_strict, shape):
    w = _w(shape)
    for variant, lib in ((orc.STOCK, ref), (orc.STRICT, ref_strict)):
        q, s = orc.quantize_weight_int8(w, variant)
        rq = np.empty_like(q)
        rs = np.empty_like(s)
        lib.ref_quantize_weight_int8(w, shape[0], shape[1], rq, rs)
        assert np.array_equal(q, rq), "packed int8 weights differ (variant %d)" % variant
        assert np.array_equal(s.view(np.uint32), rs.view(np.uint32)), "int8 scales differ (variant %d)" % variant
        assert np.abs(q.astype(np.int32)).max() <= 127


@pytest.mark.parametrize("shape", SHAPES)
def test_int4_quantiser_matches_compiled_reference(orc, ref, ref_strict, shape):
    w = _w(shape, seed=1)
    for variant, lib in ((orc.STOCK, ref), (orc.STRICT, ref_strict)):
        q, s = orc.quantize_weight_int4(w, variant)
        rq = np.empty_like(q)
        rs = np.empty_like(s)
        lib.ref_quantize_weight_int4(w, shape[0], shape[1], rq, rs)
        assert np.array_equal(q, rq), "packed int4 weights differ (variant %d)" % variant
        assert np.array_equal(s.view(np.uint32), rs.view(np.uint32)), "int4 scales differ (variant %d)" % variant


def test_quantisers_on_tie_rows_match_compiled_reference(orc, ref, ref_strict):
    w = _tie_matrix()
    n, k = w.shape
    for variant, lib in ((orc.STOCK, ref), (orc.STRICT, ref_strict)):
        q, s = orc.quantize_weight_int8(w, variant)
        rq, rs = np.empty_like(q), np.empty_like(s)
        lib.ref_quantize_weight_int8(w, n, k, rq, rs)
        assert np.array_equal(q, rq) and np.array_equal(s.view(np.uint32), rs.view(np.uint32))
        q4, s4 = orc.quantize_weight_int4(w, variant)
        rq4, rs4 = np.empty_like(q4), np.empty_like(s4)
        lib.ref_quantize_weight_int4(w, n, k, rq4, rs4)
        assert np.array_equal(q4, rq4) and np.array_equal(s4.view(np.uint32), rs4.view(np.uint32))
        for row in w:
            qx, sx = orc.quantize_act_int8(row, variant)
            rqx = np.empty_like(qx)
            rsx = lib.ref_quantize_act_int8(rqx, row, k)
            assert np.array_equal(qx, rqx)
            assert np.float32(sx).view(np.uint32) == np.float32(rsx).view(np.uint32)


def test_quantiser_brute_force_ties_and_invariants(orc):
    # half-integer grid with amax = 127: scale is exactly 1, so v == w and ties are exact
    w = np.array([[127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 0.49999997, -0.49999997, 0.0] + [0.0] * 20],
                 np.float32)
    q, s = orc.quantize_weight_int8(w, orc.STRICT)
    assert s[0] == 1.0
    # round half AWAY from zero; 0.49999997 (= 0.5 - 2^-25) becomes 1 because v + 0.5 rounds up to 1.0f
    # before the truncation -- the signature of trunc(v +- 0.5) as opposed to a true nearest rounding
    assert q[0, :12].tolist() == [127, 1, -1, 2, -2, 3, -3, 127, -127, 1, -1, 0]
    # int4: amax 7 -> scale 1; clamp to [-8, 7]; low nibble = even index
    w4 = np.zeros((1, 32), np.float32)
    w4[0, :8] = [7.0, -7.0, 0.5, -0.5, 6.5, -6.5, 3.0, -3.0]
    q4, s4 = orc.quantize_weight_int4(w4, orc.STRICT)
    assert s4[0, 0] == 1.0
    lo, hi = (q4[0] & 0x0F).astype(int) - 8, (q4[0] >> 4).astype(int) - 8
    assert [lo[0], hi[0], lo[1], hi[1], lo[2], hi[2], lo[3], hi[3]] == [7, -7, 1, -1, 7, -7, 3, -3]
    # all-zero row: scale 1, weights 0; all-zero activation: qx 0, sx 0
    q0, s0 = orc.quantize_weight_int8(np.zeros((1, 64), np.float32))
    assert s0[0] == 1.0 and not q0.any()
    qx, sx = orc.quantize_act_int8(np.zeros(64, np.float32))
    assert sx == 0.0 and not qx.any()
    # k not a multiple of 32 is refused for int4 (src/qmat.c:630)
    with pytest.raises(ValueError):
        orc.quantize_weight_int4(np.ones((2, 48), np.float32))
    # activation: |qx| <= 127 and the absmax element maps to +-127
    x = np.random.default_rng(3).standard_normal(3072).astype(np.float32)
    qx, sx = orc.quantize_act_int8(x)
    assert np.abs(qx.astype(int)).max() == 127
    assert sx == np.float32(np.abs(x).max()) / np.float32(127.0)


@pytest.mark.parametrize("shape", SHAPES)
def test_act_quant_and_accumulators(orc, ref, ref_strict, shape, nerr):
    n, k = shape
    w = _w(shape, seed=2)
    x = np.random.default_rng(5).standard_normal(k).astype(np.float32)
    bias = (np.random.default_rng(6).standard_normal(n) * 0.1).astype(np.float32)
    for variant, lib, exact in ((orc.STRICT, ref_strict, True), (orc.STOCK, ref, False)):
        qx, sx = orc.quantize_act_int8(x, variant)
        rqx = np.empty_like(qx)
        rsx = lib.ref_quantize_act_int8(rqx, x, k)
        assert np.array_equal(qx, rqx) and np.float32(sx).view(np.uint32) == np.float32(rsx).view(np.uint32)
        # int8: accumulators are exact integers -> compare with numpy int64
        q, s = orc.quantize_weight_int8(w, variant)
        out, acc = orc.matvec_q8(qx, sx, q, s, bias)
        assert np.array_equal(acc.astype(np.int64), q.astype(np.int64) @ qx.astype(np.int64))
        rout = np.empty(n, np.float32)
        lib.ref_matvec_q8(rout, qx, sx, q, s, bias.ctypes.data_as(C.c_void_p), n, k)
        if exact:
            assert np.array_equal(out.view(np.uint32), rout.view(np.uint32)), "int8 epilogue differs from the strict reference"
        assert nerr(out, rout) < 1e-6
        # int4: per-group integers exact, f32 group sum sequential
        q4, s4 = orc.quantize_weight_int4(w, variant)
        out4, acc4 = orc.matvec_q4(qx, sx, q4, s4, bias)
        lo = (q4 & 0x0F).astype(np.int64) - 8
        hi = (q4 >> 4).astype(np.int64) - 8
        full = np.empty((n, k), np.int64)
        full[:, 0::2], full[:, 1::2] = lo, hi
        want = (full * qx.astype(np.int64)).reshape(n, k // 32, 32).sum(-1)
        assert np.array_equal(acc4.astype(np.int64), want)
        rout4 = np.empty(n, np.float32)
        lib.ref_matvec_q4(rout4, qx, sx, q4, np.ascontiguousarray(s4), bias.ctypes.data_as(C.c_void_p), n, k)
        if exact:
            assert np.array_equal(out4.view(np.uint32), rout4.view(np.uint32)), "int4 epilogue differs from the strict reference"
        assert nerr(out4, rout4) < 1e-6


def test_reference_self_tests_pass(ref, ref_strict):
    """The compiled reference's own model-free self-tests (src/qmat.c:1181-1194, src/kernels.c:439-517)."""
    for lib in (ref, ref_strict):
        err = C.create_string_buffer(256)
        assert lib.mynah_qmat_self_test(err, 256) == 0, err.value
        assert lib.mynah_kernels_self_test(err, 256) == 0, err.value


def test_qmat_self_test_data_bounds(orc):
    """self_test_one (src/qmat.c:904-965): N=48, K=768 closed-form data; quantised matvec within 5 % (int8)
    / 20 % (int4) of the f32 dot with the reference's 1e-3 denominator floor."""
    N, K = 48, 768
    i = np.arange(N, dtype=np.float32)[:, None]
    j = np.arange(K, dtype=np.float32)[None, :]
    w = (np.sin(np.float32(0.017) * (i * 7 + j)) * (np.float32(0.5) + np.float32(0.5) * np.cos(np.float32(0.003) * j))).astype(np.float32)
    x = (np.cos(np.float32(0.011) * j[0]) - np.float32(0.3)).astype(np.float32)
    qx, sx = orc.quantize_act_int8(x)
    exact = w.astype(np.float64) @ x.astype(np.float64)
    denom = np.maximum(np.abs(exact), 1e-3)
    q, s = orc.quantize_weight_int8(w)
    out, _ = orc.matvec_q8(qx, sx, q, s)
    assert np.max(np.abs(out - exact) / denom) <= 0.05
    q4, s4 = orc.quantize_weight_int4(w)
    out4, _ = orc.matvec_q4(qx, sx, q4, s4)
    assert np.max(np.abs(out4 - exact) / denom) <= 0.20


def test_f16_rounding_is_ieee_rne(orc):
    # every finite half survives a round trip; random floats agree with numpy's IEEE conversion
    bits = np.arange(65536, dtype=np.uint16)
    as_f32 = bits.view(np.float16).astype(np.float32)
    finite = np.isfinite(as_f32)
    back = orc.f32_to_f16_bits(as_f32)
    assert np.array_equal(back[finite], bits[finite])
    widened = np.array([orc.lib.orc_f16_to_f32(int(b)) for b in bits[::7]], np.float32)
    assert np.array_equal(widened.view(np.uint32)[finite[::7]], as_f32[::7].view(np.uint32)[finite[::7]])
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * np.float32(s) for s in (1e-8, 1e-5, 0.02, 1.0, 300.0, 7e4)])
    # exact ties between neighbouring halves, incl. the subnormal range
    h = rng.integers(0, 0x7bff, 20000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    ties = ((lo + hi) / 2).astype(np.float32)
    x = np.concatenate([x, ties, -ties, np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -25, 2.0 ** -24], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f32_to_f16_bits(x), want)
    # the reference-held KATs (third_party/ingot/tests/test_gguf.c:439-443)
    assert orc.f32_to_f16_bits(np.array([1.0], np.float32))[0] == 0x3C00
    assert orc.lib.orc_f16_to_f32(0x3C00) == 1.0 and orc.lib.orc_f16_to_f32(0x0001) > 0.0
