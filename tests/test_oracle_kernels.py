"""Pins the oracle's f32 kernels: reference self-test KATs, float64 closed forms, the compiled reference."""
import ctypes as C
import math

import numpy as np


def test_kernel_kats(orc):
    """The literals of mynah_kernels_self_test (src/kernels.c:439-517)."""
    a = np.array([1.0, 2.0, 3.0], np.float32)
    m = np.array([[1.0, 2.0, 3.0], [-1.0, 0.0, 2.0]], np.float32)
    assert np.allclose(orc.matvec_f32(a, m), [14.0, 5.0], atol=1e-6)
    ln = orc.layernorm(np.array([1.0, 2.0, 3.0, 4.0], np.float32), np.ones(4, np.float32), np.zeros(4, np.float32), eps=1e-6)
    assert abs(ln[0] + 1.34164) < 1e-4 and abs(ln[3] - 1.34164) < 1e-4
    g = orc.gelu_scalar(np.array([-1.0, 0.0, 1.0], np.float32))
    assert abs(g[1]) < 1e-6 and abs(g[2] - 0.8411920) < 1e-5
    gp = orc.gelu_pade(np.array([-1.0, 0.0, 1.0], np.float32))
    assert abs(gp[1]) < 1e-6 and abs(gp[2] - 0.8411920) < 1e-5
    rc, p = orc.softmax(np.array([1.0, 2.0, 3.0], np.float32))
    assert rc == 0 and int(np.argmax(p)) == 2 and abs(float(p.sum()) - 1.0) < 1e-6
    assert orc.lib.orc_softmax(np.zeros(1, np.float32), np.zeros(1, np.float32), 0) == -1   # empty softmax rejected
    rc, _ = orc.softmax(np.array([1.0, np.inf], np.float32))
    assert rc == -1                                                                          # non-finite rejected
    r = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    orc.lib.orc_residual_add(r, np.array([3.0, -1.0, 2.0, -2.0], np.float32), 4)
    assert r[0] == 4.0 and r[3] == 2.0


def test_backend_matmul_kat(orc):
    """[2x3] . [4x3]^T + bias (src/backend.c:290-310)."""
    x = np.array([[1.0, 2.0, 3.0], [-1.0, 0.5, 2.0]], np.float32)
    w = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], np.float32)
    b = np.array([0.5, -0.5, 1.0, 2.0], np.float32)
    got = np.stack([orc.matvec_f32(row, w, b) for row in x])
    assert np.allclose(got, [[1.5, 1.5, 4.0, 8.0], [-0.5, 0.0, 3.0, 3.5]], atol=1e-6)


def test_f32_kernels_against_float64_and_reference(orc, ref, ref_strict, nerr):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((3, 768)).astype(np.float32) * 3 + 0.7
    gain = (1 + 0.1 * rng.standard_normal(768)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(768)).astype(np.float32)
    x64 = x.astype(np.float64)
    mu = x64.mean(-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(-1, keepdims=True)
    want = (x64 - mu) / np.sqrt(var + 1e-5) * gain
    for bias, w64 in ((None, want), (beta, want + beta)):
        got = orc.layernorm(x, gain, bias)
        assert nerr(got, w64) < 2e-6
        for lib in (ref, ref_strict):
            r = np.empty_like(x)
            lib.mynah_layernorm_f32(x, gain, None if bias is None else bias.ctypes.data_as(C.c_void_p), r, 3, 768, 1e-5)
            assert nerr(got, r) < 1e-6
    # GELU: tanh form in float64, incl. the +-6 clamp region of the Pade variant
    v = np.concatenate([np.linspace(-9, 9, 3001), rng.standard_normal(71) * 2]).astype(np.float32)
    v64 = v.astype(np.float64)
    g64 = 0.5 * v64 * (1 + np.tanh(0.7978845608 * (v64 + 0.044715 * v64 ** 3)))
    assert np.max(np.abs(orc.gelu_scalar(v) - g64)) < 2e-6
    # the Pade variant clamps tanh's argument to +-6, so beyond that it keeps tanh(6) = 1 - 1.2e-5: compare with
    # float64 inside the clamp, and with the compiled reference (below) everywhere
    inner = 0.7978845608 * (v64 + 0.044715 * v64 ** 3)
    inside = np.abs(inner) <= 6.0
    assert np.max(np.abs(orc.gelu_pade(v) - g64)[inside]) < 2e-6
    assert np.max(np.abs(orc.gelu_pade(v) - g64)) < 1e-4
    for lib in (ref, ref_strict):
        r = v.copy()
        lib.mynah_gelu_f32_scalar(r, r.size)
        assert np.max(np.abs(orc.gelu_scalar(v) - r)) < 1e-6
    # the Pade form exists only in the SIMD build (src/kernels.c:260-315); the strict build has SIMD off
    r = v.copy()
    ref.mynah_gelu_f32(r, r.size)
    assert np.max(np.abs(orc.gelu_pade(v) - r)) < 1e-6
    # softmax over 8 x 1024 (the output head's shape)
    logits = rng.standard_normal((8, 1024)).astype(np.float32) * 4
    for row in logits:
        rc, p = orc.softmax(row)
        e = np.exp(row.astype(np.float64) - row.max())
        assert rc == 0 and np.max(np.abs(p - e / e.sum())) < 2e-6
        r = np.empty_like(row)
        assert ref.mynah_softmax_f32(row, r, row.size) == 0
        assert np.max(np.abs(p - r)) < 2e-6
        q = orc.softmax_row_inplace(row)
        assert np.max(np.abs(q - p)) < 2e-6
    m = orc.softmax_masked(logits, 700)
    e = np.exp(logits[:, :700].astype(np.float64) - logits[:, :700].max(-1, keepdims=True))
    assert np.max(np.abs(m[:, :700] - e / e.sum(-1, keepdims=True))) < 2e-6 and not m[:, 700:].any()
    # f32 matvec against float64 and the compiled reference
    w = (rng.standard_normal((96, 768)) * 0.02).astype(np.float32)
    xv = rng.standard_normal(768).astype(np.float32)
    b = rng.standard_normal(96).astype(np.float32)
    got = orc.matvec_f32(xv, w, b)
    assert nerr(got, w.astype(np.float64) @ xv.astype(np.float64) + b) < 1e-6
    r = np.empty(96, np.float32)
    ref.mynah_matvec_bias_f32(w, xv, b.ctypes.data_as(C.c_void_p), r, 96, 768)
    assert nerr(got, r) < 1e-6


def test_matvec_f16_against_float64(orc, nerr):
    """self_test_f16's data (src/qmat.c:1064-1104): N=64, K=512, <= 1e-3 max-rel vs the f32 weights in
    double; and within 1e-6 of the float64 dot of the exactly widened halves (no x86 reference build
    of this kernel exists, src/qmat.c:25-28)."""
    N, K = 64, 512
    i = np.arange(N * K, dtype=np.float32)
    w = (np.sin(np.float32(0.017) * i) * (np.float32(0.5) + np.float32(0.5) * np.cos(np.float32(0.003) * i))).astype(np.float32).reshape(N, K)
    x = (np.cos(np.float32(0.011) * np.arange(K, dtype=np.float32)) - np.float32(0.3)).astype(np.float32)
    bias = (np.arange(N, dtype=np.float32) * np.float32(0.125) - np.float32(0.25)).astype(np.float32)
    bits = orc.f32_to_f16_bits(w)
    got = orc.matvec_f16(x, bits, bias)
    ref64 = w.astype(np.float64) @ x.astype(np.float64) + bias
    assert np.max(np.abs(got - ref64) / np.maximum(np.abs(ref64), 1e-3)) <= 1e-3
    widened = bits.view(np.float16).astype(np.float64)
    assert nerr(got, widened @ x.astype(np.float64) + bias) < 1e-6


def test_argmax_rules(orc):
    """src/backend.c:825-847: candidates i < codebook_size or eos; strict >, first index wins."""
    logits = np.array([0.5, 2.0, 2.0, -1.0, 9.0, 3.0], np.float32)
    assert orc.argmax_constrained(logits, 4, 5, False) == (0, 1)      # tie -> first
    assert orc.argmax_constrained(logits, 4, 5, True) == (0, 5)       # eos allowed and larger
    assert orc.argmax_constrained(logits, 4, 4, True) == (0, 4)
    assert orc.argmax_constrained(np.full(4, -np.inf, np.float32), 4, 0, False) == (0, 0)
    assert orc.argmax_constrained(np.array([np.nan, 1.0], np.float32), 2, 0, False) == (0, 1)
    assert orc.argmax_constrained(logits, 7, 0, False)[0] == -1        # codebook > vocab rejected


def test_attention_kats_and_float64(orc, nerr):
    """The resident-op KATs of gpu/metal/backend_metal_ops.m:1049-1079, then softmax(QK^T)V in float64."""
    k = np.zeros((2, 2), np.float32)
    v = np.zeros((2, 2), np.float32)
    out = orc.self_attention(np.array([1, 0, 1, 0, 2, 3], np.float32), k, v, 0, 2, 1, 1, 2, 1.0)
    assert np.allclose(out, [2.0, 3.0], atol=1e-6)
    assert np.array_equal(k[0], [1, 0]) and np.array_equal(v[0], [2, 3])     # append wrote exactly row 0
    out = orc.self_attention(np.array([1, 0, 0, 1, 4, 5], np.float32), k, v, 1, 2, 2, 1, 2, 1.0)
    e = math.e
    assert np.allclose(out, [(2 * e + 4) / (e + 1), (3 * e + 5) / (e + 1)], atol=1e-6)
    out = orc.cross_attention(np.array([1, 2], np.float32), k, v, 1, 2, 1, 2, 1.0)
    assert np.allclose(out, [2.0, 3.0], atol=1e-6)

    rng = np.random.default_rng(31)
    heads, hw, L = 12, 64, 300
    width = heads * hw
    qkv = rng.standard_normal(3 * width).astype(np.float32)
    kc = np.zeros((L + 4, width), np.float32)
    vc = np.zeros((L + 4, width), np.float32)
    kc[:L] = rng.standard_normal((L, width))
    vc[:L] = rng.standard_normal((L, width))
    before_k, before_v = kc.copy(), vc.copy()
    out = orc.self_attention(qkv, kc, vc, L, width, L + 1, heads, hw, 0.125)
    assert np.array_equal(kc[L], qkv[width:2 * width]) and np.array_equal(vc[L], qkv[2 * width:])
    assert np.array_equal(kc[:L], before_k[:L]) and np.array_equal(kc[L + 1:], before_k[L + 1:])
    assert np.array_equal(vc[:L], before_v[:L])
    q64 = qkv[:width].astype(np.float64).reshape(heads, hw)
    k64 = kc[:L + 1].astype(np.float64).reshape(L + 1, heads, hw)
    v64 = vc[:L + 1].astype(np.float64).reshape(L + 1, heads, hw)
    s = np.einsum("hd,shd->hs", q64, k64) * 0.125
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("hs,shd->hd", p, v64).reshape(-1)
    assert nerr(out, want) < 2e-6
    # convexity: every output coordinate lies inside the range of the attended V rows
    vv = vc[:L + 1].reshape(L + 1, heads, hw)
    o = out.reshape(heads, hw)
    assert np.all(o <= vv.max(0) + 1e-5) and np.all(o >= vv.min(0) - 1e-5)
    # single cross head of width 768 (what the engine passes, src/graph.c:3443-3448)
    out1 = orc.cross_attention(qkv[:width], kc, vc, L, width, 1, width, 1.0 / math.sqrt(width))
    s1 = (kc[:L].astype(np.float64) @ qkv[:width].astype(np.float64)) / math.sqrt(width)
    p1 = np.exp(s1 - s1.max())
    p1 /= p1.sum()
    assert nerr(out1, p1 @ vc[:L].astype(np.float64)) < 2e-6


def test_head_choice_against_the_reference_fused_matvec_argmax(orc, ref_strict):
    """What the GPU head test compares with -- the oracle's f32 matvec followed by its constrained first-max -- against
    the compiled reference's own fused mynah_matvec_argmax_f32 (src/kernels.c:116-139, strict build: the same
    sequential dot product), with and without the extra row, incl. a forbidden row that holds the largest value."""
    rng = np.random.default_rng(77)
    rows, cols, allowed, extra = 1024, 768, 1000, 1010
    ref_strict.mynah_matvec_argmax_f32.restype = C.c_int
    ref_strict.mynah_matvec_argmax_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int,
                                                   C.POINTER(C.c_uint)]
    for trial in range(6):
        w = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
        x = rng.standard_normal(cols).astype(np.float32)
        bias = (rng.standard_normal(rows) * 0.1).astype(np.float32)
        if trial % 2:
            bias[extra] = 40.0                # the extra row wins wherever it is allowed
        bias[1017] = 90.0                     # never allowed
        logits = orc.matvec_f32(x, w, bias)
        for allow in (0, 1):
            out = C.c_uint(0)
            rc = ref_strict.mynah_matvec_argmax_f32(w.ctypes.data, x.ctypes.data, bias.ctypes.data, rows, cols, allowed, extra, allow, C.byref(out))
            assert rc == 0
            orc_rc, got = orc.argmax_constrained(logits, allowed, extra, allow)
            assert orc_rc == 0 and got == out.value, (trial, allow, got, out.value)
            assert got != 1017 and (got == extra) == bool(allow and trial % 2)
