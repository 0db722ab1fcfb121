"""Pins of the oracle's encoder prefill, its row-times-row GEMM and its output head (CPU only).

  * orc_encoder_prefill in the reference's own form (causal mask, gain-only LayerNorm, plain or kernel-3 conv FFN)
    against the compiled reference's transformer_stack (src/graph.c:634-711 as encode_text calls it, :738-740), on
    f16-representable weights so both sides multiply the same numbers: 1e-5 normalised (the two GEMMs add in different
    orders; everything else is the same f32 arithmetic);
  * the bidirectional form with LayerNorm biases (the synthetic prefill configuration) against a float64 restatement
    written here with numpy only -- a mistake in where the scale goes, a transposed V, a shifted position row or a
    dropped bias fails it;
  * orc_gemm_nt against float64 matmul;
  * orc_output_head against the oracle's own pinned linear + softmax per head, and against float64.
"""
import numpy as np
import pytest


def _bits16(a):
    return np.asarray(a, np.float32).astype(np.float16).view(np.uint16)


def _oracle_dict(w):
    out = {"tok_table": _bits16(w["tok_table"]), "pos_table": _bits16(w["pos_table"]), "qkv_w": _bits16(w["qkv"]),
           "o_w": _bits16(w["o"]), "up_w": _bits16(w["up"]), "down_w": _bits16(w["down"])}
    for name in ("norm1_g", "norm1_b", "norm2_g", "norm2_b", "norm_out_g", "norm_out_b"):
        out[name] = w.get(name)
    return out


@pytest.mark.parametrize("tokens,layers,kernel", [(1, 2, 1), (37, 2, 1), (256, 1, 1), (1, 1, 3), (37, 2, 3), (130, 1, 3)])
@pytest.mark.parametrize("strict", [False, True])
def test_causal_encoder_matches_compiled_reference(orc, synth, nerr, tmp_path, tokens, layers, kernel, strict):
    if not orc.ref_available(strict=strict):
        pytest.skip("oracle/_ref is not built (needs the reference tree)")
    cfg = {"layers": layers, "width": 768, "heads": 12, "head_width": 64, "ffn": 3072, "vocab": 300, "max_positions": 256,
           "causal": True, "ffn_kernel": kernel}
    w = synth.encoder_weights_f16(cfg, seed=20 + kernel, kernel=kernel)
    ids = np.random.default_rng(5).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    embed, got = orc.encoder_prefill(cfg, _oracle_dict(w), ids)
    assert np.array_equal(embed, _bits16(w["tok_table"])[ids])
    want = orc.ref_transformer_stack(cfg, w, w["tok_table"][ids], kernel, strict=strict, workdir=str(tmp_path))
    assert nerr(got, want) < 1e-5


def _ln64(x, g, b):
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mean) / np.sqrt(var + 1e-5) * g
    return y + b if b is not None else y


def _encoder64(cfg, w, ids, causal, kernel):
    """float64, written from the definition: pre-LN transformer, softmax(QK^T / sqrt(d)) V, tanh GELU."""
    f8 = lambda a: None if a is None else np.asarray(a, np.float64)
    T, wd, H, hw, f = len(ids), cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
    x = f8(w["tok_table"])[ids] + f8(w["pos_table"])[:T]
    for l in range(cfg["layers"]):
        n = _ln64(x, f8(w["norm1_g"][l]), None if w["norm1_b"] is None else f8(w["norm1_b"][l]))
        qkv = n @ f8(w["qkv"][l]).T
        ctx = np.empty((T, wd))
        for h in range(H):
            q, k, v = (qkv[:, i * wd + h * hw: i * wd + (h + 1) * hw] for i in range(3))
            s = (q @ k.T) / np.sqrt(hw)
            if causal:
                s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            p /= p.sum(axis=1, keepdims=True)
            ctx[:, h * hw:(h + 1) * hw] = p @ v
        x = x + ctx @ f8(w["o"][l]).T
        n = _ln64(x, f8(w["norm2_g"][l]), None if w["norm2_b"] is None else f8(w["norm2_b"][l]))

        def conv(rows, weight, out_ch, in_ch):
            wt = f8(weight).reshape(out_ch, in_ch, kernel)
            y = np.zeros((T, out_ch))
            for j in range(kernel):            # tap j reads row t - (kernel - 1) + j
                shift = kernel - 1 - j
                src = np.zeros_like(rows)
                src[shift:] = rows[:T - shift] if shift else rows
                y += src @ wt[:, :, j].T
            return y
        hid = conv(n, w["up"][l], f, wd)
        hid = 0.5 * hid * (1.0 + np.tanh(0.7978845608028654 * (hid + 0.044715 * hid ** 3)))
        x = x + conv(hid, w["down"][l], wd, f)
    if w["norm_out_g"] is not None:
        x = _ln64(x, f8(w["norm_out_g"]), f8(w["norm_out_b"]))
    return x


@pytest.mark.parametrize("tokens,causal,kernel,biases", [(1, False, 1, True), (53, False, 1, True), (96, False, 1, False),
                                                         (53, True, 3, False), (40, True, 1, True), (31, False, 3, True)])
def test_encoder_matches_float64_definition(orc, synth, nerr, tokens, causal, kernel, biases):
    cfg = {"layers": 2, "width": 256, "heads": 4, "head_width": 64, "ffn": 512, "vocab": 97, "max_positions": 128,
           "causal": causal, "ffn_kernel": kernel}
    w = synth.encoder_weights_f16(cfg, seed=31, kernel=kernel, biases=biases)
    ids = np.random.default_rng(6).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    _, got = orc.encoder_prefill(cfg, _oracle_dict(w), ids, threads=3)
    assert nerr(got, _encoder64(cfg, w, ids, causal, kernel)) < 1e-5
    _, one_thread = orc.encoder_prefill(cfg, _oracle_dict(w), ids, threads=1)
    assert np.array_equal(got.view(np.uint32), one_thread.view(np.uint32)), "result depends on the thread count"


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 5, 7), (17, 33, 64), (64, 96, 768), (5, 8, 100)])
def test_gemm_nt_matches_float64(orc, nerr, m, n, k):
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((n, k)).astype(np.float32)
    a[0, 0] = 3.0
    b[0, 0] = -2.0      # a transposed or swapped operand changes element (0, 0) visibly
    c = np.zeros((m, n), np.float32)
    for threads in (1, 4):
        orc.lib.orc_gemm_nt(a, b, c, m, n, k, threads)
        assert nerr(c, a.astype(np.float64) @ b.astype(np.float64).T) < 1e-6
    # a row of the product is the decode matvec of that row, bit for bit
    row = orc.matvec_f32(a[m - 1], b)
    assert np.array_equal(np.asarray(row, np.float32).view(np.uint32), c[m - 1].view(np.uint32))


@pytest.mark.parametrize("qname", ["f32", "int8", "int4", "f16"])
def test_output_head_is_linear_plus_softmax_per_head(orc, nerr, qname):
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4, "f16": orc.F16}[qname]
    rng = np.random.default_rng(41)
    heads_out, vocab, width = 8, 1024, 768
    w = (rng.standard_normal((heads_out * vocab, width)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(heads_out * vocab) * 0.1).astype(np.float32)
    hidden = rng.standard_normal(width).astype(np.float32)
    pw = orc.PackedWeight(w, qtype)
    logits, probs = orc.output_head(pw, hidden, heads_out, vocab, bias)
    want_logits = orc.linear(pw, hidden, bias)
    assert np.array_equal(logits.view(np.uint32), np.asarray(want_logits, np.float32).view(np.uint32))
    for h in range(heads_out):
        rc, sm = orc.softmax(logits[h * vocab:(h + 1) * vocab])
        assert rc == 0
        assert np.array_equal(probs[h * vocab:(h + 1) * vocab].view(np.uint32), sm.view(np.uint32)), "head %d" % h
        l64 = logits[h * vocab:(h + 1) * vocab].astype(np.float64)
        p64 = np.exp(l64 - l64.max())
        p64 /= p64.sum()
        assert nerr(probs[h * vocab:(h + 1) * vocab], p64) < 5e-6   # f32 exp and a 1024-term f32 sum against float64
        assert abs(float(probs[h * vocab:(h + 1) * vocab].sum()) - 1.0) < 1e-5
    if qname == "f32":      # unquantised: the logits themselves against float64
        assert nerr(logits, w.astype(np.float64) @ hidden.astype(np.float64) + bias) < 1e-5
