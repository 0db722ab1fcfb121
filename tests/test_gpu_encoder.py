"""GPU parity of the MFMA text-encoder prefill against the oracle (f32 arithmetic on f16-rounded weights), through the C ABI.

Tolerances, both as normalised max error max|a-b|/max|b| over the whole output: the gathered token rows are
bit-exact (a gather); the encoder output is within 2e-3 -- the GPU rounds the operands of every product to f16
and accumulates in f32, the oracle keeps the activations in f32.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _oracle_weights(pkg, backend, w):
    f16 = lambda a: pkg.convert_weight_f16(backend.lib, a)
    out = {"tok_table": f16(w["tok_table"]), "pos_table": f16(w["pos_table"]), "qkv_w": f16(w["qkv"]), "o_w": f16(w["o"]),
           "up_w": f16(w["up"]), "down_w": f16(w["down"])}
    for name in ("norm1_g", "norm1_b", "norm2_g", "norm2_b", "norm_out_g", "norm_out_b"):
        out[name] = w.get(name)
    return out


def _run(pkg, backend, orc, synth, cfg, tokens, seed, final_norm=True, ln_bias=True):
    w = synth.encoder_weights(cfg, seed=seed)
    if not final_norm:
        w["norm_out_g"] = w["norm_out_b"] = None
    if not ln_bias:
        w["norm1_b"] = w["norm2_b"] = None
    rng = np.random.default_rng(seed + 100)
    ids = rng.integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    enc = pkg.Encoder(backend, cfg, w)
    width = cfg["width"]
    dembed = backend.alloc(tokens * width // 2 + 4)
    dout = backend.alloc(tokens * width)
    enc.prefill(ids, dembed.ptr, dout.ptr)
    got = dout.read().reshape(tokens, width)
    embed = dembed.read(tokens * width // 2, dtype=np.uint16).reshape(tokens, width)
    # a second call with fewer tokens on the same encoder, then the first again: nothing may leak between calls
    fewer = max(1, tokens // 3)
    enc.prefill(ids[:fewer], 0, dout.ptr)
    got_fewer = dout.read(fewer * width).reshape(fewer, width)
    enc.prefill(ids, 0, dout.ptr)
    again = dout.read().reshape(tokens, width)
    enc.destroy()
    want_embed, want = orc.encoder_prefill(cfg, _oracle_weights(pkg, backend, w), ids)
    want_embed_fewer, want_fewer = orc.encoder_prefill(cfg, _oracle_weights(pkg, backend, w), ids[:fewer])
    return got, embed, want, want_embed, again, got_fewer, want_fewer


@pytest.mark.parametrize("tokens,layers", [(256, 6), (64, 2), (37, 2), (1, 1), (200, 1)])
def test_encoder_prefill_matches_oracle(pkg, backend, orc, synth, nerr, tokens, layers):
    _announce("encoder prefill tokens=%d layers=%d" % (tokens, layers))
    cfg = synth.encoder_config(layers=layers)
    got, embed, want, want_embed, again, got_fewer, want_fewer = _run(pkg, backend, orc, synth, cfg, tokens, seed=4)
    assert np.array_equal(embed, want_embed), "gathered token rows are not bit-exact"
    assert np.all(np.isfinite(got))
    assert nerr(got, want) < 2e-3
    assert nerr(got_fewer, want_fewer) < 2e-3
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32)), "prefill is not repeatable"


def test_encoder_prefill_max_positions_and_no_final_norm(pkg, backend, orc, synth, nerr):
    _announce("encoder prefill tokens=512 (max_positions) layers=1, no final norm, gain-only LayerNorm")
    cfg = synth.encoder_config(layers=1)
    got, embed, want, want_embed, again, got_fewer, want_fewer = _run(pkg, backend, orc, synth, cfg, 512, seed=9, final_norm=False,
                                                                      ln_bias=False)
    assert np.array_equal(embed, want_embed)
    assert nerr(got, want) < 2e-3
    assert nerr(got_fewer, want_fewer) < 2e-3


def test_encoder_prefill_rejects_bad_input(pkg, backend, synth):
    _announce("encoder prefill error paths")
    cfg = synth.encoder_config(layers=1, max_positions=128)
    enc = pkg.Encoder(backend, cfg, synth.encoder_weights(cfg, seed=4))
    dout = backend.alloc(129 * cfg["width"])
    with pytest.raises(pkg.BackendError):       # id out of range (src/graph.c:730-735)
        enc.prefill(np.array([0, cfg["vocab"]], np.int32), 0, dout.ptr)
    with pytest.raises(pkg.BackendError):
        enc.prefill(np.array([-1], np.int32), 0, dout.ptr)
    with pytest.raises(pkg.BackendError):       # longer than the position table
        enc.prefill(np.zeros(129, np.int32), 0, dout.ptr)
    enc.destroy()
    bad = synth.encoder_config(layers=1, width=96, heads=2)      # 48-wide heads: not supported by the MFMA path
    with pytest.raises(pkg.BackendError):
        pkg.Encoder(backend, bad, synth.encoder_weights(bad, seed=4))


def _f16_bits(w):
    h = lambda a: np.asarray(a, np.float32).astype(np.float16).view(np.uint16)
    out = {"tok_table": h(w["tok_table"]), "pos_table": h(w["pos_table"]), "qkv_w": h(w["qkv"]), "o_w": h(w["o"]),
           "up_w": h(w["up"]), "down_w": h(w["down"])}
    for name in ("norm1_g", "norm1_b", "norm2_g", "norm2_b", "norm_out_g", "norm_out_b"):
        out[name] = w.get(name)
    return out


def _prefill(pkg, backend, cfg, w, ids):
    enc = pkg.Encoder(backend, cfg, w)
    try:
        dout = backend.alloc(ids.size * cfg["width"])
        outs = []
        for _ in range(3):                       # eager, capture, replay
            enc.prefill(ids, 0, dout.ptr)
            outs.append(dout.read().reshape(ids.size, cfg["width"]).copy())
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        assert np.array_equal(outs[0].view(np.uint32), outs[2].view(np.uint32))
        return outs[0]
    finally:
        enc.destroy()


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("kernel", [1, 3])
@pytest.mark.parametrize("tokens,layers", [(1, 1), (2, 1), (37, 2), (65, 1), (256, 2), (300, 1)])
def test_encoder_reference_form_matches_oracle(pkg, backend, orc, synth, nerr, causal, kernel, tokens, layers):
    """The stack as the reference builds it (src/graph.c:634-711): causal mask, causal conv FFN of kernel size 1 or 3,
    LayerNorm with and without bias, against the oracle (itself checked against the compiled reference on CPU)."""
    _announce("encoder reference form causal=%s kernel=%d tokens=%d layers=%d" % (causal, kernel, tokens, layers))
    cfg = dict(synth.encoder_config(layers=layers), causal=causal, ffn_kernel=kernel)
    w = synth.encoder_weights_f16(cfg, seed=60 + kernel, kernel=kernel, biases=(tokens % 2 == 0))
    ids = np.random.default_rng(61).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    got = _prefill(pkg, backend, cfg, w, ids)
    _, want = orc.encoder_prefill(cfg, _f16_bits(w), ids)
    assert np.isfinite(got).all()
    assert nerr(got, want) < 2e-3
    if causal and tokens > 2:
        # a causal stack's first rows do not depend on what follows them: bit-equal to a shorter call's
        # when both calls pad to the same number of rows (the products then see the same tiles)
        shorter = tokens - 1 if (tokens - 1 + 63) // 64 == (tokens + 63) // 64 else None
        if shorter:
            head = _prefill(pkg, backend, cfg, w, ids[:shorter])
            assert np.array_equal(head.view(np.uint32), got[:shorter].view(np.uint32))


@pytest.mark.parametrize("kernel", [1, 3])
def test_encoder_matches_the_reference_fixture(pkg, backend, synth, nerr, kernel):
    """Against the committed outputs of the compiled reference's transformer_stack (strict build) on the same weights."""
    from tests.golden import make_golden as mg
    _announce("encoder against the reference fixture, kernel=%d" % kernel)
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(mg.__file__)), "reference_vectors.npz"), allow_pickle=False)
    cfg = dict(mg.ENC_CFG, ffn_kernel=kernel)
    w = synth.encoder_weights_f16(cfg, seed=mg.ENC_SEED + kernel, kernel=kernel)
    ids = np.random.default_rng(mg.ENC_SEED).integers(0, cfg["vocab"], size=mg.ENC_TOKENS).astype(np.int32)
    if mg.crc(ids, *[w[k] for k in sorted(w) if w[k] is not None]) != gold["enc_k%d_input_crc" % kernel]:
        pytest.skip("numpy's generator produced different synthetic inputs than when the fixture was written")
    got = _prefill(pkg, backend, cfg, w, ids)
    for tag in ("strict", "stock"):
        assert nerr(got, gold["enc_k%d_%s_out" % (kernel, tag)]) < 2e-3


def test_encoder_rejects_other_conv_kernels(pkg, backend, synth):
    _announce("encoder: ffn_kernel 2 is refused")
    cfg = dict(synth.encoder_config(layers=1), ffn_kernel=2)
    with pytest.raises(pkg.BackendError, match="ffn_kernel"):
        pkg.Encoder(backend, cfg, synth.encoder_weights_f16(cfg, seed=1, kernel=2))


@pytest.mark.parametrize("width,heads,ffn,kernel", [(64, 1, 192, 3), (320, 5, 704, 1), (1024, 16, 2048, 3), (1152, 18, 2304, 1)])
def test_encoder_other_widths(pkg, backend, orc, synth, nerr, width, heads, ffn, kernel):
    """Narrow, odd-multiple and wide rows (the row pass keeps 4 or 16 pieces of a row per lane), both FFN forms."""
    _announce("encoder width=%d heads=%d ffn=%d kernel=%d" % (width, heads, ffn, kernel))
    cfg = dict(synth.encoder_config(layers=2, width=width, heads=heads, ffn=ffn, vocab=512, max_positions=128), causal=True, ffn_kernel=kernel)
    w = synth.encoder_weights_f16(cfg, seed=80, kernel=kernel)
    ids = np.random.default_rng(81).integers(0, cfg["vocab"], size=70).astype(np.int32)
    got = _prefill(pkg, backend, cfg, w, ids)
    _, want = orc.encoder_prefill(cfg, _f16_bits(w), ids)
    assert np.isfinite(got).all()
    assert nerr(got, want) < 2e-3


def _prefill_f32(pkg, backend, cfg, w, ids):
    enc = pkg.Encoder(backend, dict(cfg, operands_f32=True), w)
    try:
        dout = backend.alloc(ids.size * cfg["width"])
        outs = []
        for _ in range(2):
            enc.prefill(ids, 0, dout.ptr)
            outs.append(dout.read().reshape(ids.size, cfg["width"]).copy())
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), "the f32 form is not repeatable"
        return outs[0]
    finally:
        enc.destroy()


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("kernel", [1, 3])
@pytest.mark.parametrize("tokens,layers", [(1, 1), (19, 2), (130, 2), (256, 1)])
def test_encoder_f32_operands_match_oracle(pkg, backend, orc, synth, nerr, causal, kernel, tokens, layers):
    """The f32-operand form (transformer_stack's own arithmetic, src/graph.c:634-711) against the oracle on weights that are
    exactly representable in f16, so that both sides multiply the same numbers: 1e-5, the bar of an f32 operator."""
    _announce("encoder f32 operands causal=%s kernel=%d tokens=%d layers=%d" % (causal, kernel, tokens, layers))
    cfg = dict(synth.encoder_config(layers=layers), causal=causal, ffn_kernel=kernel)
    w = synth.encoder_weights_f16(cfg, seed=70 + kernel, kernel=kernel, biases=(tokens % 2 == 0))
    ids = np.random.default_rng(71).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    got = _prefill_f32(pkg, backend, cfg, w, ids)
    _, want = orc.encoder_prefill(cfg, _f16_bits(w), ids)
    assert np.isfinite(got).all()
    assert nerr(got, want) < 1e-5
    half = _prefill(pkg, backend, cfg, w, ids)            # and the f16-operand form stays within its own bar of it
    assert nerr(half, got) < 2e-3


@pytest.mark.parametrize("kernel", [1, 3])
def test_encoder_f32_operands_match_the_reference_fixture(pkg, backend, synth, nerr, kernel):
    """Against the committed outputs of the compiled reference's transformer_stack, both builds, at the f32 bar."""
    from tests.golden import make_golden as mg
    _announce("encoder f32 operands against the reference fixture, kernel=%d" % kernel)
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(mg.__file__)), "reference_vectors.npz"), allow_pickle=False)
    cfg = dict(mg.ENC_CFG, ffn_kernel=kernel)
    w = synth.encoder_weights_f16(cfg, seed=mg.ENC_SEED + kernel, kernel=kernel)
    ids = np.random.default_rng(mg.ENC_SEED).integers(0, cfg["vocab"], size=mg.ENC_TOKENS).astype(np.int32)
    if mg.crc(ids, *[w[k] for k in sorted(w) if w[k] is not None]) != gold["enc_k%d_input_crc" % kernel]:
        pytest.skip("numpy's generator produced different synthetic inputs than when the fixture was written")
    got = _prefill_f32(pkg, backend, cfg, w, ids)
    for tag in ("strict", "stock"):
        assert nerr(got, gold["enc_k%d_%s_out" % (kernel, tag)]) < 1e-5, tag


def test_encoder_f32_operands_return_no_f16_rows(pkg, backend, synth):
    cfg = dict(synth.encoder_config(layers=1, max_positions=64), operands_f32=True)
    enc = pkg.Encoder(backend, cfg, synth.encoder_weights(cfg, seed=4))
    dout, dembed = backend.alloc(4 * cfg["width"]), backend.alloc(4 * cfg["width"])
    with pytest.raises(pkg.BackendError, match="f32 operands"):
        enc.prefill(np.zeros(4, np.int32), dembed.ptr, dout.ptr)
    enc.destroy()
