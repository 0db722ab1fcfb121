"""GPU parity of the MFMA text-encoder prefill against the oracle (f32 arithmetic on f16-rounded weights), through the C ABI.

Tolerances, both as normalised max error max|a-b|/max|b| over the whole output: the gathered token rows are
bit-exact (a gather); the encoder output is within 2e-3 -- the GPU rounds the operands of every product to f16
and accumulates in f32, the oracle keeps the activations in f32.
"""
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
