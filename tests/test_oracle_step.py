"""Pins the oracle's whole decode step against the compiled reference's decoder_step_batch
(src/graph.c:3127-3284) on synthetic weights: f32 / int8 / int4, one stream and ragged batches."""
import numpy as np
import pytest


def _cfg(synth, layers, capacity):
    # the reference's decode step has gain-only LayerNorm and ONE cross-attention head of width xw
    cfg = synth.decoder_config(layers=layers, capacity=capacity, cross_heads=1)
    return cfg


def _run_both(orc, synth, qtype, layers, lengths, mems, strict):
    cfg = _cfg(synth, layers, max(lengths) + 3)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    B = len(lengths)
    variant = orc.STRICT if strict else orc.STOCK
    odec = orc.Decoder(cfg, weights, qtype, variant)
    ok = [s["k"].copy() for s in streams]
    ov = [s["v"].copy() for s in streams]
    want = odec.step(ok, ov, [s["ck"] for s in streams], [s["cv"] for s in streams], lengths, mems, [s["x"] for s in streams])
    rdec = orc.RefDecoder(cfg, weights, qtype, B, max(mems), strict=strict)
    rk = [s["k"].copy() for s in streams]
    rv = [s["v"].copy() for s in streams]
    got, new_lengths = rdec.step(rk, rv, [s["ck"] for s in streams], [s["cv"] for s in streams], lengths, mems,
                                 [s["x"] for s in streams])
    rdec.close()
    assert new_lengths == [n + 1 for n in lengths]
    return cfg, want, got, (ok, ov), (rk, rv)


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
@pytest.mark.parametrize("strict", [True, False])
def test_step_matches_reference_single_stream(orc, ref, ref_strict, synth, nerr, qtype_name, strict):
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}[qtype_name]
    cfg, want, got, (ok, ov), (rk, rv) = _run_both(orc, synth, qtype, 2, [37], [29], strict)
    # f32 path: 1e-5 normalised.  Quantised paths: identical packed weights on both sides (same closed-form
    # quantiser, verified bit-exact elsewhere); a last-bit LayerNorm difference can still flip one int8
    # activation by 1, hence the looser bound there.
    tol = 1e-5 if qtype == orc.F32 else 5e-3
    assert nerr(want[0], got[0]) < tol
    L = 37
    for layer in range(cfg["layers"]):
        assert nerr(ok[0][layer, L], rk[0][layer, L]) < tol
        assert nerr(ov[0][layer, L], rv[0][layer, L]) < tol
    # nothing but row `length` of each layer's cache was written
    for a, b in ((ok[0], rk[0]), (ov[0], rv[0])):
        mask = np.ones(a.shape[1], bool)
        mask[L] = False
        assert np.array_equal(a[:, mask], b[:, mask])


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
def test_step_matches_reference_ragged_batch(orc, ref_strict, synth, nerr, qtype_name):
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}[qtype_name]
    lengths = [5, 17, 0, 31, 9, 2, 25, 12]
    mems = [7, 19, 3, 32, 11, 1, 27, 16]
    cfg, want, got, _, _ = _run_both(orc, synth, qtype, 2, lengths, mems, True)
    tol = 1e-5 if qtype == orc.F32 else 5e-3
    for b in range(len(lengths)):
        assert nerr(want[b], got[b]) < tol, "stream %d" % b


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
def test_step_matches_reference_empty_memory(orc, ref_strict, synth, nerr, qtype_name):
    """Streams without any encoder memory beside streams that have one: the cross-attention context of the former is
    all zeros (src/graph.c:3237-3244: no row is ever added to the cleared output), so that sublayer leaves x as it was."""
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}[qtype_name]
    lengths = [3, 0, 12, 9]
    mems = [0, 5, 0, 13]
    cfg, want, got, _, _ = _run_both(orc, synth, qtype, 2, lengths, mems, True)
    tol = 1e-5 if qtype == orc.F32 else 5e-3   # as in the ragged batch above
    for b in range(len(lengths)):
        assert np.isfinite(want[b]).all() and np.isfinite(got[b]).all()
        assert nerr(want[b], got[b]) < tol, "stream %d" % b


def test_reference_batched_equals_solo_bitwise(orc, ref, synth):
    """The contract the GPU path inherits (src/graph.h:33-38): a stream inside a batch of 8 is bit-identical
    to the same stream run alone -- shown here on the compiled reference itself."""
    lengths = [5, 17, 0, 31, 9, 2, 25, 12]
    mems = [7, 19, 3, 32, 11, 1, 27, 16]
    cfg = _cfg(synth, 2, 40)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    for qtype in (orc.INT8, orc.INT4):
        rdec = orc.RefDecoder(cfg, weights, qtype, 8, max(mems))
        batch_out, _ = rdec.step([s["k"].copy() for s in streams], [s["v"].copy() for s in streams],
                                 [s["ck"] for s in streams], [s["cv"] for s in streams], lengths, mems,
                                 [s["x"] for s in streams])
        rdec.close()
        solo = orc.RefDecoder(cfg, weights, qtype, 1, max(mems))
        for b in (0, 3, 7):
            s = streams[b]
            one, _ = solo.step([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [lengths[b]], [mems[b]], [s["x"]])
            assert np.array_equal(one[0].view(np.uint32), batch_out[b].view(np.uint32))
        solo.close()


def test_step_capacity_error(orc, synth):
    cfg = synth.decoder_config(layers=1, capacity=8, cross_heads=1)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, [7], [4], seed=1)
    odec = orc.Decoder(cfg, weights, orc.F32)
    s = streams[0]
    odec.step([s["k"]], [s["v"]], [s["ck"]], [s["cv"]], [7], [4], [s["x"]])          # last row still fits
    with pytest.raises(RuntimeError):                                                 # src/graph.c:3152-3155
        odec.step([s["k"]], [s["v"]], [s["ck"]], [s["cv"]], [8], [4], [s["x"]])


def test_multi_head_cross_and_bias_generalisation(orc, synth, nerr):
    """The synthetic configurations use LayerNorm bias and 12x64 cross heads, which the reference's step
    does not have: check that generalisation against float64 on one layer."""
    cfg = synth.decoder_config(layers=1, capacity=24)
    w = synth.decoder_weights(cfg, seed=2)
    s = synth.decoder_streams(cfg, [20], [13], seed=3)[0]
    out = orc.Decoder(cfg, w, orc.F32).step([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [20], [13], [s["x"]])[0]

    def ln(x, g, b):
        mu = x.mean()
        return (x - mu) / np.sqrt(((x - mu) ** 2).mean() + 1e-5) * g + b

    def attend(q, K, V, heads):
        hw = q.size // heads
        o = np.empty_like(q)
        for h in range(heads):
            sl = slice(h * hw, (h + 1) * hw)
            sc = K[:, sl] @ q[sl] / np.sqrt(hw)
            p = np.exp(sc - sc.max())
            p /= p.sum()
            o[sl] = p @ V[:, sl]
        return o

    f = lambda a: np.asarray(a, np.float64)
    W = cfg["width"]
    x = f(s["x"]) + f(w["position"][20])
    qkv = f(w["qkv"][0]) @ ln(x, f(w["norm_self_g"][0]), f(w["norm_self_b"][0]))
    K = np.concatenate([f(s["k"][0, :20]), qkv[None, W:2 * W]])
    V = np.concatenate([f(s["v"][0, :20]), qkv[None, 2 * W:]])
    x = x + f(w["o_self"][0]) @ attend(qkv[:W], K, V, cfg["heads"])
    qx = f(w["q_cross"][0]) @ ln(x, f(w["norm_cross_g"][0]), f(w["norm_cross_b"][0]))
    x = x + f(w["o_cross"][0]) @ attend(qx, f(s["ck"][0]), f(s["cv"][0]), cfg["cross_heads"])
    h = f(w["ffn_up"][0]) @ ln(x, f(w["norm_ff_g"][0]), f(w["norm_ff_b"][0]))
    h = 0.5 * h * (1 + np.tanh(0.7978845608 * (h + 0.044715 * h ** 3)))
    x = x + f(w["ffn_down"][0]) @ h
    want = ln(x, f(w["norm_out_g"]), f(w["norm_out_b"]))
    assert nerr(out, want) < 1e-5


def test_forced_activations_hook(orc, synth):
    """The hook the GPU's teacher-forced comparison rests on: a step fed its own captured int8 activations is the plain step
    bit for bit with no element counted as different; moving one activation by one step is counted as exactly that and
    changes the output; the captured vectors obey quantize_act_int8's invariants (|q| <= 127, the largest is 127, scale =
    absmax / 127 > 0)."""
    cfg = synth.decoder_config(layers=2, capacity=40)
    weights = synth.decoder_weights(cfg, seed=0)
    s = synth.decoder_streams(cfg, [33], [17], seed=1)[0]
    for qtype in (orc.INT8, orc.INT4):
        dec = orc.Decoder(cfg, weights, qtype)
        args = lambda: ([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [33], [17], [s["x"]])
        plain = dec.step(*args())[0]
        outs, flips, step, (qx, sx) = dec.step_forced(*args())
        assert np.array_equal(outs[0].view(np.uint32), plain.view(np.uint32)) and flips == 0 and step == 0
        widths = [768, 768, 768, 768, 768, 3072]
        for layer in range(2):
            for slot, k in enumerate(widths):
                q = qx[layer, slot, :k].astype(np.int32)
                assert np.abs(q).max() == 127 and sx[layer, slot] > 0.0
                assert not qx[layer, slot, k:].any()
        again, flips, step, _ = dec.step_forced(*args(), qx=qx, sx=sx)
        assert np.array_equal(again[0].view(np.uint32), plain.view(np.uint32)) and flips == 0 and step == 0
        moved = qx.copy()
        at = int(np.argmin(np.abs(moved[1, 5, :3072].astype(np.int32))))     # an element away from the clamp, in the step's last projection
        moved[1, 5, at] += 1                                                 # (earlier ones would also move what the later ones quantise)
        other, flips, step, _ = dec.step_forced(*args(), qx=moved, sx=sx)
        assert flips == 1 and step == 1
        assert not np.array_equal(other[0].view(np.uint32), plain.view(np.uint32))
