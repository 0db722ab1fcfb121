"""GPU parity of the resident local-transformer frame (mynah_hip_local_frame) through the C ABI.

Two layers of evidence:
 * the token choice alone, bit for bit: the device hands back the masked logits each choice was made from, and the oracle's
   orc_local_choose (src/graph.c:1548-1616 restated) replays every choice of every item from those very floats, including
   the generator chain -- independent of any float difference in the stack before it;
 * the whole frame against the oracle's frame: logits within the step's tolerance at every position up to the first
   position where the two sides chose different tokens (after which they legitimately see different inputs), and such a
   divergence only where the oracle's two best candidates were closer than the tolerance.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

QT = {"f32": 0, "int8": 1, "int4": 2, "f16": 3}
TOL = {"f32": 1e-5, "f16": 1e-5, "int8": 2e-2, "int4": 2e-2}   # normalised max error of a projection row, as for the decode step


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _setup(synth, layers, streams, vocab, seed, eos_boost=()):
    cfg = synth.decoder_config(layers=layers, capacity=streams + 1, cross_heads=0)
    w = synth.decoder_weights(cfg, seed=seed, ln_bias=False)
    w["norm_out_g"] = w["norm_out_b"] = None
    rng = np.random.default_rng(seed + 1)
    proj = [(rng.standard_normal((vocab, cfg["width"])) * 0.05).astype(np.float32) for _ in range(streams)]
    bias = [(rng.standard_normal(vocab) * 0.1).astype(np.float32) for _ in range(streams)]
    tables = [rng.standard_normal((vocab, cfg["width"])).astype(np.float32) for _ in range(streams)]
    return cfg, w, proj, bias, tables, rng


ITEMS = [
    {"temperature": 0.0, "topk": 1, "rng_state": 11, "forbid_eos": False},
    {"temperature": 0.8, "topk": 50, "rng_state": 0x1234567, "forbid_eos": True},
    {"temperature": 1.3, "topk": 256, "rng_state": 0xDEADBEEFCAFE, "forbid_eos": False},
    {"temperature": 0.4, "topk": 2, "rng_state": 0, "forbid_eos": False},          # the all-zero state is replaced
    {"temperature": 0.7, "topk": 1, "rng_state": 5, "forbid_eos": True},           # topk 1: greedy, generator untouched
    {"temperature": 1.0, "topk": 7, "rng_state": 99, "forbid_eos": True},
]


def _replay_choices(orc, logits, items, out, codebook, eos, codebook_count):
    """Every choice of the frame again on the CPU, from the device's own masked logits."""
    B, S, _ = logits.shape
    for b in range(B):
        state = items[b]["rng_state"]
        saw, eos_frame = 0, np.iinfo(np.uint64).max
        for s in range(S):
            value, greedy, state, _ = orc.local_choose(logits[b, s], codebook, eos, items[b]["temperature"], items[b]["topk"], state,
                                                       items[b]["forbid_eos"])
            assert out["values"][b, s] == value, "item %d position %d" % (b, s)
            assert out["stored"][b, s] == (value if value < codebook else 0)
            if greedy == eos or value == eos:
                saw, eos_frame = 1, min(eos_frame, s // codebook_count)
        assert out["rng_state"][b] == state, "generator of item %d" % b
        assert out["saw_eos"][b] == saw and out["eos_frame"][b] == eos_frame


def _compare_with_oracle_frame(nerr, got, got_logits, want, items, tol):
    """A greedy item may part from the oracle only where the oracle's two candidates are within the tolerance of each
    other.  A sampling item may part wherever the tolerance is the quantised one (a 1e-2 shift of the logits moves the
    cumulative boundaries by as much, and a draw falls that close to one of them every few dozen draws); at 1e-5 it must
    not part at all."""
    B, S, _ = got_logits.shape
    compared = 0
    for b in range(B):
        sampling = items[b]["temperature"] > 0 and items[b]["topk"] > 1
        for s in range(S):
            assert nerr(got_logits[b, s], want["logits"][b, s]) < tol, "logits of item %d position %d" % (b, s)
            compared += 1
            if got["values"][b, s] != want["values"][b, s]:
                what = "item %d position %d chose %d, oracle %d" % (b, s, got["values"][b, s], want["values"][b, s])
                if sampling:
                    assert tol > 1e-4, what
                else:
                    lg = want["logits"][b, s]
                    reach = float(np.max(np.abs(lg[lg > -1e30])))
                    assert abs(float(lg[got["values"][b, s]]) - float(lg[want["values"][b, s]])) <= 2 * tol * reach, what
                break   # from here on the two sides feed different embeddings
    return compared


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4", "f16"])
def test_frame_small_vocab(pkg, backend, orc, synth, nerr, qtype_name):
    """Two layers, 16 positions, vocabulary 96, six items with every kind of sampling setting,
    forced EOS at two positions."""
    _announce("local frame vocab 96 %s" % qtype_name)
    S, V, codebook, eos, cbc = 16, 96, 80, 83, 8
    cfg, w, proj, bias, tables, rng = _setup(synth, 2, S, V, seed=41)
    for s in (6, 12):
        bias[s][eos] = 50.0
    backend.set_quant(QT[qtype_name])
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
    B = len(ITEMS)
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
    drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
    dlogits = backend.alloc(B * S * V)
    items = [dict(it, row=d.ptr) for it, d in zip(ITEMS, drows)]
    got = loc.frame(items, dlogits.ptr)
    logits = dlogits.read().reshape(B, S, V)
    _replay_choices(orc, logits, ITEMS, got, codebook, eos, cbc)
    assert got["saw_eos"][0] == 1 and got["eos_frame"][0] == 6 // cbc and got["values"][0, 6] == eos and got["stored"][0, 6] == 0
    assert got["saw_eos"][1] == 0 and np.all(got["values"][1] < codebook)           # EOS forbidden: never chosen, never seen

    qt = QT[qtype_name]
    stack = orc.Decoder(cfg, w, qt)
    oframe = orc.LocalFrame(stack, [orc.PackedWeight(p, qt) for p in proj], bias, tables, codebook, eos, cbc)
    want = oframe.frame(rows, ITEMS, want_logits=True)
    compared = _compare_with_oracle_frame(nerr, got, logits, want, ITEMS, TOL[qtype_name])
    assert compared >= B        # at least position 0 of every item
    if qtype_name == "f32":
        assert np.array_equal(got["values"], want["values"]) and got["rng_state"] == want["rng_state"]

    # a second frame: the caches restart, the captured step replays, the generators continue where they stopped
    items2 = [dict(it, rng_state=st) for it, st in zip(items, got["rng_state"])]
    again = loc.frame(items2, dlogits.ptr)
    logits2 = dlogits.read().reshape(B, S, V)
    _replay_choices(orc, logits2, [dict(it, rng_state=st) for it, st in zip(ITEMS, got["rng_state"])], again, codebook, eos, cbc)
    for b in (0, 4):   # greedy items: the same frame again, bit for bit
        assert np.array_equal(again["values"][b], got["values"][b]) and np.array_equal(logits2[b], logits[b])
    # a smaller batch afterwards gives each item what it got in the larger one (greedy item 0)
    solo = loc.frame([items[0]], dlogits.ptr)
    assert np.array_equal(solo["values"][0], got["values"][0])
    assert np.array_equal(dlogits.read(S * V).reshape(S, V), logits[0])
    loc.destroy()
    for d in drows + [dlogits]:
        d.free()
    backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["int8", "f32"])
def test_frame_model_shape_batch8(pkg, backend, orc, synth, nerr, qtype_name):
    """The model's shape: one 768-wide layer, 16 positions, 2048 logits (fused matvec path for the projection), batch 8,
    ties planted among the candidates through equal projection rows."""
    _announce("local frame vocab 2048 batch 8 %s" % qtype_name)
    S, V, codebook, eos, cbc = 16, 2048, 2016, 2017, 8
    cfg, w, proj, bias, tables, rng = _setup(synth, 1, S, V, seed=51)
    for s in range(S):
        proj[s][100:140] = proj[s][7]             # forty candidates with bit-identical logits
        bias[s][100:140] = bias[s][7]
    backend.set_quant(QT[qtype_name])
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
    B = 8
    base = [ITEMS[i % len(ITEMS)] for i in range(B)]
    base = [dict(it, rng_state=it["rng_state"] + 977 * i) for i, it in enumerate(base)]
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
    drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
    dlogits = backend.alloc(B * S * V)
    got = loc.frame([dict(it, row=d.ptr) for it, d in zip(base, drows)], dlogits.ptr)
    logits = dlogits.read().reshape(B, S, V)
    assert np.all(logits[:, :, 100:140] == logits[:, :, 7:8])
    _replay_choices(orc, logits, base, got, codebook, eos, cbc)
    qt = QT[qtype_name]
    oframe = orc.LocalFrame(orc.Decoder(cfg, w, qt), [orc.PackedWeight(p, qt) for p in proj], bias, tables, codebook, eos, cbc)
    want = oframe.frame(rows, base, want_logits=True)
    _compare_with_oracle_frame(nerr, got, logits, want, base, TOL[qtype_name])
    loc.destroy()
    for d in drows + [dlogits]:
        d.free()
    backend.set_quant(0)


def test_frame_batch16_two_tiles(pkg, backend, orc, synth, nerr):
    """Sixteen items (two passes of eight through every matvec, the many-stream attention layout), alternating greedy and
    sampling, f32: tokens and generator states equal to the oracle's frame."""
    _announce("local frame batch 16 f32")
    S, V, codebook, eos, cbc = 16, 512, 480, 481, 8
    cfg, w, proj, bias, tables, rng = _setup(synth, 1, S, V, seed=71)
    backend.set_quant(0)
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
    B = 16
    base = [dict(ITEMS[i % len(ITEMS)], rng_state=ITEMS[i % len(ITEMS)]["rng_state"] + 31 * i) for i in range(B)]
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
    drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
    dlogits = backend.alloc(B * S * V)
    for attempt in range(2):     # eager frame, then the captured one
        got = loc.frame([dict(it, row=d.ptr) for it, d in zip(base, drows)], dlogits.ptr)
        logits = dlogits.read().reshape(B, S, V)
        _replay_choices(orc, logits, base, got, codebook, eos, cbc)
    oframe = orc.LocalFrame(orc.Decoder(cfg, w, 0), [orc.PackedWeight(p, 0) for p in proj], bias, tables, codebook, eos, cbc)
    want = oframe.frame(rows, base, want_logits=True)
    _compare_with_oracle_frame(nerr, got, logits, want, base, TOL["f32"])
    assert np.array_equal(got["values"], want["values"]) and got["rng_state"] == want["rng_state"]
    loc.destroy()
    for d in drows + [dlogits]:
        d.free()


def test_frame_many_tied_candidates(pkg, backend, orc, synth, nerr):
    """Seven hundred ids share the largest logit, so more candidates reach the sampler's first bound than its fast list
    holds and the exact selection runs with short lists (top-k 2, 7, 50) as well as a long one (256): the list is the
    tied ids in ascending order, as the reference's insertion keeps the earlier id first (src/graph.c:1580-1598)."""
    _announce("local frame, 700 tied largest logits")
    S, V, codebook, eos, cbc = 4, 2048, 2016, 2017, 4
    cfg, w, proj, bias, tables, rng = _setup(synth, 1, S, V, seed=67)
    for s in range(S):
        proj[s][200:900] = proj[s][7]
        bias[s][200:900] = bias[s][7] = 25.0
    backend.set_quant(QT["f32"])
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
    B = len(ITEMS)
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
    drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
    dlogits = backend.alloc(B * S * V)
    got = loc.frame([dict(it, row=d.ptr) for it, d in zip(ITEMS, drows)], dlogits.ptr)
    logits = dlogits.read().reshape(B, S, V)
    assert np.all(logits[:, :, 200:900] == logits[:, :, 7:8]) and np.all(logits.max(axis=2) == logits[:, :, 7])
    _replay_choices(orc, logits, ITEMS, got, codebook, eos, cbc)
    for b, it in enumerate(ITEMS):   # a list of k tied ids starts 7, 200, 201, ...: nothing beyond its k-th id can be chosen
        k = it["topk"]
        assert np.all((got["values"][b] == 7) | ((got["values"][b] >= 200) & (got["values"][b] < 200 + max(k - 1, 0)))), (b, got["values"][b])
    loc.destroy()
    for d in drows + [dlogits]:
        d.free()
    backend.set_quant(0)


def test_frame_eos_outside_vocabulary(pkg, backend, orc, synth, nerr):
    """An end-of-sequence id that is no id of the vocabulary (here one whose low 32 bits are 5, a real id) matches
    nothing, as in the reference's full-width comparison (src/graph.c:1563-1574): only codebook ids are ever allowed,
    allowed or forbidden makes no difference, and no end of sequence is reported.  Likewise a codebook size above the
    vocabulary allows every id."""
    _announce("local frame, eos id outside the vocabulary")
    S, V, codebook, cbc = 8, 96, 80, 4
    eos = 2 ** 32 + 5
    cfg, w, proj, bias, tables, rng = _setup(synth, 2, S, V, seed=43)
    for s in range(S):
        bias[s][5] = 30.0       # id 5 is the greedy choice everywhere: a truncated eos id would report it as EOS
        bias[s][90] = 40.0      # above the codebook: never allowed, since it is not the eos id either
    backend.set_quant(QT["f32"])
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
    B = len(ITEMS)
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
    drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
    dlogits = backend.alloc(B * S * V)
    items = [dict(it, row=d.ptr) for it, d in zip(ITEMS, drows)]
    got = loc.frame(items, dlogits.ptr)
    logits = dlogits.read().reshape(B, S, V)
    _replay_choices(orc, logits, ITEMS, got, codebook, eos, cbc)
    assert not np.any(got["saw_eos"]) and np.all(got["values"] < codebook)
    assert np.all(got["values"][0] == 5) and np.all(got["values"][4] == 5)      # the greedy items
    stack = orc.Decoder(cfg, w, QT["f32"])
    oframe = orc.LocalFrame(stack, [orc.PackedWeight(p, QT["f32"]) for p in proj], bias, tables, codebook, eos, cbc)
    want = oframe.frame(rows, ITEMS, want_logits=True)
    _compare_with_oracle_frame(nerr, got, logits, want, ITEMS, TOL["f32"])
    assert np.array_equal(got["values"], want["values"]) and got["rng_state"] == want["rng_state"]
    loc.destroy()

    # a codebook size beyond the vocabulary: every id allowed, 90 wins everywhere for the greedy items
    loc = pkg.Local(backend, cfg, w, proj, bias, tables, 2 ** 33, eos, cbc)
    got = loc.frame(items, dlogits.ptr)
    logits = dlogits.read().reshape(B, S, V)
    _replay_choices(orc, logits, ITEMS, got, 2 ** 33, eos, cbc)
    assert np.all(got["values"][0] == 90) and np.array_equal(got["stored"], got["values"]) and not np.any(got["saw_eos"])
    loc.destroy()
    for d in drows + [dlogits]:
        d.free()
    backend.set_quant(0)


def test_frame_error_paths(pkg, backend, synth):
    _announce("local frame error paths")
    S, V = 4, 512
    cfg, w, proj, bias, tables, rng = _setup(synth, 1, S, V, seed=61)
    backend.set_quant(0)
    loc = pkg.Local(backend, cfg, w, proj, None, tables, 500, 501, 2)
    drow = backend.alloc(cfg["width"]).write(rng.standard_normal(cfg["width"]).astype(np.float32))
    ok = {"row": drow.ptr, "temperature": 0.0, "topk": 1, "rng_state": 1, "forbid_eos": False}
    with pytest.raises(pkg.BackendError, match="local frame batch exceeds MYNAH_MAX_BATCH"):
        loc.frame([ok] * 17)
    with pytest.raises(pkg.BackendError, match="local sampler scratch too small"):
        loc.frame([dict(ok, temperature=1.0, topk=300)])
    with pytest.raises(pkg.BackendError, match="no input row"):
        loc.frame([dict(ok, row=None)])
    out = loc.frame([ok])     # still usable after the refusals
    assert out["values"].shape == (1, S) and np.all(out["values"] < 502)
    assert loc.frame([])["values"].shape == (0, S)
    loc.destroy()
    # a stack with cross attention or a final norm is not a local stack
    cfg2 = synth.decoder_config(layers=1, capacity=S + 1, cross_heads=12)
    w2 = synth.decoder_weights(cfg2, seed=62, ln_bias=False)
    with pytest.raises(pkg.BackendError, match="no cross attention"):
        pkg.Local(backend, cfg2, w2, proj, None, tables, 500, 501, 2)
    drow.free()
