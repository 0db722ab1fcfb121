"""GPU parity of the resident batched decode step against the oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


class Harness:
    """Uploads a set of synthetic streams and runs mynah_hip_decoder_step on them."""

    def __init__(self, pkg, backend, cfg, weights, streams):
        self.backend, self.cfg, self.streams = backend, cfg, streams
        self.dec = pkg.Decoder(backend, cfg, weights)
        self.bufs = []
        for s in streams:
            b = {n: backend.alloc(max(s[n].size, 4)).write(s[n]) if s[n].size else backend.alloc(4) for n in ("k", "v", "ck", "cv", "x")}
            b["out"] = backend.alloc(cfg["width"])
            self.bufs.append(b)

    def slots(self, which=None):
        which = range(len(self.streams)) if which is None else which
        return [{"k": self.bufs[i]["k"].ptr, "v": self.bufs[i]["v"].ptr, "ck": self.bufs[i]["ck"].ptr, "cv": self.bufs[i]["cv"].ptr,
                 "length": self.streams[i]["length"], "memory_length": self.streams[i]["memory_length"],
                 "inp": self.bufs[i]["x"].ptr, "out": self.bufs[i]["out"].ptr} for i in which]

    def step(self, which=None):
        self.dec.step(self.slots(which))
        which = range(len(self.streams)) if which is None else which
        return [self.bufs[i]["out"].read() for i in which]

    def reset_cache(self, i):
        self.bufs[i]["k"].write(self.streams[i]["k"])
        self.bufs[i]["v"].write(self.streams[i]["v"])

    def cache_rows(self, i):
        shape = self.streams[i]["k"].shape
        return self.bufs[i]["k"].read().reshape(shape), self.bufs[i]["v"].read().reshape(shape)

    def close(self):
        self.dec.destroy()
        for b in self.bufs:
            for d in b.values():
                d.free()


def _oracle_step(orc, cfg, weights, streams, qtype):
    odec = orc.Decoder(cfg, weights, qtype)
    ks = [s["k"].copy() for s in streams]
    vs = [s["v"].copy() for s in streams]
    outs = odec.step(ks, vs, [s["ck"] for s in streams], [s["cv"] for s in streams], [s["length"] for s in streams],
                     [s["memory_length"] for s in streams], [s["x"] for s in streams])
    return outs, ks, vs


QT = {"f32": 0, "int8": 1, "int4": 2, "f16": 3}
# f32/f16 activations stay f32 end to end: 1e-5 normalised (f16: against the oracle run on the same f16 bits).
# int8/int4 re-quantise the activation of every projection.  With the same int8 activations on both sides a quantised
# step agrees like an f32 one (1e-5); but the GPU's LayerNorm adds in another order than the CPU's, and a last-bit
# difference there moves an activation that sits on a rounding boundary by one int8 step -- about 1e-3 of the output's
# scale, amplified by the layers that follow.  Roughly one (stream, layer) in thirty meets such a boundary.  So a
# quantised whole-step comparison asserts the shape of that: every stream below OUTLIER, and at most a stated number of
# streams above TOL["f32"] (quantised_errors_ok).  The per-projection integers are bit-exact in test_gpu_seam.py.
TOL = {"f32": 1e-5, "f16": 1e-5, "int8": 2e-2, "int4": 2e-2}
OUTLIER = 2e-2


def quantised_errors_ok(errors, max_outliers, what=""):
    """errors: normalised errors of the streams (or rows) of one quantised comparison."""
    errors = [float(e) for e in errors]
    above = [e for e in errors if e >= TOL["f32"]]
    print("[quantised] %s errors %s" % (what, " ".join("%.1e" % e for e in errors)), flush=True)
    assert all(e < OUTLIER for e in errors), "%s: a stream is beyond the outlier bound: %s" % (what, errors)
    assert len(above) <= max_outliers, "%s: %d streams above 1e-5 (at most %d expected): %s" % (what, len(above), max_outliers, errors)


@pytest.mark.parametrize("qtype_name", ["f32", "f16", "int8", "int4"])
def test_one_block_batch1_kv256(pkg, backend, orc, synth, nerr, qtype_name):
    """One decoder block, batch 1, KV length 256, LayerNorm gain and bias (the f32 case is the benchmark's
    CPU-runnable configuration)."""
    _announce("one block b=1 kv=256 %s" % qtype_name)
    cfg = synth.decoder_config(layers=1, capacity=258, cross_heads=0)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [256], [0], seed=1)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    got = h.step()
    want, ks, vs = _oracle_step(orc, cfg, weights, streams, QT[qtype_name])
    assert nerr(got[0], want[0]) < TOL[qtype_name]
    gk, gv = h.cache_rows(0)
    assert nerr(gk[0, 256], ks[0][0, 256]) < TOL[qtype_name] and nerr(gv[0, 256], vs[0][0, 256]) < TOL[qtype_name]
    mask = np.ones(258, bool)
    mask[256] = False
    assert np.array_equal(gk[:, mask], streams[0]["k"][:, mask]) and np.array_equal(gv[:, mask], streams[0]["v"][:, mask])
    h.close()
    backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4", "f16"])
def test_two_layers_ragged_batch8_and_bit_identity(pkg, backend, orc, synth, nerr, qtype_name):
    """Ragged B=8 (incl. an empty cache and chunk-edge lengths) against the oracle, eager and graph replay,
    and every stream bit-identical to the same stream run alone on the GPU."""
    _announce("two layers ragged b=8 %s" % qtype_name)
    lengths = [5, 64, 0, 129, 63, 2, 300, 65]
    mems = [7, 64, 3, 32, 65, 1, 27, 200]
    cfg = synth.decoder_config(layers=2, capacity=304)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    want, ks, vs = _oracle_step(orc, cfg, weights, streams, QT[qtype_name])
    first = h.step()                        # eager (first use of this batch size)
    if qtype_name in ("int8", "int4"):      # 16 (stream, layer) pairs: at most two streams may have met a rounding boundary
        quantised_errors_ok([nerr(first[b], want[b]) for b in range(8)], 2, "two layers b=8 " + qtype_name)
    else:
        for b in range(8):
            assert nerr(first[b], want[b]) < TOL[qtype_name], "stream %d" % b
    for b in (0, 3, 6):
        gk, gv = h.cache_rows(b)
        L = lengths[b]
        for layer in range(2):
            assert nerr(gk[layer, L], ks[b][layer, L]) < TOL[qtype_name]
            assert nerr(gv[layer, L], vs[b][layer, L]) < TOL[qtype_name]
    # graph capture + three replays, interleaved with host reads, must reproduce the eager result bit for bit
    for replay in range(4):
        for b in range(8):
            h.reset_cache(b)
        again = h.step()
        for b in range(8):
            assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32)), "replay %d stream %d" % (replay, b)
    # batched == solo, bitwise, for every stream
    for b in range(8):
        h.reset_cache(b)
        solo = h.step([b])[0]
        assert np.array_equal(solo.view(np.uint32), first[b].view(np.uint32)), "stream %d differs from its solo run" % b
    # a different batch composition (B = 3) keeps each stream's bits as well
    for b in (1, 4, 7):
        h.reset_cache(b)
    sub = h.step([7, 1, 4])
    for got, b in zip(sub, (7, 1, 4)):
        assert np.array_equal(got.view(np.uint32), first[b].view(np.uint32))
    h.close()
    backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["f32", "int8"])
def test_streams_without_memory(pkg, backend, orc, synth, nerr, qtype_name):
    """Streams whose encoder memory is empty (no cross cache at all) beside streams that have one: their
    cross-attention context is zero (src/graph.c:3237-3244).  Batch 4 takes the workgroup numbering over live units
    and the stand-alone fold, the pairs take the latency layout with the fold inside the output projection; a
    stream's bits are the same in both."""
    _announce("streams without memory %s" % qtype_name)
    lengths = [3, 0, 128, 40]
    mems = [0, 5, 0, 130]
    cfg = synth.decoder_config(layers=2, capacity=136)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=2)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    want, ks, vs = _oracle_step(orc, cfg, weights, streams, QT[qtype_name])
    first = h.step()
    if qtype_name == "int8":
        quantised_errors_ok([nerr(first[b], want[b]) for b in range(4)], 1, "streams without memory int8")
    for b in range(4):
        assert np.isfinite(first[b]).all(), "stream %d" % b
        assert nerr(first[b], want[b]) < TOL[qtype_name], "stream %d" % b
    for replay in range(2):   # second call of this batch size is captured, third replays the graph
        for b in range(4):
            h.reset_cache(b)
        again = h.step()
        for b in range(4):
            assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32)), "replay %d stream %d" % (replay, b)
    for pair in ((0, 1), (2, 3), (0, 2)):
        for b in pair:
            h.reset_cache(b)
        got = h.step(list(pair))
        for out, b in zip(got, pair):
            assert np.array_equal(out.view(np.uint32), first[b].view(np.uint32)), "stream %d in pair %s" % (b, pair)
    h.close()
    backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["f32", "int8"])
def test_last_row_of_the_cache(pkg, backend, orc, synth, nerr, qtype_name):
    """length == capacity - 1 appends into the last row the cache has (one more is the capacity error of
    src/graph.c:3152-3155); beside it a stream whose cache is exactly one full attention unit and one that is a row
    short of it.  Outputs and appended rows against the oracle; every other cache row untouched."""
    _announce("last cache row %s" % qtype_name)
    capacity = 256
    lengths = [capacity - 1, 128, 127]
    mems = [9, 1, 128]
    cfg = synth.decoder_config(layers=2, capacity=capacity)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=4)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    want, ks, vs = _oracle_step(orc, cfg, weights, streams, QT[qtype_name])
    got = h.step()
    for b, L in enumerate(lengths):
        assert nerr(got[b], want[b]) < TOL[qtype_name], "stream %d" % b
        gk, gv = h.cache_rows(b)
        for layer in range(2):
            assert nerr(gk[layer, L], ks[b][layer, L]) < TOL[qtype_name]
            assert nerr(gv[layer, L], vs[b][layer, L]) < TOL[qtype_name]
        mask = np.ones(capacity, bool)
        mask[L] = False
        assert np.array_equal(gk[:, mask], streams[b]["k"][:, mask]) and np.array_equal(gv[:, mask], streams[b]["v"][:, mask])
    # one row further is refused, and refusing it changes nothing
    slots = h.slots()
    slots[0]["length"] = capacity
    with pytest.raises(pkg.BackendError, match="capacity exceeded"):
        h.dec.step(slots)
    for b in range(3):
        gk, gv = h.cache_rows(b)
        assert nerr(gk[0, lengths[b]], ks[b][0, lengths[b]]) < TOL[qtype_name]
    h.close()
    backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["int8", "int4"])
@pytest.mark.parametrize("layers,length,mem,seeds", [(2, 300, 65, 10), (12, 1023, 256, 2)])
def test_teacher_forced_quantised_step(pkg, backend, orc, synth, nerr, qtype_name, layers, length, mem, seeds):
    """What the 2e-2 bar of the quantised whole-step comparisons stands for, turned into an assertion: the device reports the
    int8 activation vector and scale it formed at every projection of every layer (mynah_hip_decoder_step_probe), the
    oracle runs the same step on THOSE integers instead of its own, and the two outputs then agree like an f32 step --
    1e-5, no outlier allowance, appended cache rows included, for every one of a row of seeded inputs.  The device's
    integers differ from the oracle's own in a handful of elements at most, each by one int8 step (an activation on a
    rounding boundary that a last-bit difference in the LayerNorm sums moves), and the probing step gives the bits of the
    ordinary step."""
    _announce("teacher-forced %s step, %d layers, kv %d/%d" % (qtype_name, layers, length, mem))
    cfg = synth.decoder_config(layers=layers, capacity=length + 2)
    weights = synth.decoder_weights(cfg, seed=0)
    backend.set_quant(QT[qtype_name])
    odec = orc.Decoder(cfg, weights, QT[qtype_name])
    elements = layers * (5 * 768 + 3072)
    total_flips, unforced_outliers = 0, 0
    try:
        for seed in range(seeds):
            streams = synth.decoder_streams(cfg, [length], [mem], seed=90 + seed)
            h = Harness(pkg, backend, cfg, weights, streams)
            try:
                ordinary = h.step()[0]
                rows_ordinary = [a[:, length].copy() for a in h.cache_rows(0)]
                h.reset_cache(0)
                qx, sx = h.dec.step_probe(h.slots())
                probed = h.bufs[0]["out"].read()
                assert np.array_equal(probed.view(np.uint32), ordinary.view(np.uint32)), "the probing step is not the ordinary step"
                s = streams[0]
                ks, vs = [s["k"].copy()], [s["v"].copy()]
                want, flips, step, (own_qx, own_sx) = odec.step_forced(ks, vs, [s["ck"]], [s["cv"]], [length], [mem], [s["x"]], qx=qx, sx=sx)
                plain = odec.step([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [length], [mem], [s["x"]])[0]
                total_flips += flips
                unforced_outliers += nerr(ordinary, plain) >= 1e-5
                print("[teacher-forced] %s seed %d: %d of %d int8 activations differ from the oracle's own (largest difference %d); error forced "
                      "%.2e, unforced %.2e" % (qtype_name, seed, flips, elements, step, nerr(ordinary, want[0]), nerr(ordinary, plain)), flush=True)
                assert nerr(ordinary, want[0]) < 1e-5, "seed %d" % seed
                assert nerr(rows_ordinary[0], ks[0][:, length]) < 1e-5 and nerr(rows_ordinary[1], vs[0][:, length]) < 1e-5
                assert step <= 1, "an int8 activation differs from the oracle's by more than one step"
                assert flips <= max(4, elements // 500), "too many int8 activations differ from the oracle's own: %d" % flips
                assert np.abs(sx - own_sx).max() <= 1e-5 * np.abs(own_sx).max()
                assert flips > 0 or nerr(ordinary, plain) < 1e-5, "the unforced oracle differs although every int8 activation agrees"
            finally:
                h.close()
        print("[teacher-forced] %s: %d differing activations over %d inputs, %d inputs above 1e-5 unforced" % (qtype_name, total_flips, seeds, unforced_outliers),
              flush=True)
    finally:
        backend.set_quant(0)


def test_twelve_layers_int8_multi_step(pkg, backend, orc, synth, nerr):
    """The benchmark stack (12 layers, 12x64 cross heads, int8) at reduced cache length, two consecutive steps
    so that the second step attends over the row the first one appended."""
    _announce("12 layers int8 two steps")
    cfg = synth.decoder_config(layers=12, capacity=132)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [128, 40], [64, 48], seed=1)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    odec = orc.Decoder(cfg, weights, orc.INT8)
    ks = [s["k"].copy() for s in streams]
    vs = [s["v"].copy() for s in streams]
    lengths = [128, 40]
    for step in range(2):
        for i, s in enumerate(streams):
            s["length"] = lengths[i]
        want = odec.step(ks, vs, [s["ck"] for s in streams], [s["cv"] for s in streams], lengths, [64, 48], [s["x"] for s in streams])
        got = h.step()
        # 24 (stream, layer) pairs per step: either stream may have met a rounding boundary, neither may leave the bound
        quantised_errors_ok([nerr(got[b], want[b]) for b in range(2)], 2, "12 layers int8 step %d" % step)
        lengths = [n + 1 for n in lengths]
    h.close()
    backend.set_quant(0)


def test_step_error_paths(pkg, backend, synth):
    _announce("step error paths")
    cfg = synth.decoder_config(layers=1, capacity=8)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [7], [4], seed=1)
    h = Harness(pkg, backend, cfg, weights, streams)
    h.step()                                             # the last row still fits
    streams[0]["length"] = 8
    with pytest.raises(pkg.BackendError, match="capacity exceeded"):      # src/graph.c:3152-3155
        h.step()
    streams[0]["length"] = 7
    with pytest.raises(pkg.BackendError, match="MYNAH_MAX_BATCH"):        # src/graph.c:3133-3136
        h.dec.step(h.slots([0] * 17))
    h.dec.step([])                                       # empty batch is a no-op (src/graph.c:3132)
    h.close()


def test_output_head(pkg, backend, orc, synth, nerr):
    """Final-normed rows -> 8 x 1024 logits -> per-head softmax, int8 and f32 weights."""
    _announce("output head")
    rng = np.random.default_rng(1100)
    w = backend.keep((rng.standard_normal((8192, 768)) * 0.02).astype(np.float32))
    hidden = rng.standard_normal((3, 768)).astype(np.float32)
    for qtype in (pkg.F32, pkg.INT8, pkg.INT4):
        backend.set_quant(qtype)
        dh = [backend.alloc(768).write(hidden[b]) for b in range(3)]
        dl = [backend.alloc(8192) for _ in range(3)]
        dp = [backend.alloc(8192) for _ in range(3)]
        backend.output_head([d.ptr for d in dh], 768, w, None, 8192, 1024, [d.ptr for d in dl], [d.ptr for d in dp])
        pw = orc.PackedWeight(w, qtype)
        for b in range(3):
            logits, probs = orc.output_head(pw, hidden[b], 8, 1024)
            assert nerr(dl[b].read(), logits) < 1e-5
            got = dp[b].read()
            assert nerr(got, probs) < 1e-5
            assert np.allclose(got.reshape(8, 1024).sum(-1), 1.0, atol=1e-5)
        for d in dh + dl + dp:
            d.free()
    backend.set_quant(0)


@pytest.mark.parametrize("case", ["step", "nomem"])
@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
@pytest.mark.parametrize("arith_name", ["strict", "stock"])
def test_step_against_compiled_reference_fixture(pkg, backend, synth, nerr, qtype_name, arith_name, case):
    """The GPU step against the committed outputs of the reference's own decoder_step_batch (tests/golden): its real head
    shape -- gain-only LayerNorm, ONE 768-wide cross-attention head -- as a ragged batch of 8 ("step") and as a batch of
    four in which two streams have no encoder memory ("nomem").  That head width is not the fused attention
    kernel's, so this also covers the eight-kernel form of the step.  No oracle in between."""
    import os
    import zlib
    _announce("step vs reference fixture %s %s %s" % (case, qtype_name, arith_name))
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"), allow_pickle=False)
    if "%s_%s_%s_out" % (case, qtype_name, arith_name) not in gold.files:
        pytest.skip("the fixture holds no %s outputs for this case" % qtype_name)
    lengths = [int(n) for n in gold[case + "_lengths"]]
    mems = [int(n) for n in gold[case + "_mems"]]
    cfg = synth.decoder_config(layers=2, capacity=max(lengths) + 3, cross_heads=1)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed={"step": 1, "nomem": 2}[case])
    c = 0
    for a in [weights[k] for k in sorted(weights) if weights[k] is not None] + [s[n] for s in streams for n in ("k", "v", "ck", "cv", "x")]:
        c = zlib.crc32(np.ascontiguousarray(a).tobytes(), c)
    if np.uint32(c) != gold[case + "_input_crc"]:
        pytest.skip("numpy's generator produced different synthetic inputs than when the fixture was written")
    backend.set_quant(QT[qtype_name], 0 if arith_name == "strict" else 1)
    h = Harness(pkg, backend, cfg, weights, streams)
    got = h.step()
    tol = TOL[qtype_name]
    if qtype_name != "f32":   # 8 or 4 streams x 2 layers: at most two streams may have met a rounding boundary
        quantised_errors_ok([nerr(got[b], gold["%s_%s_%s_out" % (case, qtype_name, arith_name)][b]) for b in range(len(lengths))], 2,
                            "fixture %s %s %s" % (case, qtype_name, arith_name))
    for b in range(len(lengths)):
        assert np.isfinite(got[b]).all(), "stream %d" % b
        assert nerr(got[b], gold["%s_%s_%s_out" % (case, qtype_name, arith_name)][b]) < tol, "stream %d" % b
        gk, gv = h.cache_rows(b)
        assert nerr(gk[:, lengths[b]], gold["%s_%s_%s_newk" % (case, qtype_name, arith_name)][b]) < tol
        assert nerr(gv[:, lengths[b]], gold["%s_%s_%s_newv" % (case, qtype_name, arith_name)][b]) < tol
    h.close()
    backend.set_quant(0)


def test_batch16_two_lanes(pkg, backend, orc, synth, nerr):
    """MYNAH_MAX_BATCH streams: two lanes of eight streams side by side (each one pass over the weights); oracle parity,
    graph replay == eager, batched == solo bitwise, and the same bits in one lane (two passes one after the other) and in three."""
    _announce("one layer ragged b=16 int8")
    rng = np.random.default_rng(16)
    lengths = [int(n) for n in rng.integers(0, 200, size=16)]
    mems = [int(n) for n in rng.integers(1, 70, size=16)]
    cfg = synth.decoder_config(layers=1, capacity=204)
    weights = synth.decoder_weights(cfg, seed=5)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=6)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        want, ks, vs = _oracle_step(orc, cfg, weights, streams, 1)
        first = h.step()
        quantised_errors_ok([nerr(first[b], want[b]) for b in range(16)], 2, "b=16 int8, one layer")
        for replay in range(2):                # captured graphs, then their replay
            for b in range(16):
                h.reset_cache(b)
            again = h.step()
            for b in range(16):
                assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32)), "replay %d stream %d" % (replay, b)
        for b in (0, 7, 8, 15):
            h.reset_cache(b)
            solo = h.step([b])[0]
            assert np.array_equal(solo.view(np.uint32), first[b].view(np.uint32)), "stream %d differs from its solo run" % b
        for lanes in (1, 3):
            backend.set_step_lanes(lanes)
            for attempt in range(3):           # eager, capture, replay in this lane layout
                for b in range(16):
                    h.reset_cache(b)
                got = h.step()
                for b in range(16):
                    assert np.array_equal(got[b].view(np.uint32), first[b].view(np.uint32)), "%d lanes, attempt %d, stream %d" % (lanes, attempt, b)
    finally:
        backend.set_step_lanes(0)
        h.close()
        backend.set_quant(0)


@pytest.mark.parametrize("qtype_name", ["int8", "f32"])
def test_lanes_keep_every_bit(pkg, backend, synth, qtype_name):
    """A ragged batch of eight stepped in one, two and three lanes (groups of streams on HIP streams of their own, dealt by
    cache length): outputs and appended cache rows are the same bits in every layout, eagerly, at capture and on replay, and
    so is a batch of five that follows on the same decoder (other lane sizes, the lanes' graphs of those sizes)."""
    _announce("lanes keep every bit, %s" % qtype_name)
    lengths = [5, 640, 0, 129, 63, 2, 300, 65]
    mems = [7, 64, 3, 32, 65, 0, 27, 200]
    cfg = synth.decoder_config(layers=3, capacity=648)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=11)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        ref = {}
        for lanes in (1, 2, 3, 2):
            backend.set_step_lanes(lanes)
            for which in (list(range(8)), [6, 1, 3, 7, 0]):
                for attempt in range(3):
                    for b in which:
                        h.reset_cache(b)
                    got = h.step(which)
                    rows = [tuple(a[:, lengths[b]].copy() for a in h.cache_rows(b)) for b in which]
                    key = len(which)
                    if key not in ref:
                        ref[key] = (got, rows)
                        assert all(np.isfinite(o).all() for o in got)
                    for i, b in enumerate(which):
                        what = "%d lanes, batch %d, attempt %d, stream %d" % (lanes, key, attempt, b)
                        assert np.array_equal(got[i].view(np.uint32), ref[key][0][i].view(np.uint32)), what
                        assert np.array_equal(rows[i][0], ref[key][1][i][0]) and np.array_equal(rows[i][1], ref[key][1][i][1]), what + " (appended rows)"
        for i, b in enumerate([6, 1, 3, 7, 0]):   # and a stream's bits do not depend on the batch it is in
            assert np.array_equal(ref[5][0][i].view(np.uint32), ref[8][0][b].view(np.uint32))
    finally:
        backend.set_step_lanes(0)
        h.close()
        backend.set_quant(0)


def test_stage_enqueue_leaves_the_step_intact(pkg, backend, synth):
    """The per-stage timing entry replays single stages of the step; a full step afterwards gives the same bits as before."""
    _announce("stage enqueue")
    cfg = synth.decoder_config(layers=2, capacity=140)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [130, 17, 64], [20, 33, 1], seed=1)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    with pytest.raises(pkg.BackendError):            # needs one earlier step with this batch size
        h.dec.stage_enqueue(3, 0)
    first = h.step()
    for stage in range(6):
        for _ in range(2):
            h.dec.stage_enqueue(3, stage)
    backend.sync()
    with pytest.raises(pkg.BackendError):
        h.dec.stage_enqueue(3, 6)
    for b in range(3):
        h.reset_cache(b)
    again = h.step()
    for b in range(3):
        assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32))
    h.close()
    backend.set_quant(0)


def test_full_size_ragged_batch8_int8(pkg, backend, orc, synth, nerr):
    """The benchmark's batch-8 configuration at full size (12 layers, self KV up to 2048 rows, 12x64 cross heads, int8):
    four streams against the oracle, graph replay == eager, and EVERY stream bit-identical to the same stream alone."""
    _announce("12 layers int8 ragged b=8 full size")
    self_len, cross_len = synth.ragged_lengths(8, seed=3)
    lengths = [n - 1 for n in self_len]
    cfg = synth.decoder_config(layers=12, capacity=2048)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, cross_len, seed=1)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    first = h.step()
    assert all(np.all(np.isfinite(o)) for o in first)
    check = (1, 6, 3, 7)                                # the shortest and the longest stream, and two in between
    odec = orc.Decoder(cfg, weights, orc.INT8)
    errs = []
    for b in check:
        s = streams[b]
        want = odec.step([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [lengths[b]], [cross_len[b]], [s["x"]])[0]
        errs.append(nerr(first[b], want))
    quantised_errors_ok(errs, 3, "full size b=8 int8")     # 12 layers each: roughly one (stream, layer) in thirty meets a rounding boundary
    for b in range(8):
        h.reset_cache(b)
    again = h.step()                                    # captured graph
    for b in range(8):
        assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32)), "replay differs for stream %d" % b
    for b in range(8):
        h.reset_cache(b)
        solo = h.step([b])[0]
        assert np.array_equal(solo.view(np.uint32), first[b].view(np.uint32)), "stream %d differs from its solo run" % b
    h.close()
    backend.set_quant(0)


def test_full_size_batch16_int8(pkg, backend, orc, synth, nerr):
    """Sixteen streams of the 12-layer int8 stack at full size (self caches of 700 to 1023 rows, memories of 100 to 256 rows), stepped
    as two lanes of eight: three streams against the oracle, graph replay == eager, and four streams (both lanes, both ends
    of the length order) bit-identical to themselves alone."""
    _announce("12 layers int8 b=16 full size")
    rng = np.random.default_rng(160)
    lengths = [int(n) for n in rng.integers(700, 1024, size=16)]
    mems = [int(n) for n in rng.integers(100, 257, size=16)]
    lengths[5], mems[5] = 1023, 256
    cfg = synth.decoder_config(layers=12, capacity=1024)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=21)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        first = h.step()
        assert all(np.all(np.isfinite(o)) for o in first)
        odec = orc.Decoder(cfg, weights, orc.INT8)
        errs = []
        for b in (5, 0, 11):
            s = streams[b]
            want = odec.step([s["k"].copy()], [s["v"].copy()], [s["ck"]], [s["cv"]], [lengths[b]], [mems[b]], [s["x"]])[0]
            errs.append(nerr(first[b], want))
        quantised_errors_ok(errs, 2, "full size b=16 int8")
        for replay in range(2):
            for b in range(16):
                h.reset_cache(b)
            again = h.step()
            for b in range(16):
                assert np.array_equal(again[b].view(np.uint32), first[b].view(np.uint32)), "replay %d differs for stream %d" % (replay, b)
        order = sorted(range(16), key=lambda b: lengths[b] + mems[b])
        for b in (order[0], order[1], order[-1], order[-2]):
            h.reset_cache(b)
            solo = h.step([b])[0]
            assert np.array_equal(solo.view(np.uint32), first[b].view(np.uint32)), "stream %d differs from its solo run" % b
    finally:
        h.close()
        backend.set_quant(0)


def test_config2_int4_full_stack_with_head(pkg, backend, orc, synth, nerr):
    """The benchmark's int4 configuration at full size: 12 layers, int4 group-32 weights, batch 1, self KV 1024 rows, 256
    encoder states under 12 x 64 cross heads, LayerNorm gain and bias, final LayerNorm, then the 768 -> 8 x 1024 output
    projection and a softmax per head.  Hidden row, logits and probabilities against the oracle; the captured graph's
    replay against the eager step bit for bit."""
    _announce("config 2: 12 layers int4 b=1 kv=1024/256 + head")
    cfg = synth.decoder_config(layers=12, capacity=1025)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [1024], [256], seed=1)
    rng = np.random.default_rng(1102)
    head_w = backend.keep((rng.standard_normal((8192, 768)) * 0.02).astype(np.float32))
    backend.set_quant(pkg.INT4)
    h = Harness(pkg, backend, cfg, weights, streams)
    want, ks, vs = _oracle_step(orc, cfg, weights, streams, orc.INT4)
    first = h.step()
    assert np.isfinite(first[0]).all()
    quantised_errors_ok([nerr(first[0], want[0])], 1, "config 2 hidden row")
    gk, gv = h.cache_rows(0)
    quantised_errors_ok([nerr(gk[:, 1024], ks[0][:, 1024]), nerr(gv[:, 1024], vs[0][:, 1024])], 2, "config 2 appended rows")
    mask = np.ones(1025, bool)
    mask[1024] = False
    assert np.array_equal(gk[:, mask], streams[0]["k"][:, mask]) and np.array_equal(gv[:, mask], streams[0]["v"][:, mask])
    # the head on the device's own hidden row: checked against the oracle's head of that same row, so the head's bar is the
    # matvec's (1e-5) whatever the stack did before it
    dl, dp = backend.alloc(8192), backend.alloc(8192)
    backend.output_head([h.bufs[0]["out"].ptr], 768, head_w, None, 8192, 1024, [dl.ptr], [dp.ptr])
    logits, probs = orc.output_head(orc.PackedWeight(head_w, orc.INT4), first[0], 8, 1024)
    assert nerr(dl.read(), logits) < 1e-5
    got_probs = dp.read()
    assert nerr(got_probs, probs) < 1e-5
    assert np.allclose(got_probs.reshape(8, 1024).sum(-1), 1.0, atol=1e-5)
    for replay in range(3):                  # second call captures, the others replay
        h.reset_cache(0)
        again = h.step()
        assert np.array_equal(again[0].view(np.uint32), first[0].view(np.uint32)), "replay %d" % replay
    dl.free()
    dp.free()
    h.close()
    backend.set_quant(0)


def test_captured_step_survives_a_growing_backend_workspace(pkg, backend, synth):
    """A decoder whose cross head is not 64 wide runs the eight-kernel layer, whose attention partials are the decoder's own
    memory: after its graph has been captured, a second decoder with a far larger cache (which makes the backend replace
    its shared attention workspace) and a step of that one, the first decoder's graph still gives its first result."""
    _announce("captured graph vs workspace growth")
    cfg_a = synth.decoder_config(layers=2, capacity=70, cross_heads=1)
    weights_a = synth.decoder_weights(cfg_a, seed=0, ln_bias=False)
    streams_a = synth.decoder_streams(cfg_a, [66, 3], [9, 20], seed=1)
    a = Harness(pkg, backend, cfg_a, weights_a, streams_a)
    first = a.step()
    for b in range(2):
        a.reset_cache(b)
    second = a.step()                                  # captured here
    cfg_b = synth.decoder_config(layers=1, capacity=20000, cross_heads=1)
    weights_b = synth.decoder_weights(cfg_b, seed=3, ln_bias=False, position=False)
    streams_b = synth.decoder_streams(cfg_b, [19990], [40], seed=2)
    bh = Harness(pkg, backend, cfg_b, weights_b, streams_b)
    bh.step()
    for b in range(2):
        a.reset_cache(b)
    third = a.step()                                   # replay of the graph captured before the workspace moved
    for b in range(2):
        assert np.array_equal(second[b].view(np.uint32), first[b].view(np.uint32))
        assert np.array_equal(third[b].view(np.uint32), first[b].view(np.uint32)), "stream %d changed after the workspace grew" % b
    bh.close()
    a.close()


@pytest.mark.parametrize("qtype_name", ["int8", "f32", "int4"])
def test_many_stream_forms_agree(pkg, backend, synth, qtype_name):
    """Five ragged streams (one with an empty cache, one without encoder memory) stepped by the many-stream attention launches
    in each of their forms -- partials folded inside the launch (the default), by a fold kernel behind it, and with two or
    more cache chunks per workgroup -- give the same bits, outputs and appended cache rows, eagerly and as a captured graph."""
    import os
    _announce("many-stream forms agree, %s" % qtype_name)
    lengths, mems = [700, 0, 129, 383, 512], [40, 7, 0, 130, 129]
    cfg = synth.decoder_config(layers=3, capacity=800)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=5)
    backend.set_quant(QT[qtype_name])
    results = {}
    try:
        for name, env in (("default", {}), ("fold kernel", {"MYNAH_HIP_FOLD_IN_LAUNCH": "0"}), ("grouped to the device", {"MYNAH_HIP_ATTN_SLOTS": "device"}),
                          ("grouped into 100 slots", {"MYNAH_HIP_ATTN_SLOTS": "100"})):
            os.environ.update(env)
            try:
                h = Harness(pkg, backend, cfg, weights, streams)     # the decoder reads the switches when it is created
            finally:
                for k in env:
                    del os.environ[k]
            outs = []
            for _ in range(3):                                      # eager, capture, replay
                for b in range(len(lengths)):
                    h.reset_cache(b)
                outs.append(h.step())
            rows = [tuple(a[:, lengths[b]].copy() for a in h.cache_rows(b)) for b in range(len(lengths))]
            h.close()
            for b in range(len(lengths)):
                assert np.isfinite(outs[0][b]).all()
                for o in outs[1:]:
                    assert np.array_equal(o[b].view(np.uint32), outs[0][b].view(np.uint32)), "%s: replay differs, stream %d" % (name, b)
            results[name] = (outs[0], rows)
        ref_out, ref_rows = results["default"]
        for name, (out, rows) in results.items():
            for b in range(len(lengths)):
                assert np.array_equal(out[b].view(np.uint32), ref_out[b].view(np.uint32)), "%s differs from the default, stream %d" % (name, b)
                assert np.array_equal(rows[b][0], ref_rows[b][0]) and np.array_equal(rows[b][1], ref_rows[b][1]), "%s: appended rows differ" % name
    finally:
        backend.set_quant(0)


def test_long_cache_takes_the_fold_kernel(pkg, backend, orc, synth, nerr):
    """A capacity whose per-(stream, head) partial records exceed the LDS a launch may use without asking (more than
    about 19,000 rows): the many-stream step then folds in a kernel of its own.  Three streams, one of them 20,000 rows
    long, against the oracle and against each stream alone."""
    _announce("long cache: fold kernel form")
    lengths, mems = [20000, 5, 700], [33, 0, 129]
    cfg = synth.decoder_config(layers=1, capacity=20480)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=8)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        outs = h.step()
        want, _, _ = _oracle_step(orc, cfg, weights, streams, QT["int8"])
        quantised_errors_ok([nerr(outs[b], want[b]) for b in range(3)], 1, "long cache int8")
        for b in range(3):
            h.reset_cache(b)
        again = h.step()
        for b in range(3):
            assert np.array_equal(again[b].view(np.uint32), outs[b].view(np.uint32))
            h.reset_cache(b)
            solo = h.step([b])[0]
            assert np.array_equal(solo.view(np.uint32), outs[b].view(np.uint32)), "stream %d differs from its solo run" % b
    finally:
        h.close()
        backend.set_quant(0)


@pytest.mark.parametrize("qtype_name,batch", [("int8", 1), ("int8", 2), ("int8", 5), ("int8", 8), ("int4", 3), ("f32", 2), ("f16", 4), ("int8", 11)])
def test_step_and_head_in_one_call(pkg, backend, synth, nerr, qtype_name, batch):
    """mynah_hip_decoder_step_head against mynah_hip_decoder_step followed by mynah_hip_output_head on the same streams: the
    slots' outputs (the final-normed rows), the appended cache rows, logits and probabilities, all bit for bit -- the head
    product's LayerNorm prologue forms its sums as the end kernel does; eight steps in a row: eager, captured, replayed; the
    same three with other rows for the results (the head travels in the step's graph, whose nodes hold its pointers: one eager
    step, then captured again); and two with a head whose weight the library has not seen before (converted and uploaded in
    the eager step, outside any capture);
    eleven streams take the two-call form inside the library (two lanes)."""
    _announce("step + head in one call %s b=%d" % (qtype_name, batch))
    rng = np.random.default_rng(11)
    lengths = [int(v) for v in rng.integers(0, 290, batch)]
    mems = [int(v) for v in rng.integers(0, 200, batch)]
    cfg = synth.decoder_config(layers=2, capacity=304)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    first_w = (rng.standard_normal((2 * 256, cfg["width"])) * 0.02).astype(np.float32)
    first_b = (rng.standard_normal(2 * 256) * 0.1).astype(np.float32)
    backend.set_quant(QT[qtype_name])
    h = Harness(pkg, backend, cfg, weights, streams)
    later_w = (rng.standard_normal((2 * 256, cfg["width"])) * 0.02).astype(np.float32)
    later_b = (rng.standard_normal(2 * 256) * 0.1).astype(np.float32)
    first = [backend.alloc(512) for _ in range(2 * batch)]
    other = [backend.alloc(512) for _ in range(2 * batch)]
    for step in range(8):
        dl, dp = (other[:batch], other[batch:]) if 3 <= step < 6 else (first[:batch], first[batch:])
        head_w, head_b = (later_w, later_b) if step >= 6 else (first_w, first_b)
        def two_calls():
            for i in range(batch):
                h.reset_cache(i)
            rows = h.step()
            backend.output_head([b["out"].ptr for b in h.bufs], cfg["width"], head_w, head_b, 512, 256, [d.ptr for d in dl], [d.ptr for d in dp])
            return rows, [d.read() for d in dl], [d.read() for d in dp], [h.cache_rows(i) for i in range(batch)]

        def one_call():
            for i in range(batch):
                h.reset_cache(i)
                h.bufs[i]["out"].write(np.zeros(cfg["width"], np.float32))
                dl[i].write(np.zeros(512, np.float32))
                dp[i].write(np.zeros(512, np.float32))
            h.dec.step_head(h.slots(), head_w, head_b, 512, 256, [d.ptr for d in dl], [d.ptr for d in dp])
            return [b["out"].read() for b in h.bufs], [d.read() for d in dl], [d.read() for d in dp], [h.cache_rows(i) for i in range(batch)]

        if step == 6:   # the new head's first sight is the one-call form's
            got, want = one_call(), two_calls()
        else:
            want, got = two_calls(), one_call()
        for i in range(batch):
            assert np.array_equal(got[0][i].view(np.uint32), want[0][i].view(np.uint32)), "step %d stream %d: output row" % (step, i)
            assert np.array_equal(got[3][i][0], want[3][i][0]) and np.array_equal(got[3][i][1], want[3][i][1]), "step %d stream %d: cache" % (step, i)
            assert np.array_equal(got[1][i].view(np.uint32), want[1][i].view(np.uint32)), "step %d stream %d: logits" % (step, i)
            assert np.array_equal(got[2][i].view(np.uint32), want[2][i].view(np.uint32)), "step %d stream %d: probabilities" % (step, i)
    for d in first + other:
        d.free()
    h.close()
    backend.set_quant(0)
