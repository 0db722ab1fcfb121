"""The resident decode step as one persistent launch (graph mode 2, opt-in) against the same step as a captured graph (mode 1,
the default) and
as separate launches (mode 0), through the C ABI: the three forms must give the same bits -- outputs and appended cache rows --
for int8 and int4 weights, one and two streams.  Also: the persistent form against the oracle, several steps in a row, streams
it hands back to the launched form (too many attention units, more than two streams), and the bounded wait: with a spin limit
of zero every wait gives up at once, all workgroups leave, and the next synchronisation reports it.
"""
import os

import numpy as np
import pytest

from tests.test_gpu_step import Harness, QT, _oracle_step, quantised_errors_ok

pytestmark = pytest.mark.gpu


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _run_mode(h, backend, mode, which=None):
    backend.set_graph_mode(mode)
    for b in range(len(h.streams)):
        h.reset_cache(b)
    outs = []
    for _ in range(3 if mode == 1 else 2):          # the graph form captures at its second call: take the replay
        for b in range(len(h.streams)):
            h.reset_cache(b)
        outs = h.step(which)
    which = range(len(h.streams)) if which is None else which
    rows = []
    for i in which:
        gk, gv = h.cache_rows(i)
        L = h.streams[i]["length"]
        rows.append((gk[:, L].copy(), gv[:, L].copy(), gk, gv))
    return outs, rows


def _same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint32), np.ascontiguousarray(b).view(np.uint32))


CASES = [
    # layers, capacity, cross heads, lengths, memory lengths
    (2, 300, 12, [129], [40]),
    (2, 300, 12, [0], [1]),                 # empty cache: the new row is the only unit
    (2, 300, 12, [128, 299], [0, 130]),     # a full unit beside the cache's last row; a stream without encoder memory
    (2, 140, 0, [63, 130], [0, 0]),         # a stack without cross attention
    (12, 1025, 12, [1024], [256]),          # the benchmark's batch-1 line
    (12, 1025, 12, [1000, 517], [256, 33]),   # too many attention units to sit beside the row stages: runs as the graph under mode 2
    (12, 520, 12, [400, 300], [256, 33]),     # two streams that fit
]


@pytest.mark.parametrize("qname", ["int8", "int4"])
@pytest.mark.parametrize("layers,capacity,cross_heads,lengths,mems", CASES)
def test_persistent_equals_graph_equals_launches(pkg, backend, orc, synth, nerr, qname, layers, capacity, cross_heads, lengths, mems):
    _announce("persistent step %s layers=%d lengths=%s mems=%s cross_heads=%d" % (qname, layers, lengths, mems, cross_heads))
    cfg = synth.decoder_config(layers=layers, capacity=capacity, cross_heads=cross_heads)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    backend.set_quant(QT[qname])
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        eager, eager_rows = _run_mode(h, backend, 0)
        graph, graph_rows = _run_mode(h, backend, 1)
        persistent, persistent_rows = _run_mode(h, backend, 2)
        for b in range(len(lengths)):
            assert np.isfinite(persistent[b]).all()
            assert _same_bits(graph[b], eager[b]), "graph differs from launches, stream %d" % b
            assert _same_bits(persistent[b], eager[b]), "persistent differs from launches, stream %d" % b
            assert _same_bits(persistent_rows[b][0], eager_rows[b][0]) and _same_bits(persistent_rows[b][1], eager_rows[b][1]), \
                "appended cache rows differ, stream %d" % b
            mask = np.ones(capacity, bool)
            mask[lengths[b]] = False
            assert np.array_equal(persistent_rows[b][2][:, mask], streams[b]["k"][:, mask]), "a cache row that is not the appended one changed"
            assert np.array_equal(persistent_rows[b][3][:, mask], streams[b]["v"][:, mask])
        if layers <= 2:
            want, _, _ = _oracle_step(orc, cfg, weights, streams, QT[qname])
            quantised_errors_ok([nerr(persistent[b], want[b]) for b in range(len(lengths))], 1, "persistent vs oracle " + qname)
        # each stream alone: same bits as inside the pair
        if len(lengths) == 2:
            for b in range(2):
                h.reset_cache(b)
                solo = h.step([b])[0]
                assert _same_bits(solo, persistent[b]), "stream %d differs from its solo run" % b
    finally:
        backend.set_graph_mode(1)
        h.close()
        backend.set_quant(0)


def test_persistent_steps_in_a_row(pkg, backend, orc, synth, nerr):
    """Five consecutive steps of two streams (each attends over the rows the earlier ones appended; the tags move on every
    step) in the persistent form, against the same five steps as launches."""
    _announce("persistent step: five steps in a row")
    cfg = synth.decoder_config(layers=3, capacity=140)
    weights = synth.decoder_weights(cfg, seed=0)
    lengths = [126, 5]
    streams = synth.decoder_streams(cfg, lengths, [30, 128], seed=7)
    backend.set_quant(1)
    h = Harness(pkg, backend, cfg, weights, streams)
    try:
        results = {}
        for mode in (0, 2):
            backend.set_graph_mode(mode)
            for b in range(2):
                h.reset_cache(b)
                streams[b]["length"] = lengths[b]
            outs = []
            for step in range(5):
                outs.append(h.step())
                for b in range(2):
                    streams[b]["length"] += 1
            results[mode] = (outs, [h.cache_rows(b) for b in range(2)])
        for step in range(5):
            for b in range(2):
                assert _same_bits(results[2][0][step][b], results[0][0][step][b]), "step %d stream %d" % (step, b)
        for b in range(2):
            assert np.array_equal(results[2][1][b][0], results[0][1][b][0]) and np.array_equal(results[2][1][b][1], results[0][1][b][1])
    finally:
        for b in range(2):
            streams[b]["length"] = lengths[b]
        backend.set_graph_mode(1)
        h.close()
        backend.set_quant(0)


def test_persistent_hands_back_what_it_does_not_take(pkg, backend, synth):
    """Three streams, f32 weights, and a cache so long that its attention units outnumber the compute units all run as
    launched kernels under graph mode 2, with the bits of mode 1."""
    _announce("persistent step: shapes it does not take")
    for qt, lengths, mems, capacity in ((1, [10, 20, 30], [5, 6, 7], 40), (0, [33], [9], 40), (1, [3000], [40], 3002)):
        cfg = synth.decoder_config(layers=1, capacity=capacity)
        weights = synth.decoder_weights(cfg, seed=0)
        streams = synth.decoder_streams(cfg, lengths, mems, seed=3)
        backend.set_quant(qt)
        h = Harness(pkg, backend, cfg, weights, streams)
        try:
            graph, _ = _run_mode(h, backend, 1)
            persistent, _ = _run_mode(h, backend, 2)
            for b in range(len(lengths)):
                assert _same_bits(persistent[b], graph[b])
        finally:
            backend.set_graph_mode(1)
            h.close()
            backend.set_quant(0)


def test_bounded_waits_fall_back_instead_of_hanging(pkg, backend, synth):
    """A backend opened with a spin limit of zero: every wait between workgroups gives up at its first look when what it
    waits for is not there yet, the kernel drains, and the synchronisation after the step repeats the step in the form
    without such waits -- the caller gets the bits of the normal run and a counter says how often that happened.  Two steps
    without a synchronisation in between cannot be repeated (the first one's inputs may be gone): that is the error."""
    _announce("bounded waits: fallback")
    os.environ["MYNAH_HIP_PERSIST_SPIN"] = "0"
    try:
        b2 = pkg.Backend(quant=pkg.INT8)
    finally:
        del os.environ["MYNAH_HIP_PERSIST_SPIN"]
    backend.set_quant(pkg.INT8)
    try:
        # the persistent launch: its second stage cannot find the first stage's partials at its first look
        cfg = synth.decoder_config(layers=2, capacity=200)
        weights = synth.decoder_weights(cfg, seed=0)
        streams = synth.decoder_streams(cfg, [150], [20], seed=1)
        ref_h = Harness(pkg, backend, cfg, weights, streams)
        want = ref_h.step()
        want_rows = ref_h.cache_rows(0)
        ref_h.close()
        h = Harness(pkg, b2, cfg, weights, streams)
        b2.set_graph_mode(2)
        assert b2.wait_fallbacks() == 0
        got = h.step()                      # the read of the output row synchronises
        assert b2.wait_fallbacks() == 1, "a persistent step with a spin limit of zero must have given up a wait"
        assert _same_bits(got[0], want[0])
        rows = h.cache_rows(0)
        assert np.array_equal(rows[0], want_rows[0]) and np.array_equal(rows[1], want_rows[1])
        h.reset_cache(0)
        h.dec.step(h.slots())               # two steps, no synchronisation between them
        h.dec.step(h.slots())
        with pytest.raises(pkg.BackendError, match="bounded wait"):
            b2.sync()
        b2.set_graph_mode(1)
        h.reset_cache(0)
        again = h.step()
        assert _same_bits(again[0], want[0])
        h.close()
        # the same bound holds the fold workgroups of the many-stream attention launches: eight long streams make more
        # workgroups than the device holds at once, so folds usually start while cache chunks are still being read and give
        # up at their first look; whether or not one did, the step's results are those of the normal run
        cfg = synth.decoder_config(layers=1, capacity=2048)
        weights = synth.decoder_weights(cfg, seed=0)
        streams = synth.decoder_streams(cfg, [2000, 1990, 1980, 1970, 1960, 1950, 1940, 1930], [16] * 8, seed=2)
        ref_h = Harness(pkg, backend, cfg, weights, streams)
        want = ref_h.step()
        ref_h.close()
        h = Harness(pkg, b2, cfg, weights, streams)
        before = b2.wait_fallbacks()
        for attempt in range(3):            # eager, capture, replay
            for b in range(8):
                h.reset_cache(b)
            got = h.step()
            for b in range(8):
                assert _same_bits(got[b], want[b]), "attempt %d stream %d" % (attempt, b)
        print("[fallback] many-stream steps repeated: %d of 3" % (b2.wait_fallbacks() - before), flush=True)
        h.close()
    finally:
        backend.set_quant(0)
        b2.close()


def test_spin_limit_must_be_a_number(pkg):
    os.environ["MYNAH_HIP_PERSIST_SPIN"] = "lots"
    try:
        with pytest.raises(pkg.BackendError, match="MYNAH_HIP_PERSIST_SPIN"):
            pkg.Backend(quant=pkg.INT8)
    finally:
        del os.environ["MYNAH_HIP_PERSIST_SPIN"]
