"""The packed-weight file: converted weights written by one backend and taken by the next instead of converting again."""
import os
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from tests.test_gpu_step import Harness, QT   # noqa: E402


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _copy_weights(weights):
    return {k: (None if v is None else np.array(v, copy=True)) for k, v in weights.items()}   # same contents, new host addresses


@pytest.mark.parametrize("qtype_name", ["int8", "int4", "f16"])
def test_pack_round_trip(pkg, synth, tmp_path, qtype_name):
    """Export from one backend, import into a fresh one: every matrix of the decoder comes out of the file (none is
    converted), the step's outputs are the same bits, and with verification switched on the file's bytes equal a fresh
    conversion's.  A backend with the other quantiser arithmetic takes nothing from the file."""
    _announce("packed-weight file round trip, %s" % qtype_name)
    cfg = synth.decoder_config(layers=2, capacity=40)
    weights = synth.decoder_weights(cfg, seed=0)
    streams = synth.decoder_streams(cfg, [33, 7], [17, 5], seed=1)
    path = str(tmp_path / "weights.mynahqw")
    matrices = 2 * 6
    a = pkg.Backend(quant=QT[qtype_name])
    try:
        h = Harness(pkg, a, cfg, weights, streams)
        want = h.step()
        h.close()
        assert a.weights_export(path) == matrices
        assert a.weights_from_pack() == 0
    finally:
        a.close()
    assert os.path.getsize(path) > 0
    b = pkg.Backend(quant=QT[qtype_name])
    try:
        assert b.weights_import(path) == matrices
        t0 = time.perf_counter()
        h = Harness(pkg, b, cfg, _copy_weights(weights), streams)
        load_s = time.perf_counter() - t0
        assert b.weights_from_pack() == matrices, "a matrix was converted although the file holds it"
        got = h.step()
        for g, w in zip(got, want):
            assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
        h.close()
        print("[pack] %s: decoder created from the file in %.3f s" % (qtype_name, load_s), flush=True)
    finally:
        b.close()
    os.environ["MYNAH_HIP_PACK_VERIFY"] = "1"
    try:
        c = pkg.Backend(quant=QT[qtype_name])
    finally:
        del os.environ["MYNAH_HIP_PACK_VERIFY"]
    try:
        assert c.weights_import(path) == matrices
        h = Harness(pkg, c, cfg, _copy_weights(weights), streams)          # converts everything and compares with the file
        assert c.weights_from_pack() == matrices
        h.close()
    finally:
        c.close()
    if qtype_name != "f16":
        d = pkg.Backend(quant=QT[qtype_name], arith=pkg.ARITH_STOCK)       # the file was written with the other arithmetic
        try:
            assert d.weights_import(path) == matrices
            h = Harness(pkg, d, cfg, _copy_weights(weights), streams)
            assert d.weights_from_pack() == 0
            h.close()
        finally:
            d.close()


def test_pack_refuses_what_it_cannot_trust(pkg, synth, tmp_path):
    """A file that is not one, a file cut short, and -- under verification -- a file whose bytes are not what the tensor
    converts to: each is an error with a message, and a backend goes on converting by itself afterwards."""
    _announce("packed-weight file: damaged files")
    cfg = synth.decoder_config(layers=1, capacity=16, cross_heads=0)
    weights = synth.decoder_weights(cfg, seed=3)
    streams = synth.decoder_streams(cfg, [5], [0], seed=1)
    path = str(tmp_path / "weights.mynahqw")
    a = pkg.Backend(quant=pkg.INT8)
    try:
        h = Harness(pkg, a, cfg, weights, streams)
        want = h.step()
        h.close()
        assert a.weights_export(path) == 4
        junk = str(tmp_path / "junk")
        open(junk, "wb").write(b"not a packed-weight file at all")
        with pytest.raises(pkg.BackendError, match="not a packed-weight file"):
            a.weights_import(junk)
        blob = open(path, "rb").read()
        short = str(tmp_path / "short")
        open(short, "wb").write(blob[:len(blob) // 2])
        with pytest.raises(pkg.BackendError, match="ends inside an entry|damaged entry"):
            a.weights_import(short)
        with pytest.raises(pkg.BackendError, match="cannot open"):
            a.weights_import(str(tmp_path / "missing"))
    finally:
        a.close()
    flipped = bytearray(blob)
    flipped[len(flipped) // 2] ^= 0x55                     # somewhere inside a weight's values or scales
    bad = str(tmp_path / "flipped")
    open(bad, "wb").write(bytes(flipped))
    os.environ["MYNAH_HIP_PACK_VERIFY"] = "1"
    try:
        b = pkg.Backend(quant=pkg.INT8)
    finally:
        del os.environ["MYNAH_HIP_PACK_VERIFY"]
    try:
        assert b.weights_import(bad) == 4
        with pytest.raises(pkg.BackendError, match="does not hold what this tensor converts to"):
            Harness(pkg, b, cfg, _copy_weights(weights), streams)
    finally:
        b.close()
    c = pkg.Backend(quant=pkg.INT8)                        # no file: converts by itself, same bits
    try:
        h = Harness(pkg, c, cfg, _copy_weights(weights), streams)
        got = h.step()
        assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32))
        h.close()
    finally:
        c.close()
