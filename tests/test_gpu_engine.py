"""The reference's own engine code as the consumer of the library: decoder_run's resident single-row path
(src/graph.c:3368-3491) and local_step_device (src/graph.c:1106-1158), compiled from the reference's sources, call the
library through the reference's `struct mynah_backend` filled as a `MYNAH_ENABLE_HIP` block would fill it
(oracle/ref_shim_backend.c).  The same engine functions run on the reference's CPU backend beside it, on the same
seeded weights, caches and inputs, so the only thing that differs between the two sides is the backend.

Needs oracle/_ref (built from the reference tree where that is present; the built library travels with the tree)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

QT = {"f32": 0, "int8": 1, "int4": 2}
# f32: 1e-5 normalised (max|a-b| / max|b|).  Quantised storage: the packed weights are identical on both sides; a
# last-bit difference in a LayerNorm output can move one int8 activation by one step, which later layers amplify.
TOL = {"f32": 1e-5, "int8": 2e-2, "int4": 2e-2}


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


@pytest.fixture()
def quant_env():
    """The backend reads its storage type from MYNAH_QUANT when it is opened (same strings as src/qmat.c:571-576)."""
    saved = {k: os.environ.get(k) for k in ("MYNAH_QUANT", "MYNAH_QUANT_ARITH")}

    def choose(qname):
        os.environ.pop("MYNAH_QUANT_ARITH", None)
        if qname == "f32":
            os.environ.pop("MYNAH_QUANT", None)
        else:
            os.environ["MYNAH_QUANT"] = qname

    yield choose
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


def test_backend_struct_self_test(pkg, orc, ref_strict, synth, quant_env):
    """The library's self-test, reached through the function pointer the reference's open call receives."""
    _announce("engine: self-test through struct mynah_backend")
    quant_env("f32")
    cfg = synth.decoder_config(layers=1, capacity=8, cross_heads=1)
    w = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    dec = orc.RefDecoder(cfg, w, orc.F32, 1, 4, strict=True)
    dec.use_hip(pkg.LIB_PATH)
    dec.self_test()
    dec.close()


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
def test_decoder_run_resident_path(pkg, orc, ref_strict, synth, nerr, quant_env, qtype_name):
    """Three consecutive decoder_run calls per stream, two streams with their own caches: the reference engine on the
    library against the reference engine on its CPU backend (where a single row is decoder_step_batch with one slot,
    src/graph.c:3493-3506).  Checks the output rows, that the resident path was the one taken, and the rows the
    library appended to the device caches."""
    _announce("engine: decoder_run resident path, %s" % qtype_name)
    qtype = QT[qtype_name]
    tol = TOL[qtype_name]
    lengths, mems = [5, 17], [7, 19]
    steps = 3
    cfg = synth.decoder_config(layers=2, capacity=max(lengths) + steps + 1, cross_heads=1)
    w = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=5)
    rng = np.random.default_rng(6)
    xs = [[rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(steps)] for _ in streams]

    quant_env(qtype_name)
    cpu = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip.use_hip(pkg.LIB_PATH)
    try:
        for slot, s in enumerate(streams):
            ck, cv = s["k"].copy(), s["v"].copy()       # the CPU side appends into these
            hk, hv = s["k"].copy(), s["v"].copy()       # uploaded once by the engine, then left alone
            clen = hlen = s["length"]
            for t in range(steps):
                want, clen, cpu_resident = cpu.run_one(slot, ck, cv, s["ck"], s["cv"], clen, s["memory_length"], xs[slot][t])
                got, hlen, resident = hip.run_one(slot, hk, hv, s["ck"], s["cv"], hlen, s["memory_length"], xs[slot][t])
                assert not cpu_resident
                assert resident, "the engine fell back to its CPU path"
                assert hlen == clen == s["length"] + t + 1
                e = nerr(got, want)
                assert e < tol, "stream %d step %d: %.3g" % (slot, t, e)
                row = s["length"] + t
                for layer in range(cfg["layers"]):
                    dk, dv = hip.device_kv_row(slot, layer, row)
                    assert nerr(dk, ck[layer, row]) < tol and nerr(dv, cv[layer, row]) < tol
            # the engine's host copies were never written by the resident path
            assert np.array_equal(hk, s["k"]) and np.array_equal(hv, s["v"])
            # rows below the first appended one arrived on the device unchanged
            if s["length"]:
                dk, dv = hip.device_kv_row(slot, 1, s["length"] - 1)
                assert np.array_equal(dk, s["k"][1, s["length"] - 1]) and np.array_equal(dv, s["v"][1, s["length"] - 1])
    finally:
        hip.close()
        cpu.close()


@pytest.mark.parametrize("qtype_name", ["f32", "int8"])
def test_local_step_device(pkg, orc, ref_strict, synth, nerr, quant_env, qtype_name):
    """Four positions of the local transformer: the reference's local_step_device on the library against its
    local_step_batch on the CPU backend.  The engine passes the position row, a pointer into host weight memory, in a
    device-pointer argument of residual_inplace (src/graph.c:1118-1120); the library resolves it through its weight
    cache."""
    _announce("engine: local_step_device, %s" % qtype_name)
    qtype = QT[qtype_name]
    tol = {"f32": 1e-5, "int8": 5e-3}[qtype_name]
    cfg = synth.decoder_config(layers=2, cross_heads=0, capacity=17)
    w = synth.decoder_weights(cfg, seed=21, ln_bias=False)
    rng = np.random.default_rng(22)
    quant_env(qtype_name)
    cpu = orc.RefLocal(cfg, w, qtype, 1, strict=True)
    hip = orc.RefLocal(cfg, w, qtype, 1, strict=True)
    hip.use_hip(pkg.LIB_PATH)
    shape = (cfg["layers"], cfg["capacity"], cfg["width"])
    ck, cv = [np.zeros(shape, np.float32)], [np.zeros(shape, np.float32)]
    try:
        length = 0
        for pos in range(4):
            x = rng.standard_normal(cfg["width"]).astype(np.float32)
            want, _ = cpu.step(ck, cv, [pos], [x])
            got, length = hip.device_step(0, length, x)
            assert length == pos + 1
            e = nerr(got, want[0])
            assert e < tol, "position %d: %.3g" % (pos, e)
    finally:
        hip.close()
        cpu.close()


def test_codec_decode_resident(pkg, orc, ref_strict, nerr, quant_env, tmp_path):
    """The reference's decode_codec on a file of synthetic codec weights (every tensor at the codec's real shape): on
    the library it takes decode_codec_resident (src/graph.c:2508-2638: pre-conv, five stages of snake, grouped
    transposed conv and res_layer_device, post-conv, clip -- about 290 operator calls), on the CPU backend its own CPU
    sequence (im2col + sgemm convolutions).  Three raw frames -> 3072 samples.  Ninety-five convolutions in a row, each
    adding in a different order on the matrix cores than the CPU does: 1e-4 normalised on the clipped waveform."""
    _announce("engine: decode_codec resident, 3 raw frames")
    quant_env("f32")
    path = str(tmp_path / "codec.safetensors")
    orc.write_safetensors(path, orc.codec_weights(seed=11))
    codes = np.random.default_rng(1).integers(0, 2016, (8, 3)).astype(np.uint32)
    cpu = orc.RefCodecEngine(path, None, strict=True)
    hip = orc.RefCodecEngine(path, pkg.LIB_PATH, strict=True)
    try:
        want, cpu_resident = cpu.decode(codes)
        got, resident = hip.decode(codes)
        assert resident and not cpu_resident
        assert np.all(np.isfinite(got)) and np.abs(got).max() <= 1.0
        assert np.std(want) > 0.05, "degenerate waveform"
        e = nerr(got, want)
        assert e < 1e-4, "codec waveform: %.3g" % e
        again, _ = hip.decode(codes)          # weights now come from the library's device cache
        assert np.array_equal(again, got)
    finally:
        hip.close()
        cpu.close()
