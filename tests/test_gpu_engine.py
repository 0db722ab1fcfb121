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


@pytest.mark.parametrize("tokens,layers,kernel", [(37, 2, 1), (130, 1, 3), (256, 2, 3)])
def test_transformer_stack_on_the_library(pkg, orc, ref_strict, synth, nerr, tmp_path, tokens, layers, kernel):
    """The reference's own text-encoder stack (transformer_stack as encode_text calls it, src/graph.c:634-711, :738-740:
    causal attention, gain-only LayerNorm, plain or kernel-3 conv FFN) with the library as its backend against the same
    function on the CPU backend: every projection is a host-pointer `matmul` of `tokens` rows, QK^T and PV one `sgemm` each
    per head, the conv FFN two `sgemm` calls over the unfolded rows -- the seam's many-row products (f32 matrix cores from 24
    rows on, the scalar kernels below) as the unmodified engine drives them.  f32 on both sides: 1e-5 normalised."""
    _announce("engine: transformer_stack on the library, %d tokens, %d layers, kernel %d" % (tokens, layers, kernel))
    cfg = {"layers": layers, "width": 768, "heads": 12, "head_width": 64, "ffn": 3072, "vocab": 300, "max_positions": 256,
           "causal": True, "ffn_kernel": kernel}
    w = synth.encoder_weights_f16(cfg, seed=30 + kernel, kernel=kernel)
    ids = np.random.default_rng(6).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    states = w["tok_table"][ids]
    want = orc.ref_transformer_stack(cfg, w, states, kernel, strict=True, workdir=str(tmp_path))
    got = orc.ref_transformer_stack(cfg, w, states, kernel, strict=True, workdir=str(tmp_path), hip_library=pkg.LIB_PATH)
    assert np.isfinite(got).all()
    e = nerr(got, want)
    assert e < 1e-5, "%.3g" % e


@pytest.mark.parametrize("qtype_name", ["f32", "int8"])
def test_decoder_run_prefill_then_resident_steps(pkg, orc, ref_strict, synth, nerr, quant_env, qtype_name):
    """decoder_run with 24 rows at once -- the reference's context prefill (src/graph.c:3506-3654) -- on the library and
    on the CPU backend: with more than sixteen rows every projection is a host-pointer f32 product of 24 rows through the
    backend's `matmul`, and self-attention two `sgemm` calls per head (QK^T over the rows the cache already holds plus the
    new ones, then PV), so this is the seam's many-row side as the engine drives it.  Then two single-row calls per stream,
    which on the library upload the prefilled host caches once and continue resident."""
    _announce("engine: decoder_run prefill of 24 rows, then resident steps, %s" % qtype_name)
    qtype = QT[qtype_name]
    tol = TOL[qtype_name]
    lengths, mems = [0, 6], [9, 19]
    rows, steps = 24, 2
    cfg = synth.decoder_config(layers=2, capacity=max(lengths) + rows + steps + 1, cross_heads=1)
    w = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=7)
    rng = np.random.default_rng(8)
    prompts = [rng.standard_normal((rows, cfg["width"])).astype(np.float32) for _ in streams]
    xs = [[rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(steps)] for _ in streams]

    quant_env(qtype_name)
    cpu = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip.use_hip(pkg.LIB_PATH)
    try:
        for slot, s in enumerate(streams):
            ck, cv = s["k"].copy(), s["v"].copy()
            hk, hv = s["k"].copy(), s["v"].copy()
            want, clen = cpu.run_rows(slot, ck, cv, s["ck"], s["cv"], s["length"], s["memory_length"], prompts[slot])
            got, hlen = hip.run_rows(slot, hk, hv, s["ck"], s["cv"], s["length"], s["memory_length"], prompts[slot])
            assert hlen == clen == s["length"] + rows
            e = nerr(got, want)
            assert e < 1e-5, "stream %d prefill: %.3g" % (slot, e)   # f32 products on both sides whatever the weight storage
            new = slice(s["length"], s["length"] + rows)
            for layer in range(cfg["layers"]):
                assert nerr(hk[layer, new], ck[layer, new]) < 1e-5 and nerr(hv[layer, new], cv[layer, new]) < 1e-5
            assert np.array_equal(hk[:, :s["length"]], s["k"][:, :s["length"]])
            for t in range(steps):
                want, clen, _ = cpu.run_one(slot, ck, cv, s["ck"], s["cv"], clen, s["memory_length"], xs[slot][t])
                got, hlen, resident = hip.run_one(slot, hk, hv, s["ck"], s["cv"], hlen, s["memory_length"], xs[slot][t])
                assert resident, "the engine fell back to its CPU path"
                assert hlen == clen == s["length"] + rows + t + 1
                e = nerr(got, want)
                assert e < tol, "stream %d step %d after the prefill: %.3g" % (slot, t, e)
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


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
def test_integration_text_batched_decoder_step(pkg, orc, ref_strict, synth, nerr, quant_env, qtype_name):
    """The engine-side code that the integration notes quote for the batched step (oracle/integration_batched.inc), compiled against the
    reference's own decoder_cache: eight ragged streams, two consecutive steps through hip_decoder_step_batch on the
    library, against the reference's CPU decoder_step_batch on the same caches and inputs.  The device caches are the
    ones the reference's decoder_gpu_attention_init uploads; lengths advance as the reference's do; the rows the step
    appended are read back through the backend."""
    _announce("engine: integration text, batched decoder step, %s" % qtype_name)
    from tests.test_gpu_step import quantised_errors_ok
    qtype = QT[qtype_name]
    lengths = [5, 17, 0, 31, 9, 2, 25, 12]
    mems = [7, 19, 3, 32, 11, 1, 27, 16]
    steps = 2
    cfg = synth.decoder_config(layers=2, capacity=max(lengths) + steps + 1, cross_heads=1)
    w = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    rng = np.random.default_rng(9)
    xs = [[rng.standard_normal(cfg["width"]).astype(np.float32) for _ in streams] for _ in range(steps)]
    quant_env(qtype_name)
    cpu = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip = orc.RefDecoder(cfg, w, qtype, len(streams), max(mems), strict=True)
    hip.use_hip(pkg.LIB_PATH)
    try:
        ck, cv = [s["k"].copy() for s in streams], [s["v"].copy() for s in streams]
        hk, hv = [s["k"].copy() for s in streams], [s["v"].copy() for s in streams]
        clens, hlens = list(lengths), list(lengths)
        for t in range(steps):
            want, clens = cpu.step(ck, cv, [s["ck"] for s in streams], [s["cv"] for s in streams], clens, mems, xs[t])
            got, hlens = hip.hip_step_batch(pkg.LIB_PATH, hk, hv, [s["ck"] for s in streams], [s["cv"] for s in streams], hlens, mems, xs[t])
            assert hlens == clens == [n + t + 1 for n in lengths]
            errs = [nerr(got[b], want[b]) for b in range(len(streams))]
            if qtype_name == "f32":
                assert max(errs) < 1e-5, errs
            else:   # 16 (stream, layer) pairs per step; the second step inherits what the first one's rounding did
                quantised_errors_ok(errs, 2 + 2 * t, "integration text step %d %s" % (t, qtype_name))
            for b in (0, 2, 7):
                row = lengths[b] + t
                for layer in range(cfg["layers"]):
                    dk, dv = hip.device_kv_row(b, layer, row)
                    assert nerr(dk, ck[b][layer, row]) < TOL[qtype_name] and nerr(dv, cv[b][layer, row]) < TOL[qtype_name]
        for b in range(len(streams)):      # the host copies were uploaded once and never written
            assert np.array_equal(hk[b], streams[b]["k"]) and np.array_equal(hv[b], streams[b]["v"])
    finally:
        hip.close()
        cpu.close()


def test_integration_text_local_frame(pkg, orc, ref_strict, synth, quant_env):
    """The engine-side code that the integration notes quote for the local frame, compiled against the reference's own local_cache and
    local_batch_item: one frame of three items (greedy with rng_state == NULL, two sampling items, one of them with EOS
    forbidden) through hip_sample_local_frame_batch on the library, f32 weights, against the oracle's frame: the codes
    land where the reference's loop stores them (src/graph.c:1620-1628: codebook * code_stride + raw_offset + frame),
    the generators advance in place, EOS flags and frames agree."""
    _announce("engine: integration text, local frame")
    S, V, codebook, eos, cbc = 16, 96, 80, 83, 8
    cfg = synth.decoder_config(layers=2, capacity=S + 1, cross_heads=0)
    w = synth.decoder_weights(cfg, seed=41, ln_bias=False)
    w["norm_out_g"] = w["norm_out_b"] = None
    rng = np.random.default_rng(42)
    proj = [(rng.standard_normal((V, cfg["width"])) * 0.05).astype(np.float32) for _ in range(S)]
    bias = [(rng.standard_normal(V) * 0.1).astype(np.float32) for _ in range(S)]
    tables = [rng.standard_normal((V, cfg["width"])).astype(np.float32) for _ in range(S)]
    bias[6][eos] = 50.0                        # position 6 chooses EOS unless it is forbidden
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(3)]
    items = [
        {"row": rows[0], "temperature": 0.9, "topk": 40, "rng_state": None, "generated_raw_length": 10, "min_raw_length": 4},   # greedy
        {"row": rows[1], "temperature": 0.8, "topk": 50, "rng_state": 0x1234567, "generated_raw_length": 1, "min_raw_length": 4},  # EOS forbidden
        {"row": rows[2], "temperature": 1.1, "topk": 7, "rng_state": 99, "generated_raw_length": 4, "min_raw_length": 4},
    ]
    oracle_items = [{"temperature": it["temperature"], "topk": it["topk"] if it["rng_state"] is not None else 1,
                     "rng_state": it["rng_state"] or 0, "forbid_eos": it["generated_raw_length"] < it["min_raw_length"]} for it in items]
    quant_env("f32")
    hip = orc.RefLocal(cfg, w, orc.F32, 3, strict=True)
    hip.use_hip(pkg.LIB_PATH)
    try:
        code_stride, raw_offset = 11, 5
        codes, saw, eos_frame, states = hip.hip_frame(pkg.LIB_PATH, proj, bias, tables, V, codebook, eos, cbc, items, code_stride, raw_offset)
        stack = orc.Decoder(cfg, w, orc.F32)
        want = orc.LocalFrame(stack, [orc.PackedWeight(p, orc.F32) for p in proj], bias, tables, codebook, eos, cbc).frame(rows, oracle_items)
        for i in range(3):
            for s in range(S):
                assert codes[i, s % cbc, raw_offset + s // cbc] == want["stored"][i, s], "item %d position %d" % (i, s)
            untouched = np.ones(code_stride, bool)
            untouched[raw_offset:raw_offset + S // cbc] = False
            assert np.all(codes[i][:, untouched] == 0xffffffff), "codes outside the frame's columns were written"
            assert saw[i] == want["saw_eos"][i]
            assert eos_frame[i] == want["eos_frame"][i]
            if items[i]["rng_state"] is not None:
                assert states[i] == want["rng_state"][i], "generator of item %d" % i
        assert saw[0] == 1 and eos_frame[0] == 6 // cbc and saw[1] == 0
    finally:
        hip.close()
