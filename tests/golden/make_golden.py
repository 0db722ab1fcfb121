"""Writes tests/golden/reference_vectors.npz: inputs and outputs of the reference's own CPU code for the decode-step
path, produced by the reference compiled from its sources (oracle/_ref, both flag sets: "stock" = its Makefile's
-O3 -ffast-math build, "strict" = the source as written under IEEE rules).

    make -C oracle ref && python tests/golden/make_golden.py

The fixture is data only.  Small cases carry their inputs; the whole-step cases are seeded (the generators live in
mynah-tts_amd/synth.py) and carry a checksum of the generated inputs, so a drift of the generator is noticed rather
than misread as a parity failure.  tests/test_golden.py checks the oracle against this file wherever the compiled
reference itself is absent.
"""
import ctypes as C
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

STEP_LENGTHS = [5, 17, 0, 31, 9, 2, 25, 12]
STEP_MEMS = [7, 19, 3, 32, 11, 1, 27, 16]
STEP_LAYERS = 2
# streams without any encoder memory beside streams that have one (src/graph.c:3237-3244: their context stays zero)
NOMEM_LENGTHS = [3, 0, 12, 9]
NOMEM_MEMS = [0, 5, 0, 13]
ENC_CFG = {"layers": 2, "width": 768, "heads": 12, "head_width": 64, "ffn": 3072, "vocab": 300, "max_positions": 64,
           "causal": True}
ENC_KERNELS = (1, 3)
ENC_TOKENS = 19
ENC_SEED = 50


def crc(*arrays):
    c = 0
    for a in arrays:
        c = zlib.crc32(np.ascontiguousarray(a).tobytes(), c)
    return np.uint32(c)


def quant_inputs():
    """8 rows x 96: rounding ties at several magnitudes, an all-zero row, a denormal-scale row, a random row."""
    rng = np.random.default_rng(11)
    k = 96
    rows = []
    for amax in (127.0, 63.5, 7.0, 3.5, 1e-3):
        grid = (np.arange(k, dtype=np.float32) - np.float32(k // 2)) + np.float32(0.5)
        row = (grid * np.float32(amax / 127.0)).astype(np.float32)
        row[0] = amax
        rows.append(row)
    rows.append(np.zeros(k, np.float32))
    rows.append(np.full(k, 1e-30, np.float32))
    rows.append((rng.standard_normal(k) * 0.02).astype(np.float32))
    return np.stack(rows)


def step_case(orc, synth, out, prefix, lengths, mems, stream_seed, qnames):
    """Outputs and appended cache rows of the compiled reference's decoder_step_batch on seeded synthetic streams."""
    batch = len(lengths)
    cfg = synth.decoder_config(layers=STEP_LAYERS, capacity=max(lengths) + 3, cross_heads=1)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    streams = synth.decoder_streams(cfg, lengths, mems, seed=stream_seed)
    out[prefix + "_lengths"] = np.array(lengths, np.int64)
    out[prefix + "_mems"] = np.array(mems, np.int64)
    out[prefix + "_input_crc"] = crc(*[weights[k] for k in sorted(weights) if weights[k] is not None],
                                     *[s[n] for s in streams for n in ("k", "v", "ck", "cv", "x")])
    qtypes = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}
    for qname in qnames:
        for tag, strict in (("stock", False), ("strict", True)):
            dec = orc.RefDecoder(cfg, weights, qtypes[qname], batch, max(mems), strict=strict)
            ks = [s["k"].copy() for s in streams]
            vs = [s["v"].copy() for s in streams]
            outs, _ = dec.step(ks, vs, [s["ck"] for s in streams], [s["cv"] for s in streams], lengths, mems,
                               [s["x"] for s in streams])
            dec.close()
            out["%s_%s_%s_out" % (prefix, qname, tag)] = np.stack(outs)
            out["%s_%s_%s_newk" % (prefix, qname, tag)] = np.stack([ks[b][:, lengths[b]] for b in range(batch)])
            out["%s_%s_%s_newv" % (prefix, qname, tag)] = np.stack([vs[b][:, lengths[b]] for b in range(batch)])


def main():
    orc = entry.load_oracle()
    pkg = entry.load_package()     # only for the seeded generators in synth.py
    import mynah_tts_amd.synth as synth
    out = {}

    # ---- quantisers, activation quantisation, integer matvecs (src/qmat.c:39-115,117-383)
    w = quant_inputs()
    rng = np.random.default_rng(12)
    x = rng.standard_normal(96).astype(np.float32)
    x[3] = np.float32(2.5)      # makes a few exact ties after scaling by 127/amax
    bias = (rng.standard_normal(8) * 0.1).astype(np.float32)
    out["quant_w"], out["quant_x"], out["quant_bias"] = w, x, bias
    for tag, strict in (("stock", False), ("strict", True)):
        lib = orc.load_ref(strict=strict)
        n, k = w.shape
        q8 = np.empty((n, k), np.int8)
        s8 = np.empty(n, np.float32)
        lib.ref_quantize_weight_int8(w, n, k, q8, s8)
        q4 = np.empty((n, k // 2), np.uint8)
        s4 = np.empty((n, k // 32), np.float32)
        lib.ref_quantize_weight_int4(w, n, k, q4, s4)
        qx = np.empty(k, np.int8)
        sx = np.float32(lib.ref_quantize_act_int8(qx, x, k))
        y8 = np.empty(n, np.float32)
        lib.ref_matvec_q8(y8, qx, sx, q8, s8, bias.ctypes.data_as(C.c_void_p), n, k)
        y4 = np.empty(n, np.float32)
        lib.ref_matvec_q4(y4, qx, sx, q4, np.ascontiguousarray(s4), bias.ctypes.data_as(C.c_void_p), n, k)
        # activation quantisation of every weight row too (covers amax == 0 and tiny magnitudes)
        qrows = np.empty((n, k), np.int8)
        srows = np.empty(n, np.float32)
        for i in range(n):
            srows[i] = lib.ref_quantize_act_int8(qrows[i], w[i], k)
        for name, val in (("q8", q8), ("s8", s8), ("q4", q4), ("s4", s4), ("qx", qx), ("sx", sx), ("y8", y8), ("y4", y4),
                          ("qrows", qrows), ("srows", srows)):
            out["quant_%s_%s" % (tag, name)] = val

    # ---- LayerNorm / GELU / softmax (src/kernels.c:186-257,373-433), strict build = the scalar source
    lib = orc.load_ref(strict=True)
    rng = np.random.default_rng(13)
    v = rng.standard_normal((3, 64)).astype(np.float32) * np.float32(2.0)
    gain = (1.0 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(64)).astype(np.float32)
    ln = np.empty_like(v)
    lib.mynah_layernorm_f32(v, gain, beta.ctypes.data_as(C.c_void_p), ln, 3, 64, C.c_float(1e-5))
    g = v.copy().reshape(-1)
    lib.mynah_gelu_f32_scalar(g, g.size)
    sm = np.empty(64, np.float32)
    assert lib.mynah_softmax_f32(np.ascontiguousarray(v[0]), sm, 64) == 0
    out.update(kern_x=v, kern_gain=gain, kern_beta=beta, kern_layernorm=ln, kern_gelu=g.reshape(v.shape), kern_softmax=sm)

    # ---- the whole decode step (src/graph.c:3127-3284), 2 layers: a ragged batch of 8, and a batch of 4 in which two
    # streams have no encoder memory
    step_case(orc, synth, out, "step", STEP_LENGTHS, STEP_MEMS, 1, ("f32", "int8", "int4"))
    step_case(orc, synth, out, "nomem", NOMEM_LENGTHS, NOMEM_MEMS, 2, ("f32", "int8", "int4"))

    # ---- the text encoder's layer stack (transformer_stack, src/graph.c:634-711, as encode_text calls it): causal,
    # gain-only LayerNorm, plain FFN and the model's kernel-3 conv FFN, 19 tokens, 2 layers
    for kernel in ENC_KERNELS:
        cfg = dict(ENC_CFG, ffn_kernel=kernel)
        w = synth.encoder_weights_f16(cfg, seed=ENC_SEED + kernel, kernel=kernel)
        ids = np.random.default_rng(ENC_SEED).integers(0, cfg["vocab"], size=ENC_TOKENS).astype(np.int32)
        out["enc_k%d_input_crc" % kernel] = crc(ids, *[w[k] for k in sorted(w) if w[k] is not None])
        for tag, strict in (("stock", False), ("strict", True)):
            out["enc_k%d_%s_out" % (kernel, tag)] = orc.ref_transformer_stack(cfg, w, w["tok_table"][ids], kernel, strict=strict)

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
