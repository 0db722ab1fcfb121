"""Seeded sweeps of shapes the hand-picked cases do not name: the resident decode step (layers, capacity, with and without
cross attention, 1-8 streams, every storage type; lengths drawn from {0, 1, capacity - 1, anything} and memories from the chunk
edges) against the oracle, batched against solo bit for bit, the caches' untouched rows unchanged and a replay equal to the
first run; and the local frame (vocabularies from 96 to 8192 ids, 2-16 positions, 1-8 items, planted ties, an end-of-sequence
id that wins wherever it is allowed) with every token choice replayed on the CPU from the device's own masked logits; and the
codec's causal convolution at channel counts, lengths and tap counts between the named cases, with guard values around the output."""
import numpy as np
import pytest

import test_gpu_local as L
import test_gpu_step as S

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12])
def test_decode_step_shape_sweep(pkg, backend, orc, synth, nerr, seed):
    rng = np.random.default_rng(seed)
    for case in range(8):
        layers = int(rng.integers(1, 3))
        capacity = int(rng.choice([17, 64, 129, 257, 300, 513, 1025]))
        cross = bool(rng.integers(0, 4) > 0)
        batch = int(rng.integers(1, 9))
        qname = str(rng.choice(["f32", "int8", "int4", "f16"]))
        lengths = [int(rng.choice([0, 1, capacity - 1, int(rng.integers(0, capacity))])) for _ in range(batch)]
        # a memory is at most as long as the self cache's capacity (the step refuses longer ones)
        mems = [min(capacity, int(rng.choice([1, 2, 127, 128, 129, 256, int(rng.integers(1, 257))]))) for _ in range(batch)] if cross else [0] * batch
        what = "sweep %d/%d: layers %d capacity %d cross %s batch %d %s lengths %s mems %s" % (seed, case, layers, capacity, cross, batch, qname, lengths, mems)
        S._announce(what)
        cfg = synth.decoder_config(layers=layers, capacity=capacity) if cross else synth.decoder_config(layers=layers, capacity=capacity, cross_heads=0)
        weights = synth.decoder_weights(cfg, seed=seed * 100 + case)
        streams = synth.decoder_streams(cfg, lengths, mems, seed=seed * 100 + case + 50)
        backend.set_quant(S.QT[qname])
        h = S.Harness(pkg, backend, cfg, weights, streams)
        want, ks, vs = S._oracle_step(orc, cfg, weights, streams, S.QT[qname])
        got = h.step()
        errors = [nerr(got[b], want[b]) for b in range(batch)]
        quantised = qname in ("int8", "int4")
        if quantised:
            S.quantised_errors_ok(errors, max(1, (batch * layers) // 6), what)
        else:
            assert all(e < S.TOL[qname] for e in errors), (what, errors)
        for b in range(batch):
            gk, gv = h.cache_rows(b)
            mask = np.ones(capacity, bool)
            mask[lengths[b]] = False
            assert np.array_equal(gk[:, mask], streams[b]["k"][:, mask]) and np.array_equal(gv[:, mask], streams[b]["v"][:, mask]), what
            assert nerr(gk[:, lengths[b]], ks[b][:, lengths[b]]) < (S.OUTLIER if quantised else S.TOL[qname]), what
        pick = int(rng.integers(0, batch))
        h.reset_cache(pick)
        assert np.array_equal(h.step([pick])[0], got[pick]), what + ": stream %d alone" % pick
        for b in range(batch):
            h.reset_cache(b)
        again = h.step()
        assert all(np.array_equal(again[b], got[b]) for b in range(batch)), what + ": replay"
        h.close()
        backend.set_quant(0)


@pytest.mark.parametrize("seed", [21])
def test_local_frame_shape_sweep(pkg, backend, orc, synth, seed):
    rng = np.random.default_rng(seed)
    for case in range(10):
        V = int(rng.choice([96, 1000, 2048, 2049, 4100, 8192]))
        positions = int(rng.integers(2, 17))
        B = int(rng.integers(1, 9))
        cbc = int(rng.choice([1, 2, 4, 8]))
        codebook = int(rng.integers(V // 2, V - 2))
        eos = codebook + 1
        qname = str(rng.choice(["f32", "int8"]))
        items = [{"temperature": float(rng.choice([0.0, 0.3, 0.8, 1.0, 1.5])), "topk": int(rng.choice([1, 2, 7, 50, 64, 65, 200, 256])),
                  "rng_state": int(rng.integers(0, 2 ** 62)), "forbid_eos": bool(rng.integers(0, 2))} for _ in range(B)]
        ties = int(rng.choice([0, 0, 40, 70, 600]))
        what = "local sweep %d/%d: vocab %d positions %d items %d codebooks %d codebook size %d %s ties %d" % (seed, case, V, positions, B, cbc, codebook, qname, ties)
        L._announce(what)
        cfg, w, proj, bias, tables, r2 = L._setup(synth, 1, positions, V, seed=seed * 100 + case)
        if ties and ties + 10 < codebook:
            lo = int(rng.integers(8, codebook - ties))
            level = float(rng.choice([0.0, 25.0]))
            for s in range(positions):
                proj[s][lo:lo + ties] = proj[s][3]
                bias[s][lo:lo + ties] = bias[s][3] = level
        if rng.integers(0, 2):
            for s in range(positions):
                bias[s][eos] = 30.0
        backend.set_quant(L.QT[qname])
        loc = pkg.Local(backend, cfg, w, proj, bias, tables, codebook, eos, cbc)
        rows = [r2.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
        drows = [backend.alloc(cfg["width"]).write(r) for r in rows]
        dlogits = backend.alloc(B * positions * V)
        frame_items = [dict(it, row=d.ptr) for it, d in zip(items, drows)]
        got = loc.frame(frame_items, dlogits.ptr)
        L._replay_choices(orc, dlogits.read().reshape(B, positions, V), items, got, codebook, eos, cbc)
        again = loc.frame(frame_items, dlogits.ptr)
        assert np.array_equal(again["values"], got["values"]) and list(again["rng_state"]) == list(got["rng_state"]), what + ": replay"
        loc.destroy()
        for d in drows + [dlogits]:
            d.free()
        backend.set_quant(0)


@pytest.mark.parametrize("seed", [31])
def test_codec_conv_shape_sweep(backend, orc, nerr, seed):
    """Twenty seeded causal convolutions at shapes the named cases leave out -- channel counts that end inside a block of
    eight or a tile of 32, rows shorter than a tap's reach or ending one position into a tile, every tap count from 1 to 16
    within the reach limit of 128 positions -- against the oracle (1e-5 normalised: the matrix cores add in another order);
    the output buffer carries guard values on both sides, which must survive; and with 3, 7 or 11 taps three convolutions
    side by side in one launch give the bits of three launches."""
    import test_gpu_codec as K
    rng = np.random.default_rng(seed)
    guard = 256
    for case in range(20):
        in_ch = int(rng.choice([1, 7, 8, 9, 31, 33, 64, 108, int(rng.integers(1, 261))]))
        out_ch = int(rng.choice([1, 31, 32, 33, 63, 65, 108, int(rng.integers(1, 261))]))
        length = int(rng.choice([1, 2, 31, 33, 63, 64, 65, 127, 129, 255, 257, int(rng.integers(1, 1501))]))
        kernel = int(rng.choice([1, 2, 3, 3, 5, 7, 7, 11, 11, 16]))
        dilation = int(rng.choice([d for d in (1, 2, 3, 5, 8) if (kernel - 1) * d <= 128]))
        what = "conv sweep %d/%d: in %d out %d length %d kernel %d dilation %d" % (seed, case, in_ch, out_ch, length, kernel, dilation)
        K._announce(what)
        x = rng.standard_normal((in_ch, length)).astype(np.float32)
        w = (rng.standard_normal((out_ch, in_ch, kernel)) / np.sqrt(in_ch * kernel)).astype(np.float32)
        b = rng.standard_normal(out_ch).astype(np.float32)
        want = orc.conv1d_causal(x, w, b, dilation)
        din = backend.alloc(x.size).write(x)
        fence = np.full(guard, 12345.0, np.float32)
        padded = np.concatenate([fence, np.zeros(out_ch * length, np.float32), fence])
        dbuf = backend.alloc(padded.size).write(padded)
        backend.conv1d(din.ptr, dbuf.ptr + 4 * guard, in_ch, out_ch, length, kernel, dilation, w, b)
        back = dbuf.read()
        assert np.array_equal(back[:guard], fence) and np.array_equal(back[-guard:], fence), what + ": wrote outside its rows"
        single = back[guard:-guard].reshape(out_ch, length)
        e = nerr(single, want)
        assert e < 1e-5, (what, e)
        if kernel in (3, 7, 11):
            outs = [backend.alloc(out_ch * length) for _ in range(3)]
            weights = [w, (w * 0.5).astype(np.float32), (w[::-1] * 1.0).astype(np.float32).copy()]
            items = [{"din": din.ptr, "dout": o.ptr, "kernel": kernel, "dilation": dilation, "weight": wt, "bias": b} for o, wt in zip(outs, weights)]
            backend.conv1d_fused_batch(items, in_ch, out_ch, length)
            together = [o.read() for o in outs]
            for o, wt in zip(outs, weights):
                backend.conv1d_fused(din.ptr, o.ptr, in_ch, out_ch, length, kernel, dilation, wt, b)
            for got, o in zip(together, outs):
                assert np.array_equal(got.view(np.uint32), o.read().view(np.uint32)), what + ": side by side"
            assert np.array_equal(together[0].view(np.uint32), single.reshape(-1).view(np.uint32)), what + ": fused against the seam's conv1d"
            for o in outs:
                o.free()
        din.free()
        dbuf.free()
