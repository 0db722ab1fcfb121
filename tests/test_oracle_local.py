"""Pins the oracle's local-transformer frame (src/graph.c:1234-1343 local step, :1374-1656 frame loop).

The step is pinned against the compiled reference's own local_step_batch.  The token choice (constraint mask, first-max
argmax, top-k insertion, temperature softmax, xorshift64 draw, cumulative pick) is pinned by what fixes it without the
reference: a numpy uint64 xorshift, a stable descending sort, float32 sequential sums, and brute-force cases on tiny
inputs with ties.
"""
import numpy as np
import pytest


def _local_cfg(synth, layers=1):
    return synth.decoder_config(layers=layers, capacity=17, cross_heads=0)


@pytest.mark.parametrize("qtype_name", ["f32", "int8", "int4"])
@pytest.mark.parametrize("strict", [True, False])
def test_local_step_matches_reference(orc, ref, ref_strict, synth, nerr, qtype_name, strict):
    """Three consecutive positions of a batch of three: the oracle's step without cross attention and final norm is the
    reference's local_step_batch."""
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}[qtype_name]
    cfg = _local_cfg(synth, layers=2)
    w = synth.decoder_weights(cfg, seed=21, ln_bias=False)
    w["norm_out_g"] = w["norm_out_b"] = None
    B = 3
    rng = np.random.default_rng(22)
    odec = orc.Decoder(cfg, w, qtype, orc.STRICT if strict else orc.STOCK)
    rdec = orc.RefLocal(cfg, w, qtype, B, strict=strict)
    shape = (cfg["layers"], cfg["capacity"], cfg["width"])
    ok, ov = [np.zeros(shape, np.float32) for _ in range(B)], [np.zeros(shape, np.float32) for _ in range(B)]
    rk, rv = [np.zeros(shape, np.float32) for _ in range(B)], [np.zeros(shape, np.float32) for _ in range(B)]
    # f32: 1e-5.  Quantised: identical packed weights on both sides; a last-bit LayerNorm difference can flip one int8
    # activation by one step, which moves an output by ~1/127 of a weight row's reach (more visible with int4 weights).
    tol = {orc.F32: 1e-5, orc.INT8: 5e-3, orc.INT4: 2e-2}[qtype]
    for pos in range(3):
        xs = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(B)]
        none = [np.zeros((cfg["layers"], 0, 1), np.float32)] * B
        want, new_len = rdec.step(rk, rv, [pos] * B, xs)
        got = odec.step(ok, ov, none, none, [pos] * B, [0] * B, xs)
        assert new_len == [pos + 1] * B
        for b in range(B):
            assert nerr(got[b], want[b]) < tol, "position %d stream %d" % (pos, b)
            for layer in range(cfg["layers"]):
                assert nerr(ok[b][layer, pos], rk[b][layer, pos]) < tol
                assert nerr(ov[b][layer, pos], rv[b][layer, pos]) < tol
    rdec.close()


def _xorshift(state):
    s = np.uint64(state)
    s ^= s << np.uint64(13)
    s ^= s >> np.uint64(7)
    s ^= s << np.uint64(17)
    return int(s) if int(s) != 0 else 0x9E3779B97F4A7C15


def _choose_numpy(logits, codebook_size, eos_id, temperature, topk, rng_state, forbid_eos):
    """Independent restatement: stable sort instead of the insertion loop, float32 sequential sums."""
    lg = np.array(logits, np.float32)
    V = lg.size
    allowed = np.arange(V) < codebook_size
    if not forbid_eos and eos_id < V:
        allowed[eos_id] = True
    lg[~allowed] = -np.finfo(np.float32).max
    masked = np.where(allowed, lg, -np.inf)
    greedy = int(np.argmax(masked)) if np.any(np.where(allowed, lg, -np.inf) > -np.finfo(np.float32).max) else 0
    if not (temperature > 0 and topk > 1):
        return greedy, greedy, rng_state
    k = min(topk, V)
    order = np.argsort(-lg.astype(np.float64), kind="stable")[:k]      # descending, earlier index first among equals
    top = lg[order]
    with np.errstate(over="ignore"):      # (-FLT_MAX - max) / T overflows to -inf, exp gives 0: the same in C
        p = np.exp(((top - top[0]) / np.float32(temperature)).astype(np.float32)).astype(np.float32)
    total = np.float32(0)
    for q in p:
        total = np.float32(total + q)
    state = _xorshift(rng_state)
    draw = np.float32(np.float32((state >> 40) & 0xFFFFFF) / np.float32(16777216.0)) * total
    cum = np.float32(0)
    value = int(order[-1])
    for q in range(k):
        cum = np.float32(cum + p[q])
        if draw <= cum or q + 1 == k:
            value = int(order[q])
            break
    return value, greedy, state


def test_xorshift_and_draw_sequence(orc):
    """The generator alone: 1000 steps against numpy uint64 arithmetic (sampling over two equal logits exposes the state)."""
    state = 0x1234567
    for _ in range(1000):
        _, _, new_state, _ = orc.local_choose([0.0, 0.0], 2, 9, 1.0, 2, state, True)
        assert new_state == _xorshift(state)
        state = new_state
    assert orc.local_choose([0.0, 0.0], 2, 9, 1.0, 2, 0, True)[2] == 0x9E3779B97F4A7C15     # the all-zero state is replaced


def test_constraint_mask_and_first_max(orc):
    lg = [1.0, 3.0, 3.0, 2.0, 9.0, 8.0]                       # codes 0..3, EOS = 4, 5 is another special token
    v, g, _, masked = orc.local_choose(lg, 4, 4, 0.0, 1, 7, False)
    assert (v, g) == (4, 4) and masked[5] == -np.finfo(np.float32).max and masked[4] == 9.0
    v, g, _, masked = orc.local_choose(lg, 4, 4, 0.0, 1, 7, True)     # EOS forbidden: first of the two equal maxima
    assert (v, g) == (1, 1) and masked[4] == -np.finfo(np.float32).max
    v, g, state, _ = orc.local_choose(lg, 4, 4, 0.7, 1, 7, False)     # topk 1 is greedy and leaves the generator alone
    assert (v, g, state) == (4, 4, 7)


@pytest.mark.parametrize("seed", range(6))
def test_sampling_matches_independent_restatement(orc, seed):
    rng = np.random.default_rng(100 + seed)
    V, codebook, eos = 2024, 2016, 2017
    state = int(rng.integers(1, 2 ** 62))
    for trial in range(40):
        lg = (rng.standard_normal(V) * 3).astype(np.float32)
        if trial % 5 == 0:
            lg[rng.integers(0, codebook, 40)] = lg[3]                 # ties among the candidates
        topk = int(rng.choice([2, 5, 80, 300, 5000]))
        temperature = float(rng.choice([0.3, 0.7, 1.0, 1.5]))
        forbid = bool(trial % 2)
        want = _choose_numpy(lg, codebook, eos, temperature, topk, state, forbid)
        got = orc.local_choose(lg, codebook, eos, temperature, topk, state, forbid)
        assert got[:3] == want, "trial %d" % trial
        state = got[2]


def test_brute_force_distribution_tiny(orc):
    """Three candidates, temperature 1, top-3: over many draws the frequencies follow softmax (sanity of the draw mapping)."""
    lg = np.array([0.0, 1.0, 2.0], np.float32)
    p = np.exp(lg - lg.max())
    p /= p.sum()
    state, counts = 99, np.zeros(3)
    for _ in range(20000):
        v, _, state, _ = orc.local_choose(lg, 3, 7, 1.0, 3, state, True)
        counts[v] += 1
    assert np.abs(counts / counts.sum() - p).max() < 0.01


def test_local_frame_bookkeeping(orc, synth):
    """A whole frame on a tiny vocabulary: greedy items are reproducible, tokens are fed back through the audio tables,
    EOS is seen when greedy or sampled value is EOS, special tokens are stored as 0."""
    cfg = _local_cfg(synth)
    w = synth.decoder_weights(cfg, seed=31, ln_bias=False)
    w["norm_out_g"] = w["norm_out_b"] = None
    stack = orc.Decoder(cfg, w, orc.F32)
    rng = np.random.default_rng(32)
    S, V, codebook, eos, cbc = 16, 40, 32, 33, 8
    proj = [orc.PackedWeight((rng.standard_normal((V, cfg["width"])) * 0.05).astype(np.float32), orc.F32) for _ in range(S)]
    bias = [(rng.standard_normal(V) * 0.1).astype(np.float32) for _ in range(S)]
    for s in (5, 11):
        bias[s][eos] = 50.0                                                  # force EOS at streams 5 and 11
    tables = [rng.standard_normal((V, cfg["width"])).astype(np.float32) for _ in range(S)]
    frame = orc.LocalFrame(stack, proj, bias, tables, codebook, eos, cbc)
    rows = [rng.standard_normal(cfg["width"]).astype(np.float32) for _ in range(2)]
    items = [{"temperature": 0.0, "topk": 1, "rng_state": 5, "forbid_eos": False},
             {"temperature": 0.0, "topk": 1, "rng_state": 6, "forbid_eos": True}]
    out = frame.frame(rows, items, want_logits=True)
    again = frame.frame(rows, items)
    assert np.array_equal(out["values"], again["values"])
    assert out["values"][0, 5] == eos and out["stored"][0, 5] == 0 and out["saw_eos"][0] == 1 and out["eos_frame"][0] == 5 // cbc
    assert out["saw_eos"][1] == 0 and out["eos_frame"][1] == np.iinfo(np.uint64).max and np.all(out["values"][1] < codebook)
    assert out["rng_state"] == [5, 6]                                        # greedy items never touch the generator
    # stream s + 1 really consumed the embedding of stream s's token: recompute stream 1 of item 0 by hand
    lg0 = out["logits"][0, 0]
    assert out["values"][0, 0] == int(np.argmax(lg0))
