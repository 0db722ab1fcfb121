"""The allocation-free self-attention entry point against the ordinary one, through the C ABI.

mynah_hip_self_attention_dev_noalloc keeps its split-L partials in a fixed array inside the library instead of the
backend's growable workspace.  Every case runs two calls in a row on the shared array, the second with a smaller input,
and compares output row and caches with mynah_hip_self_attention_dev bit for bit (the same kernels run on both sides;
the bar for this f32 operator against the oracle is 1e-5, checked as well).
"""
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _case(backend, rng, heads, hw, L):
    width = heads * hw
    qkv = rng.standard_normal(3 * width).astype(np.float32)
    kc = np.zeros((L + 1, width), np.float32)
    vc = np.zeros((L + 1, width), np.float32)
    kc[:L - 1] = rng.standard_normal((L - 1, width))
    vc[:L - 1] = rng.standard_normal((L - 1, width))
    kc[L:] = 55.0      # a row beyond `valid`: ignored and left alone
    vc[L:] = -55.0
    return qkv, kc, vc


def _run(backend, call, qkv, kc, vc, heads, hw, L):
    width = heads * hw
    dq, dk, dv, do = backend.alloc(qkv.size).write(qkv), backend.alloc(kc.size).write(kc), backend.alloc(vc.size).write(vc), backend.alloc(width)
    call(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, 1.0 / math.sqrt(hw), do.ptr)
    out, k_after, v_after = do.read(), dk.read().reshape(kc.shape), dv.read().reshape(vc.shape)
    for d in (dq, dk, dv, do):
        d.free()
    return out, k_after, v_after


# (heads, head width, first length, second smaller length): the step's 12 x 64 heads over many chunks and then a single one;
# a head width the 64-wide kernel does not take (arrival counters in the fixed array); one wide head; an unaligned width
@pytest.mark.parametrize("heads,hw,first,second", [(12, 64, 1100, 70), (12, 64, 300, 1), (4, 128, 260, 40), (1, 768, 200, 65),
                                                   (3, 50, 150, 9)])
def test_noalloc_matches_the_allocating_entry_twice_in_a_row(backend, orc, nerr, heads, hw, first, second):
    _announce("no-alloc self attention heads=%d hw=%d L=%d then %d" % (heads, hw, first, second))
    rng = np.random.default_rng(4200 + heads * 7 + hw + first)
    for L in (first, second):
        qkv, kc, vc = _case(backend, rng, heads, hw, L)
        want_out, want_k, want_v = _run(backend, backend.self_attention_dev, qkv, kc, vc, heads, hw, L)
        got_out, got_k, got_v = _run(backend, backend.self_attention_dev_noalloc, qkv, kc, vc, heads, hw, L)
        assert np.array_equal(got_out.view(np.uint32), want_out.view(np.uint32)), "output row differs at L=%d" % L
        assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v), "caches differ at L=%d" % L
        ok, ov = kc.copy(), vc.copy()
        oracle = orc.self_attention(qkv, ok, ov, L - 1, heads * hw, L, heads, hw, 1.0 / math.sqrt(hw))
        assert nerr(got_out, oracle) < 1e-5
        assert np.array_equal(got_k, ok) and np.array_equal(got_v, ov)


def test_noalloc_refuses_what_does_not_fit(pkg, backend):
    _announce("no-alloc self attention beyond its workspace")
    heads, hw = 12, 64
    width = heads * hw
    L = 20500                                   # 12 * (321 + 1) * 68 floats > 2^18
    dq, dk, dv, do = backend.alloc(3 * width), backend.alloc(L * width), backend.alloc(L * width), backend.alloc(width)
    with pytest.raises(pkg.BackendError, match="allocation-free workspace"):
        backend.self_attention_dev_noalloc(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, 0.125, do.ptr)
    for d in (dq, dk, dv, do):
        d.free()


def test_noalloc_allocates_nothing(pkg):
    """What names the entry point: on a backend whose first attention call it is (no workspace, no counters, no chunk-count
    word exist yet), two calls leave the device's free memory exactly where it was, and a call of the allocating entry
    afterwards does take some (so the reading would have shown an allocation)."""
    _announce("no-alloc self attention: device memory before and after")
    fresh = pkg.Backend()
    try:
        heads, hw = 12, 64
        width = heads * hw
        rng = np.random.default_rng(4300)
        bufs = []
        for L in (1100, 70):
            qkv, kc, vc = _case(fresh, rng, heads, hw, L)
            bufs.append((L, fresh.alloc(qkv.size).write(qkv), fresh.alloc(kc.size).write(kc), fresh.alloc(vc.size).write(vc), fresh.alloc(width)))
        fresh.sync()
        before = fresh.device_memory()[0]
        for L, dq, dk, dv, do in bufs:
            fresh.self_attention_dev_noalloc(dq.ptr, dk.ptr, dv.ptr, L - 1, width, L, heads, hw, 1.0 / math.sqrt(hw), do.ptr)
        fresh.sync()
        after = fresh.device_memory()[0]
        assert after == before, "the allocation-free entry point changed the device's free memory by %d bytes" % (before - after)
        L, dq, dk, dv, do = bufs[0]
        dbig = [fresh.alloc(32 << 20) for _ in range(2)]      # an allocation of a size the reading cannot miss
        assert fresh.device_memory()[0] < after
        for d in dbig:
            d.free()
        for L, dq, dk, dv, do in bufs:
            for d in (dq, dk, dv, do):
                d.free()
    finally:
        fresh.close()
