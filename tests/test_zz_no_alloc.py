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
