"""GPU parity of the codec operators (mynah_hip_conv1d / _conv_transpose_dev / _snake_dev) against the oracle, through the
C ABI.  conv1d runs on the f32 matrix cores and adds in a different order than the CPU: 1e-5 normalised.  The transposed
conv adds in the reference's order: bit-exact.  snake: the device sine against libm's, 1e-6 normalised."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _announce(msg):
    print("[gpu-case] " + msg, flush=True)


def _run_conv1d(backend, x, w, b, dilation):
    in_ch, length = x.shape
    out_ch, _, kernel = w.shape
    din = backend.alloc(x.size).write(x)
    dout = backend.alloc(out_ch * length)
    backend.conv1d(din.ptr, dout.ptr, in_ch, out_ch, length, kernel, dilation, w, b)
    got = dout.read().reshape(out_ch, length)
    din.free()
    dout.free()
    return got


def test_known_answer(backend):
    """gpu/metal/backend_metal_ops.m:1026-1027,1099-1106: input 1 2 3, taps 1 2, no bias -> 2 5 8."""
    _announce("conv1d known answer")
    got = _run_conv1d(backend, np.array([[1, 2, 3]], np.float32), np.array([[[1, 2]]], np.float32), None, 1)
    assert got.tolist() == [[2.0, 5.0, 8.0]]


# (in, out, length, kernel, dilation): the codec's pre-conv, its residual convs at three stages (kernels 3/7/11, dilations
# 1/3/5), the post-conv, and shapes that end inside a tile or are shorter than a tap's reach
SHAPES = [(32, 864, 75, 7, 1), (432, 432, 600, 3, 1), (216, 216, 700, 7, 3), (108, 108, 1000, 11, 5), (54, 54, 3000, 11, 1),
          (27, 27, 5000, 7, 5), (27, 1, 9000, 3, 1), (5, 70, 33, 1, 1), (9, 33, 20, 11, 5), (8, 64, 128, 2, 1),
          (40, 48, 300, 16, 8), (64, 40, 257, 5, 2), (33, 65, 129, 4, 1), (128, 96, 64, 1, 1)]   # generic tap counts, the largest reach, odd edges


@pytest.mark.parametrize("shape", SHAPES)
def test_conv1d_against_oracle(backend, orc, nerr, shape):
    in_ch, out_ch, length, kernel, dilation = shape
    _announce("conv1d in=%d out=%d length=%d kernel=%d dilation=%d" % shape)
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((in_ch, length)).astype(np.float32)
    w = (rng.standard_normal((out_ch, in_ch, kernel)) / np.sqrt(in_ch * kernel)).astype(np.float32)
    b = rng.standard_normal(out_ch).astype(np.float32)
    got = _run_conv1d(backend, x, w, b, dilation)
    want = orc.conv1d_causal(x, w, b, dilation)
    assert nerr(got, want) < 1e-5
    got_nobias = _run_conv1d(backend, x, w, None, dilation)
    assert nerr(got_nobias, want - b[:, None]) < 1e-5


@pytest.mark.parametrize("shape", [(864, 432, 75, 8), (432, 216, 600, 8), (54, 27, 3000, 2), (8, 4, 5, 4), (12, 4, 7, 3)])
def test_conv_transpose_bit_exact(backend, orc, shape):
    in_ch, out_ch, length, stride = shape
    _announce("conv_transpose in=%d out=%d length=%d stride=%d" % shape)
    kernel = 2 * stride
    groups = out_ch if in_ch % out_ch == 0 and shape != (12, 4, 7, 3) else 2
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((in_ch, length)).astype(np.float32)
    w = rng.standard_normal((in_ch, out_ch // groups, kernel)).astype(np.float32)
    b = rng.standard_normal(out_ch).astype(np.float32)
    want = orc.conv_transpose_causal(x, w, b, stride, groups)
    din = backend.alloc(x.size).write(x)
    dout = backend.alloc(want.size)
    backend.conv_transpose_dev(din.ptr, dout.ptr, in_ch, out_ch, length, want.shape[1], kernel, stride, groups, w, b)
    got = dout.read().reshape(want.shape)
    assert np.array_equal(got, want)
    din.free()
    dout.free()


def test_snake(backend, orc, nerr):
    _announce("snake 432 x 600")
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((432, 600)) * 2).astype(np.float32)
    alpha = (np.abs(rng.standard_normal(216)) + 0.05).astype(np.float32)
    d = backend.alloc(x.size).write(x)
    backend.snake_dev(d.ptr, alpha, 432, 600, 216)
    got = d.read().reshape(x.shape)
    want = orc.snake(x, alpha, 216)
    assert nerr(got[:216], want[:216]) < 1e-6
    assert np.array_equal(got[216:], want[216:])
    d.free()


def test_res_block_chain(backend, orc, nerr):
    """snake -> conv -> snake -> conv -> residual add, as res_layer_device chains them (src/graph.c:2444-2491)."""
    _announce("residual block chain 108 x 800")
    rng = np.random.default_rng(10)
    C, L, K, D = 108, 800, 7, 3
    x = rng.standard_normal((C, L)).astype(np.float32)
    a1, a2 = [(np.abs(rng.standard_normal(C // 2)) + 0.1).astype(np.float32) for _ in range(2)]
    w1, w2 = [(rng.standard_normal((C, C, K)) / np.sqrt(C * K)).astype(np.float32) for _ in range(2)]
    b1, b2 = [rng.standard_normal(C).astype(np.float32) * np.float32(0.1) for _ in range(2)]
    cur = backend.alloc(x.size).write(x)
    act, res, br = backend.alloc(x.size), backend.alloc(x.size), backend.alloc(x.size)
    backend.copy_dev(act.ptr, cur.ptr, x.size)
    backend.snake_dev(act.ptr, a1, C, L, C // 2)
    backend.conv1d(act.ptr, res.ptr, C, C, L, K, D, w1, b1)
    backend.snake_dev(res.ptr, a2, C, L, C // 2)
    backend.conv1d(res.ptr, br.ptr, C, C, L, K, 1, w2, b2)
    backend.residual_inplace(cur.ptr, br.ptr, x.size)
    got = cur.read().reshape(C, L)
    want = x + orc.conv1d_causal(orc.snake(orc.conv1d_causal(orc.snake(x, a1, C // 2), w1, b1, D), a2, C // 2), w2, b2, 1)
    assert nerr(got, want) < 1e-5
    for d in (cur, act, res, br):
        d.free()


def test_error_paths(pkg, backend):
    _announce("codec error paths")
    d = backend.alloc(64)
    w = np.zeros((1, 1, 17), np.float32)
    with pytest.raises(pkg.BackendError, match="kernel above 16 taps"):
        backend.conv1d(d.ptr, d.ptr, 1, 1, 8, 17, 1, w)
    with pytest.raises(pkg.BackendError, match="invalid conv1d arguments"):
        backend.conv1d(d.ptr, d.ptr, 1, 1, 0, 3, 1, w)
    with pytest.raises(pkg.BackendError, match="invalid conv_transpose arguments"):
        backend.conv_transpose_dev(d.ptr, d.ptr, 3, 2, 4, 8, 4, 2, 2, w)
    with pytest.raises(pkg.BackendError, match="invalid snake arguments"):
        backend.snake_dev(d.ptr, np.ones(4, np.float32), 2, 8, 3)
    d.free()
