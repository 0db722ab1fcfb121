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


def _res_layer_inputs(C, L, seed):
    rng = np.random.default_rng(seed)
    alpha = lambda: (np.abs(rng.standard_normal(C // 2)) + 0.1).astype(np.float32)
    conv = lambda k: ((rng.standard_normal((C, C, k)) / np.sqrt(C * k)).astype(np.float32), rng.standard_normal(C).astype(np.float32) * np.float32(0.1))
    blocks = [[(alpha(), conv(k), alpha(), conv(k), d) for d in (1, 3, 5)] for k in (3, 7, 11)]
    return rng.standard_normal((C, L)).astype(np.float32), blocks


# channels x length: the 64 x 128 tiles, the channel-split small tiles in both widths, at most 32 output channels, ragged edges
@pytest.mark.parametrize("C,L", [(108, 1000), (432, 96), (216, 300), (54, 700), (28, 1300), (70, 33)])
def test_fused_res_layer_is_the_operator_sequence(pkg, backend, orc, nerr, C, L):
    """The residual layer from fused calls (conv1d_fused, snake_copy_dev) against the same layer from the seam's operators
    in res_layer_device's order (src/graph.c:2423-2498): every value bit for bit.  And, for one shape, both against the oracle."""
    import importlib
    codec = importlib.import_module(pkg.__name__ + ".codec")
    _announce("fused residual layer %d x %d" % (C, L))
    x, blocks = _res_layer_inputs(C, L, 20 + C)
    n = C * L
    din = backend.alloc(n).write(x)
    bufs = [backend.alloc(n) for _ in range(8)]
    out_a, out_b = bufs[0], bufs[1]
    codec.res_layer(backend, blocks, din.ptr, out_a.ptr, C, L, *(b.ptr for b in bufs[2:6]))
    codec.res_layer_fused(backend, blocks, din.ptr, out_b.ptr, C, L, *(b.ptr for b in bufs[5:8]))
    seq, fused = out_a.read().reshape(C, L), out_b.read().reshape(C, L)
    assert np.isfinite(seq).all()
    assert np.array_equal(seq.view(np.uint32), fused.view(np.uint32))
    assert np.array_equal(din.read().reshape(C, L), x), "the layer's input was written"
    # the three branches' convolutions of a block and position in one launch each (conv1d_fused_batch): the same bits again
    more = [backend.alloc(n) for _ in range(10)]
    codec.res_layer_batched(backend, blocks, din.ptr, more[0].ptr, C, L, [b.ptr for b in more[1:4]], [b.ptr for b in more[4:7]],
                            [b.ptr for b in more[7:10]])
    batched = more[0].read().reshape(C, L)
    assert np.array_equal(seq.view(np.uint32), batched.view(np.uint32))
    assert np.array_equal(din.read().reshape(C, L), x), "the layer's input was written"
    for d in more:
        d.free()
    if C == 70:
        total = np.zeros_like(x)
        for branch in blocks:
            cur = x.copy()
            for a_in, (w_in, b_in), a_skip, (w_skip, b_skip), d in branch:
                cur = cur + orc.conv1d_causal(orc.snake(orc.conv1d_causal(orc.snake(cur, a_in, C // 2), w_in, b_in, d), a_skip, C // 2), w_skip, b_skip, 1)
            total += cur
        assert nerr(fused, total * np.float32(1.0 / 3.0)) < 1e-5
    for d in bufs + [din]:
        d.free()


def test_conv_batch_members_and_refusals(pkg, backend):
    """conv1d_fused_batch, two to four members: with tap counts outside 3 / 7 / 11 (run one after the other) and with them
    (one launch) every member gets its own conv1d_fused result bit for bit; a member that writes what another reads is refused."""
    _announce("conv1d_fused_batch members")
    rng = np.random.default_rng(77)
    C, O, L = 40, 72, 210
    x = rng.standard_normal((4, C, L)).astype(np.float32)
    r = rng.standard_normal((O, L)).astype(np.float32)
    alpha = (np.abs(rng.standard_normal(O // 2)) + 0.1).astype(np.float32)
    dins = [backend.alloc(C * L).write(x[i]) for i in range(4)]
    dres = backend.alloc(O * L).write(r)
    for taps in ((3, 7, 11), (11, 11, 3), (5, 7, 11), (7, 3), (11, 3, 7, 11)):
        ws = [(rng.standard_normal((O, C, k)) / np.sqrt(C * k)).astype(np.float32) for k in taps]
        bs = [rng.standard_normal(O).astype(np.float32) for _ in taps]
        single = [backend.alloc(O * L) for _ in taps]
        together = [backend.alloc(O * L) for _ in taps]
        acts = [backend.alloc(O * L) for _ in range(2)]
        extras = [dict(residual=dres.ptr, scale=0.5), dict(alpha=alpha, activated=acts[0].ptr), dict(), dict(alpha=alpha)][:len(taps)]
        for i, k in enumerate(taps):
            e = dict(extras[i])
            if "activated" in e:
                e["activated"] = acts[1].ptr
            backend.conv1d_fused(dins[i].ptr, single[i].ptr, C, O, L, k, 1 + i, ws[i], bs[i], **e)
        backend.conv1d_fused_batch([dict(din=dins[i].ptr, dout=together[i].ptr, kernel=k, dilation=1 + i, weight=ws[i], bias=bs[i], **extras[i])
                                    for i, k in enumerate(taps)], C, O, L)
        for a, b in zip(single, together):
            assert np.array_equal(a.read().view(np.uint32), b.read().view(np.uint32)), taps
        assert np.array_equal(acts[0].read().view(np.uint32), acts[1].read().view(np.uint32)), taps
        with pytest.raises(pkg.BackendError, match="another member"):
            backend.conv1d_fused_batch([dict(din=dins[0].ptr, dout=together[0].ptr, kernel=taps[0], dilation=1, weight=ws[0]),
                                        dict(din=together[0].ptr, dout=together[1].ptr, kernel=taps[1], dilation=1, weight=ws[1])], C, O, L)
        for d in single + together + acts:
            d.free()
    with pytest.raises(pkg.BackendError, match="one to four"):
        backend.conv1d_fused_batch([], C, O, L)
    for d in dins + [dres]:
        d.free()


def test_conv_batch_on_the_wider_split_tiles(backend):
    """432 channels x 512 positions: alone a convolution takes the channel-split kernel's 32 x 32 tiles, three side by side
    its 32 x 64 tiles.  The tile's width is not part of a value's arithmetic: every member keeps its single call's bits."""
    _announce("conv1d_fused_batch on 432 x 512")
    rng = np.random.default_rng(78)
    C, L, taps = 432, 512, (3, 7, 11)
    x = rng.standard_normal((C, L)).astype(np.float32)
    din = backend.alloc(C * L).write(x)
    ws = [(rng.standard_normal((C, C, k)) / np.sqrt(C * k)).astype(np.float32) for k in taps]
    bs = [rng.standard_normal(C).astype(np.float32) for _ in taps]
    single = [backend.alloc(C * L) for _ in taps]
    together = [backend.alloc(C * L) for _ in taps]
    for i, k in enumerate(taps):
        backend.conv1d_fused(din.ptr, single[i].ptr, C, C, L, k, 1 + 2 * i, ws[i], bs[i], residual=din.ptr)
    backend.conv1d_fused_batch([dict(din=din.ptr, dout=together[i].ptr, kernel=k, dilation=1 + 2 * i, weight=ws[i], bias=bs[i], residual=din.ptr)
                                for i, k in enumerate(taps)], C, C, L)
    for a, b in zip(single, together):
        got = b.read()
        assert np.isfinite(got).all()
        assert np.array_equal(a.read().view(np.uint32), got.view(np.uint32))
    for d in single + together + [din]:
        d.free()


def test_rows_combine_is_the_operator_sequence(pkg, backend):
    """rows_combine_dev against residual_inplace per addend, scale_dev and snake_dev / snake_copy_dev: bit for bit."""
    _announce("rows_combine_dev")
    rng = np.random.default_rng(91)
    C, L = 54, 333
    rows = (rng.standard_normal((3, C, L)) * 3).astype(np.float32)
    alphas = [(np.abs(rng.standard_normal(C // 2)) + 0.1).astype(np.float32) for _ in range(3)]
    dins = [backend.alloc(C * L).write(rows[i]) for i in range(3)]
    outs = [backend.alloc(C * L) for _ in range(3)]
    want = backend.alloc(C * L)
    bits = lambda d: d.read().view(np.uint32)
    # one input, three activated outputs
    backend.rows_combine_dev([dins[0].ptr], 1.0, [o.ptr for o in outs], alphas, C, L)
    for o, al in zip(outs, alphas):
        backend.snake_copy_dev(dins[0].ptr, want.ptr, al, C, L, C // 2)
        assert np.array_equal(bits(o), bits(want))
    # three inputs summed in order, scaled, one output plain and one activated
    backend.rows_combine_dev([d.ptr for d in dins], 1.0 / 3.0, [outs[0].ptr, outs[1].ptr], [None, alphas[1]], C, L)
    backend.copy_dev(want.ptr, dins[0].ptr, C * L)
    backend.residual_inplace(want.ptr, dins[1].ptr, C * L)
    backend.residual_inplace(want.ptr, dins[2].ptr, C * L)
    backend.scale_dev(want.ptr, C * L, 1.0 / 3.0)
    assert np.array_equal(bits(outs[0]), bits(want))
    backend.snake_dev(want.ptr, alphas[1], C, L, C // 2)
    assert np.array_equal(bits(outs[1]), bits(want))
    # an output that is also the first input
    backend.rows_combine_dev([d.ptr for d in dins], 1.0 / 3.0, [dins[0].ptr], [alphas[1]], C, L)
    assert np.array_equal(bits(dins[0]), bits(want))
    with pytest.raises(pkg.BackendError, match="named twice"):
        backend.rows_combine_dev([dins[1].ptr], 1.0, [outs[0].ptr, outs[0].ptr], [None, None], C, L)
    with pytest.raises(pkg.BackendError, match="one to four"):
        backend.rows_combine_dev([], 1.0, [outs[0].ptr], [None], C, L)
    for d in dins + outs + [want]:
        d.free()


def test_fused_conv_pieces(backend, orc, nerr):
    """Each optional step of conv1d_fused alone against the operator it stands for, bit for bit."""
    _announce("conv1d_fused steps")
    rng = np.random.default_rng(31)
    C, O, L, K, D = 40, 72, 210, 7, 3
    x = rng.standard_normal((C, L)).astype(np.float32)
    w = (rng.standard_normal((O, C, K)) / np.sqrt(C * K)).astype(np.float32)
    b = rng.standard_normal(O).astype(np.float32)
    r1, r2 = rng.standard_normal((2, O, L)).astype(np.float32)
    alpha = (np.abs(rng.standard_normal(O // 2)) + 0.1).astype(np.float32)
    din, dr1, dr2 = backend.alloc(x.size).write(x), backend.alloc(r1.size).write(r1), backend.alloc(r2.size).write(r2)
    plain, got, act = backend.alloc(O * L), backend.alloc(O * L), backend.alloc(O * L)
    bits = lambda d: d.read().view(np.uint32)

    backend.conv1d(din.ptr, plain.ptr, C, O, L, K, D, w, b)
    backend.conv1d_fused(din.ptr, got.ptr, C, O, L, K, D, w, b)                       # nothing added: the plain operator
    assert np.array_equal(bits(got), bits(plain))

    backend.conv1d_fused(din.ptr, got.ptr, C, O, L, K, D, w, b, residual=dr1.ptr, residual2=dr2.ptr, scale=0.25)
    backend.residual_inplace(dr1.ptr, plain.ptr, O * L)                                # dr1 += conv
    backend.residual_inplace(dr2.ptr, dr1.ptr, O * L)                                  # dr2 += that
    backend.scale_dev(dr2.ptr, O * L, 0.25)
    assert np.array_equal(bits(got), bits(dr2))

    backend.conv1d_fused(din.ptr, got.ptr, C, O, L, K, D, w, b, alpha=alpha, snake_channels=O // 2, activated=act.ptr)
    assert np.array_equal(bits(got), bits(plain)), "the plain value must stay beside the activated one"
    backend.snake_dev(plain.ptr, alpha, O, L, O // 2)
    assert np.array_equal(bits(act), bits(plain))
    backend.conv1d_fused(din.ptr, got.ptr, C, O, L, K, D, w, b, alpha=alpha, snake_channels=O // 2)
    assert np.array_equal(bits(got), bits(plain))

    # sine arguments beyond the short routine's range take the epilogue's other path (and the library's sine in both kernels)
    big = (alpha * np.float32(3.0e4)).astype(np.float32)
    backend.conv1d(din.ptr, plain.ptr, C, O, L, K, D, w, b)
    backend.snake_dev(plain.ptr, big, O, L, O // 2)
    backend.conv1d_fused(din.ptr, got.ptr, C, O, L, K, D, w, b, alpha=big, snake_channels=O // 2)
    assert np.array_equal(bits(got), bits(plain))
    conv = _run_conv1d(backend, x, w, b, D)
    assert nerr(got.read().reshape(O, L), orc.snake(conv, big, O // 2)) < 1e-6

    backend.snake_copy_dev(din.ptr, got.ptr, alpha[:C // 2], C, L, C // 2)
    assert nerr(got.read(x.size).reshape(C, L), orc.snake(x, alpha[:C // 2], C // 2)) < 1e-6
    assert np.array_equal(din.read().reshape(C, L), x)
    for d in (din, dr1, dr2, plain, got, act):
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
    e = backend.alloc(64)
    w3 = np.zeros((1, 1, 3), np.float32)
    with pytest.raises(pkg.BackendError, match="conv1d_fused"):      # the activated copy may not be the output itself
        backend.conv1d_fused(d.ptr, e.ptr, 1, 1, 8, 3, 1, w3, alpha=np.ones(1, np.float32), snake_channels=1, activated=e.ptr)
    with pytest.raises(pkg.BackendError, match="conv1d_fused"):      # more snake channels than output channels
        backend.conv1d_fused(d.ptr, e.ptr, 1, 1, 8, 3, 1, w3, alpha=np.ones(2, np.float32), snake_channels=2)
    e.free()
    d.free()
