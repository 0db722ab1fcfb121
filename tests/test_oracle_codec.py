"""Pins the oracle's codec operators (causal conv1d, grouped transposed conv, snake): against the compiled reference's own
conv1d_causal / conv_transpose_causal / snake fallback run on a synthetic safetensors file the test writes, against the
reference's resident-op known answers (gpu/metal/backend_metal_ops.m:1026-1106) and against float64 numpy."""
import ctypes as C

import numpy as np
import pytest


def _conv1d_f64(x, w, b, dilation):
    out_ch, in_ch, kernel = w.shape
    length = x.shape[1]
    out = np.zeros((out_ch, length), np.float64) + (0.0 if b is None else b.astype(np.float64)[:, None])
    for k in range(kernel):
        shift = (kernel - 1 - k) * dilation
        if shift >= length:
            continue
        out[:, shift:] += w[:, :, k].astype(np.float64) @ x[:, :length - shift].astype(np.float64)
    return out


def _convt_f64(x, w, b, stride, groups):
    in_ch, opg, kernel = w.shape
    length = x.shape[1]
    out_ch = opg * groups
    ipg = in_ch // groups
    full = np.zeros((out_ch, (length - 1) * stride + kernel), np.float64)
    for o in range(out_ch):
        g, ol = divmod(o, opg)
        for i in range(g * ipg, (g + 1) * ipg):
            for k in range(kernel):
                full[o, k:k + (length - 1) * stride + 1:stride] += x[i].astype(np.float64) * float(w[i, ol, k])
    out = full[:, :length * stride] if kernel >= stride else full
    return out + (0.0 if b is None else b.astype(np.float64)[:, None])


def test_known_answers(orc):
    # conv1d: input 1 2 3, taps 1 2, no bias -> 2 5 8 (gpu/metal/backend_metal_ops.m:1026-1027,1099-1106)
    out = orc.conv1d_causal(np.array([[1, 2, 3]], np.float32), np.array([[[1, 2]]], np.float32), None, 1)
    assert out.tolist() == [[2.0, 5.0, 8.0]]
    # snake with alpha 1: x + sin(x)^2; leaky half
    x = np.array([[0.5, -2.0], [3.0, -4.0]], np.float32)
    got = orc.snake(x, np.array([1.0], np.float32), 1)
    want0 = x[0].astype(np.float64) + np.sin(x[0].astype(np.float64)) ** 2
    assert np.abs(got[0] - want0).max() < 1e-6 and got[1].tolist() == [3.0, np.float32(-4.0) * np.float32(0.01)]


@pytest.mark.parametrize("shape", [(32, 864, 40, 7, 1), (54, 54, 300, 11, 5), (27, 1, 500, 3, 1), (16, 24, 9, 7, 3)])
def test_conv1d_against_reference_and_float64(orc, ref, nerr, tmp_path, shape):
    in_ch, out_ch, length, kernel, dilation = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((in_ch, length)).astype(np.float32)
    w = (rng.standard_normal((out_ch, in_ch, kernel)) / np.sqrt(in_ch * kernel)).astype(np.float32)
    b = rng.standard_normal(out_ch).astype(np.float32)
    got = orc.conv1d_causal(x, w, b, dilation)
    assert nerr(got, _conv1d_f64(x, w, b, dilation)) < 1e-5
    path = str(tmp_path / "codec.safetensors")
    orc.write_safetensors(path, {"w": w, "b": b})
    r = orc.ref_codec()
    out = np.zeros((out_ch, length), np.float32)
    err = C.create_string_buffer(256)
    rc = r.ref_conv1d(path.encode(), b"w", b"b", x.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data_as(C.POINTER(C.c_float)),
                      in_ch, out_ch, length, kernel, dilation, err, 256)
    assert rc == 0, err.value
    assert nerr(got, out) < 1e-5     # the reference sums through its im2col + sgemm, the oracle in scalar-loop order


@pytest.mark.parametrize("shape", [(864, 432, 30, 8), (108, 54, 77, 2), (8, 4, 5, 4)])
def test_conv_transpose_bit_exact_against_reference(orc, ref_strict, nerr, tmp_path, shape):
    in_ch, out_ch, length, stride = shape
    kernel, groups = 2 * stride, out_ch
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((in_ch, length)).astype(np.float32)
    w = rng.standard_normal((in_ch, out_ch // groups, kernel)).astype(np.float32)
    b = rng.standard_normal(out_ch).astype(np.float32)
    got = orc.conv_transpose_causal(x, w, b, stride, groups)
    assert got.shape == (out_ch, length * stride)
    assert nerr(got, _convt_f64(x, w, b, stride, groups)) < 1e-5
    path = str(tmp_path / "codec.safetensors")
    orc.write_safetensors(path, {"w": w, "b": b})
    r = orc.ref_codec(strict=True)
    out = np.zeros_like(got)
    err = C.create_string_buffer(256)
    rc = r.ref_conv_transpose(path.encode(), b"w", b"b", x.ctypes.data_as(C.POINTER(C.c_float)),
                              out.ctypes.data_as(C.POINTER(C.c_float)), in_ch, out_ch, length, kernel, stride, groups, err, 256)
    assert rc == 0, err.value
    assert np.array_equal(got, out)      # same order of the same IEEE operations (strict build of the reference)


def test_snake_against_reference(orc, ref_strict, nerr):
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((10, 333)) * 3).astype(np.float32)
    alpha = (np.abs(rng.standard_normal(5)) + 0.1).astype(np.float32)
    got = orc.snake(x, alpha, 5)
    want = x.copy()
    r = orc.ref_codec(strict=True)
    assert r.ref_snake(want.ctypes.data_as(C.POINTER(C.c_float)), alpha.ctypes.data_as(C.POINTER(C.c_float)), 10, 333, 5) == 0
    assert np.array_equal(got, want)
    f64 = x[:5].astype(np.float64) + np.sin(alpha[:, None].astype(np.float64) * x[:5]) ** 2 / (alpha[:, None].astype(np.float64) + 1e-9)
    assert nerr(got[:5], f64) < 1e-6
    assert np.array_equal(got[5:], np.where(x[5:] < 0, x[5:] * np.float32(0.01), x[5:]))
