"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header declares, and
its host-side load-time converters produce the reference's bytes.  No GPU call is made here."""
import ctypes as C
import os
import re

import numpy as np
import pytest


def _declared_functions(header_path):
    text = open(header_path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(mynah_(?:hip|backend_hip)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.load_library()
    names = _declared_functions(pkg.HEADER_PATH)
    assert len(names) >= 45
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, "declared in include/mynah_hip.h but not exported: %s" % missing


def test_missing_library_fails_loudly(pkg, tmp_path):
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.load_library(str(tmp_path / "absent.so"))


def test_header_is_plain_c(tmp_path):
    """The boundary must compile as C11 with nothing but the standard headers."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "t.c"
    src.write_text('#include "mynah_hip.h"\nint main(void) { return MYNAH_HIP_MAX_BATCH == 16 ? 0 : 1; }\n')
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(root, "include"), "-c", str(src),
                    "-o", str(tmp_path / "t.o")], check=True)


SHAPES = [(2304, 768), (768, 768), (96, 3072)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("arith", [0, 1])
def test_host_quantisers_match_oracle_and_reference(pkg, orc, shape, arith):
    """The library's load-time quantisers (host code) against the oracle; the oracle is pinned against the
    compiled reference in test_oracle_quant.py, and directly here when oracle/_ref is present."""
    lib = pkg.load_library()
    rng = np.random.default_rng(shape[0] + arith)
    w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    w[3] = 0.0                                        # all-zero row
    w[5, :32] = np.arange(32, dtype=np.float32) - 15.5  # half-integer grid after scaling
    q, s = pkg.quantize_weight_int8(lib, w, arith)
    oq, os_ = orc.quantize_weight_int8(w, arith)
    assert np.array_equal(q, oq) and np.array_equal(s.view(np.uint32), os_.view(np.uint32))
    rc, q4, s4 = pkg.quantize_weight_int4(lib, w, arith)
    oq4, os4 = orc.quantize_weight_int4(w, arith)
    assert rc == 0 and np.array_equal(q4, oq4) and np.array_equal(s4.view(np.uint32), os4.view(np.uint32))
    if orc.ref_available(strict=(arith == 0)):
        r = orc.load_ref(strict=(arith == 0))
        rq, rs = np.empty_like(q), np.empty_like(s)
        r.ref_quantize_weight_int8(w, shape[0], shape[1], rq, rs)
        assert np.array_equal(q, rq) and np.array_equal(s.view(np.uint32), rs.view(np.uint32))
        rq4, rs4 = np.empty_like(q4), np.empty_like(s4)
        r.ref_quantize_weight_int4(w, shape[0], shape[1], rq4, rs4)
        assert np.array_equal(q4, rq4) and np.array_equal(s4.view(np.uint32), rs4.view(np.uint32))


def test_host_int4_refuses_ragged_width(pkg):
    lib = pkg.load_library()
    rc, _, _ = pkg.quantize_weight_int4(lib, np.ones((4, 48), np.float32))
    assert rc == -1


def test_host_f16_conversion_is_ieee(pkg, orc):
    lib = pkg.load_library()
    rng = np.random.default_rng(9)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * np.float32(s) for s in (1e-8, 1e-5, 0.02, 1.0, 7e4)])
    h = rng.integers(0, 0x7bff, 20000).astype(np.uint16)
    ties = ((h.view(np.float16).astype(np.float64) + (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, ties, -ties, np.array([0.0, -0.0, 65504.0, 65520.0, np.inf, -np.inf, 2.0 ** -25, 2.0 ** -24], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = pkg.convert_weight_f16(lib, x)
    assert np.array_equal(got, want)
    assert np.array_equal(got, orc.f32_to_f16_bits(x))


def test_reference_backend_struct_binds_every_seam_symbol(orc, ref_strict, pkg, synth):
    """oracle/ref_shim_backend.c fills the reference's own backend struct (src/backend.c:26-70) from the library by
    symbol name, through pointers of the prototypes in include/mynah_hip.h: it compiled, so every prototype fits the
    struct's field; here it must find every symbol and reach the library's open call.  Without a GPU that call refuses
    with its own message (no CPU fallback); with one it succeeds."""
    cfg = synth.decoder_config(layers=1, capacity=8, cross_heads=1)
    w = synth.decoder_weights(cfg, seed=0, ln_bias=False)
    dec = orc.RefDecoder(cfg, w, orc.F32, 1, 4, strict=True)
    try:
        dec.use_hip(pkg.LIB_PATH)
    except RuntimeError as e:
        assert "missing symbol" not in str(e) and "dlopen" not in str(e), str(e)
        assert "HIP" in str(e) or "device" in str(e), str(e)
    finally:
        dec.close()


def test_entry_points_refuse_a_null_state(pkg):
    """Every resident entry point that only forwards to a launch returns -1 with a message for a NULL state, before it
    touches a device (no GPU is needed to see that)."""
    import ctypes as C
    lib = pkg.load_library()
    err = C.create_string_buffer(256)
    fake = C.c_void_p(0x1000)          # never dereferenced: the state is looked at first
    one = C.c_size_t(1)
    calls = {
        "mynah_hip_sgemm_dev": (None, 0, 0, one, one, one, C.c_float(1.0), fake, one, fake, one, C.c_float(0.0), fake, one),
        "mynah_hip_softmax_dev": (None, fake, one, one, one),
        "mynah_hip_copy_dev": (None, fake, fake, one),
        "mynah_hip_scale_dev": (None, fake, one, C.c_float(1.0)),
        "mynah_hip_clip_dev": (None, fake, one),
        "mynah_hip_self_attention_dev": (None, fake, fake, fake, C.c_size_t(0), one, one, one, C.c_size_t(64), C.c_float(1.0), fake),
        "mynah_hip_cross_attention_dev": (None, fake, fake, fake, one, one, one, C.c_size_t(64), C.c_float(1.0), fake),
        "mynah_hip_sync": (None,),
    }
    for name, args in calls.items():
        err.value = b""
        rc = getattr(lib, name)(*args, err, C.c_size_t(len(err)))
        assert rc == -1, name
        assert b"state is null" in err.value, (name, err.value)
