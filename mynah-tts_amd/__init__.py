"""Host-side bindings of the gfx950 HIP backend for Mynah TTS's decode-step kernels.

The product is the C-ABI shared library libmynah_hip.so (sources in csrc/, declarations in
include/mynah_hip.h).  This module only loads it through ctypes and mirrors the reference's
backend seam (src/backend.h) with the same names, argument meaning and error behaviour
(0 / -1 + message), so the parity tests read like the reference's own self-tests.

There is no CPU fallback: if the library is missing or no MI355X is present, loading or opening
fails loudly.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmynah_hip.so")
HEADER_PATH = os.path.join(HERE, "..", "include", "mynah_hip.h")

F32, INT8, INT4, F16 = 0, 1, 2, 3
ARITH_STRICT, ARITH_STOCK = 0, 1
MAX_BATCH = 16
QTYPE_NAMES = {F32: "f32", INT8: "int8", INT4: "int4", F16: "f16"}

_sz = C.c_size_t
_vp = C.c_void_p
_err = (C.c_char_p, _sz)

MATMUL_FN = C.CFUNCTYPE(C.c_int, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, C.c_char_p, _sz)
SGEMM_FN = C.CFUNCTYPE(C.c_int, _vp, C.c_int, C.c_int, _sz, _sz, _sz, C.c_float, _vp, _sz, _vp, _sz, C.c_float,
                       _vp, _sz, C.c_char_p, _sz)
CLOSE_FN = C.CFUNCTYPE(None, _vp)
SELF_TEST_FN = C.CFUNCTYPE(C.c_int, _vp, C.c_char_p, _sz)


class DecoderDesc(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn_width", _sz),
                ("cross_heads", _sz), ("cross_head_width", _sz), ("capacity", _sz),
                ("norm_self", _vp), ("norm_self_bias", _vp), ("norm_xattn_query", _vp), ("norm_xattn_query_bias", _vp),
                ("norm_pos_ff", _vp), ("norm_pos_ff_bias", _vp),
                ("qkv_w", _vp), ("o_self_w", _vp), ("q_cross_w", _vp), ("o_cross_w", _vp), ("ffn_up_w", _vp),
                ("ffn_down_w", _vp), ("norm_out", _vp), ("norm_out_bias", _vp), ("position", _vp)]


class DecoderSlot(C.Structure):
    _fields_ = [("dev_self_k", _vp), ("dev_self_v", _vp), ("dev_cross_k", _vp), ("dev_cross_v", _vp),
                ("length", _sz), ("memory_length", _sz), ("dev_input", _vp), ("dev_output", _vp)]


class Conv1dExtra(C.Structure):
    _fields_ = [("dev_residual", _vp), ("dev_residual2", _vp), ("scale", C.c_float), ("activate", C.c_int),
                ("snake_alpha", _vp), ("snake_channels", _sz), ("dev_activated", _vp)]


class Conv1dItem(C.Structure):
    _fields_ = [("dev_input", _vp), ("dev_output", _vp), ("kernel", C.c_int), ("dilation", C.c_int), ("weight", _vp), ("bias", _vp),
                ("extra", Conv1dExtra)]


class EncoderDesc(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn_width", _sz),
                ("vocab", _sz), ("max_positions", _sz), ("tok_table", _vp), ("pos_table", _vp),
                ("qkv_w", _vp), ("o_w", _vp), ("up_w", _vp), ("down_w", _vp),
                ("norm1", _vp), ("norm1_bias", _vp), ("norm2", _vp), ("norm2_bias", _vp),
                ("norm_out", _vp), ("norm_out_bias", _vp), ("causal", C.c_int), ("ffn_kernel", _sz), ("operands_f32", C.c_int)]


class LocalItem(C.Structure):
    _fields_ = [("dev_decoder_last", _vp), ("temperature", C.c_float), ("topk", _sz), ("rng_state", C.c_uint64),
                ("forbid_eos", C.c_int)]


class LocalDesc(C.Structure):
    _fields_ = [("streams", _sz), ("vocab", _sz), ("codebook_size", _sz), ("eos_id", _sz), ("codebook_count", _sz),
                ("projection_w", _vp), ("projection_bias", _vp), ("audio_table", _vp)]


def load_library(path=LIB_PATH):
    """dlopen the backend.  Raises (never falls back) when it has not been built."""
    if not os.path.exists(path):
        raise RuntimeError(
            "libmynah_hip.so is not built: run `python mynah-tts_amd/build.py` (needs hipcc for gfx950). "
            "There is no CPU fallback for the HIP backend.")
    lib = C.CDLL(path)
    lib.mynah_backend_hip_open.argtypes = [C.POINTER(_vp), C.POINTER(MATMUL_FN), C.POINTER(SGEMM_FN),
                                           C.POINTER(CLOSE_FN), C.POINTER(SELF_TEST_FN), *_err]
    lib.mynah_hip_dev_alloc.argtypes = [_vp, _sz, C.POINTER(_vp), *_err]
    lib.mynah_hip_dev_free.argtypes = [_vp, _vp]
    lib.mynah_hip_dev_free.restype = None
    lib.mynah_hip_h2d.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_d2h.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_upload.argtypes = [_vp, _vp, _sz, C.POINTER(_vp), *_err]
    lib.mynah_hip_download.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_sync.argtypes = [_vp, *_err]
    lib.mynah_hip_batch_begin.argtypes = [_vp, *_err]
    lib.mynah_hip_gelu_inplace.argtypes = [_vp, _vp, _sz, *_err]
    lib.mynah_hip_gelu_dev.argtypes = [_vp, _vp, _sz, *_err]
    lib.mynah_hip_residual_inplace.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_residual_add_dev.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_layer_norm_inplace.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, *_err]
    lib.mynah_hip_layer_norm_dev.argtypes = [_vp, _vp, _vp, _vp, _vp, _sz, _sz, *_err]
    for name in ("mynah_hip_matmul_d2d", "mynah_hip_matmul_dev", "mynah_hip_matmul_to_dev"):
        getattr(lib, name).argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, *_err]
    lib.mynah_hip_matvec_dev.argtypes = [_vp, _vp, _vp, _sz, _sz, _vp, _vp, *_err]
    lib.mynah_hip_sgemm_dev.argtypes = [_vp, C.c_int, C.c_int, _sz, _sz, _sz, C.c_float, _vp, _sz, _vp, _sz,
                                        C.c_float, _vp, _sz, *_err]
    lib.mynah_hip_softmax_dev.argtypes = [_vp, _vp, _sz, _sz, _sz, *_err]
    lib.mynah_hip_self_attention_dev.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_float, _vp, *_err]
    lib.mynah_hip_cross_attention_dev.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.c_float, _vp, *_err]
    lib.mynah_hip_self_attention_dev_noalloc.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_float, _vp, *_err]
    lib.mynah_hip_copy_dev.argtypes = [_vp, _vp, _vp, _sz, *_err]
    lib.mynah_hip_scale_dev.argtypes = [_vp, _vp, _sz, C.c_float, *_err]
    lib.mynah_hip_clip_dev.argtypes = [_vp, _vp, _sz, *_err]
    lib.mynah_hip_argmax_dev.argtypes = [_vp, _vp, _sz, _sz, _sz, C.c_int, C.POINTER(C.c_uint), *_err]
    lib.mynah_hip_conv1d.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _vp, *_err]
    lib.mynah_hip_conv_transpose_dev.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _vp,
                                                 *_err]
    lib.mynah_hip_snake_dev.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, *_err]
    lib.mynah_hip_snake_copy_dev.argtypes = [_vp, _vp, _vp, _vp, _sz, _sz, _sz, *_err]
    lib.mynah_hip_rows_combine_dev.argtypes = [_vp, C.POINTER(_vp), _sz, C.c_float, C.POINTER(_vp), C.POINTER(_vp), _sz, _sz, _sz, _sz, *_err]
    lib.mynah_hip_conv1d_fused_batch.argtypes = [_vp, C.POINTER(Conv1dItem), _sz, C.c_int, C.c_int, C.c_int, *_err]
    lib.mynah_hip_conv1d_fused.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _vp,
                                           C.POINTER(Conv1dExtra), *_err]
    lib.mynah_hip_set_quant.argtypes = [_vp, C.c_int, C.c_int, *_err]
    lib.mynah_hip_quantize_weight_int8.argtypes = [_vp, _sz, _sz, _vp, _vp, C.c_int]
    lib.mynah_hip_quantize_weight_int8.restype = None
    lib.mynah_hip_quantize_weight_int4.argtypes = [_vp, _sz, _sz, _vp, _vp, C.c_int]
    lib.mynah_hip_convert_weight_f16.argtypes = [_vp, _sz, _vp]
    lib.mynah_hip_convert_weight_f16.restype = None
    lib.mynah_hip_matmul_d2d_batched.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, *_err]
    lib.mynah_hip_matmul_d2d_probe.argtypes = [_vp, _vp, _vp, _sz, _sz, _vp, _vp, _vp, _vp, _vp, *_err]
    lib.mynah_hip_self_attention_dev_batched.argtypes = [_vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _sz, _sz, C.c_float,
                                                         _vp, *_err]
    lib.mynah_hip_cross_attention_dev_batched.argtypes = [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.c_float, _vp,
                                                          *_err]
    lib.mynah_hip_head_argmax.argtypes = [_vp, _vp, _sz, _sz, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp, _vp, *_err]
    lib.mynah_hip_cross_kv_dev.argtypes = [_vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp, _sz, _vp, _vp, *_err]
    lib.mynah_hip_embed_gather.argtypes = [_vp, _vp, _vp, _sz, _vp, _sz, _sz, C.c_float, _vp, _sz, _vp, *_err]
    lib.mynah_hip_decoder_create.argtypes = [_vp, C.POINTER(DecoderDesc), C.POINTER(_vp), *_err]
    lib.mynah_hip_decoder_destroy.argtypes = [_vp, _vp]
    lib.mynah_hip_decoder_destroy.restype = None
    lib.mynah_hip_decoder_step.argtypes = [_vp, _vp, C.POINTER(DecoderSlot), _sz, *_err]
    lib.mynah_hip_output_head.argtypes = [_vp, _vp, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _vp, *_err]
    lib.mynah_hip_decoder_stage_enqueue.argtypes = [_vp, _vp, _sz, C.c_int, *_err]
    lib.mynah_hip_decoder_step_probe.argtypes = [_vp, _vp, C.POINTER(DecoderSlot), _sz, _vp, _vp, *_err]
    lib.mynah_hip_local_create.argtypes = [_vp, C.POINTER(DecoderDesc), C.POINTER(LocalDesc), C.POINTER(_vp), *_err]
    lib.mynah_hip_local_destroy.argtypes = [_vp, _vp]
    lib.mynah_hip_local_destroy.restype = None
    lib.mynah_hip_local_frame.argtypes = [_vp, _vp, C.POINTER(LocalItem), _sz, _vp, _vp, _vp, _vp, _vp, *_err]
    lib.mynah_hip_encoder_create.argtypes = [_vp, C.POINTER(EncoderDesc), C.POINTER(_vp), *_err]
    lib.mynah_hip_encoder_destroy.argtypes = [_vp, _vp]
    lib.mynah_hip_encoder_destroy.restype = None
    lib.mynah_hip_encoder_prefill.argtypes = [_vp, _vp, _vp, _sz, _vp, _vp, *_err]
    lib.mynah_hip_timer_begin.argtypes = [_vp, *_err]
    lib.mynah_hip_timer_end.argtypes = [_vp, C.POINTER(C.c_float), *_err]
    lib.mynah_hip_flush_cache.argtypes = [_vp, _sz, *_err]
    lib.mynah_hip_set_graph_mode.argtypes = [_vp, C.c_int, *_err]
    lib.mynah_hip_set_step_lanes.argtypes = [_vp, C.c_int, *_err]
    lib.mynah_hip_im2col.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, *_err]
    lib.mynah_hip_gelu_host.argtypes = [_vp, _vp, _sz, *_err]
    lib.mynah_hip_gelu_host_f64.argtypes = [_vp, _vp, _sz, *_err]
    lib.mynah_hip_matmul_graph.argtypes = [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp, *_err]
    lib.mynah_hip_device_memory.argtypes = [_vp, C.POINTER(_sz), C.POINTER(_sz), *_err]
    lib.mynah_hip_weights_export.argtypes = [_vp, C.c_char_p, C.POINTER(_sz), *_err]
    lib.mynah_hip_weights_import.argtypes = [_vp, C.c_char_p, C.POINTER(_sz), *_err]
    lib.mynah_hip_weights_from_pack.argtypes = [_vp]
    lib.mynah_hip_weights_from_pack.restype = C.c_size_t
    lib.mynah_hip_wait_fallbacks.argtypes = [_vp]
    lib.mynah_hip_wait_fallbacks.restype = C.c_size_t
    lib.mynah_hip_dependent_launch_probe.argtypes = [_vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float), *_err]
    lib.mynah_hip_cached_weight_bytes.argtypes = [_vp]
    lib.mynah_hip_cached_weight_bytes.restype = _sz
    return lib


class BackendError(RuntimeError):
    pass


def _np_ptr(a):
    return None if a is None else a.ctypes.data_as(_vp)


class DeviceBuffer:
    """n floats of device memory owned through mynah_hip_dev_alloc / dev_free."""

    def __init__(self, backend, n):
        self.backend, self.n = backend, int(n)
        p = _vp()
        backend._call("mynah_hip_dev_alloc", _sz(self.n), C.byref(p))
        self.ptr = p.value

    def at(self, offset_floats):
        return self.ptr + 4 * int(offset_floats)

    def write(self, host, offset=0):
        host = np.ascontiguousarray(host)
        assert host.nbytes % 4 == 0 and host.nbytes // 4 + offset <= self.n
        self.backend._call("mynah_hip_h2d", _np_ptr(host), _vp(self.at(offset)), _sz(host.nbytes // 4))
        return self

    def read(self, n=None, offset=0, dtype=np.float32):
        n = self.n - offset if n is None else n
        out = np.empty(n, np.float32)
        self.backend._call("mynah_hip_d2h", _vp(self.at(offset)), _np_ptr(out), _sz(n))
        return out.view(dtype)

    def free(self):
        if self.ptr:
            self.backend.lib.mynah_hip_dev_free(self.backend.state, _vp(self.ptr))
            self.ptr = None


class Backend:
    """mynah_backend_open(MYNAH_TTS_DEVICE_HIP) as the reference's backend.c would wire it
    (src/backend.c:367-475): one opaque state plus the function pointers handed back by open."""

    def __init__(self, quant=None, arith=None):
        self.lib = load_library()
        self.state = _vp()
        self._matmul, self._sgemm = MATMUL_FN(), SGEMM_FN()
        self._close, self._self_test = CLOSE_FN(), SELF_TEST_FN()
        err = C.create_string_buffer(512)
        rc = self.lib.mynah_backend_hip_open(C.byref(self.state), C.byref(self._matmul), C.byref(self._sgemm),
                                             C.byref(self._close), C.byref(self._self_test), err, 512)
        if rc != 0:
            raise BackendError("mynah_backend_hip_open failed: " + err.value.decode())
        self._keep = []   # host arrays whose addresses key the device weight cache
        if quant is not None or arith is not None:
            self.set_quant(F32 if quant is None else quant, ARITH_STRICT if arith is None else arith)

    # -- plumbing
    def _call(self, name, *args):
        err = C.create_string_buffer(512)
        rc = getattr(self.lib, name)(self.state, *args, err, 512)
        if rc != 0:
            raise BackendError("%s: %s" % (name, err.value.decode()))
        return rc

    def keep(self, array):
        """Pin a host tensor for the life of the backend (the cache keys on its address)."""
        a = np.ascontiguousarray(array, np.float32)
        self._keep.append(a)
        return a

    def close(self):
        if self.state:
            self._close(self.state)
            self.state = _vp()

    def alloc(self, n):
        return DeviceBuffer(self, n)

    def sync(self):
        self._call("mynah_hip_sync")

    def upload(self, array):
        """mynah_backend_upload (src/backend.h:79-81): host floats into the backend's one upload buffer.  Returns the
        device address, valid until the next upload or host-pointer matmul."""
        a = np.ascontiguousarray(array, np.float32)
        dev = _vp()
        self._call("mynah_hip_upload", _np_ptr(a), _sz(a.size), C.byref(dev))
        return dev.value

    def download(self, dev_ptr, n):
        """mynah_backend_download (src/backend.h:83-85): n floats from a device address, synchronous."""
        out = np.empty(n, np.float32)
        self._call("mynah_hip_download", _vp(dev_ptr), _np_ptr(out), _sz(n))
        return out

    def set_quant(self, qtype, arith=ARITH_STRICT):
        self._call("mynah_hip_set_quant", C.c_int(qtype), C.c_int(arith))

    # -- host-pointer seam ops
    def self_test(self):
        err = C.create_string_buffer(512)
        rc = self._self_test(self.state, err, 512)
        return rc, err.value.decode()

    def matmul(self, inp, weight, bias=None):
        inp = np.ascontiguousarray(inp, np.float32)
        rows, iw = inp.shape
        ow = weight.shape[0]
        out = np.empty((rows, ow), np.float32)
        err = C.create_string_buffer(512)
        rc = self._matmul(self.state, _np_ptr(inp), _np_ptr(out), rows, iw, ow, _np_ptr(weight), _np_ptr(bias), err, 512)
        if rc != 0:
            raise BackendError(err.value.decode())
        return out

    def sgemm(self, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
        err = C.create_string_buffer(512)
        rc = self._sgemm(self.state, ta, tb, m, n, k, alpha, _np_ptr(a), lda, _np_ptr(b), ldb, beta, _np_ptr(c), ldc,
                         err, 512)
        if rc != 0:
            raise BackendError(err.value.decode())
        return c

    # -- resident seam ops (device buffers in, host weights)
    def matmul_d2d(self, din, dout, rows, iw, ow, weight, bias=None):
        self._call("mynah_hip_matmul_d2d", _vp(din), _vp(dout), _sz(rows), _sz(iw), _sz(ow), _np_ptr(weight), _np_ptr(bias))

    def matmul_d2d_batched(self, dins, douts, iw, ow, weight, bias=None):
        B = len(dins)
        arr = _vp * B
        self._call("mynah_hip_matmul_d2d_batched", arr(*dins), arr(*douts), _sz(B), _sz(iw), _sz(ow), _np_ptr(weight),
                   _np_ptr(bias))

    def matmul_probe(self, din, dout, iw, ow, weight, bias, dqx, dsx, dacc):
        self._call("mynah_hip_matmul_d2d_probe", _vp(din), _vp(dout), _sz(iw), _sz(ow), _np_ptr(weight), _np_ptr(bias),
                   _vp(dqx), _vp(dsx), _vp(dacc))

    def layer_norm_inplace(self, din, dout, gain, rows, width):
        self._call("mynah_hip_layer_norm_inplace", _vp(din), _vp(dout), _np_ptr(gain), _sz(rows), _sz(width))

    def layer_norm_dev(self, din, dout, gain, bias, rows, width):
        self._call("mynah_hip_layer_norm_dev", _vp(din), _vp(dout), _np_ptr(gain), _np_ptr(bias), _sz(rows), _sz(width))

    def gelu_inplace(self, d, n):
        self._call("mynah_hip_gelu_inplace", _vp(d), _sz(n))

    def residual_inplace(self, dout, din, n):
        self._call("mynah_hip_residual_inplace", _vp(dout), _vp(din), _sz(n))

    def softmax_dev(self, d, rows, cols, valid):
        self._call("mynah_hip_softmax_dev", _vp(d), _sz(rows), _sz(cols), _sz(valid))

    def head_argmax(self, dev_hidden, width, weight, bias, streams, vocab, codebook_size, eos_id, codebook_count, forbid_eos):
        """Returns (values, stored) [batch, streams], saw_eos [batch], eos_frame [batch] (None where no EOS)."""
        B = len(dev_hidden)
        values, stored = np.zeros((B, streams), np.uint32), np.zeros((B, streams), np.uint32)
        saw = np.zeros(B, np.int32)
        frame = np.zeros(B, np.uint64)
        forbid = np.ascontiguousarray(forbid_eos, np.int32)
        self._call("mynah_hip_head_argmax", (_vp * B)(*dev_hidden), _sz(B), _sz(width), _np_ptr(weight), _np_ptr(bias), _sz(streams), _sz(vocab),
                   _sz(codebook_size), _sz(eos_id), _sz(codebook_count), _np_ptr(forbid), _np_ptr(values), _np_ptr(stored), _np_ptr(saw),
                   _np_ptr(frame))
        return values, stored, saw, [None if f == np.iinfo(np.uint64).max else int(f) for f in frame]

    def cross_kv_dev(self, dmemory, memory_length, width, norm_gains, norm_biases, kv_ws, xattn_width, dck, dcv):
        """norm_gains / kv_ws: per-layer lists of kept host arrays (norm_biases may be None)."""
        layers = len(kv_ws)
        g, w = _ptr_array(norm_gains), _ptr_array(kv_ws)
        b = _ptr_array(norm_biases) if norm_biases is not None else None
        self._call("mynah_hip_cross_kv_dev", _vp(dmemory), _sz(memory_length), _sz(width), _sz(layers), C.cast(g, _vp),
                   C.cast(b, _vp) if b is not None else None, C.cast(w, _vp), _sz(xattn_width), _vp(dck), _vp(dcv))

    def copy_dev(self, dst, src, n):
        self._call("mynah_hip_copy_dev", _vp(dst), _vp(src), _sz(n))

    def scale_dev(self, d, n, scale):
        self._call("mynah_hip_scale_dev", _vp(d), _sz(n), C.c_float(scale))

    def clip_dev(self, d, n):
        self._call("mynah_hip_clip_dev", _vp(d), _sz(n))

    def conv1d(self, din, dout, in_ch, out_ch, length, kernel, dilation, weight, bias=None):
        self._call("mynah_hip_conv1d", din, dout, in_ch, out_ch, length, kernel, dilation, _np_ptr(self.keep(weight)),
                   None if bias is None else _np_ptr(self.keep(bias)))

    def conv_transpose_dev(self, din, dout, in_ch, out_ch, length, output_length, kernel, stride, groups, weight, bias=None):
        self._call("mynah_hip_conv_transpose_dev", din, dout, in_ch, out_ch, length, output_length, kernel, stride, groups,
                   _np_ptr(self.keep(weight)), None if bias is None else _np_ptr(self.keep(bias)))

    def snake_dev(self, d, alpha, channels, length, snake_channels):
        self._call("mynah_hip_snake_dev", d, _np_ptr(self.keep(alpha)), _sz(channels), _sz(length), _sz(snake_channels))

    def snake_copy_dev(self, din, dout, alpha, channels, length, snake_channels):
        self._call("mynah_hip_snake_copy_dev", din, dout, _np_ptr(self.keep(alpha)), _sz(channels), _sz(length), _sz(snake_channels))

    def conv1d_fused(self, din, dout, in_ch, out_ch, length, kernel, dilation, weight, bias=None, residual=None, residual2=None,
                     scale=1.0, alpha=None, snake_channels=None, activated=None):
        """conv1d, then per value: + residual, + residual2, * scale, and (alpha given) the half-snake, written to dout or,
        with `activated`, beside the plain value."""
        extra = Conv1dExtra(residual, residual2, scale, 0 if alpha is None else 1,
                            None if alpha is None else _np_ptr(self.keep(alpha)),
                            0 if alpha is None else (out_ch // 2 if snake_channels is None else snake_channels), activated)
        self._call("mynah_hip_conv1d_fused", din, dout, in_ch, out_ch, length, kernel, dilation, _np_ptr(self.keep(weight)),
                   None if bias is None else _np_ptr(self.keep(bias)), C.byref(extra))

    def conv1d_fused_batch(self, items, in_ch, out_ch, length):
        """Up to four conv1d_fused calls of one shape in one launch.  items: dicts with din, dout, kernel, dilation, weight and,
        optionally, bias, residual, residual2, scale, alpha, snake_channels, activated (conv1d_fused's arguments)."""
        arr = (Conv1dItem * len(items))()
        for slot, it in zip(arr, items):
            alpha = it.get("alpha")
            snake = 0 if alpha is None else (out_ch // 2 if it.get("snake_channels") is None else it["snake_channels"])
            slot.dev_input, slot.dev_output, slot.kernel, slot.dilation = it["din"], it["dout"], it["kernel"], it["dilation"]
            slot.weight = _np_ptr(self.keep(it["weight"]))
            slot.bias = None if it.get("bias") is None else _np_ptr(self.keep(it["bias"]))
            slot.extra = Conv1dExtra(it.get("residual"), it.get("residual2"), it.get("scale", 1.0), 0 if alpha is None else 1,
                                     None if alpha is None else _np_ptr(self.keep(alpha)), snake, it.get("activated"))
        self._call("mynah_hip_conv1d_fused_batch", arr, _sz(len(items)), in_ch, out_ch, length)

    def rows_combine_dev(self, dins, scale, douts, alphas, channels, length, snake_channels=None):
        """((in0 + in1) + ...) * scale into every output, through the half-snake of alphas[j] where that is not None."""
        arr_in, arr_out = (_vp * len(dins))(*dins), (_vp * len(douts))(*douts)
        arr_al = (_vp * len(douts))(*[None if a is None else _np_ptr(self.keep(a)) for a in alphas])
        self._call("mynah_hip_rows_combine_dev", arr_in, _sz(len(dins)), C.c_float(scale), arr_out, arr_al, _sz(len(douts)), _sz(channels),
                   _sz(length), _sz(channels // 2 if snake_channels is None else snake_channels))

    def argmax_dev(self, dlogits, vocab, codebook_size, eos_id, allow_eos):
        out = C.c_uint(0)
        self._call("mynah_hip_argmax_dev", _vp(dlogits), _sz(vocab), _sz(codebook_size), _sz(eos_id), C.c_int(int(allow_eos)),
                   C.byref(out))
        return out.value

    def self_attention_dev(self, dqkv, dk, dv, position, stride, valid, heads, hw, scale, dout):
        self._call("mynah_hip_self_attention_dev", _vp(dqkv), _vp(dk), _vp(dv), _sz(position), _sz(stride), _sz(valid),
                   _sz(heads), _sz(hw), C.c_float(scale), _vp(dout))

    def self_attention_dev_noalloc(self, dqkv, dk, dv, position, stride, valid, heads, hw, scale, dout):
        self._call("mynah_hip_self_attention_dev_noalloc", _vp(dqkv), _vp(dk), _vp(dv), _sz(position), _sz(stride), _sz(valid),
                   _sz(heads), _sz(hw), C.c_float(scale), _vp(dout))

    def cross_attention_dev(self, dq, dk, dv, valid, stride, heads, hw, scale, dout):
        self._call("mynah_hip_cross_attention_dev", _vp(dq), _vp(dk), _vp(dv), _sz(valid), _sz(stride), _sz(heads), _sz(hw),
                   C.c_float(scale), _vp(dout))

    def self_attention_dev_batched(self, dqkv, dk, dv, positions, stride, valids, heads, hw, scale, douts):
        B = len(dqkv)
        arr, szs = _vp * B, _sz * B
        self._call("mynah_hip_self_attention_dev_batched", arr(*dqkv), arr(*dk), arr(*dv), szs(*positions), _sz(stride),
                   szs(*valids), _sz(B), _sz(heads), _sz(hw), C.c_float(scale), arr(*douts))

    def cross_attention_dev_batched(self, dq, dk, dv, valids, stride, heads, hw, scale, douts):
        B = len(dq)
        arr, szs = _vp * B, _sz * B
        self._call("mynah_hip_cross_attention_dev_batched", arr(*dq), arr(*dk), arr(*dv), szs(*valids), _sz(stride), _sz(B),
                   _sz(heads), _sz(hw), C.c_float(scale), arr(*douts))

    def embed_gather(self, tables, ids, width, scale, position, position_offset, dout):
        ids = np.ascontiguousarray(ids, np.int32)
        T = len(tables)
        tokens = ids.size // T
        arr = _vp * T
        rows = (_sz * T)(*[t.shape[0] for t in tables])
        self._call("mynah_hip_embed_gather", arr(*[_np_ptr(t) for t in tables]), rows, _sz(T), _np_ptr(ids), _sz(tokens),
                   _sz(width), C.c_float(scale), _np_ptr(position), _sz(position_offset), _vp(dout))

    def output_head(self, dhidden, width, weight, bias, rows, vocab, dlogits, dprobs):
        B = len(dhidden)
        arr = _vp * B
        self._call("mynah_hip_output_head", arr(*dhidden), _sz(B), _sz(width), _np_ptr(weight), _np_ptr(bias), _sz(rows),
                   _sz(vocab), arr(*dlogits), None if dprobs is None else arr(*dprobs))

    # -- measurement
    def timer_begin(self):
        self._call("mynah_hip_timer_begin")

    def timer_end(self):
        ms = C.c_float(0)
        self._call("mynah_hip_timer_end", C.byref(ms))
        return ms.value

    def flush_cache(self, nbytes=512 << 20):
        self._call("mynah_hip_flush_cache", _sz(nbytes))

    def set_graph_mode(self, enabled):
        self._call("mynah_hip_set_graph_mode", C.c_int(int(enabled)))

    def dependent_launch_probe(self, nodes=72, workgroups=192, floats=768, chains=1, repeats=20):
        """Microseconds per dependent graph node that only hands a `floats`-long vector to the next node (no weights, no caches)."""
        us = C.c_float(0.0)
        self._call("mynah_hip_dependent_launch_probe", C.c_int(nodes), C.c_int(workgroups), C.c_int(floats), C.c_int(chains), C.c_int(repeats),
                   C.byref(us))
        return float(us.value)

    def device_memory(self):
        """(free bytes, total bytes) of the device."""
        free, total = _sz(0), _sz(0)
        self._call("mynah_hip_device_memory", C.byref(free), C.byref(total))
        return int(free.value), int(total.value)

    def weights_export(self, path):
        """Writes every converted weight the backend holds to a packed-weight file; returns the number of entries."""
        n = _sz(0)
        self._call("mynah_hip_weights_export", os.fsencode(path), C.byref(n))
        return int(n.value)

    def weights_import(self, path):
        """Reads a packed-weight file: matching tensors are then uploaded from it instead of being converted."""
        n = _sz(0)
        self._call("mynah_hip_weights_import", os.fsencode(path), C.byref(n))
        return int(n.value)

    def weights_from_pack(self):
        return int(self.lib.mynah_hip_weights_from_pack(self.state))

    def wait_fallbacks(self):
        """Steps that were repeated in the wait-free form because a workgroup had given up a bounded wait."""
        return int(self.lib.mynah_hip_wait_fallbacks(self.state))

    def im2col(self, din, dcolumns, in_channels, length, kernel, dilation):
        self._call("mynah_hip_im2col", _vp(din), _vp(dcolumns), C.c_int(in_channels), C.c_int(length), C.c_int(kernel), C.c_int(dilation))

    def gelu_host(self, data, in_double=False):
        """tanh-GELU of a host float32 array, in place (upload, kernel, download, synchronise)."""
        assert data.dtype == np.float32 and data.flags["C_CONTIGUOUS"]
        self._call("mynah_hip_gelu_host_f64" if in_double else "mynah_hip_gelu_host", _np_ptr(data), _sz(data.size))
        return data

    def matmul_graph(self, x, weight, bias=None):
        x = np.ascontiguousarray(x, np.float32)
        rows, iw = x.shape
        out = np.empty((rows, weight.shape[0]), np.float32)
        self._call("mynah_hip_matmul_graph", _np_ptr(x), _np_ptr(out), _sz(rows), _sz(iw), _sz(weight.shape[0]), _np_ptr(weight), _np_ptr(bias))
        return out

    def set_step_lanes(self, lanes):
        """Groups a resident step above two streams is cut into, each stepping on a stream of its own (0: chosen from the batch size)."""
        self._call("mynah_hip_set_step_lanes", C.c_int(int(lanes)))

    def cached_weight_bytes(self):
        return self.lib.mynah_hip_cached_weight_bytes(self.state)


def _ptr_array(arrays):
    """C array of host pointers (one per layer); None entries stay NULL."""
    arr = (_vp * len(arrays))(*[_np_ptr(a) for a in arrays])
    return arr


def _decoder_desc(backend, cfg, weights, hold):
    """Fills a DecoderDesc with host pointers the backend keeps alive; `hold` collects the pointer arrays."""
    L = cfg["layers"]

    def per_layer(name):
        if weights.get(name) is None:
            return None
        rows = [backend.keep(weights[name][l]) for l in range(L)]
        arr = _ptr_array(rows)
        hold.append(arr)
        return C.cast(arr, _vp)

    def single(name):
        if weights.get(name) is None:
            return None
        return _np_ptr(backend.keep(weights[name]))

    d = DecoderDesc()
    d.layers, d.width, d.heads, d.head_width, d.ffn_width = L, cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
    d.cross_heads, d.cross_head_width, d.capacity = cfg["cross_heads"], cfg["cross_head_width"], cfg["capacity"]
    d.norm_self, d.norm_self_bias = per_layer("norm_self_g"), per_layer("norm_self_b")
    if cfg["cross_heads"]:
        d.norm_xattn_query, d.norm_xattn_query_bias = per_layer("norm_cross_g"), per_layer("norm_cross_b")
        d.q_cross_w, d.o_cross_w = per_layer("q_cross"), per_layer("o_cross")
    d.norm_pos_ff, d.norm_pos_ff_bias = per_layer("norm_ff_g"), per_layer("norm_ff_b")
    d.qkv_w, d.o_self_w = per_layer("qkv"), per_layer("o_self")
    d.ffn_up_w, d.ffn_down_w = per_layer("ffn_up"), per_layer("ffn_down")
    d.norm_out, d.norm_out_bias, d.position = single("norm_out_g"), single("norm_out_b"), single("position")
    return d


class Decoder:
    """mynah_hip_decoder_create + step: the batched resident decode step."""

    def __init__(self, backend, cfg, weights):
        self.backend, self.cfg = backend, cfg
        self._hold = []
        self.desc = _decoder_desc(backend, cfg, weights, self._hold)
        h = _vp()
        backend._call("mynah_hip_decoder_create", C.byref(self.desc), C.byref(h))
        self.handle = h

    def step(self, slots):
        """slots: list of dicts with k, v, ck, cv (device addresses), length, memory_length, inp, out."""
        B = len(slots)
        arr = (DecoderSlot * B)()
        for i, s in enumerate(slots):
            arr[i] = DecoderSlot(s["k"], s["v"], s.get("ck"), s.get("cv"), s["length"], s.get("memory_length", 0),
                                 s["inp"], s["out"])
        self.backend._call("mynah_hip_decoder_step", self.handle, arr, _sz(B))

    def step_head(self, slots, weight, bias, rows, vocab, dlogits, dprobs):
        """The step and the output head on the slots' outputs as one call (mynah_hip_decoder_step_head)."""
        B = len(slots)
        arr = (DecoderSlot * B)()
        for i, s in enumerate(slots):
            arr[i] = DecoderSlot(s["k"], s["v"], s.get("ck"), s.get("cv"), s["length"], s.get("memory_length", 0), s["inp"], s["out"])
        ptrs = _vp * B
        self.backend._call("mynah_hip_decoder_step_head", self.handle, arr, _sz(B), _np_ptr(weight), _np_ptr(bias), _sz(rows), _sz(vocab),
                           ptrs(*dlogits), None if dprobs is None else ptrs(*dprobs))

    def step_probe(self, slots):
        """One step of one or two streams as plain launches; returns (qx [layers, 6, ffn] int8, sx [layers, 6] f32) of stream 0:
        the int8 activations and scales the device formed at each projection (qkv, o_self, q_cross, o_cross, up, down)."""
        B = len(slots)
        arr = (DecoderSlot * B)()
        for i, s in enumerate(slots):
            arr[i] = DecoderSlot(s["k"], s["v"], s.get("ck"), s.get("cv"), s["length"], s.get("memory_length", 0), s["inp"], s["out"])
        layers, ffn = int(self.desc.layers), int(self.desc.ffn_width)
        dqx = self.backend.alloc((layers * 6 * ffn + 3) // 4)
        dsx = self.backend.alloc(layers * 6)
        dqx.write(np.zeros((layers * 6 * ffn + 3) // 4, np.float32))
        try:
            self.backend._call("mynah_hip_decoder_step_probe", self.handle, arr, _sz(B), _vp(dqx.ptr), _vp(dsx.ptr))
            qx = dqx.read().view(np.int8)[:layers * 6 * ffn].reshape(layers, 6, ffn).copy()
            sx = dsx.read().reshape(layers, 6).copy()
        finally:
            dqx.free()
            dsx.free()
        return qx, sx

    def stage_enqueue(self, batch, stage):
        """Measurement helper: one stage of the step (all layers) as its own graph, see mynah_hip_decoder_stage_enqueue."""
        self.backend._call("mynah_hip_decoder_stage_enqueue", self.handle, _sz(batch), C.c_int(stage))

    def destroy(self):
        if self.handle:
            self.backend.lib.mynah_hip_decoder_destroy(self.backend.state, self.handle)
            self.handle = None


class Local:
    """mynah_hip_local_create + frame: the local transformer's per-frame token loop, resident on the device."""

    def __init__(self, backend, cfg, weights, projections, biases, tables, codebook_size, eos_id, codebook_count):
        self.backend, self.cfg = backend, cfg
        self._hold = []
        self.stack_desc = _decoder_desc(backend, cfg, weights, self._hold)
        self.streams, self.vocab = len(projections), int(projections[0].shape[0])
        d = LocalDesc()
        d.streams, d.vocab, d.codebook_size, d.eos_id, d.codebook_count = self.streams, self.vocab, codebook_size, eos_id, codebook_count
        for name, arrays in (("projection_w", projections), ("projection_bias", biases), ("audio_table", tables)):
            if arrays is None:
                continue
            arr = _ptr_array([None if a is None else backend.keep(a) for a in arrays])
            self._hold.append(arr)
            setattr(d, name, C.cast(arr, _vp))
        self.desc = d
        h = _vp()
        backend._call("mynah_hip_local_create", C.byref(self.stack_desc), C.byref(d), C.byref(h))
        self.handle = h

    def frame(self, items, dev_logits_copy=None):
        """items: list of dicts {row (device address of the decoder's output row), temperature, topk, rng_state,
        forbid_eos}.  Returns values, stored [B, streams], saw_eos, eos_frame, rng_state (advanced)."""
        B = len(items)
        arr = (LocalItem * B)()
        for i, it in enumerate(items):
            arr[i] = LocalItem(it["row"], it["temperature"], it["topk"], it["rng_state"], int(bool(it["forbid_eos"])))
        values = np.zeros((B, self.streams), np.uint32)
        stored = np.zeros((B, self.streams), np.uint32)
        saw = np.zeros(B, np.int32)
        eos_frame = np.zeros(B, np.uint64)
        self.backend._call("mynah_hip_local_frame", self.handle, arr, _sz(B), _np_ptr(values), _np_ptr(stored), _np_ptr(saw),
                           _np_ptr(eos_frame), dev_logits_copy)
        return {"values": values, "stored": stored, "saw_eos": saw, "eos_frame": eos_frame,
                "rng_state": [int(arr[i].rng_state) for i in range(B)]}

    def destroy(self):
        if self.handle:
            self.backend.lib.mynah_hip_local_destroy(self.backend.state, self.handle)
            self.handle = None


class Encoder:
    """mynah_hip_encoder_create + prefill: the dense MFMA text-encoder path."""

    def __init__(self, backend, cfg, weights):
        self.backend, self.cfg = backend, cfg
        L = cfg["layers"]
        self._hold = []

        def per_layer(name):
            if weights.get(name) is None:
                return None
            rows = [backend.keep(weights[name][l]) for l in range(L)]
            arr = _ptr_array(rows)
            self._hold.append(arr)
            return C.cast(arr, _vp)

        def single(name):
            return None if weights.get(name) is None else _np_ptr(backend.keep(weights[name]))

        e = EncoderDesc()
        e.layers, e.width, e.heads, e.head_width, e.ffn_width = L, cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
        e.vocab, e.max_positions = cfg["vocab"], cfg["max_positions"]
        e.tok_table, e.pos_table = single("tok_table"), single("pos_table")
        e.qkv_w, e.o_w, e.up_w, e.down_w = per_layer("qkv"), per_layer("o"), per_layer("up"), per_layer("down")
        e.norm1, e.norm1_bias = per_layer("norm1_g"), per_layer("norm1_b")
        e.norm2, e.norm2_bias = per_layer("norm2_g"), per_layer("norm2_b")
        e.norm_out, e.norm_out_bias = single("norm_out_g"), single("norm_out_b")
        e.causal, e.ffn_kernel = int(bool(cfg.get("causal", False))), int(cfg.get("ffn_kernel", 1))
        e.operands_f32 = int(bool(cfg.get("operands_f32", False)))
        self.desc = e
        h = _vp()
        backend._call("mynah_hip_encoder_create", C.byref(e), C.byref(h))
        self.handle = h

    def prefill(self, ids, dembed, dout):
        ids = np.ascontiguousarray(ids, np.int32)
        self.backend._call("mynah_hip_encoder_prefill", self.handle, _np_ptr(ids), _sz(ids.size), _vp(dembed), _vp(dout))

    def destroy(self):
        if self.handle:
            self.backend.lib.mynah_hip_encoder_destroy(self.backend.state, self.handle)
            self.handle = None


# ---- host-side converters (exposed by the library, used by callers that pre-pack and by tests)
def quantize_weight_int8(lib, w, arith=ARITH_STRICT):
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    q = np.empty((n, k), np.int8)
    s = np.empty(n, np.float32)
    lib.mynah_hip_quantize_weight_int8(_np_ptr(w), n, k, _np_ptr(q), _np_ptr(s), arith)
    return q, s


def quantize_weight_int4(lib, w, arith=ARITH_STRICT):
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    q = np.empty((n, k // 2), np.uint8)
    s = np.empty((n, max(k // 32, 1)), np.float32)
    rc = lib.mynah_hip_quantize_weight_int4(_np_ptr(w), n, k, _np_ptr(q), _np_ptr(s), arith)
    return rc, q, s


def convert_weight_f16(lib, w):
    w = np.ascontiguousarray(w, np.float32)
    out = np.empty(w.shape, np.uint16)
    lib.mynah_hip_convert_weight_f16(_np_ptr(w), w.size, _np_ptr(out))
    return out
