"""TEST INFRASTRUCTURE ONLY: ctypes bindings for the CPU oracle (liboracle.so) and, when built,
the compiled reference (oracle/_ref/libmynah_ref*.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
The shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
F32, INT8, INT4, F16 = 0, 1, 2, 3
STRICT, STOCK = 0, 1

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(dtype=np.int8, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_sz = C.c_size_t


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def build_oracle():
    subprocess.run(["make", "-C", HERE, "oracle"], check=True, stdout=subprocess.DEVNULL)


def _load_oracle():
    path = os.path.join(HERE, "liboracle.so")
    if not os.path.exists(path):
        build_oracle()
    lib = C.CDLL(path)
    lib.orc_quantize_weight_int8.argtypes = [_f32p, _sz, _sz, _i8p, _f32p, C.c_int]
    lib.orc_quantize_weight_int8.restype = None
    lib.orc_quantize_weight_int4.argtypes = [_f32p, _sz, _sz, _u8p, _f32p, C.c_int]
    lib.orc_quantize_weight_int4.restype = C.c_int
    lib.orc_f32_to_f16_array.argtypes = [_f32p, _u16p, _sz]
    lib.orc_f32_to_f16_array.restype = None
    lib.orc_f16_to_f32.argtypes = [C.c_uint16]
    lib.orc_f16_to_f32.restype = C.c_float
    lib.orc_quantize_act_int8.argtypes = [_i8p, _f32p, _sz, C.c_int]
    lib.orc_quantize_act_int8.restype = C.c_float
    lib.orc_matvec_q8.argtypes = [_f32p, C.c_void_p, _i8p, C.c_float, _i8p, _f32p, C.c_void_p, _sz, _sz]
    lib.orc_matvec_q8.restype = None
    lib.orc_matvec_q4.argtypes = [_f32p, C.c_void_p, _i8p, C.c_float, _u8p, _f32p, C.c_void_p, _sz, _sz]
    lib.orc_matvec_q4.restype = None
    lib.orc_matvec_f16.argtypes = [_f32p, _f32p, _u16p, C.c_void_p, _sz, _sz]
    lib.orc_matvec_f16.restype = None
    lib.orc_matvec_f32.argtypes = [_f32p, _f32p, _f32p, C.c_void_p, _sz, _sz]
    lib.orc_matvec_f32.restype = None
    lib.orc_layernorm.argtypes = [_f32p, _f32p, C.c_void_p, _f32p, _sz, _sz, C.c_float]
    lib.orc_layernorm.restype = None
    lib.orc_gelu_scalar.argtypes = [_f32p, _sz]
    lib.orc_gelu_pade.argtypes = [_f32p, _sz]
    lib.orc_softmax.argtypes = [_f32p, _f32p, _sz]
    lib.orc_softmax.restype = C.c_int
    lib.orc_softmax_row_inplace.argtypes = [_f32p, _sz]
    lib.orc_softmax_masked.argtypes = [_f32p, _sz, _sz, _sz]
    lib.orc_residual_add.argtypes = [_f32p, _f32p, _sz]
    lib.orc_argmax_constrained.argtypes = [_f32p, _sz, _sz, _sz, C.c_int, C.POINTER(C.c_uint)]
    lib.orc_argmax_constrained.restype = C.c_int
    lib.orc_self_attention.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, C.c_float, _f32p, _f32p]
    lib.orc_cross_attention.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, C.c_float, _f32p, _f32p]
    lib.orc_decoder_step.restype = C.c_int
    lib.orc_decoder_step_forced.restype = C.c_int
    lib.orc_output_head.restype = None
    lib.orc_encoder_prefill.restype = C.c_int
    lib.orc_gemm_nt.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, C.c_int]
    lib.orc_local_choose.restype = C.c_uint
    lib.orc_local_frame.restype = C.c_int
    return lib


lib = _load_oracle()


class OrcWeight(C.Structure):
    _fields_ = [("qtype", C.c_int), ("n", _sz), ("k", _sz), ("data", C.c_void_p), ("scales", C.c_void_p)]


class OrcDecoder(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn", _sz),
                ("cross_heads", _sz), ("cross_head_width", _sz), ("capacity", _sz),
                ("qkv", C.POINTER(OrcWeight)), ("o_self", C.POINTER(OrcWeight)),
                ("q_cross", C.POINTER(OrcWeight)), ("o_cross", C.POINTER(OrcWeight)),
                ("ffn_up", C.POINTER(OrcWeight)), ("ffn_down", C.POINTER(OrcWeight)),
                ("norm_self_g", C.c_void_p), ("norm_self_b", C.c_void_p),
                ("norm_cross_g", C.c_void_p), ("norm_cross_b", C.c_void_p),
                ("norm_ff_g", C.c_void_p), ("norm_ff_b", C.c_void_p),
                ("norm_out_g", C.c_void_p), ("norm_out_b", C.c_void_p),
                ("position", C.c_void_p), ("act_variant", C.c_int)]


class OrcEncoder(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn", _sz),
                ("vocab", _sz), ("max_positions", _sz),
                ("tok_table", C.c_void_p), ("pos_table", C.c_void_p),
                ("qkv_w", C.c_void_p), ("o_w", C.c_void_p), ("up_w", C.c_void_p), ("down_w", C.c_void_p),
                ("norm1_g", C.c_void_p), ("norm1_b", C.c_void_p), ("norm2_g", C.c_void_p),
                ("norm2_b", C.c_void_p), ("norm_out_g", C.c_void_p), ("norm_out_b", C.c_void_p),
                ("causal", C.c_int), ("ffn_kernel", _sz)]


# ----------------------------------------------------------------------------- numpy-level helpers
def quantize_weight_int8(w, variant=STRICT):
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    q = np.empty((n, k), np.int8)
    s = np.empty(n, np.float32)
    lib.orc_quantize_weight_int8(w, n, k, q, s, variant)
    return q, s


def quantize_weight_int4(w, variant=STRICT):
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    q = np.empty((n, k // 2), np.uint8)
    s = np.empty((n, k // 32), np.float32)
    if lib.orc_quantize_weight_int4(w, n, k, q, s, variant) != 0:
        raise ValueError("int4 needs k % 32 == 0")
    return q, s


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f32_to_f16_array(x.reshape(-1), out.reshape(-1), x.size)
    return out


def quantize_act_int8(x, variant=STRICT):
    x = np.ascontiguousarray(x, dtype=np.float32)
    qx = np.empty(x.shape, np.int8)
    sx = lib.orc_quantize_act_int8(qx, x, x.size, variant)
    return qx, np.float32(sx)


def matvec_q8(qx, sx, q, scales, bias=None):
    n, k = q.shape
    out = np.empty(n, np.float32)
    acc = np.empty(n, np.int32)
    lib.orc_matvec_q8(out, _ptr(acc), qx, float(sx), q, scales, _ptr(bias), n, k)
    return out, acc


def matvec_q4(qx, sx, q, scales, bias=None):
    n, k2 = q.shape
    k = k2 * 2
    out = np.empty(n, np.float32)
    acc = np.empty((n, k // 32), np.int32)
    lib.orc_matvec_q4(out, _ptr(acc), qx, float(sx), q, np.ascontiguousarray(scales), _ptr(bias), n, k)
    return out, acc


def matvec_f16(x, wbits, bias=None):
    n, k = wbits.shape
    out = np.empty(n, np.float32)
    lib.orc_matvec_f16(out, np.ascontiguousarray(x, np.float32), wbits, _ptr(bias), n, k)
    return out


def matvec_f32(x, w, bias=None):
    n, k = w.shape
    out = np.empty(n, np.float32)
    lib.orc_matvec_f32(out, np.ascontiguousarray(x, np.float32), np.ascontiguousarray(w, np.float32), _ptr(bias), n, k)
    return out


def layernorm(x, gain, bias=None, eps=1e-5):
    x = np.ascontiguousarray(x, np.float32)
    x2 = x.reshape(-1, x.shape[-1])
    out = np.empty_like(x2)
    lib.orc_layernorm(x2, np.ascontiguousarray(gain, np.float32), _ptr(bias), out, x2.shape[0], x2.shape[1], eps)
    return out.reshape(x.shape)


def gelu_scalar(x):
    y = np.array(x, dtype=np.float32, copy=True).reshape(-1)
    lib.orc_gelu_scalar(y, y.size)
    return y.reshape(np.shape(x))


def gelu_pade(x):
    y = np.array(x, dtype=np.float32, copy=True).reshape(-1)
    lib.orc_gelu_pade(y, y.size)
    return y.reshape(np.shape(x))


def softmax(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    rc = lib.orc_softmax(x, out, x.size)
    return rc, out


def softmax_row_inplace(x):
    y = np.array(x, dtype=np.float32, copy=True)
    lib.orc_softmax_row_inplace(y, y.size)
    return y


def softmax_masked(x, valid):
    y = np.array(x, dtype=np.float32, copy=True)
    lib.orc_softmax_masked(y, y.shape[0], y.shape[1], valid)
    return y


def argmax_constrained(logits, codebook_size, eos_id, allow_eos):
    out = C.c_uint(0)
    rc = lib.orc_argmax_constrained(np.ascontiguousarray(logits, np.float32), logits.size, codebook_size, eos_id,
                                    int(allow_eos), C.byref(out))
    return rc, out.value


def self_attention(qkv, k_cache, v_cache, position, stride, valid, heads, hw, scale):
    out = np.empty(heads * hw, np.float32)
    scratch = np.empty(valid + 1, np.float32)
    lib.orc_self_attention(qkv, k_cache, v_cache, position, stride, valid, heads, hw, scale, out, scratch)
    return out


def cross_attention(q, k_cache, v_cache, valid, stride, heads, hw, scale):
    out = np.empty(heads * hw, np.float32)
    scratch = np.empty(valid + 1, np.float32)
    lib.orc_cross_attention(q, k_cache, v_cache, valid, stride, heads, hw, scale, out, scratch)
    return out


class PackedWeight:
    """A weight matrix converted once on the host; keeps the numpy arrays alive for ctypes."""

    def __init__(self, w, qtype, variant=STRICT):
        w = np.ascontiguousarray(w, np.float32)
        self.qtype, self.n, self.k = qtype, w.shape[0], w.shape[1]
        self.scales = None
        if qtype == F32:
            self.data = w
        elif qtype == F16:
            self.data = f32_to_f16_bits(w)
        elif qtype == INT8:
            self.data, self.scales = quantize_weight_int8(w, variant)
        elif qtype == INT4:
            self.data, self.scales = quantize_weight_int4(w, variant)
        else:
            raise ValueError(qtype)

    def struct(self):
        return OrcWeight(self.qtype, self.n, self.k, _ptr(self.data), _ptr(self.scales))

    def nbytes(self):
        return self.data.nbytes + (0 if self.scales is None else self.scales.nbytes)


def linear(pw, x, bias=None, act_variant=STRICT):
    out = np.empty(pw.n, np.float32)
    s = pw.struct()
    lib.orc_linear(C.byref(s), _ptr(np.ascontiguousarray(x, np.float32)), _ptr(out), _ptr(bias), act_variant)
    return out


class Decoder:
    """Synthetic decoder stack: holds packed weights and runs orc_decoder_step."""

    def __init__(self, cfg, weights, qtype, variant=STRICT):
        # weights: dict of per-layer f32 arrays (see tests/synth.py)
        self.cfg = cfg
        L = cfg["layers"]
        has_cross = cfg["cross_heads"] * cfg["cross_head_width"] != 0
        self.packed = {name: [PackedWeight(weights[name][l], qtype if (has_cross or "cross" not in name) else F32, variant)
                              for l in range(L)]
                       for name in ("qkv", "o_self", "q_cross", "o_cross", "ffn_up", "ffn_down")}
        self._arrays = {name: (OrcWeight * L)(*[p.struct() for p in self.packed[name]]) for name in self.packed}
        self.norms = {k: (None if weights.get(k) is None else np.ascontiguousarray(weights[k], np.float32))
                      for k in ("norm_self_g", "norm_self_b", "norm_cross_g", "norm_cross_b", "norm_ff_g",
                                "norm_ff_b", "norm_out_g", "norm_out_b", "position")}
        d = OrcDecoder()
        d.layers, d.width, d.heads, d.head_width, d.ffn = L, cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
        d.cross_heads, d.cross_head_width, d.capacity = cfg["cross_heads"], cfg["cross_head_width"], cfg["capacity"]
        for name in self._arrays:
            setattr(d, name, self._arrays[name])
        for k, v in self.norms.items():
            setattr(d, k, _ptr(v))
        d.act_variant = variant
        self.d = d

    def step(self, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs):
        B = len(inputs)
        outs = [np.empty(self.cfg["width"], np.float32) for _ in range(B)]
        pp = C.c_void_p * B
        szs = _sz * B
        rc = lib.orc_decoder_step(C.byref(self.d), _sz(B), pp(*[_ptr(a) for a in self_k]), pp(*[_ptr(a) for a in self_v]),
                                  pp(*[_ptr(a) for a in cross_k]), pp(*[_ptr(a) for a in cross_v]),
                                  szs(*lengths), szs(*memory_lengths), pp(*[_ptr(a) for a in inputs]),
                                  pp(*[_ptr(a) for a in outs]))
        if rc != 0:
            raise RuntimeError("decoder cache capacity exceeded")
        return outs

    def step_forced(self, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs, qx=None, sx=None):
        """The same step with stream 0's int8 activations taken from the caller: qx [layers, 6, ffn] int8 and sx [layers, 6] f32,
        one slot per projection (qkv, o_self, q_cross, o_cross, ffn_up, ffn_down); None: nothing forced.  Returns (outs,
        elements in which qx differs from the oracle's own quantisation, the largest such difference in int8 steps, and the
        activations the oracle quantised itself, in the same layout: (own_qx, own_sx))."""
        B = len(inputs)
        L, ffn = self.cfg["layers"], self.cfg["ffn"]
        if qx is not None:
            qx = np.ascontiguousarray(qx, np.int8)
            sx = np.ascontiguousarray(sx, np.float32)
            assert qx.shape == (L, 6, ffn) and sx.shape == (L, 6)
        own_qx, own_sx = np.zeros((L, 6, ffn), np.int8), np.zeros((L, 6), np.float32)
        outs = [np.empty(self.cfg["width"], np.float32) for _ in range(B)]
        pp = C.c_void_p * B
        szs = _sz * B
        counts = (_sz * 2)(0, 0)
        rc = lib.orc_decoder_step_forced(C.byref(self.d), _sz(B), pp(*[_ptr(a) for a in self_k]), pp(*[_ptr(a) for a in self_v]),
                                         pp(*[_ptr(a) for a in cross_k]), pp(*[_ptr(a) for a in cross_v]),
                                         szs(*lengths), szs(*memory_lengths), pp(*[_ptr(a) for a in inputs]),
                                         pp(*[_ptr(a) for a in outs]), _ptr(qx), _ptr(sx), counts, _ptr(own_qx), _ptr(own_sx))
        if rc != 0:
            raise RuntimeError("decoder cache capacity exceeded")
        return outs, int(counts[0]), int(counts[1]), (own_qx, own_sx)


def output_head(pw, hidden, heads_out, vocab, bias=None, act_variant=STRICT):
    logits = np.empty(heads_out * vocab, np.float32)
    probs = np.empty(heads_out * vocab, np.float32)
    s = pw.struct()
    lib.orc_output_head(C.byref(s), _ptr(bias), _ptr(np.ascontiguousarray(hidden, np.float32)), _sz(heads_out),
                        _sz(vocab), _ptr(logits), _ptr(probs), C.c_int(act_variant))
    return logits, probs


def encoder_prefill(cfg, w, ids, threads=8):
    """w: dict with f16-bit tables/weights (uint16) and f32 norms.  cfg["causal"] (default False) masks row t to rows
    [0, t]; cfg["ffn_kernel"] (default 1) > 1 takes up_w [ffn, width, k] / down_w [width, ffn, k] of the causal conv FFN.
    Returns (embed_bits, out)."""
    e = OrcEncoder()
    e.causal = 1 if cfg.get("causal") else 0
    e.ffn_kernel = int(cfg.get("ffn_kernel", 1))
    e.layers, e.width, e.heads, e.head_width, e.ffn = cfg["layers"], cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
    e.vocab, e.max_positions = cfg["vocab"], cfg["max_positions"]
    keep = []
    for name in ("tok_table", "pos_table", "qkv_w", "o_w", "up_w", "down_w"):
        a = np.ascontiguousarray(w[name], np.uint16)
        keep.append(a)
        setattr(e, name, _ptr(a))
    for name in ("norm1_g", "norm1_b", "norm2_g", "norm2_b", "norm_out_g", "norm_out_b"):
        a = None if w.get(name) is None else np.ascontiguousarray(w[name], np.float32)
        keep.append(a)
        setattr(e, name, _ptr(a))
    ids = np.ascontiguousarray(ids, np.int32)
    T = ids.size
    embed = np.empty((T, cfg["width"]), np.uint16)
    out = np.empty((T, cfg["width"]), np.float32)
    rc = lib.orc_encoder_prefill(C.byref(e), _ptr(ids), _sz(T), _ptr(embed), _ptr(out), C.c_int(threads))
    if rc != 0:
        raise ValueError("invalid ids or length")
    return embed, out


# ----------------------------------------------------------------------------- local transformer frame
class OrcLocalItem(C.Structure):
    _fields_ = [("temperature", C.c_float), ("topk", _sz), ("rng_state", C.c_uint64), ("forbid_eos", C.c_int)]


class OrcLocal(C.Structure):
    _fields_ = [("stack", C.POINTER(OrcDecoder)), ("streams", _sz), ("vocab", _sz), ("codebook_size", _sz), ("eos_id", _sz),
                ("codebook_count", _sz), ("projection", C.POINTER(OrcWeight)), ("projection_bias", C.c_void_p),
                ("audio_table", C.c_void_p)]


def local_choose(logits, codebook_size, eos_id, temperature, topk, rng_state, forbid_eos):
    """One token from one row of logits.  Returns (value, greedy, new_rng_state, masked_logits)."""
    lg = np.array(logits, dtype=np.float32, copy=True)
    item = OrcLocalItem(float(temperature), int(topk), int(rng_state), int(bool(forbid_eos)))
    greedy = C.c_uint(0)
    n = max(1, min(int(topk), lg.size))
    top_i = (_sz * n)()
    top_v = (C.c_float * n)()
    value = lib.orc_local_choose(_ptr(lg), _sz(lg.size), _sz(codebook_size), _sz(eos_id), C.byref(item), C.byref(greedy), top_i, top_v)
    return int(value), int(greedy.value), int(item.rng_state), lg


class LocalFrame:
    """orc_local_frame on a local stack (an orc.Decoder without cross attention or final norm), per-stream projections
    (PackedWeight list), optional biases and f32 audio tables."""

    def __init__(self, stack, projections, biases, audio_tables, codebook_size, eos_id, codebook_count):
        self.stack, self.projections = stack, projections
        S = len(projections)
        self.S, self.vocab = S, projections[0].struct().n
        self._proj = (OrcWeight * S)(*[p.struct() for p in projections])
        self._bias_arrays = None if biases is None else [np.ascontiguousarray(b, np.float32) for b in biases]
        self._tables = [np.ascontiguousarray(t, np.float32) for t in audio_tables]
        pp = C.c_void_p * S
        self._bias_ptrs = None if biases is None else pp(*[_ptr(b) for b in self._bias_arrays])
        self._table_ptrs = pp(*[_ptr(t) for t in self._tables])
        L = OrcLocal()
        L.stack = C.pointer(stack.d)
        L.streams, L.vocab, L.codebook_size, L.eos_id, L.codebook_count = S, self.vocab, codebook_size, eos_id, codebook_count
        L.projection = self._proj
        L.projection_bias = None if biases is None else C.cast(self._bias_ptrs, C.c_void_p)
        L.audio_table = C.cast(self._table_ptrs, C.c_void_p)
        self.L = L

    def frame(self, decoder_last, items, want_logits=False):
        """items: list of dicts temperature/topk/rng_state/forbid_eos.  Returns dict with values, stored, saw_eos, eos_frame,
        rng_state (advanced) and optionally logits [batch, streams, vocab]."""
        B = len(decoder_last)
        cfg = self.stack.cfg
        arr = (OrcLocalItem * B)(*[OrcLocalItem(float(i["temperature"]), int(i["topk"]), int(i["rng_state"]), int(bool(i["forbid_eos"])))
                                   for i in items])
        ks = [np.zeros((cfg["layers"], cfg["capacity"], cfg["width"]), np.float32) for _ in range(B)]
        vs = [np.zeros((cfg["layers"], cfg["capacity"], cfg["width"]), np.float32) for _ in range(B)]
        rows = [np.ascontiguousarray(r, np.float32) for r in decoder_last]
        pp = C.c_void_p * B
        values = np.zeros((B, self.S), np.uint32)
        stored = np.zeros((B, self.S), np.uint32)
        saw = np.zeros(B, np.int32)
        eosf = np.zeros(B, np.uint64)
        logits = np.zeros((B, self.S, self.vocab), np.float32) if want_logits else None
        rc = lib.orc_local_frame(C.byref(self.L), _sz(B), pp(*[_ptr(r) for r in rows]), arr, pp(*[_ptr(a) for a in ks]),
                                 pp(*[_ptr(a) for a in vs]), _ptr(values), _ptr(stored), _ptr(saw), _ptr(eosf), _ptr(logits))
        if rc != 0:
            raise RuntimeError("orc_local_frame failed")
        return {"values": values, "stored": stored, "saw_eos": saw, "eos_frame": eosf,
                "rng_state": [int(arr[b].rng_state) for b in range(B)], "logits": logits}


# ----------------------------------------------------------------------------- compiled reference
class RefDecoderDesc(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn", _sz), ("xw", _sz),
                ("capacity", _sz),
                ("norm_self", C.c_void_p), ("norm_xq", C.c_void_p), ("norm_ff", C.c_void_p),
                ("qkv_w", C.c_void_p), ("o_w", C.c_void_p), ("qx_w", C.c_void_p), ("ox_w", C.c_void_p),
                ("up_w", C.c_void_p), ("down_w", C.c_void_p), ("norm_out", C.c_void_p), ("position", C.c_void_p)]


def ref_available(strict=False):
    return os.path.exists(os.path.join(HERE, "_ref", "libmynah_ref_strict.so" if strict else "libmynah_ref.so"))


_ref_cache = {}


def load_ref(strict=False):
    """The reference's own CPU code, compiled from the reference tree by oracle/Makefile `ref`."""
    key = bool(strict)
    if key in _ref_cache:
        return _ref_cache[key]
    path = os.path.join(HERE, "_ref", "libmynah_ref_strict.so" if strict else "libmynah_ref.so")
    r = C.CDLL(path)
    r.ref_quantize_weight_int8.argtypes = [_f32p, _sz, _sz, _i8p, _f32p]
    r.ref_quantize_weight_int8.restype = None
    r.ref_quantize_weight_int4.argtypes = [_f32p, _sz, _sz, _u8p, _f32p]
    r.ref_quantize_weight_int4.restype = None
    r.ref_quantize_act_int8.argtypes = [_i8p, _f32p, _sz]
    r.ref_quantize_act_int8.restype = C.c_float
    r.ref_matvec_q8.argtypes = [_f32p, _i8p, C.c_float, _i8p, _f32p, C.c_void_p, _sz, _sz]
    r.ref_matvec_q8.restype = None
    r.ref_matvec_q4.argtypes = [_f32p, _i8p, C.c_float, _u8p, _f32p, C.c_void_p, _sz, _sz]
    r.ref_matvec_q4.restype = None
    r.ref_matvec_rows_blocked.argtypes = [_f32p, _i8p, C.c_float, C.c_void_p, _f32p, C.c_void_p, _sz, _sz, C.c_int]
    r.ref_matvec_q_rows.argtypes = [_f32p, _i8p, C.c_float, C.c_void_p, _f32p, C.c_void_p, _sz, _sz, C.c_int]
    r.ref_num_threads.restype = C.c_int
    r.mynah_qmat_self_test.argtypes = [C.c_char_p, _sz]
    r.mynah_qmat_self_test.restype = C.c_int
    r.mynah_kernels_self_test.argtypes = [C.c_char_p, _sz]
    r.mynah_kernels_self_test.restype = C.c_int
    r.mynah_layernorm_f32.argtypes = [_f32p, _f32p, C.c_void_p, _f32p, _sz, _sz, C.c_float]
    r.mynah_layernorm_f32.restype = None
    r.mynah_gelu_f32_scalar.argtypes = [_f32p, _sz]
    r.mynah_gelu_f32.argtypes = [_f32p, _sz]
    r.mynah_softmax_f32.argtypes = [_f32p, _f32p, _sz]
    r.mynah_softmax_f32.restype = C.c_int
    r.mynah_matvec_bias_f32.argtypes = [_f32p, _f32p, C.c_void_p, _f32p, _sz, _sz]
    r.ref_softmax_row_inplace.argtypes = [_f32p, _sz]
    r.ref_decoder_new.argtypes = [C.POINTER(RefDecoderDesc), C.c_int, _sz, _sz]
    r.ref_decoder_new.restype = C.c_void_p
    r.ref_decoder_free.argtypes = [C.c_void_p]
    r.ref_decoder_step.restype = C.c_int
    _ref_cache[key] = r
    return r


class RefLocalDesc(C.Structure):
    _fields_ = [("layers", _sz), ("width", _sz), ("heads", _sz), ("head_width", _sz), ("ffn", _sz), ("capacity", _sz),
                ("norm_self", C.c_void_p), ("norm_ff", C.c_void_p), ("qkv_w", C.c_void_p), ("o_w", C.c_void_p),
                ("up_w", C.c_void_p), ("down_w", C.c_void_p), ("position", C.c_void_p)]


class RefLocal:
    """The reference's local_step_batch (src/graph.c:1234-1343) on synthetic weights."""

    def __init__(self, cfg, weights, qtype, batch, strict=False):
        self.r = load_ref(strict)
        self.r.ref_local_new.argtypes = [C.POINTER(RefLocalDesc), C.c_int, _sz]
        self.r.ref_local_new.restype = C.c_void_p
        self.r.ref_local_free.argtypes = [C.c_void_p]
        self.r.ref_local_step.restype = C.c_int
        self.cfg, self.batch = cfg, batch
        self.keep = {}
        d = RefLocalDesc()
        d.layers, d.width, d.heads, d.head_width, d.ffn, d.capacity = (cfg["layers"], cfg["width"], cfg["heads"], cfg["head_width"],
                                                                       cfg["ffn"], cfg["capacity"])
        names = {"norm_self": "norm_self_g", "norm_ff": "norm_ff_g", "qkv_w": "qkv", "o_w": "o_self", "up_w": "ffn_up",
                 "down_w": "ffn_down", "position": "position"}
        for field, key in names.items():
            a = np.ascontiguousarray(weights[key], np.float32)
            self.keep[field] = a
            setattr(d, field, _ptr(a))
        self.h = self.r.ref_local_new(C.byref(d), qtype, batch)
        if not self.h:
            raise RuntimeError("ref_local_new failed")

    def step(self, ks, vs, lengths, inputs):
        B = self.batch
        outs = [np.empty(self.cfg["width"], np.float32) for _ in range(B)]
        pp = C.c_void_p * B
        lens = (_sz * B)(*lengths)
        err = C.create_string_buffer(256)
        rc = self.r.ref_local_step(C.c_void_p(self.h), pp(*[_ptr(a) for a in ks]), pp(*[_ptr(a) for a in vs]), lens,
                                   pp(*[_ptr(a) for a in inputs]), pp(*[_ptr(a) for a in outs]), err, _sz(256))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return outs, list(lens)

    def use_hip(self, library_path):
        """Hands the reference engine this repository's library as its backend (oracle/ref_shim_backend.c)."""
        err = C.create_string_buffer(512)
        self.r.ref_local_use_hip.restype = C.c_int
        if self.r.ref_local_use_hip(C.c_void_p(self.h), os.fsencode(library_path), err, _sz(512)) != 0:
            raise RuntimeError(err.value.decode())
        self.device = True

    def device_step(self, slot, length, x):
        """The reference's local_step_device (src/graph.c:1106-1158) for one slot; returns (row, new length)."""
        out = np.empty(self.cfg["width"], np.float32)
        x = np.ascontiguousarray(x, np.float32)
        n = _sz(length)
        err = C.create_string_buffer(512)
        self.r.ref_local_device_step.restype = C.c_int
        rc = self.r.ref_local_device_step(C.c_void_p(self.h), _sz(slot), C.byref(n), _ptr(x), _ptr(out), err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return out, int(n.value)

    def hip_frame(self, library_path, projections, biases, audio_tables, vocab, codebook_size, eos_id, codebook_count, items,
                  code_stride, raw_offset):
        """One device frame through the integration text's hip_sample_local_frame_batch (oracle/integration_batched.inc) on the
        reference's own local_batch_item.  items: dicts with row, temperature, topk, rng_state (None = greedy),
        generated_raw_length, min_raw_length.  Returns (codes [count, codebook_count, code_stride], saw_eos, eos_frame,
        rng states)."""
        streams, count = len(projections), len(items)
        keep = [np.ascontiguousarray(a, np.float32) for a in projections]
        keep_b = [None if biases is None or b is None else np.ascontiguousarray(b, np.float32) for b in (biases or [None] * streams)]
        keep_t = [np.ascontiguousarray(a, np.float32) for a in audio_tables]
        self._frame_keep = (keep, keep_b, keep_t)        # the device weight cache keys on these addresses
        pp, pc = C.c_void_p * streams, C.c_void_p * count
        rows = [np.ascontiguousarray(it["row"], np.float32) for it in items]
        temperature = (C.c_float * count)(*[it["temperature"] for it in items])
        topk = (C.c_uint * count)(*[it["topk"] for it in items])
        rng = (C.c_uint64 * count)(*[it["rng_state"] or 0 for it in items])
        has_rng = (C.c_int * count)(*[0 if it["rng_state"] is None else 1 for it in items])
        generated = (_sz * count)(*[it["generated_raw_length"] for it in items])
        minimum = (_sz * count)(*[it["min_raw_length"] for it in items])
        codes = np.full((count, codebook_count, code_stride), 0xffffffff, np.uint32)
        saw = (C.c_int * count)()
        eos_frame = (_sz * count)()
        err = C.create_string_buffer(512)
        self.r.ref_local_hip_frame.restype = C.c_int
        rc = self.r.ref_local_hip_frame(C.c_void_p(self.h), os.fsencode(library_path), _sz(streams), _sz(vocab), _sz(codebook_size),
                                        _sz(eos_id), _sz(codebook_count), pp(*[_ptr(a) for a in keep]),
                                        None if biases is None else pp(*[_ptr(a) for a in keep_b]), pp(*[_ptr(a) for a in keep_t]),
                                        _sz(count), pc(*[_ptr(a) for a in rows]), temperature, topk, rng, has_rng, generated, minimum,
                                        _ptr(codes), _sz(code_stride), _sz(raw_offset), saw, eos_frame, err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        self.hip_batched = True
        return codes, list(saw), list(eos_frame), list(rng)

    def close(self):
        if self.h:
            if getattr(self, "hip_batched", False):
                self.r.ref_local_hip_batch_release(C.c_void_p(self.h))
            if getattr(self, "device", False):
                self.r.ref_local_release(C.c_void_p(self.h))
            self.r.ref_local_free(C.c_void_p(self.h))
            self.h = None


class RefDecoder:
    """The reference's decoder_step_batch on synthetic weights (gain-only LayerNorm, one cross head)."""

    def __init__(self, cfg, weights, qtype, batch, max_memory, strict=False):
        assert cfg["cross_heads"] == 1, "the reference's decode step has a single cross-attention head"
        self.r = load_ref(strict)
        self.cfg, self.batch = cfg, batch
        self.keep = {}
        d = RefDecoderDesc()
        d.layers, d.width, d.heads, d.head_width, d.ffn = cfg["layers"], cfg["width"], cfg["heads"], cfg["head_width"], cfg["ffn"]
        d.xw, d.capacity = cfg["cross_head_width"], cfg["capacity"]
        names = {"norm_self": "norm_self_g", "norm_xq": "norm_cross_g", "norm_ff": "norm_ff_g", "qkv_w": "qkv",
                 "o_w": "o_self", "qx_w": "q_cross", "ox_w": "o_cross", "up_w": "ffn_up", "down_w": "ffn_down",
                 "norm_out": "norm_out_g", "position": "position"}
        for field, key in names.items():
            a = np.ascontiguousarray(weights[key], np.float32)
            self.keep[field] = a
            setattr(d, field, _ptr(a))
        self.desc = d
        self.h = self.r.ref_decoder_new(C.byref(d), qtype, batch, max_memory)
        if not self.h:
            raise RuntimeError("ref_decoder_new failed")

    def step(self, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs):
        B = self.batch
        outs = [np.empty(self.cfg["width"], np.float32) for _ in range(B)]
        pp = C.c_void_p * B
        szs = _sz * B
        lens = szs(*lengths)
        err = C.create_string_buffer(256)
        rc = self.r.ref_decoder_step(C.c_void_p(self.h), pp(*[_ptr(a) for a in self_k]), pp(*[_ptr(a) for a in self_v]),
                                     pp(*[_ptr(a) for a in cross_k]), pp(*[_ptr(a) for a in cross_v]), lens,
                                     szs(*memory_lengths), pp(*[_ptr(a) for a in inputs]),
                                     pp(*[_ptr(a) for a in outs]), err, _sz(256))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return outs, list(lens)

    def use_hip(self, library_path):
        """Hands the reference engine this repository's library as its backend (oracle/ref_shim_backend.c)."""
        err = C.create_string_buffer(512)
        self.r.ref_decoder_use_hip.restype = C.c_int
        if self.r.ref_decoder_use_hip(C.c_void_p(self.h), os.fsencode(library_path), err, _sz(512)) != 0:
            raise RuntimeError(err.value.decode())
        self.device = True

    def self_test(self):
        err = C.create_string_buffer(512)
        self.r.ref_decoder_self_test.restype = C.c_int
        if self.r.ref_decoder_self_test(C.c_void_p(self.h), err, _sz(512)) != 0:
            raise RuntimeError(err.value.decode())

    def run_one(self, slot, self_k, self_v, cross_k, cross_v, length, memory_length, x):
        """The reference's decoder_run with one row (src/graph.c:3292-3654); returns (row, new length, resident)."""
        out = np.empty(self.cfg["width"], np.float32)
        x = np.ascontiguousarray(x, np.float32)
        n = _sz(length)
        resident = C.c_int(0)
        err = C.create_string_buffer(512)
        self.r.ref_decoder_run_one.restype = C.c_int
        rc = self.r.ref_decoder_run_one(C.c_void_p(self.h), _sz(slot), _ptr(self_k), _ptr(self_v), _ptr(cross_k), _ptr(cross_v),
                                        C.byref(n), _sz(memory_length), _ptr(x), _ptr(out), C.byref(resident), err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return out, int(n.value), bool(resident.value)

    def run_rows(self, slot, self_k, self_v, cross_k, cross_v, length, memory_length, rows):
        """The reference's decoder_run with several rows, its context prefill (src/graph.c:3506-3654): the host caches are
        appended in place; returns (the last row after the final norm, new length)."""
        rows = np.ascontiguousarray(rows, np.float32)
        out = np.empty(self.cfg["width"], np.float32)
        n = _sz(length)
        err = C.create_string_buffer(512)
        self.r.ref_decoder_run_rows.restype = C.c_int
        rc = self.r.ref_decoder_run_rows(C.c_void_p(self.h), _sz(slot), _ptr(self_k), _ptr(self_v), _ptr(cross_k), _ptr(cross_v),
                                         C.byref(n), _sz(memory_length), _ptr(rows), _sz(rows.shape[0]), _ptr(out), err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        return out, int(n.value)

    def device_kv_row(self, slot, layer, row):
        k = np.empty(self.cfg["width"], np.float32)
        v = np.empty(self.cfg["width"], np.float32)
        err = C.create_string_buffer(512)
        self.r.ref_decoder_read_device_kv.restype = C.c_int
        if self.r.ref_decoder_read_device_kv(C.c_void_p(self.h), _sz(slot), _sz(layer), _sz(row), _ptr(k), _ptr(v), err,
                                             _sz(512)) != 0:
            raise RuntimeError(err.value.decode() or "no device caches")
        return k, v

    def hip_step_batch(self, library_path, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs):
        """One batched device step through the integration text's hip_decoder_step_batch (oracle/integration_batched.inc) on
        the reference's own decoder_cache slots; returns (rows, new lengths)."""
        B = self.batch
        outs = [np.empty(self.cfg["width"], np.float32) for _ in range(B)]
        pp, szs = C.c_void_p * B, _sz * B
        lens = szs(*lengths)
        err = C.create_string_buffer(512)
        self.r.ref_decoder_hip_step_batch.restype = C.c_int
        rc = self.r.ref_decoder_hip_step_batch(C.c_void_p(self.h), os.fsencode(library_path), pp(*[_ptr(a) for a in self_k]),
                                               pp(*[_ptr(a) for a in self_v]), pp(*[_ptr(a) for a in cross_k]),
                                               pp(*[_ptr(a) for a in cross_v]), lens, szs(*memory_lengths),
                                               pp(*[_ptr(np.ascontiguousarray(a, np.float32)) for a in inputs]),
                                               pp(*[_ptr(a) for a in outs]), err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        self.hip_batched = True
        return outs, list(lens)

    def close(self):
        if self.h:
            if getattr(self, "hip_batched", False):
                self.r.ref_decoder_hip_batch_release(C.c_void_p(self.h))
            if getattr(self, "device", False):
                self.r.ref_decoder_release(C.c_void_p(self.h))
            self.r.ref_decoder_free(C.c_void_p(self.h))
            self.h = None


# ----------------------------------------------------------------------------- codec operators
_vp = C.c_void_p
lib.orc_conv1d_causal.argtypes = [_vp, _vp, _sz, _sz, _sz, _sz, _sz, _vp, _vp]
lib.orc_conv1d_causal.restype = None
lib.orc_conv_transpose_causal.argtypes = [_vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _sz, _vp, _vp]
lib.orc_conv_transpose_causal.restype = None
lib.orc_snake.argtypes = [_vp, _vp, _sz, _sz, _sz]
lib.orc_snake.restype = None


def conv1d_causal(x, weight, bias, dilation):
    """x [in, length], weight [out, in, kernel], bias [out] or None -> [out, length]."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(weight, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    out = np.zeros((w.shape[0], x.shape[1]), np.float32)
    lib.orc_conv1d_causal(_ptr(x), _ptr(out), x.shape[0], w.shape[0], x.shape[1], w.shape[2], dilation, _ptr(w), _ptr(b))
    return out


def conv_transpose_causal(x, weight, bias, stride, groups, output_length=None):
    """x [in, length], weight [in, out / groups, kernel] -> [out, output_length] (default: length * stride)."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(weight, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    out_ch = w.shape[1] * groups
    kernel = w.shape[2]
    if output_length is None:
        output_length = (x.shape[1] - 1) * stride + kernel - (kernel - stride)
    out = np.zeros((out_ch, output_length), np.float32)
    lib.orc_conv_transpose_causal(_ptr(x), _ptr(out), x.shape[0], out_ch, x.shape[1], output_length, kernel, stride, groups, _ptr(w),
                                  _ptr(b))
    return out


def snake(x, alpha, snake_channels):
    out = np.array(x, np.float32, copy=True)
    a = np.ascontiguousarray(alpha, np.float32)
    lib.orc_snake(_ptr(out), _ptr(a), out.shape[0], out.shape[1], snake_channels)
    return out


def write_safetensors(path, tensors):
    """A minimal safetensors file (8-byte little-endian header length, JSON header, raw little-endian f32 data) holding the
    given name -> float32 array map: what the compiled reference's weight loader opens for the codec operators."""
    import json
    import struct
    header, blobs, offset = {}, [], 0
    for name, value in tensors.items():
        a = np.ascontiguousarray(value, "<f4")
        header[name] = {"dtype": "F32", "shape": list(a.shape), "data_offsets": [offset, offset + a.nbytes]}
        blobs.append(a.tobytes())
        offset += a.nbytes
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * ((8 - len(text) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for blob in blobs:
            f.write(blob)


def ref_transformer_stack(cfg, w, states, kernel, strict=False, workdir=None, hip_library=None):
    """The compiled reference's transformer_stack (src/graph.c:634-711) exactly as encode_text calls it (:738-740):
    causal self-attention, gain-only LayerNorm, FFN with `kernel` taps, final norm when w["norm_out_g"] is given.
    w holds f32 arrays: pos_table [P, width], qkv [L, 3w, w], o [L, w, w], up [L, ffn, w(, kernel)],
    down [L, w, ffn(, kernel)], norm1_g / norm2_g [L, w].  states: the gathered token rows [T, width].
    hip_library: the same function on the reference's backend struct filled with that library's entry points."""
    import tempfile
    r = load_ref(strict)
    fp = C.POINTER(C.c_float)
    r.ref_transformer_stack_on.argtypes = [C.c_char_p, C.c_char_p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int, fp, fp, C.c_char_p, _sz]
    r.ref_transformer_stack_on.restype = C.c_int
    L, width, ffn = cfg["layers"], cfg["width"], cfg["ffn"]
    tensors = {"encoder.position_embeddings.weight": w["pos_table"]}
    for l in range(L):
        base = "encoder.layers.%d." % l
        tensors[base + "norm_self.weight"] = w["norm1_g"][l]
        tensors[base + "self_attention.qkv_net.weight"] = w["qkv"][l]
        tensors[base + "self_attention.o_net.weight"] = w["o"][l]
        tensors[base + "norm_pos_ff.weight"] = w["norm2_g"][l]
        tensors[base + "pos_ff.proj.conv.weight"] = np.asarray(w["up"][l]).reshape(ffn, width, kernel)
        tensors[base + "pos_ff.o_net.conv.weight"] = np.asarray(w["down"][l]).reshape(width, ffn, kernel)
    final = w.get("norm_out_g") is not None
    if final:
        tensors["encoder.norm_out.weight"] = w["norm_out_g"]
    states = np.ascontiguousarray(states, np.float32)
    T = states.shape[0]
    out = np.empty((T, width), np.float32)
    err = C.create_string_buffer(512)
    with tempfile.TemporaryDirectory(dir=workdir) as tmp:
        path = os.path.join(tmp, "encoder.safetensors")
        write_safetensors(path, tensors)
        rc = r.ref_transformer_stack_on(os.fsencode(path), None if hip_library is None else os.fsencode(hip_library), L, T, width, ffn,
                                        cfg["heads"], kernel, 1 if final else 0, states.ctypes.data_as(fp), out.ctypes.data_as(fp), err, 512)
    if rc != 0:
        raise RuntimeError(err.value.decode())
    return out


def ref_codec(strict=False):
    r = load_ref(strict)
    fp = C.POINTER(C.c_float)
    r.ref_conv1d.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, fp, fp, _sz, _sz, _sz, _sz, _sz, C.c_char_p, _sz]
    r.ref_conv1d.restype = C.c_int
    r.ref_conv_transpose.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, fp, fp, _sz, _sz, _sz, _sz, _sz, _sz, C.c_char_p, _sz]
    r.ref_conv_transpose.restype = C.c_int
    r.ref_snake.argtypes = [fp, fp, _sz, _sz, _sz]
    r.ref_snake.restype = C.c_int
    return r


class RefCodecEngine:
    """The reference's decode_codec (src/graph.c:2640-2790) on a safetensors file of synthetic codec weights: with
    hip_library=None its CPU sequence on the CPU backend, otherwise decode_codec_resident on that library."""

    def __init__(self, weights_path, hip_library=None, strict=False):
        self.r = load_ref(strict)
        self.r.ref_codec_engine_new.restype = C.c_void_p
        self.r.ref_codec_engine_new.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, _sz]
        self.r.ref_codec_engine_free.argtypes = [C.c_void_p]
        self.r.ref_codec_engine_decode.restype = C.c_int
        err = C.create_string_buffer(512)
        self.h = self.r.ref_codec_engine_new(os.fsencode(weights_path), None if hip_library is None else os.fsencode(hip_library),
                                             err, 512)
        if not self.h:
            raise RuntimeError(err.value.decode())

    def decode(self, codes):
        codes = np.ascontiguousarray(codes, np.uint32)
        assert codes.ndim == 2 and codes.shape[0] == 8
        raw = codes.shape[1]
        samples = np.empty(raw * 1024, np.float32)
        count, resident = _sz(0), C.c_int(0)
        err = C.create_string_buffer(512)
        rc = self.r.ref_codec_engine_decode(C.c_void_p(self.h), _ptr(codes), _sz(raw), _ptr(samples), _sz(samples.size),
                                            C.byref(count), C.byref(resident), err, _sz(512))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        assert count.value == samples.size
        return samples, bool(resident.value)

    def close(self):
        if self.h:
            self.r.ref_codec_engine_free(C.c_void_p(self.h))
            self.h = None


def codec_weights(seed=11):
    """Synthetic NanoCodec decoder weights under the tensor names the reference's codec decode looks up
    (src/graph.c:2345-2400,2444-2480,2547-2617): 32 -> 864 pre-conv (7 taps), five stages of half-snake alpha, grouped
    transposed conv (rates 8 8 4 2 2, one group per output channel) and 3 x 3 residual blocks (taps 3 / 7 / 11), the post
    snake alpha and the 1-channel post-conv (3 taps)."""
    rng = np.random.default_rng(seed)
    t = {}

    def conv(prefix, out_ch, in_ch, k):
        t[prefix + ".weight"] = rng.standard_normal((out_ch, in_ch, k), dtype=np.float32) * np.float32(1.0 / np.sqrt(in_ch * k))
        t[prefix + ".bias"] = rng.standard_normal(out_ch, dtype=np.float32) * np.float32(0.1)

    def alpha(name, channels):
        t[name] = np.abs(rng.standard_normal(channels // 2, dtype=np.float32)) + np.float32(0.1)

    conv("audio_decoder.pre_conv.conv", 864, 32, 7)
    c = 864
    for stage, rate in enumerate((8, 8, 4, 2, 2)):
        alpha("audio_decoder.activations.%d.activation.snake_act.alpha" % stage, c)
        nc = c // 2
        t["audio_decoder.up_sample_conv_layers.%d.conv.weight" % stage] = rng.standard_normal((c, 1, 2 * rate), dtype=np.float32) * np.float32(0.3)
        t["audio_decoder.up_sample_conv_layers.%d.conv.bias" % stage] = rng.standard_normal(nc, dtype=np.float32) * np.float32(0.1)
        for branch, k in enumerate((3, 7, 11)):
            for block in range(3):
                p = "audio_decoder.res_layers.%d.res_blocks.%d.res_blocks.%d." % (stage, branch, block)
                alpha(p + "input_activation.activation.snake_act.alpha", nc)
                conv(p + "input_conv.conv", nc, nc, k)
                alpha(p + "skip_activation.activation.snake_act.alpha", nc)
                conv(p + "skip_conv.conv", nc, nc, k)
        c = nc
    alpha("audio_decoder.post_activation.activation.snake_act.alpha", c)
    conv("audio_decoder.post_conv.conv", 1, c, 3)
    return t
