"""Seeded synthetic workloads: the decoder stack, KV caches and encoder of the benchmark configurations.

One numpy Generator per workload, drawn in the order written here, so the CPU checkers and the GPU
read identical bytes.  Weights ~ N(0, 0.02), activations and caches ~ N(0, 1), LayerNorm gain
1 + N(0, 0.1), LayerNorm bias N(0, 0.02).
"""
import numpy as np


def decoder_config(layers=12, width=768, heads=12, ffn=3072, cross_heads=12, capacity=1025):
    return {"layers": layers, "width": width, "heads": heads, "head_width": width // heads, "ffn": ffn,
            "cross_heads": cross_heads, "cross_head_width": (width // cross_heads) if cross_heads else 0,
            "capacity": capacity}


def _normal(rng, shape, std, mean=0.0):
    a = rng.standard_normal(shape, dtype=np.float32)
    a *= np.float32(std)
    if mean:
        a += np.float32(mean)
    return a


def decoder_weights(cfg, seed=0, ln_bias=True, position=True):
    """Per-layer f32 tensors keyed as the oracle and the backend bindings expect."""
    rng = np.random.default_rng(seed)
    L, w, f = cfg["layers"], cfg["width"], cfg["ffn"]
    xw = cfg["cross_heads"] * cfg["cross_head_width"]
    out = {}
    for name in ("norm_self", "norm_cross", "norm_ff"):
        out[name + "_g"] = _normal(rng, (L, w), 0.1, 1.0)
        out[name + "_b"] = _normal(rng, (L, w), 0.02) if ln_bias else None
    out["qkv"] = _normal(rng, (L, 3 * w, w), 0.02)
    out["o_self"] = _normal(rng, (L, w, w), 0.02)
    out["q_cross"] = _normal(rng, (L, max(xw, 1), w), 0.02)
    out["o_cross"] = _normal(rng, (L, w, max(xw, 1)), 0.02)
    out["ffn_up"] = _normal(rng, (L, f, w), 0.02)
    out["ffn_down"] = _normal(rng, (L, w, f), 0.02)
    out["norm_out_g"] = _normal(rng, (w,), 0.1, 1.0)
    out["norm_out_b"] = _normal(rng, (w,), 0.02) if ln_bias else None
    out["position"] = _normal(rng, (cfg["capacity"], w), 0.02) if position else None
    return out


def decoder_streams(cfg, lengths, memory_lengths, seed=1):
    """Per-stream hidden input and KV caches.  Cache rows at and beyond `length` are zero."""
    rng = np.random.default_rng(seed)
    L, w, cap = cfg["layers"], cfg["width"], cfg["capacity"]
    xw = cfg["cross_heads"] * cfg["cross_head_width"]
    streams = []
    for length, mem in zip(lengths, memory_lengths):
        s = {"length": int(length), "memory_length": int(mem)}
        s["x"] = _normal(rng, (w,), 1.0)
        k = np.zeros((L, cap, w), np.float32)
        v = np.zeros((L, cap, w), np.float32)
        k[:, :length] = _normal(rng, (L, length, w), 1.0)
        v[:, :length] = _normal(rng, (L, length, w), 1.0)
        s["k"], s["v"] = k, v
        s["ck"] = _normal(rng, (L, max(mem, 1), max(xw, 1)), 1.0)[:, :mem].copy() if xw else np.zeros((L, 0, 1), np.float32)
        s["cv"] = _normal(rng, (L, max(mem, 1), max(xw, 1)), 1.0)[:, :mem].copy() if xw else np.zeros((L, 0, 1), np.float32)
        streams.append(s)
    return streams


def ragged_lengths(batch, seed=3, self_range=(64, 2048), cross_range=(32, 256)):
    """Continuous-batching lengths: self KV ~ U[64, 2048], cross ~ U[32, 256] (inclusive)."""
    rng = np.random.default_rng(seed)
    self_len = rng.integers(self_range[0], self_range[1] + 1, size=batch)
    cross_len = rng.integers(cross_range[0], cross_range[1] + 1, size=batch)
    return [int(x) for x in self_len], [int(x) for x in cross_len]


def encoder_config(layers=6, width=768, heads=12, ffn=3072, vocab=4096, max_positions=512):
    return {"layers": layers, "width": width, "heads": heads, "head_width": width // heads, "ffn": ffn,
            "vocab": vocab, "max_positions": max_positions}


def encoder_weights(cfg, seed=4):
    rng = np.random.default_rng(seed)
    L, w, f = cfg["layers"], cfg["width"], cfg["ffn"]
    out = {"tok_table": _normal(rng, (cfg["vocab"], w), 0.02), "pos_table": _normal(rng, (cfg["max_positions"], w), 0.02)}
    out["qkv"] = _normal(rng, (L, 3 * w, w), 0.02)
    out["o"] = _normal(rng, (L, w, w), 0.02)
    out["up"] = _normal(rng, (L, f, w), 0.02)
    out["down"] = _normal(rng, (L, w, f), 0.02)
    for name in ("norm1", "norm2"):
        out[name + "_g"] = _normal(rng, (L, w), 0.1, 1.0)
        out[name + "_b"] = _normal(rng, (L, w), 0.02)
    out["norm_out_g"] = _normal(rng, (w,), 0.1, 1.0)
    out["norm_out_b"] = _normal(rng, (w,), 0.02)
    return out


def encoder_weights_f16(cfg, seed, kernel=1, biases=False):
    """Encoder tensors whose matrices and tables are exactly representable in f16 (as f32 arrays), so that a checker that
    reads f32 weights and one that reads f16 bits multiply the same numbers.  kernel > 1: the FFN weights are those of
    the causal conv FFN, up [L, ffn, width * kernel] and down [L, width, ffn * kernel] (rows [in][kernel] flattened).
    LayerNorm gains stay f32; biases only when asked for (the reference's LayerNorm has none)."""
    rng = np.random.default_rng(seed)
    L, w, f = cfg["layers"], cfg["width"], cfg["ffn"]

    def n(shape, std, mean=0.0):
        return (rng.standard_normal(shape) * std + mean).astype(np.float32)

    def h(a):
        return a.astype(np.float16).astype(np.float32)
    out = {"tok_table": h(n((cfg["vocab"], w), 0.02)), "pos_table": h(n((cfg["max_positions"], w), 0.02)),
           "qkv": h(n((L, 3 * w, w), 0.02)), "o": h(n((L, w, w), 0.02)),
           "up": h(n((L, f, w * kernel), 0.02)), "down": h(n((L, w, f * kernel), 0.02)),
           "norm1_g": n((L, w), 0.1, 1.0), "norm2_g": n((L, w), 0.1, 1.0), "norm_out_g": n((w,), 0.1, 1.0)}
    for name in ("norm1_b", "norm2_b", "norm_out_b"):
        out[name] = n((L, w) if name != "norm_out_b" else (w,), 0.02) if biases else None
    return out


# ---- algorithmic bytes (what roofline.achieved is computed from) --------------------------------
def weight_bytes(n, k, qtype):
    """Packed bytes of one [n, k] matrix incl. scales: f32 4nk; int8 nk + 4n; int4 nk/2 + 4nk/32; f16 2nk."""
    return {0: 4 * n * k, 1: n * k + 4 * n, 2: n * k // 2 + 4 * n * (k // 32), 3: 2 * n * k}[qtype]


def decoder_step_bytes(cfg, qtype, lengths, memory_lengths):
    """Algorithmic HBM bytes of one decode step: every packed weight and scale once (weight-stationary
    over the batch), each stream's self K/V rows [0, length] and cross K/V rows read once, the appended
    K/V row written, LayerNorm vectors; activations (a few KB) are not counted."""
    L, w, f = cfg["layers"], cfg["width"], cfg["ffn"]
    xw = cfg["cross_heads"] * cfg["cross_head_width"]
    per_layer = (weight_bytes(3 * w, w, qtype) + weight_bytes(w, w, qtype) + weight_bytes(f, w, qtype) +
                 weight_bytes(w, f, qtype))
    if xw:
        per_layer += weight_bytes(xw, w, qtype) + weight_bytes(w, xw, qtype)
    weights = L * per_layer
    kv = 0
    for length, mem in zip(lengths, memory_lengths):
        kv += L * 2 * (length + 1) * w * 4      # rows [0, length] incl. the appended one
        kv += L * 2 * mem * xw * 4
    # the same bytes split by stage kernel, per launch (one layer): order of the MYNAH_HIP_STAGE_* values
    self_kv = sum(2 * (n + 1) * w * 4 for n in lengths)
    cross_kv = sum(2 * m * xw * 4 for m in memory_lengths)
    stages = [weight_bytes(3 * w, w, qtype) + self_kv, weight_bytes(w, w, qtype),
              (weight_bytes(xw, w, qtype) + cross_kv) if xw else 0, weight_bytes(w, xw, qtype) if xw else 0,
              weight_bytes(f, w, qtype), weight_bytes(w, f, qtype)]
    return {"weights": weights, "kv": kv, "total": weights + kv, "stage_bytes_per_launch": stages}
