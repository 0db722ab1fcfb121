"""Decode-step benchmark: us per step and achieved HBM GB/s of the int8 12-layer decoder stack on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--quant int8] [--skip-b8]

Workload (named in config.workload): the 12-layer d=768 decoder stack (12 heads x 64, FFN 3072, a 12 x 64
cross-attention sublayer per layer), int8 weights, batch 1, self-KV length 1024, cross-KV length 256, followed by the
final LayerNorm, the 768 -> 8 x 1024 output projection and the per-head softmax.  Synthetic seeded data, random
weights.  A "step" is one decode step of that stack for the whole batch.

HBM honesty: the int8 weights (106 MB) and one stream's KV (94 MB) would fit in the 256 MB last-level cache, so the
timed loop rotates over several independent copies of weights AND caches (ROTATE sets, > 600 MB in total): every step
streams its bytes from HBM.  Inputs are resident in HBM before the timed region starts; nothing crosses PCIe in it.

The JSON line also carries the same stack at batch 8 with ragged cache lengths (continuous batching) under "b8",
the roofline of the step and the CPU baseline (the reference's own CPU decode step, compiled from its sources).
"""
import argparse
import importlib
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

METRIC = "decode-step µs + achieved HBM GB/s (% of 8 TB/s peak), int8 b=1 and b=8"
PEAK_GBPS = 8000.0
ROTATE = 3


def build_sets(pkg, synth, backend, cfg, qtype, lengths, mems, head_rows, rotate):
    """`rotate` independent copies of the decoder weights, the output head and the per-stream caches."""
    base = synth.decoder_weights(cfg, seed=0)
    rng = np.random.default_rng(7)
    head = (rng.standard_normal((head_rows, cfg["width"]), dtype=np.float32) * np.float32(0.02))
    sets = []
    streams = synth.decoder_streams(cfg, lengths, mems, seed=1)
    for r in range(rotate):
        weights = {k: (None if v is None else np.array(v, copy=True)) for k, v in base.items()}   # new host addresses
        dec = pkg.Decoder(backend, cfg, weights)
        head_w = backend.keep(np.array(head, copy=True))
        slots, outs, logits, probs = [], [], [], []
        for s in streams:
            bufs = {n: backend.alloc(max(s[n].size, 4)).write(s[n]) for n in ("k", "v", "ck", "cv", "x")}
            out = backend.alloc(cfg["width"])
            slots.append({"k": bufs["k"].ptr, "v": bufs["v"].ptr, "ck": bufs["ck"].ptr, "cv": bufs["cv"].ptr,
                          "length": s["length"], "memory_length": s["memory_length"], "inp": bufs["x"].ptr, "out": out.ptr})
            outs.append(out)
            logits.append(backend.alloc(head_rows))
            probs.append(backend.alloc(head_rows))
        sets.append({"dec": dec, "head": head_w, "slots": slots, "outs": outs, "logits": logits, "probs": probs})
    return sets, streams


def run_steps(backend, sets, cfg, head_rows, vocab, count, start=0, with_head=True):
    for i in range(start, start + count):
        s = sets[i % len(sets)]
        if with_head:   # the step and the output head on its rows, as the one call a serving loop makes per step
            s["dec"].step_head(s["slots"], s["head"], None, head_rows, vocab, [d.ptr for d in s["logits"]], [d.ptr for d in s["probs"]])
        else:
            s["dec"].step(s["slots"])


def timed_steps(backend, sets, cfg, head_rows, vocab, steps, warmup, with_head=True):
    run_steps(backend, sets, cfg, head_rows, vocab, warmup, with_head=with_head)
    backend.sync()
    backend.timer_begin()
    run_steps(backend, sets, cfg, head_rows, vocab, steps, with_head=with_head)
    return backend.timer_end() * 1000.0 / steps


GRAPH_MODE = 1   # 0 with --launches: every stage kernel a launch of its own (runs under a profiler)


def time_config(pkg, synth, backend, qtype, lengths, mems, capacity, steps, warmup, rotate=ROTATE, stages=True):
    """Times the step of one configuration as the library runs it by default (a captured graph of stage kernels) with the
    output head -- the figure `value` is made from --, the decoder stack's part of it alone, each stage kernel of the
    graph alone, and, where it applies, the same step as one persistent launch (graph mode 2, opt-in)."""
    cfg = synth.decoder_config(layers=12, capacity=capacity)
    head_rows, vocab = 8 * 1024, 1024
    backend.set_quant(qtype)
    t0 = time.time()
    sets, streams = build_sets(pkg, synth, backend, cfg, qtype, lengths, mems, head_rows, rotate)
    setup_s = time.time() - t0
    warm = max(warmup, 2 * rotate)      # every set runs eagerly once and captures its graph before anything is timed
    batch = len(streams)
    backend.set_graph_mode(GRAPH_MODE)
    stages = stages and GRAPH_MODE == 1
    step_us = timed_steps(backend, sets, cfg, head_rows, vocab, steps, warm)
    probs = sets[0]["probs"][0].read()
    assert np.all(np.isfinite(probs)) and abs(float(probs[:vocab].sum()) - 1.0) < 1e-3, "benchmark output is not a distribution"
    stack_us = timed_steps(backend, sets, cfg, head_rows, vocab, steps, warm, with_head=False)
    persistent_us = persistent_stack_us = None
    if GRAPH_MODE == 1 and batch <= 2 and qtype in (pkg.INT8, pkg.INT4):      # the same step as one persistent launch (opt-in form)
        backend.set_graph_mode(2)
        persistent_us = timed_steps(backend, sets, cfg, head_rows, vocab, steps, warm)
        persistent_stack_us = timed_steps(backend, sets, cfg, head_rows, vocab, steps, warm, with_head=False)
        backend.set_graph_mode(1)
    b = synth.decoder_step_bytes(cfg, qtype, [s["length"] for s in streams], [s["memory_length"] for s in streams])
    head_bytes = synth.weight_bytes(head_rows, cfg["width"], qtype)
    total = b["total"] + head_bytes
    # per-stage launch times of the graph form: each of the six stage kernels alone (its 12 launches per step as one graph),
    # rotating over the same weight/cache sets so its bytes come from HBM, timed with HIP events on the backend's stream
    stage_us = []
    reps = max(4, steps // 4)
    for stage in range(6 if stages else 0):
        for i in range(2 * rotate):
            sets[i % rotate]["dec"].stage_enqueue(batch, stage)
        backend.sync()
        backend.timer_begin()
        for i in range(reps):
            sets[i % rotate]["dec"].stage_enqueue(batch, stage)
        stage_us.append(backend.timer_end() * 1000.0 / (reps * cfg["layers"]))
    for s in sets:
        s["dec"].destroy()
    return {"step_us": step_us, "stack_us": stack_us, "persistent_step_us": persistent_us, "persistent_stack_us": persistent_stack_us, "bytes": total,
            "stack_bytes": b["total"], "weight_bytes": b["weights"] + head_bytes, "kv_bytes": b["kv"],
            "gbps": total / (step_us * 1e-6) / 1e9, "setup_s": setup_s, "stage_us": stage_us,
            "stage_bytes": b["stage_bytes_per_launch"], "layers": cfg["layers"]}


def time_prefill(pkg, synth, backend, tokens=256, runs=30, warmup=5):
    """Text-encoder prefill: 6 layers, d=768, 12x64 heads, FFN 3072, f16 weights, `tokens` tokens, on the matrix cores."""
    cfg = synth.encoder_config()
    enc = pkg.Encoder(backend, cfg, synth.encoder_weights(cfg, seed=4))
    ids = np.random.default_rng(5).integers(0, cfg["vocab"], size=tokens).astype(np.int32)
    dout = backend.alloc(tokens * cfg["width"])
    for _ in range(warmup):
        enc.prefill(ids, 0, dout.ptr)
    backend.sync()
    backend.timer_begin()
    for _ in range(runs):
        enc.prefill(ids, 0, dout.ptr)
    us = backend.timer_end() * 1000.0 / runs
    out = dout.read()
    assert np.all(np.isfinite(out)), "prefill output is not finite"
    enc.destroy()
    w, f, L = cfg["width"], cfg["ffn"], cfg["layers"]
    flops = L * (2 * tokens * (3 * w * w + w * w + 2 * f * w) + 4 * tokens * tokens * w)
    return {"us": us, "flops": flops, "tflops": flops / (us * 1e-6) / 1e12, "tokens": tokens}


def time_local(pkg, synth, backend, qtype, batch, frames=40, warmup=5, streams=16, vocab=2048):
    """The local transformer's frame (16 sequential positions: one 768-wide layer step + 768 -> 2048 projection + token
    choice), resident on the device.  Every item samples (temperature 0.8, top-k 50).  The frame call is synchronous, so
    the clock is the host's; the items go up and the tokens come down once per frame inside the timed region."""
    cfg = synth.decoder_config(layers=1, capacity=streams + 1, cross_heads=0)
    w = synth.decoder_weights(cfg, seed=7, ln_bias=False)
    w["norm_out_g"] = w["norm_out_b"] = None
    rng = np.random.default_rng(8)
    proj = [(rng.standard_normal((vocab, cfg["width"]), dtype=np.float32) * np.float32(0.05)) for _ in range(streams)]
    tables = [rng.standard_normal((vocab, cfg["width"]), dtype=np.float32) for _ in range(streams)]
    loc = pkg.Local(backend, cfg, w, proj, None, tables, vocab - 32, vocab - 31, streams // 2)
    drows = [backend.alloc(cfg["width"]).write(rng.standard_normal(cfg["width"], dtype=np.float32)) for _ in range(batch)]
    items = [{"row": d.ptr, "temperature": 0.8, "topk": 50, "rng_state": 1000 + b, "forbid_eos": True} for b, d in enumerate(drows)]
    out = None
    for _ in range(warmup):
        out = loc.frame(items)
        for it, st in zip(items, out["rng_state"]):
            it["rng_state"] = st
    t0 = time.perf_counter()
    for _ in range(frames):
        out = loc.frame(items)
        for it, st in zip(items, out["rng_state"]):
            it["rng_state"] = st
    us = (time.perf_counter() - t0) * 1e6 / frames
    assert np.all(out["values"] < vocab - 32), "forbidden token chosen"
    loc.destroy()
    for d in drows:
        d.free()
    wd, f = cfg["width"], cfg["ffn"]
    layer = sum(synth.weight_bytes(n, k, qtype) for n, k in ((3 * wd, wd), (wd, wd), (f, wd), (wd, f)))
    nbytes = streams * (layer + synth.weight_bytes(vocab, wd, qtype))
    return {"batch": batch, "frame_us": us, "position_us": us / streams, "bytes": nbytes, "gbps": nbytes / (us * 1e-6) / 1e9}


def time_codec(pkg, backend, frames=64, runs=4, warmup=2):
    """The resident NanoCodec decode's operator sequence (decode_codec_resident / res_layer_device, src/graph.c:2423-2638)
    on synthetic weights: 32 -> 864 pre-conv, five stages of half-snake, grouped transposed conv (rates 8 8 4 2 2, channels
    halving) and a residual layer of 3 branches x 3 x (snake, conv k, snake, conv k) with k = 3 / 7 / 11 and dilations
    1 / 3 / 5, then snake, the 1-channel post-conv and the clip.  f32 throughout; the convolutions run on the f32 matrix
    cores.  Timed with HIP events on the backend's stream over whole decodes of `frames` raw frames."""
    rng = np.random.default_rng(11)

    def conv_w(out_ch, in_ch, k):
        return (rng.standard_normal((out_ch, in_ch, k), dtype=np.float32) * np.float32(1.0 / np.sqrt(in_ch * k))), \
               rng.standard_normal(out_ch, dtype=np.float32) * np.float32(0.1)

    def alpha(c):
        return (np.abs(rng.standard_normal(c // 2, dtype=np.float32)) + np.float32(0.1))

    rates, kernels, dilations = (8, 8, 4, 2, 2), (3, 7, 11), (1, 3, 5)
    pre = conv_w(864, 32, 7)
    stages, flops = [], 2.0 * 864 * 32 * 7 * frames
    C, L = 864, frames
    for rate in rates:
        nc, nl = C // 2, L * rate
        up_w = rng.standard_normal((C, 1, 2 * rate), dtype=np.float32) * np.float32(0.3)
        blocks = [[(alpha(nc), conv_w(nc, nc, k), alpha(nc), conv_w(nc, nc, k), d) for d in dilations] for k in kernels]
        stages.append({"alpha": alpha(C), "up": (up_w, rng.standard_normal(nc, dtype=np.float32) * np.float32(0.1)), "blocks": blocks,
                       "rate": rate})
        flops += 2.0 * nc * 2 * 2 * nl + sum(2 * 2.0 * nc * nc * k * nl * len(dilations) for k in kernels)
        C, L = nc, nl
    post_alpha, post = alpha(C), conv_w(1, C, 3)
    flops += 2.0 * C * 3 * L
    latent = backend.alloc(32 * frames).write(rng.uniform(-1, 1, 32 * frames).astype(np.float32))
    biggest = max((864 >> (i + 1)) * frames * int(np.prod(rates[:i + 1])) for i in range(5))
    bufs = [backend.alloc(max(biggest, 864 * frames)) for _ in range(13)]
    cur, up, out, act, res, br, work = bufs[:7]
    side = [b.ptr for b in bufs[4:13]]   # the batched form's buffers: three each of current, activated, residual
    audio = backend.alloc(L)

    codec = importlib.import_module(pkg.__name__ + ".codec")

    def decode(fused):
        """fused: the element-wise operators inside the convolutions' epilogues (mynah_hip_conv1d_fused), with "batched" also a
        residual layer's three branches side by side in one launch per block and position (mynah_hip_conv1d_fused_batch);
        else the operator sequence decode_codec_resident issues through the seam.  All give the same samples, bit for bit."""
        nonlocal cur, up, out
        C, L = 864, frames
        if fused:
            backend.conv1d_fused(latent.ptr, cur.ptr, 32, 864, L, 7, 1, *pre, alpha=stages[0]["alpha"])
        else:
            backend.conv1d(latent.ptr, cur.ptr, 32, 864, L, 7, 1, *pre)
        for index, st in enumerate(stages):
            nc, nl = C // 2, L * st["rate"]
            if not fused:
                backend.snake_dev(cur.ptr, st["alpha"], C, L, C // 2)
            backend.conv_transpose_dev(cur.ptr, up.ptr, C, nc, L, nl, 2 * st["rate"], st["rate"], nc, *st["up"])
            if fused:
                then_alpha = stages[index + 1]["alpha"] if index + 1 < len(stages) else post_alpha
                if fused == "batched":
                    codec.res_layer_batched(backend, st["blocks"], up.ptr, out.ptr, nc, nl, side[0:3], side[3:6], side[6:9], then_alpha=then_alpha)
                else:
                    codec.res_layer_fused(backend, st["blocks"], up.ptr, out.ptr, nc, nl, work.ptr, act.ptr, res.ptr, then_alpha=then_alpha)
            else:
                codec.res_layer(backend, st["blocks"], up.ptr, out.ptr, nc, nl, work.ptr, act.ptr, res.ptr, br.ptr)
            cur, out = out, cur
            C, L = nc, nl
        if not fused:
            backend.snake_dev(cur.ptr, post_alpha, C, L, C // 2)
        backend.conv1d(cur.ptr, audio.ptr, C, 1, L, 3, 1, *post)
        backend.clip_dev(audio.ptr, L)

    timings, waves = {}, {}
    for fused in (False, True, "batched"):
        for _ in range(warmup):
            decode(fused)
        backend.sync()
        backend.timer_begin()
        for _ in range(runs):
            decode(fused)
        timings[fused] = backend.timer_end() / runs
        waves[fused] = audio.read()
    assert np.array_equal(waves[False].view(np.uint32), waves[True].view(np.uint32)), "the fused sequence changed the samples"
    assert np.array_equal(waves[False].view(np.uint32), waves["batched"].view(np.uint32)), "the batched sequence changed the samples"
    ms, samples = timings["batched"], waves["batched"]
    assert np.all(np.isfinite(samples)) and np.abs(samples).max() <= 1.0, "codec output is not a clipped waveform"
    for d in bufs + [latent, audio]:
        d.free()
    return {"frames": frames, "samples": int(L), "ms": ms, "flops": flops, "tflops": flops / (ms * 1e-3) / 1e12,
            "ms_seam_operator_sequence": timings[False], "ms_one_launch_per_convolution": timings[True]}


# (with one or two streams the attention partials are folded by the output projection that follows; with more, by
# workgroups of the attention launch itself, and the stage timing of those launches includes, per twelve launches, the two
# small launches that give the step its counter)
STAGES = [("self-attention", "k_step_attention<self>", "LayerNorm + int8 act-quant + per-head Q/K/V rows + KV append + attention over the self cache (+ fold of the partials when more than two streams)"),
          ("self-out", "k_linear<k=768, residual>", "(fold of attention partials, up to two streams) + act-quant + O matvec + residual"),
          ("cross-attention", "k_step_attention<cross>", "LayerNorm + act-quant + per-head Q rows + attention over the cross cache (+ fold when more than two streams)"),
          ("cross-out", "k_linear<k=768, residual>", "(fold, up to two streams) + act-quant + O matvec + residual"),
          ("ffn-up", "k_linear<k=768, LayerNorm, GELU>", "LayerNorm + act-quant + up matvec + GELU"),
          ("ffn-down", "k_linear<k=3072, residual>", "act-quant + down matvec + residual")]

# HBM bytes per launch of the dominant kernels of the batch-1 and batch-8 int8 lines, from two rocprofv3 --pmc runs (FETCH_SIZE,
# then WRITE_SIZE), each scaled by what the same counter reads for the library's plain 256 MiB read+write kernel.  A figure
# belongs to the kernel sources it was measured on: it is reported only while their hash is the one recorded here.
MEASURED_TRAFFIC = {
    1: {"kernel": "k_linear<k=768, residual>", "bytes": 937934, "profile": "profiles/decode_step_int8_hbm_counters.md",
        "sources": ("kernels_linear.hip", "device_common.h", "kernels.h", "common.h"), "csrc_sha256": "21040170f4024ffc"},
    8: {"kernel": "k_step_attention<self>", "bytes": 54469598, "profile": "profiles/decode_step_int8_hbm_counters.md",
        "sources": ("kernels_step_attention.hip", "step_attention_core.h", "step_items.h", "tagged_exchange.h", "device_common.h",
                    "kernels.h", "common.h"), "csrc_sha256": "186dff1ded534a42"},
}


def latency_floor(backend, step_us, launches):
    """What the step's chain of dependent launches costs with every byte taken out: the library's probe runs graph nodes
    that only hand a 768-float vector (3072 for one stage in six) from all workgroups of one node to all workgroups of the
    next -- the skeleton of a matvec stage -- and the floor is that node time x the step's dependent launches."""
    node768 = backend.dependent_launch_probe(72, 192, 768, 1, 40)
    node3072 = backend.dependent_launch_probe(72, 192, 3072, 1, 40)
    two = backend.dependent_launch_probe(72, 192, 768, 2, 40)
    three = backend.dependent_launch_probe(72, 192, 768, 3, 40)
    floor_us = node768 * launches
    return {"what": "dependent graph nodes that only hand a 768-float vector from 192 workgroups to the next node's 192 (mynah_hip_dependent_launch_probe): "
                    "no weights, no caches",
            "node_us": round(node768, 3), "node_us_3072_floats": round(node3072, 3), "dependent_launches_per_step": launches,
            "floor_us": round(floor_us, 1), "step_over_floor": round(step_us / floor_us, 3),
            "node_us_two_chains_side_by_side": round(two, 3), "node_us_three_chains_side_by_side": round(three, 3)}


def csrc_hash(sources):
    import hashlib
    h = hashlib.sha256()
    for name in sources:
        with open(os.path.join(ROOT, "mynah-tts_amd", "csrc", name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    return h.hexdigest()[:16]


def roofline(r):
    """The dominant kernel is chosen by kernel symbol: launches of one template instance are summed (the two output
    projections of a layer are the same kernel), and the instance with the largest share of the step is the one whose
    achieved = average algorithmic bytes per launch over average launch time (HIP events around graphs holding only that
    stage, all layers, sets rotating) goes into the line.  The per-stage list is given as well."""
    rows = []
    for (name, symbol, what), us, nbytes in zip(STAGES, r["stage_us"], r["stage_bytes"]):
        rows.append({"stage": name, "kernel": symbol, "does": what, "launch_us": round(us, 3), "algorithmic_bytes_per_launch": nbytes,
                     "gbps": round(nbytes / (us * 1e-6) / 1e9, 1), "frac": round(nbytes / (us * 1e-6) / 1e9 / PEAK_GBPS, 4),
                     "share_of_step": round(us * r["layers"] / r["step_us"], 3)})
    groups = {}
    for row in rows:
        g = groups.setdefault(row["kernel"], {"us": 0.0, "bytes": 0, "launches": 0})
        g["us"] += row["launch_us"]
        g["bytes"] += row["algorithmic_bytes_per_launch"]
        g["launches"] += 1
    name, g = max(groups.items(), key=lambda kv: kv[1]["us"])
    kernel, launch_us, nbytes = name, g["us"] / g["launches"], g["bytes"] // g["launches"]
    share = g["us"] * r["layers"] / r["step_us"]
    gbps = nbytes / (launch_us * 1e-6) / 1e9
    traffic, measured = None, MEASURED_TRAFFIC.get(r.get("traffic_batch"))
    if measured is not None and measured["kernel"] == kernel and measured["csrc_sha256"] == csrc_hash(measured["sources"]):
        traffic = measured["bytes"]
    return {"bound": "hbm", "kernel": kernel, "achieved": round(gbps, 1), "peak": PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / PEAK_GBPS, 4),
            "traffic": traffic, "traffic_source": measured["profile"] if traffic is not None else None,
            "launch_us": round(launch_us, 3), "algorithmic_bytes_per_launch": nbytes, "share_of_step": round(share, 3),
            "launches_per_step": g["launches"] * r["layers"], "stages": rows,
            "whole_step": {"step_us": round(r["step_us"], 2), "algorithmic_bytes_per_step": r["bytes"], "weight_bytes": r["weight_bytes"],
                           "kv_bytes": r["kv_bytes"], "gbps": round(r["gbps"], 2), "frac": round(r["gbps"] / PEAK_GBPS, 4)}}


CPU_STEPS, CPU_WARMUP = 400, 20   # about 5 s per leg at 11.5 ms per step


def cpu_baseline(steps=CPU_STEPS, warmup=CPU_WARMUP):
    """The reference's own CPU decode step (compiled from its sources into oracle/_ref), timed on this box's host
    cores in a child process per thread count (its pool reads MYNAH_THREADS once per process): every core this process
    may run on, then 1, 2 and 4 threads on a shorter sample, and the same step with caches of one row at 1 and all
    threads -- what is left then are the weight products, the only part of the step the reference's pool splits
    (src/qmat.c:386-451, src/backend.c:246-252); its attention loops run on the calling thread (src/graph.c:3172-3247)."""
    out = {}
    affinity = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(os.cpu_count() or 1, affinity))
    short = max(steps // 4, 20)
    legs = [("all", "reference", cores, steps, []), ("one", "reference", 1, steps, []), ("two", "reference", 2, short, []),
            ("four", "reference", 4, short, []),
            ("products_one", "reference", 1, short, ["--length", "2", "--memory", "1"]),
            ("products_all", "reference", cores, short, ["--length", "2", "--memory", "1"]),
            ("engine", "engine", 1, steps, [])]
    for label, kind, threads, count, extra in legs:
        cmd = [sys.executable, os.path.join(ROOT, "oracle", "cpu_baseline.py"), "--kind", kind,
               "--threads", str(threads), "--steps", str(count), "--warmup", str(warmup)] + extra
        try:
            proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
            out[label] = json.loads(proc.stdout.strip().splitlines()[-1])
        except Exception as e:   # the baseline is reported, never required for the GPU number
            out[label] = {"error": str(e)[:200]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--quant", default="int8", choices=["int8", "int4", "f16", "f32"])
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--skip-b8", action="store_true")
    ap.add_argument("--skip-int4", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true")
    ap.add_argument("--skip-local", action="store_true")
    ap.add_argument("--skip-codec", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run the library's plain read+write kernel over 256 MiB three times (a known-size reference for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--launches", action="store_true",
                    help="run every kernel as a launch of its own instead of captured graphs, skip the per-stage and persistent timings "
                         "and print a reduced line: for runs under rocprofv3, whose interception of graph launches has crashed here")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X: the decode step has no multi-GPU form (streams shard by request, with no "
              "exchange step); run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    pkg = entry.load_package()
    import mynah_tts_amd.synth as synth
    qtype = {"f32": pkg.F32, "int8": pkg.INT8, "int4": pkg.INT4, "f16": pkg.F16}[args.quant]
    backend = pkg.Backend(quant=qtype)
    if args.launches:
        global GRAPH_MODE
        GRAPH_MODE = 0
        backend.set_graph_mode(0)
    if args.calibrate:
        for _ in range(3):
            backend.flush_cache(256 << 20)
        backend.sync()

    b1 = time_config(pkg, synth, backend, qtype, [1023], [256], 1024, args.steps, args.warmup)
    b1["traffic_batch"] = 1 if args.quant == "int8" else None
    # dependent launches of a step: six stages a layer, begin, the head product (which also does the final LayerNorm), its softmax
    floor = None if args.launches else latency_floor(backend, b1["step_us"], 6 * b1["layers"] + 3)
    int4 = None
    if args.quant == "int8" and not args.skip_int4:
        int4 = time_config(pkg, synth, backend, pkg.INT4, [1023], [256], 1024, max(args.steps // 3, 20), max(args.warmup // 3, 6), stages=False)
        backend.set_quant(qtype)
    b8 = None
    if not args.skip_b8:
        self_len, cross_len = synth.ragged_lengths(8, seed=3)
        b8 = time_config(pkg, synth, backend, qtype, [n - 1 for n in self_len], cross_len, 2048, max(args.steps // 3, 20),
                         max(args.warmup // 3, 6), rotate=ROTATE)
        b8["self_lengths"], b8["cross_lengths"] = self_len, cross_len
        b8["traffic_batch"] = 8 if args.quant == "int8" else None   # the counters were taken on these ragged lengths
    prefill = None if args.skip_prefill else time_prefill(pkg, synth, backend)
    local = None if args.skip_local else [time_local(pkg, synth, backend, qtype, b) for b in (1, 8)]
    codec = None if args.skip_codec else time_codec(pkg, backend)
    backend.close()
    if args.launches:
        line = {"mode": "every kernel a launch of its own (profiling run: not the benchmark figure)", "b1_step_us": round(b1["step_us"], 2)}
        if b8 is not None:
            line["b8_step_us"] = round(b8["step_us"], 2)
        if int4 is not None:
            line["int4_b1_step_us"] = round(int4["step_us"], 2)
        if prefill is not None:
            line["prefill_us"] = round(prefill["us"], 2)
        if local is not None:
            line["local_frame_us"] = [round(f["frame_us"], 1) for f in local]
        if codec is not None:
            line["codec_ms"] = round(codec["ms"], 3)
        print(json.dumps(line))
        return

    result = {
        "metric": METRIC,
        "value": round(b1["gbps"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(b1["step_us"] / 1000.0, 6),
        "step_us": round(b1["step_us"], 2),
        "pct_of_peak": round(100.0 * b1["gbps"] / PEAK_GBPS, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"int8": "int8 weights x int8 activations -> int32, f32 epilogue", "int4": "int4 x int8 -> int32 per group",
                  "f16": "f16 weights, f32 accumulate", "f32": "f32"}[args.quant],
        "data": "synthetic (seeded N(0,1) activations and caches, N(0,0.02) weights quantised at load time)",
        "config": {"workload": "12-layer d=768 decoder stack decode step, %s weights, batch 1, self-KV 1024, cross-KV 256 "
                               "(12x64 heads), final LayerNorm + 768->8x1024 output head + softmax" % args.quant,
                   "batch": 1, "layers": 12, "width": 768, "self_kv": 1024, "cross_kv": 256, "quant": args.quant,
                   "step_form": "captured graph of stage kernels",
                   "rotating_sets": ROTATE},
        "roofline": roofline(b1),
    }
    result["roofline"]["latency_floor"] = floor
    result["config"]["step_over_latency_floor"] = floor["step_over_floor"]
    if b1["persistent_step_us"] is not None:
        result["persistent_form"] = {"what": "the same step as ONE persistent launch (graph mode 2, opt-in): stage hand-overs through tagged "
                                             "(value, tag) pairs in memory instead of kernel boundaries",
                                     "step_us": round(b1["persistent_step_us"], 2), "stack_launch_us": round(b1["persistent_stack_us"], 2),
                                     "stack_algorithmic_bytes": b1["stack_bytes"],
                                     "frac": round(b1["stack_bytes"] / (b1["persistent_stack_us"] * 1e-6) / 1e9 / PEAK_GBPS, 4)}
    if int4 is not None:
        result["int4_b1"] = {"workload": "the same stack and lengths with int4 group-32 weights, batch 1, + output head",
                             "step_us": round(int4["step_us"], 2), "persistent_step_us": round(int4["persistent_step_us"], 2),
                             "algorithmic_bytes_per_step": int4["bytes"], "gbps": round(int4["gbps"], 2),
                             "pct_of_peak": round(100.0 * int4["gbps"] / PEAK_GBPS, 2)}
    if b8 is not None:
        result["b8"] = {"step_us": round(b8["step_us"], 2), "gbps": round(b8["gbps"], 2),
                        "pct_of_peak": round(100.0 * b8["gbps"] / PEAK_GBPS, 2), "algorithmic_bytes_per_step": b8["bytes"],
                        "weight_bytes": b8["weight_bytes"], "kv_bytes": b8["kv_bytes"], "self_lengths": b8["self_lengths"],
                        "cross_lengths": b8["cross_lengths"],
                        "us_per_stream_step": round(b8["step_us"] / 8.0, 2), "roofline": roofline(b8)}
    if prefill is not None:
        result["prefill"] = {"workload": "text-encoder prefill, 6 layers d=768 12x64 heads FFN 3072, f16 weights and operands, f32 "
                                         "accumulate, %d tokens" % prefill["tokens"],
                             "us": round(prefill["us"], 2), "flops": prefill["flops"], "tflops": round(prefill["tflops"], 2),
                             "bound": "mfma", "peak_tflops": 2500.0, "frac": round(prefill["tflops"] / 2500.0, 4)}
    if local is not None:
        result["local"] = {"workload": "local-transformer frame: 16 sequential positions of (one d=768 layer step, %s weights + "
                                       "768->2048 projection + top-50 temperature sampling), tokens chosen on the device, one "
                                       "host round trip per frame" % args.quant,
                           "frames": [{"batch": r["batch"], "frame_us": round(r["frame_us"], 1), "position_us": round(r["position_us"], 2),
                                       "algorithmic_bytes_per_frame": r["bytes"], "gbps": round(r["gbps"], 1),
                                       "frac": round(r["gbps"] / PEAK_GBPS, 4)} for r in local]}
    if codec is not None:
        result["codec"] = {"workload": "NanoCodec decode operator sequence, %d raw frames -> %d samples, f32: causal conv1d (kernels 3/7/11, "
                                       "dilations 1/3/5, 864..27 channels) on the f32 matrix cores, grouped transposed conv, half-snake"
                                       % (codec["frames"], codec["samples"]),
                           "ms": round(codec["ms"], 3), "flops": codec["flops"], "tflops": round(codec["tflops"], 2), "bound": "mfma",
                           "peak_tflops": 157.3, "frac": round(codec["tflops"] / 157.3, 4),
                           "form": "element-wise operators in the convolutions' epilogues and a residual layer's three branches side by side, "
                                   "one launch per block and position (mynah_hip_conv1d_fused_batch); samples bit-identical to the seam's "
                                   "operator sequence",
                           "ms_one_launch_per_convolution": round(codec["ms_one_launch_per_convolution"], 3),
                           "ms_seam_operator_sequence": round(codec["ms_seam_operator_sequence"], 3)}
    if not args.no_cpu:
        cpu = cpu_baseline()
        allc = cpu.get("all", {})
        us = lambda leg: round(cpu[leg]["median_us"], 1) if "median_us" in cpu.get(leg, {}) else None
        timed = [cpu[leg] for leg in ("all", "four", "two", "one") if "median_us" in cpu.get(leg, {})]
        best = min(timed, key=lambda r: r["median_us"]) if timed else {}
        result["cpu_baseline"] = {
            # the fastest of the thread counts tried is the baseline; all of them are listed below
            "value": round(best.get("median_us", float("nan")), 1), "unit": "us per decode step (batch 1)",
            "cores": best.get("threads"), "kind": best.get("kind", "reference"),
            "sample": "median of %d steps after %d warm-ups of the reference's own decoder_step_batch (stock flags, its pthread "
                      "pool) on the same 12-layer int8 stack, self-KV 1024, cross-KV 256; that function has gain-only LayerNorm and "
                      "one 768-wide cross head (same bytes and flops) and no output head.  Threads: the pool splits only the weight "
                      "products' rows; the single-token attention loops over the f32 caches run on the calling thread, so the step "
                      "gains from threads only what `weight_products_only_us` gains, and with every core busy the pool's waiting threads cost "
                      "more than they bring" % (best.get("steps", CPU_STEPS), best.get("warmup", CPU_WARMUP)),
            "all_threads_us": us("all"), "all_threads": allc.get("threads"),
            "one_thread_us": us("one"), "two_threads_us": us("two"), "four_threads_us": us("four"),
            "weight_products_only_us": {"what": "the same step with caches of one row (what the pool can split)", "one_thread": us("products_one"),
                                        "all_threads": us("products_all")},
            "online_cores": allc.get("online_cores"), "affinity_cores": allc.get("affinity_cores"),
            # not a CPU figure: the same engine's single-row decoder_run (src/graph.c:3292-3654) with this library as its
            # backend, through the reference's backend struct -- the per-operator seam, 18 calls per layer
            "same_engine_on_this_library_us": us("engine"),
            "gpu_speedup": round(best.get("median_us", float("nan")) / b1["step_us"], 1) if "median_us" in best else None,
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
