"""TEST/BENCH INFRASTRUCTURE ONLY: times the CPU path of the decode step on this machine's host cores.

Run as a subprocess by bench.py's cpu_baseline leg (the reference's thread pool reads MYNAH_THREADS once per
process, src/threads.c:36-44, so each thread count needs its own process):

    python oracle/cpu_baseline.py --kind reference --threads 16 --steps 5 --warmup 2 [--layers 12 --length 1024 --memory 256]

kind=reference : the reference's own decoder_step_batch (oracle/_ref/libmynah_ref.so, stock flags, its pthread pool)
                 -- gain-only LayerNorm and ONE cross-attention head of width 768, the only form that function has;
                 same weight bytes, KV bytes and flops as the benchmark workload.
kind=engine    : the same reference engine function one level up (decoder_run, src/graph.c:3292-3654, single row) with the
                 gfx950 library as its backend through the reference's backend struct (oracle/ref_shim_backend.c): the
                 resident path, 18 seam calls per layer.  Not a CPU figure: it is what the unmodified engine gets from the
                 library, reported beside the CPU figure of the same engine.
kind=port      : this repository's restatement (liboracle.so), single thread, exact benchmark workload.
Protocol as the reference's own bench (cli/main.c:382-406): warm-ups, then the median of the measured runs.
Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--kind", default="reference")
    ap.add_argument("--threads", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--length", type=int, default=1024)
    ap.add_argument("--memory", type=int, default=256)
    ap.add_argument("--quant", default="int8")
    args = ap.parse_args()
    os.environ["MYNAH_THREADS"] = str(args.threads)
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry
    entry.load_package()
    import mynah_tts_amd.synth as synth
    orc = entry.load_oracle()
    qtype = {"f32": orc.F32, "int8": orc.INT8, "int4": orc.INT4}[args.quant]
    kind = args.kind
    if kind == "reference" and not orc.ref_available():
        kind = "port"
    if kind == "engine" and not orc.ref_available():
        print(json.dumps({"kind": "engine", "error": "oracle/_ref is not built"}))
        return
    cross_heads = 1 if kind in ("reference", "engine") else 12
    extra = args.steps + args.warmup if kind == "engine" else 0    # the engine run appends a row per step
    cfg = synth.decoder_config(layers=args.layers, capacity=args.length + 8 + extra, cross_heads=cross_heads)
    weights = synth.decoder_weights(cfg, seed=0, ln_bias=(kind == "port"))
    length = args.length - 1
    s = synth.decoder_streams(cfg, [length], [args.memory], seed=1)[0]
    if kind == "engine":
        if args.quant == "f32":
            os.environ.pop("MYNAH_QUANT", None)
        else:
            os.environ["MYNAH_QUANT"] = args.quant
        os.environ["MYNAH_QUANT_ARITH"] = "stock"
        dec = orc.RefDecoder(cfg, weights, qtype, 1, args.memory)
        dec.use_hip(entry.load_package().LIB_PATH)
        state = {"n": length}

        def run():
            _, state["n"], resident = dec.run_one(0, s["k"], s["v"], s["ck"], s["cv"], state["n"], args.memory, s["x"])
            assert resident, "the engine fell back to its CPU path"
        threads = 1
    elif kind == "reference":
        dec = orc.RefDecoder(cfg, weights, qtype, 1, args.memory)
        run = lambda: dec.step([s["k"]], [s["v"]], [s["ck"]], [s["cv"]], [length], [args.memory], [s["x"]])
        threads = orc.load_ref().ref_num_threads()
    else:
        dec = orc.Decoder(cfg, weights, qtype)
        run = lambda: dec.step([s["k"]], [s["v"]], [s["ck"]], [s["cv"]], [length], [args.memory], [s["x"]])
        threads = 1
    for _ in range(args.warmup):
        run()
    times = []
    for _ in range(args.steps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    median = times[len(times) // 2]
    # cores this process may run on (a container's share can be smaller than the machine's count) beside the machine's count
    affinity = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else None
    print(json.dumps({"kind": kind, "threads": threads, "median_us": median * 1e6, "min_us": times[0] * 1e6,
                      "steps": args.steps, "warmup": args.warmup, "online_cores": os.cpu_count(), "affinity_cores": affinity,
                      "length": args.length, "memory": args.memory}))


if __name__ == "__main__":
    main()
