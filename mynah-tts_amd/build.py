"""Builds libmynah_hip.so (the gfx950 backend) in-tree with hipcc.

Usage: python mynah-tts_amd/build.py [--force]
The shared object is written next to this file; it is the only artefact the package loads.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmynah_hip.so")
OBJ = os.path.join(HERE, "_obj")   # per-source objects (git-ignored); a source is recompiled when it or a header is newer

# -ffp-contract=off / -fno-fast-math: the quantisers and the LayerNorm/GELU/softmax arithmetic must be
# the IEEE operations the source names; fused multiply-adds appear only where written explicitly.
# The packed-fp32 feature is switched off for device code on purpose.
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",   # leading scalar kernel arguments arrive in registers (no fetch at kernel start)
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def headers():
    return sorted(glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h")))


def is_stale():
    if not os.path.exists(LIB):
        return True
    built = os.path.getmtime(LIB)
    return any(os.path.getmtime(p) > built for p in sources() + headers())


def _compile(hipcc, src, obj):
    cmd = [hipcc] + FLAGS + ["-x", "hip", "-c", src, "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    return proc.returncode, out


def build(force=True, verbose=False):
    """Compile every HIP source for gfx950 (one object each, in parallel) and link them into one shared object.
    force=True recompiles everything; otherwise only what is older than its source or any header."""
    if not force and not is_stale():
        return LIB
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    newest_header = max(os.path.getmtime(p) for p in headers())
    jobs = []
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        fresh = os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header)
        if force or not fresh:
            jobs.append((src, obj))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as pool:
        results = list(pool.map(lambda j: _compile(hipcc, *j), jobs))
    log = "\n".join(out for _, out in results if out.strip())
    if any(rc != 0 for rc, _ in results):
        raise RuntimeError("hipcc failed:\n" + log)
    objs = [os.path.join(OBJ, os.path.basename(src) + ".o") for src in sources()]
    proc = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout)
    if verbose and log.strip():
        print(log)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
