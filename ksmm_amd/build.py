"""Builds libksmm_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m ksmm_amd.build          # rebuild everything
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libksmm_hip.so")
SOURCES = ["ksmm_api.hip", "ksmm_generic.hip", "ksmm_wave.hip", "ksmm_tile.hip", "ksmm_stream.hip", "ksmm_tile_bf.hip", "ksmm_rows_bf.hip", "ksmm_gemm.hip", "ksmm_chain16.hip", "ksmm_transpose.hip", "ksmm_backward.hip"]
# measurement aids of bench.py: a library of their own, outside the drop-in ABI
BENCH_LIB = os.path.join(HERE, "libksmm_bench.so")
BENCH_SOURCES = ["ksmm_probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are switched off on purpose for this hardware pool
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr[-8000:]))
    noise = "is not a recognized feature for this target"
    warn = "\n".join(l for l in r.stderr.splitlines() if l.strip() and noise not in l)
    return obj, warn


def build(verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, SOURCES + BENCH_SOURCES))
    objs = [o for o, _ in results[:len(SOURCES)]]
    bench_objs = [o for o, _ in results[len(SOURCES):]]
    if verbose:
        for _, w in results:
            if w:
                print(w, file=sys.stderr)
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr[-4000:])
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", BENCH_LIB] + bench_objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr[-4000:])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
