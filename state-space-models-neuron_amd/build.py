"""Build libmamba2_hip.so (gfx950) in-tree with hipcc.

    python state-space-models-neuron_amd/build.py [--force] [-j N]

The library is the C-ABI boundary declared in include/mamba2_hip.h.  hipcc
cross-compiles for gfx950 without a GPU, so this runs anywhere ROCm is installed.
"""
import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "mamba2", "libmamba2_hip.so")
SOURCES = ["api.hip", "conv1d.hip", "decode.hip", "glue.hip", "ssd_fwd.hip", "ssd_bwd.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm",
         # packed-FP32 VALU forms are kept out of the generated code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, jobs=None, verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    headers.append(os.path.join(os.path.dirname(HERE), "include", "mamba2_hip.h"))
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    todo = []
    for s in srcs:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJ, s.replace(".hip", ".o"))
        if force or _stale(obj, [src] + headers):
            todo.append((src, obj))
    jobs = jobs or min(8, max(1, len(todo)))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = {ex.submit(_run, [hipcc] + FLAGS + ["-c", src, "-o", obj]): src for src, obj in todo}
        for f in cf.as_completed(futs):
            out = f.result()
            if verbose:
                print("compiled", os.path.basename(futs[f]), flush=True)
                if out.strip():
                    print(out)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in srcs]
    if force or todo or _stale(LIB, objs):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
        if verbose:
            print("linked", LIB, flush=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    build(force=a.force, jobs=a.j)
