"""Builds rex-sc_amd/librexsc.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python rex-sc_amd/build.py            # rebuild what changed
    python rex-sc_amd/build.py --force    # rebuild everything

The library is built in-tree; nothing is installed.  Compilation needs no GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "librexsc.so")
SOURCES = ["sc_api.hip", "sng.hip", "sc_compute.hip", "pointwise.hip", "fixed_conv.hip", "profile.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wall", "-Wno-unused-function"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force, extra):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(ROOT, "include", "rexsc.h"))
    if force or _newer(obj, [os.path.join(CSRC, src)] + headers):
        cmd = [_hipcc()] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stdout))
        out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if out:
            print(out)
    return obj


def build(force=False, extra_flags=()):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, list(extra_flags)), SOURCES))
    if force or _newer(LIB, objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("link failed:\n" + proc.stdout)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
