"""Build recipes for the test oracle (TEST INFRASTRUCTURE, not product code).

build_oracle()  gcc -> oracle/_build/librexsc_oracle.so   (the plain-C restatement)
build_ref()     g++ -> oracle/_ref/{sc_extension,fixed_extension}.so
                the reference's own CPU extension, compiled from its sources where they lie
                under /root/reference (nothing is copied); only possible where that tree
                exists.  The reference's build system (setuptools) is not run: its three
                sources are compiled directly against the torch headers of this image with
                the flags its setup.py asks for (-march=native -fopenmp).

Run as a script to build both:  python oracle/build.py
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SRC = "/root/reference/torch_c/sc-extension"
ORACLE_SO = os.path.join(HERE, "_build", "librexsc_oracle.so")
REF_DIR = os.path.join(HERE, "_ref")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def build_oracle(force=True):
    """Compile the C restatement.  x86-64-v3 (AVX2+POPCNT) so the library also runs on a
    host whose CPU differs from the build machine's."""
    os.makedirs(os.path.dirname(ORACLE_SO), exist_ok=True)
    src = os.path.join(HERE, "rexsc_oracle.c")
    if not force and os.path.exists(ORACLE_SO) and os.path.getmtime(ORACLE_SO) >= os.path.getmtime(src):
        return ORACLE_SO
    _run(["gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-fPIC", "-shared", "-std=gnu11",
          "-Wall", "-o", ORACLE_SO, src, "-lm"])
    return ORACLE_SO


ORACLE_SAN_SO = os.path.join(os.path.dirname(ORACLE_SO), "librexsc_oracle_san.so")


def build_oracle_sanitized():
    """The same source with AddressSanitizer and UndefinedBehaviorSanitizer (host code only; any finding aborts).
    -> (library path, path of the ASan runtime that a process loading it has to preload)."""
    os.makedirs(os.path.dirname(ORACLE_SAN_SO), exist_ok=True)
    src = os.path.join(HERE, "rexsc_oracle.c")
    _run(["gcc", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
          "-fno-sanitize-recover=undefined", "-march=x86-64-v3", "-fopenmp", "-fPIC", "-shared", "-std=gnu11",
          "-Wall", "-o", ORACLE_SAN_SO, src, "-lm"])
    runtime = subprocess.run(["gcc", "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    return ORACLE_SAN_SO, runtime


def ref_available():
    return os.path.isdir(REF_SRC)


def build_ref(force=False):
    """Compile the reference CPU extension into oracle/_ref/ (git-ignored)."""
    if not ref_available():
        return None
    from torch.utils import cpp_extension
    import torch
    os.makedirs(REF_DIR, exist_ok=True)
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"]]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    common = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-march=native", "-fopenmp", "-w",
              "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi())]
    link = ["-L" + libdir, "-Wl,-rpath," + libdir, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python"]
    targets = {
        "sc_extension": ["sc.cpp", "sc_conv.cpp", "sc_matmul.cpp"],
        "fixed_extension": ["fixed.cpp"],
    }
    built = {}
    for name, srcs in targets.items():
        out = os.path.join(REF_DIR, name + ".so")
        built[name] = out
        if not force and os.path.exists(out):
            continue
        cmd = common + ["-DTORCH_EXTENSION_NAME=" + name] + inc + \
            [os.path.join(REF_SRC, s) for s in srcs] + ["-o", out] + link
        _run(cmd)
    return built


if __name__ == "__main__":
    print(build_oracle())
    print(build_ref(force="--force" in sys.argv))
