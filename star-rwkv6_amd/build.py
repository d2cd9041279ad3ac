"""Compiles the HIP sources in csrc/ into lib/libwkv6_gfx950.so (gfx950 only).

Usage: python star-rwkv6_amd/build.py            (hipcc cross-compiles; no GPU needed)
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libwkv6_gfx950.so")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fno-gpu-rdc",
    # packed-fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm", "-Wno-unknown-warning-option", "-Wno-unknown-attributes",
    "-I" + INCLUDE, "-I" + CSRC,
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose=False, extra_flags=()):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []

    def compile_one(src):
        obj = os.path.join(LIBDIR, src[:-4] + ".o")
        cmd = [HIPCC, *FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        p = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(l for l in (p.stdout + p.stderr).splitlines()
                        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(compile_one, sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stdout + p.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
