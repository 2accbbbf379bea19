"""Builds lib2by4_gfx950.so (the C-ABI library of include/tf24.h) with hipcc, for gfx950 only.

    python 2by4-pretrain_amd/build.py [-j N] [--force]

Objects go to 2by4-pretrain_amd/build/, the library next to the Python package that loads it
(2by4-pretrain_amd/sparse/lib2by4_gfx950.so).
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "sparse", "lib2by4_gfx950.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",                                            # bit-exact with unfused CPU arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",    # no packed-fp32 instructions
    "-Wno-unused-command-line-argument", "-Wno-ignored-optimization-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, force):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    src_path = os.path.join(CSRC, src)
    deps = [src_path] + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".hpp")]
    deps.append(os.path.join(ROOT, "include", "tf24.h"))
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj, ""
    cmd = [HIPCC, *FLAGS, "-c", src_path, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj, res.stderr


def build_library(jobs=8, force=True, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        results = list(pool.map(lambda s: _compile(s, force), sources()))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-v", action="store_true")
    a = ap.parse_args()
    print(build_library(a.j, a.force, a.v))
