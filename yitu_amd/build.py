"""Builds libyitu_hip.so (gfx950) in-tree with hipcc.

Usage: ``python -m yitu_amd.build [-j N] [--force]``. Objects are cached under
``yitu_amd/csrc/build/`` and rebuilt when a source or header is newer.
"""
import argparse
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libyitu_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 instructions are kept out of generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _newest_header():
    hs = glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, force):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    if (not force and os.path.exists(obj) and os.path.getmtime(obj) > os.path.getmtime(src)
            and os.path.getmtime(obj) > _newest_header()):
        return obj
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    if out.strip():
        sys.stderr.write(out + "\n")
    return obj


HOST_LIB = os.path.join(HERE, "libyitu_host.so")
# x86-64-v3: built in one container, loaded on another host
HOST_FLAGS = ["-O3", "-mavx2", "-mfma", "-std=c++17", "-fopenmp", "-fPIC", "-fvisibility=hidden",
              "-Wall", "-Wextra", "-shared"]


def build_host(force=False):
    """libyitu_host.so: the CPU graph-preparation code (g++, OpenMP)."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "host", "*.cpp")))
    newest = max([os.path.getmtime(s) for s in srcs] +
                 [os.path.getmtime(os.path.join(HERE, "..", "include", "yitu_host.h"))])
    if not force and os.path.exists(HOST_LIB) and os.path.getmtime(HOST_LIB) > newest:
        return HOST_LIB
    cmd = [os.environ.get("CXX", "g++")] + HOST_FLAGS + srcs + ["-o", HOST_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("g++ failed:\n" + r.stdout + r.stderr)
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    return HOST_LIB


def build(force=False, jobs=8):
    build_host(force)
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    print(build(force=a.force, jobs=a.j))
