"""Builds libshv_hip.so (the C-ABI HIP library for gfx950) in-tree with hipcc.

    python strix-halo-vulkan_amd/build.py [-j N] [--force]

Every .hip file under csrc/ is compiled for gfx950 only and linked into one shared library that
sits next to this file, so it travels with the tree.  Packed-FP32 instruction selection is
switched off for all device code; the quantiser additionally forbids floating-point contraction
because its results must be bit-identical to a CPU that never fuses a multiply-add.
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
LIB = os.path.join(HERE, "libshv_hip.so")
HOST = os.path.join(HERE, "host")
HOST_LIB = os.path.join(HERE, "libshv_llm.so")
CXX = os.environ.get("CXX", "g++")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
PER_FILE = {"quantize_q4k.hip": ["-ffp-contract=off"]}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    hs.append(os.path.join(ROOT, "include", "shv_hip.h"))
    return hs


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + headers()):
        # SHV_EXTRA_HIPCC_FLAGS: extra compiler flags for an experiment (e.g. a -D switch)
        cmd = [HIPCC] + COMMON + PER_FILE.get(src, []) + os.environ.get("SHV_EXTRA_HIPCC_FLAGS", "").split() + ["-c", path, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr))
        # the host pass warns that it does not know the packed-fp32 target feature; drop that
        noise = "is not a recognized feature for this target"
        rest = [l for l in r.stderr.splitlines() if l.strip() and noise not in l and "warning generated" not in l]
        if rest:
            sys.stderr.write("\n".join(rest) + "\n")
    return obj


def build(jobs=8, force=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
    build_host(force)
    return LIB


def build_host(force=False):
    """The C++ host layer (host/*.cpp) above the C ABI: plain g++, linked against libshv_hip.so."""
    srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp"))
    deps = srcs + [os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith((".hpp", ".h"))]
    deps += [os.path.join(ROOT, "include", "shv_hip.h"), LIB]
    if force or _stale(HOST_LIB, deps):
        cmd = [CXX, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-I" + os.path.join(ROOT, "include"),
               "-I" + HOST, "-o", HOST_LIB] + srcs + ["-L" + HERE, "-lshv_hip", "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host build failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
        if r.stderr.strip():
            sys.stderr.write(r.stderr)
    return HOST_LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    print(build(a.j, a.force))
