"""Compiles the gfx950 kernels and the C ABI into libtokspur_hip.so, in-tree, with hipcc.

hipcc cross-compiles without a GPU. Each source is compiled to an object (in parallel) and the
objects are linked into one shared library next to this file.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtokspur_hip.so")
HOST_LIB = os.path.join(HERE, "libtokspur_graph.so")

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-ffp-contract=off", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _compile(src, out_dir):
    obj = os.path.join(out_dir, os.path.basename(src) + ".o")
    cmd = ["hipcc", "-x", "hip", "-c", src, "-o", obj] + HIP_FLAGS
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}")
    noise = "unknown target feature"
    warnings = "\n".join(line for line in proc.stdout.splitlines() if line.strip() and noise not in line)
    return obj, warnings


def build(verbose=False, jobs=8):
    out_dir = os.path.join(HERE, "build")
    os.makedirs(out_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda s: _compile(s, out_dir), sources()))
    objs = [r[0] for r in results]
    if verbose:
        for _, w in results:
            if w:
                print(w)
    link = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", LIB] + objs
    proc = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode:
        raise RuntimeError(f"link failed:\n{proc.stdout}")
    return LIB


def build_host():
    """The C++ host side over the C ABI (tokspur::HipGraph, the GGUF reader and the Pack v3 builder / adopter): host/*.cpp -> libtokspur_graph.so."""
    root = os.path.dirname(HERE)
    host = os.path.join(HERE, "host")
    cmd = ["hipcc", "-std=c++20", "-O2", "-fPIC", "-shared", "-Wall", "-pthread"] + sorted(os.path.join(host, f) for f in os.listdir(host) if f.endswith(".cpp")) + [
        "-I", os.path.join(root, "include"), "-L", HERE, "-ltokspur_hip", "-Wl,-rpath,$ORIGIN", "-o", HOST_LIB]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode:
        raise RuntimeError(f"host library build failed:\n{proc.stdout}")
    return HOST_LIB


def build_native_tests():
    """tests/native/*.cpp -> tests/native/bin/ (they link the host library, the C ABI and the CPU oracle as checker)."""
    root = os.path.dirname(HERE)
    src_dir, out_dir = os.path.join(root, "tests", "native"), os.path.join(root, "tests", "native", "bin")
    os.makedirs(out_dir, exist_ok=True)
    built = []
    for name in sorted(f for f in os.listdir(src_dir) if f.endswith(".cpp")):
        out = os.path.join(out_dir, name[:-4])
        cmd = ["hipcc", "-std=c++20", "-O2", "-Wall", os.path.join(src_dir, name), "-I", os.path.join(HERE, "host"), "-I", os.path.join(root, "include"),
               "-I", os.path.join(root, "oracle"), "-L", HERE, "-ltokspur_graph", "-ltokspur_hip", "-L", os.path.join(root, "oracle"), "-loracle",
               "-Wl,-rpath," + HERE, "-Wl,-rpath," + os.path.join(root, "oracle"), "-o", out]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode:
            raise RuntimeError(f"native test build failed for {name}:\n{proc.stdout}")
        built.append(out)
    return built


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print(build_host())
