"""Builds libbsa_hip.so for gfx950 with hipcc (no torch headers, no cmake).

    python build.py            # rebuild when a source is newer than the library
    python build.py --force    # always rebuild
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["api.hip", "layout_build.hip", "matmul.hip", "dsd_runs.hip", "softmax.hip", "attention.hip", "block_copy.hip"]
HEADERS = ["bench_yardstick.hip", "bsa_device.hpp", "lds_tiles.hpp", "lds_index_math.hpp", "bsa_internal.hpp", "group_walk.hpp", os.path.join("..", "..", "include", "bsa.h")]
LIB = os.path.join(HERE, "libbsa_hip.so")

# The same library built with the compile-time alternative of a hand-rolled sequence, for the test that pins the
# default against it (tests/test_gpu_build_variants.py): full agent-scope fences around the counter of split
# groups instead of atomic accesses + a wait.
CHECK_VARIANTS = {
    "fences": (os.path.join(HERE, "libbsa_hip_fences.so"), ["-DBSA_SPLIT_MODE=1"]),
}

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def out_of_date() -> bool:
    if not os.path.exists(LIB) or not all(os.path.exists(path) for path, _ in CHECK_VARIANTS.values()):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(os.path.join(HERE, f)) > t for f in SOURCES + HEADERS + ["build.py"])


def build(force: bool = False, verbose: bool = False, extra_flags=(), lib: str = LIB) -> str:
    """Compiles every source to an object file (in parallel, one hipcc each) and links them."""
    if not force and lib == LIB and not out_of_date():
        return LIB
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build", os.path.basename(lib))
    os.makedirs(objdir, exist_ok=True)
    flags = [f for f in FLAGS if f != "-shared"] + list(extra_flags)
    jobs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src + ".o")
        cmd = [hipcc] + flags + ["-c", os.path.join(HERE, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        jobs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, obj, proc in jobs:
        out = proc.communicate()[0]
        out = "\n".join(ln for ln in out.splitlines() if "packed-fp32-ops" not in ln)   # the host pass does not know the feature
        if proc.returncode != 0:
            failed = True
            sys.stderr.write(out + "\n")
        elif verbose and out.strip():
            sys.stderr.write(out + "\n")
    if failed:
        raise RuntimeError("hipcc failed building " + os.path.basename(lib))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + [j[1] for j in jobs] + ["-o", lib]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed linking " + os.path.basename(lib))
    if lib == LIB:
        build_index_host(verbose)
        build_bench_yardstick(verbose)
        for _, (path, flags) in CHECK_VARIANTS.items():
            build(force=True, verbose=verbose, extra_flags=flags, lib=path)
    return lib


def build_bench_yardstick(verbose: bool = False) -> str:
    """The streaming-copy yardstick bench.py times beside the kernels (its own small library)."""
    out = os.path.join(HERE, "libbsa_bench.so")
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")] + FLAGS + [os.path.join(HERE, "bench_yardstick.hip"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building libbsa_bench.so")
    return out


def build_index_host(verbose: bool = False) -> str:
    """g++ build of the LDS index arithmetic (no GPU code) for the bank-model tests."""
    out = os.path.join(HERE, "liblds_index.so")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           os.path.join(HERE, "lds_index_host.cpp"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
