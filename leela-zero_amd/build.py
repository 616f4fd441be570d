"""Builds csrc/liblzhip.so (gfx950 code objects + host runtime) with hipcc.

hipcc cross-compiles for gfx950 without a GPU present.  The library is built
in-tree so that it travels with the source tree; nothing is installed.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "liblzhip.so")

SOURCES = ["kernels.hip", "hip_pipe.hip", "hip_scheduler.cpp", "goboard.cpp", "search.cpp",
           "weights_file.cpp",
           "c_api.cpp"]

# -packed-fp32-ops off: v_pk_*_f32 forms are kept out of the generated code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-result",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build(verbose=False):
    """Compile every source and link the shared library.  Always recompiles."""
    objs = []
    inc = ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc()] + HIP_FLAGS + inc + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
        if verbose and err.strip():
            print(err, file=sys.stderr)
        objs.append(obj)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread", "-lz"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    build_engine_path_test(verbose)
    return LIB


ENGINE_TEST = os.path.join(CSRC, "engine_path_test")


def build_engine_path_test(verbose=False):
    """tests/cpp/test_engine_path.cpp linked against the library: the C++ drop-in
    path (HIPScheduler as a ForwardPipe) exercised on a GPU box by the GPU tests.
    Built here so that no compiler has to run there."""
    src = os.path.join(ROOT, "tests", "cpp", "test_engine_path.cpp")
    cmd = [hipcc(), "-O1", "-std=c++17", "-x", "c++", src, "-x", "none",
           "-I", os.path.join(ROOT, "include"), "-L", CSRC, "-llzhip", "-lpthread",
           "-Wl,-rpath,$ORIGIN", "-o", ENGINE_TEST]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("engine path test failed to build:\n" + r.stderr)
    return ENGINE_TEST


if __name__ == "__main__":
    print(build(verbose=True))
