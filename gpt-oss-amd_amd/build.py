"""Builds libmoe_gfx950.so from csrc/*.hip with hipcc for gfx950 (cross-compiles without a GPU).

Usage: python gpt-oss-amd_amd/build.py [--force]
The library is written next to this file so it travels with the source tree.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe_gfx950.so")
OBJ_DIR = os.path.join(HERE, "build")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-munsafe-fp-atomics",
    # never let the compiler form packed fp32 arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-warning-option",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def headers():
    inc = os.path.join(os.path.dirname(HERE), "include")
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs += [os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h")]
    return hs


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    return obj, err


def up_to_date():
    if not os.path.exists(LIB):
        return False
    t = os.path.getmtime(LIB)
    return all(os.path.getmtime(p) <= t for p in sources() + headers() + [os.path.abspath(__file__)])


HOST_DIR = os.path.join(HERE, "host")
HOST_BIN_DIR = os.path.join(HOST_DIR, "bin")
HOST_PROGRAMS = ["moe_stack_main", "example_layer_loop"]


def build_host_programs():
    """The C++ host side (layer loop, forward(), decode loop) as programs linked against the library:
    compiled here so that the GPU box only has to run them.  Plain C++ against the HIP runtime API."""
    os.makedirs(HOST_BIN_DIR, exist_ok=True)
    out = []
    for name in HOST_PROGRAMS:
        exe = os.path.join(HOST_BIN_DIR, name)
        cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
               "-I" + os.path.join(ROCM, "include"), os.path.join(HOST_DIR, name + ".cpp"), "-o", exe, "-L" + HERE,
               "-lmoe_gfx950", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN/../..",
               "-Wl,-rpath," + os.path.join(ROCM, "lib")]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("building %s failed:\n%s" % (name, r.stderr))
        out.append(exe)
    return out


def build(force=True, verbose=True):
    """Compile every .hip file and link the shared library, then the host programs.  Returns the library path."""
    if not force and up_to_date():
        return LIB
    os.makedirs(OBJ_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        results = list(ex.map(_compile, sources()))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    build_host_programs()
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
