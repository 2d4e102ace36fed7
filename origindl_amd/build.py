"""Builds the gfx950 HIP library in-tree: origindl_amd/csrc/*.hip -> origindl_amd/lib/libodl_hip.so.

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm toolchain is installed. The
library is the only thing the Python layer loads; there is no fallback when it is missing."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libodl_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops: the compiler must not form packed FP32 VALU instructions on this hardware.
# -ffp-contract=off: elementwise chains round after every step, as the reference's separate Mat ops do.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src):
    obj = os.path.join(LIB_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(sources()))) as ex:
        results = list(ex.map(_compile, sources()))
    objs = [o for o, _ in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    for o in objs:
        os.remove(o)
    return LIB_PATH


HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIB_DIR, "liborigin_host.so")
CXX = os.environ.get("CXX", "g++")


def build_host(verbose=False):
    """C++ host layer (Mat / Tensor / operators / nn / optim over the C ABI) -> lib/liborigin_host.so.
    Plain g++: no device code."""
    os.makedirs(LIB_DIR, exist_ok=True)
    inc = ["-I" + os.path.join(HOST_DIR, "include"), "-I" + os.path.join(os.path.dirname(HERE), "include")]
    common = [CXX, "-std=c++17", "-O2", "-fPIC", "-Wall", "-Wno-unused-variable"] + inc
    srcs = sorted(glob.glob(os.path.join(HOST_DIR, "src", "*.cpp")))
    link = ["-L" + LIB_DIR, "-lodl_hip", "-Wl,-rpath,$ORIGIN"]
    cmd = common + ["-shared", "-o", HOST_LIB] + srcs + link
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose and res.stdout.strip():
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("host build failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    return HOST_LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print(build_host(verbose="-v" in sys.argv))
