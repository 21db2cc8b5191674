"""Build libsvox_hip.so for gfx950 with hipcc, in-tree (next to the sources)."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libsvox_hip.so"
SOURCES = ["svox_hip.hip"]
HEADERS = ["fpmath.h", "tree_walk.h", "basis.h", "query_kernels.h", "march_kernels.h",
           os.path.join("..", "..", "include", "svox_hip.h")]

# -ffp-contract=off: the kernels spell their fused multiply-adds out; the compiler adds none.
# -munsafe-fp-atomics: floating-point atomicAdd becomes the hardware global_atomic_add.
# -packed-fp32-ops off: no packed fp32 instructions are generated from scalar code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    "-ffp-contract=off", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def library_path():
    return os.path.join(HERE, LIB_NAME)


def build_library(verbose=True):
    """Compile the HIP sources into svox_amd/csrc/libsvox_hip.so.  Raises on failure."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = library_path()
    tmp = out + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", tmp] + [os.path.join(HERE, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    build_library()
    sys.exit(0)
