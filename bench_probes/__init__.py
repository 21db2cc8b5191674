"""Measurement aids of bench.py (not part of the product library): two probe launches that measure what the GPU's
memory system serves -- scattered cache lines per microsecond and fp32 atomic-add requests per microsecond -- the
ceilings the benchmark prices the march kernels against.  `build()` compiles probes.hip into libbench_probes.so
beside it; the callers time the launches themselves."""
import ctypes
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbench_probes.so")
_lib = None


def build(verbose=False):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", LIB_PATH + ".tmp", os.path.join(HERE, "probes.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def _load():
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (the HIP runtime the library binds to)
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        v, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
        lib.bench_gather_probe.restype = ctypes.c_int
        lib.bench_gather_probe.argtypes = [v, i64, i32, i32, i32, i32, v, v]
        lib.bench_atomic_probe.restype = ctypes.c_int
        lib.bench_atomic_probe.argtypes = [v, i64, i32, i32, i32, v]
        _lib = lib
    return _lib


def _stream(device):
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def gather_probe(buffer, unit_bytes=64, iters=64, blocks=2048, lanes_per_unit=1):
    """Queues the gather probe on `buffer` (a contiguous GPU tensor): blocks * 256 lanes, every `lanes_per_unit`
    consecutive lanes reading the first lanes_per_unit * 16 bytes of 4 * iters pseudo-random `unit_bytes`-sized
    units (64, 128 or 256), four reads in flight per lane.  Returns the number of units read; the caller times the
    call.  A buffer that fits one L2 gives the rate of L2 hits, a large one the rate of L2 misses."""
    import torch
    if not buffer.is_contiguous():
        raise ValueError("gather_probe: buffer must be contiguous")
    sink = torch.empty((int(blocks) * 256, 4), dtype=torch.int32, device=buffer.device)
    with torch.cuda.device(buffer.device):
        rc = _load().bench_gather_probe(buffer.data_ptr(), buffer.numel() * buffer.element_size(), int(unit_bytes),
                                        int(lanes_per_unit), int(iters), int(blocks), sink.data_ptr(),
                                        _stream(buffer.device))
    if rc:
        raise RuntimeError(f"gather_probe: arguments out of range or launch failed ({rc})")
    return int(blocks) * 256 * 4 * int(iters) // int(lanes_per_unit)


def atomic_probe(scratch, run_floats=16, iters=64, blocks=4096):
    """Queues the atomic-add probe on `scratch` (a contiguous float32 GPU tensor whose contents are given up):
    blocks * 256 lanes, each adding 1.0f `iters` times, the lanes of a wavefront to runs of `run_floats`
    consecutive floats (1, 4, 16 or 64) at pseudo-random places.  Returns (adds, 64-byte requests); the caller
    times the call."""
    import torch
    if not scratch.is_contiguous() or scratch.dtype != torch.float32:
        raise ValueError("atomic_probe: scratch must be a contiguous float32 tensor")
    with torch.cuda.device(scratch.device):
        rc = _load().bench_atomic_probe(scratch.data_ptr(), scratch.numel() * 4, int(run_floats), int(iters),
                                        int(blocks), _stream(scratch.device))
    if rc:
        raise RuntimeError(f"atomic_probe: arguments out of range or launch failed ({rc})")
    adds = int(blocks) * 256 * int(iters)
    return adds, adds // min(int(run_floats), 16)
