// probes.hip -- measurement aids of bench.py, NOT part of the product library: two launches whose only use is to
// measure what the memory system of the GPU serves (scattered cache lines per microsecond, fp32 atomic-add requests
// per microsecond), the ceilings bench.py prices the march kernels against.  Built into libbench_probes.so by
// bench_probes/__init__.py; nothing under svox_amd/ loads it.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// Every group of `lanes` consecutive lanes reads the first lanes * 16 bytes of 4 * iters pseudo-random units of
// the buffer, 16 bytes per lane, four reads in flight.  The checksum keeps the reads alive; the store never
// happens for data a caller can have (it would need two exact 32-bit values).
__global__ __launch_bounds__(256) void gather_probe_kernel(const uint4* __restrict__ buffer, uint64_t n_units,
                                                           int unit16, int lanes, int iters,
                                                           uint4* __restrict__ sink) {
    uint4 acc = make_uint4(0u, 0u, 0u, 0u);
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    const uint32_t piece = tid % (uint32_t)lanes;
    uint32_t seed = tid / (uint32_t)lanes;
    for (int it = 0; it < iters; ++it) {
        uint4 v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            seed = probe_hash(seed + 0x9e3779b9u * (uint32_t)(k + 1));
            const uint64_t unit = ((uint64_t)seed * n_units) >> 32;
            v[k] = buffer[unit * (uint64_t)unit16 + piece];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            acc.x ^= v[k].x;
            acc.y += v[k].y;
            acc.z ^= v[k].z;
            acc.w += v[k].w;
        }
    }
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[blockIdx.x * 256u + threadIdx.x] = acc;
}

// Per round the wavefront adds 1.0f to 64 / run consecutive-float runs at pseudo-random run-aligned places.
__global__ __launch_bounds__(256) void atomic_probe_kernel(float* __restrict__ scratch, uint64_t n_runs, int run,
                                                           int iters) {
    const int lane = threadIdx.x & 63;
    uint32_t seed = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 977u;
    for (int it = 0; it < iters; ++it) {
        seed = probe_hash(seed + 0x9e3779b9u);
        const uint32_t s = probe_hash(seed + (uint32_t)(lane / run));
        const uint64_t at = ((uint64_t)s * n_runs) >> 32;
        atomicAdd(scratch + at * (uint64_t)run + (lane % run), 1.0f);
    }
}

}  // namespace

// Both return 0, -2 for arguments out of range, -5 for a failed launch.
extern "C" __attribute__((visibility("default"))) int bench_gather_probe(const void* buffer, int64_t bytes,
                                                                         int32_t unit_bytes, int32_t lanes_per_unit,
                                                                         int32_t iters, int32_t blocks, void* sink,
                                                                         void* stream) {
    if (!buffer || !sink) return -2;
    if (unit_bytes != 64 && unit_bytes != 128 && unit_bytes != 256) return -2;
    if ((lanes_per_unit != 1 && lanes_per_unit != 4 && lanes_per_unit != 8 && lanes_per_unit != 16) ||
        lanes_per_unit * 16 > unit_bytes)
        return -2;
    if (((uintptr_t)buffer & 15u) || bytes < unit_bytes || bytes / unit_bytes > 0xffffffffll || iters < 1 ||
        blocks < 1 || blocks > (1 << 20))
        return -2;
    hipLaunchKernelGGL(gather_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)buffer, (uint64_t)(bytes / unit_bytes), unit_bytes / 16, lanes_per_unit, iters,
                       (uint4*)sink);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

extern "C" __attribute__((visibility("default"))) int bench_atomic_probe(void* scratch, int64_t bytes,
                                                                         int32_t run_floats, int32_t iters,
                                                                         int32_t blocks, void* stream) {
    if (!scratch) return -2;
    if (run_floats != 1 && run_floats != 4 && run_floats != 16 && run_floats != 64) return -2;
    const int64_t n_runs = bytes / (4 * (int64_t)run_floats);
    if (((uintptr_t)scratch & 63u) || n_runs < 1 || n_runs > 0xffffffffll || iters < 1 || blocks < 1 ||
        blocks > (1 << 20))
        return -2;
    hipLaunchKernelGGL(atomic_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (float*)scratch, (uint64_t)n_runs, run_floats, iters);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}
