// query_kernels.h -- point queries on the N^3 tree (reference: svox/csrc/svox_kernel.cu:42-115).
//
// query / query-backward / assign run in two phases per wavefront:
//   1. one lane per point: world->tree transform, clamp, root-to-leaf walk.  For an fp32 octree the
//      walk runs on integer cell coordinates and reads the child rows of the first `lds_nodes`
//      nodes (the top of the tree: nodes are stored parents-before-children) from LDS;
//   2. the 64 lanes together move the 64 leaf records: the output (or grad_output / values) of a
//      wavefront is one contiguous run of 64*K scalars, so consecutive lanes touch consecutive
//      addresses on that side and K-long runs on the tree side, instead of one lane copying K
//      scalars in a serial loop.
// Blocks are persistent (grid-stride over tiles of 256 points) so the LDS copy of the child rows
// is filled once per block.
#pragma once

#include "tree_walk.h"

namespace svox {

constexpr int kQueryThreads = 256;
constexpr int kWave = 64;

enum QueryMode { kQueryGather = 0, kQueryScatterAdd = 1, kQueryAssign = 2 };

template <typename T, bool kOctree>
__device__ __forceinline__ int64_t query_leaf(const TreeDev<T>& tr, const int32_t* lds_child,
                                              int32_t lds_nodes, const T* offset, const T* scaling,
                                              const T* p) {
    T xyz[3] = {p[0], p[1], p[2]};
    transform_coord(xyz, offset, scaling);
    if constexpr (kOctree) {
        const float cx = clamp01(xyz[0]), cy = clamp01(xyz[1]), cz = clamp01(xyz[2]);
        int levels;
        const int32_t leaf = descend_octree(tr.child, lds_child, lds_nodes, tr.capacity,
                                            cell_coord(cx), cell_coord(cy), cell_coord(cz), &levels);
        if (leaf >= 0) return leaf;
        // deeper than the integer coordinates resolve: repeat with the floating-point walk
    }
    T cube;
    int levels;
    return descend_generic<T>(tr.child, tr.capacity, tr.N, xyz, &cube, &levels);
}

// MODE gather:      values[q][0..Kx) = data[leaf_q][0..Kx), ids[q] = leaf_q        (Kx = K)
// MODE scatter-add: target[leaf_q][0..Kx) += values[q][0..Kx)   (target row stride Kx)
// MODE assign:      data[leaf_q][0..Kx) = values[q][0..Kx)      (tree row stride K)
template <typename T, int MODE, bool kOctree>
__global__ __launch_bounds__(kQueryThreads) void query_kernel(TreeDev<T> tr, const T* __restrict__ points,
                                                              int64_t n_points, T* values, T* target,
                                                              int64_t* __restrict__ ids, int32_t Kx,
                                                              int32_t lds_nodes) {
    extern __shared__ int32_t lds_child[];
    if constexpr (kOctree) {
        for (int i = threadIdx.x; i < lds_nodes * 8; i += kQueryThreads) lds_child[i] = tr.child[i];
        __syncthreads();
    }
    T offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t n_tiles = (n_points + kQueryThreads - 1) / kQueryThreads;
    const int64_t row = (MODE == kQueryAssign) ? (int64_t)tr.K : (int64_t)Kx;
    const int step_e = kWave % Kx, step_p = kWave / Kx;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t wave_base = tile * kQueryThreads + (threadIdx.x & ~(kWave - 1));
        const int64_t q = wave_base + lane;
        int64_t leaf = -1;
        if (q < n_points) {
            leaf = query_leaf<T, kOctree>(tr, lds_child, lds_nodes, offset, scaling, points + q * 3);
            if (MODE == kQueryGather && ids) ids[q] = leaf;
        }
        // phase 2: flat index f = p*Kx + e over the wavefront's 64 rows
        const int64_t remaining = n_points - wave_base;
        const int n_rows = remaining < kWave ? (int)(remaining > 0 ? remaining : 0) : kWave;
        const int total = n_rows * Kx;
        int p = lane / Kx, e = lane % Kx;
        T* lin = values + wave_base * Kx;
        for (int f = lane; __any(f < total); f += kWave) {
            // every lane takes part in the shuffle; rows past the end read lane 0's leaf
            const int src_lane = f < total ? p : 0;
            const int lo = __shfl((int)(leaf & 0xffffffff), src_lane);
            const int hi = __shfl((int)(leaf >> 32), src_lane);
            const int64_t lf = ((int64_t)hi << 32) | (uint32_t)lo;
            if (f < total && lf >= 0) {
                if (MODE == kQueryGather) {
                    lin[f] = tr.data[lf * row + e];
                } else if (MODE == kQueryScatterAdd) {
                    atomicAdd(target + lf * row + e, lin[f]);
                } else {
                    tr.data[lf * row + e] = lin[f];
                }
            }
            e += step_e;
            p += step_p;
            if (e >= Kx) {
                e -= Kx;
                p += 1;
            }
        }
    }
}

// calc_corner_kernel, svox_kernel.cu:91-115: climb parent links from the leaf's node to the
// root; per level result = (result + cell index) / N.
template <typename T>
__global__ __launch_bounds__(kQueryThreads) void corners_kernel(const int32_t* __restrict__ parent_depth,
                                                                int32_t N, int64_t capacity,
                                                                const int64_t* __restrict__ indexer,
                                                                int64_t n_leaves, T* __restrict__ out) {
    const int64_t q = blockIdx.x * (int64_t)kQueryThreads + threadIdx.x;
    if (q >= n_leaves) return;
    int32_t node = (int32_t)indexer[q * 4];
    int32_t c[3] = {(int32_t)indexer[q * 4 + 1], (int32_t)indexer[q * 4 + 2],
                    (int32_t)indexer[q * 4 + 3]};
    T res[3] = {T(0), T(0), T(0)};
    const T Nf = (T)N;
    for (int guard = 0; guard < kMaxWalkLevels; ++guard) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            res[i] += (T)c[i];
            res[i] /= Nf;
        }
        if (node <= 0 || node >= capacity) break;
        int32_t packed = parent_depth[(int64_t)node * 2];
        c[2] = packed % N;
        packed /= N;
        c[1] = packed % N;
        packed /= N;
        c[0] = packed % N;
        node = packed / N;
    }
    out[q * 3] = res[0];
    out[q * 3 + 1] = res[1];
    out[q * 3 + 2] = res[2];
}

// Zero-fill used in place of a memset so that a caller may capture the call in a graph.
__global__ __launch_bounds__(256) void zero_kernel(uint4* __restrict__ p16, int64_t n16,
                                                   uint32_t* __restrict__ tail, int n_tail) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const uint4 z = make_uint4(0u, 0u, 0u, 0u);
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n16; i += stride) p16[i] = z;
    if (blockIdx.x == 0 && (int)threadIdx.x < n_tail) tail[threadIdx.x] = 0u;
}

}  // namespace svox
