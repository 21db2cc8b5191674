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
// Blocks are persistent (grid-stride over tiles of 512 points, two per lane) so the LDS copy of the
// child rows is filled once per block.
#pragma once

#include "tree_walk.h"

namespace svox {

constexpr int kQueryThreads = 256;
constexpr int kWave = 64;

enum QueryMode { kQueryGather = 0, kQueryScatterAdd = 1, kQueryAssign = 2 };
typedef unsigned int Piece16 __attribute__((ext_vector_type(4)));   // 16 bytes as the non-temporal builtins take them

constexpr int kQueryPts = 2;   // points a lane walks in lockstep (their child reads overlap)

// Leaves of a lane's kQueryPts points: leaf[u] = packed leaf id or -1.
template <typename T, bool kOctree>
__device__ __forceinline__ void query_leaves(const TreeDev<T>& tr, const int32_t* lds_child, int32_t lds_nodes,
                                             const T* offset, const T* scaling, const T* __restrict__ points,
                                             const int64_t* q, int64_t n_points, int64_t* leaf) {
    T xyz[kQueryPts][3];
    bool valid[kQueryPts];
#pragma unroll
    for (int u = 0; u < kQueryPts; ++u) {
        valid[u] = q[u] < n_points;
        leaf[u] = -1;
#pragma unroll
        for (int k = 0; k < 3; ++k) xyz[u][k] = valid[u] ? points[q[u] * 3 + k] : T(0);
        transform_coord(xyz[u], offset, scaling);
    }
    if constexpr (kOctree) {
        uint32_t ix[kQueryPts], iy[kQueryPts], iz[kQueryPts];
        int32_t cell[kQueryPts];
#pragma unroll
        for (int u = 0; u < kQueryPts; ++u) {
            ix[u] = cell_coord(clamp01(xyz[u][0]));
            iy[u] = cell_coord(clamp01(xyz[u][1]));
            iz[u] = cell_coord(clamp01(xyz[u][2]));
        }
        descend_octree_multi<kQueryPts>(tr.child, lds_child, lds_nodes, tr.capacity, ix, iy, iz, valid, cell);
#pragma unroll
        for (int u = 0; u < kQueryPts; ++u) {
            leaf[u] = cell[u];
            valid[u] = valid[u] && cell[u] < 0;   // deeper than the integer coordinates resolve:
        }                                         // repeat those with the floating-point walk
    }
#pragma unroll
    for (int u = 0; u < kQueryPts; ++u) {
        if (valid[u]) {
            T cube;
            int levels;
            leaf[u] = descend_generic<T>(tr.child, tr.capacity, tr.N, xyz[u], &cube, &levels);
        }
    }
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
    constexpr int kTile = kQueryThreads * kQueryPts;   // points per block and iteration
    const int64_t n_tiles = (n_points + kTile - 1) / kTile;
    const int64_t row = (MODE == kQueryAssign) ? (int64_t)tr.K : (int64_t)Kx;
    // records and output rows start on 16-byte boundaries: move 16-byte pieces
    const bool vec16 = (Kx * (int)sizeof(T)) % 16 == 0 && (((uintptr_t)tr.data | (uintptr_t)values) & 15u) == 0;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        // a wavefront owns kQueryPts runs of 64 consecutive points; lane l walks point l of each run
        const int64_t wave_first = tile * kTile + (int64_t)(threadIdx.x / kWave) * (kWave * kQueryPts);
        int64_t q[kQueryPts], leaves[kQueryPts];
#pragma unroll
        for (int u = 0; u < kQueryPts; ++u) q[u] = wave_first + u * kWave + lane;
        query_leaves<T, kOctree>(tr, lds_child, lds_nodes, offset, scaling, points, q, n_points, leaves);
        if (MODE == kQueryGather && ids) {
#pragma unroll
            for (int u = 0; u < kQueryPts; ++u)
                if (q[u] < n_points) ids[q[u]] = leaves[u];
        }
        // phase 2, run by run: the 64 rows of a run, flat index f = p * Kx + e
#pragma unroll
        for (int u = 0; u < kQueryPts; ++u) {
            const int64_t wave_base = wave_first + u * kWave;
            const int64_t leaf = leaves[u];
            const int64_t remaining = n_points - wave_base;
            const int n_rows = remaining < kWave ? (int)(remaining > 0 ? remaining : 0) : kWave;
            T* lin = values + wave_base * Kx;
            const int leaf_lo = (int)(leaf & 0xffffffff), leaf_hi = (int)(leaf >> 32);
            if (MODE == kQueryGather && vec16) {
                // 16-byte pieces: a record is `pieces` of them, and kBatch loads per lane are in flight
                // before the first store (the compiler must assume that the output aliases the tree)
                constexpr int kPer = 16 / (int)sizeof(T);
                constexpr int kBatch = 4;
                const int pieces = Kx / kPer;
                const int total = n_rows * pieces;
                const int step_e = kWave % pieces, step_p = kWave / pieces;
                int p = lane / pieces, e = lane % pieces;
                uint4* lin16 = (uint4*)lin;
                for (int f0 = 0; f0 < total; f0 += kWave * kBatch) {
                    uint4 buf[kBatch];
#pragma unroll
                    for (int b = 0; b < kBatch; ++b) {
                        const int f = f0 + b * kWave + lane;
                        // every lane takes part in the shuffle; rows past the end read lane 0's leaf
                        const int src_lane = f < total ? p : 0;
                        const int lo = __shfl(leaf_lo, src_lane);
                        const int hi = __shfl(leaf_hi, src_lane);
                        const int64_t lf = ((int64_t)hi << 32) | (uint32_t)lo;
                        buf[b] = make_uint4(0u, 0u, 0u, 0u);
                        if (f < total && lf >= 0) buf[b] = ((const uint4*)(tr.data + lf * row))[e];
                        e += step_e;
                        p += step_p;
                        if (e >= pieces) {
                            e -= pieces;
                            p += 1;
                        }
                    }
#pragma unroll
                    for (int b = 0; b < kBatch; ++b) {
                        const int f = f0 + b * kWave + lane;
                        // (stored past the caches' keep-list: the output is written once, and the tree it is gathered
                        // from should stay in the last-level cache: 4 Mi points of a 268 MB tree 0.346 -> 0.332 ms)
                        if (f < total) __builtin_nontemporal_store((Piece16){buf[b].x, buf[b].y, buf[b].z, buf[b].w}, (Piece16*)lin16 + f);
                    }
                }
                continue;
            }
            const int total = n_rows * Kx;
            const int step_e = kWave % Kx, step_p = kWave / Kx;
            int p = lane / Kx, e = lane % Kx;
            for (int f = lane; __any(f < total); f += kWave) {
                const int src_lane = f < total ? p : 0;
                const int lo = __shfl(leaf_lo, src_lane);
                const int hi = __shfl(leaf_hi, src_lane);
                const int64_t lf = ((int64_t)hi << 32) | (uint32_t)lo;
                if (f < total && lf >= 0) {
                    if (MODE == kQueryGather) {
                        __builtin_nontemporal_store(tr.data[lf * row + e], &lin[f]);
                    } else if (MODE == kQueryScatterAdd) {
                        atomicAdd(target + lf * row + e, __builtin_nontemporal_load(&lin[f]));
                    } else {
                        tr.data[lf * row + e] = lin[f];
                    }
                } else if (MODE == kQueryGather && f < total) {
                    lin[f] = T(0);   // malformed tree: no leaf
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

// The child table with the leaves a render skips marked: a leaf cell (child == 0) whose density -- after the shifted
// softplus of rt_kernel.cu:276-277 where `softplus` says so -- is not > thresh receives SVOX_EMPTY_LEAF, every other
// cell its child entry.  One thread per cell.
template <typename T>
__global__ __launch_bounds__(256) void mark_leaves_kernel(const T* __restrict__ data, const int32_t* __restrict__ child,
                                                          int64_t cells, int K, T thresh, bool softplus,
                                                          int32_t* __restrict__ marks) {
    const int64_t i = blockIdx.x * 256ll + threadIdx.x;
    if (i >= cells) return;
    const int32_t c = child[i];
    int32_t m = c;
    if (c == 0) {
        // read past the caches' keep-list: a density is 4 bytes of a line nobody asks for again soon, and 0.7 GB of
        // such lines would push the child table and the marks out of L2 ahead of the render that follows
        // (8 poses of 800x800: marking 0.141 -> 0.129 ms, the render call as a whole 0.811 -> 0.790 ms)
        T sigma = __builtin_nontemporal_load(&data[i * K + (K - 1)]);
        if (softplus) sigma = softplus_m1(sigma);
        m = sigma > thresh ? 0 : SVOX_EMPTY_LEAF;
    }
    marks[i] = m;
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
