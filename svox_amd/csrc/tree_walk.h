// tree_walk.h -- root-to-leaf descent of the N^3 tree (reference: query_single_from_root,
// svox/csrc/include/common.cuh:52-90).
//
// Two formulations that return the same leaf and the same leaf-local position:
//
//   descend_generic<T>   the reference's floating-point walk (multiply by N, floor, subtract) for
//                        any branching factor and scalar type.
//
//   OctreeCursor         N == 2, fp32.  Multiplying by 2, taking the floor and subtracting it are
//                        exact in binary floating point, so the cell chosen at level l is bit
//                        (24 - l) of trunc(p * 2^24) and the leaf-local position at depth L is
//                        frac(p * 2^L).  The walk therefore runs on integers, and because a ray's
//                        next sample is close to the previous one, it restarts from the deepest
//                        node whose cell still contains the new point instead of from the root:
//                        the node ids of the previous path are kept in LDS, one column per lane
//                        (keeping only the deepest four levels in registers was measured slower:
//                        more restarts from the root and select chains on the critical path).
#pragma once

#include "fpmath.h"

namespace svox {

constexpr int kMaxWalkLevels = 64;   // a deeper (malformed) tree ends the walk with leaf -1
constexpr int kCoordBits = 24;       // integer cell coordinates hold 24 levels of an octree
constexpr int kPathLevels = 11;      // levels of the previous path remembered per lane

template <typename T>
struct TreeDev {
    T* data;
    const int32_t* child;
    const int32_t* parent_depth;
    const T* extra;
    const T* offset;   // may be null: zero
    const T* scaling;  // may be null: one
    T* weight_accum;
    int64_t capacity;
    int32_t N;
    int32_t K;
    int32_t extra_cols;
    int32_t weight_accum_max;
};

// The octree march kernels may be given, in place of the child table, the copy svox_mark_empty_leaves
// made of it, in which a negative entry is a leaf whose density is not > 0.  Their walk reads every
// negative entry so (the child table of a well-formed tree has none on a cell that can be reached)
// and sets this bit in the leaf id it returns for such a leaf (octree leaf ids stay below 2^30).
constexpr int32_t kEmptyLeafBit = 1 << 30;

template <typename T>
__device__ __forceinline__ void load_transform(const TreeDev<T>& tr, T* offset, T* scaling) {
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        offset[i] = tr.offset ? tr.offset[i] : T(0);
        scaling[i] = tr.scaling ? tr.scaling[i] : T(1);
    }
}

// transform_coord, common.cuh:43-50
template <typename T>
__device__ __forceinline__ void transform_coord(T* q, const T* offset, const T* scaling) {
#pragma unroll
    for (int i = 0; i < 3; ++i) q[i] = fma_(scaling[i], q[i], offset[i]);
}

// The reference's walk.  xyz: in = point in tree coordinates, out = position inside the leaf.
// Returns the packed leaf id node*N^3 + u*N^2 + v*N + w, or -1 for a malformed tree.
template <typename T>
__device__ __forceinline__ int64_t descend_generic(const int32_t* __restrict__ child,
                                                   int64_t capacity, int32_t Ni, T* xyz,
                                                   T* cube_sz, int* levels, bool marked = false) {
    const T N = (T)Ni;
    xyz[0] = clamp01(xyz[0]);
    xyz[1] = clamp01(xyz[1]);
    xyz[2] = clamp01(xyz[2]);
    int64_t node = 0;
    *cube_sz = N;
    for (int level = 1; level <= kMaxWalkLevels; ++level) {
        xyz[0] *= N;
        xyz[1] *= N;
        xyz[2] *= N;
        const int32_t u = (int32_t)floor_(xyz[0]);
        const int32_t v = (int32_t)floor_(xyz[1]);
        const int32_t w = (int32_t)floor_(xyz[2]);
        xyz[0] -= (T)u;
        xyz[1] -= (T)v;
        xyz[2] -= (T)w;
        const int64_t cell = ((node * Ni + u) * Ni + v) * Ni + w;
        const int32_t skip = child[cell];
        if (skip == 0 || (marked && skip < 0)) {
            *levels = level;
            return cell;
        }
        *cube_sz *= N;
        node += skip;
        if (node < 0 || node >= capacity) return -1;
    }
    return -1;
}

// Integer cell coordinates of a clamped point: trunc(p * 2^24), exact.
__device__ __forceinline__ uint32_t cell_coord(float pc) { return (uint32_t)(pc * 16777216.0f); }

__device__ __forceinline__ int cell_at(uint32_t ix, uint32_t iy, uint32_t iz, int level) {
    const unsigned s = (unsigned)(kCoordBits - level);
    const unsigned bx = __builtin_amdgcn_ubfe(ix, s, 1u), by = __builtin_amdgcn_ubfe(iy, s, 1u),
                   bz = __builtin_amdgcn_ubfe(iz, s, 1u);
    return (int)((((bx << 1) | by) << 1) | bz);
}

// One child entry for the point queries: from the rows staged in LDS for nodes below lds_nodes, else
// from memory.  Written as an LDS read that every lane makes (of entry 0 where the node is not
// staged) and a memory read under a condition: a choice between the two pointers would leave the
// compiler with one load through the generic address path, which is the slower way into LDS.
__device__ __forceinline__ int32_t child_entry(const int32_t* __restrict__ child, const int32_t* lds_child,
                                               int32_t lds_nodes, int32_t node, int32_t cell) {
    const bool staged = node < lds_nodes;
    int32_t skip = lds_child[staged ? cell : 0];
    asm volatile("" : "+v"(skip));   // (keeps the two reads apart)
    if (!staged) skip = child[cell];
    return skip;
}

// Octree walk over integer coordinates with no path memory (point queries).
// `lds_child` holds the child rows of nodes [0, lds_nodes); deeper nodes are read from memory.
// Returns the leaf cell index node*8 + cell (or -1) and the number of levels visited.
__device__ __forceinline__ int32_t descend_octree(const int32_t* __restrict__ child,
                                                  const int32_t* lds_child, int32_t lds_nodes,
                                                  int64_t capacity, uint32_t ix, uint32_t iy,
                                                  uint32_t iz, int* levels) {
    int32_t node = 0;
    for (int level = 1; level <= kCoordBits; ++level) {
        const int32_t cell = node * 8 + cell_at(ix, iy, iz, level);
        const int32_t skip = child_entry(child, lds_child, lds_nodes, node, cell);
        if (skip == 0) {
            *levels = level;
            return cell;
        }
        node += skip;
        if (node < 0 || node >= capacity) return -1;
    }
    return -1;  // deeper than the integer coordinates resolve; the host routes such trees elsewhere
}

// The same walk for kPts points of one lane in lockstep: the child reads of the points are
// independent, so they are in flight together and the lane waits once per level instead of once
// per level and point.  leaf[u] = cell index or -1.
template <int kPts>
__device__ __forceinline__ void descend_octree_multi(const int32_t* __restrict__ child, const int32_t* lds_child,
                                                     int32_t lds_nodes, int64_t capacity, const uint32_t* ix,
                                                     const uint32_t* iy, const uint32_t* iz, const bool* valid,
                                                     int32_t* leaf) {
    int32_t node[kPts];
    bool live[kPts];
    bool any_live = false;
#pragma unroll
    for (int u = 0; u < kPts; ++u) {
        node[u] = 0;
        leaf[u] = -1;
        live[u] = valid[u];
        any_live |= live[u];
    }
    for (int level = 1; level <= kCoordBits && any_live; ++level) {
        int32_t cell[kPts], skip[kPts];
#pragma unroll
        for (int u = 0; u < kPts; ++u) {
            cell[u] = node[u] * 8 + cell_at(ix[u], iy[u], iz[u], level);
            skip[u] = 0;
            if (live[u]) skip[u] = child_entry(child, lds_child, lds_nodes, node[u], cell[u]);
        }
        any_live = false;
#pragma unroll
        for (int u = 0; u < kPts; ++u) {
            if (live[u]) {
                if (skip[u] == 0) {
                    leaf[u] = cell[u];
                    live[u] = false;
                } else {
                    node[u] += skip[u];
                    if (node[u] < 0 || node[u] >= capacity) live[u] = false;
                }
            }
            any_live |= live[u];
        }
    }
}

// leaf-local position frac(pc * 2^levels): s - floor(s), exact for the non-negative s of a clamped coordinate, in
// one instruction
__device__ __forceinline__ float leaf_local(float pc, float cube_sz) {
    return __builtin_amdgcn_fractf(pc * cube_sz);
}

// Per-lane cursor that remembers the previous descent.  `path` points at this lane's column of an
// LDS array laid out [kPathLevels + 1][block threads]: path[l * stride], l < kPathLevels, is the node
// whose child row is indexed at level l + 1 (path[0] is the root, node 0); the last row is a dump
// for the levels below kPathLevels, which a restart never resumes from.
struct OctreeCursor {
    int32_t* path;
    int stride;
    uint32_t ix, iy, iz;  // coordinates of the previous query
    int levels;           // levels of the previous leaf, 0 = no previous query
    int32_t leaf;         // its cell index
    int pend_level;       // > 0: a descent was interrupted before reading the child row at this level
    int32_t pend_node;    //      of this node

    static constexpr int32_t kPending = -2;

    __device__ __forceinline__ void reset(int32_t* lane_path, int lane_stride) {
        path = lane_path;
        stride = lane_stride;
        levels = 0;
        leaf = -1;
        pend_level = 0;
        pend_node = 0;
        ix = iy = iz = 0;
    }

    // forget the previous query (a new ray)
    __device__ __forceinline__ void restart() {
        levels = 0;
        pend_level = 0;
    }

    static constexpr int32_t kIdle = -3;

    // Finds the leaf of the point with integer coordinates (nx, ny, nz), reading at most kBudget
    // child entries.  Returns the leaf cell index; kPending if the budget ran out (call again with
    // the same point to go on); -1 if the tree has more levels than the coordinates hold (`levels`
    // becomes 0).  The budget bounds how long the lanes of a wavefront wait for the one lane that
    // has to descend many levels: that lane continues in its next turn instead.
    // Node ids read from the table are clamped into [0, capacity): a malformed tree yields a wrong
    // leaf, never an access outside the table.  The table is smaller than 4 GiB (checked on the
    // host): a 32-bit byte offset from the uniform base lets the load use the scalar-base form.
    //
    // The bookkeeping is written as selects: every lane runs every instruction (in a wavefront that
    // costs nothing more than running it for one lane) and only the table reads sit under a
    // condition.  `go`: this lane searches; a lane that does not keeps its state and returns kIdle.
    template <int kBudget>
    __device__ __forceinline__ int32_t seek_flat(bool go, const int32_t* __restrict__ child, int32_t last_node,
                                                 uint32_t nx, uint32_t ny, uint32_t nz) {
        const bool pending = pend_level > 0;
        const bool have = levels > 0;
        const uint32_t diff = (ix ^ nx) | (iy ^ ny) | (iz ^ nz);
        const int first_diff = diff ? (kCoordBits - 31 + __builtin_clz(diff)) : kCoordBits + 1;
        const bool same = !pending && have && first_diff > levels;   // still inside the previous leaf
        const int from = first_diff < kPathLevels ? first_diff : kPathLevels;
        const int32_t remembered = path[(from - 1) * stride];   // a row of the array for every lane
        int level = pending ? pend_level : (have ? from : 1);
        int32_t node = pending ? pend_node : (have ? remembered : 0);
        const bool moved = go && !pending;
        ix = moved ? nx : ix;
        iy = moved ? ny : iy;
        iz = moved ? nz : iz;
        const bool search = go && !same;
        bool want = search;
        int32_t cell = 0, skip = 0;
#pragma unroll
        for (int it = 0; it < kBudget; ++it) {
            if (want) {
                path[((level <= kPathLevels ? level : kPathLevels + 1) - 1) * stride] = node;
                cell = (node << 3) | cell_at(nx, ny, nz, level);
                skip = *(const int32_t*)((const char*)child + ((uint32_t)cell << 2));
            }
            want = want && skip > 0 && level != kCoordBits;
            node = want ? (int32_t)min((uint32_t)(node + skip), (uint32_t)last_node) : node;
            level = want ? level + 1 : level;
        }
        // want: the budget ran out; skip == 0: found; else more levels than the coordinates hold
        const bool empty = skip < 0;   // a leaf marked empty
        const bool found = search && skip <= 0;
        const bool open = search && skip > 0;
        pend_level = go ? (want ? level : 0) : pend_level;
        pend_node = want ? node : pend_node;
        levels = found ? level : (open ? 0 : levels);
        leaf = found ? (empty ? cell | kEmptyLeafBit : cell) : (open ? -1 : leaf);
        return !go ? kIdle : (want ? kPending : leaf);
    }
};

}  // namespace svox
