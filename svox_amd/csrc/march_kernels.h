// march_kernels.h -- ray marching through the leaves of the N^3 tree: forward rendering, its
// backward pass, the squared-error gradient / Hessian diagonal, the dense-grid weight render and
// the visit counters (reference: svox/csrc/rt_kernel.cu:189-1003).
//
// The tree kernels exist in two flavours that compute the same numbers:
//   GenericPolicy<T>   any branching factor, scalar type, data format, component range, softplus;
//                      the reference's floating-point walk from the root for every sample.
//   OctreePolicy<FMT,D> fp32 octree with the default options (SH with D in {1,4,9,16,25}, or RGBA
//                      with 3 colours): integer-coordinate walk restarted from the previous path
//                      (OctreeCursor), record length and basis size known at compile time.
#pragma once

#include <cstddef>

#include "basis.h"
#include "tree_walk.h"

namespace svox {

constexpr int kMarchThreads = 64;  // one wavefront per block: finished tiles free their slot at once

// Orders the LDS traffic of the block's single wavefront: what a lane wrote before is read by
// any lane after.  The hardware keeps a wavefront's LDS operations in order; this keeps the compiler
// from moving them across and waits for the LDS counter only.  (__syncthreads would also wait for
// every outstanding global load, store and atomic of the wavefront -- the gradient atomics, which
// nothing here has to wait for.)
__device__ __forceinline__ void wave_lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// ------------------------------------------------------------------------------------------------
// ray sources
// ------------------------------------------------------------------------------------------------
template <typename T>
struct RayBatch {
    const T* origins;
    const T* dirs;
    const T* vdirs;
    int64_t n_rays;
};

template <typename T>
struct Camera {
    const T* c2w;
    float fx, fy;
    int width, height;
};

// _dda_unit, rt_kernel.cu:203-220: the segment of the ray inside the unit cube
template <typename T>
__device__ __forceinline__ void dda_unit(const T* cen, const T* invdir, T* tmin, T* tmax) {
    T lo = T(0), hi = T(1e9f);
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const T t1 = -cen[i] * invdir[i];
        const T t2 = t1 + invdir[i];
        lo = max_(lo, min_(t1, t2));
        hi = min_(hi, max_(t1, t2));
    }
    *tmin = lo;
    *tmax = hi;
}

// _dda_unit for a point inside the unit cube -- the leaf-local position of a sample, every coordinate in [0, 1) --
// as the octree walk uses it: the length tmax - tmin of the segment.  There the entry distance is 0 (on every axis
// t1 = -c * inv and t2 = t1 + inv lie on either side of 0, so min(t1, t2) <= 0), and the larger of t1 and t2 is t2
// where inv > 0 and t1 elsewhere, i.e. t1 + max(inv, 0): the same roundings and the same value as dda_unit gives
// (an axis whose inv is NaN drops out of both), in half the instructions of the walk's innermost turn.
__device__ __forceinline__ float leaf_exit(const float* cen, const float* invdir) {
    float hi = 1e9f;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const float t1 = -cen[i] * invdir[i];
        hi = min_(hi, t1 + max_(invdir[i], 0.0f));
    }
    return hi;
}

// cam2world_ray, rt_kernel.cu:758-772: pixel corner (no half-pixel offset), camera looking down
// -z with +y up.  x and y are formed in double and rounded; the radicand is widened for `+ 1.0`.
template <typename T>
__device__ __forceinline__ void cam2world_ray(int ix, int iy, const Camera<T>& cam, T* dir, T* origin) {
    T x = (T)(((double)ix - 0.5 * (double)cam.width) / (double)cam.fx);
    T y = (T)(-((double)iy - 0.5 * (double)cam.height) / (double)cam.fy);
    T z = (T)__builtin_sqrtf((float)((double)fma_(x, x, y * y) + 1.0));
    x /= z;
    y /= z;
    z = (T)(-1.0f / z);
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const T* row = cam.c2w + r * 4;
        dir[r] = fma_(row[2], z, fma_(row[0], x, row[1] * y));
        origin[r] = row[3];
    }
}

// maybe_world2ndc, rt_kernel.cu:775-796 with near = 1
template <typename T>
__device__ __forceinline__ void maybe_world2ndc(const SvoxRenderOptions& opt, T* dir, T* cen) {
    if (opt.ndc_width < 0) return;
    const T near = T(1);
    const T t = -(near + cen[2]) / dir[2];
#pragma unroll
    for (int i = 0; i < 3; ++i) cen[i] = fma_(t, dir[i], cen[i]);
    const float two_f = 2 * opt.ndc_focal;
    const T kx = (T)(two_f / (float)opt.ndc_width);
    const T ky = (T)(two_f / (float)opt.ndc_height);
    dir[0] = -kx * (dir[0] / dir[2] - cen[0] / cen[2]);
    dir[1] = -ky * (dir[1] / dir[2] - cen[1] / cen[2]);
    dir[2] = T(-2) * near / cen[2];
    cen[0] = -kx * (cen[0] / cen[2]);
    cen[1] = -ky * (cen[1] / cen[2]);
    cen[2] = T(1) + T(2) * near / cen[2];
    const T n = norm3(dir);
    dir[0] /= n;
    dir[1] /= n;
    dir[2] /= n;
}

// Ray sources.  The rays of a launch are numbered 0 .. total()-1 ("items"); a wavefront owns the
// `per_wave` consecutive items of chunk chunk_of_block(blockIdx.x) and feeds them to its 64 lanes.
//   Batch: item i is ray i.
//   Image: items are numbered so that 64 consecutive items are one 8x8 pixel tile and 256
//          consecutive items one 16x16 block (four tiles), image after image: the rays a wavefront
//          holds at any time stay close in the tree, and the dispatcher starts the next image's
//          blocks as the previous image's last ones drain.  Items that fall outside the image
//          (sizes that are not multiples of 16) have no ray.  The blocks of an image are counted
//          row by row or (inside_out) ring by ring from the middle of the image: a launch lasts as
//          long as its longest rays, a camera that looks at an object has them in the middle of
//          the picture, and counted from there they start first instead of after the dispatcher
//          has gone through the upper half of the image.
// fetch_item returns the output slot of the item (ray index / pixel index) or -1, and the ray in
// tree coordinates.
template <typename T>
struct BatchSource {
    RayBatch<T> rays;
    int per_wave;
    int refill_at;   // idle lanes that trigger taking new rays
    int xcd_group;   // see chunk_of_block; 1 for unrelated rays
    // > 0 (per_wave a power of two): the wavefront that owns items [w * per_wave, (w + 1) * per_wave)
    // takes the groups of four rays w, w + n_waves, w + 2 * n_waves, ... of the batch instead of one
    // contiguous range.  A batch in some coherent order (the rays of an image, row by row) keeps its
    // long rays together, and the wavefronts that own them would finish long after the others (1M
    // rays of 8 images in tile order: 3x the time of the same rays shuffled, backward 5x); dealt
    // out like this every wavefront gets its share whatever the order, at 2-3 % for a shuffled batch
    // (groups of four keep the reads of the rays in whole 48-byte pieces; single rays cost 14 %).
    int64_t n_waves;
    __device__ __forceinline__ int64_t total() const { return n_waves > 0 ? n_waves * per_wave : rays.n_rays; }
    // rays are numbered as they lie in the batch; with n_waves == 0 item i is ray i
    static constexpr bool kItemsAreSlots = true;
    __device__ __forceinline__ int64_t n_slots() const { return rays.n_rays; }
    __device__ __forceinline__ void view_dir(int64_t slot, T* vdir) const {
#pragma unroll
        for (int k = 0; k < 3; ++k) vdir[k] = rays.vdirs[slot * 3 + k];
    }
    __device__ __forceinline__ int64_t fetch_item(int64_t i, const SvoxRenderOptions&, const T* offset,
                                                  const T* scaling, T* origin, T* dir, T* vdir) const {
        if (n_waves > 0) {
            const int shift = __builtin_ctz((unsigned)per_wave);
            const int64_t j = i & (per_wave - 1), w = i >> shift;
            i = ((((j >> 2) * n_waves + w) << 2) | (j & 3));
        }
        if (i >= rays.n_rays) return -1;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            origin[k] = rays.origins[i * 3 + k];
            dir[k] = rays.dirs[i * 3 + k];
            vdir[k] = rays.vdirs[i * 3 + k];
        }
        transform_coord(origin, offset, scaling);
        return i;
    }
};

__host__ __device__ inline int blocks16_of(int extent) { return (extent + 15) / 16; }

// Which chunk of items the wavefront of block `b` (of gridDim.x) works on.  Workgroups are handed
// to the 8 XCDs in turn (block b runs on XCD b mod 8), and every XCD has its own L2.  With
// group > 1, runs of `group` consecutive chunks go to one XCD, so neighbouring image tiles, whose
// rays read the same child rows and leaf records, share that L2; the runs themselves still rotate
// over the XCDs, which keeps the load balanced.  A bijection on [0, gridDim.x).
__device__ __forceinline__ int64_t chunk_of_block(unsigned b, unsigned n_blocks, int group) {
    constexpr unsigned kXcds = 8;
    if (group <= 1) return b;
    const unsigned span = kXcds * (unsigned)group;
    const unsigned full = n_blocks / span * span;
    if (b >= full) return b;
    const unsigned xcd = b % kXcds, j = b / kXcds;
    return (int64_t)((j / group) * kXcds + xcd) * group + j % group;
}

// Block `rank` of an nbx x nby grid of blocks counted from the middle outwards: the innermost
// rectangle first, then ring after ring (each ring clockwise from its top left corner).
__device__ __forceinline__ void block_inside_out(int rank, int nbx, int nby, int& bx, int& by) {
    int p = (min(nbx, nby) - 1) / 2;
    while (p > 0 && rank >= (nbx - 2 * p) * (nby - 2 * p)) --p;
    const int w = nbx - 2 * p, h = nby - 2 * p;
    const int inner = (w > 2 && h > 2) ? (w - 2) * (h - 2) : 0;
    const int k = rank - inner;
    if (h == 1) {
        bx = p + k; by = p;
    } else if (w == 1) {
        bx = p; by = p + k;
    } else if (k < w) {
        bx = p + k; by = p;
    } else if (k < w + h - 1) {
        bx = p + w - 1; by = p + (k - w + 1);
    } else if (k < 2 * w + h - 2) {
        bx = p + w - 1 - (k - (w + h - 2)); by = p + h - 1;
    } else {
        bx = p; by = p + h - 1 - (k - (2 * w + h - 3));
    }
}

template <typename T>
struct ImageSource {
    Camera<T> cam;          // cam.c2w: pose of image 0
    int n_images;
    int64_t pose_stride;    // scalars between consecutive poses
    int per_wave;           // 64 (one 8x8 tile) or 256 (one 16x16 block)
    int refill_at;          // idle lanes that trigger taking new rays
    int xcd_group;          // see chunk_of_block
    int run;                // > 0: the images advance together, `run` 16x16 blocks at a time
    int inside_out;         // != 0: the blocks of an image are counted from its middle outwards
    // pixels are numbered image by image, row by row; the items run through the tiles instead
    static constexpr bool kItemsAreSlots = false;
    __device__ __forceinline__ int64_t n_slots() const { return (int64_t)n_images * cam.height * cam.width; }
    __device__ __forceinline__ void view_dir(int64_t slot, T* vdir) const {
        const int64_t per_image = (int64_t)cam.height * cam.width;
        const int64_t image = slot / per_image;
        const int pixel = (int)(slot - image * per_image);
        const int iy = pixel / cam.width, ix = pixel - iy * cam.width;
        Camera<T> c = cam;
        c.c2w = cam.c2w + image * pose_stride;
        T origin[3];
        cam2world_ray(ix, iy, c, vdir, origin);
    }
    __device__ __forceinline__ int64_t total() const {
        const int64_t per_image = (int64_t)blocks16_of(cam.width) * blocks16_of(cam.height);
        const int64_t padded = run > 0 ? (per_image + run - 1) / run * run : per_image;
        return (int64_t)n_images * padded * 256;
    }
    __device__ __forceinline__ int64_t fetch_item(int64_t i, const SvoxRenderOptions& opt, const T* offset,
                                                  const T* scaling, T* origin, T* dir, T* vdir) const {
        const int nbx = blocks16_of(cam.width), nby = blocks16_of(cam.height);
        const int64_t block = i >> 8;
        const int within = (int)(i & 255);
        int image, b;
        if (run > 0) {
            // runs of `run` blocks, image after image, then the next run of every image
            const int64_t r = block / run;
            const int64_t round = r / n_images;
            image = (int)(r - round * n_images);
            b = (int)(round * run + (block - r * run));
            if (b >= nbx * nby) return -1;
        } else {
            image = (int)(block / (nbx * nby));
            if (image >= n_images) return -1;
            b = (int)(block - (int64_t)image * (nbx * nby));
        }
        int by = b / nbx, bx = b - by * nbx;
        if (inside_out) block_inside_out(b, nbx, nby, bx, by);
        const int sub = within >> 6, pos = within & 63;
        const int ix = bx * 16 + (sub & 1) * 8 + (pos & 7);
        const int iy = by * 16 + (sub >> 1) * 8 + (pos >> 3);
        if (ix >= cam.width || iy >= cam.height) return -1;
        Camera<T> c = cam;
        c.c2w = cam.c2w + (int64_t)image * pose_stride;
        cam2world_ray(ix, iy, c, dir, origin);
#pragma unroll
        for (int k = 0; k < 3; ++k) vdir[k] = dir[k];
        maybe_world2ndc(opt, dir, origin);
        transform_coord(origin, offset, scaling);
        return ((int64_t)image * cam.height + iy) * cam.width + ix;
    }
};

// ------------------------------------------------------------------------------------------------
// per-ray march state
// ------------------------------------------------------------------------------------------------
template <typename T>
struct RayState {
    T o[3], d[3], inv[3];
    T t, tmax, dscale;
};

// rt_kernel.cu:228-247: scale and normalise the direction, reciprocal in double, clip to the cube
template <typename T>
__device__ __forceinline__ bool setup_ray(RayState<T>& r, const T* origin, const T* dir, const T* scaling) {
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        r.o[i] = origin[i];
        r.d[i] = dir[i] * scaling[i];
    }
    const T s = T(1) / norm3(r.d);
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        r.d[i] *= s;
        r.inv[i] = (T)(1.0 / ((double)r.d[i] + 1e-9));
    }
    r.dscale = s;
    T tmin, tmax;
    dda_unit(r.o, r.inv, &tmin, &tmax);
    r.t = tmin;
    r.tmax = tmax;
    return !(tmax < T(0) || tmin > tmax);
}

// t += delta_t.  If t cannot advance any more (a delta below the spacing of floats at t, or NaN), the
// reference's `while (t < tmax)` loop would never end; the ray is ended after this sample instead.
template <typename T>
__device__ __forceinline__ void advance(RayState<T>& r, T delta_t) {
    const T t_next = r.t + delta_t;
    r.t = t_next > r.t ? t_next : r.tmax;
}

struct Visit {
    int64_t leaf;  // cell index node*N^3 + cell; -1 ends the ray (malformed tree); -2 descent pending
    int levels;
};

// Child entries one lane reads per turn of the octree walk (OctreeCursor::seek_flat).  A lane that needs
// more (its ray crossed the boundary of a large cell and has to descend many levels) goes on in its
// next turn, so that the other lanes of the wavefront do not wait for it: measured, the lanes need
// 2.0 entries per leaf on average, but the slowest lane of a wavefront 4.8.  (Budgets of 1 and 3, and
// extra turns per round for the interrupted lanes, were measured slower.)
constexpr int kSeekBudget = 2;

// One sample with the reference's walk: position, leaf, step length.  rt_kernel.cu:262-275.
template <typename T>
__device__ __forceinline__ Visit step_generic(const TreeDev<T>& tr, const RayState<T>& r, T step_size,
                                              T* delta_t) {
    T pos[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) pos[j] = fma_(r.t, r.d[j], r.o[j]);
    T cube;
    Visit v;
    v.leaf = descend_generic<T>(tr.child, tr.capacity, tr.N, pos, &cube, &v.levels);
    T s0, s1;
    dda_unit(pos, r.inv, &s0, &s1);
    *delta_t = (s1 - s0) / cube + step_size;
    return v;
}

// One turn of the octree walk for the whole wavefront, written flat: the lanes with `go` take one
// sample (slot_leaf, slot_dt) and advance, or keep a descent pending (slot_leaf -1); the others run
// the same instructions without effect.  `broken`: the tree is malformed, the ray ends here.
__device__ __forceinline__ void walk_turn_flat(const TreeDev<float>& tr, RayState<float>& r, OctreeCursor& cur,
                                               float step_size, bool go, bool& broken, int32_t& slot_leaf,
                                               float& slot_dt) {
    float pc[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) pc[j] = clamp01(fma_(r.t, r.d[j], r.o[j]));
    // (trees with another branching factor have no exact integer formulation: every lane takes the reference's
    // floating-point walk below, from the root for every sample, and shares everything else with the octrees)
    const bool octree = tr.N == 2;
    int32_t leaf = go ? -1 : OctreeCursor::kIdle;
    if (octree)
        leaf = cur.seek_flat<kSeekBudget>(go, tr.child, (int32_t)(tr.capacity - 1), cell_coord(pc[0]), cell_coord(pc[1]),
                                          cell_coord(pc[2]));
    // 2^levels and 2^-levels: dividing by the power of two is the multiplication by its reciprocal
    const float cube = __uint_as_float((uint32_t)(127 + cur.levels) << 23);
    float inv_cube = __uint_as_float((uint32_t)(127 - cur.levels) << 23);
    float cells_per_axis = 1.0f;   // N^levels where it is no power of two
    float local[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) local[j] = leaf_local(pc[j], cube);
    const bool deep = leaf == -1;
    if (__any(deep)) {
        if (deep) {
            // more levels than the integer coordinates hold, another branching factor, or a broken tree
            int levels_f;
#pragma unroll
            for (int j = 0; j < 3; ++j) local[j] = pc[j];
            leaf = (int32_t)descend_generic<float>(tr.child, tr.capacity, tr.N, local, &cells_per_axis, &levels_f, true);
            inv_cube = 1.0f / cells_per_axis;
            broken = broken || leaf < 0;
        }
    }
    const float segment = leaf_exit(local, r.inv);
    // (rt_kernel.cu:274 divides by the cell count; for a power of two the product with the reciprocal is the same number)
    const float delta_t = (octree ? segment * inv_cube : segment / cells_per_axis) + step_size;
    const bool ok = leaf >= 0;
    slot_leaf = ok ? leaf : -1;
    slot_dt = ok ? delta_t : 0.0f;
    const float t_next = r.t + delta_t;
    r.t = ok ? (t_next > r.t ? t_next : r.tmax) : r.t;
}

// ------------------------------------------------------------------------------------------------
// policies
// ------------------------------------------------------------------------------------------------
template <typename T>
struct GenericPolicy {
    using scalar = T;
    static constexpr bool kOctree = false;
};

template <int FMT, int D>
struct OctreePolicy {
    using scalar = float;
    static constexpr bool kOctree = true;
    static constexpr int kFormat = FMT;                                // RGBA, SH, or SG for both kinds of lobes
    static constexpr int kBasis = D;                                   // 0 for RGBA
    static constexpr int kRecord = (FMT == SVOX_FORMAT_RGBA) ? 4 : 3 * D + 1;
    // SH: the basis is a closed form of the view direction, cheap enough to evaluate again wherever a
    // colour is formed; lobes (SG, ASG): D exponentials, evaluated once per ray and kept as a row in LDS
    static constexpr bool kForwardRows = FMT == SVOX_FORMAT_SG;
};

// The table of lobes of a tree of spherical gaussians (TreeSpec.extra_data: basis_dim rows [lambda, mu])
// or anisotropic ones ([lambda_x, lambda_y, x-axis, y-axis, z-axis]), and which of the two it is: the two
// formats differ in nothing but the basis of a ray, which is evaluated once per ray, so one set of
// kernels (OctreePolicy<SVOX_FORMAT_SG, D>) serves both and looks at `format` there.
struct Lobes {
    const float* table;
    int cols;
    int format;
};
// A launch that renders only the components [min_comp, max_comp] of the basis (rt_kernel.cu:286-288: the loops over
// the coefficients run over that range) runs on the kernels that keep a ray's basis as a row in LDS (the lobe
// policy, whatever the format: its rows are made by precalc_basis, which knows spherical harmonics too), with the
// row zero outside the range: the full-length colour sums then add 0 * coefficient = 0 for the terms the reference
// leaves out, which leaves the running sum as it is -- the same bits for every finite coefficient (a coefficient
// that is infinite or NaN outside the range would show here and not in the reference) -- and the gradient terms
// of those components are zeros added to zeros.
template <int D>
__device__ __forceinline__ bool partial_range(const SvoxRenderOptions& opt) {
    return opt.min_comp > 0 || opt.max_comp < D - 1;   // (uniform: the same for every lane of the launch)
}
template <int D>
__device__ __forceinline__ void keep_range(const SvoxRenderOptions& opt, float* x) {
#pragma unroll
    for (int i = 0; i < D; ++i) x[i] = (i >= opt.min_comp && i <= opt.max_comp) ? x[i] : 0.0f;
}

// The basis of one ray (maybe_precalc_basis, rt_kernel.cu:111-187) for the policy's format, zero outside the
// launch's component range.
template <class P>
__device__ __forceinline__ void policy_basis(const Lobes& lobes, const SvoxRenderOptions& opt, const float* vdir,
                                             float* out) {
    if constexpr (P::kFormat == SVOX_FORMAT_SH) {
        sh_basis<float>(P::kBasis, vdir, out);
    } else {
        precalc_basis<float>(lobes.format, P::kBasis, lobes.table, lobes.cols, vdir, out);
    }
    if (partial_range<P::kBasis>(opt)) keep_range<P::kBasis>(opt, out);
}

// atomicMax of the reference (common.cuh:152-172): compare-and-swap loop around fmaxf
__device__ __forceinline__ void atomic_max_float(float* addr, float value) {
    unsigned* a = (unsigned*)addr;
    unsigned old = *a, assumed;
    do {
        assumed = old;
        old = atomicCAS(a, assumed, __float_as_uint(max_(value, __uint_as_float(assumed))));
    } while (old != assumed);
}
__device__ __forceinline__ void atomic_max_float(double* addr, double value) {
    unsigned long long* a = (unsigned long long*)addr;
    unsigned long long old = *a, assumed;
    do {
        assumed = old;
        const double m = (double)max_((float)value, (float)__longlong_as_double((long long)assumed));
        old = atomicCAS(a, assumed, (unsigned long long)__double_as_longlong(m));
    } while (old != assumed);
}

// ------------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------------
// trace_ray, rt_kernel.cu:222-321, generic flavour.  `basis` and `acc` are this lane's columns of two LDS arrays
// laid out [index][lane] (stride kMarchThreads): the reference's loops index them at run time, and as register
// arrays they would live in scratch memory.
template <typename T>
__device__ void trace_generic(const TreeDev<T>& tr, const SvoxRenderOptions& opt, const T* origin,
                              const T* dir, const T* vdir, const T* scaling, int out_dim, T* out, T* basis, T* acc) {
    constexpr int S = kMarchThreads;
    RayState<T> r;
    if (!setup_ray(r, origin, dir, scaling)) {
        for (int j = 0; j < out_dim; ++j) out[j] = (T)opt.background_brightness;
        return;
    }
    for (int j = 0; j < out_dim; ++j) acc[j * S] = T(0);
    if (opt.format != SVOX_FORMAT_RGBA) {
        T b[SVOX_MAX_BASIS_DIM];
        precalc_basis<T>(opt.format, opt.basis_dim, tr.extra, tr.extra_cols, vdir, b);
#pragma unroll
        for (int i = 0; i < SVOX_MAX_BASIS_DIM; ++i)
            if (i < opt.basis_dim) basis[i * S] = b[i];
    }
    T light = T(1);
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    bool stopped = false;
    while (r.t < r.tmax) {
        T delta_t;
        const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
        if (v.leaf < 0) break;
        const T* val = tr.data + v.leaf * tr.K;
        T sigma = val[tr.K - 1];
        if (opt.density_softplus) sigma = softplus_m1(sigma);
        if (sigma > (T)opt.sigma_thresh) {
            const T att = exp_sp<T>(-delta_t * r.dscale * sigma);
            const T weight = light * (T(1) - att);
            if (opt.format != SVOX_FORMAT_RGBA) {
                for (int c = 0; c < out_dim; ++c) {
                    const int off = c * opt.basis_dim;
                    T tmp = T(0);
                    for (int i = opt.min_comp; i <= opt.max_comp; ++i) tmp = fma_(basis[i * S], val[off + i], tmp);
                    acc[c * S] = fma_(weight, fma_(sigmoid_(tmp), d_rgb_pad, -pad), acc[c * S]);
                }
            } else {
                for (int c = 0; c < out_dim; ++c)
                    acc[c * S] = fma_(weight, fma_(sigmoid_(val[c]), d_rgb_pad, -pad), acc[c * S]);
            }
            light *= att;
            if (tr.weight_accum) {
                if (tr.weight_accum_max)
                    atomic_max_float(tr.weight_accum + v.leaf, weight);
                else
                    atomicAdd(tr.weight_accum + v.leaf, weight);
            }
            if (light <= (T)opt.stop_thresh) {
                const T scale = (T)(1.0 / (1.0 - (double)light));
                for (int j = 0; j < out_dim; ++j) acc[j * S] *= scale;
                stopped = true;
                break;
            }
        }
        advance(r, delta_t);
    }
    if (!stopped)
        for (int j = 0; j < out_dim; ++j) acc[j * S] = fma_(light, (T)opt.background_brightness, acc[j * S]);
    for (int j = 0; j < out_dim; ++j) out[j] = acc[j * S];
}

// number of set bits of `mask` below this lane
__device__ __forceinline__ int rank_in(unsigned long long mask) {
    return (int)__builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

// trace_ray for the generic policy: one ray per lane, no sharing of work between lanes
template <typename T>
__host__ __device__ inline size_t generic_forward_lds_bytes(int basis_dim, int out_dim) {
    return (size_t)kMarchThreads * (size_t)(basis_dim + out_dim) * sizeof(T);
}
template <typename T, class Source>
__global__ __launch_bounds__(kMarchThreads) void render_forward_generic_kernel(TreeDev<T> tr, Source src,
                                                                               SvoxRenderOptions opt, int out_dim,
                                                                               T* __restrict__ out) {
    // dynamic LDS: (basis_dim + out_dim) scalars of T per lane, generic_forward_lds_bytes
    extern __shared__ __align__(16) unsigned char generic_lds[];
    T* const sh_basis = (T*)generic_lds;
    T* const sh_acc = sh_basis + kMarchThreads * (opt.format == SVOX_FORMAT_RGBA ? 1 : opt.basis_dim);
    T offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    T origin[3], dir[3], vdir[3];
    const int64_t item = blockIdx.x * (int64_t)kMarchThreads + threadIdx.x;
    const int64_t slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
    if (slot < 0) return;
    trace_generic<T>(tr, opt, origin, dir, vdir, scaling, out_dim, out + slot * out_dim, sh_basis + threadIdx.x,
                     sh_acc + threadIdx.x);
}

constexpr int kQueue = 4;  // leaves a lane walks ahead before the wavefront shades them
static_assert(kQueue <= 4, "ShadeShared::who packs the queue slot into two bits");

// Shade list shared by the wavefront: the (lane, slot) pairs of one round whose leaf has to be
// shaded, compacted so that consecutive lanes can take consecutive entries.  kRows: the basis of
// every lane's ray is kept as a row (needed where other lanes multiply with it); otherwise only
// the view direction is kept and the basis is re-evaluated where it is used.
template <int D, bool kRows>
struct ShadeShared;
template <int D>
struct ShadeShared<D, true> {
    int32_t leaf[kQueue * kMarchThreads];       // leaf cell index of entry e
    uint8_t who[kQueue * kMarchThreads];        // owner lane | slot << 6
    float colour[kQueue * kMarchThreads * 3];   // [slot][lane][channel]: sigmoid(basis . coefficients)
    float basis[kMarchThreads * D];             // [lane][coefficient]
};
template <int D>
struct ShadeShared<D, false> {
    int32_t leaf[kQueue * kMarchThreads];
    uint8_t who[kQueue * kMarchThreads];
    float colour[kQueue * kMarchThreads * 3];
    float vdir[kMarchThreads * 3];              // [lane][xyz]
};

// Colours of all list entries, computed by the whole wavefront: item p = 3 * entry + channel goes to
// lane p mod 64.  One item is the reference's dot product for one channel, evaluated in the
// reference's order (coefficient 0 first) from 16-byte loads of the leaf record and the owner
// lane's basis, followed by the sigmoid.
// kWithSigma: the densities of the entries are not known yet (a launch whose marks say that every leaf on the list
// is shaded): the lane of an entry's last channel also reads the density, the scalar after its coefficients, and
// leaves it in sigma_out[slot * 64 + owner].
template <class P, bool kRows, bool kWithSigma = false>
__device__ __forceinline__ void shade_entries(const float* __restrict__ data,
                                              ShadeShared<(P::kBasis > 0 ? P::kBasis : 1), kRows>& sh,
                                              int n_entries, int lane, float* sigma_out = nullptr) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    const int n_items = n_entries * 3;
    for (int p = lane; p < n_items; p += kMarchThreads) {
        const int e = p / 3, c = p - 3 * e;
        const int32_t leaf = sh.leaf[e];
        const int who = sh.who[e];
        const int owner = who & 63, slot = who >> 6;
        const float* rec = data + (int64_t)leaf * K;
        float density = 0.0f;
        if constexpr (kWithSigma) {
            if (c == 2) density = rec[K - 1];
        }
        float s;
        if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
            s = sigmoid_(rec[c]);
        } else {
            const float* co = rec + c * D;
            // the coefficients are asked for first: the basis is evaluated while they arrive
            float cv[D];
#pragma unroll
            for (int i = 0; i < D; ++i) cv[i] = co[i];
            float b[D];
            if constexpr (kRows) {
#pragma unroll
                for (int i = 0; i < D; ++i) b[i] = sh.basis[owner * D + i];
            } else {
                const float vd[3] = {sh.vdir[owner * 3], sh.vdir[owner * 3 + 1], sh.vdir[owner * 3 + 2]};
                sh_basis<float>(P::kBasis, vd, b);
            }
            float tmp = 0.0f;
#pragma unroll
            for (int i = 0; i < D; ++i) tmp = fma_(b[i], cv[i], tmp);
            s = sigmoid_(tmp);
        }
        sh.colour[(slot * kMarchThreads + owner) * 3 + c] = s;
        if constexpr (kWithSigma) {
            if (c == 2) sigma_out[slot * kMarchThreads + owner] = density;
        }
    }
}

// ---- phases of a round shared by the octree kernels --------------------------------------------
// Refill: once `refill_at` lanes are idle and the wavefront's range [next, end) is not used up, the
// idle lanes take the next items, ranked by ballot.  Returns kRoundRefilled (look again), kRoundDone
// (every lane idle, range used up) or kRoundWork.
enum RoundState { kRoundWork, kRoundRefilled, kRoundDone };
template <class Start>
__device__ __forceinline__ RoundState refill_lanes(bool active, int64_t& next, int64_t end, int refill_at,
                                                   Start&& start) {
    const unsigned long long idle = __ballot(!active);
    const int n_idle = __popcll(idle);
    if (next < end && n_idle >= refill_at) {
        if (!active) {
            const int64_t item = next + rank_in(idle);
            if (item < end) start(item);
        }
        next += n_idle;
        return kRoundRefilled;
    }
    return n_idle == kMarchThreads ? kRoundDone : kRoundWork;
}

// Walk: kQueue turns; slot q receives the leaf found in turn q and its step length, or -1 (no live
// ray, or a descent still under way).  `broken` reports a malformed tree: the ray ends there.
__device__ __forceinline__ void walk_turns(const TreeDev<float>& tr, RayState<float>& r, OctreeCursor& cur,
                                           float step, bool active, bool& broken, int32_t* q_leaf, float* q_dt) {
    broken = false;
#pragma unroll
    for (int q = 0; q < kQueue; ++q) {
        const bool go = active && !broken && r.t < r.tmax;
        q_leaf[q] = -1;
        q_dt[q] = 0.0f;
        if (__any(go)) walk_turn_flat(tr, r, cur, step, go, broken, q_leaf[q], q_dt[q]);
    }
}

// Sigma: the densities of the queued leaves, fetched together (the last scalar of each record).
template <int K>
__device__ __forceinline__ void fetch_sigma(const float* __restrict__ data, const int32_t* q_leaf, float* q_sigma) {
#pragma unroll
    for (int q = 0; q < kQueue; ++q) {
        // no leaf in the slot (-1) or a leaf marked empty (kEmptyLeafBit): nothing to read
        q_sigma[q] = (uint32_t)q_leaf[q] < (uint32_t)kEmptyLeafBit ? data[(int64_t)q_leaf[q] * K + (K - 1)] : 0.0f;
    }
}

// density_softplus (rt_kernel.cu:276-277): the march works on log(1 + exp(sigma - 1)) of the stored density.
// q_sigma: in the stored densities of the queued leaves, out the densities the march uses; q_raw keeps the stored
// ones (the gradient's chain factor sigmoid(raw - 1), rt_kernel.cu:471-474, and the notes need them).  A slot
// without a leaf, or with a leaf marked empty, stays at 0.
__device__ __forceinline__ void soften_sigma(bool softplus, const int32_t* q_leaf, float* q_sigma, float* q_raw) {
#pragma unroll
    for (int q = 0; q < kQueue; ++q) q_raw[q] = q_sigma[q];
    if (softplus) {
#pragma unroll
        for (int q = 0; q < kQueue; ++q)
            q_sigma[q] = (uint32_t)q_leaf[q] < (uint32_t)kEmptyLeafBit ? softplus_m1(q_raw[q]) : 0.0f;
    }
}

// Shade list: the (lane, slot) pairs with sigma > thresh, compacted by ballot and prefix count
// (`skip`: none of this lane's).  Returns the number of entries.
template <class Shared>
__device__ __forceinline__ int build_shade_list(Shared& sh, const int32_t* q_leaf, const float* q_sigma,
                                                float thresh, int lane, bool skip = false) {
    int n_entries = 0;
#pragma unroll
    for (int q = 0; q < kQueue; ++q) {
        const bool want = !skip && q_leaf[q] >= 0 && q_sigma[q] > thresh;
        const unsigned long long m = __ballot(want);
        if (want) {
            const int e = n_entries + rank_in(m);
            sh.leaf[e] = q_leaf[q];
            sh.who[e] = (uint8_t)(lane | (q << 6));
        }
        n_entries += __popcll(m);
    }
    return n_entries;
}

// The same list where the marks of the launch say that every leaf they let through is shaded (the marks were made
// with the launch's own sigma_thresh): every queued leaf that is not marked joins, its density still unread.
template <class Shared>
__device__ __forceinline__ int build_shade_list_all(Shared& sh, const int32_t* q_leaf, int lane) {
    int n_entries = 0;
#pragma unroll
    for (int q = 0; q < kQueue; ++q) {
        const bool want = (uint32_t)q_leaf[q] < (uint32_t)kEmptyLeafBit;
        const unsigned long long m = __ballot(want);
        if (want) {
            const int e = n_entries + rank_in(m);
            sh.leaf[e] = q_leaf[q];
            sh.who[e] = (uint8_t)(lane | (q << 6));
        }
        n_entries += __popcll(m);
    }
    return n_entries;
}

// Workspace of the replaying backward: chunks of kChunkRecords records of 3 float2 (leaf and step
// length, density and first sigmoid, the other two sigmoids) followed by one float2 whose x
// holds the index of the ray's next chunk.  Ray number i starts in chunk i; further chunks come
// from the rest of the workspace, of which a wavefront takes a stock of 64 chunks at a time through
// one atomic counter (a heavy image tile needs hundreds, most tiles none); the lanes that need a
// chunk in the same step are ranked by ballot.
constexpr int kStampWords = 6;   // ray count; tree data, child; ray origins, directions; step size and threshold
struct ReplaySpace {
    float2* base;          // chunk c starts at base + c * kChunkFloat2
    int64_t first_shared;  // chunks [0, first_shared) are the rays' first chunks
    int64_t n_chunks;      // chunks [first_shared, n_chunks) are handed out in stocks of kChunkStock
    unsigned long long* stocks_taken;   // counter of the stocks handed out (zero when the launch starts)
    // the noting forward kernels write `stamp` (what the notes belong to) to stamp_at; replay_backward_kernel uses
    // the notes only if it finds its own stamp there
    unsigned long long* stamp_at;
    unsigned long long stamp[kStampWords];
    // one bit per ray (ray i: bit i % 64 of word i / 64).  replay_backward_kernel sets the bits of the
    // rays it could not do from their notes; a launch of render_backward_kernel that is given the
    // bitmap as `only` does those rays and no others
    unsigned long long* undone;
    const unsigned long long* only;
    // > 0: the looks in a row after which a waiting wavefront of render_forward_split_kernel gives up, in place of
    // kSpinLimit (set by a debug flag, so that a test can see what a give-up leaves behind)
    int32_t spin_limit;
};

// whether the workspace carries the stamp this launch expects
__device__ __forceinline__ bool stamp_matches(const ReplaySpace& ws) {
    bool same = true;
#pragma unroll
    for (int i = 0; i < kStampWords; ++i) same = same && ws.stamp_at[i] == ws.stamp[i];
    return same;
}

// The first ray at or after `next` (a wavefront-uniform ray number below `end`) whose 64-ray word of
// the bitmap `only` is not zero, found 64 words at a time; a value >= end if there is none.
__device__ __forceinline__ int64_t skip_clear_words(const unsigned long long* __restrict__ only, int64_t next,
                                                    int64_t end, int lane) {
    while (next < end) {
        const int64_t word = next >> 6, last_word = (end - 1) >> 6;
        const bool some = word + lane <= last_word && only[word + lane] != 0ull;
        const unsigned long long nz = __ballot(some);
        if (nz == 0ull) {
            next = (word + kMarchThreads) << 6;
            continue;
        }
        const int64_t first = (word + __builtin_ctzll(nz)) << 6;
        if (first > next) next = first;
        break;
    }
    return next;
}

// What a launch of render_backward_kernel does:
//   kBackwardPlain   both marches walk the tree;
//   kBackwardSecond  only the second march: the first was made by a noting forward kernel.
// (Notes are taken by render_forward_kernel and render_forward_split_kernel with kNoted and used by
// replay_backward_kernel; render_backward_kernel serves the rays that have none.)
enum BackwardMode { kBackwardPlain = 0, kBackwardSecond = 1 };

// Head of a ray's notes, kept in the spare floats of its first chunk (after the 15 records): the
// link to the next chunk, the number of notes (-1: they did not fit; 0 also for a ray that misses
// the tree), the ray's delta_scale (rt_kernel.cu:228), a flag (1.0f: the ray misses the tree, 2.0f:
// its walk broke off in a malformed tree, 3.0f: the launch gave up on the ray -- count -1, no sum --, else 0.0f)
// and the sum of the backward pass's first march where the noting pass could form it (NoteTaker::finish).
constexpr int kChunkRecords = 15;
constexpr int kChunkFloat2 = (kChunkRecords + 1) * 3;   // 384 bytes
constexpr int kHeadFloat2 = kChunkRecords * 3;          // float2 index of {link, count}, then {delta_scale, -}
constexpr int kChunkStock = 64;   // further chunks a wavefront takes at a time (at most 64 lanes ask at once)

// The notes of one lane's ray while they are taken (by the forward kernels, for replay_backward_kernel
// and replay_se_grad_kernel): every leaf with sigma > 0, in the order the ray meets them.
struct NoteTaker {
    int count, pos;     // notes so far; place in the chunk being written
    bool lost;          // the workspace ran out: the backward pass of this ray will march
    float2* first;      // the ray's own chunk, which also holds the head of its notes
    float2* chunk;      // the chunk being written

    __device__ __forceinline__ void begin(const ReplaySpace& ws, int64_t slot) {
        count = 0;
        pos = 0;
        lost = false;
        first = ws.base + slot * kChunkFloat2;
        chunk = first;
    }
    // A ray that misses the tree: no notes, flagged as a miss.
    static __device__ __forceinline__ void missed(const ReplaySpace& ws, int64_t slot) {
        ws.base[slot * kChunkFloat2 + kHeadFloat2] = make_float2(0.0f, __int_as_float(0));
        ws.base[slot * kChunkFloat2 + kHeadFloat2 + 1] = make_float2(0.0f, 1.0f);
    }
    // Called by all lanes of the wavefront together; `note`: this lane has a leaf to note.  Lanes whose
    // chunk is full take the next chunks of the wavefront's stock [shared_next, shared_end), in lane
    // order; a new stock costs one atomic on the workspace's counter (what is left of the old one is
    // given up).
    __device__ __forceinline__ void take(const ReplaySpace& ws, int64_t& shared_next, int64_t& shared_end, int lane,
                                         bool note, int32_t leaf, float dt, float sigma, const float* s) {
        const bool need = note && !lost && pos == kChunkRecords;
        const unsigned long long m = __ballot(need);
        if (m) {
            if (shared_next + __popcll(m) > shared_end) {
                unsigned long long t = 0;
                if (lane == 0) t = atomicAdd(ws.stocks_taken, 1ull);
                const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)t);
                const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(t >> 32));
                const int64_t stock = (int64_t)(((unsigned long long)hi << 32) | lo);
                shared_next = ws.first_shared + stock * kChunkStock;
                shared_end = shared_next + kChunkStock < ws.n_chunks ? shared_next + kChunkStock : ws.n_chunks;
                if (shared_next > shared_end) shared_next = shared_end;
            }
            const int64_t mine = shared_next + rank_in(m);
            if (need) {
                if (mine < shared_end) {
                    chunk[kHeadFloat2] = make_float2(__int_as_float((int32_t)mine), 0.0f);
                    chunk = ws.base + mine * kChunkFloat2;
                    pos = 0;
                } else {
                    lost = true;
                }
            }
            shared_next += __popcll(m);
        }
        if (note) {
            if (!lost) {
                float2* e = chunk + pos * 3;
                e[0] = make_float2(__int_as_float(leaf), dt);
                e[1] = make_float2(sigma, s[0]);
                e[2] = make_float2(s[1], s[2]);
                pos += 1;
            }
            count += 1;
        }
    }
    // The head of the notes: the count beside the link (written when the first chunk filled up), -1 if
    // the notes are incomplete; then the ray's delta_scale and 2.0f if the walk broke off in a
    // malformed tree; then, from a noting pass that had the gradient of the picture at hand, the sum
    // the backward pass forms in its first march (render_backward_kernel<kBackwardSecond> starts from it).
    // The notes of a ray whose launch gave up on it (the bounded wait of render_forward_split_kernel ran out): no
    // count and no sum of the first march (flag 3.0f): the backward pass marches this ray twice.
    __device__ __forceinline__ void give_up(float dscale) {
        ((float*)(first + kHeadFloat2))[1] = __int_as_float(-1);
        first[kHeadFloat2 + 1] = make_float2(dscale, 3.0f);
        first[kHeadFloat2 + 2] = make_float2(0.0f, 0.0f);
    }
    __device__ __forceinline__ void finish(bool broken, float dscale, float march1_sum = 0.0f) {
        ((float*)(first + kHeadFloat2))[1] = __int_as_float(lost || broken ? -1 : count);
        first[kHeadFloat2 + 1] = make_float2(dscale, broken ? 2.0f : 0.0f);
        first[kHeadFloat2 + 2] = make_float2(march1_sum, 0.0f);
    }
};

// What a noting pass that has the gradient of the picture at hand accumulates per ray beside its notes:
// the sum the backward pass forms in its first march (rt_kernel.cu:358-419; the same expressions, in
// the same order, as march 1 of render_backward_kernel), so that a ray whose notes do not fit needs
// only the second march afterwards.
struct March1Sum {
    float go[3], light, accum;
    __device__ __forceinline__ void begin(const float* __restrict__ grad_out, int64_t slot) {
        go[0] = grad_out[slot * 3];
        go[1] = grad_out[slot * 3 + 1];
        go[2] = grad_out[slot * 3 + 2];
        light = 1.0f;
        accum = 0.0f;
    }
    // a leaf with sigma > 0 and the sigmoids s of its colour
    __device__ __forceinline__ void leaf(float dt, float sigma, float dscale, const float* s, float d_rgb_pad, float pad) {
        const float att = expf_fixed(-dt * sigma * dscale);
        const float weight = light * (1.0f - att);
        float total_color = 0.0f;
#pragma unroll
        for (int c = 0; c < 3; ++c) total_color = fma_(fma_(s[c], d_rgb_pad, -pad), go[c], total_color);
        light *= att;
        accum = fma_(weight, total_color, accum);
    }
    __device__ __forceinline__ float end(float bg) const {
        const float total_grad = (go[0] + go[1]) + go[2];
        return fma_(light * bg, total_grad, accum);
    }
};

// trace_ray, octree flavour: a persistent wavefront working in rounds.
//
//   refill    lanes whose ray has ended take the next rays of the wavefront's range (ranked by
//             ballot among the idle lanes) once `refill_at` lanes are idle: rays differ wildly in
//             length, and a finished lane does not wait for the longest ray of the wavefront;
//   walk      kQueue turns; in a turn every live lane advances its ray by one leaf and remembers
//             (leaf, step length), or, if the descent needs more than kSeekBudget child reads,
//             goes on with it in its next turn.  The next position depends only on the tree, not
//             on the leaf's contents, so this phase waits for child-table reads only;
//   sigma     the densities of the remembered leaves are fetched together (kQueue loads in flight);
//   shade     the leaves with sigma > sigma_thresh of all lanes form one list, and the wavefront
//             evaluates their colours together (shade_entries), all 64 lanes busy whatever the
//             number of rays that hit something;
//   composite every lane folds its leaves, in order, into its colour and transmittance, stops at
//             stop_thresh and writes the pixel when the ray ends.
// A ray that stops early has walked at most kQueue - 1 leaves too far; the values are the same as
// when every leaf is shaded on the spot.
// kAccum: the compositing weight of every shaded leaf is also added to (or maximised into)
// tr.weight_accum at the leaf's cell index (rt_kernel.cu:298-304).
// kRefill: the wavefront owns more than 64 rays and refills idle lanes; without it the 64 rays are
// set up once before the loop, and nothing the set-up needs stays live inside it.
// kNoted: the forward pass of a training step.  The picture is composed as without it; beside it the
// launch leaves in the workspace the notes the backward pass works from (NoteTaker): every leaf with
// sigma > 0 of the whole ray, so a ray is walked to its end also after its picture stopped early, and
// the colours of the leaves at or below sigma_thresh are evaluated too.  With out == nullptr only the
// notes are taken (the backward pass without a forward pass before it); kGrad: that backward pass's
// grad_out is given, and the sum of its first march is formed on the way (March1Sum).
// kAllShaded: tr.child is a marked copy of the child table made with this launch's sigma_thresh (and softplus
// setting): a leaf that is not marked has sigma > sigma_thresh, so the round has no density phase -- every
// unmarked leaf goes on the shade list and its density arrives with its coefficients (one round trip to memory
// per round instead of two that wait for one another).
template <class P, class Source, bool kAccum, bool kRefill, bool kNoted = false, bool kGrad = false,
          bool kAllShaded = false>
__global__ __launch_bounds__(kMarchThreads) void render_forward_kernel(TreeDev<float> tr, Source src,
                                                                       SvoxRenderOptions opt,
                                                                       float* __restrict__ out, ReplaySpace ws,
                                                                       const float* __restrict__ grad_out = nullptr) {
    static_assert(!kAllShaded || (!kNoted && !kAccum), "notes and weights look at leaves the marks may hide");
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    __shared__ int32_t path[(kPathLevels + 1) * kMarchThreads];
    __shared__ ShadeShared<D, P::kForwardRows> sh;
    __shared__ float sh_sigma[kAllShaded ? kQueue * kMarchThreads : 1];
    const int lane = threadIdx.x;
    float offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    const float step = opt.step_size, sigma_thresh = opt.sigma_thresh, stop_thresh = opt.stop_thresh;

    int64_t next = chunk_of_block(blockIdx.x, gridDim.x, src.xcd_group) * (int64_t)src.per_wave;
    const int64_t total = src.total();
    const int64_t end = next + src.per_wave < total ? next + src.per_wave : total;

    if constexpr (kNoted) {
        if (blockIdx.x == 0 && lane < kStampWords) ws.stamp_at[lane] = ws.stamp[lane];
    }

    RayState<float> r;
    float acc[3] = {0.f, 0.f, 0.f};
    float light = 1.0f;
    int64_t slot = -1;
    bool active = false;
    bool painted = false;   // kNoted: the ray's picture is finished (early stop), its notes go on
    NoteTaker notes;
    March1Sum sum1;
    int64_t shared_next = 0, shared_end = 0;   // the wavefront's stock of chunks for notes (uniform)
    OctreeCursor cur;
    cur.reset(path + lane, kMarchThreads);

    // takes ray `item` into this lane: a miss is answered at once, a hit becomes the lane's ray
    auto start = [&](int64_t item) {
        float origin[3], dir[3], vdir[3];
        slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
        if (slot < 0) return;
        if (setup_ray(r, origin, dir, scaling)) {
            if constexpr (P::kFormat == SVOX_FORMAT_SH) {
                sh.vdir[lane * 3] = vdir[0];
                sh.vdir[lane * 3 + 1] = vdir[1];
                sh.vdir[lane * 3 + 2] = vdir[2];
            } else if constexpr (P::kForwardRows) {
                float basis[D];
                policy_basis<P>(Lobes{tr.extra, tr.extra_cols, opt.format}, opt, vdir, basis);
#pragma unroll
                for (int i = 0; i < D; ++i) sh.basis[lane * D + i] = basis[i];
            }
            acc[0] = acc[1] = acc[2] = 0.0f;
            light = 1.0f;
            cur.restart();
            active = true;
            if constexpr (kNoted) {
                painted = out == nullptr;   // no picture asked for: nothing to compose
                notes.begin(ws, slot);
                if constexpr (kGrad) sum1.begin(grad_out, slot);
            }
        } else {
            if (!kNoted || out) {
                out[slot * 3] = bg;
                out[slot * 3 + 1] = bg;
                out[slot * 3 + 2] = bg;
            }
            if constexpr (kNoted) NoteTaker::missed(ws, slot);
        }
    };
    if constexpr (!kRefill) {
        if (next + lane < end) start(next + lane);
    }

    while (true) {
        if constexpr (kRefill) {
            const RoundState state = refill_lanes(active, next, end, src.refill_at, start);
            if (state == kRoundRefilled) continue;
            if (state == kRoundDone) break;
        } else {
            if (!__any(active)) break;
        }

        // ---- walk
        int32_t q_leaf[kQueue];
        float q_dt[kQueue];
        bool broken;
        walk_turns(tr, r, cur, step, active, broken, q_leaf, q_dt);
        // ---- sigma
        float q_sigma[kQueue], q_raw[kQueue];   // (q_raw: what the notes keep, the stored density)
        int n_entries;
        if constexpr (kAllShaded) {
            n_entries = build_shade_list_all(sh, q_leaf, lane);
        } else {
            fetch_sigma<K>(tr.data, q_leaf, q_sigma);
            soften_sigma(opt.density_softplus, q_leaf, q_sigma, q_raw);
            // ---- shade list
            n_entries = build_shade_list(sh, q_leaf, q_sigma, kNoted ? 0.0f : sigma_thresh, lane);
        }
        bool stopped = false;
        if (n_entries > 0) {   // most rounds of a ray pass through empty space: nothing to shade
            wave_lds_sync();   // list and view directions are visible to every lane
            shade_entries<P, P::kForwardRows, kAllShaded>(tr.data, sh, n_entries, lane, sh_sigma);
            wave_lds_sync();
            if constexpr (kAllShaded) {
#pragma unroll
                for (int q = 0; q < kQueue; ++q) {
                    const bool listed = (uint32_t)q_leaf[q] < (uint32_t)kEmptyLeafBit;
                    const float raw = sh_sigma[q * kMarchThreads + lane];
                    q_sigma[q] = listed ? (opt.density_softplus ? softplus_m1(raw) : raw) : 0.0f;
                }
            }
            // ---- composite
            // the attenuations and padded colours of the four slots do not depend on one another: they
            // are evaluated side by side, and only the products with the transmittance form a chain
            float q_att[kQueue], q_rgb[kQueue][3], q_s[kQueue][3];
#pragma unroll
            for (int q = 0; q < kQueue; ++q) {
                q_att[q] = expf_fixed(-q_dt[q] * r.dscale * q_sigma[q]);
                const float* s = sh.colour + (q * kMarchThreads + lane) * 3;
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    q_s[q][c] = s[c];
                    q_rgb[q][c] = fma_(s[c], d_rgb_pad, -pad);
                }
            }
#pragma unroll
            for (int q = 0; q < kQueue; ++q) {
                const bool take = active && !painted && q_leaf[q] >= 0 && !stopped && q_sigma[q] > sigma_thresh;
                const float weight = light * (1.0f - q_att[q]);
#pragma unroll
                for (int c = 0; c < 3; ++c) acc[c] = take ? fma_(weight, q_rgb[q][c], acc[c]) : acc[c];
                light = take ? light * q_att[q] : light;
                if constexpr (kAccum) {
                    if (take) {
                        if (tr.weight_accum_max)
                            atomic_max_float(tr.weight_accum + q_leaf[q], weight);
                        else
                            atomicAdd(tr.weight_accum + q_leaf[q], weight);
                    }
                }
                stopped = stopped || (take && light <= stop_thresh);
                if constexpr (kNoted) {
                    const bool note = active && q_leaf[q] >= 0 && q_sigma[q] > 0.0f;
                    notes.take(ws, shared_next, shared_end, lane, note, q_leaf[q], q_dt[q], q_raw[q], q_s[q]);
                    if constexpr (kGrad) {
                        if (note) sum1.leaf(q_dt[q], q_sigma[q], r.dscale, q_s[q], d_rgb_pad, pad);
                    }
                }
            }
        }
        if (active) {
            if (stopped) {
                // rt_kernel.cu:306-313: rescale and leave without the background (done here, once
                // per round, with the transmittance the ray stopped at)
                const float scale = (float)(1.0 / (1.0 - (double)light));
                out[slot * 3] = acc[0] * scale;
                out[slot * 3 + 1] = acc[1] * scale;
                out[slot * 3 + 2] = acc[2] * scale;
                if constexpr (kNoted)
                    painted = true;   // the notes go on to the end of the ray
                else
                    active = false;
            }
            if (active && (broken || !(r.t < r.tmax))) {
                if (!painted) {
                    out[slot * 3] = fma_(light, bg, acc[0]);
                    out[slot * 3 + 1] = fma_(light, bg, acc[1]);
                    out[slot * 3 + 2] = fma_(light, bg, acc[2]);
                }
                if constexpr (kNoted) notes.finish(broken, r.dscale, kGrad ? sum1.end(bg) : 0.0f);
                active = false;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// backward
// ------------------------------------------------------------------------------------------------
// trace_ray_backward, rt_kernel.cu:323-477, generic flavour: one ray per lane, the reference's two marches --
// <render, grad_out> and the colour gradient in the first, the density gradient in the second; both test
// sigma > 0 and never stop early.  The colour terms are the reference's products (basis[i] * tmp2) but are not
// scattered lane by lane: a lane whose sample has density leaves its factors (tmp2 per channel) and the offset of its
// leaf in LDS, the lanes of a step that did so are listed, and the wavefront adds the listed records flat -- scalar f
// of the list from lane f mod 64, so that consecutive scalars of a record go out together, one request per 64 bytes
// instead of one per scalar (the memory system takes atomic adds at a fixed rate of requests).  For that the lanes
// of a wavefront stay in the loop of the first march until the last of them is through.  The basis of a ray and its
// grad_out sit in LDS as well, where the runtime-indexed loops of the reference can address them (in registers such
// arrays end up in scratch memory).
// Dynamic LDS, in scalars of T per lane: basis_dim (1 for RGBA) made odd, so that the lanes' rows start in different
// banks, + 2 * out_dim, then 8 bytes (leaf offset) and 1 byte (list) per lane: generic_backward_lds_bytes.
template <typename T>
__host__ __device__ inline size_t generic_backward_lds_bytes(int basis_dim, int out_dim) {
    return (size_t)kMarchThreads * ((size_t)((basis_dim | 1) + 2 * out_dim) * sizeof(T) + sizeof(int64_t) + 1);
}

template <typename T, class Source>
__global__ __launch_bounds__(kMarchThreads) void render_backward_generic_kernel(
    TreeDev<T> tr, Source src, SvoxRenderOptions opt, int out_dim, const T* __restrict__ grad_out,
    T* __restrict__ grad_data) {
    extern __shared__ __align__(16) unsigned char generic_lds[];
    const int lane = threadIdx.x;
    const bool rgba = opt.format == SVOX_FORMAT_RGBA;
    const int bd = (rgba ? 1 : opt.basis_dim) | 1;                          // row length, odd
    T* const sh_basis = (T*)generic_lds;                                    // [lane * bd + i]
    T* const sh_go = sh_basis + kMarchThreads * bd;                         // [c * 64 + lane]: grad_out of the ray
    T* const sh_factor = sh_go + kMarchThreads * out_dim;                   // [c * 64 + lane]: tmp2 of the sample
    int64_t* const sh_base = (int64_t*)(sh_factor + kMarchThreads * out_dim);   // [lane]: leaf * K
    uint8_t* const sh_list = (uint8_t*)(sh_base + kMarchThreads);           // lanes with a record in this step

    T offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    T origin[3], dir[3], vdir[3];
    const int64_t item = blockIdx.x * (int64_t)kMarchThreads + lane;
    const int64_t slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
    RayState<T> r;
    bool alive = slot >= 0 && setup_ray(r, origin, dir, scaling);
    if (alive) {
        if (!rgba) {
            T basis[SVOX_MAX_BASIS_DIM];
            precalc_basis<T>(opt.format, opt.basis_dim, tr.extra, tr.extra_cols, vdir, basis);
#pragma unroll
            for (int i = 0; i < SVOX_MAX_BASIS_DIM; ++i)
                if (i < opt.basis_dim) sh_basis[lane * bd + i] = basis[i];
        }
        for (int j = 0; j < out_dim; ++j) sh_go[j * kMarchThreads + lane] = grad_out[slot * out_dim + j];
    }
    wave_lds_sync();
    const T* const my_basis = sh_basis + lane * bd;
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    const int lo = rgba ? 0 : opt.min_comp;
    const int n_comp = rgba ? 1 : (opt.max_comp - opt.min_comp + 1 > 0 ? opt.max_comp - opt.min_comp + 1 : 0);
    const int per_record = out_dim * n_comp;
    const T tmin = alive ? r.t : T(0);
    T accum = T(0);
    {
        T light = T(1);
        while (__any(alive && r.t < r.tmax)) {
            bool emit = false;
            if (alive && r.t < r.tmax) {
                T delta_t;
                const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
                if (v.leaf < 0) {
                    alive = false;   // a broken tree: the reference leaves the ray here, second march included
                } else {
                    const int64_t base = v.leaf * tr.K;
                    const T* val = tr.data + base;
                    T sigma = val[tr.K - 1];
                    if (opt.density_softplus) sigma = softplus_m1(sigma);
                    if (sigma > T(0)) {
                        const T att = exp_sp<T>(-delta_t * sigma * r.dscale);
                        const T weight = light * (T(1) - att);
                        T total_color = T(0);
                        for (int c = 0; c < out_dim; ++c) {
                            const T go_c = sh_go[c * kMarchThreads + lane];
                            T sg;
                            if (!rgba) {
                                const int off = c * opt.basis_dim;
                                T tmp = T(0);
                                for (int i = opt.min_comp; i <= opt.max_comp; ++i)
                                    tmp = fma_(my_basis[i], val[off + i], tmp);
                                sg = sigmoid_(tmp);
                                sh_factor[c * kMarchThreads + lane] =
                                    (T)((double)(weight * sg) * (1.0 - (double)sg) * (double)go_c * (double)d_rgb_pad);
                            } else {
                                sg = sigmoid_(val[c]);
                                sh_factor[c * kMarchThreads + lane] = weight * sg * (T(1) - sg) * go_c * d_rgb_pad;
                            }
                            total_color = fma_(fma_(sg, d_rgb_pad, -pad), go_c, total_color);
                        }
                        sh_base[lane] = base;
                        emit = per_record > 0;
                        light *= att;
                        accum = fma_(weight, total_color, accum);
                    }
                    advance(r, delta_t);
                }
            }
            // the records of this step, added by the whole wavefront
            const unsigned long long m = __ballot(emit);
            if (m != 0) {
                if (emit) sh_list[rank_in(m)] = (uint8_t)lane;
                wave_lds_sync();
                const int n_scalars = __popcll(m) * per_record;
                for (int f = lane; f < n_scalars; f += kMarchThreads) {
                    const int rec = f / per_record, e = f - rec * per_record;
                    const int c = e / n_comp, i = lo + (e - c * n_comp);
                    const int owner = sh_list[rec];
                    const T factor = sh_factor[c * kMarchThreads + owner];
                    if (rgba)
                        atomicAdd(grad_data + sh_base[owner] + c, factor);
                    else
                        atomicAdd(grad_data + sh_base[owner] + c * opt.basis_dim + i, sh_basis[owner * bd + i] * factor);
                }
                wave_lds_sync();
            }
        }
        if (alive) {
            T total_grad = T(0);
            for (int j = 0; j < out_dim; ++j) total_grad += sh_go[j * kMarchThreads + lane];
            accum = fma_(light * (T)opt.background_brightness, total_grad, accum);
        }
    }
    if (alive) {
        T light = T(1);
        r.t = tmin;
        while (r.t < r.tmax) {
            T delta_t;
            const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
            if (v.leaf < 0) break;
            const int64_t base = v.leaf * tr.K;
            const T* val = tr.data + base;
            T sigma = val[tr.K - 1];
            const T raw_sigma = sigma;
            if (opt.density_softplus) sigma = softplus_m1(sigma);
            if (sigma > T(0)) {
                const T att = exp_sp<T>(-delta_t * sigma * r.dscale);
                const T weight = light * (T(1) - att);
                T total_color = T(0);
                for (int c = 0; c < out_dim; ++c) {
                    const T go_c = sh_go[c * kMarchThreads + lane];
                    T sg;
                    if (!rgba) {
                        const int off = c * opt.basis_dim;
                        T tmp = T(0);
                        for (int i = opt.min_comp; i <= opt.max_comp; ++i) tmp = fma_(my_basis[i], val[off + i], tmp);
                        sg = sigmoid_(tmp);
                    } else {
                        sg = sigmoid_(val[c]);
                    }
                    total_color = fma_(fma_(sg, d_rgb_pad, -pad), go_c, total_color);
                }
                light *= att;
                accum = fma_(-weight, total_color, accum);
                const T chain = opt.density_softplus ? sigmoid_(raw_sigma - T(1)) : T(1);
                atomicAdd(grad_data + base + tr.K - 1, delta_t * r.dscale * fma_(total_color, light, -accum) * chain);
            }
            advance(r, delta_t);
        }
    }
}

// value of `v` in lane `k` (k uniform across the wavefront)
__device__ __forceinline__ float read_lane(float v, int k) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), k));
}

// trace_ray_backward, octree flavour: a persistent wavefront working in the forward kernel's rounds
// (refill, walk, sigma, shade, composite).
//
// A lane runs its ray twice.  March 1 accumulates <render, grad_out> and writes nothing.  March 2
// replays the ray and produces, per visited leaf with sigma > 0, the reference's gradient record:
// basis[i] * tmp2[c] for the colour coefficients and the density term.  The records are not
// scattered lane by lane: the records of a round are listed in LDS (RecordList) and added by the
// whole wavefront, and where several rays of the wavefront sit in the same leaf their records are
// summed first (group_by_leaf), so that the leaf receives one atomic per element instead of one per
// ray.  The per-term products are the reference's; only the order in which they are added up differs.
// Both marches test sigma > 0 and never stop early (rt_kernel.cu:377, 441).
//
// Gradient records of a round.  A record is the K-long vector (basis[i] * tmp2[c] for the colour
// coefficients, g_sigma last) of a lane, to be added at a leaf.  The records of the queue slots are
// collected in LDS -- in the shade list's storage, which is dead once the colours are evaluated --
// and added together.  The list is flushed when it is full and at the end of the round.  Two forms:
//   flat        the n * K scalars of the list, scalar f from lane f mod 64, so that every atomic
//               instruction covers 64 consecutive scalars whatever K is;
//   by record   the lanes tied to elements (add_records_by_leaf): the list is cut into 64 / K slices
//               of consecutive records and lane l serves element l % K of slice l / K (of every
//               record, in two or more steps, if K > 64).  Which element a lane serves never changes,
//               so an addition costs about half the instructions of running over the flat list; the
//               price is idle lanes where K does not divide 64.  Consecutive records of the same leaf
//               are summed in registers and added once.  term(rec, e, t) gives the NV values of
//               element e of record rec, emit(leaf, e, sum) adds them.
// Records longer than half a wavefront (K > 32: one record at a time either way) are added by
// RecordList::add_held in both forms: the by-record scheme with the values of a record handed round by
// readlane instead of read through LDS one after the other.
// Before either, group_by_leaf looks for leaves that several records of the list share; if enough do,
// the list is put in an order that brings the records of a leaf together and added by record.

// Scratch of group_by_leaf, in LDS that is dead while records are added.
struct GroupScratch {
    uint8_t table[256];              // hash of a leaf -> some record of the list with that hash
    uint8_t order[kMarchThreads];    // position in the grouped order -> record
    int32_t leaf[kMarchThreads];     // position in the grouped order -> its leaf
};
// The list is regrouped if at least one record in kMergeMinShare repeats the leaf of another one.
// Where rays do not share leaves (a shuffled training batch) looking for repeats is pure cost, so a
// wavefront that found too few looks again only kMergeRecheck flushes later; one that found enough
// looks at every flush (the look is small beside the regrouping it decides on).
constexpr int kMergeMinShare = 2;
constexpr int kMergeRecheck = 8;
struct MergeState {
    int skip = 0;   // flushes left before the next look (wavefront-uniform)
};

// n <= 64 records; record r's leaf is leaves[r] (visible to every lane).  Estimates how many records
// repeat the leaf of another record: every record writes its number at its leaf's hash, reads the
// number that stayed there and compares leaves (a record that reads its own number repeats nothing it
// can see; two leaves with one hash hide each other's repeats, which only makes the estimate low).
// If they are too few, returns false.  Otherwise fills gs.order / gs.leaf with the records grouped by
// leaf (groups in the order of their first record, records of a group in list order) and returns true.
__device__ __forceinline__ bool group_by_leaf(GroupScratch& gs, MergeState& state, const int32_t* leaves, int n,
                                              int lane) {
    if (state.skip > 0) {
        state.skip -= 1;
        return false;
    }
    const bool mine = lane < n;
    const int32_t leaf = mine ? leaves[lane] : -1;
    const unsigned h = ((uint32_t)leaf * 2654435761u) >> 24;
    if (mine) gs.table[h] = (uint8_t)lane;
    wave_lds_sync();
    bool repeat = false;
    if (mine) {
        const int j = gs.table[h];
        repeat = j != lane && leaves[j] == leaf;
    }
    if (__popcll(__ballot(repeat)) * kMergeMinShare < n) {
        state.skip = kMergeRecheck;
        return false;
    }
    unsigned long long todo = __ballot(mine);
    int base = 0, pos = 0;
    while (todo) {
        const int lead = __builtin_ctzll(todo);
        const int32_t l = __builtin_amdgcn_readlane(leaf, lead);
        const unsigned long long same = __ballot(mine && leaf == l);
        if ((same >> lane) & 1ull) pos = base + rank_in(same);
        base += __popcll(same);
        todo &= ~same;
    }
    if (mine) {
        gs.order[pos] = (uint8_t)lane;
        gs.leaf[pos] = leaf;
    }
    wave_lds_sync();
    return true;
}

template <int K, int NV, class Term, class Emit>
__device__ __forceinline__ void add_records_by_leaf(int n, int lane, const int32_t* leaves, Term&& term,
                                                    Emit&& emit) {
    constexpr int kPer = K <= kMarchThreads ? kMarchThreads / K : 1;
    const int r = K <= kMarchThreads ? lane / K : 0;
    if (r >= kPer) return;
    const int per = (n + kPer - 1) / kPer;
    const int lo = r * per;
    const int hi = lo + per < n ? lo + per : n;
    for (int e = K <= kMarchThreads ? lane - r * K : lane; e < K; e += kMarchThreads) {
        int32_t cur = -1;
        float acc[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
        for (int rec = lo; rec < hi; ++rec) {
            const int32_t leaf = leaves[rec];
            if (leaf != cur) {
                if (cur >= 0) emit(cur, e, acc);
                cur = leaf;
#pragma unroll
                for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
            }
            float t[NV];
            term(rec, e, t);
#pragma unroll
            for (int v = 0; v < NV; ++v) acc[v] += t[v];
        }
        if (cur >= 0) emit(cur, e, acc);
    }
}

// One record per lane of a wavefront: a step in which all 64 lanes emit fills the list once.  Leaves,
// density terms and colour factors (20 bytes a record) fill ShadeShared::leaf and ::who exactly; the
// owners follow the GroupScratch in ShadeShared::colour.
constexpr int kEmitCap = kMarchThreads;
template <class P, int D, bool kByRecord = false>
struct RecordList {
    static constexpr int K = P::kRecord;
    ShadeShared<D, true>& sh;
    float* grad_data;
    int lane;
    MergeState& merge;
    int n = 0;   // wavefront-uniform

    __device__ __forceinline__ int32_t* leaves() const { return sh.leaf; }
    // per record four factors: the three colour factors tmp2[c], then the density term
    __device__ __forceinline__ float* factors() const { return (float*)(sh.leaf + kEmitCap); }
    __device__ __forceinline__ uint8_t* owners() const { return (uint8_t*)sh.colour + sizeof(GroupScratch); }

    // element e of record rec: basis[i] * tmp2[c] for a colour coefficient, g_sigma for the density
    __device__ __forceinline__ float element(int rec, int e) const {
        const int c = P::kFormat == SVOX_FORMAT_RGBA ? e : e / D;
        if (c < 3) {
            const float v = factors()[rec * 4 + c];
            return P::kFormat == SVOX_FORMAT_RGBA ? v : sh.basis[owners()[rec] * D + (e - c * D)] * v;
        }
        return factors()[rec * 4 + 3];
    }

    // The colours of the round are in registers by the time records are added: their LDS is free.
    __device__ __forceinline__ GroupScratch& scratch() const { return *(GroupScratch*)sh.colour; }

    // add_records_by_leaf for records longer than half a wavefront (one record at a time, lane e on
    // element e).  What the lanes need to find a record's values -- its place in the list, its leaf,
    // its owner -- is first taken into registers, record r by lane r, and then handed round by
    // readlane: per record that leaves two LDS reads (the factor of the lane's channel, the owner's
    // basis value) whose addresses come from scalars, so the reads of kHeldBlock records are in flight
    // together.  (Through LDS alone a record costs three reads that wait for one another: place, owner,
    // basis.)  order: the records' adding order (grouped by leaf), or nullptr for the list's own.
    static constexpr bool kHeld = K > kMarchThreads / 2;
    static constexpr int kHeldBlock = 4;
    __device__ __forceinline__ void add_held(const uint8_t* order) {
        const bool mine = lane < n;
        const int rec = mine ? (order ? order[lane] : lane) : 0;
        const int my_rec = rec;
        const int my_leaf = leaves()[rec];
        const int my_owner = owners()[rec];
        // readlane looks into other lanes, so every lane must hold its record and must stay in step with the
        // others: the loop below is one every lane runs (its trip count depends on K alone), and a lane whose
        // element lies beyond the record only leaves out the additions.
        for (int e0 = 0; e0 < K; e0 += kMarchThreads) {
            const int e = e0 + lane;
            const bool on = e < K;
            const int c_raw = P::kFormat == SVOX_FORMAT_RGBA ? e : e / D;
            const int c = c_raw < 3 ? c_raw : 3;                              // (3: the density element, and lanes that are not `on`)
            const int i = P::kFormat == SVOX_FORMAT_RGBA || c == 3 ? 0 : e - c * D;
            const bool with_basis = P::kFormat != SVOX_FORMAT_RGBA && c < 3;
            int32_t cur = -1;
            float acc = 0.0f;
            for (int at = 0; at < n; at += kHeldBlock) {
                int32_t leaf[kHeldBlock];
                float val[kHeldBlock], leaf_basis[kHeldBlock];
#pragma unroll
                for (int u = 0; u < kHeldBlock; ++u) {
                    const int a = at + u < n ? at + u : n - 1;   // (past the end: the last record again, unused)
                    leaf[u] = __builtin_amdgcn_readlane(my_leaf, a);
                    const int owner = __builtin_amdgcn_readlane(my_owner, a);
                    const float t = factors()[__builtin_amdgcn_readlane(my_rec, a) * 4 + c];
                    // (every lane reads, also the lane of the density element, whose i is 0: a read under a
                    // condition would be waited for on the spot)
                    float basis_value = 1.0f;
                    if constexpr (P::kFormat != SVOX_FORMAT_RGBA) basis_value = sh.basis[owner * D + i];
                    leaf_basis[u] = basis_value;
                    val[u] = t;
                }
#pragma unroll
                for (int u = 0; u < kHeldBlock; ++u) val[u] = with_basis ? leaf_basis[u] * val[u] : val[u];
#pragma unroll
                for (int u = 0; u < kHeldBlock; ++u) {
                    if (at + u < n) {
                        if (leaf[u] != cur) {
                            if (on && cur >= 0) atomicAdd(grad_data + (int64_t)cur * K + e, acc);
                            cur = leaf[u];
                            acc = 0.0f;
                        }
                        acc += val[u];
                    }
                }
            }
            if (on && cur >= 0) atomicAdd(grad_data + (int64_t)cur * K + e, acc);
        }
    }

    // Adds the list with the records of every leaf summed first, if enough records share a leaf.
    __device__ __forceinline__ bool flush_grouped() {
        GroupScratch& gs = scratch();
        if (!group_by_leaf(gs, merge, leaves(), n, lane)) return false;
        if constexpr (kHeld) {
            add_held(gs.order);
        } else {
            add_records_by_leaf<K, 1>(
                n, lane, gs.leaf, [&](int at, int e, float* t) { t[0] = element(gs.order[at], e); },
                [&](int32_t leaf, int e, const float* sum) { atomicAdd(grad_data + (int64_t)leaf * K + e, sum[0]); });
        }
        wave_lds_sync();
        n = 0;
        return true;
    }

    __device__ __forceinline__ void flush() {
        if constexpr (kByRecord) {
            flush_by_record();
            return;
        }
        if (n == 0) return;
        wave_lds_sync();
        if (flush_grouped()) return;
        if constexpr (kHeld) {
            // long records: one at a time with its values handed round by readlane (measured on the
            // marching backward of an 800x800 image: 2.55 -> 2.38 ms, with a workspace 2.07 -> 1.80 ms;
            // for records of up to 32 scalars the flat form below is as fast)
            add_held(nullptr);
            wave_lds_sync();
            n = 0;
            return;
        }
        const int total = n * K;
        for (int f = lane; f < total; f += kMarchThreads) {
            const int rec = f / K, e = f - rec * K;
            float val;
            if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
                val = factors()[rec * 4 + e];
            } else {
                if (e < 3 * D) {
                    const int c = e / D;
                    val = sh.basis[owners()[rec] * D + (e - c * D)] * factors()[rec * 4 + c];
                } else {
                    val = factors()[rec * 4 + 3];
                }
            }
            atomicAdd(grad_data + (int64_t)leaves()[rec] * K + e, val);
        }
        wave_lds_sync();
        n = 0;
    }

    // The same additions by add_records_by_leaf.  (Measured: 12 % off replay_backward_kernel, whose
    // time is mostly these additions; nothing for render_backward_kernel.)
    __device__ __forceinline__ void flush_by_record() {
        if (n == 0) return;
        wave_lds_sync();
        if (flush_grouped()) return;
        if constexpr (kHeld) {
            add_held(nullptr);
        } else {
            add_records_by_leaf<K, 1>(
                n, lane, leaves(), [&](int rec, int e, float* t) { t[0] = element(rec, e); },
                [&](int32_t leaf, int e, const float* sum) { atomicAdd(grad_data + (int64_t)leaf * K + e, sum[0]); });
        }
        wave_lds_sync();
        n = 0;
    }

    // the record of every lane with `emit` set joins the list (in lane order)
    __device__ __forceinline__ void append(bool emit, int32_t leaf, const float* tmp2, float g_sigma) {
        unsigned long long todo = __ballot(emit);
        while (todo) {
            if (n == kEmitCap) flush();
            const bool pending = (todo >> lane) & 1ull;
            const int slot = n + rank_in(todo);
            const bool take = pending && slot < kEmitCap;
            if (take) {
                leaves()[slot] = leaf;
                owners()[slot] = (uint8_t)lane;
                factors()[slot * 4] = tmp2[0];
                factors()[slot * 4 + 1] = tmp2[1];
                factors()[slot * 4 + 2] = tmp2[2];
                factors()[slot * 4 + 3] = g_sigma;
            }
            const unsigned long long taken = __ballot(take);
            n += __popcll(taken);
            todo &= ~taken;
        }
    }
};
static_assert(5 * kEmitCap * 4 <= kQueue * kMarchThreads * 5, "record list exceeds the shade list");
static_assert(kEmitCap <= kMarchThreads, "group_by_leaf holds one record per lane");
static_assert(sizeof(GroupScratch) + kEmitCap <= sizeof(float) * kQueue * kMarchThreads * 3,
              "GroupScratch and the owners live in ShadeShared::colour");
using ShadeSharedProbe = ShadeShared<1, true>;
static_assert(offsetof(ShadeSharedProbe, who) == sizeof(int32_t) * kQueue * kMarchThreads,
              "the record list runs from ShadeShared::leaf into ShadeShared::who");


// ------------------------------------------------------------------------------------------------
// forward, walk and shading on two wavefronts
// ------------------------------------------------------------------------------------------------
// The round of render_forward_kernel is one chain per wavefront: four turns of the walk (child reads
// that hit in L2), then the densities and the records of the leaves found (reads that go to HBM), then
// the colours, then the next walk.  The walk does not depend on what the leaves hold, but a
// wavefront's loads come back in the order they were issued, so within one wavefront the next walk
// cannot run while the records are on their way.  Here a block is two wavefronts that share the 64
// rays of a tile: the first only walks and hands every leaf it finds (that is not marked empty) to
// the second through a ring in LDS, a few leaves per lane deep; the second takes the leaves as they
// come, fetches densities and records, evaluates colours and composites exactly as
// render_forward_kernel does, and tells the walk which rays have stopped.  Same arithmetic, same
// pictures.  Each wavefront sets the rays up for itself (the same instructions give the same rays).
// A wavefront that finds nothing to do sleeps a few cycles and looks again; after kSpinLimit looks in a
// row it gives up, so that a launch ends whatever happens.
//
// kNoted: as in render_forward_kernel, the launch also leaves the notes of every ray for the backward
// pass: every leaf with sigma > 0 of the whole ray, so the walk goes on after the picture's early stop,
// and the colours of leaves below sigma_thresh are evaluated too; the picture itself is composed as
// without notes.
constexpr int kSplitThreads = 2 * kMarchThreads;
constexpr int kRing = 8;               // leaves a lane's walk may be ahead of its shading (a power of two)
constexpr int kSpinLimit = 1 << 22;
constexpr int32_t kEndedBit = 1 << 30;   // in SplitBox::written: the ray's walk is over; in ::taken: the ray wants no more leaves
constexpr int32_t kBrokenBit = 1 << 29;  // in SplitBox::written, beside kEndedBit: the walk ended in a malformed tree

struct SplitBox {
    int32_t leaf[kRing * kMarchThreads];   // [place in the ring][lane]
    float dt[kRing * kMarchThreads];
    int32_t written[kMarchThreads];        // set by the walk: leaves put into the lane's ring so far (| kEndedBit)
    int32_t taken[kMarchThreads];          // set by the shading: leaves taken out so far (| kEndedBit)
};

// The two counters are read and written as atomics of the workgroup (unlike a volatile access, which the compiler
// leaves on the generic address path -- a flat instruction with a wait for every store --, it still knows that they
// live in LDS and issues plain LDS reads and writes).  A count is published with release order after the ring
// entries it covers were written (or read), and read with acquire order before they are read (or overwritten):
// the hand-over does not lean on the order in which one wavefront's LDS operations happen to be carried out.
#ifdef SVOX_BOX_RELAXED
constexpr int kBoxLoadOrder = __ATOMIC_RELAXED, kBoxStoreOrder = __ATOMIC_RELAXED;
#else
constexpr int kBoxLoadOrder = __ATOMIC_ACQUIRE, kBoxStoreOrder = __ATOMIC_RELEASE;
#endif
__device__ __forceinline__ int32_t box_read(const int32_t* at) {
    return __hip_atomic_load(at, kBoxLoadOrder, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void box_write(int32_t* at, int32_t value) {
    __hip_atomic_store(at, value, kBoxStoreOrder, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Wavefronts of render_forward_split_kernel that gave up waiting since the library was loaded (svox_give_up_count).
__device__ unsigned int split_give_ups = 0;

// (The density phase stays also where the marks of a launch say that every leaf they let through is shaded,
// render_forward_kernel's kAllShaded: here the walk is the critical path, and the density read of a leaf brings the
// last line of its record into L2 ahead of the coefficient reads.)
template <class P, class Source, bool kNoted = false, bool kGrad = false>
__global__ __launch_bounds__(kSplitThreads) void render_forward_split_kernel(TreeDev<float> tr, Source src,
                                                                             SvoxRenderOptions opt,
                                                                             float* __restrict__ out, ReplaySpace ws,
                                                                             const float* __restrict__ grad_out = nullptr) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    __shared__ int32_t path[(kPathLevels + 1) * kMarchThreads];
    __shared__ ShadeShared<D, P::kForwardRows> sh;
    __shared__ SplitBox box;
    if constexpr (kNoted) {
        if (blockIdx.x == 0 && threadIdx.x < kStampWords) ws.stamp_at[threadIdx.x] = ws.stamp[threadIdx.x];
    }
    const int lane = threadIdx.x & (kMarchThreads - 1);
    const bool walks = threadIdx.x < kMarchThreads;   // uniform in a wavefront
    float offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    const float step = opt.step_size, sigma_thresh = opt.sigma_thresh, stop_thresh = opt.stop_thresh;
    const int spin_limit = ws.spin_limit > 0 ? ws.spin_limit : kSpinLimit;

    const int64_t item = chunk_of_block(blockIdx.x, gridDim.x, src.xcd_group) * (int64_t)kMarchThreads + lane;
    RayState<float> r;
    int64_t slot = -1;
    bool active = false;
    {
        float origin[3], dir[3], vdir[3];
        if (item < src.total()) slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
        if (slot >= 0) active = setup_ray(r, origin, dir, scaling);
        if (!walks) {
            if (slot >= 0 && !active) {
                if (!kNoted || out) {
                    out[slot * 3] = bg;
                    out[slot * 3 + 1] = bg;
                    out[slot * 3 + 2] = bg;
                }
                if constexpr (kNoted) NoteTaker::missed(ws, slot);
            }
            if constexpr (P::kFormat == SVOX_FORMAT_SH) {
                if (active) {
                    sh.vdir[lane * 3] = vdir[0];
                    sh.vdir[lane * 3 + 1] = vdir[1];
                    sh.vdir[lane * 3 + 2] = vdir[2];
                }
            } else if constexpr (P::kForwardRows) {
                if (active) {
                    float basis[D];
                    policy_basis<P>(Lobes{tr.extra, tr.extra_cols, opt.format}, opt, vdir, basis);
#pragma unroll
                    for (int i = 0; i < D; ++i) sh.basis[lane * D + i] = basis[i];
                }
            }
        }
    }
    if (!__any(active)) return;   // (both wavefronts see the same rays: both leave or both stay)
    if (walks)
        box.written[lane] = 0;
    else
        box.taken[lane] = active ? 0 : kEndedBit;
    __syncthreads();

    if (walks) {
        // ---- the walk: one leaf per live lane and turn, into the ring
        OctreeCursor cur;
        cur.reset(path + lane, kMarchThreads);
        int32_t written = 0;
        bool live = active, broken = false;
        int spins = 0;
        // the walk is the longest chain of a tile: it goes first where wavefronts share a SIMD
        // (measured: -10 % on a dense image, nothing elsewhere)
        __builtin_amdgcn_s_setprio(3);
        while (true) {
            // (reading the shading's count only every few turns was measured slower: rays that have
            // stopped are then walked further)
            const int32_t taken = box_read(&box.taken[lane]);
            live = live && !(taken & kEndedBit);
            if (live && (broken || !(r.t < r.tmax))) {   // the walk of this ray is over: say so once
                box_write(&box.written[lane], written | kEndedBit | (broken ? kBrokenBit : 0));
                live = false;
            }
            if (!__any(live)) break;
            const bool go = live && written - (taken & ~kEndedBit) < kRing;
            if (!__any(go)) {   // every ring is full: the shading is behind
                if (++spins > spin_limit) {
                    if (lane == 0) atomicAdd(&split_give_ups, 1u);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
                continue;
            }
            spins = 0;
            int32_t leaf;
            float dt;
            walk_turn_flat(tr, r, cur, step, go, broken, leaf, dt);
            const bool put = go && leaf >= 0 && !(leaf & kEmptyLeafBit);
            if (put) {
                const int at = (written & (kRing - 1)) * kMarchThreads + lane;
                box.leaf[at] = leaf;
                box.dt[at] = dt;
                written += 1;
            }
            // (release: the leaf is in the ring before the count says so)
            if (put) box_write(&box.written[lane], written);
        }
        return;
    }

    // ---- the shading: takes up to kQueue leaves per lane at a time, as render_forward_kernel's round
    float acc[3] = {0.f, 0.f, 0.f};
    float light = 1.0f;
    int32_t taken = 0;
    int spins = 0;
    // kNoted: the picture of a ray may be finished (early stop) while its notes go on; without `out`
    // there is no picture to compose
    bool painted = kNoted && out == nullptr;
    NoteTaker notes;
    March1Sum sum1;
    int64_t shared_next = 0, shared_end = 0;   // the wavefront's stock of chunks for notes (uniform)
    if constexpr (kNoted) notes.begin(ws, active ? slot : 0);
    if constexpr (kNoted && kGrad) sum1.begin(grad_out, active ? slot : 0);
    while (true) {
        const int32_t w = box_read(&box.written[lane]);   // (acquire: the ring is read after the count, not before)
        const int32_t avail = (w & ~(kEndedBit | kBrokenBit)) - taken;
        if (active && (w & kEndedBit) && avail == 0) {
            // the ray left the tree: the background shows through what is left of the light
            if (!painted) {
                out[slot * 3] = fma_(light, bg, acc[0]);
                out[slot * 3 + 1] = fma_(light, bg, acc[1]);
                out[slot * 3 + 2] = fma_(light, bg, acc[2]);
            }
            if constexpr (kNoted) notes.finish((w & kBrokenBit) != 0, r.dscale, kGrad ? sum1.end(bg) : 0.0f);
            active = false;
        }
        if (!__any(active)) break;
        const int n_take = active ? (avail < kQueue ? avail : kQueue) : 0;
        // (waiting for fuller hands -- two or four leaves per lane, a few looks of patience -- and a ring
        // of 16 were measured: no gain, the larger ring costs LDS)
        if (!__any(n_take > 0)) {   // the walk has found nothing new yet
            if (++spins > spin_limit) {
                // Cannot happen while the walk runs.  If it ever does, nothing plausible is left behind: the pixel
                // is NaN, the ray's notes say "march me" (the backward pass then does, twice), and the library's
                // give-up counter tells the host (svox_give_up_count).
                if (active && out && !painted)
                    out[slot * 3] = out[slot * 3 + 1] = out[slot * 3 + 2] = __int_as_float(0x7fc00000);
                if constexpr (kNoted) {
                    if (active) notes.give_up(r.dscale);
                }
                if (lane == 0) atomicAdd(&split_give_ups, 1u);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
            continue;
        }
        spins = 0;
        int32_t q_leaf[kQueue];
        float q_dt[kQueue];
#pragma unroll
        for (int q = 0; q < kQueue; ++q) {
            const int at = ((taken + q) & (kRing - 1)) * kMarchThreads + lane;
            q_leaf[q] = q < n_take ? box.leaf[at] : -1;
            q_dt[q] = q < n_take ? box.dt[at] : 0.0f;
        }
        wave_lds_sync();   // the leaves are out of the ring before the count gives their places back
        taken += n_take;
        if (n_take > 0) box_write(&box.taken[lane], taken);
        float q_sigma[kQueue], q_raw[kQueue];
        fetch_sigma<K>(tr.data, q_leaf, q_sigma);
        soften_sigma(opt.density_softplus, q_leaf, q_sigma, q_raw);
        const int n_entries = build_shade_list(sh, q_leaf, q_sigma, kNoted ? 0.0f : sigma_thresh, lane);
        bool stopped = false;
        if (n_entries > 0) {
            wave_lds_sync();
            shade_entries<P, P::kForwardRows>(tr.data, sh, n_entries, lane);
            wave_lds_sync();
            float q_att[kQueue], q_rgb[kQueue][3], q_s[kQueue][3];
#pragma unroll
            for (int q = 0; q < kQueue; ++q) {
                q_att[q] = expf_fixed(-q_dt[q] * r.dscale * q_sigma[q]);
                const float* s = sh.colour + (q * kMarchThreads + lane) * 3;
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    q_s[q][c] = s[c];
                    q_rgb[q][c] = fma_(s[c], d_rgb_pad, -pad);
                }
            }
#pragma unroll
            for (int q = 0; q < kQueue; ++q) {
                const bool take = active && !painted && q_leaf[q] >= 0 && !stopped && q_sigma[q] > sigma_thresh;
                const float weight = light * (1.0f - q_att[q]);
#pragma unroll
                for (int c = 0; c < 3; ++c) acc[c] = take ? fma_(weight, q_rgb[q][c], acc[c]) : acc[c];
                light = take ? light * q_att[q] : light;
                stopped = stopped || (take && light <= stop_thresh);
                if constexpr (kNoted) {
                    const bool note = active && q_leaf[q] >= 0 && q_sigma[q] > 0.0f;
                    notes.take(ws, shared_next, shared_end, lane, note, q_leaf[q], q_dt[q], q_raw[q], q_s[q]);
                    if constexpr (kGrad) {
                        if (note) sum1.leaf(q_dt[q], q_sigma[q], r.dscale, q_s[q], d_rgb_pad, pad);
                    }
                }
            }
            wave_lds_sync();   // the colours are read before the next list overwrites them
        }
        if (active && stopped) {
            // rt_kernel.cu:306-313: rescale and leave without the background; the walk may stop
            const float scale = (float)(1.0 / (1.0 - (double)light));
            out[slot * 3] = acc[0] * scale;
            out[slot * 3 + 1] = acc[1] * scale;
            out[slot * 3 + 2] = acc[2] * scale;
            if constexpr (kNoted) {
                painted = true;   // the picture is done; the notes go on to the end of the ray
            } else {
                active = false;
                box_write(&box.taken[lane], taken | kEndedBit);
            }
        }
    }
}

// kMode: kBackwardPlain runs both marches; kBackwardSecond runs only the second, for rays whose first
// march a noting forward kernel has already made (with grad_out at hand: NoteTaker keeps the sum of
// march 1 in the head of the ray's notes) but whose notes did not fit the workspace.
template <class P, class Source, bool kRefill, int kMode>
__global__ __launch_bounds__(kMarchThreads) void render_backward_kernel(TreeDev<float> tr, Source src,
                                                                        SvoxRenderOptions opt,
                                                                        const float* __restrict__ grad_out,
                                                                        float* __restrict__ grad_data,
                                                                        ReplaySpace ws) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    __shared__ int32_t path[(kPathLevels + 1) * kMarchThreads];
    __shared__ ShadeShared<D, true> sh;
    const int lane = threadIdx.x;
    float offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    const float step = opt.step_size;

    int64_t next = chunk_of_block(blockIdx.x, gridDim.x, src.xcd_group) * (int64_t)src.per_wave;
    const int64_t total = src.total();
    const int64_t end = next + src.per_wave < total ? next + src.per_wave : total;

    enum { kMarch1 = 0, kMarch2 = 1 };
    RayState<float> r;
    float go[3] = {0.f, 0.f, 0.f};
    float light = 1.0f, accum = 0.0f, tmin = 0.0f;
    bool active = false;
    int phase = kMarch1;
    MergeState merge;
    OctreeCursor cur;
    cur.reset(path + lane, kMarchThreads);

    // takes ray `item` into this lane if it hits the tree
    auto start = [&](int64_t item) {
        float origin[3], dir[3], vdir[3];
        // (with a bitmap a batch launch does not deal its rays out: its items are ray numbers)
        if (Source::kItemsAreSlots && ws.only && !((ws.only[item >> 6] >> (item & 63)) & 1ull)) return;
        const int64_t slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
        if (!Source::kItemsAreSlots && ws.only && slot >= 0 && !((ws.only[slot >> 6] >> (slot & 63)) & 1ull)) return;
        if (slot >= 0 && setup_ray(r, origin, dir, scaling)) {
            float march1_sum = 0.0f;
            bool first_march_too = false;
            if constexpr (kMode == kBackwardSecond) {
                const float2* head = ws.base + slot * kChunkFloat2 + kHeadFloat2;
                // (a walk that broke off in a malformed tree: the reference adds nothing for such a ray)
                if (head[1].y == 2.0f) return;
                // (a ray the noting launch gave up on has no sum: both marches)
                first_march_too = head[1].y == 3.0f;
                march1_sum = first_march_too ? 0.0f : head[2].x;
            }
            if constexpr (P::kFormat != SVOX_FORMAT_RGBA) {
                float basis[D];
                policy_basis<P>(Lobes{tr.extra, tr.extra_cols, opt.format}, opt, vdir, basis);
#pragma unroll
                for (int i = 0; i < D; ++i) sh.basis[lane * D + i] = basis[i];
            }
            go[0] = grad_out[slot * 3];
            go[1] = grad_out[slot * 3 + 1];
            go[2] = grad_out[slot * 3 + 2];
            light = 1.0f;
            accum = march1_sum;
            tmin = r.t;
            cur.restart();
            phase = kMode == kBackwardSecond && !first_march_too ? kMarch2 : kMarch1;
            active = true;
        }
    };
    if constexpr (!kRefill) {
        if (next + lane < end) start(next + lane);
    }

    while (true) {
        if constexpr (kRefill) {
            if (Source::kItemsAreSlots && ws.only) next = skip_clear_words(ws.only, next, end, lane);
            const RoundState state = refill_lanes(active, next, end, src.refill_at, start);
            if (state == kRoundRefilled) continue;
            if (state == kRoundDone) break;
        } else {
            if (!__any(active)) break;
        }

        // ---- walk
        int32_t q_leaf[kQueue];
        float q_dt[kQueue];
        bool broken;
        float q_sigma[kQueue];
        walk_turns(tr, r, cur, step, active, broken, q_leaf, q_dt);
        // ---- sigma
        float q_raw[kQueue];
        fetch_sigma<K>(tr.data, q_leaf, q_sigma);
        soften_sigma(opt.density_softplus, q_leaf, q_sigma, q_raw);
        // ---- shade list: every leaf with density
        const int n_entries = build_shade_list(sh, q_leaf, q_sigma, 0.0f, lane);
        wave_lds_sync();
        if (n_entries > 0) shade_entries<P, true>(tr.data, sh, n_entries, lane);
        wave_lds_sync();
        // ---- composite slot by slot; the gradient records of the round are added together
        RecordList<P, D> records{sh, grad_data, lane, merge};
        // what does not depend on the transmittance is evaluated for the four slots side by side
        float q_att[kQueue], q_total[kQueue], q_s[kQueue][3];
#pragma unroll
        for (int q = 0; q < kQueue; ++q) {
            q_att[q] = expf_fixed(-q_dt[q] * q_sigma[q] * r.dscale);
            const float* s = sh.colour + (q * kMarchThreads + lane) * 3;
            float total_color = 0.0f;
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                q_s[q][c] = s[c];
                total_color = fma_(fma_(s[c], d_rgb_pad, -pad), go[c], total_color);
            }
            q_total[q] = total_color;
        }
#pragma unroll
        for (int q = 0; q < kQueue; ++q) {
            bool emit = false;
            float tmp2[3] = {0.f, 0.f, 0.f};
            float g_sigma = 0.f;
            if (active && q_leaf[q] >= 0 && q_sigma[q] > 0.0f) {
                const float att = q_att[q];
                const float weight = light * (1.0f - att);
                const float* s = q_s[q];
                const float total_color = q_total[q];
                light *= att;
                if (phase == kMarch1) {
                    accum = fma_(weight, total_color, accum);
                } else {
#pragma unroll
                    for (int c = 0; c < 3; ++c) {
                        if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
                            tmp2[c] = weight * s[c] * (1.0f - s[c]) * go[c] * d_rgb_pad;
                        } else {
                            tmp2[c] = (float)((double)(weight * s[c]) * (1.0 - (double)s[c]) * (double)go[c] *
                                              (double)d_rgb_pad);
                        }
                    }
                    accum = fma_(-weight, total_color, accum);
                    g_sigma = q_dt[q] * r.dscale * fma_(total_color, light, -accum);
                    if (opt.density_softplus) g_sigma *= sigmoid_(q_raw[q] - 1.0f);   // rt_kernel.cu:471-474
                    emit = true;
                }
            }
            records.append(emit, q_leaf[q], tmp2, g_sigma);
        }
        records.flush();
        // ---- end of a march
        if (active && (broken || !(r.t < r.tmax))) {
            if (phase == kMarch1 && !broken) {
                const float total_grad = (go[0] + go[1]) + go[2];
                accum = fma_(light * bg, total_grad, accum);
                light = 1.0f;
                phase = kMarch2;
                r.t = tmin;
            } else {
                active = false;
            }
        }
    }
}

// The backward pass from the notes a noting forward kernel left (NoteTaker): one lane per ray, no
// tree walk.  The notes of a ray (leaf, step length, sigma, the three sigmoids of every leaf with
// sigma > 0) are read twice, five at a time: first for the sum the reference's first march forms
// (rt_kernel.cu:358-419), then for the gradient records of its second march (:421-475), which the
// wavefront adds together as render_backward_kernel does.  A ray whose notes are incomplete, or every
// ray if the workspace carries another stamp, is left to a launch of render_backward_kernel with the
// bitmap this kernel writes (one word per wavefront).
constexpr int kReplayGroup = 5;
static_assert(kChunkRecords % kReplayGroup == 0, "a group of notes never straddles two chunks");

template <class P, class Source>
__global__ __launch_bounds__(kMarchThreads) __attribute__((amdgpu_waves_per_eu(3))) void replay_backward_kernel(Source src, SvoxRenderOptions opt,
                                                                        const float* __restrict__ grad_out,
                                                                        float* __restrict__ grad_data,
                                                                        ReplaySpace ws, int ray_shift,
                                                                        int march1_known, Lobes lobes) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    __shared__ ShadeShared<D, true> sh;
    const int lane = threadIdx.x;
    // A wavefront takes 2^ray_shift consecutive rays (64 or 16), one per lane from lane 0.  Adding a
    // step's records is work of the whole wavefront, one record after the other; where the rays of a
    // wavefront are neighbours (the pixels of an image) they are all long or all short together, and
    // fewer of them per wavefront spread a long run of pixels over several wavefronts.
    const int64_t ray = ((int64_t)blockIdx.x << ray_shift) + lane;
    const bool seated = lane < (1 << ray_shift);
    const bool stamped = stamp_matches(ws);
    const float2* first = ws.base + ray * kChunkFloat2;
    int count = 0;
    int32_t first_link = 0;
    float dscale = 0.0f;
    if (seated && ray < src.n_slots()) {
        const float2 head = first[kHeadFloat2], tail = first[kHeadFloat2 + 1];
        first_link = __float_as_int(head.x);
        count = stamped ? __float_as_int(head.y) : -1;
        dscale = tail.x;
    }
    // (the wavefront's part of the bitmap: a word or a quarter of one)
    const unsigned long long undone = __ballot(count < 0);
    if (lane == 0) {
        if (ray_shift == 6)
            ws.undone[blockIdx.x] = undone;
        else
            ((uint16_t*)ws.undone)[blockIdx.x] = (uint16_t)undone;
    }
    const bool work = count > 0;
    if (!__any(work)) return;

    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    float go[3] = {0.f, 0.f, 0.f};
    if (work) {
        if constexpr (P::kFormat != SVOX_FORMAT_RGBA) {
            float vdir[3];
            src.view_dir(ray, vdir);
            float basis[D];
            policy_basis<P>(lobes, opt, vdir, basis);
#pragma unroll
            for (int i = 0; i < D; ++i) sh.basis[lane * D + i] = basis[i];
        }
        go[0] = grad_out[ray * 3];
        go[1] = grad_out[ray * 3 + 1];
        go[2] = grad_out[ray * 3 + 2];
    }
    wave_lds_sync();   // the basis rows are read by other lanes when the records are added

    float light = 1.0f, accum = 0.0f;
    // march1_known: the pass that took the notes had grad_out and left the sum of the first march in
    // the head of the ray's notes (March1Sum: the same expressions in the same order as pass 0 below)
    if (march1_known && work) accum = first[kHeadFloat2 + 2].x;
    MergeState merge{2};   // (a wavefront of 64 unrelated rays flushes about twice: it never looks)
    RecordList<P, D, true> records{sh, grad_data, lane, merge};
    struct Group {
        float2 note[kReplayGroup][3];
    };
#pragma unroll 1
    for (int pass = march1_known ? 1 : 0; pass < 2; ++pass) {
        const float2* chunk = first;
        int32_t link = first_link;
        int pos = 0;
        // asks for the group of notes that starts at note `base` (the loads are waited for where the
        // group is worked on: meanwhile the group before it is)
        auto fetch = [&](Group& g, int base) {
            if (work && base < count) {
                if (pos == kChunkRecords) {
                    chunk = ws.base + (int64_t)link * kChunkFloat2;
                    link = __float_as_int(chunk[kHeadFloat2].x);
                    pos = 0;
                }
#pragma unroll
                for (int k = 0; k < kReplayGroup; ++k) {
#pragma unroll
                    for (int j = 0; j < 3; ++j) g.note[k][j] = chunk[(pos + k) * 3 + j];
                }
                pos += kReplayGroup;
            }
        };
        auto work_on = [&](const Group& g, int base) {
#pragma unroll
            for (int k = 0; k < kReplayGroup; ++k) {
                const bool have = work && base + k < count;
                const int32_t leaf = __float_as_int(g.note[k][0].x);
                const float dt = g.note[k][0].y, raw = g.note[k][1].x;   // (the stored density)
                const float s[3] = {g.note[k][1].y, g.note[k][2].x, g.note[k][2].y};
                float tmp2[3] = {0.f, 0.f, 0.f};
                float g_sigma = 0.0f;
                if (have) {
                    const float sigma = opt.density_softplus ? softplus_m1(raw) : raw;
                    const float att = expf_fixed(-dt * sigma * dscale);
                    const float weight = light * (1.0f - att);
                    float total_color = 0.0f;
#pragma unroll
                    for (int c = 0; c < 3; ++c) total_color = fma_(fma_(s[c], d_rgb_pad, -pad), go[c], total_color);
                    light *= att;
                    if (pass == 0) {
                        accum = fma_(weight, total_color, accum);
                    } else {
#pragma unroll
                        for (int c = 0; c < 3; ++c) {
                            if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
                                tmp2[c] = weight * s[c] * (1.0f - s[c]) * go[c] * d_rgb_pad;
                            } else {
                                tmp2[c] = (float)((double)(weight * s[c]) * (1.0 - (double)s[c]) * (double)go[c] *
                                                  (double)d_rgb_pad);
                            }
                        }
                        accum = fma_(-weight, total_color, accum);
                        g_sigma = dt * dscale * fma_(total_color, light, -accum);
                        if (opt.density_softplus) g_sigma *= sigmoid_(raw - 1.0f);
                    }
                }
                if (pass == 1) records.append(have, leaf, tmp2, g_sigma);
            }
        };
        Group a, b;
        fetch(a, 0);
        for (int base = 0; __any(work && base < count); base += 2 * kReplayGroup) {
            fetch(b, base + kReplayGroup);
            work_on(a, base);
            fetch(a, base + 2 * kReplayGroup);
            work_on(b, base + kReplayGroup);
        }
        if (pass == 0) {
            const float total_grad = (go[0] + go[1]) + go[2];
            accum = fma_(light * bg, total_grad, accum);
            light = 1.0f;
        }
    }
    records.flush();
}

// ------------------------------------------------------------------------------------------------
// squared-error gradient and Gauss-Newton Hessian diagonal
// ------------------------------------------------------------------------------------------------
// sigmoid(basis . coefficients) of channel c, rt_kernel.cu:541-547
template <typename T>
__device__ __forceinline__ T channel_sigmoid(const SvoxRenderOptions& opt, const T* basis, const T* val, int c) {
    if (opt.format == SVOX_FORMAT_RGBA) return sigmoid_(val[c]);
    const int off = c * opt.basis_dim;
    T tmp = T(0);
    for (int i = opt.min_comp; i <= opt.max_comp; ++i) tmp = fma_(basis[i], val[off + i], tmp);
    return sigmoid_(tmp);
}

// trace_ray_se_grad_hess, rt_kernel.cu:479-715, generic flavour: one ray per lane, three marches (residual; colour
// gradients and the rendered colour as a running suffix; density gradients), all with sigma > 0 and
// no early stop.  The attenuation argument is spelled -delta_t * delta_scale * sigma in the first
// march and -delta_t * sigma * delta_scale in the other two, as in the reference.  The reference's
// out_dim atomics per sample on the density entry are summed first and added once.  The colour terms of the second
// march are added by the whole wavefront, flat over the records of the lanes that have one in the step, as in
// render_backward_generic_kernel (same LDS layout: the second block of out_dim scalars per lane holds the ray's
// residual instead of grad_out), into both arrays.
template <typename T, class Source>
__global__ __launch_bounds__(kMarchThreads) void se_grad_generic_kernel(TreeDev<T> tr, Source src,
                                                                        SvoxRenderOptions opt, int out_dim,
                                                                        const T* __restrict__ color_ref,
                                                                        T* __restrict__ color_out,
                                                                        T* __restrict__ grad, T* __restrict__ hess) {
    extern __shared__ __align__(16) unsigned char generic_lds[];
    const int lane = threadIdx.x;
    const bool rgba = opt.format == SVOX_FORMAT_RGBA;
    const int bd = (rgba ? 1 : opt.basis_dim) | 1;                          // row length, odd
    T* const sh_basis = (T*)generic_lds;                                    // [lane * bd + i]
    T* const sh_resid = sh_basis + kMarchThreads * bd;                      // [c * 64 + lane]: residual of the ray
    T* const sh_factor = sh_resid + kMarchThreads * out_dim;                // [c * 64 + lane]: grad_ci of the sample
    int64_t* const sh_base = (int64_t*)(sh_factor + kMarchThreads * out_dim);   // [lane]: leaf * K
    uint8_t* const sh_list = (uint8_t*)(sh_base + kMarchThreads);           // lanes with a record in this step

    T offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    T origin[3], dir[3], vdir[3];
    const int64_t item = blockIdx.x * (int64_t)kMarchThreads + lane;
    const int64_t slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
    const T bg = (T)opt.background_brightness;
    RayState<T> r;
    bool alive = slot >= 0 && setup_ray(r, origin, dir, scaling);
    if (slot >= 0 && !alive) {
        for (int j = 0; j < out_dim; ++j) color_out[slot * out_dim + j] = bg;
    }
    if (alive && !rgba) {
        T basis[SVOX_MAX_BASIS_DIM];
        precalc_basis<T>(opt.format, opt.basis_dim, tr.extra, tr.extra_cols, vdir, basis);
#pragma unroll
        for (int i = 0; i < SVOX_MAX_BASIS_DIM; ++i)
            if (i < opt.basis_dim) sh_basis[lane * bd + i] = basis[i];
    }
    wave_lds_sync();
    const T* const my_basis = sh_basis + lane * bd;
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    const int lo = rgba ? 0 : opt.min_comp;
    const int n_comp = rgba ? 1 : (opt.max_comp - opt.min_comp + 1 > 0 ? opt.max_comp - opt.min_comp + 1 : 0);
    const int per_record = out_dim * n_comp;
    const T tmin = alive ? r.t : T(0);
    T resid[4] = {T(0), T(0), T(0), T(0)};
    if (alive) {
        T light = T(1);
        while (r.t < r.tmax) {
            T delta_t;
            const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
            if (v.leaf < 0) break;
            const T* val = tr.data + v.leaf * tr.K;
            T sigma = val[tr.K - 1];
            if (opt.density_softplus) sigma = softplus_m1(sigma);
            if (sigma > T(0)) {
                const T att = exp_sp<T>(-delta_t * r.dscale * sigma);
                const T weight = light * (T(1) - att);
                for (int c = 0; c < out_dim; ++c)
                    resid[c] = fma_(weight, fma_(channel_sigmoid(opt, my_basis, val, c), d_rgb_pad, -pad), resid[c]);
                light *= att;
            }
            advance(r, delta_t);
        }
        for (int j = 0; j < out_dim; ++j) {
            resid[j] += fma_(light, bg, -color_ref[slot * out_dim + j]);
            sh_resid[j * kMarchThreads + lane] = resid[j];
        }
    }
    wave_lds_sync();
    T color_accum[4] = {T(0), T(0), T(0), T(0)};
    {
        T light = T(1);
        if (alive) r.t = tmin;
        bool marching = alive;   // (a broken tree ends this march, not the ray: the reference breaks out of the loop)
        while (__any(marching && r.t < r.tmax)) {
            bool emit = false;
            if (marching && r.t < r.tmax) {
                T delta_t;
                const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
                if (v.leaf < 0) {
                    marching = false;
                } else {
                    const int64_t base = v.leaf * tr.K;
                    const T* val = tr.data + base;
                    T sigma = val[tr.K - 1];
                    if (opt.density_softplus) sigma = softplus_m1(sigma);
                    if (sigma > T(0)) {
                        const T att = exp_sp<T>(-delta_t * sigma * r.dscale);
                        const T weight = light * (T(1) - att);
                        for (int c = 0; c < out_dim; ++c) {
                            const T sg = channel_sigmoid(opt, my_basis, val, c);
                            sh_factor[c * kMarchThreads + lane] =
                                rgba ? weight * sg * (T(1) - sg) * d_rgb_pad
                                     : (T)((double)(weight * sg) * (1.0 - (double)sg) * (double)d_rgb_pad);
                            color_accum[c] = fma_(weight, fma_(sg, d_rgb_pad, -pad), color_accum[c]);
                        }
                        sh_base[lane] = base;
                        emit = per_record > 0;
                        light *= att;
                    }
                    advance(r, delta_t);
                }
            }
            const unsigned long long m = __ballot(emit);
            if (m != 0) {
                if (emit) sh_list[rank_in(m)] = (uint8_t)lane;
                wave_lds_sync();
                const int n_scalars = __popcll(m) * per_record;
                for (int f = lane; f < n_scalars; f += kMarchThreads) {
                    const int rec = f / per_record, e = f - rec * per_record;
                    const int c = e / n_comp, i = lo + (e - c * n_comp);
                    const int owner = sh_list[rec];
                    const T grad_ci = sh_factor[c * kMarchThreads + owner];
                    const T grad_wi = rgba ? grad_ci : sh_basis[owner * bd + i] * grad_ci;
                    const int64_t at = sh_base[owner] + (rgba ? c : c * opt.basis_dim + i);
                    atomicAdd(grad + at, grad_wi * sh_resid[c * kMarchThreads + owner]);
                    atomicAdd(hess + at, grad_wi * grad_wi);
                }
                wave_lds_sync();
            }
        }
        if (alive)
            for (int j = 0; j < out_dim; ++j) color_accum[j] = fma_(light, bg, color_accum[j]);
    }
    if (!alive) return;
    {
        T light = T(1);
        r.t = tmin;
        while (r.t < r.tmax) {
            T delta_t;
            const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
            if (v.leaf < 0) break;
            const int64_t base = v.leaf * tr.K;
            const T* val = tr.data + base;
            const T raw_sigma = val[tr.K - 1];
            const T sigma = opt.density_softplus ? softplus_m1(raw_sigma) : raw_sigma;
            if (sigma > T(0)) {
                const T att = exp_sp<T>(-delta_t * sigma * r.dscale);
                const T weight = light * (T(1) - att);
                T color_curr[4];
                for (int c = 0; c < out_dim; ++c) {
                    color_curr[c] = fma_(channel_sigmoid(opt, my_basis, val, c), d_rgb_pad, -pad);
                    color_accum[c] = fma_(-weight, color_curr[c], color_accum[c]);
                }
                light *= att;
                T g = T(0), h = T(0);
                for (int j = 0; j < out_dim; ++j) {
                    const T grad_sigma = delta_t * r.dscale * fma_(color_curr[j], light, -color_accum[j]);
                    const T grad2_sigma = grad_sigma * grad_sigma;
                    if (opt.density_softplus) {
                        const T sg = sigmoid_(raw_sigma - T(1));
                        const T d_sg = sg * (T(1) - sg);
                        g += grad_sigma * resid[j] * sg;
                        h += fma_(grad2_sigma * sg, sg, grad_sigma * d_sg);
                    } else {
                        g += grad_sigma * resid[j];
                        h += grad2_sigma;
                    }
                }
                atomicAdd(grad + base + tr.K - 1, g);
                atomicAdd(hess + base + tr.K - 1, h);
            }
            advance(r, delta_t);
        }
    }
    for (int j = 0; j < out_dim; ++j) color_out[slot * out_dim + j] = resid[j] + color_ref[slot * out_dim + j];
}

// trace_ray_se_grad_hess, octree flavour: the backward kernel's persistent wavefront and rounds.
// Two marches instead of three: march 1 forms the residual with the first spelling of the
// attenuation and, beside it, the rendered colour with the second spelling (what the reference's
// second march accumulates); march 2 then produces, per leaf with sigma > 0, both the colour terms
// (the reference's second march) and the density terms (its third).  Every term has the reference's
// value; records are added cooperatively, one coalesced atomic instruction per record element and
// output array, after summing the lanes whose rays sit in the same leaf.
template <class P, class Source, bool kRefill>
__global__ __launch_bounds__(kMarchThreads) void se_grad_kernel(TreeDev<float> tr, Source src, SvoxRenderOptions opt,
                                                                const float* __restrict__ color_ref,
                                                                float* __restrict__ color_out,
                                                                float* __restrict__ grad_data,
                                                                float* __restrict__ hess_data,
                                                                const unsigned long long* __restrict__ only) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    __shared__ int32_t path[(kPathLevels + 1) * kMarchThreads];
    __shared__ ShadeShared<D, true> sh;
    const int lane = threadIdx.x;
    float offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    const float step = opt.step_size;

    int64_t next = chunk_of_block(blockIdx.x, gridDim.x, src.xcd_group) * (int64_t)src.per_wave;
    const int64_t total = src.total();
    const int64_t end = next + src.per_wave < total ? next + src.per_wave : total;

    RayState<float> r;
    float ref[3] = {0.f, 0.f, 0.f};
    float resid[3] = {0.f, 0.f, 0.f};    // march 1: colour so far; afterwards the residual
    float caccum[3] = {0.f, 0.f, 0.f};   // rendered colour not yet passed (second spelling)
    float light = 1.0f, light1 = 1.0f, tmin = 0.0f;
    int64_t slot = -1;
    bool active = false, second = false;
    OctreeCursor cur;
    cur.reset(path + lane, kMarchThreads);

    // takes ray `item` into this lane: a miss is answered at once, a hit becomes the lane's ray
    // (with a bitmap `only` the launch does the rays whose bit is set and no others; a batch launch
    // then does not deal its rays out: its items are ray numbers)
    auto start = [&](int64_t item) {
        float origin[3], dir[3], vdir[3];
        if (Source::kItemsAreSlots && only && !((only[item >> 6] >> (item & 63)) & 1ull)) return;
        slot = src.fetch_item(item, opt, offset, scaling, origin, dir, vdir);
        if (slot < 0) return;
        if (!Source::kItemsAreSlots && only && !((only[slot >> 6] >> (slot & 63)) & 1ull)) return;
        if (setup_ray(r, origin, dir, scaling)) {
            if constexpr (P::kFormat != SVOX_FORMAT_RGBA) {
                float basis[D];
                policy_basis<P>(Lobes{tr.extra, tr.extra_cols, opt.format}, opt, vdir, basis);
#pragma unroll
                for (int i = 0; i < D; ++i) sh.basis[lane * D + i] = basis[i];
            }
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                ref[c] = color_ref[slot * 3 + c];
                resid[c] = 0.0f;
                caccum[c] = 0.0f;
            }
            light = light1 = 1.0f;
            tmin = r.t;
            cur.restart();
            second = false;
            active = true;
        } else {
            color_out[slot * 3] = bg;
            color_out[slot * 3 + 1] = bg;
            color_out[slot * 3 + 2] = bg;
        }
    };
    if constexpr (!kRefill) {
        if (next + lane < end) start(next + lane);
    }

    while (true) {
        if constexpr (kRefill) {
            if (Source::kItemsAreSlots && only) next = skip_clear_words(only, next, end, lane);
            const RoundState state = refill_lanes(active, next, end, src.refill_at, start);
            if (state == kRoundRefilled) continue;
            if (state == kRoundDone) break;
        } else {
            if (!__any(active)) break;
        }

        // ---- walk
        int32_t q_leaf[kQueue];
        float q_dt[kQueue];
        bool broken;
        walk_turns(tr, r, cur, step, active, broken, q_leaf, q_dt);
        // ---- sigma
        float q_sigma[kQueue], q_raw[kQueue];
        fetch_sigma<K>(tr.data, q_leaf, q_sigma);
        soften_sigma(opt.density_softplus, q_leaf, q_sigma, q_raw);
        // ---- shade list
        const int n_entries = build_shade_list(sh, q_leaf, q_sigma, 0.0f, lane);
        wave_lds_sync();
        shade_entries<P, true>(tr.data, sh, n_entries, lane);
        wave_lds_sync();
        // ---- composite and emit, slot by slot
#pragma unroll
        for (int q = 0; q < kQueue; ++q) {
            bool emit = false;
            float gci[3] = {0.f, 0.f, 0.f};
            float g_sigma = 0.f, h_sigma = 0.f;
            if (active && q_leaf[q] >= 0 && q_sigma[q] > 0.0f) {
                const float att = expf_fixed(-q_dt[q] * q_sigma[q] * r.dscale);
                const float weight = light * (1.0f - att);
                const float* s = sh.colour + (q * kMarchThreads + lane) * 3;
                float col[3];
#pragma unroll
                for (int c = 0; c < 3; ++c) col[c] = fma_(s[c], d_rgb_pad, -pad);
                light *= att;
                if (!second) {
                    const float att1 = expf_fixed(-q_dt[q] * r.dscale * q_sigma[q]);
                    const float weight1 = light1 * (1.0f - att1);
                    light1 *= att1;
#pragma unroll
                    for (int c = 0; c < 3; ++c) {
                        resid[c] = fma_(weight1, col[c], resid[c]);
                        caccum[c] = fma_(weight, col[c], caccum[c]);
                    }
                } else {
                    // (density_softplus: the chain factor of rt_kernel.cu:693-703; 1 and 0 without it)
                    const float sg = opt.density_softplus ? sigmoid_(q_raw[q] - 1.0f) : 1.0f;
                    const float d_sg = sg * (1.0f - sg);
#pragma unroll
                    for (int c = 0; c < 3; ++c) {
                        if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
                            gci[c] = weight * s[c] * (1.0f - s[c]) * d_rgb_pad;
                        } else {
                            gci[c] = (float)((double)(weight * s[c]) * (1.0 - (double)s[c]) * (double)d_rgb_pad);
                        }
                        caccum[c] = fma_(-weight, col[c], caccum[c]);
                        const float gs = q_dt[q] * r.dscale * fma_(col[c], light, -caccum[c]);
                        if (opt.density_softplus) {
                            g_sigma += gs * resid[c] * sg;
                            h_sigma += fma_(gs * gs * sg, sg, gs * d_sg);
                        } else {
                            g_sigma += gs * resid[c];
                            h_sigma += gs * gs;
                        }
                    }
                    emit = true;
                }
            }
            unsigned long long todo = __ballot(emit);
            while (todo) {
                const int leader = __ffsll((long long)todo) - 1;
                const int32_t leaf_l = __builtin_amdgcn_readlane(q_leaf[q], leader);
                const unsigned long long same = __ballot(emit && q_leaf[q] == leaf_l);
                todo &= ~same;
                float* g = grad_data + (int64_t)leaf_l * K;
                float* h = hess_data + (int64_t)leaf_l * K;
#pragma unroll
                for (int e0 = 0; e0 < K; e0 += 64) {
                    const int e = e0 + lane;
                    float g_val = 0.0f, h_val = 0.0f;
                    unsigned long long members = same;
                    while (members) {
                        const int k = __ffsll((long long)members) - 1;
                        members &= members - 1;
                        const float t0 = read_lane(gci[0], k), t1 = read_lane(gci[1], k), t2 = read_lane(gci[2], k);
                        const float r0 = read_lane(resid[0], k), r1 = read_lane(resid[1], k),
                                    r2 = read_lane(resid[2], k);
                        const float gs = read_lane(g_sigma, k), hs = read_lane(h_sigma, k);
                        float g_term, h_term;
                        if constexpr (P::kFormat == SVOX_FORMAT_RGBA) {
                            const float tc = e == 0 ? t0 : e == 1 ? t1 : t2;
                            const float rc = e == 0 ? r0 : e == 1 ? r1 : r2;
                            g_term = e < 3 ? tc * rc : gs;
                            h_term = e < 3 ? tc * tc : hs;
                        } else {
                            const int c = e / D;
                            const float b = e < 3 * D ? sh.basis[k * D + (e - c * D)] : 0.0f;
                            const float gw = b * (c == 0 ? t0 : c == 1 ? t1 : t2);
                            const float rc = c == 0 ? r0 : c == 1 ? r1 : r2;
                            g_term = e < 3 * D ? gw * rc : gs;
                            h_term = e < 3 * D ? gw * gw : hs;
                        }
                        g_val += g_term;
                        h_val += h_term;
                    }
                    if (e < K) {
                        atomicAdd(g + e, g_val);
                        atomicAdd(h + e, h_val);
                    }
                }
            }
        }
        // ---- end of a march
        if (active && (broken || !(r.t < r.tmax))) {
            if (!second && !broken) {
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    resid[c] += fma_(light1, bg, -ref[c]);
                    caccum[c] = fma_(light, bg, caccum[c]);
                }
                light = 1.0f;
                r.t = tmin;
                second = true;
            } else {
#pragma unroll
                for (int c = 0; c < 3; ++c) color_out[slot * 3 + c] = resid[c] + ref[c];
                active = false;
            }
        }
    }
}

// se_grad from the notes a noting forward kernel left (NoteTaker; taken with both thresholds at
// zero): one lane per ray, no tree walk.  The first pass over a ray's notes forms the residual and the
// rendered colour as march 1 of se_grad_kernel does, the second pass the gradient and Hessian records
// of its march 2, term by term the same values; the wavefront adds the records of its rays together,
// each lane serving one element of one record (RecordList::flush_by_record's scheme, with two output
// arrays).  Rays that miss the tree keep the background colour the noting launch wrote; a ray whose
// notes are incomplete, or every ray if the workspace carries another stamp, is marked in the bitmap
// for a launch of se_grad_kernel.
constexpr int kSeRecordCap = 48;
static_assert(kSeRecordCap <= kMarchThreads, "group_by_leaf holds one record per lane");

template <class P, class Source>
__global__ __launch_bounds__(kMarchThreads) void replay_se_grad_kernel(Source src, SvoxRenderOptions opt,
                                                                       const float* __restrict__ color_ref,
                                                                       float* __restrict__ color_out,
                                                                       float* __restrict__ grad_data,
                                                                       float* __restrict__ hess_data,
                                                                       ReplaySpace ws, int ray_shift, Lobes lobes) {
    constexpr int D = P::kBasis > 0 ? P::kBasis : 1;
    constexpr int K = P::kRecord;
    constexpr bool kRgba = P::kFormat == SVOX_FORMAT_RGBA;
    __shared__ float basis_rows[kMarchThreads * D];
    __shared__ float resid_rows[kMarchThreads * 3];
    __shared__ int32_t l_leaf[kSeRecordCap];
    // per record four gradient factors (the three colour factors, then the density term) and the
    // density term of the Hessian
    __shared__ float l_factor[kSeRecordCap * 4], l_hs[kSeRecordCap];
    __shared__ uint8_t l_owner[kSeRecordCap];
    __shared__ GroupScratch group;
    const int lane = threadIdx.x;
    // 2^ray_shift consecutive rays per wavefront (64, or 16 for the pixels of images), as in
    // replay_backward_kernel
    const int64_t ray = ((int64_t)blockIdx.x << ray_shift) + lane;
    const bool seated = lane < (1 << ray_shift);
    const bool stamped = stamp_matches(ws);
    const float2* first = ws.base + ray * kChunkFloat2;
    int count = 0;
    int32_t first_link = 0;
    float dscale = 0.0f;
    bool missed = true;
    if (seated && ray < src.n_slots()) {
        const float2 head = first[kHeadFloat2], tail = first[kHeadFloat2 + 1];
        first_link = __float_as_int(head.x);
        count = stamped ? __float_as_int(head.y) : -1;
        dscale = tail.x;
        missed = tail.y != 0.0f;
    }
    const unsigned long long undone = __ballot(count < 0);
    if (lane == 0) {
        if (ray_shift == 6)
            ws.undone[blockIdx.x] = undone;
        else
            ((uint16_t*)ws.undone)[blockIdx.x] = (uint16_t)undone;
    }
    const bool hit = count >= 0 && !missed;   // the rays this launch answers
    const bool work = hit && count > 0;
    if (!__any(hit)) return;

    const float bg = opt.background_brightness;
    const float pad = opt.rgb_padding;
    const float d_rgb_pad = 1 + 2 * opt.rgb_padding;
    float ref[3] = {0.f, 0.f, 0.f};
    if (hit) {
        ref[0] = color_ref[ray * 3];
        ref[1] = color_ref[ray * 3 + 1];
        ref[2] = color_ref[ray * 3 + 2];
    }
    if (work) {
        if constexpr (!kRgba) {
            float vdir[3];
            src.view_dir(ray, vdir);
            float basis[D];
            policy_basis<P>(lobes, opt, vdir, basis);
#pragma unroll
            for (int i = 0; i < D; ++i) basis_rows[lane * D + i] = basis[i];
        }
    }

    int n = 0;   // records in the list (wavefront-uniform)
    MergeState merge{2};
    auto flush = [&]() {
        if (n == 0) return;
        wave_lds_sync();
        // where enough records share a leaf, the records of a leaf are brought together first
        const bool grouped = group_by_leaf(group, merge, l_leaf, n, lane);
        auto emit = [&](int32_t leaf, int e, const float* sum) {
            const int64_t at = (int64_t)leaf * K + e;
            atomicAdd(grad_data + at, sum[0]);
            atomicAdd(hess_data + at, sum[1]);
        };
        if constexpr (K > kMarchThreads / 2) {
            // One record at a time, lane e on element e; place, leaf and owner of the records are held
            // in registers, record r by lane r, and handed round by readlane, so that the LDS reads of a
            // record have their addresses from scalars and those of four records are in flight together
            // (RecordList::add_held).
            const bool mine = lane < n;
            const int my_rec = mine ? (grouped ? group.order[lane] : lane) : 0;
            const int my_leaf = l_leaf[my_rec];
            const int my_owner = l_owner[my_rec];
            constexpr int kBlock = 4;
            // (a loop every lane runs, so that every lane holds its record when readlane looks: see add_held)
            for (int e0 = 0; e0 < K; e0 += kMarchThreads) {
                const int e = e0 + lane;
                const bool on = e < K;
                const int c_raw = kRgba ? e : e / D;
                const int c = c_raw < 3 ? c_raw : 3;
                const int i = kRgba || c == 3 ? 0 : e - c * D;
                const int cc = c < 3 ? c : 0;
                int32_t cur = -1;
                float acc[2] = {0.0f, 0.0f};
                for (int at = 0; at < n; at += kBlock) {
                    int32_t leaf[kBlock];
                    float f[kBlock], b[kBlock], rs[kBlock], hs[kBlock];
#pragma unroll
                    for (int u = 0; u < kBlock; ++u) {
                        const int a = at + u < n ? at + u : n - 1;   // (past the end: the last record again, unused)
                        const int rec = __builtin_amdgcn_readlane(my_rec, a);
                        const int owner = __builtin_amdgcn_readlane(my_owner, a);
                        leaf[u] = __builtin_amdgcn_readlane(my_leaf, a);
                        f[u] = l_factor[rec * 4 + c];
                        b[u] = kRgba ? 1.0f : basis_rows[owner * D + i];
                        rs[u] = resid_rows[owner * 3 + cc];
                        hs[u] = l_hs[rec];
                    }
#pragma unroll
                    for (int u = 0; u < kBlock; ++u) {
                        if (at + u < n) {
                            if (leaf[u] != cur) {
                                if (on && cur >= 0) emit(cur, e, acc);
                                cur = leaf[u];
                                acc[0] = acc[1] = 0.0f;
                            }
                            const float gw = kRgba ? f[u] : b[u] * f[u];
                            acc[0] += c < 3 ? gw * rs[u] : f[u];
                            acc[1] += c < 3 ? gw * gw : hs[u];
                        }
                    }
                }
                if (on && cur >= 0) emit(cur, e, acc);
            }
        } else {
            add_records_by_leaf<K, 2>(
                n, lane, grouped ? group.leaf : l_leaf,
                // element e of a record: colour coefficient (c, i) or, last, the density
                [&](int at, int e, float* t) {
                    const int rec = grouped ? group.order[at] : at;
                    const int c = kRgba ? e : e / D;
                    if (c < 3) {
                        const int owner = l_owner[rec];
                        const float v = l_factor[rec * 4 + c];
                        const float gw = kRgba ? v : basis_rows[owner * D + (e - c * D)] * v;
                        t[0] = gw * resid_rows[owner * 3 + c];
                        t[1] = gw * gw;
                    } else {
                        t[0] = l_factor[rec * 4 + 3];
                        t[1] = l_hs[rec];
                    }
                },
                emit);
        }
        wave_lds_sync();
        n = 0;
    };
    // the record of every lane with `emit` set joins the list (in lane order)
    auto append = [&](bool emit, int32_t leaf, const float* gci, float g_sigma, float h_sigma) {
        unsigned long long todo = __ballot(emit);
        while (todo) {
            if (n == kSeRecordCap) flush();
            const bool pending = (todo >> lane) & 1ull;
            const int at = n + rank_in(todo);
            const bool take = pending && at < kSeRecordCap;
            if (take) {
                l_leaf[at] = leaf;
                l_owner[at] = (uint8_t)lane;
                l_hs[at] = h_sigma;
                l_factor[at * 4] = gci[0];
                l_factor[at * 4 + 1] = gci[1];
                l_factor[at * 4 + 2] = gci[2];
                l_factor[at * 4 + 3] = g_sigma;
            }
            const unsigned long long taken = __ballot(take);
            n += __popcll(taken);
            todo &= ~taken;
        }
    };

    float resid[3] = {0.f, 0.f, 0.f};    // pass 0: colour so far; afterwards the residual
    float caccum[3] = {0.f, 0.f, 0.f};   // rendered colour not yet passed (second spelling)
    float light = 1.0f, light1 = 1.0f;
    struct Group {
        float2 note[kReplayGroup][3];
    };
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
        const float2* chunk = first;
        int32_t link = first_link;
        int pos = 0;
        auto fetch = [&](Group& g, int base) {
            if (work && base < count) {
                if (pos == kChunkRecords) {
                    chunk = ws.base + (int64_t)link * kChunkFloat2;
                    link = __float_as_int(chunk[kHeadFloat2].x);
                    pos = 0;
                }
#pragma unroll
                for (int k = 0; k < kReplayGroup; ++k) {
#pragma unroll
                    for (int j = 0; j < 3; ++j) g.note[k][j] = chunk[(pos + k) * 3 + j];
                }
                pos += kReplayGroup;
            }
        };
        auto work_on = [&](const Group& g, int base) {
#pragma unroll
            for (int k = 0; k < kReplayGroup; ++k) {
                const bool have = work && base + k < count;
                const int32_t leaf = __float_as_int(g.note[k][0].x);
                const float dt = g.note[k][0].y, raw = g.note[k][1].x;   // (the stored density)
                const float s[3] = {g.note[k][1].y, g.note[k][2].x, g.note[k][2].y};
                float gci[3] = {0.f, 0.f, 0.f};
                float g_sigma = 0.0f, h_sigma = 0.0f;
                if (have) {
                    const float sigma = opt.density_softplus ? softplus_m1(raw) : raw;
                    const float att = expf_fixed(-dt * sigma * dscale);
                    const float weight = light * (1.0f - att);
                    float col[3];
#pragma unroll
                    for (int c = 0; c < 3; ++c) col[c] = fma_(s[c], d_rgb_pad, -pad);
                    light *= att;
                    if (pass == 0) {
                        const float att1 = expf_fixed(-dt * dscale * sigma);
                        const float weight1 = light1 * (1.0f - att1);
                        light1 *= att1;
#pragma unroll
                        for (int c = 0; c < 3; ++c) {
                            resid[c] = fma_(weight1, col[c], resid[c]);
                            caccum[c] = fma_(weight, col[c], caccum[c]);
                        }
                    } else {
                        const float sg = opt.density_softplus ? sigmoid_(raw - 1.0f) : 1.0f;
                        const float d_sg = sg * (1.0f - sg);
#pragma unroll
                        for (int c = 0; c < 3; ++c) {
                            if constexpr (kRgba) {
                                gci[c] = weight * s[c] * (1.0f - s[c]) * d_rgb_pad;
                            } else {
                                gci[c] = (float)((double)(weight * s[c]) * (1.0 - (double)s[c]) * (double)d_rgb_pad);
                            }
                            caccum[c] = fma_(-weight, col[c], caccum[c]);
                            const float gs = dt * dscale * fma_(col[c], light, -caccum[c]);
                            if (opt.density_softplus) {
                                g_sigma += gs * resid[c] * sg;
                                h_sigma += fma_(gs * gs * sg, sg, gs * d_sg);
                            } else {
                                g_sigma += gs * resid[c];
                                h_sigma += gs * gs;
                            }
                        }
                    }
                }
                if (pass == 1) append(have, leaf, gci, g_sigma, h_sigma);
            }
        };
        Group a, b;
        fetch(a, 0);
        for (int base = 0; __any(work && base < count); base += 2 * kReplayGroup) {
            fetch(b, base + kReplayGroup);
            work_on(a, base);
            fetch(a, base + 2 * kReplayGroup);
            work_on(b, base + kReplayGroup);
        }
        if (pass == 0) {
            // the end of march 1 (rt_kernel.cu:560-563, the background of :635-637, and :711-713)
            if (hit) {
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    resid[c] += fma_(light1, bg, -ref[c]);
                    caccum[c] = fma_(light, bg, caccum[c]);
                    color_out[ray * 3 + c] = resid[c] + ref[c];
                    resid_rows[lane * 3 + c] = resid[c];
                }
            }
            light = 1.0f;
            wave_lds_sync();   // basis and residual rows are read by other lanes when the records are added
        }
    }
    flush();
}

// ------------------------------------------------------------------------------------------------
// dense-grid weight render
// ------------------------------------------------------------------------------------------------
// grid_trace_ray + grid_weight_render_kernel, rt_kernel.cu:898-1003: one pixel ray per lane through a
// dense reso^3 density grid; per cell with sigma > sigma_thresh the largest compositing weight any
// ray gave it and the number of visits.
template <typename T>
__global__ __launch_bounds__(kMarchThreads) void grid_weight_kernel(const T* __restrict__ data, int reso,
                                                                    ImageSource<T> src, SvoxRenderOptions opt,
                                                                    const T* __restrict__ offset_p,
                                                                    const T* __restrict__ scaling_p,
                                                                    T* __restrict__ grid_weight,
                                                                    T* __restrict__ grid_hit) {
    T offset[3], scaling[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        offset[i] = offset_p[i];
        scaling[i] = scaling_p[i];
    }
    T origin[3], dir[3], vdir[3];
    const int64_t item = blockIdx.x * (int64_t)kMarchThreads + threadIdx.x;
    if (src.fetch_item(item, opt, offset, scaling, origin, dir, vdir) < 0) return;
    RayState<T> r;
    if (!setup_ray(r, origin, dir, scaling)) return;
    const T cube_sz = (T)reso;
    T light = T(1);
    while (r.t < r.tmax) {
        T pos[3];
        int32_t uvw[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            pos[j] = clamp01(fma_(r.t, r.d[j], r.o[j])) * cube_sz;
            uvw[j] = (int32_t)floor_(pos[j]);
            pos[j] -= (T)uvw[j];
        }
        const int32_t node_id = uvw[0] * reso * reso + uvw[1] * reso + uvw[2];
        T s0, s1;
        dda_unit(pos, r.inv, &s0, &s1);
        const T delta_t = (s1 - s0) / cube_sz + (T)opt.step_size;
        const T sigma = data[node_id];
        if (sigma > (T)opt.sigma_thresh) {
            const T att = exp_sp<T>(-delta_t * r.dscale * sigma);
            const T weight = light * (T(1) - att);
            light *= att;
            atomic_max_float(grid_weight + node_id, weight);
            atomicAdd(grid_hit + node_id, T(1));
        }
        advance(r, delta_t);
    }
}

// ------------------------------------------------------------------------------------------------
// visit counters
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long wave_sum(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned lo = __shfl_down((unsigned)(v & 0xffffffffull), off);
        const unsigned hi = __shfl_down((unsigned)(v >> 32), off);
        v += ((unsigned long long)hi << 32) | lo;
    }
    return v;
}

// Counts, with the reference's walk, what the forward march (thresholds, early stop) and one
// backward march (sigma > 0, no stop) of every ray visit.
template <typename T, class Source>
__global__ __launch_bounds__(kMarchThreads) void render_stats_kernel(TreeDev<T> tr, Source src,
                                                                     SvoxRenderOptions opt,
                                                                     unsigned long long* __restrict__ stats) {
    T offset[3], scaling[3];
    load_transform(tr, offset, scaling);
    T origin[3], dir[3], vdir[3];
    const int64_t slot = src.fetch_item(blockIdx.x * (int64_t)kMarchThreads + threadIdx.x, opt, offset, scaling,
                                        origin, dir, vdir);
    unsigned long long c_rays = 0, c_hit = 0, c_samples = 0, c_shaded = 0, c_bwd = 0, c_bwd_pos = 0, c_levels = 0;
    unsigned long long c_tail = 0;
    if (slot >= 0) {
        c_rays = 1;
        RayState<T> r;
        if (setup_ray(r, origin, dir, scaling)) {
            c_hit = 1;
            T light = T(1);
            bool fwd_live = true;
            unsigned since_shaded = 0;   // forward visits since the ray's last shaded leaf
            while (r.t < r.tmax) {
                T delta_t;
                const Visit v = step_generic<T>(tr, r, (T)opt.step_size, &delta_t);
                if (v.leaf < 0) break;
                T sigma = tr.data[v.leaf * tr.K + tr.K - 1];
                if (opt.density_softplus) sigma = softplus_m1(sigma);
                c_bwd += 1;
                if (sigma > T(0)) c_bwd_pos += 1;
                if (fwd_live) {
                    c_samples += 1;
                    c_levels += (unsigned)v.levels;
                    since_shaded += 1;
                    if (sigma > (T)opt.sigma_thresh) {
                        c_shaded += 1;
                        since_shaded = 0;
                        light *= exp_sp<T>(-delta_t * r.dscale * sigma);
                        if (light <= (T)opt.stop_thresh) fwd_live = false;
                    }
                }
                advance(r, delta_t);
            }
            c_tail = since_shaded;
        }
    }
    // every lane reaches the reductions
    c_rays = wave_sum(c_rays);
    c_hit = wave_sum(c_hit);
    c_samples = wave_sum(c_samples);
    c_shaded = wave_sum(c_shaded);
    c_bwd = wave_sum(c_bwd);
    c_bwd_pos = wave_sum(c_bwd_pos);
    c_levels = wave_sum(c_levels);
    c_tail = wave_sum(c_tail);
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(stats + 0, c_rays);
        atomicAdd(stats + 1, c_hit);
        atomicAdd(stats + 2, c_samples);
        atomicAdd(stats + 3, c_shaded);
        atomicAdd(stats + 4, c_bwd);
        atomicAdd(stats + 5, c_bwd_pos);
        atomicAdd(stats + 6, c_levels);
        atomicAdd(stats + 7, c_tail);
    }
}

}  // namespace svox
