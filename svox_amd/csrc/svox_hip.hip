// svox_hip.hip -- the extern "C" entry points of libsvox_hip.so (declared in include/svox_hip.h):
// argument validation, kernel selection and launches.  Each entry point stands where one function
// of the reference's extension module stood (svox/csrc/svox.cpp:106-121; host launchers
// svox/csrc/svox_kernel.cu:120-203 and svox/csrc/rt_kernel.cu:1009-1109).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/svox_hip.h"
#include "march_kernels.h"
#include "query_kernels.h"

#include <mutex>

// Workspace of svox_volume_render_backward_static: one array per GPU, inside the library's code object.
// In host code the name `scratch` is only a handle for hipGetSymbolAddress (static_workspace below); it
// is never passed to a kernel or a runtime call as an address.
static_assert(SVOX_STATIC_WORKSPACE_BYTES % 256 == 0, "whole 256-byte units");
static __device__ __align__(256) unsigned char scratch[SVOX_STATIC_WORKSPACE_BYTES];

namespace {

using namespace svox;

thread_local char g_error[512] = "";
// Debug flags of the calling thread (svox_set_debug_flags): bit 0: always take the generic kernels; bit 1: small
// batches run like large ones; bit 2: forward launches never take the two-wavefront kernel; bit 3: they always
// do (where it applies).  Per thread, so that one thread's tests cannot change the kernels of another's calls.
thread_local int g_debug_flags = 0;

// Launch-shape overrides for experiments, read from the environment once, when the first launch of the process
// picks a shape; the library has no other mutable state besides g_error / g_debug_flags (per thread) and the
// per-device address of `scratch`.  Every field is 0 / -1 ("not set") in normal use:
//   SVOX_PER_WAVE      rays a persistent wavefront of a batch launch owns (64, 128, 256, 512 or 1024)
//   SVOX_REFILL        idle lanes at which such a wavefront takes new rays (1..64)
//   SVOX_XCD_GROUP     consecutive image tiles handed to one XCD (1..4096)
//   SVOX_TILE_ORDER    0: 16x16 blocks of an image row by row, 1: ring by ring from the middle
//   SVOX_IMAGE_RUN     16x16 blocks of one image in a row before the next image's, in multi-image launches
//   SVOX_SPLIT_FORWARD 0 / 1: forward launches never / always on two wavefronts per tile
//   SVOX_SPLIT_BLOCKS  largest forward launch (in tiles) that takes two wavefronts per tile
//   SVOX_REPLAY_SHIFT  4 or 6: log2 of the rays a wavefront of the replay kernels takes
struct Tuning {
    int per_wave = 0, refill = 0, xcd_group = 0, tile_order = -1, image_run = -1, split_forward = -1, replay_shift = -1;
    long split_blocks = -1;
};
const Tuning& tuning() {
    static const Tuning t = [] {
        Tuning v;
        auto num = [](const char* name, long unset) {
            const char* e = getenv(name);
            return e ? atol(e) : unset;
        };
        v.per_wave = (int)num("SVOX_PER_WAVE", 0);
        v.refill = (int)num("SVOX_REFILL", 0);
        v.xcd_group = (int)num("SVOX_XCD_GROUP", 0);
        v.tile_order = (int)num("SVOX_TILE_ORDER", -1);
        v.image_run = (int)num("SVOX_IMAGE_RUN", -1);
        v.split_forward = (int)num("SVOX_SPLIT_FORWARD", -1);
        v.split_blocks = num("SVOX_SPLIT_BLOCKS", -1);
        v.replay_shift = (int)num("SVOX_REPLAY_SHIFT", -1);
        return v;
    }();
    return t;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(SVOX_ERR_LAUNCH, "svox.%s: %s", what, hipGetErrorString(err));
    return SVOX_OK;
}

int check_tree(const SvoxTreeSpec* t, bool need_data) {
    if (!t) return fail(SVOX_ERR_NULL_POINTER, "tree spec is NULL");
    if (need_data && !t->data) return fail(SVOX_ERR_NULL_POINTER, "tree.data is NULL");
    if (!t->child) return fail(SVOX_ERR_NULL_POINTER, "tree.child is NULL");
    if (!t->parent_depth) return fail(SVOX_ERR_NULL_POINTER, "tree.parent_depth is NULL");
    if (t->dtype != SVOX_F32 && t->dtype != SVOX_F64)
        return fail(SVOX_ERR_BAD_DTYPE, "tree.dtype must be SVOX_F32 or SVOX_F64, got %d", t->dtype);
    if (t->capacity < 1) return fail(SVOX_ERR_BAD_SHAPE, "tree.capacity must be >= 1, got %lld", (long long)t->capacity);
    if (t->N < 2) return fail(SVOX_ERR_BAD_SHAPE, "tree.N must be >= 2, got %d", t->N);
    if (t->data_dim < 1) return fail(SVOX_ERR_BAD_SHAPE, "tree.data_dim must be >= 1, got %d", t->data_dim);
    const double cells = (double)t->capacity * t->N * t->N * t->N;
    if (cells >= 9.0e18 / (double)(t->data_dim > 0 ? t->data_dim : 1))
        return fail(SVOX_ERR_BAD_SHAPE, "tree is too large to index");
    if (t->capacity > 0x7fffffffll)
        return fail(SVOX_ERR_BAD_SHAPE, "tree.capacity exceeds the int32 node ids of the child table");
    return SVOX_OK;
}

template <typename T>
TreeDev<T> make_tree(const SvoxTreeSpec* t) {
    TreeDev<T> d;
    d.data = (T*)t->data;
    d.child = t->child;
    d.parent_depth = t->parent_depth;
    d.extra = (const T*)t->extra_data;
    d.offset = (const T*)t->offset;
    d.scaling = (const T*)t->scaling;
    d.weight_accum = (T*)t->weight_accum;
    d.capacity = t->capacity;
    d.N = t->N;
    d.K = t->data_dim;
    d.extra_cols = t->extra_cols;
    d.weight_accum_max = t->weight_accum_max;
    return d;
}

// an fp32 tree whose cells number less than 2^30 (int32 cell indices with two spare bits; for an octree that is
// fewer than 2^27 nodes and a child table below 4 GiB, which its walk addresses with 32-bit byte offsets).  Octrees
// walk on integer coordinates from the previous path; other branching factors take the reference's floating-point
// walk inside the same kernels and share the rounds, the shade list, the record lists and the notes.
bool march_fast_ok(const SvoxTreeSpec* t) {
    return !(g_debug_flags & 1) && t->dtype == SVOX_F32 && (double)t->capacity * t->N * t->N * t->N < 1073741824.0;
}
// ... and an octree among them: the point queries' integer walk
bool octree_fast_ok(const SvoxTreeSpec* t) { return march_fast_ok(t) && t->N == 2; }

int zero_fill(void* ptr, int64_t bytes, hipStream_t stream) {
    if (bytes <= 0) return SVOX_OK;
    if (((uintptr_t)ptr & 15u) != 0 || (bytes & 3) != 0)
        return fail(SVOX_ERR_BAD_SHAPE, "gradient buffer must be 16-byte aligned and a multiple of 4 bytes");
    const int64_t n16 = bytes / 16;
    const int n_tail = (int)((bytes - n16 * 16) / 4);
    int64_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint4*)ptr, n16,
                       (uint32_t*)((char*)ptr + n16 * 16), n_tail);
    return check_launch("zero_fill");
}

// ---------------------------------------------------------------------------------------------
// queries
// ---------------------------------------------------------------------------------------------
constexpr int kLdsNodesMax = 584;  // child rows kept in LDS per block: 584 * 32 B = 18.25 KiB

template <typename T, int MODE>
int launch_query(const SvoxTreeSpec* tree, const void* points, int64_t n, void* values, void* target,
                 int64_t* ids, int32_t Kx, hipStream_t stream, const char* what) {
    if (n == 0) return SVOX_OK;
    const TreeDev<T> tr = make_tree<T>(tree);
    const int64_t per_tile = (int64_t)kQueryThreads * kQueryPts;
    const int64_t tiles = (n + per_tile - 1) / per_tile;
    const int64_t blocks = tiles < 256 * 8 ? tiles : 256 * 8;
    if constexpr (sizeof(T) == 4) {
        if (octree_fast_ok(tree)) {
            const int32_t lds_nodes = tree->capacity < kLdsNodesMax ? (int32_t)tree->capacity : kLdsNodesMax;
            hipLaunchKernelGGL((query_kernel<T, MODE, true>), dim3((unsigned)blocks), dim3(kQueryThreads),
                               (size_t)lds_nodes * 32, stream, tr, (const T*)points, n, (T*)values,
                               (T*)target, ids, Kx, lds_nodes);
            return check_launch(what);
        }
    }
    hipLaunchKernelGGL((query_kernel<T, MODE, false>), dim3((unsigned)blocks), dim3(kQueryThreads), 0, stream,
                       tr, (const T*)points, n, (T*)values, (T*)target, ids, Kx, 0);
    return check_launch(what);
}

// ---------------------------------------------------------------------------------------------
// rendering
// ---------------------------------------------------------------------------------------------
int check_render(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, int* out_dim) {
    int rc = check_tree(tree, true);
    if (rc) return rc;
    if (!opt) return fail(SVOX_ERR_NULL_POINTER, "render options are NULL");
    if (opt->format < SVOX_FORMAT_RGBA || opt->format > SVOX_FORMAT_ASG)
        return fail(SVOX_ERR_BAD_SHAPE, "unknown data format %d", opt->format);
    const int od = svox_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    if (od < 0)
        return fail(SVOX_ERR_BAD_SHAPE, "basis_dim %d is invalid for format %d", opt->basis_dim, opt->format);
    if (od > SVOX_MAX_OUT_DIM)
        return fail(SVOX_ERR_UNSUPPORTED, "rendered colour dimension %d exceeds %d", od, SVOX_MAX_OUT_DIM);
    if (opt->format != SVOX_FORMAT_RGBA) {
        if (opt->basis_dim > SVOX_MAX_BASIS_DIM)
            return fail(SVOX_ERR_UNSUPPORTED, "basis_dim %d exceeds %d", opt->basis_dim, SVOX_MAX_BASIS_DIM);
        if (opt->min_comp < 0 || opt->max_comp >= opt->basis_dim)
            return fail(SVOX_ERR_BAD_SHAPE, "component range [%d, %d] outside [0, %d)", opt->min_comp,
                        opt->max_comp, opt->basis_dim);
        if (opt->format == SVOX_FORMAT_SG || opt->format == SVOX_FORMAT_ASG) {
            const int need = opt->format == SVOX_FORMAT_SG ? 4 : 11;
            if (!tree->extra_data || tree->extra_rows < opt->basis_dim || tree->extra_cols < need)
                return fail(SVOX_ERR_BAD_SHAPE, "extra_data must be (%d, >=%d) for this format", opt->basis_dim, need);
        }
    }
    *out_dim = od;
    return SVOX_OK;
}

int check_camera(const SvoxCameraSpec* cam, int n_images = 1, int64_t pose_stride = 12) {
    if (!cam) return fail(SVOX_ERR_NULL_POINTER, "camera spec is NULL");
    if (!cam->c2w) return fail(SVOX_ERR_NULL_POINTER, "cam.c2w is NULL");
    if (cam->width < 0 || cam->height < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative image size");
    if (n_images < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative image count");
    if (n_images > 1 && pose_stride < 12) return fail(SVOX_ERR_BAD_SHAPE, "pose_stride must be >= 12 scalars");
    // (+ 64: multi-image launches pad every image to a whole number of block runs)
    const double tiles = 4.0 * ((double)blocks16_of(cam->width) * blocks16_of(cam->height) + 64.0) * (n_images > 0 ? n_images : 1);
    if (tiles >= 2147483647.0) return fail(SVOX_ERR_BAD_SHAPE, "too many pixels for one launch");
    return SVOX_OK;
}

int check_rays(const SvoxRaysSpec* rays) {
    if (!rays) return fail(SVOX_ERR_NULL_POINTER, "rays spec is NULL");
    if (rays->n_rays < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative ray count");
    if (rays->n_rays >= (1ll << 36)) return fail(SVOX_ERR_BAD_SHAPE, "too many rays for one launch");
    if (rays->n_rays > 0 && (!rays->origins || !rays->dirs || !rays->vdirs))
        return fail(SVOX_ERR_NULL_POINTER, "rays.origins / dirs / vdirs is NULL");
    return SVOX_OK;
}

// default options on an fp32 octree whose record matches the format: the specialised kernels (with or without
// density_softplus, which they apply to the densities they fetch).  Returns what SVOX_DISPATCH_OCTREE
// switches on: 0 for RGBA, basis_dim for spherical harmonics, kLobeKernels + basis_dim for lobes (spherical
// gaussians and anisotropic ones), -1 for everything the generic kernels serve.
constexpr int kLobeKernels = 100;
int fast_basis(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    if (!march_fast_ok(tree)) return -1;
    if (opt->format == SVOX_FORMAT_RGBA) return tree->data_dim == 4 ? 0 : -1;
    if (opt->format != SVOX_FORMAT_SH && opt->format != SVOX_FORMAT_SG && opt->format != SVOX_FORMAT_ASG) return -1;
    const int D = opt->basis_dim;
    if (D != 1 && D != 4 && D != 9 && D != 16 && D != 25) return -1;
    if (tree->data_dim != 3 * D + 1 || opt->min_comp < 0 || opt->max_comp > D - 1) return -1;
    // A range of components narrower than the basis runs on the kernels that keep a ray's basis as a row in LDS (the
    // lobe policy: its rows come from precalc_basis, for spherical harmonics too), the row zero outside the range;
    // min_comp > max_comp is the reference's empty range, mid grey.
    const bool partial = opt->min_comp > 0 || opt->max_comp < D - 1;
    if (opt->format == SVOX_FORMAT_SH && partial) return kLobeKernels + D;
    if (opt->format != SVOX_FORMAT_SH) {
        // lobes: the table must be there, [lambda, mu] per spherical gaussian (rt_kernel.cu:133-139),
        // [lambda_x, lambda_y, three axes] per anisotropic one (rt_kernel.cu:120-131)
        const int need = opt->format == SVOX_FORMAT_SG ? 4 : 11;
        if (!tree->extra_data || tree->extra_rows < D || tree->extra_cols < need) return -1;
        return kLobeKernels + D;
    }
    return D;
}

Lobes lobes_of(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    return Lobes{(const float*)tree->extra_data, tree->extra_cols, opt->format};
}

// Whether a launch that works on every leaf with density > need_thresh (the forward pass: opt->sigma_thresh; the
// backward passes, se_grad and the noting passes: 0) may read the caller's marks in place of the child table: the
// marks hide the leaves whose density is not > child_marks_thresh, which must all be leaves the launch skips.
bool marks_apply(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, float need_thresh) {
    return tree->child_marks && tree->child_marks_thresh >= 0.0f && need_thresh >= tree->child_marks_thresh &&
           (tree->child_marks_softplus != 0) == (opt->density_softplus != 0);
}
// ... and whether the marks hide exactly the leaves the launch skips: every leaf they let through is shaded.
bool marks_decide(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, float need_thresh) {
    return marks_apply(tree, opt, need_thresh) && need_thresh == tree->child_marks_thresh;
}

// The tree as the octree march kernels see it: with the caller's marks in place of the child table where they apply.
TreeDev<float> march_tree(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, float need_thresh = 0.0f) {
    TreeDev<float> d = make_tree<float>(tree);
    if (marks_apply(tree, opt, need_thresh)) d.child = tree->child_marks;
    return d;
}

// the workspace argument of a forward launch that takes no notes
ReplaySpace no_notes() {
    ReplaySpace ws{};
    ws.spin_limit = (g_debug_flags & 16) ? 1 : 0;
    return ws;
}

// Items (rays) a persistent wavefront owns.  With few rays every wavefront gets one 64-item chunk so
// that the launch spreads over as many SIMDs as possible; with many, several chunks, which lets lanes
// whose rays end early pick up new ones (measured on 1M random rays: forward best at 256 rays per
// wavefront, backward -- two marches per ray, longer-lived lanes -- at 512).
int pick_per_wave(int64_t total_items, bool backward) {
    const int forced = tuning().per_wave;
    if (forced == 64 || forced == 128 || forced == 256 || forced == 512 || forced == 1024) return forced;
    if (total_items < (int64_t)64 * 1024 * 8 && !(g_debug_flags & 2)) return 64;
    return backward ? 512 : 256;
}

int pick_refill() {
    const int forced = tuning().refill;
    return forced >= 1 && forced <= 64 ? forced : 16;
}

// Image tiles handed to one XCD in a row (chunk_of_block): 16 tiles are four 16x16 pixel blocks.
// Measured on 8 poses of 800x800: 1 -> 16 shortens the launch by 2-3 %, larger runs gain no more and
// start to unbalance the XCDs.
int pick_xcd_group() {
    const int forced = tuning().xcd_group;
    return forced >= 1 && forced <= 4096 ? forced : 16;
}

template <typename T>
BatchSource<T> batch_source(const SvoxRaysSpec* rays, bool backward = false) {
    BatchSource<T> s;
    s.rays.origins = (const T*)rays->origins;
    s.rays.dirs = (const T*)rays->dirs;
    s.rays.vdirs = (const T*)rays->vdirs;
    s.rays.n_rays = rays->n_rays;
    s.per_wave = pick_per_wave(rays->n_rays, backward);
    s.refill_at = pick_refill();
    s.xcd_group = 1;
    s.n_waves = 0;
    return s;
}

// The persistent kernels deal the rays of a batch out over their wavefronts (BatchSource::n_waves).
template <typename T>
BatchSource<T> dealt_out(BatchSource<T> s, unsigned n_waves) {
    if (s.per_wave > kMarchThreads && (s.per_wave & (s.per_wave - 1)) == 0) s.n_waves = n_waves;
    return s;
}
template <typename T>
ImageSource<T> dealt_out(const ImageSource<T>& s, unsigned) { return s; }

// bytes after the chunks and the bitmap of a workspace: the stamp of the notes
constexpr int64_t kTailBytes = 256;

template <typename T>
ImageSource<T> image_source(const SvoxCameraSpec* cam, int n_images, int64_t pose_stride,
                            const SvoxRenderOptions* opt) {
    ImageSource<T> s;
    s.cam.c2w = (const T*)cam->c2w;
    s.cam.fx = cam->fx;
    s.cam.fy = cam->fy;
    s.cam.width = cam->width;
    s.cam.height = cam->height;
    s.n_images = n_images;
    s.pose_stride = pose_stride;
    // image tiles are coherent (rays of a tile end together) and only part of an image hits the
    // tree: one tile per wavefront keeps the busy tiles spread over the whole GPU
    s.per_wave = 64;
    s.refill_at = pick_refill();
    s.xcd_group = pick_xcd_group();
    s.run = 0;
    // Blocks from the middle of the image outwards, unless the camera is an NDC one: there every
    // ray crosses the whole tree, no part of the picture is longer than another, and rows of
    // blocks (slabs of the tree) share more leaves in L2 than rings do.  Measured (us, rows / rings):
    // one 800x800 pose of the sparse SH16 tree 317 / 304, 2 poses 344 / 314, 8 poses 695 / 670,
    // 16 poses 1159 / 1174; one pose of the dense 128^3 tree 385 / 340; 4 NDC poses 3538 / 3957.
    {
        const int forced = tuning().tile_order;
        s.inside_out = forced == 0 || forced == 1 ? forced : (opt->ndc_width > 0 ? 0 : 1);
    }
    if (n_images > 1) {
        const int forced = tuning().image_run;
        s.run = forced >= 0 ? forced : 4;
    }
    return s;
}

template <typename T>
int64_t total_items_of(const BatchSource<T>& s) { return s.rays.n_rays; }
template <typename T>
int64_t total_items_of(const ImageSource<T>& s) {
    const int64_t per_image = (int64_t)blocks16_of(s.cam.width) * blocks16_of(s.cam.height);
    const int64_t padded = s.run > 0 ? (per_image + s.run - 1) / s.run * s.run : per_image;
    return (int64_t)s.n_images * padded * 256;
}

unsigned blocks_for(int64_t items, int per_block) { return (unsigned)((items + per_block - 1) / per_block); }

#define SVOX_DISPATCH_OCTREE(D, ...)                                         \
    switch (D) {                                                             \
        case 0: { using P = OctreePolicy<SVOX_FORMAT_RGBA, 0>; __VA_ARGS__; } break; \
        case 1: { using P = OctreePolicy<SVOX_FORMAT_SH, 1>; __VA_ARGS__; } break;   \
        case 4: { using P = OctreePolicy<SVOX_FORMAT_SH, 4>; __VA_ARGS__; } break;   \
        case 9: { using P = OctreePolicy<SVOX_FORMAT_SH, 9>; __VA_ARGS__; } break;   \
        case 16: { using P = OctreePolicy<SVOX_FORMAT_SH, 16>; __VA_ARGS__; } break; \
        case 25: { using P = OctreePolicy<SVOX_FORMAT_SH, 25>; __VA_ARGS__; } break; \
        case kLobeKernels + 1: { using P = OctreePolicy<SVOX_FORMAT_SG, 1>; __VA_ARGS__; } break;   \
        case kLobeKernels + 4: { using P = OctreePolicy<SVOX_FORMAT_SG, 4>; __VA_ARGS__; } break;   \
        case kLobeKernels + 9: { using P = OctreePolicy<SVOX_FORMAT_SG, 9>; __VA_ARGS__; } break;   \
        case kLobeKernels + 16: { using P = OctreePolicy<SVOX_FORMAT_SG, 16>; __VA_ARGS__; } break; \
        default: { using P = OctreePolicy<SVOX_FORMAT_SG, 25>; __VA_ARGS__; } break; \
    }

// Whether a forward launch of `blocks` 64-ray wavefronts takes render_forward_split_kernel (two wavefronts per 64
// rays: one walks, one shades).  It shortens the chain of a tile's longest ray, which is what a launch that does not
// fill the GPU with heavy tiles waits for; where every tile is heavy and the GPU full, the second wavefront only
// takes a place another tile could have.  Measured on 800x800 poses of the sparse 512^3 SH16 tree (ms, one / two
// wavefronts per tile), orbit of radius 4 (18 % of the rays hit the tree): 1 pose 0.41 / 0.34, 2 poses 0.45 / 0.37,
// 4 poses 0.62 / 0.56, 8 poses 0.90 / 0.85, 16 poses 1.55 / 1.60; radius 2.5 (49 % hit): 0.43 / 0.38, 0.57 / 0.54,
// 0.97 / 0.95, 1.61 / 1.64, 2.91 / 3.14; radius 1.5 (every ray hits): 0.54 / 0.52, 0.88 / 0.90, 1.71 / 1.82,
// 3.14 / 3.40, 5.92 / 6.49.  With marks that decide the shading (`decided`: the one-wavefront kernel then reads a
// leaf's density with its coefficients, the two-wavefront kernel gains nothing from them) the balance tips earlier,
// launches alone: radius 4, 4 poses 0.48 / 0.47, 8 poses 0.69 / 0.72, 16 poses 1.13 / 1.30; radius 2.5, 8 poses
// 1.22 / 1.33.  The launcher cannot know how many rays hit, so the rule goes by tiles: images of up to 65 536 tiles
// (six 800x800 poses) -- 49 152 with deciding marks, 16 384 under NDC, where every ray passes through the tree --,
// ray batches of up to 128 Ki rays (dense 128^3 tree: 1 pose 0.54 / 0.37, 4 poses 0.84 / 0.75; 4 NDC poses of 47 628
// tiles 3.54 / 3.67; 256 Ki unrelated rays 0.29 / 0.39).
bool use_split_forward(unsigned blocks, bool image, const SvoxRenderOptions* opt, bool decided) {
    const int forced = tuning().split_forward;
    const long limit = tuning().split_blocks;
    if (g_debug_flags & 12) return (g_debug_flags & 8) != 0;
    if (forced >= 0) return forced > 0;
    if (limit >= 0) return (long)blocks <= limit;
    if (!image) return blocks <= 2048u;
    if (opt->ndc_width > 0) return blocks <= 16384u;
    return blocks <= (decided ? 49152u : 65536u);
}
template <typename T>
constexpr bool is_image_source(const ImageSource<T>&) { return true; }
template <typename T>
constexpr bool is_image_source(const BatchSource<T>&) { return false; }

template <class Source, typename T>
void launch_forward(const SvoxTreeSpec* tree, const Source& src, const SvoxRenderOptions* opt, int out_dim,
                    void* out, hipStream_t stream) {
    const int64_t items = total_items_of(src);
    if constexpr (sizeof(T) == 4) {
        const int D = fast_basis(tree, opt);
        if (D >= 0) {
            const unsigned blocks = blocks_for(items, src.per_wave);
            const Source dealt = dealt_out(src, blocks);
            const TreeDev<float> tr = march_tree(tree, opt, opt->sigma_thresh);
            const ReplaySpace none = no_notes();
            // Marks made with this launch's own threshold: every leaf they let through is shaded, and the kernel with
            // one wavefront per tile or chunk then reads a leaf's density with its coefficients (one round trip per
            // round instead of two that wait for one another: 4 NDC poses 3.10 -> 2.93 ms).  The two-wavefront kernel
            // keeps its density phase: there the walk is the critical path, the density read of a leaf brings the
            // last line of its record into L2 ahead of the coefficient reads, and without it the kernel needs more
            // registers (5 instead of 6 wavefronts per SIMD): measured 0.70 -> 0.73 ms on 8 poses of 800x800,
            // although the launch sends 17 % fewer requests to L2.
            const bool all_shaded = !tree->weight_accum && marks_decide(tree, opt, opt->sigma_thresh);
#define SVOX_LAUNCH_FORWARD(ACCUM, REFILL, ALL)                                                                   \
    SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((render_forward_kernel<P, Source, ACCUM, REFILL, false, false, ALL>), \
                                               dim3(blocks), dim3(kMarchThreads), 0, stream, tr, dealt, *opt,      \
                                               (float*)out, none))
            const bool refill = src.per_wave > kMarchThreads;
            if (!refill && !tree->weight_accum && use_split_forward(blocks, is_image_source(src), opt, all_shaded)) {
                SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((render_forward_split_kernel<P, Source, false>),
                                                           dim3(blocks), dim3(kSplitThreads), 0, stream, tr, dealt,
                                                           *opt, (float*)out, none));
                return;
            }
            if (tree->weight_accum) {
                // accumulation is an analysis pass: one variant is enough
                SVOX_LAUNCH_FORWARD(true, true, false);
            } else if (refill) {
                if (all_shaded) { SVOX_LAUNCH_FORWARD(false, true, true); } else { SVOX_LAUNCH_FORWARD(false, true, false); }
            } else {
                if (all_shaded) { SVOX_LAUNCH_FORWARD(false, false, true); } else { SVOX_LAUNCH_FORWARD(false, false, false); }
            }
#undef SVOX_LAUNCH_FORWARD
            return;
        }
    }
    const int basis_rows = opt->format == SVOX_FORMAT_RGBA ? 1 : opt->basis_dim;
    hipLaunchKernelGGL((render_forward_generic_kernel<T, Source>), dim3(blocks_for(items, kMarchThreads)),
                       dim3(kMarchThreads), generic_forward_lds_bytes<T>(basis_rows, out_dim), stream,
                       make_tree<T>(tree), src, *opt, out_dim, (T*)out);
}

constexpr int64_t kChunkBytes = (int64_t)kChunkFloat2 * 8;   // 384: 15 records and a link

// What the notes in a workspace belong to (ReplaySpace::stamp).
struct NoteStamp {
    unsigned long long word[kStampWords];
};
NoteStamp stamp_of(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt) {
    NoteStamp st;
    uint32_t step_bits, thresh_bits;
    memcpy(&step_bits, &opt->step_size, 4);
    memcpy(&thresh_bits, &opt->sigma_thresh, 4);
    st.word[0] = 0x73766f786e6f7465ull ^ (unsigned long long)rays->n_rays ^ (opt->density_softplus ? 1ull << 62 : 0ull);
    st.word[1] = (unsigned long long)(uintptr_t)tree->data;
    st.word[2] = (unsigned long long)(uintptr_t)rays->origins;
    st.word[3] = ((unsigned long long)thresh_bits << 32) | step_bits;
    st.word[4] = (unsigned long long)(uintptr_t)tree->child;
    st.word[5] = (unsigned long long)(uintptr_t)rays->dirs;
    return st;
}

// The workspace of the replaying kernels: chunks of notes, then one bit per ray (rays left undone by
// replay_backward_kernel), then 256 bytes that hold the stamp of the notes and, from byte 128 on, the
// counter of the chunk stocks (cleared before every launch that takes notes).
constexpr int64_t kStampOffset = 0;
constexpr int64_t kStockCounterOffset = 128;
int64_t bitmap_bytes(int64_t n_slots) { return ((n_slots + 63) / 64 * 8 + 15) / 16 * 16; }
bool carve_workspace(void* workspace, int64_t workspace_bytes, int64_t n_slots, ReplaySpace* ws) {
    *ws = ReplaySpace{nullptr, 0, 0, nullptr, nullptr, {0, 0, 0, 0, 0, 0}, nullptr, nullptr};
    const int64_t chunks = workspace && n_slots > 0
                               ? (workspace_bytes - kTailBytes - bitmap_bytes(n_slots)) / kChunkBytes : 0;
    if (n_slots <= 0 || chunks < n_slots || chunks >= 0x7fffffffll || ((uintptr_t)workspace & 15u) != 0) return false;
    ws->base = (float2*)workspace;
    ws->first_shared = n_slots;
    ws->n_chunks = chunks;
    ws->undone = (unsigned long long*)((char*)workspace + chunks * kChunkBytes);
    ws->stamp_at = (unsigned long long*)((char*)ws->undone + bitmap_bytes(n_slots) + kStampOffset);
    ws->stocks_taken = (unsigned long long*)((char*)ws->undone + bitmap_bytes(n_slots) + kStockCounterOffset);
    return true;
}

// The backward pass by two marches per ray (no workspace, or one that cannot serve: see backward_by_noting).
template <class Source, typename T>
void launch_backward(const SvoxTreeSpec* tree, const Source& src, const SvoxRenderOptions* opt, int out_dim,
                     const void* grad_out, void* grad_data, hipStream_t stream) {
    const int64_t items = total_items_of(src);
    if constexpr (sizeof(T) == 4) {
        const int D = fast_basis(tree, opt);
        if (D >= 0) {
            const unsigned blocks = blocks_for(items, src.per_wave);
            const Source dealt = dealt_out(src, blocks);
            const ReplaySpace none{};
            if (src.per_wave > kMarchThreads) {
                SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((render_backward_kernel<P, Source, true, kBackwardPlain>),
                                                           dim3(blocks), dim3(kMarchThreads), 0, stream,
                                                           march_tree(tree, opt), dealt, *opt, (const float*)grad_out,
                                                           (float*)grad_data, none));
            } else {
                SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((render_backward_kernel<P, Source, false, kBackwardPlain>),
                                                           dim3(blocks), dim3(kMarchThreads), 0, stream,
                                                           march_tree(tree, opt), dealt, *opt, (const float*)grad_out,
                                                           (float*)grad_data, none));
            }
            return;
        }
    }
    const int basis_rows = opt->format == SVOX_FORMAT_RGBA ? 1 : opt->basis_dim;
    hipLaunchKernelGGL((render_backward_generic_kernel<T, Source>), dim3(blocks_for(items, kMarchThreads)),
                       dim3(kMarchThreads), generic_backward_lds_bytes<T>(basis_rows, out_dim), stream,
                       make_tree<T>(tree), src, *opt, out_dim, (const T*)grad_out, (T*)grad_data);
}

// The launch shape of the noting forward pass for the rays of `s`: that of a forward pass (a batch
// source made for a backward pass gives its wavefronts more rays than the forward kernels like).
template <typename T>
BatchSource<T> noting_shape(BatchSource<T> s) {
    s.per_wave = pick_per_wave(s.rays.n_rays, false);
    return s;
}
template <typename T>
ImageSource<T> noting_shape(const ImageSource<T>& s) { return s; }

// The forward pass of a training step: the picture into `out` and, in the workspace, the notes of
// every ray under `stamp`.  Needs a usable workspace and the octree kernels, which noted_ok() tells
// beforehand.  A launch that does not fill the GPU runs on two wavefronts per 64 rays.  out may be
// nullptr (notes only); grad_out, if given, is the gradient of the picture the backward pass will be
// called with: the notes' heads then also carry the sum of that pass's first march.
template <class Source>
int launch_noted(const SvoxTreeSpec* tree, const Source& src, const SvoxRenderOptions* opt, void* out,
                 void* workspace, int64_t workspace_bytes, int64_t n_slots, const NoteStamp& stamp,
                 hipStream_t stream, const void* grad_out = nullptr) {
    const int D = fast_basis(tree, opt);
    const unsigned blocks = blocks_for(total_items_of(src), src.per_wave);
    const Source dealt = dealt_out(src, blocks);
    ReplaySpace ws;
    if (D < 0 || !carve_workspace(workspace, workspace_bytes, n_slots, &ws))
        return fail(SVOX_ERR_BAD_SHAPE, "notes asked for where they cannot be taken");
    const int rc = zero_fill(ws.stocks_taken, 16, stream);
    if (rc) return rc;
    memcpy(ws.stamp, stamp.word, sizeof(ws.stamp));
    ws.spin_limit = (g_debug_flags & 16) ? 1 : 0;
    const bool refill = src.per_wave > kMarchThreads;
    const bool split = !refill && use_split_forward(blocks, is_image_source(src), opt, false);
    const dim3 threads(split ? kSplitThreads : kMarchThreads);
#define SVOX_LAUNCH_NOTING(KERNEL)                                                                                   \
    SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL(KERNEL, dim3(blocks), threads, 0, stream, march_tree(tree, opt), dealt, \
                                               *opt, (float*)out, ws, (const float*)grad_out))
    if (grad_out) {
        if (split) {
            SVOX_LAUNCH_NOTING((render_forward_split_kernel<P, Source, true, true>));
        } else if (refill) {
            SVOX_LAUNCH_NOTING((render_forward_kernel<P, Source, false, true, true, true>));
        } else {
            SVOX_LAUNCH_NOTING((render_forward_kernel<P, Source, false, false, true, true>));
        }
    } else {
        if (split) {
            SVOX_LAUNCH_NOTING((render_forward_split_kernel<P, Source, true, false>));
        } else if (refill) {
            SVOX_LAUNCH_NOTING((render_forward_kernel<P, Source, false, true, true, false>));
        } else {
            SVOX_LAUNCH_NOTING((render_forward_kernel<P, Source, false, false, true, false>));
        }
    }
#undef SVOX_LAUNCH_NOTING
    return SVOX_OK;
}

// The device address of `scratch` on the current device, looked up once per device (every GPU holds
// its own copy of the array at its own address).
constexpr int kStaticDevicesMax = 64;
int static_workspace(void** out) {
    static std::mutex guard;
    static void* address[kStaticDevicesMax] = {nullptr};
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess || device < 0 || device >= kStaticDevicesMax)
        return fail(SVOX_ERR_NO_DEVICE, "svox.volume_render_backward_static: no usable current device (%s)",
                    err != hipSuccess ? hipGetErrorString(err) : "device index out of range");
    std::lock_guard<std::mutex> lock(guard);
    if (!address[device]) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !ptr)
            return fail(SVOX_ERR_LAUNCH, "svox.volume_render_backward_static: hipGetSymbolAddress failed (%s)",
                        hipGetErrorString(err));
        address[device] = ptr;
    }
    *out = address[device];
    return SVOX_OK;
}

int64_t data_bytes(const SvoxTreeSpec* t) {
    const int64_t esz = t->dtype == SVOX_F32 ? 4 : 8;
    return t->capacity * t->N * t->N * t->N * t->data_dim * esz;
}

// `only`: a bitmap of the rays to do (octree kernels only; the batch rays are then not dealt out)
template <class Source, typename T>
void launch_se_grad(const SvoxTreeSpec* tree, const Source& src, const SvoxRenderOptions* opt, int out_dim,
                    const void* color_ref, void* color_out, void* grad, void* hess, hipStream_t stream,
                    const unsigned long long* only = nullptr) {
    const int64_t items = total_items_of(src);
    if constexpr (sizeof(T) == 4) {
        const int D = fast_basis(tree, opt);
        if (D >= 0) {
            const unsigned blocks = blocks_for(items, src.per_wave);
            const Source dealt = only ? src : dealt_out(src, blocks);
            if (src.per_wave > kMarchThreads) {
                SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((se_grad_kernel<P, Source, true>), dim3(blocks),
                                                           dim3(kMarchThreads), 0, stream, march_tree(tree, opt),
                                                           dealt, *opt, (const float*)color_ref, (float*)color_out,
                                                           (float*)grad, (float*)hess, only));
            } else {
                SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((se_grad_kernel<P, Source, false>), dim3(blocks),
                                                           dim3(kMarchThreads), 0, stream, march_tree(tree, opt),
                                                           src, *opt, (const float*)color_ref, (float*)color_out,
                                                           (float*)grad, (float*)hess, only));
            }
            return;
        }
    }
    const int basis_rows = opt->format == SVOX_FORMAT_RGBA ? 1 : opt->basis_dim;
    hipLaunchKernelGGL((se_grad_generic_kernel<T, Source>), dim3(blocks_for(items, kMarchThreads)),
                       dim3(kMarchThreads), generic_backward_lds_bytes<T>(basis_rows, out_dim), stream,
                       make_tree<T>(tree), src, *opt, out_dim, (const T*)color_ref, (T*)color_out, (T*)grad, (T*)hess);
}

// shared argument checks and zero-fills of the two squared-error entry points
int se_grad_prepare(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, void* grad, void* hess, int* od,
                    hipStream_t stream) {
    int rc = check_render(tree, opt, od);
    if (rc) return rc;
    if (*od > 4) return fail(SVOX_ERR_BAD_SHAPE, "Tree's output dim cannot be > 4 for se_grad");
    if (!grad || !hess) return fail(SVOX_ERR_NULL_POINTER, "grad_out / hessdiag_out is NULL");
    rc = zero_fill(grad, data_bytes(tree), stream);
    if (rc) return rc;
    return zero_fill(hess, data_bytes(tree), stream);
}

// Can notes be taken (launch_noted) and used (replay_backward_kernel)?  The octree kernels, a forward
// pass whose threshold does not admit leaves the backward pass ignores, no weight accumulator, and a
// workspace with a chunk for every ray.
bool notes_possible(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    return tree->dtype == SVOX_F32 && fast_basis(tree, opt) >= 0 && !tree->weight_accum && opt->sigma_thresh >= 0.0f;
}
bool noted_ok(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt, int64_t n_slots, void* workspace,
                     int64_t workspace_bytes) {
    if (!notes_possible(tree, opt)) return false;
    ReplaySpace ws;
    return carve_workspace(workspace, workspace_bytes, n_slots, &ws);
}

NoteStamp stamp_of_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                                const SvoxRenderOptions* opt) {
    SvoxRaysSpec as_rays;
    as_rays.origins = cam->c2w;
    as_rays.dirs = nullptr;
    as_rays.n_rays = ((int64_t)n_images * cam->height * cam->width) ^ ((int64_t)cam->width << 40);
    return stamp_of(tree, &as_rays, opt);
}

// log2 of the rays a wavefront of the replay kernels takes: 16 rays for the pixels of images (neighbours,
// long together) and for batches that do not fill the GPU with 64 (up to 64 Ki rays: 4 096 rays of a 16^3
// tree 246 -> 196 us, 64 Ki rays 350 -> 333 us), 64 for larger ray batches (1 Mi rays: 0.68 against 0.83 ms
// with 16).
int replay_ray_shift(bool image, int64_t n_rays) {
    const int forced_shift = tuning().replay_shift;
    return forced_shift == 4 || forced_shift == 6 ? forced_shift : (image || n_rays <= 65536 ? 4 : 6);
}

// The backward pass of `all` from the notes in the workspace: the rays with complete notes by
// replay_backward_kernel, the others, which it marks in the bitmap, by marching (`rest`: the launch
// shape for those): twice, or -- march1_known: the noting pass had grad_output and left the sum of
// the first march in the heads of the notes -- once.
template <class Source>
int backward_from_notes(const SvoxTreeSpec* tree, const Source& all, Source rest, const SvoxRenderOptions* opt,
                               const void* grad_output, void* grad_data_out, void* workspace, int64_t workspace_bytes,
                               int64_t n_slots, const NoteStamp& stamp, hipStream_t stream, bool march1_known = false) {
    const int D = fast_basis(tree, opt);
    const int ray_shift = replay_ray_shift(is_image_source(all), n_slots);
    const unsigned waves = blocks_for(n_slots, 1 << ray_shift);
    ReplaySpace ws;
    carve_workspace(workspace, workspace_bytes, n_slots, &ws);
    memcpy(ws.stamp, stamp.word, sizeof(ws.stamp));
    SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((replay_backward_kernel<P, Source>), dim3(waves), dim3(kMarchThreads), 0,
                                               stream, all, *opt, (const float*)grad_output, (float*)grad_data_out, ws,
                                               ray_shift, march1_known ? 1 : 0, lobes_of(tree, opt)));
    int rc = check_launch("volume_render_backward_noted");
    if (rc) return rc;
    ReplaySpace only{};
    only.base = ws.base;
    only.only = ws.undone;
    const unsigned blocks = blocks_for(total_items_of(rest), rest.per_wave);
#define SVOX_LAUNCH_REST(REFILL, MODE)                                                                              \
    SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((render_backward_kernel<P, Source, REFILL, MODE>), dim3(blocks),      \
                                               dim3(kMarchThreads), 0, stream, march_tree(tree, opt), rest, *opt,    \
                                               (const float*)grad_output, (float*)grad_data_out, only))
    if (rest.per_wave > kMarchThreads) {
        if (march1_known) { SVOX_LAUNCH_REST(true, kBackwardSecond); } else { SVOX_LAUNCH_REST(true, kBackwardPlain); }
    } else {
        if (march1_known) { SVOX_LAUNCH_REST(false, kBackwardSecond); } else { SVOX_LAUNCH_REST(false, kBackwardPlain); }
    }
#undef SVOX_LAUNCH_REST
    return check_launch("volume_render_backward_noted");
}

// the options under which notes are taken where no picture hangs on them (se_grad, the backward pass alone): every leaf with sigma > 0, no early stop
SvoxRenderOptions without_thresholds(const SvoxRenderOptions* opt) {
    SvoxRenderOptions o = *opt;
    o.sigma_thresh = 0.0f;
    o.stop_thresh = 0.0f;
    return o;
}

// The backward pass of a call that brings a workspace but no notes: one noting march without a picture
// (thresholds play no part in the backward pass, rt_kernel.cu:377, 441), then backward_from_notes.  The
// reference's two marches per ray become one walk of the tree and one pass over 24 bytes per leaf with
// density.  `all`, `rest` as in backward_from_notes; returns 1 if notes cannot be taken here (the
// caller then marches twice), else a status.
template <class Source>
int backward_by_noting(const SvoxTreeSpec* tree, const Source& all, const Source& rest, const SvoxRenderOptions* opt,
                       const void* grad_output, void* grad_data_out, void* workspace, int64_t workspace_bytes,
                       int64_t n_slots, NoteStamp stamp, hipStream_t stream) {
    SvoxTreeSpec quiet = *tree;
    quiet.weight_accum = nullptr;   // (the backward pass accumulates no weights)
    const SvoxRenderOptions plain = without_thresholds(opt);
    if (!noted_ok(&quiet, &plain, n_slots, workspace, workspace_bytes)) return 1;
    // (the notes belong to this call alone: the stamp carries its gradient buffer too)
    stamp.word[0] ^= (unsigned long long)(uintptr_t)grad_output;
    int rc = launch_noted(&quiet, noting_shape(all), &plain, nullptr, workspace, workspace_bytes, n_slots, stamp, stream,
                          grad_output);
    if (rc) return rc;
    rc = check_launch("volume_render_backward");
    if (rc) return rc;
    return backward_from_notes(&quiet, all, rest, &plain, grad_output, grad_data_out, workspace, workspace_bytes,
                               n_slots, stamp, stream, true);
}

// se_grad of the rays of `all` with their notes kept in the workspace between its two halves: one
// march that takes the notes (thresholds play no part in se_grad, rt_kernel.cu:479-715), then
// replay_se_grad_kernel; rays it marks in the bitmap are done by se_grad_kernel (`rest`: the launch
// shape for those).  The caller has checked noted_ok() with the same options.
template <class Source>
int se_grad_from_notes(const SvoxTreeSpec* tree, const Source& all, const Source& rest, const SvoxRenderOptions* opt,
                       const void* color_ref, void* color_out, void* grad, void* hess, void* workspace,
                       int64_t workspace_bytes, int64_t n_slots, const NoteStamp& stamp, hipStream_t stream) {
    const int D = fast_basis(tree, opt);
    int rc = launch_noted(tree, noting_shape(all), opt, color_out, workspace, workspace_bytes, n_slots, stamp, stream);
    if (rc) return rc;
    rc = check_launch("se_grad");
    if (rc) return rc;
    ReplaySpace ws;
    carve_workspace(workspace, workspace_bytes, n_slots, &ws);
    memcpy(ws.stamp, stamp.word, sizeof(ws.stamp));
    const int ray_shift = replay_ray_shift(is_image_source(all), n_slots);
    SVOX_DISPATCH_OCTREE(D, hipLaunchKernelGGL((replay_se_grad_kernel<P, Source>), dim3(blocks_for(n_slots, 1 << ray_shift)),
                                               dim3(kMarchThreads), 0, stream, all, *opt, (const float*)color_ref,
                                               (float*)color_out, (float*)grad, (float*)hess, ws, ray_shift,
                                               lobes_of(tree, opt)));
    rc = check_launch("se_grad");
    if (rc) return rc;
    launch_se_grad<Source, float>(tree, rest, opt, 3, color_ref, color_out, grad, hess, stream, ws.undone);
    return check_launch("se_grad");
}


}  // namespace

#pragma GCC visibility push(default)
extern "C" {

int svox_abi_version(void) { return SVOX_ABI_VERSION; }

const char* svox_last_error(void) { return g_error; }

const char* svox_status_string(int status) {
    switch (status) {
        case SVOX_OK: return "ok";
        case SVOX_ERR_NULL_POINTER: return "null pointer";
        case SVOX_ERR_BAD_SHAPE: return "bad shape";
        case SVOX_ERR_BAD_DTYPE: return "bad dtype";
        case SVOX_ERR_UNSUPPORTED: return "unsupported";
        case SVOX_ERR_LAUNCH: return "kernel launch failed";
        case SVOX_ERR_NO_DEVICE: return "no device";
        default: return "unknown status";
    }
}

// Debugging aid: bit 0 routes every call to the generic kernels.
void svox_set_debug_flags(int flags) { g_debug_flags = flags; }

int svox_out_data_dim(int32_t format, int32_t basis_dim, int32_t data_dim) {
    if (data_dim < 1) return -1;
    if (format != SVOX_FORMAT_RGBA) {
        if (basis_dim <= 0) return -1;
        return (data_dim - 1) / basis_dim;
    }
    return data_dim - 1;
}

int svox_query_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points, void* values_out,
                        int64_t* node_ids_out, void* stream) {
    int rc = check_tree(tree, true);
    if (rc) return rc;
    if (n_points < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative point count");
    if (n_points == 0) return SVOX_OK;
    if (!indices || !values_out || !node_ids_out) return fail(SVOX_ERR_NULL_POINTER, "indices / values_out / node_ids_out is NULL");
    if (tree->dtype == SVOX_F32)
        return launch_query<float, kQueryGather>(tree, indices, n_points, values_out, nullptr, node_ids_out,
                                                 tree->data_dim, (hipStream_t)stream, "query_vertical");
    return launch_query<double, kQueryGather>(tree, indices, n_points, values_out, nullptr, node_ids_out,
                                              tree->data_dim, (hipStream_t)stream, "query_vertical");
}

int svox_query_vertical_backward(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                                 const void* grad_output, int32_t grad_dim, void* grad_data_out,
                                 int32_t accumulate, void* stream) {
    int rc = check_tree(tree, false);
    if (rc) return rc;
    if (n_points < 0 || grad_dim < 1) return fail(SVOX_ERR_BAD_SHAPE, "negative point count or grad_dim < 1");
    if (!grad_data_out) return fail(SVOX_ERR_NULL_POINTER, "grad_data_out is NULL");
    const int64_t esz = tree->dtype == SVOX_F32 ? 4 : 8;
    if (!accumulate) {
        rc = zero_fill(grad_data_out, tree->capacity * tree->N * tree->N * tree->N * grad_dim * esz,
                       (hipStream_t)stream);
        if (rc) return rc;
    }
    if (n_points == 0) return SVOX_OK;
    if (!indices || !grad_output) return fail(SVOX_ERR_NULL_POINTER, "indices / grad_output is NULL");
    if (tree->dtype == SVOX_F32)
        return launch_query<float, kQueryScatterAdd>(tree, indices, n_points, (void*)grad_output, grad_data_out,
                                                     nullptr, grad_dim, (hipStream_t)stream,
                                                     "query_vertical_backward");
    return launch_query<double, kQueryScatterAdd>(tree, indices, n_points, (void*)grad_output, grad_data_out,
                                                  nullptr, grad_dim, (hipStream_t)stream,
                                                  "query_vertical_backward");
}

int svox_assign_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points, const void* values,
                         int32_t value_dim, void* stream) {
    int rc = check_tree(tree, true);
    if (rc) return rc;
    if (n_points < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative point count");
    if (value_dim < 1 || value_dim > tree->data_dim)
        return fail(SVOX_ERR_BAD_SHAPE, "value_dim %d outside [1, data_dim=%d]", value_dim, tree->data_dim);
    if (n_points == 0) return SVOX_OK;
    if (!indices || !values) return fail(SVOX_ERR_NULL_POINTER, "indices / values is NULL");
    if (tree->dtype == SVOX_F32)
        return launch_query<float, kQueryAssign>(tree, indices, n_points, (void*)values, nullptr, nullptr,
                                                 value_dim, (hipStream_t)stream, "assign_vertical");
    return launch_query<double, kQueryAssign>(tree, indices, n_points, (void*)values, nullptr, nullptr, value_dim,
                                              (hipStream_t)stream, "assign_vertical");
}

int svox_calc_corners(const SvoxTreeSpec* tree, const int64_t* indexer, int64_t n_leaves, void* corners_out,
                      void* stream) {
    int rc = check_tree(tree, false);
    if (rc) return rc;
    if (n_leaves < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative leaf count");
    if (n_leaves == 0) return SVOX_OK;
    if (!indexer || !corners_out) return fail(SVOX_ERR_NULL_POINTER, "indexer / corners_out is NULL");
    const unsigned blocks = (unsigned)((n_leaves + kQueryThreads - 1) / kQueryThreads);
    if (tree->dtype == SVOX_F32)
        hipLaunchKernelGGL((corners_kernel<float>), dim3(blocks), dim3(kQueryThreads), 0, (hipStream_t)stream,
                           tree->parent_depth, tree->N, tree->capacity, indexer, n_leaves, (float*)corners_out);
    else
        hipLaunchKernelGGL((corners_kernel<double>), dim3(blocks), dim3(kQueryThreads), 0, (hipStream_t)stream,
                           tree->parent_depth, tree->N, tree->capacity, indexer, n_leaves, (double*)corners_out);
    return check_launch("calc_corners");
}

// The forward pass of a training step: the picture of svox_volume_render, and in the workspace the notes
// svox_volume_render_backward_noted works from (where noted_ok() allows; else the plain forward pass).
int svox_volume_render_noted(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                             void* out, void* workspace, int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_rays(rays);
    if (rc) return rc;
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    if (rays->n_rays == 0) return SVOX_OK;
    if (!out) return fail(SVOX_ERR_NULL_POINTER, "out is NULL");
    if (!noted_ok(tree, opt, rays->n_rays, workspace, workspace_bytes))
        return svox_volume_render(tree, rays, opt, out, stream);
    const NoteStamp stamp = stamp_of(tree, rays, opt);
    rc = launch_noted(tree, batch_source<float>(rays, false), opt, out, workspace, workspace_bytes, rays->n_rays, stamp,
                      (hipStream_t)stream);
    if (rc) return rc;
    return check_launch("volume_render_noted");
}

int svox_volume_render_backward_noted(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                      const SvoxRenderOptions* opt, const void* grad_output, void* grad_data_out,
                                      int32_t accumulate, void* workspace, int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_rays(rays);
    if (rc) return rc;
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    if (!noted_ok(tree, opt, rays->n_rays, workspace, workspace_bytes))
        return svox_volume_render_backward_ws(tree, rays, opt, grad_output, grad_data_out, accumulate, workspace,
                                              workspace_bytes, stream);
    if (!grad_data_out) return fail(SVOX_ERR_NULL_POINTER, "grad_data_out is NULL");
    if (!accumulate) {
        rc = zero_fill(grad_data_out, data_bytes(tree), (hipStream_t)stream);
        if (rc) return rc;
    }
    if (rays->n_rays == 0) return SVOX_OK;
    if (!grad_output) return fail(SVOX_ERR_NULL_POINTER, "grad_output is NULL");
    const BatchSource<float> all = batch_source<float>(rays, true);
    return backward_from_notes(tree, all, all, opt, grad_output, grad_data_out, workspace, workspace_bytes,
                               rays->n_rays, stamp_of(tree, rays, opt), (hipStream_t)stream);
}

int svox_volume_render_images_noted(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                                    int64_t pose_stride, const SvoxRenderOptions* opt, void* out, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_camera(cam, n_images, pose_stride);
    if (rc) return rc;
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    if (cam->width == 0 || cam->height == 0 || n_images == 0) return SVOX_OK;
    if (!out) return fail(SVOX_ERR_NULL_POINTER, "out is NULL");
    const int64_t n_slots = (int64_t)n_images * cam->width * cam->height;
    if (!noted_ok(tree, opt, n_slots, workspace, workspace_bytes))
        return svox_volume_render_images(tree, cam, n_images, pose_stride, opt, out, stream);
    const NoteStamp stamp = stamp_of_image(tree, cam, n_images, opt);
    rc = launch_noted(tree, image_source<float>(cam, n_images, pose_stride, opt), opt, out, workspace, workspace_bytes,
                      n_slots, stamp, (hipStream_t)stream);
    if (rc) return rc;
    return check_launch("volume_render_images_noted");
}

int svox_volume_render_images_backward_noted(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                                             int64_t pose_stride, const SvoxRenderOptions* opt,
                                             const void* grad_output, void* grad_data_out, int32_t accumulate,
                                             void* workspace, int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_camera(cam, n_images, pose_stride);
    if (rc) return rc;
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    const int64_t n_slots = (int64_t)n_images * cam->width * cam->height;
    if (!noted_ok(tree, opt, n_slots, workspace, workspace_bytes))
        return svox_volume_render_images_backward_ws(tree, cam, n_images, pose_stride, opt, grad_output, grad_data_out,
                                                     accumulate, workspace, workspace_bytes, stream);
    if (!grad_data_out) return fail(SVOX_ERR_NULL_POINTER, "grad_data_out is NULL");
    if (!accumulate) {
        rc = zero_fill(grad_data_out, data_bytes(tree), (hipStream_t)stream);
        if (rc) return rc;
    }
    if (n_slots == 0) return SVOX_OK;
    if (!grad_output) return fail(SVOX_ERR_NULL_POINTER, "grad_output is NULL");
    const ImageSource<float> all = image_source<float>(cam, n_images, pose_stride, opt);
    return backward_from_notes(tree, all, all, opt, grad_output, grad_data_out, workspace, workspace_bytes, n_slots,
                               stamp_of_image(tree, cam, n_images, opt), (hipStream_t)stream);
}

int svox_volume_render(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt, void* out,
                       void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_rays(rays);
    if (rc) return rc;
    if (rays->n_rays == 0) return SVOX_OK;
    if (!out) return fail(SVOX_ERR_NULL_POINTER, "out is NULL");
    if (tree->dtype == SVOX_F32)
        launch_forward<BatchSource<float>, float>(tree, batch_source<float>(rays), opt, od, out,
                                                  (hipStream_t)stream);
    else
        launch_forward<BatchSource<double>, double>(tree, batch_source<double>(rays), opt, od, out,
                                                    (hipStream_t)stream);
    return check_launch("volume_render");
}

int svox_volume_render_images(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                              int64_t pose_stride, const SvoxRenderOptions* opt, void* out, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_camera(cam, n_images, pose_stride);
    if (rc) return rc;
    if (cam->width == 0 || cam->height == 0 || n_images == 0) return SVOX_OK;
    if (!out) return fail(SVOX_ERR_NULL_POINTER, "out is NULL");
    if (tree->dtype == SVOX_F32) {
        const auto src = image_source<float>(cam, n_images, pose_stride, opt);
        launch_forward<ImageSource<float>, float>(tree, src, opt, od, out, (hipStream_t)stream);
    } else {
        const auto src = image_source<double>(cam, n_images, pose_stride, opt);
        launch_forward<ImageSource<double>, double>(tree, src, opt, od, out, (hipStream_t)stream);
    }
    return check_launch("volume_render_image");
}

int svox_volume_render_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                             void* out, void* stream) {
    return svox_volume_render_images(tree, cam, 1, 12, opt, out, stream);
}

int svox_volume_render_backward(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                                const void* grad_output, void* grad_data_out, int32_t accumulate, void* stream) {
    return svox_volume_render_backward_ws(tree, rays, opt, grad_output, grad_data_out, accumulate, nullptr, 0,
                                          stream);
}

int svox_notes_pool_info(int64_t n_rays, int64_t workspace_bytes, int64_t* counter_offset, int64_t* pool_stocks) {
    if (!counter_offset || !pool_stocks) return fail(SVOX_ERR_NULL_POINTER, "svox_notes_pool_info: NULL output");
    ReplaySpace ws;
    // (any 16-byte aligned address does for the arithmetic)
    char* const base = (char*)(uintptr_t)4096;
    if (!carve_workspace(base, workspace_bytes, n_rays, &ws))
        return fail(SVOX_ERR_BAD_SHAPE, "svox_notes_pool_info: the workspace does not hold a chunk per ray");
    *counter_offset = (int64_t)((char*)ws.stocks_taken - base);
    *pool_stocks = (ws.n_chunks - ws.first_shared + kChunkStock - 1) / kChunkStock;
    return SVOX_OK;
}

int64_t svox_volume_render_backward_workspace_bytes(int64_t n_rays, int32_t records_per_ray) {
    if (n_rays <= 0 || records_per_ray <= 0) return 0;
    const int64_t chunks_per_ray = (records_per_ray + kChunkRecords - 1) / kChunkRecords;
    return n_rays * chunks_per_ray * kChunkBytes + bitmap_bytes(n_rays) + kTailBytes;
}

int svox_volume_render_backward_ws(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                                   const void* grad_output, void* grad_data_out, int32_t accumulate,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_rays(rays);
    if (rc) return rc;
    if (!grad_data_out) return fail(SVOX_ERR_NULL_POINTER, "grad_data_out is NULL");
    if (!accumulate) {
        rc = zero_fill(grad_data_out, data_bytes(tree), (hipStream_t)stream);
        if (rc) return rc;
    }
    if (rays->n_rays == 0) return SVOX_OK;
    if (!grad_output) return fail(SVOX_ERR_NULL_POINTER, "grad_output is NULL");
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    if (tree->dtype == SVOX_F32 && workspace) {
        const BatchSource<float> all = batch_source<float>(rays, true);
        rc = backward_by_noting(tree, all, all, opt, grad_output, grad_data_out, workspace, workspace_bytes,
                                rays->n_rays, stamp_of(tree, rays, opt), (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    if (tree->dtype == SVOX_F32)
        launch_backward<BatchSource<float>, float>(tree, batch_source<float>(rays, true), opt, od, grad_output,
                                                   grad_data_out, (hipStream_t)stream);
    else
        launch_backward<BatchSource<double>, double>(tree, batch_source<double>(rays, true), opt, od, grad_output,
                                                     grad_data_out, (hipStream_t)stream);
    return check_launch("volume_render_backward");
}

// svox_volume_render_backward_ws on the library's own array: no allocation anywhere on the way (the
// stock counter in the array's tail is cleared by the fill kernel of launch_noted before the noting
// launch; everything else in the array is written by that launch before the launches after it read it).
int svox_volume_render_backward_static(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                       const SvoxRenderOptions* opt, const void* grad_output, void* grad_data_out,
                                       int32_t accumulate, void* stream) {
    int rc = check_rays(rays);
    if (rc) return rc;
    if (rays->n_rays > SVOX_STATIC_RAYS_MAX)
        return fail(SVOX_ERR_BAD_SHAPE,
                    "svox.volume_render_backward_static: %lld rays exceed the %d rays the library's fixed "
                    "workspace serves per call; split the batch (accumulate = 1 from the second part on) or "
                    "call svox_volume_render_backward_ws with a workspace of your own",
                    (long long)rays->n_rays, (int)SVOX_STATIC_RAYS_MAX);
    void* ws = nullptr;
    rc = static_workspace(&ws);
    if (rc) return rc;
    return svox_volume_render_backward_ws(tree, rays, opt, grad_output, grad_data_out, accumulate, ws,
                                          (int64_t)SVOX_STATIC_WORKSPACE_BYTES, stream);
}

int svox_volume_render_images_backward(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                                       int64_t pose_stride, const SvoxRenderOptions* opt,
                                       const void* grad_output, void* grad_data_out, int32_t accumulate,
                                       void* stream) {
    return svox_volume_render_images_backward_ws(tree, cam, n_images, pose_stride, opt, grad_output, grad_data_out,
                                                 accumulate, nullptr, 0, stream);
}

int svox_volume_render_images_backward_ws(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                                          int64_t pose_stride, const SvoxRenderOptions* opt,
                                          const void* grad_output, void* grad_data_out, int32_t accumulate,
                                          void* workspace, int64_t workspace_bytes, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    rc = check_camera(cam, n_images, pose_stride);
    if (rc) return rc;
    if (!grad_data_out) return fail(SVOX_ERR_NULL_POINTER, "grad_data_out is NULL");
    if (!accumulate) {
        rc = zero_fill(grad_data_out, data_bytes(tree), (hipStream_t)stream);
        if (rc) return rc;
    }
    if (cam->width == 0 || cam->height == 0 || n_images == 0) return SVOX_OK;
    if (!grad_output) return fail(SVOX_ERR_NULL_POINTER, "grad_output is NULL");
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    if (tree->dtype == SVOX_F32) {
        const auto src = image_source<float>(cam, n_images, pose_stride, opt);
        if (workspace) {
            rc = backward_by_noting(tree, src, src, opt, grad_output, grad_data_out, workspace, workspace_bytes,
                                    (int64_t)n_images * cam->width * cam->height,
                                    stamp_of_image(tree, cam, n_images, opt), (hipStream_t)stream);
            if (rc <= 0) return rc;
        }
        launch_backward<ImageSource<float>, float>(tree, src, opt, od, grad_output, grad_data_out, (hipStream_t)stream);
    } else {
        const auto src = image_source<double>(cam, n_images, pose_stride, opt);
        launch_backward<ImageSource<double>, double>(tree, src, opt, od, grad_output, grad_data_out, (hipStream_t)stream);
    }
    return check_launch("volume_render_image_backward");
}

int svox_volume_render_image_backward(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                      const SvoxRenderOptions* opt, const void* grad_output, void* grad_data_out,
                                      int32_t accumulate, void* stream) {
    return svox_volume_render_images_backward(tree, cam, 1, 12, opt, grad_output, grad_data_out, accumulate, stream);
}

int svox_se_grad(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                 const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* stream) {
    int od;
    int rc = check_rays(rays);
    if (rc) return rc;
    rc = se_grad_prepare(tree, opt, grad_out, hessdiag_out, &od, (hipStream_t)stream);
    if (rc) return rc;
    if (rays->n_rays == 0) return SVOX_OK;
    if (!color_ref || !color_out) return fail(SVOX_ERR_NULL_POINTER, "color_ref / color_out is NULL");
    if (tree->dtype == SVOX_F32)
        launch_se_grad<BatchSource<float>, float>(tree, batch_source<float>(rays, true), opt, od, color_ref,
                                                  color_out, grad_out, hessdiag_out, (hipStream_t)stream);
    else
        launch_se_grad<BatchSource<double>, double>(tree, batch_source<double>(rays, true), opt, od, color_ref,
                                                    color_out, grad_out, hessdiag_out, (hipStream_t)stream);
    return check_launch("se_grad");
}

int svox_se_grad_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                       const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* stream) {
    int od;
    int rc = check_camera(cam, 1, 12);
    if (rc) return rc;
    rc = se_grad_prepare(tree, opt, grad_out, hessdiag_out, &od, (hipStream_t)stream);
    if (rc) return rc;
    if (cam->width == 0 || cam->height == 0) return SVOX_OK;
    if (!color_ref || !color_out) return fail(SVOX_ERR_NULL_POINTER, "color_ref / color_out is NULL");
    if (tree->dtype == SVOX_F32) {
        const auto src = image_source<float>(cam, 1, 12, opt);
        launch_se_grad<ImageSource<float>, float>(tree, src, opt, od, color_ref, color_out, grad_out, hessdiag_out,
                                                  (hipStream_t)stream);
    } else {
        const auto src = image_source<double>(cam, 1, 12, opt);
        launch_se_grad<ImageSource<double>, double>(tree, src, opt, od, color_ref, color_out, grad_out,
                                                    hessdiag_out, (hipStream_t)stream);
    }
    return check_launch("se_grad_persp");
}

int svox_se_grad_ws(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                    const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* workspace,
                    int64_t workspace_bytes, void* stream) {
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    int od;
    int rc = check_rays(rays);
    if (rc) return rc;
    rc = check_render(tree, opt, &od);
    if (rc) return rc;
    const SvoxRenderOptions plain = without_thresholds(opt);
    if (od != 3 || rays->n_rays == 0 || !color_ref || !color_out ||
        !noted_ok(tree, &plain, rays->n_rays, workspace, workspace_bytes))
        return svox_se_grad(tree, rays, opt, color_ref, color_out, grad_out, hessdiag_out, stream);
    rc = se_grad_prepare(tree, opt, grad_out, hessdiag_out, &od, (hipStream_t)stream);
    if (rc) return rc;
    const BatchSource<float> all = batch_source<float>(rays, true);
    return se_grad_from_notes(tree, all, all, &plain, color_ref, color_out, grad_out, hessdiag_out, workspace,
                              workspace_bytes, rays->n_rays, stamp_of(tree, rays, &plain), (hipStream_t)stream);
}

int svox_se_grad_image_ws(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                          const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out,
                          void* workspace, int64_t workspace_bytes, void* stream) {
    if (workspace_bytes < 0) return fail(SVOX_ERR_BAD_SHAPE, "negative workspace size");
    int od;
    int rc = check_camera(cam, 1, 12);
    if (rc) return rc;
    rc = check_render(tree, opt, &od);
    if (rc) return rc;
    const SvoxRenderOptions plain = without_thresholds(opt);
    const int64_t n_slots = (int64_t)cam->width * cam->height;
    if (od != 3 || n_slots == 0 || !color_ref || !color_out ||
        !noted_ok(tree, &plain, n_slots, workspace, workspace_bytes))
        return svox_se_grad_image(tree, cam, opt, color_ref, color_out, grad_out, hessdiag_out, stream);
    rc = se_grad_prepare(tree, opt, grad_out, hessdiag_out, &od, (hipStream_t)stream);
    if (rc) return rc;
    const ImageSource<float> all = image_source<float>(cam, 1, 12, opt);
    return se_grad_from_notes(tree, all, all, &plain, color_ref, color_out, grad_out, hessdiag_out, workspace,
                              workspace_bytes, n_slots, stamp_of_image(tree, cam, 1, &plain), (hipStream_t)stream);
}

int svox_mark_leaves_below(const SvoxTreeSpec* tree, float sigma_thresh, int32_t density_softplus, int32_t* marks_out,
                           void* stream) {
    int rc = check_tree(tree, true);
    if (rc) return rc;
    if (!marks_out) return fail(SVOX_ERR_NULL_POINTER, "marks_out is NULL");
    if (!(sigma_thresh >= 0.0f)) return fail(SVOX_ERR_BAD_SHAPE, "marks need a sigma_thresh >= 0, got %g", (double)sigma_thresh);
    const int64_t cells = tree->capacity * tree->N * tree->N * tree->N;
    if (cells == 0) return SVOX_OK;
    const unsigned blocks = blocks_for(cells, 256);
    if (tree->dtype == SVOX_F32)
        hipLaunchKernelGGL((mark_leaves_kernel<float>), dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                           (const float*)tree->data, tree->child, cells, tree->data_dim, sigma_thresh,
                           density_softplus != 0, marks_out);
    else
        hipLaunchKernelGGL((mark_leaves_kernel<double>), dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                           (const double*)tree->data, tree->child, cells, tree->data_dim, (double)sigma_thresh,
                           density_softplus != 0, marks_out);
    return check_launch("mark_leaves_below");
}

int svox_mark_empty_leaves(const SvoxTreeSpec* tree, int32_t* marks_out, void* stream) {
    return svox_mark_leaves_below(tree, 0.0f, 0, marks_out, stream);
}

int svox_grid_weight_render(const void* data, int32_t reso, int32_t dtype, const SvoxCameraSpec* cam,
                            const SvoxRenderOptions* opt, const void* offset, const void* scaling,
                            void* grid_weight_out, void* grid_hit_out, void* stream) {
    if (!data || !opt || !offset || !scaling || !grid_weight_out || !grid_hit_out)
        return fail(SVOX_ERR_NULL_POINTER, "grid_weight_render: NULL argument");
    if (dtype != SVOX_F32 && dtype != SVOX_F64) return fail(SVOX_ERR_BAD_DTYPE, "dtype must be SVOX_F32 or SVOX_F64");
    // cell ids are 32-bit, as in the reference (reso^3 < 2^31)
    if (reso < 1 || reso > 1290) return fail(SVOX_ERR_BAD_SHAPE, "grid resolution must be in [1, 1290]");
    int rc = check_camera(cam, 1, 12);
    if (rc) return rc;
    const int64_t bytes = (int64_t)reso * reso * reso * (dtype == SVOX_F32 ? 4 : 8);
    rc = zero_fill(grid_weight_out, bytes, (hipStream_t)stream);
    if (rc) return rc;
    rc = zero_fill(grid_hit_out, bytes, (hipStream_t)stream);
    if (rc) return rc;
    if (cam->width == 0 || cam->height == 0) return SVOX_OK;
    if (dtype == SVOX_F32) {
        const auto src = image_source<float>(cam, 1, 12, opt);
        hipLaunchKernelGGL((grid_weight_kernel<float>), dim3(blocks_for(total_items_of(src), kMarchThreads)),
                           dim3(kMarchThreads), 0, (hipStream_t)stream, (const float*)data, reso, src, *opt,
                           (const float*)offset, (const float*)scaling, (float*)grid_weight_out,
                           (float*)grid_hit_out);
    } else {
        const auto src = image_source<double>(cam, 1, 12, opt);
        hipLaunchKernelGGL((grid_weight_kernel<double>), dim3(blocks_for(total_items_of(src), kMarchThreads)),
                           dim3(kMarchThreads), 0, (hipStream_t)stream, (const double*)data, reso, src, *opt,
                           (const double*)offset, (const double*)scaling, (double*)grid_weight_out,
                           (double*)grid_hit_out);
    }
    return check_launch("grid_weight_render");
}

int svox_volume_render_stats(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxCameraSpec* cam,
                             const SvoxRenderOptions* opt, SvoxMarchStats* stats_out, void* stream) {
    int od;
    int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    if (!stats_out) return fail(SVOX_ERR_NULL_POINTER, "stats_out is NULL");
    if ((rays != nullptr) == (cam != nullptr))
        return fail(SVOX_ERR_BAD_SHAPE, "exactly one of rays and cam must be given");
    unsigned long long* st = (unsigned long long*)stats_out;
    if (rays) {
        rc = check_rays(rays);
        if (rc) return rc;
        if (rays->n_rays == 0) return SVOX_OK;
        const unsigned blocks = blocks_for(rays->n_rays, kMarchThreads);
        if (tree->dtype == SVOX_F32)
            hipLaunchKernelGGL((render_stats_kernel<float, BatchSource<float>>), dim3(blocks), dim3(kMarchThreads), 0,
                               (hipStream_t)stream, make_tree<float>(tree), batch_source<float>(rays), *opt, st);
        else
            hipLaunchKernelGGL((render_stats_kernel<double, BatchSource<double>>), dim3(blocks), dim3(kMarchThreads),
                               0, (hipStream_t)stream, make_tree<double>(tree), batch_source<double>(rays), *opt, st);
    } else {
        rc = check_camera(cam);
        if (rc) return rc;
        if (cam->width == 0 || cam->height == 0) return SVOX_OK;
        if (tree->dtype == SVOX_F32) {
            const auto src = image_source<float>(cam, 1, 12, opt);
            const unsigned blocks = blocks_for(total_items_of(src), kMarchThreads);
            hipLaunchKernelGGL((render_stats_kernel<float, ImageSource<float>>), dim3(blocks), dim3(kMarchThreads), 0,
                               (hipStream_t)stream, make_tree<float>(tree), src, *opt, st);
        } else {
            const auto src = image_source<double>(cam, 1, 12, opt);
            const unsigned blocks = blocks_for(total_items_of(src), kMarchThreads);
            hipLaunchKernelGGL((render_stats_kernel<double, ImageSource<double>>), dim3(blocks), dim3(kMarchThreads),
                               0, (hipStream_t)stream, make_tree<double>(tree), src, *opt, st);
        }
    }
    return check_launch("volume_render_stats");
}

int svox_octree_kernels_serve(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    int od;
    const int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    return fast_basis(tree, opt) >= 0 ? 1 : 0;
}

int svox_notes_serve(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    int od;
    const int rc = check_render(tree, opt, &od);
    if (rc) return rc;
    return notes_possible(tree, opt) ? 1 : 0;
}

int svox_give_up_count(int64_t* count_out) {
    if (!count_out) return fail(SVOX_ERR_NULL_POINTER, "count_out is NULL");
    unsigned int n = 0;
    hipError_t err = hipDeviceSynchronize();
    if (err == hipSuccess) err = hipMemcpyFromSymbol(&n, HIP_SYMBOL(split_give_ups), sizeof(n), 0, hipMemcpyDeviceToHost);
    if (err != hipSuccess) return fail(SVOX_ERR_LAUNCH, "svox.give_up_count: %s", hipGetErrorString(err));
    *count_out = (int64_t)n;
    return SVOX_OK;
}

}  // extern "C"
#pragma GCC visibility pop
