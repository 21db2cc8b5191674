/*
 * svox_hip.h -- C ABI of libsvox_hip.so: N^3-tree point queries and differentiable volume
 * rendering on AMD gfx950 (MI355X).
 *
 * Every entry point below replaces one function of the reference's pybind11 module `svox.csrc`
 * (svox/csrc/svox.cpp:63-122).  Where the reference passes torch::Tensor members, this ABI passes
 * raw device pointers plus sizes; where the reference allocates and returns a tensor, the caller
 * passes the output buffer.  Nothing here depends on torch or on HIP headers: `stream` is a
 * hipStream_t carried as void* (NULL = the null stream).
 *
 * Conventions
 *   - all pointers are device pointers valid on the current HIP device unless stated otherwise;
 *   - all arrays are dense and row-major (the reference requires contiguous tensors,
 *     svox/csrc/include/data_spec.hpp:37-42);
 *   - `dtype` selects the scalar type of every `void*` array in the call: SVOX_F32 or SVOX_F64
 *     (the reference dispatches with AT_DISPATCH_FLOATING_TYPES);
 *   - every function returns SVOX_OK (0) or a negative SvoxStatus; svox_last_error() returns a
 *     per-thread message for the last failing call.  Launches are asynchronous on `stream`;
 *   - the library never allocates or frees device memory.
 */
#ifndef SVOX_HIP_H_
#define SVOX_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SVOX_ABI_VERSION 3

typedef enum SvoxStatus {
    SVOX_OK = 0,
    SVOX_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
    SVOX_ERR_BAD_SHAPE = -2,      /* a size is negative / zero where it may not be, or inconsistent */
    SVOX_ERR_BAD_DTYPE = -3,      /* dtype is neither SVOX_F32 nor SVOX_F64 */
    SVOX_ERR_UNSUPPORTED = -4,    /* valid in the reference but outside what this build covers */
    SVOX_ERR_LAUNCH = -5,         /* hipGetLastError() after the launch was not hipSuccess */
    SVOX_ERR_NO_DEVICE = -6       /* no usable HIP device */
} SvoxStatus;

typedef enum SvoxDType { SVOX_F32 = 0, SVOX_F64 = 1 } SvoxDType;

/* svox/csrc/include/data_spec.hpp:44-49 */
typedef enum SvoxDataFormat {
    SVOX_FORMAT_RGBA = 0,
    SVOX_FORMAT_SH = 1,
    SVOX_FORMAT_SG = 2,
    SVOX_FORMAT_ASG = 3
} SvoxDataFormat;

#define SVOX_MAX_BASIS_DIM 25 /* size of the reference's basis_fn array, rt_kernel.cu:250 */
#define SVOX_MAX_OUT_DIM 16   /* widest rendered colour vector this build accumulates */

/* TreeSpec, svox/csrc/include/data_spec.hpp:65-89 */
typedef struct SvoxTreeSpec {
    void* data;                  /* (capacity, N, N, N, data_dim) scalar; leaf records, sigma last */
    const int32_t* child;        /* (capacity, N, N, N) relative child offset, 0 = leaf */
    const int32_t* parent_depth; /* (capacity, 2): packed parent cell, node depth */
    const void* extra_data;      /* (extra_rows, extra_cols) scalar for SG/ASG, else NULL */
    const void* offset;          /* 3 scalars on the device, NULL = (0,0,0) */
    const void* scaling;         /* 3 scalars on the device, NULL = (1,1,1) */
    void* weight_accum;          /* (capacity, N, N, N) scalar, or NULL */
    int64_t capacity;            /* M = child.shape[0] */
    int32_t N;                   /* branching factor */
    int32_t data_dim;            /* K */
    int32_t extra_rows;
    int32_t extra_cols;
    int32_t weight_accum_max;    /* nonzero: max-reduce into weight_accum, zero: sum */
    int32_t dtype;               /* SvoxDType of data/extra_data/offset/scaling/weight_accum */
    const int32_t* child_marks;  /* optional (NULL: none): what svox_mark_empty_leaves / svox_mark_leaves_below wrote for this tree */
    float child_marks_thresh;    /* the sigma_thresh those marks were made with (0 for svox_mark_empty_leaves) */
    int32_t child_marks_softplus;/* nonzero: they were made with density_softplus */
} SvoxTreeSpec;

/* RaysSpec, svox/csrc/include/data_spec.hpp:51-63 */
typedef struct SvoxRaysSpec {
    const void* origins; /* (n_rays, 3) scalar */
    const void* dirs;    /* (n_rays, 3) scalar */
    const void* vdirs;   /* (n_rays, 3) scalar */
    int64_t n_rays;
} SvoxRaysSpec;

/* CameraSpec, svox/csrc/include/data_spec.hpp:91-104 */
typedef struct SvoxCameraSpec {
    const void* c2w; /* device pointer, (3 or 4, 4) scalar; only the first 3 rows are read */
    float fx;
    float fy;
    int32_t width;
    int32_t height;
} SvoxCameraSpec;

/* RenderOptions, svox/csrc/include/data_spec.hpp:107-126 (bool widened to int32_t) */
typedef struct SvoxRenderOptions {
    float step_size;
    float background_brightness;
    int32_t format;    /* SvoxDataFormat */
    int32_t basis_dim; /* -1 for RGBA */
    int32_t ndc_width; /* < 0 disables NDC */
    int32_t ndc_height;
    float ndc_focal;
    int32_t min_comp;
    int32_t max_comp;
    float sigma_thresh;
    float stop_thresh;
    int32_t density_softplus;
    float rgb_padding;
} SvoxRenderOptions;

/* Per-launch march statistics written by svox_volume_render_stats (no counterpart in the
 * reference; used to price a launch in algorithmic bytes). */
typedef struct SvoxMarchStats {
    uint64_t rays;            /* rays traced */
    uint64_t rays_hit;        /* rays whose segment intersects the unit cube */
    uint64_t samples;         /* leaf visits of the forward march */
    uint64_t samples_shaded;  /* leaf visits with sigma > sigma_thresh */
    uint64_t samples_bwd;     /* leaf visits of one backward march (no early stop) */
    uint64_t samples_bwd_pos; /* of those, visits with sigma > 0 */
    uint64_t levels;          /* child-table entries read by a root-to-leaf walk, forward march */
    uint64_t samples_tail;    /* of `samples`: visits after the last shaded leaf of their ray (all visits of a ray
                                 that shades nothing); not counted where the march stops early (stop_thresh) */
} SvoxMarchStats;

int svox_abi_version(void);
const char* svox_last_error(void);
const char* svox_status_string(int status);

/* Debugging aid without a counterpart in the reference.  Bit 0: route every call to the generic
 * kernels (any N, any dtype) even where a specialised octree kernel exists.  Bit 1: ray batches of
 * any size run the way batches of 512 Ki rays and more do (several 64-ray chunks per wavefront, idle
 * lanes refilled), so that small test batches reach those kernels.  Bit 2: forward renders never take
 * the kernel that walks and shades on two wavefronts; bit 3: they always do where it applies (launches
 * of one 64-ray wavefront per tile or chunk, no weight accumulator), whatever their size.  Bit 4: the bounded waits
 * of that kernel give up at the first look that finds nothing (so that a test can see what a give-up leaves
 * behind; every kernel still ends normally).  The flags belong to the calling thread. */
void svox_set_debug_flags(int flags);

/* No counterpart in the reference.  The forward kernel that walks and shades on two wavefronts hands leaves over
 * through bounded waits (4 Mi looks); a wavefront whose wait ever ran out leaves NaN in its pixels, marks its rays'
 * notes "to be marched" (the backward pass then marches them: the gradient stays right) and counts itself here.
 * *count_out: such wavefronts since the library was loaded, on the current device; 0 in any healthy run.  The call
 * waits for all work queued on the device. */
int svox_give_up_count(int64_t* count_out);

/* query_vertical(TreeSpec&, Tensor indices) -> (values, node_ids); svox/csrc/svox_kernel.cu:120-143.
 * indices (n_points,3) scalar; values_out (n_points, data_dim) scalar; node_ids_out (n_points) int64. */
int svox_query_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                        void* values_out, int64_t* node_ids_out, void* stream);

/* query_vertical_backward(TreeSpec&, indices, grad_output) -> grad_data; svox_kernel.cu:160-182.
 * grad_output (n_points, grad_dim); grad_data_out (capacity, N, N, N, grad_dim).  The reference
 * returns a fresh zero-filled tensor; here the library zero-fills grad_data_out first unless
 * `accumulate` is nonzero. */
int svox_query_vertical_backward(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                                 const void* grad_output, int32_t grad_dim, void* grad_data_out,
                                 int32_t accumulate, void* stream);

/* assign_vertical(TreeSpec&, indices, values); svox_kernel.cu:145-158.  values (n_points, value_dim),
 * value_dim <= data_dim.  Two points in one leaf race; the last writer wins, as in the reference. */
int svox_assign_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                         const void* values, int32_t value_dim, void* stream);

/* calc_corners(TreeSpec&, indexer) -> (n,3); svox_kernel.cu:184-203.  indexer (n_leaves,4) int64
 * rows [node, x, y, z]; corners_out (n_leaves,3) scalar of tree->dtype. */
int svox_calc_corners(const SvoxTreeSpec* tree, const int64_t* indexer, int64_t n_leaves,
                      void* corners_out, void* stream);

/* volume_render(TreeSpec&, RaysSpec&, RenderOptions&) -> (n_rays, out_dim); rt_kernel.cu:1019-1036.
 * out_dim = svox_out_data_dim(opt->format, opt->basis_dim, tree->data_dim). */
int svox_volume_render(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                       const SvoxRenderOptions* opt, void* out, void* stream);

/* volume_render_image(TreeSpec&, CameraSpec&, RenderOptions&) -> (H, W, out_dim);
 * rt_kernel.cu:1038-1057. */
int svox_volume_render_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                             const SvoxRenderOptions* opt, void* out, void* stream);

/* No counterpart in the reference (its extension renders one image per call): n_images pinhole
 * images of one size, focal length and option set in ONE launch, so that the tiles of several
 * poses fill the GPU together.  cam->c2w points at the first pose; pose i starts pose_stride
 * scalars after pose i-1 (12 for packed (3,4) poses, 16 for (4,4)).  out is (n_images, H, W, out_dim).
 * With n_images == 1 this is svox_volume_render_image. */
int svox_volume_render_images(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, int32_t n_images,
                              int64_t pose_stride, const SvoxRenderOptions* opt, void* out,
                              void* stream);

/* Backward of svox_volume_render_images; grad_output is (n_images, H, W, out_dim). */
int svox_volume_render_images_backward(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                       int32_t n_images, int64_t pose_stride,
                                       const SvoxRenderOptions* opt, const void* grad_output,
                                       void* grad_data_out, int32_t accumulate, void* stream);

/* volume_render_backward(TreeSpec&, RaysSpec&, RenderOptions&, grad_output) -> zeros_like(data) +
 * scatter; rt_kernel.cu:1059-1083.  grad_output (n_rays, out_dim); grad_data_out has the shape of
 * tree->data and is zero-filled first unless `accumulate` is nonzero. */
int svox_volume_render_backward(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                const SvoxRenderOptions* opt, const void* grad_output,
                                void* grad_data_out, int32_t accumulate, void* stream);

/* No counterpart in the reference.  svox_volume_render_backward with a workspace in device memory
 * (16-byte aligned, any contents, overwritten): the first of the two marches of a ray notes in the
 * workspace what the second march needs of the leaves with sigma > 0 (24 bytes per leaf, in chunks
 * of 384 bytes = 15 leaves and a link), and a second launch forms the gradient of every ray whose
 * notes fit from those notes, without the tree; the other rays are marched a second time.  The first n_rays chunks are the rays' own; the rest of
 * the workspace is shared out among the wavefronts for rays with more than 15 such leaves.  After
 * the chunks come one bit per ray and 256 bytes of bookkeeping (used by the two calls below), so
 * the workspace holds (workspace_bytes - 256 - 16 * ceil(n_rays / 128)) / 384 chunks and is useful
 * from n_rays chunks on.
 * The gradient is the one svox_volume_render_backward gives (the same terms; the order of the
 * atomic additions differs from call to call either way).  Without a workspace (NULL, or fewer
 * than n_rays chunks), for fp64 trees and wherever the generic kernels run, the call is
 * svox_volume_render_backward.  svox_volume_render_backward_workspace_bytes gives the size that
 * holds `records_per_ray` leaves per ray on average (rounded up to whole chunks). */
int svox_volume_render_backward_ws(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                   const SvoxRenderOptions* opt, const void* grad_output,
                                   void* grad_data_out, int32_t accumulate, void* workspace,
                                   int64_t workspace_bytes, void* stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): svox_volume_render_backward_ws
 * whose workspace is a fixed array inside the library (SVOX_STATIC_WORKSPACE_BYTES of device memory per
 * GPU the library runs on, held until the process ends) instead of a caller's buffer.  The call
 * allocates and frees nothing.  At most SVOX_STATIC_RAYS_MAX rays per call: more is SVOX_ERR_BAD_SHAPE
 * (split the batch and pass accumulate = 1 from the second part on).  The array holds 30 noted leaves
 * per ray at the maximum ray count and more per ray for smaller batches; rays whose notes do not fit
 * are marched twice, as by svox_volume_render_backward.  Same gradient as svox_volume_render_backward_ws.
 * All calls on one GPU share that GPU's array: two such calls that overlap in time on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe. */
#define SVOX_STATIC_RAYS_MAX 65536
#define SVOX_STATIC_WORKSPACE_BYTES (65536LL * 768 + 8192 + 256)
int svox_volume_render_backward_static(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                       const SvoxRenderOptions* opt, const void* grad_output,
                                       void* grad_data_out, int32_t accumulate, void* stream);

/* No counterpart in the reference: the pair a training step calls instead of svox_volume_render and
 * svox_volume_render_backward when it runs both on the same rays (what an autograd function keeps
 * between its forward and its backward).  svox_volume_render_noted gives the output of
 * svox_volume_render and, in the same march, leaves in the workspace the notes of every leaf with
 * sigma > 0 of every ray (the whole ray, also behind the point where the rendering stops early).
 * svox_volume_render_backward_noted, called with the same tree, rays, options and workspace, gives
 * the gradient of svox_volume_render_backward without walking the tree: it replays the notes twice.
 * A ray whose notes did not fit is marched twice as in svox_volume_render_backward; so is every ray
 * if the workspace does not carry the stamp (ray count, tree->data, tree->child, rays->origins,
 * rays->dirs, step size, sigma_thresh) the first call left.  The caller must not change tree->data, the rays or the
 * workspace between the two calls.  Workspace as for svox_volume_render_backward_ws (same size
 * function).  Where notes cannot be taken (fp64 or generic kernels, a weight accumulator, a negative
 * sigma_thresh, a workspace with fewer than n_rays chunks) the two calls are svox_volume_render and
 * svox_volume_render_backward_ws. */
int svox_volume_render_noted(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                             const SvoxRenderOptions* opt, void* out, void* workspace,
                             int64_t workspace_bytes, void* stream);
int svox_volume_render_backward_noted(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                      const SvoxRenderOptions* opt, const void* grad_output,
                                      void* grad_data_out, int32_t accumulate, void* workspace,
                                      int64_t workspace_bytes, void* stream);

/* The same pair for images (svox_volume_render_images / svox_volume_render_images_backward): one
 * ray per pixel, n_rays = n_images * H * W; the stamp holds cam->c2w in place of rays->origins. */
int svox_volume_render_images_noted(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                    int32_t n_images, int64_t pose_stride,
                                    const SvoxRenderOptions* opt, void* out, void* workspace,
                                    int64_t workspace_bytes, void* stream);
int svox_volume_render_images_backward_noted(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                             int32_t n_images, int64_t pose_stride,
                                             const SvoxRenderOptions* opt, const void* grad_output,
                                             void* grad_data_out, int32_t accumulate, void* workspace,
                                             int64_t workspace_bytes, void* stream);
int64_t svox_volume_render_backward_workspace_bytes(int64_t n_rays, int32_t records_per_ray);

/* No counterpart in the reference.  How full a workspace of notes ran: after a call that takes notes
 * (svox_volume_render_noted, svox_volume_render_images_noted, the _ws calls) the 64-bit word at byte
 * *counter_offset of the workspace holds the number of 64-chunk stocks its wavefronts asked for
 * beyond the rays' own chunks, and the workspace has *pool_stocks of them (rounded up).  A count at
 * or above that number says the shared chunks ran out: some rays' notes are incomplete (those rays are
 * marched by the backward pass: correct, slower) and a larger workspace would serve the same rays
 * better.  Returns 0, or SVOX_ERR_BAD_SHAPE for a workspace too small to hold n_rays chunks. */
int svox_notes_pool_info(int64_t n_rays, int64_t workspace_bytes, int64_t* counter_offset, int64_t* pool_stocks);

/* The same for svox_volume_render_images_backward: one ray per pixel, n_rays = n_images * H * W. */
int svox_volume_render_images_backward_ws(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                          int32_t n_images, int64_t pose_stride,
                                          const SvoxRenderOptions* opt, const void* grad_output,
                                          void* grad_data_out, int32_t accumulate, void* workspace,
                                          int64_t workspace_bytes, void* stream);

/* volume_render_image_backward(TreeSpec&, CameraSpec&, RenderOptions&, grad_output);
 * rt_kernel.cu:1085-1109.  grad_output (H, W, out_dim). */
int svox_volume_render_image_backward(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                      const SvoxRenderOptions* opt, const void* grad_output,
                                      void* grad_data_out, int32_t accumulate, void* stream);

/* se_grad(TreeSpec&, RaysSpec&, color, RenderOptions&) -> (color_out, grad, hessdiag);
 * svox.cpp:54-55, 115, rt_kernel.cu:1111-1139 (kernel :479-715, :846-868).
 * Rendered colour plus gradient and Gauss-Newton Hessian diagonal of 0.5 * |render - color_ref|^2 with
 * respect to tree.data.  color_ref and color_out are (B, out_dim), out_dim <= 4; grad_out and
 * hessdiag_out have the shape of tree.data and are zero-filled by the library.  Thresholds are not
 * applied (the kernel tests sigma > 0 and never stops early). */
int svox_se_grad(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                 const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* stream);

/* se_grad_persp(TreeSpec&, CameraSpec&, RenderOptions&, color) -> (color_out, grad, hessdiag);
 * svox.cpp:56-57, 116, rt_kernel.cu:1141-1173 (kernel :870-897).  color_ref and color_out are
 * (H, W, out_dim). */
int svox_se_grad_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                       const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* stream);

/* svox_se_grad / svox_se_grad_image with a caller workspace (no reference counterpart: the reference
 * marches every ray three times, rt_kernel.cu:518-710): one march notes the leaves with sigma > 0 of
 * every ray in the workspace, the residual, gradient and Hessian terms are then formed from the notes.
 * Same terms, same results as the plain entry points up to the order of the atomic additions; the
 * rendered colour is bit-identical.  The workspace is the one of svox_volume_render_backward_ws
 * (svox_volume_render_backward_workspace_bytes(n_rays or H * W, per_ray); 16-byte aligned); rays whose
 * notes do not fit are marched as without a workspace.  Without a usable workspace, with fp64 data or
 * options the octree kernels do not cover, the call is the plain one.  The notes left in the workspace
 * are those svox_volume_render_noted would leave with both thresholds at zero. */
int svox_se_grad_ws(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                    const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out, void* workspace,
                    int64_t workspace_bytes, void* stream);
int svox_se_grad_image_ws(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                          const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* Marks the empty leaves of a tree for the renderers (no reference counterpart; for trees that are
 * rendered many times between changes, e.g. when serving views of a finished model).
 * marks_out (capacity, N, N, N) int32 receives a copy of tree->child in which every leaf cell whose
 * density is not > 0 holds SVOX_EMPTY_LEAF instead of 0.  Passed as SvoxTreeSpec.child_marks, it lets
 * the fp32 octree render kernels pass through such leaves without reading their density (a 128-byte
 * line for 4 bytes, four fifths of the leaves a ray of a sparse scene visits).  Results are bit-identical:
 * no kernel lets a leaf with sigma <= 0 contribute (the marks are ignored for a negative sigma_thresh,
 * for fp64 trees, N != 2 and density_softplus).  The marks describe data and child as they were when
 * the call ran: after any write to the densities or to the structure they must be made again or left
 * out -- the library cannot tell.  Point queries and svox_calc_corners never use them. */
#define SVOX_EMPTY_LEAF (-2)
int svox_mark_empty_leaves(const SvoxTreeSpec* tree, int32_t* marks_out, void* stream);

/* No counterpart in the reference.  svox_mark_empty_leaves for a forward render with thresholds: a leaf is marked
 * when its density -- after the shifted softplus of rt_kernel.cu:276-277 if density_softplus is nonzero -- is not
 * > sigma_thresh (>= 0), i.e. exactly when trace_ray skips it (rt_kernel.cu:278).  The caller passes the marks
 * with SvoxTreeSpec.child_marks_thresh = sigma_thresh and .child_marks_softplus = density_softplus.  A forward
 * render whose options carry the same two values then shades every leaf that is not marked and reads its density
 * together with its colour coefficients instead of in a round trip of its own.  Calls that need leaves the marks
 * hide (a smaller or negative sigma_thresh, the other softplus setting; the backward passes, se_grad and the noting
 * forward passes, which work on every leaf with sigma > 0, unless the marks were made with threshold 0) leave the
 * marks aside and read the child table.  Results are bit-identical with and without marks. */
int svox_mark_leaves_below(const SvoxTreeSpec* tree, float sigma_thresh, int32_t density_softplus,
                           int32_t* marks_out, void* stream);

/* grid_weight_render(data, CameraSpec&, RenderOptions&, offset, scaling) -> {grid_weight, grid_hit};
 * svox.cpp:38-40, 120, rt_kernel.cu:1174-1203 (kernel :898-1003).
 * Marches the pixel rays of one camera through a dense density grid data (reso, reso, reso): per
 * cell with sigma > opt->sigma_thresh, grid_weight_out holds the largest compositing weight any ray
 * gave the cell and grid_hit_out the number of such visits.  offset and scaling are 3 scalars each
 * in device memory (world -> grid coordinates).  Both outputs are zero-filled by the library and
 * must be 16-byte aligned.  `dtype` is the scalar type of data, offset, scaling, c2w and outputs. */
int svox_grid_weight_render(const void* data, int32_t reso, int32_t dtype, const SvoxCameraSpec* cam,
                            const SvoxRenderOptions* opt, const void* offset, const void* scaling,
                            void* grid_weight_out, void* grid_hit_out, void* stream);

/* get_out_data_dim, rt_kernel.cu:1009-1015.  Returns -1 for an invalid combination. */
int svox_out_data_dim(int32_t format, int32_t basis_dim, int32_t data_dim);

/* No counterpart in the reference.  Walks the same marches as svox_volume_render (rays != NULL) or
 * svox_volume_render_image (cam != NULL) and adds the visit counts of the launch into *stats_out
 * (device pointer to one SvoxMarchStats, which the caller zeroes). */
int svox_volume_render_stats(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                             const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                             SvoxMarchStats* stats_out, void* stream);

/* No counterpart in the reference.  Which family of kernels serves the render calls of this tree under
 * these options (forward, backward and se_grad alike, with or without density_softplus): 1 the
 * wavefront-per-tile kernels (fp32, any branching factor, fewer than 2^30 cells, RGBA / SH / SG / ASG records
 * with basis_dim 1, 4, 9, 16 or 25, any range of components), 0 the one-ray-per-lane kernels that cover
 * everything else the reference accepts (fp64, other basis sizes and record shapes), or
 * a negative SvoxStatus for a tree or options no kernel accepts.  Results do not depend on the family. */
int svox_octree_kernels_serve(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt);

/* No counterpart in the reference.  1 if the noting calls (svox_volume_render_noted, svox_volume_render_images_noted)
 * take notes for this tree under these options when given a workspace with a chunk per ray, 0 if they run as the
 * plain forward calls and leave the workspace untouched (fp64, the one-ray-per-lane kernels, a weight accumulator, a
 * negative sigma_thresh), or a negative SvoxStatus.  A caller that would only allocate the workspace for the notes
 * asks first. */
int svox_notes_serve(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt);

#ifdef __cplusplus
}
#endif
#endif /* SVOX_HIP_H_ */
