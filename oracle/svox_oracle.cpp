// svox_oracle.cpp -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A scalar CPU restatement of the reference's CUDA kernels for N^3-tree queries and volume
// rendering, used only as the checker for the HIP library (by tests, by the smoke check and by the
// CPU-baseline leg of the benchmark).  The product never links, loads or calls this file.
//
// Each function cites the reference lines it restates (paths relative to the reference tree).
// It is written for clarity, one ray / one point at a time, with the reference's re-descent from
// the root for every sample; the HIP kernels are formulated differently (integer cell coordinates,
// cached descent paths) and are compared against this file's outputs.
//
// Floating-point contract.  The reference is compiled by nvcc with its default contraction
// (-fmad=true): a product whose only use is an addend becomes one fused multiply-add.  This file is
// compiled with -ffp-contract=off and spells those fusions explicitly (fma_()), following LLVM's
// rule: in `a*b + c*d` the left product is the fused one.  Division and square root are IEEE
// (correctly rounded).  exp() is the reference's single-precision expf even in double builds; it is
// restated here as oracle_expf (Cody-Waite reduction + degree-5 polynomial, <= 1 ulp, flushed to 0
// below e^-87) so that the value is a fixed function of its argument on every machine.
//
// Sums of gradient terms.  The reference adds every term to d(data) with an fp32 atomicAdd, in an
// order no two runs share; any fp32 order is within the comparison tolerance only while few terms
// meet in one element.  The backward and se_grad entry points therefore take `exact_sum`: every
// term is still formed in the tree's scalar type exactly as the reference forms it, but the terms of
// one element are added in double (SumBuffer) and rounded once at the end.  That result does not
// depend on the order of the rays or on the thread count beyond the last bit of the double sum, and
// it is what any fp32 summation order is an approximation of: the checker for many rays per leaf.
// With it the adder can report, per element, how far a sum of the same terms in the scalar type may
// stray from the exact one whatever the order (`slack`): sqrt(n) * u * sum |term| for n terms and
// unit roundoff u -- every one of the n - 1 additions rounds a partial sum no larger than sum |term|,
// and the roundings add up like a random walk.  The reference's own atomics are subject to it.
//
// Parity pins (which test fixes which function) are listed in tests/ and in oracle/README.md.

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#include "../include/svox_hip.h"

extern "C" int oracle_out_data_dim(int32_t format, int32_t basis_dim, int32_t data_dim);

namespace {

// ----------------------------------------------------------------------------------------------
// arithmetic helpers
// ----------------------------------------------------------------------------------------------
inline float fma_(float a, float b, float c) { return std::fmaf(a, b, c); }
inline double fma_(double a, double b, double c) { return std::fma(a, b, c); }

inline float bits_to_float(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// Single-precision e^x.  Stands in for the reference's expf (rt_kernel.cu:86-87 _SOFTPLUS_M1 /
// _SIGMOID, :280 att).  |error| <= 1 ulp on [-87, 88.72]; exactly 0 below -87; +inf above 88.7228.
float expf_fixed(float x) {
    if (!(x == x)) return x;
    if (x < -87.0f) return 0.0f;
    if (x > 88.72283f) return std::numeric_limits<float>::infinity();
    const float n = std::nearbyintf(x * 1.44269504088896341f);
    float r = std::fmaf(n, -0.693145751953125f, x);       // ln2 high part, 0x3f317200
    r = std::fmaf(n, -1.428606765330187045e-06f, r);      // ln2 low part
    float p = 1.9875691500e-4f;
    p = std::fmaf(p, r, 1.3981999507e-3f);
    p = std::fmaf(p, r, 8.3334519073e-3f);
    p = std::fmaf(p, r, 4.1665795894e-2f);
    p = std::fmaf(p, r, 1.6666665459e-1f);
    p = std::fmaf(p, r, 5.0000001201e-1f);
    const float z = r * r;
    float y = std::fmaf(p, z, r);
    y = y + 1.0f;
    const int ni = (int)n;
    const int n1 = ni >> 1, n2 = ni - n1;
    const float s1 = bits_to_float((uint32_t)(n1 + 127) << 23);
    const float s2 = bits_to_float((uint32_t)(n2 + 127) << 23);
    return (y * s1) * s2;
}

template <typename T>
inline T exp_sp(T x) {  // expf applied to a scalar_t argument, result widened back
    return (T)expf_fixed((float)x);
}
template <typename T>
inline T sigmoid_(T x) {  // _SIGMOID, rt_kernel.cu:87
    return T(1) / (T(1) + exp_sp<T>(-x));
}
template <typename T>
inline T softplus_m1(T x) {  // _SOFTPLUS_M1, rt_kernel.cu:86 (logf of a float argument)
    return (T)std::log((float)(T(1) + exp_sp<T>(x - T(1))));
}

template <typename T>
struct TreeView {
    T* data;
    const int32_t* child;
    const int32_t* parent_depth;
    const T* extra;
    T offset[3];
    T scaling[3];
    T* weight_accum;
    bool weight_accum_max;
    int64_t M;
    int N, K, extra_rows, extra_cols;
};

template <typename T>
TreeView<T> make_view(const SvoxTreeSpec* s) {
    TreeView<T> t;
    t.data = (T*)s->data;
    t.child = s->child;
    t.parent_depth = s->parent_depth;
    t.extra = (const T*)s->extra_data;
    for (int i = 0; i < 3; ++i) {
        t.offset[i] = s->offset ? ((const T*)s->offset)[i] : T(0);
        t.scaling[i] = s->scaling ? ((const T*)s->scaling)[i] : T(1);
    }
    t.weight_accum = (T*)s->weight_accum;
    t.weight_accum_max = s->weight_accum_max != 0;
    t.M = s->capacity;
    t.N = s->N;
    t.K = s->data_dim;
    t.extra_rows = s->extra_rows;
    t.extra_cols = s->extra_cols;
    return t;
}

// clamp_coord, common.cuh:36-41.  The upper bound 1 - 1e-6 is formed and compared in double and
// rounded when stored; fmin/fmax return the non-NaN operand, so NaN maps to the upper bound.
template <typename T>
inline void clamp_coord(T* q) {
    for (int i = 0; i < 3; ++i) {
        double v = std::fmin(1.0 - 1e-6, (double)q[i]);
        v = std::fmax(0.0, v);
        q[i] = (T)v;
    }
}

// transform_coord, common.cuh:43-50.
template <typename T>
inline void transform_coord(T* q, const T* offset, const T* scaling) {
    for (int i = 0; i < 3; ++i) q[i] = fma_(scaling[i], q[i], offset[i]);
}

// query_single_from_root, common.cuh:52-90.  Returns the packed leaf id
// node*N^3 + u*N^2 + v*N + w; xyz becomes the position inside the leaf in [0,1)^3, *cube_sz the
// number of leaf-sized cells per axis (N^levels).  Returns -1 if the walk exceeds 64 levels or
// leaves the node table (malformed tree) instead of looping forever.
template <typename T>
inline int64_t descend(const TreeView<T>& tr, T* xyz, T* cube_sz, int* levels_out) {
    const T N = (T)tr.N;
    clamp_coord(xyz);
    int64_t node = 0;
    *cube_sz = N;
    for (int level = 1; level <= 64; ++level) {
        xyz[0] *= N;
        xyz[1] *= N;
        xyz[2] *= N;
        const int32_t u = (int32_t)std::floor(xyz[0]);
        const int32_t v = (int32_t)std::floor(xyz[1]);
        const int32_t w = (int32_t)std::floor(xyz[2]);
        xyz[0] -= (T)u;
        xyz[1] -= (T)v;
        xyz[2] -= (T)w;
        const int64_t cell = ((node * tr.N + u) * tr.N + v) * tr.N + w;
        const int32_t skip = tr.child[cell];
        if (skip == 0) {
            if (levels_out) *levels_out = level;
            return cell;
        }
        *cube_sz *= N;
        node += skip;
        if (node < 0 || node >= tr.M) return -1;
    }
    return -1;
}

// _norm / _normalize / _dot3, rt_kernel.cu:89-108 (sqrtf: single precision in every build).
template <typename T>
inline T norm3(const T* d) {
    const T s = fma_(d[2], d[2], fma_(d[0], d[0], d[1] * d[1]));
    return (T)std::sqrt((float)s);
}
template <typename T>
inline T dot3(const T* u, const T* v) {
    return fma_(u[2], v[2], fma_(u[0], v[0], u[1] * v[1]));
}

const float kC0 = 0.28209479177387814f;
const float kC1 = 0.4886025119029199f;
const float kC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                      -1.0925484305920792f, 0.5462742152960396f};
const float kC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                      0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                      -0.5900435899266435f};
const float kC4[9] = {2.5033429417967046f, -1.7701307697799304f, 0.9461746957575601f,
                      -0.6690465435572892f, 0.10578554691520431f, -0.6690465435572892f,
                      0.47308734787878004f, -1.7701307697799304f, 0.6258357354491761f};

// maybe_precalc_basis, rt_kernel.cu:111-187.  Differences of products such as 3*xx - yy are
// fused on the left product; constants are single precision as in the reference's __constant__
// tables, integer literals take the scalar type, `2.0 * zz` and friends are evaluated in double.
template <typename T>
void precalc_basis(int format, int basis_dim, const T* extra, int extra_cols, const T* dir,
                   T* out) {
    if (format == SVOX_FORMAT_ASG) {
        for (int i = 0; i < basis_dim; ++i) {
            const T* p = extra + (int64_t)i * extra_cols;
            const T S = dot3(dir, p + 8);
            const T dx = dot3(dir, p + 2);
            const T dy = dot3(dir, p + 5);
            // -ptr[0]*dot_x*dot_x - ptr[1]*dot_y*dot_y : the left product is the fused one
            const T arg = fma_(-p[0] * dx, dx, -((p[1] * dy) * dy));
            out[i] = S * exp_sp<T>(arg) / (T)basis_dim;
        }
    } else if (format == SVOX_FORMAT_SG) {
        for (int i = 0; i < basis_dim; ++i) {
            const T* p = extra + (int64_t)i * extra_cols;
            out[i] = exp_sp<T>(p[0] * (dot3(dir, p + 1) - T(1))) / (T)basis_dim;
        }
    } else if (format == SVOX_FORMAT_SH) {
        out[0] = (T)kC0;
        const T x = dir[0], y = dir[1], z = dir[2];
        const T xx = x * x, yy = y * y, zz = z * z;
        const T xy = x * y, yz = y * z, xz = x * z;
        if (basis_dim == 25) {
            out[16] = (T)kC4[0] * xy * (xx - yy);
            out[17] = (T)kC4[1] * yz * fma_(T(3), xx, -yy);
            out[18] = (T)kC4[2] * xy * fma_(T(7), zz, T(-1));
            out[19] = (T)kC4[3] * yz * fma_(T(7), zz, T(-3));
            out[20] = (T)kC4[4] * fma_(zz, fma_(T(35), zz, T(-30)), T(3));
            out[21] = (T)kC4[5] * xz * fma_(T(7), zz, T(-3));
            out[22] = (T)kC4[6] * (xx - yy) * fma_(T(7), zz, T(-1));
            out[23] = (T)kC4[7] * xz * fma_(T(-3), yy, xx);
            out[24] = (T)kC4[8] * fma_(xx, fma_(T(-3), yy, xx), -(yy * fma_(T(3), xx, -yy)));
        }
        if (basis_dim == 25 || basis_dim == 16) {
            out[9] = (T)kC3[0] * y * fma_(T(3), xx, -yy);
            out[10] = (T)kC3[1] * xy * z;
            out[11] = (T)kC3[2] * y * (fma_(T(4), zz, -xx) - yy);
            out[12] = (T)kC3[3] * z * fma_(T(-3), yy, fma_(T(2), zz, -(T(3) * xx)));
            out[13] = (T)kC3[4] * x * (fma_(T(4), zz, -xx) - yy);
            out[14] = (T)kC3[5] * z * (xx - yy);
            out[15] = (T)kC3[6] * x * fma_(T(-3), yy, xx);
        }
        if (basis_dim == 25 || basis_dim == 16 || basis_dim == 9) {
            out[4] = (T)kC2[0] * xy;
            out[5] = (T)kC2[1] * yz;
            out[6] = (T)((double)kC2[2] * (std::fma(2.0, (double)zz, -(double)xx) - (double)yy));
            out[7] = (T)kC2[3] * xz;
            out[8] = (T)kC2[4] * (xx - yy);
        }
        if (basis_dim == 25 || basis_dim == 16 || basis_dim == 9 || basis_dim == 4) {
            out[1] = -(T)kC1 * y;
            out[2] = (T)kC1 * z;
            out[3] = -(T)kC1 * x;
        }
    }
}

// _get_delta_scale, rt_kernel.cu:189-201.
template <typename T>
inline T delta_scale_of(const T* scaling, T* dir) {
    dir[0] *= scaling[0];
    dir[1] *= scaling[1];
    dir[2] *= scaling[2];
    const T s = T(1) / norm3(dir);
    dir[0] *= s;
    dir[1] *= s;
    dir[2] *= s;
    return s;
}

// _dda_unit, rt_kernel.cu:203-220.  t1 is used by min/max as well as by the sum, so it stays a
// rounded product.
template <typename T>
inline void dda_unit(const T* cen, const T* invdir, T* tmin, T* tmax) {
    *tmin = T(0);
    *tmax = T(1e9f);
    for (int i = 0; i < 3; ++i) {
        const T t1 = -cen[i] * invdir[i];
        const T t2 = t1 + invdir[i];
        *tmin = std::fmax(*tmin, std::fmin(t1, t2));
        *tmax = std::fmin(*tmax, std::fmax(t1, t2));
    }
}

// t += delta_t.  Where t can no longer advance (delta below the spacing of floats at t, or NaN) the
// reference's `while (t < tmax)` never ends; the ray is ended after this sample instead (the one
// deliberate departure from the reference, shared with the kernels).
template <typename T>
inline T advance_t(T t, T delta_t, T tmax) {
    const T t_next = t + delta_t;
    return t_next > t ? t_next : tmax;
}

struct Counters {
    uint64_t rays = 0, rays_hit = 0, samples = 0, shaded = 0, bwd = 0, bwd_pos = 0, levels = 0, tail = 0;
};

struct LeafVisit {
    int64_t leaf;
    double t, delta_t, sigma;
};

template <typename T>
struct RaySetup {
    T origin[3], dir[3], invdir[3], basis[SVOX_MAX_BASIS_DIM];
    T delta_scale, tmin, tmax;
    bool hit;
};

// The part of trace_ray / trace_ray_backward before the march, rt_kernel.cu:228-255 / :331-354.
// `origin` is already in tree coordinates, `dir` is the caller's direction (scaled here).
template <typename T>
void setup_ray(const TreeView<T>& tr, const SvoxRenderOptions& opt, const T* origin, const T* dir,
               const T* vdir, RaySetup<T>* rs) {
    for (int i = 0; i < 3; ++i) {
        rs->origin[i] = origin[i];
        rs->dir[i] = dir[i];
    }
    rs->delta_scale = delta_scale_of(tr.scaling, rs->dir);
    for (int i = 0; i < 3; ++i) rs->invdir[i] = (T)(1.0 / ((double)rs->dir[i] + 1e-9));
    dda_unit(rs->origin, rs->invdir, &rs->tmin, &rs->tmax);
    rs->hit = !(rs->tmax < T(0) || rs->tmin > rs->tmax);
    if (rs->hit)
        precalc_basis(opt.format, opt.basis_dim, tr.extra, tr.extra_cols, vdir, rs->basis);
}

// trace_ray, rt_kernel.cu:222-321.
template <typename T>
void trace_ray(const TreeView<T>& tr, const SvoxRenderOptions& opt, const T* origin, const T* dir,
               const T* vdir, int out_dim, T* out, Counters* cnt, std::vector<LeafVisit>* visits) {
    RaySetup<T> rs;
    setup_ray(tr, opt, origin, dir, vdir, &rs);
    if (cnt) cnt->rays++;
    if (!rs.hit) {
        for (int j = 0; j < out_dim; ++j) out[j] = (T)opt.background_brightness;
        return;
    }
    if (cnt) cnt->rays_hit++;
    for (int j = 0; j < out_dim; ++j) out[j] = T(0);
    T light = T(1);
    T t = rs.tmin;
    const T step = (T)opt.step_size;
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    T pos[3];
    uint64_t since_shaded = 0;   // (statistics only: visits since the ray's last shaded leaf)
    while (t < rs.tmax) {
        for (int j = 0; j < 3; ++j) pos[j] = fma_(t, rs.dir[j], rs.origin[j]);
        T cube_sz;
        int levels = 0;
        const int64_t leaf = descend(tr, pos, &cube_sz, &levels);
        if (leaf < 0) {  // malformed tree
            if (cnt) cnt->tail += since_shaded;
            return;
        }
        const T* val = tr.data + leaf * tr.K;
        T s0, s1;
        dda_unit(pos, rs.invdir, &s0, &s1);
        const T t_subcube = (s1 - s0) / cube_sz;
        const T delta_t = t_subcube + step;
        T sigma = val[tr.K - 1];
        if (opt.density_softplus) sigma = softplus_m1(sigma);
        if (cnt) {
            cnt->samples++;
            cnt->levels += (uint64_t)levels;
        }
        since_shaded += 1;
        if (visits) visits->push_back({leaf, (double)t, (double)delta_t, (double)sigma});
        if (sigma > (T)opt.sigma_thresh) {
            if (cnt) cnt->shaded++;
            since_shaded = 0;
            const T att = exp_sp<T>(-delta_t * rs.delta_scale * sigma);
            const T weight = light * (T(1) - att);
            if (opt.format != SVOX_FORMAT_RGBA) {
                for (int c = 0; c < out_dim; ++c) {
                    const int off = c * opt.basis_dim;
                    T tmp = T(0);
                    for (int i = opt.min_comp; i <= opt.max_comp; ++i)
                        tmp = fma_(rs.basis[i], val[off + i], tmp);
                    out[c] = fma_(weight, fma_(sigmoid_(tmp), d_rgb_pad, -pad), out[c]);
                }
            } else {
                for (int c = 0; c < out_dim; ++c)
                    out[c] = fma_(weight, fma_(sigmoid_(val[c]), d_rgb_pad, -pad), out[c]);
            }
            light *= att;
            if (tr.weight_accum) {
                T* w = tr.weight_accum + leaf;
                if (tr.weight_accum_max) {
                    *w = (T)std::fmax((float)weight, (float)*w);  // atomicMax uses fmaxf, common.cuh:152-172
                } else {
                    *w += weight;
                }
            }
            if (light <= (T)opt.stop_thresh) {
                const T scale = (T)(1.0 / (1.0 - (double)light));
                for (int j = 0; j < out_dim; ++j) out[j] *= scale;
                return;
            }
        }
        t = advance_t(t, delta_t, rs.tmax);
    }
    if (cnt) cnt->tail += since_shaded;
    for (int j = 0; j < out_dim; ++j) out[j] = fma_(light, (T)opt.background_brightness, out[j]);
}

// trace_ray_backward, rt_kernel.cu:323-477.  Both passes test sigma > 0 and never stop early.
// `add(offset, value)` receives every atomicAdd of the reference in the reference's order.
template <typename T, typename Adder>
void trace_ray_backward(const TreeView<T>& tr, const SvoxRenderOptions& opt, const T* origin,
                        const T* dir, const T* vdir, int out_dim, const T* grad_out, Adder add,
                        Counters* cnt) {
    RaySetup<T> rs;
    setup_ray(tr, opt, origin, dir, vdir, &rs);
    if (!rs.hit) return;
    const T step = (T)opt.step_size;
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    T accum = T(0);
    T pos[3];
    // PASS 1, rt_kernel.cu:358-419
    {
        T light = T(1), t = rs.tmin;
        while (t < rs.tmax) {
            for (int j = 0; j < 3; ++j) pos[j] = fma_(t, rs.dir[j], rs.origin[j]);
            T cube_sz;
            const int64_t leaf = descend(tr, pos, &cube_sz, (int*)nullptr);
            if (leaf < 0) return;
            const int64_t base = leaf * tr.K;
            const T* val = tr.data + base;
            T s0, s1;
            dda_unit(pos, rs.invdir, &s0, &s1);
            const T delta_t = (s1 - s0) / cube_sz + step;
            T sigma = val[tr.K - 1];
            if (opt.density_softplus) sigma = softplus_m1(sigma);
            if (cnt) cnt->bwd++;
            if (sigma > T(0)) {
                if (cnt) cnt->bwd_pos++;
                const T att = exp_sp<T>(-delta_t * sigma * rs.delta_scale);
                const T weight = light * (T(1) - att);
                T total_color = T(0);
                if (opt.format != SVOX_FORMAT_RGBA) {
                    for (int c = 0; c < out_dim; ++c) {
                        const int off = c * opt.basis_dim;
                        T tmp = T(0);
                        for (int i = opt.min_comp; i <= opt.max_comp; ++i)
                            tmp = fma_(rs.basis[i], val[off + i], tmp);
                        const T sg = sigmoid_(tmp);
                        // weight * sigmoid * (1.0 - sigmoid) * grad * d_rgb_pad: the literal 1.0
                        // makes everything after weight*sigmoid double; rounded on store
                        const T tmp2 = (T)((double)(weight * sg) * (1.0 - (double)sg) *
                                           (double)grad_out[c] * (double)d_rgb_pad);
                        for (int i = opt.min_comp; i <= opt.max_comp; ++i)
                            add(base + off + i, rs.basis[i] * tmp2);
                        total_color = fma_(fma_(sg, d_rgb_pad, -pad), grad_out[c], total_color);
                    }
                } else {
                    for (int c = 0; c < out_dim; ++c) {
                        const T sg = sigmoid_(val[c]);
                        const T toadd = weight * sg * (T(1) - sg) * grad_out[c] * d_rgb_pad;
                        add(base + c, toadd);
                        total_color = fma_(fma_(sg, d_rgb_pad, -pad), grad_out[c], total_color);
                    }
                }
                light *= att;
                accum = fma_(weight, total_color, accum);
            }
            t = advance_t(t, delta_t, rs.tmax);
        }
        T total_grad = T(0);
        for (int j = 0; j < out_dim; ++j) total_grad += grad_out[j];
        accum = fma_(light * (T)opt.background_brightness, total_grad, accum);
    }
    // PASS 2, rt_kernel.cu:421-475
    {
        T light = T(1), t = rs.tmin;
        while (t < rs.tmax) {
            for (int j = 0; j < 3; ++j) pos[j] = fma_(t, rs.dir[j], rs.origin[j]);
            T cube_sz;
            const int64_t leaf = descend(tr, pos, &cube_sz, (int*)nullptr);
            if (leaf < 0) return;
            const int64_t base = leaf * tr.K;
            const T* val = tr.data + base;
            T s0, s1;
            dda_unit(pos, rs.invdir, &s0, &s1);
            const T delta_t = (s1 - s0) / cube_sz + step;
            T sigma = val[tr.K - 1];
            const T raw_sigma = sigma;
            if (opt.density_softplus) sigma = softplus_m1(sigma);
            if (sigma > T(0)) {
                const T att = exp_sp<T>(-delta_t * sigma * rs.delta_scale);
                const T weight = light * (T(1) - att);
                T total_color = T(0);
                if (opt.format != SVOX_FORMAT_RGBA) {
                    for (int c = 0; c < out_dim; ++c) {
                        const int off = c * opt.basis_dim;
                        T tmp = T(0);
                        for (int i = opt.min_comp; i <= opt.max_comp; ++i)
                            tmp = fma_(rs.basis[i], val[off + i], tmp);
                        total_color =
                            fma_(fma_(sigmoid_(tmp), d_rgb_pad, -pad), grad_out[c], total_color);
                    }
                } else {
                    for (int c = 0; c < out_dim; ++c)
                        total_color =
                            fma_(fma_(sigmoid_(val[c]), d_rgb_pad, -pad), grad_out[c], total_color);
                }
                light *= att;
                accum = fma_(-weight, total_color, accum);
                const T chain = opt.density_softplus ? sigmoid_(raw_sigma - T(1)) : T(1);
                add(base + tr.K - 1,
                    delta_t * rs.delta_scale * fma_(total_color, light, -accum) * chain);
            }
            t = advance_t(t, delta_t, rs.tmax);
        }
    }
}

// One sample of the squared-error marches (rt_kernel.cu:520-537 and the same lines of the later
// passes): position, leaf, step length, density.
template <typename T>
struct SeSample {
    int64_t leaf;
    T delta_t, sigma, raw_sigma;
};

template <typename T>
inline bool se_sample(const TreeView<T>& tr, const SvoxRenderOptions& opt, const RaySetup<T>& rs,
                      T t, SeSample<T>* s) {
    T pos[3];
    for (int j = 0; j < 3; ++j) pos[j] = fma_(t, rs.dir[j], rs.origin[j]);
    T cube_sz;
    s->leaf = descend(tr, pos, &cube_sz, (int*)nullptr);
    if (s->leaf < 0) return false;
    T s0, s1;
    dda_unit(pos, rs.invdir, &s0, &s1);
    s->delta_t = (s1 - s0) / cube_sz + (T)opt.step_size;
    s->raw_sigma = tr.data[s->leaf * tr.K + tr.K - 1];
    s->sigma = opt.density_softplus ? softplus_m1(s->raw_sigma) : s->raw_sigma;
    return true;
}

// sigmoid(basis . coefficients) of channel c of a leaf record (rt_kernel.cu:541-547)
template <typename T>
inline T channel_sigmoid(const SvoxRenderOptions& opt, const T* basis, const T* val, int c) {
    if (opt.format == SVOX_FORMAT_RGBA) return sigmoid_(val[c]);
    const int off = c * opt.basis_dim;
    T tmp = T(0);
    for (int i = opt.min_comp; i <= opt.max_comp; ++i) tmp = fma_(basis[i], val[off + i], tmp);
    return sigmoid_(tmp);
}

// trace_ray_se_grad_hess, rt_kernel.cu:479-715: rendered colour, gradient and Gauss-Newton Hessian
// diagonal of 0.5 * |render - color_ref|^2.  Three marches, all with sigma > 0 and no early stop.
// `add_grad` / `add_hess` receive the reference's atomicAdds in the reference's order.
// Note the two spellings of the attenuation argument: -delta_t * delta_scale * sigma in the first
// march (:538), -delta_t * sigma * delta_scale in the other two (:586, :653).
template <typename T, typename AddG, typename AddH>
void trace_ray_se_grad(const TreeView<T>& tr, const SvoxRenderOptions& opt, const T* origin,
                       const T* dir, const T* vdir, int out_dim, const T* color_ref, T* color_out,
                       AddG add_grad, AddH add_hess) {
    RaySetup<T> rs;
    setup_ray(tr, opt, origin, dir, vdir, &rs);
    if (!rs.hit) {
        for (int j = 0; j < out_dim; ++j) color_out[j] = (T)opt.background_brightness;
        return;
    }
    const T pad = (T)opt.rgb_padding;
    const T d_rgb_pad = (T)(1 + 2 * opt.rgb_padding);
    const T bg = (T)opt.background_brightness;
    SeSample<T> s;
    // PASS 1: residual, :516-566 (color_out arrives zero-filled)
    {
        T light = T(1), t = rs.tmin;
        while (t < rs.tmax) {
            if (!se_sample(tr, opt, rs, t, &s)) return;
            if (s.sigma > T(0)) {
                const T* val = tr.data + s.leaf * tr.K;
                const T att = exp_sp<T>(-s.delta_t * rs.delta_scale * s.sigma);
                const T weight = light * (T(1) - att);
                for (int c = 0; c < out_dim; ++c)
                    color_out[c] = fma_(weight, fma_(channel_sigmoid(opt, rs.basis, val, c), d_rgb_pad, -pad),
                                        color_out[c]);
                light *= att;
            }
            t = advance_t(t, s.delta_t, rs.tmax);
        }
        for (int j = 0; j < out_dim; ++j) color_out[j] += fma_(light, bg, -color_ref[j]);
    }
    // PASS 2: colour gradient and the rendered colour as a suffix sum, :568-637
    T color_accum[4] = {T(0), T(0), T(0), T(0)};
    {
        T light = T(1), t = rs.tmin;
        while (t < rs.tmax) {
            if (!se_sample(tr, opt, rs, t, &s)) return;
            if (s.sigma > T(0)) {
                const int64_t base = s.leaf * tr.K;
                const T* val = tr.data + base;
                const T att = exp_sp<T>(-s.delta_t * s.sigma * rs.delta_scale);
                const T weight = light * (T(1) - att);
                for (int c = 0; c < out_dim; ++c) {
                    const T sg = channel_sigmoid(opt, rs.basis, val, c);
                    if (opt.format != SVOX_FORMAT_RGBA) {
                        // `1.0 - sigmoid`: double from there on, rounded on store (:604-605)
                        const T grad_ci = (T)((double)(weight * sg) * (1.0 - (double)sg) * (double)d_rgb_pad);
                        const int off = c * opt.basis_dim;
                        for (int i = opt.min_comp; i <= opt.max_comp; ++i) {
                            const T grad_wi = rs.basis[i] * grad_ci;
                            add_grad(base + off + i, grad_wi * color_out[c]);
                            add_hess(base + off + i, grad_wi * grad_wi);
                        }
                    } else {
                        const T grad_ci = weight * sg * (T(1) - sg) * d_rgb_pad;
                        add_grad(base + c, grad_ci * color_out[c]);
                        add_hess(base + c, grad_ci * grad_ci);
                    }
                    color_accum[c] = fma_(weight, fma_(sg, d_rgb_pad, -pad), color_accum[c]);
                }
                light *= att;
            }
            t = advance_t(t, s.delta_t, rs.tmax);
        }
        for (int j = 0; j < out_dim; ++j) color_accum[j] = fma_(light, bg, color_accum[j]);
    }
    // PASS 3: density gradient, :639-708
    {
        T light = T(1), t = rs.tmin;
        T color_curr[4];
        while (t < rs.tmax) {
            if (!se_sample(tr, opt, rs, t, &s)) return;
            if (s.sigma > T(0)) {
                const int64_t base = s.leaf * tr.K;
                const T* val = tr.data + base;
                const T att = exp_sp<T>(-s.delta_t * s.sigma * rs.delta_scale);
                const T weight = light * (T(1) - att);
                for (int c = 0; c < out_dim; ++c) {
                    color_curr[c] = fma_(channel_sigmoid(opt, rs.basis, val, c), d_rgb_pad, -pad);
                    color_accum[c] = fma_(-weight, color_curr[c], color_accum[c]);
                }
                light *= att;
                for (int j = 0; j < out_dim; ++j) {
                    const T grad_sigma = s.delta_t * rs.delta_scale * fma_(color_curr[j], light, -color_accum[j]);
                    const T grad2_sigma = grad_sigma * grad_sigma;
                    if (opt.density_softplus) {
                        const T sg = sigmoid_(s.raw_sigma - T(1));
                        const T d_sg = sg * (T(1) - sg);
                        add_grad(base + tr.K - 1, grad_sigma * color_out[j] * sg);
                        add_hess(base + tr.K - 1, fma_(grad2_sigma * sg, sg, grad_sigma * d_sg));
                    } else {
                        add_grad(base + tr.K - 1, grad_sigma * color_out[j]);
                        add_hess(base + tr.K - 1, grad2_sigma);
                    }
                }
            }
            t = advance_t(t, s.delta_t, rs.tmax);
        }
    }
    // residual -> colour, :710-713
    for (int j = 0; j < out_dim; ++j) color_out[j] += color_ref[j];
}

// cam2world_ray, rt_kernel.cu:758-772.  x and y are formed in double (0.5 * width) and rounded;
// the radicand x*x + y*y is a scalar_t sum widened to double for `+ 1.0`, then sqrtf.
template <typename T>
void cam2world_ray(int ix, int iy, const T* c2w, float fx, float fy, int width, int height,
                   T* dir, T* origin) {
    T x = (T)(((double)ix - 0.5 * (double)width) / (double)fx);
    T y = (T)(-((double)iy - 0.5 * (double)height) / (double)fy);
    T z = (T)std::sqrt((float)((double)fma_(x, x, y * y) + 1.0));
    x /= z;
    y /= z;
    z = (T)(-1.0f / z);
    for (int r = 0; r < 3; ++r) {
        const T* row = c2w + r * 4;
        dir[r] = fma_(row[2], z, fma_(row[0], x, row[1] * y));
        origin[r] = row[3];
    }
}

// maybe_world2ndc, rt_kernel.cu:775-796 (near = 1).
template <typename T>
void maybe_world2ndc(const SvoxRenderOptions& opt, T* dir, T* cen) {
    if (opt.ndc_width < 0) return;
    const T near = T(1);
    const T t = -(near + cen[2]) / dir[2];
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

template <typename T>
void pixel_ray(const TreeView<T>& tr, const SvoxCameraSpec& cam, const SvoxRenderOptions& opt,
               int64_t pix, T* origin, T* dir, T* vdir) {
    // render_image_kernel, rt_kernel.cu:799-819
    const int iy = (int)(pix / cam.width), ix = (int)(pix % cam.width);
    cam2world_ray(ix, iy, (const T*)cam.c2w, cam.fx, cam.fy, cam.width, cam.height, dir, origin);
    for (int i = 0; i < 3; ++i) vdir[i] = dir[i];
    maybe_world2ndc(opt, dir, origin);
    transform_coord(origin, tr.offset, tr.scaling);
}

template <typename T>
void batch_ray(const TreeView<T>& tr, const SvoxRaysSpec& rays, int64_t r, T* origin, T* dir,
               T* vdir) {
    // render_ray_kernel, rt_kernel.cu:717-733
    for (int i = 0; i < 3; ++i) {
        origin[i] = ((const T*)rays.origins)[r * 3 + i];
        dir[i] = ((const T*)rays.dirs)[r * 3 + i];
        vdir[i] = ((const T*)rays.vdirs)[r * 3 + i];
    }
    transform_coord(origin, tr.offset, tr.scaling);
}

void merge(SvoxMarchStats* dst, const Counters& c) {
    dst->rays += c.rays;
    dst->rays_hit += c.rays_hit;
    dst->samples += c.samples;
    dst->samples_shaded += c.shaded;
    dst->samples_bwd += c.bwd;
    dst->samples_bwd_pos += c.bwd_pos;
    dst->levels += c.levels;
    dst->samples_tail += c.tail;
}

int check_render_args(const SvoxTreeSpec* tree, const SvoxRenderOptions* opt) {
    if (!tree || !opt || !tree->data || !tree->child) return SVOX_ERR_NULL_POINTER;
    if (tree->dtype != SVOX_F32 && tree->dtype != SVOX_F64) return SVOX_ERR_BAD_DTYPE;
    const int od = oracle_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    if (od < 0 || od > SVOX_MAX_OUT_DIM) return SVOX_ERR_BAD_SHAPE;
    if (opt->format != SVOX_FORMAT_RGBA &&
        (opt->basis_dim > SVOX_MAX_BASIS_DIM || opt->max_comp >= opt->basis_dim || opt->min_comp < 0))
        return SVOX_ERR_BAD_SHAPE;
    return SVOX_OK;
}

template <typename T>
int render_impl(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxCameraSpec* cam,
                const SvoxRenderOptions* opt, void* out_v, SvoxMarchStats* stats, int n_threads) {
    const TreeView<T> tr = make_view<T>(tree);
    const int od = oracle_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    const int64_t n = rays ? rays->n_rays : (int64_t)cam->width * cam->height;
    T* out = (T*)out_v;
    Counters total;
    // weight accumulation writes shared leaves: keep it serial
    if (tr.weight_accum) n_threads = 1;
#pragma omp parallel num_threads(n_threads > 0 ? n_threads : 1)
    {
        Counters local;
#pragma omp for schedule(dynamic, 256)
        for (int64_t r = 0; r < n; ++r) {
            T origin[3], dir[3], vdir[3];
            if (rays)
                batch_ray(tr, *rays, r, origin, dir, vdir);
            else
                pixel_ray(tr, *cam, *opt, r, origin, dir, vdir);
            trace_ray(tr, *opt, origin, dir, vdir, od, out + r * od, stats ? &local : nullptr,
                      (std::vector<LeafVisit>*)nullptr);
        }
#pragma omp critical
        {
            total.rays += local.rays;
            total.rays_hit += local.rays_hit;
            total.samples += local.samples;
            total.shaded += local.shaded;
            total.levels += local.levels;
            total.tail += local.tail;
        }
    }
    if (stats) merge(stats, total);
    return SVOX_OK;
}

// Destination of the reference's atomicAdds.  Plain: dst[off] += v in the scalar type, in the order the
// calls arrive (an OpenMP atomic when several threads add).  Exact: the terms are added in double
// into a zero-initialised side buffer (untouched pages are never committed) and finish() adds the
// rounded sums to dst.
template <typename T>
struct SumBuffer {
    T* dst;
    T* slack;                  // optional output of the exact mode: sqrt(n) * u * sum |term| per element
    double* wide = nullptr;
    double* wide_abs = nullptr;
    uint32_t* terms = nullptr;
    int64_t n;
    bool par;
    SumBuffer(T* dst_, int64_t n_, bool exact, bool par_, T* slack_ = nullptr)
        : dst(dst_), slack(exact ? slack_ : nullptr), n(n_), par(par_) {
        if (exact) wide = (double*)std::calloc((size_t)n_, sizeof(double));
        if (slack) {
            wide_abs = (double*)std::calloc((size_t)n_, sizeof(double));
            terms = (uint32_t*)std::calloc((size_t)n_, sizeof(uint32_t));
        }
    }
    SumBuffer(const SumBuffer&) = delete;
    ~SumBuffer() {
        std::free(wide);
        std::free(wide_abs);
        std::free(terms);
    }
    bool failed(bool exact) const { return (exact && !wide) || (slack && (!wide_abs || !terms)); }
    inline void add(int64_t off, T v) const {
        if (slack) {
            const double a = std::fabs((double)v);
            if (par) {
#pragma omp atomic
                wide_abs[off] += a;
#pragma omp atomic
                terms[off] += 1u;
            } else {
                wide_abs[off] += a;
                terms[off] += 1u;
            }
        }
        if (wide) {
            if (par) {
#pragma omp atomic
                wide[off] += (double)v;
            } else {
                wide[off] += (double)v;
            }
        } else if (par) {
#pragma omp atomic
            dst[off] += v;
        } else {
            dst[off] += v;
        }
    }
    void finish() const {
        if (!wide) return;
#pragma omp parallel for schedule(static) if (par)
        for (int64_t i = 0; i < n; ++i)
            if (wide[i] != 0.0) dst[i] = (T)((double)dst[i] + wide[i]);
        if (!slack) return;
        const double u = 0.5 * (double)std::numeric_limits<T>::epsilon();
#pragma omp parallel for schedule(static) if (par)
        for (int64_t i = 0; i < n; ++i) slack[i] = (T)(std::sqrt((double)terms[i]) * u * wide_abs[i]);
    }
};

template <typename T>
int render_backward_impl(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                         const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                         const void* grad_out_v, void* grad_data_v, int accumulate,
                         SvoxMarchStats* stats, int n_threads, int exact_sum, void* slack_v) {
    const TreeView<T> tr = make_view<T>(tree);
    const int od = oracle_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    const int64_t n = rays ? rays->n_rays : (int64_t)cam->width * cam->height;
    const T* grad_out = (const T*)grad_out_v;
    T* grad = (T*)grad_data_v;
    const int64_t total_elems = tr.M * tr.N * tr.N * tr.N * tr.K;
    if (!accumulate) std::memset(grad, 0, sizeof(T) * (size_t)total_elems);
    Counters total;
    const bool par = n_threads > 1;
    const SumBuffer<T> sum(grad, total_elems, exact_sum != 0, par, (T*)slack_v);
    if (sum.failed(exact_sum != 0)) return SVOX_ERR_BAD_SHAPE;
#pragma omp parallel num_threads(n_threads > 0 ? n_threads : 1)
    {
        Counters local;
#pragma omp for schedule(dynamic, 256)
        for (int64_t r = 0; r < n; ++r) {
            T origin[3], dir[3], vdir[3];
            if (rays)
                batch_ray(tr, *rays, r, origin, dir, vdir);
            else
                pixel_ray(tr, *cam, *opt, r, origin, dir, vdir);
            trace_ray_backward(
                tr, *opt, origin, dir, vdir, od, grad_out + r * od,
                [&sum](int64_t off, T v) { sum.add(off, v); }, stats ? &local : nullptr);
        }
#pragma omp critical
        {
            total.bwd += local.bwd;
            total.bwd_pos += local.bwd_pos;
        }
    }
    sum.finish();
    if (stats) merge(stats, total);
    return SVOX_OK;
}

// grid_trace_ray + grid_weight_render_kernel, rt_kernel.cu:898-1003: march through a dense
// reso^3 density grid; per visited cell with sigma > sigma_thresh the largest compositing weight any
// ray gave it (atomicMax) and the number of such visits.
template <typename T>
int grid_weight_impl(const void* data_v, int reso, const SvoxCameraSpec* cam,
                     const SvoxRenderOptions* opt, const void* offset_v, const void* scaling_v,
                     void* weight_v, void* hit_v) {
    const T* data = (const T*)data_v;
    T* grid_weight = (T*)weight_v;
    T* grid_hit = (T*)hit_v;
    const size_t cells = (size_t)reso * reso * reso;
    std::memset(grid_weight, 0, sizeof(T) * cells);
    std::memset(grid_hit, 0, sizeof(T) * cells);
    TreeView<T> tr{};   // only the transform is used
    for (int i = 0; i < 3; ++i) {
        tr.offset[i] = ((const T*)offset_v)[i];
        tr.scaling[i] = ((const T*)scaling_v)[i];
    }
    const int64_t n = (int64_t)cam->width * cam->height;
    for (int64_t pix = 0; pix < n; ++pix) {
        T origin[3], dir[3], vdir[3];
        pixel_ray(tr, *cam, *opt, pix, origin, dir, vdir);
        const T delta_scale = delta_scale_of(tr.scaling, dir);
        T invdir[3], tmin, tmax;
        for (int i = 0; i < 3; ++i) invdir[i] = (T)(1.0 / ((double)dir[i] + 1e-9));
        dda_unit(origin, invdir, &tmin, &tmax);
        if (tmax < T(0) || tmin > tmax) continue;
        T light = T(1), t = tmin;
        const T cube_sz = (T)reso;
        while (t < tmax) {
            T pos[3];
            for (int j = 0; j < 3; ++j) pos[j] = fma_(t, dir[j], origin[j]);
            clamp_coord(pos);
            int32_t uvw[3];
            for (int j = 0; j < 3; ++j) {
                pos[j] *= (T)reso;
                uvw[j] = (int32_t)std::floor(pos[j]);
                pos[j] -= (T)uvw[j];
            }
            const int32_t node_id = uvw[0] * reso * reso + uvw[1] * reso + uvw[2];
            T s0, s1;
            dda_unit(pos, invdir, &s0, &s1);
            const T delta_t = (s1 - s0) / cube_sz + (T)opt->step_size;
            const T sigma = data[node_id];
            if (sigma > (T)opt->sigma_thresh) {
                const T att = exp_sp<T>(-delta_t * delta_scale * sigma);
                const T weight = light * (T(1) - att);
                light *= att;
                grid_weight[node_id] = (T)std::fmax((float)weight, (float)grid_weight[node_id]);
                grid_hit[node_id] += T(1);
            }
            t = advance_t(t, delta_t, tmax);
        }
    }
    return SVOX_OK;
}

// se_grad / se_grad_persp, rt_kernel.cu:1111-1173
template <typename T>
int se_grad_impl(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxCameraSpec* cam,
                 const SvoxRenderOptions* opt, const void* color_ref_v, void* color_out_v,
                 void* grad_v, void* hess_v, int n_threads, int exact_sum, void* grad_slack_v,
                 void* hess_slack_v) {
    const TreeView<T> tr = make_view<T>(tree);
    const int od = oracle_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    if (od > 4) return SVOX_ERR_BAD_SHAPE;  // "Tree's output dim cannot be > 4 for se_grad"
    const int64_t n = rays ? rays->n_rays : (int64_t)cam->width * cam->height;
    const T* ref = (const T*)color_ref_v;
    T* out = (T*)color_out_v;
    T* grad = (T*)grad_v;
    T* hess = (T*)hess_v;
    const int64_t total_elems = tr.M * tr.N * tr.N * tr.N * tr.K;
    std::memset(grad, 0, sizeof(T) * (size_t)total_elems);
    std::memset(hess, 0, sizeof(T) * (size_t)total_elems);
    std::memset(out, 0, sizeof(T) * (size_t)(n * od));
    const bool par = n_threads > 1;
    const SumBuffer<T> grad_sum(grad, total_elems, exact_sum != 0, par, (T*)grad_slack_v),
        hess_sum(hess, total_elems, exact_sum != 0, par, (T*)hess_slack_v);
    if (grad_sum.failed(exact_sum != 0) || hess_sum.failed(exact_sum != 0)) return SVOX_ERR_BAD_SHAPE;
#pragma omp parallel for schedule(dynamic, 256) num_threads(n_threads > 0 ? n_threads : 1)
    for (int64_t r = 0; r < n; ++r) {
        T origin[3], dir[3], vdir[3];
        if (rays)
            batch_ray(tr, *rays, r, origin, dir, vdir);
        else
            pixel_ray(tr, *cam, *opt, r, origin, dir, vdir);
        trace_ray_se_grad(tr, *opt, origin, dir, vdir, od, ref + r * od, out + r * od,
                          [&grad_sum](int64_t off, T v) { grad_sum.add(off, v); },
                          [&hess_sum](int64_t off, T v) { hess_sum.add(off, v); });
    }
    grad_sum.finish();
    hess_sum.finish();
    return SVOX_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// C interface (host pointers everywhere; same structs as the device library)
// ------------------------------------------------------------------------------------------------
extern "C" {

// get_out_data_dim, rt_kernel.cu:1009-1015
int oracle_out_data_dim(int32_t format, int32_t basis_dim, int32_t data_dim) {
    if (data_dim < 1) return -1;
    if (format != SVOX_FORMAT_RGBA) {
        if (basis_dim <= 0) return -1;
        return (data_dim - 1) / basis_dim;
    }
    return data_dim - 1;
}

float oracle_expf(float x) { return expf_fixed(x); }

float oracle_sigmoid(float x) { return sigmoid_<float>(x); }

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// basis functions for one direction; out has basis_dim entries of `dtype`
int oracle_basis(int32_t format, int32_t basis_dim, const void* extra, int32_t extra_cols,
                 const void* dir, void* out, int32_t dtype) {
    if (basis_dim > SVOX_MAX_BASIS_DIM) return SVOX_ERR_BAD_SHAPE;
    if (dtype == SVOX_F32)
        precalc_basis<float>(format, basis_dim, (const float*)extra, extra_cols, (const float*)dir,
                             (float*)out);
    else
        precalc_basis<double>(format, basis_dim, (const double*)extra, extra_cols,
                              (const double*)dir, (double*)out);
    return SVOX_OK;
}

// query_single_kernel + query_vertical, svox_kernel.cu:42-66, 120-143.
// levels_out (optional, int32 per point) receives the number of child entries read.
int oracle_query_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                          void* values_out, int64_t* node_ids_out, int32_t* levels_out) {
    if (!tree || !tree->data || !tree->child) return SVOX_ERR_NULL_POINTER;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const TreeView<T> tr = make_view<T>(tree);
        const T* idx = (const T*)indices;
        T* vals = (T*)values_out;
        for (int64_t q = 0; q < n_points; ++q) {
            T xyz[3] = {idx[q * 3], idx[q * 3 + 1], idx[q * 3 + 2]};
            transform_coord(xyz, tr.offset, tr.scaling);
            T cube;
            int levels = 0;
            const int64_t leaf = descend(tr, xyz, &cube, &levels);
            if (leaf < 0) return (int)SVOX_ERR_BAD_SHAPE;
            if (vals)
                for (int i = 0; i < tr.K; ++i) vals[q * tr.K + i] = tr.data[leaf * tr.K + i];
            if (node_ids_out) node_ids_out[q] = leaf;
            if (levels_out) levels_out[q] = levels;
        }
        return (int)SVOX_OK;
    };
    return tree->dtype == SVOX_F32 ? run(float()) : run(double());
}

// query_single_kernel_backward + query_vertical_backward, svox_kernel.cu:68-78, 160-182
int oracle_query_vertical_backward(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                                   const void* grad_output, int32_t grad_dim, void* grad_data_out,
                                   int32_t accumulate) {
    if (!tree || !tree->child || !grad_data_out) return SVOX_ERR_NULL_POINTER;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const TreeView<T> tr = make_view<T>(tree);
        const T* idx = (const T*)indices;
        const T* go = (const T*)grad_output;
        T* gd = (T*)grad_data_out;
        const int64_t cells = tr.M * tr.N * tr.N * tr.N;
        if (!accumulate) std::memset(gd, 0, sizeof(T) * (size_t)(cells * grad_dim));
        for (int64_t q = 0; q < n_points; ++q) {
            T xyz[3] = {idx[q * 3], idx[q * 3 + 1], idx[q * 3 + 2]};
            transform_coord(xyz, tr.offset, tr.scaling);
            T cube;
            const int64_t leaf = descend(tr, xyz, &cube, (int*)nullptr);
            if (leaf < 0) return (int)SVOX_ERR_BAD_SHAPE;
            for (int i = 0; i < grad_dim; ++i) gd[leaf * grad_dim + i] += go[q * grad_dim + i];
        }
        return (int)SVOX_OK;
    };
    return tree->dtype == SVOX_F32 ? run(float()) : run(double());
}

// assign_single_kernel + assign_vertical, svox_kernel.cu:80-89, 145-158 (points in order, so the
// last point written to a leaf wins)
int oracle_assign_vertical(const SvoxTreeSpec* tree, const void* indices, int64_t n_points,
                           const void* values, int32_t value_dim) {
    if (!tree || !tree->data || !tree->child) return SVOX_ERR_NULL_POINTER;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const TreeView<T> tr = make_view<T>(tree);
        const T* idx = (const T*)indices;
        const T* v = (const T*)values;
        for (int64_t q = 0; q < n_points; ++q) {
            T xyz[3] = {idx[q * 3], idx[q * 3 + 1], idx[q * 3 + 2]};
            transform_coord(xyz, tr.offset, tr.scaling);
            T cube;
            const int64_t leaf = descend(tr, xyz, &cube, (int*)nullptr);
            if (leaf < 0) return (int)SVOX_ERR_BAD_SHAPE;
            for (int i = 0; i < value_dim; ++i) tr.data[leaf * tr.K + i] = v[q * value_dim + i];
        }
        return (int)SVOX_OK;
    };
    return tree->dtype == SVOX_F32 ? run(float()) : run(double());
}

// calc_corner_kernel + calc_corners, svox_kernel.cu:91-115, 184-203
int oracle_calc_corners(const SvoxTreeSpec* tree, const int64_t* indexer, int64_t n_leaves,
                        void* corners_out) {
    if (!tree || !tree->parent_depth || !corners_out) return SVOX_ERR_NULL_POINTER;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const int N = tree->N;
        T* out = (T*)corners_out;
        for (int64_t q = 0; q < n_leaves; ++q) {
            int32_t curr[4] = {(int32_t)indexer[q * 4], (int32_t)indexer[q * 4 + 1],
                               (int32_t)indexer[q * 4 + 2], (int32_t)indexer[q * 4 + 3]};
            T res[3] = {T(0), T(0), T(0)};
            for (int guard = 0; guard < 64; ++guard) {
                for (int i = 0; i < 3; ++i) {
                    res[i] += (T)curr[i + 1];
                    res[i] /= (T)N;
                }
                if (curr[0] == 0) break;
                curr[0] = tree->parent_depth[(int64_t)curr[0] * 2];
                for (int i = 3; i > 0; --i) {
                    curr[i] = curr[0] % N;
                    curr[0] /= N;
                }
            }
            for (int i = 0; i < 3; ++i) out[q * 3 + i] = res[i];
        }
        return (int)SVOX_OK;
    };
    return tree->dtype == SVOX_F32 ? run(float()) : run(double());
}

// volume_render, rt_kernel.cu:1019-1036
int oracle_volume_render(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                         const SvoxRenderOptions* opt, void* out, SvoxMarchStats* stats,
                         int32_t n_threads) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!rays || !out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? render_impl<float>(tree, rays, nullptr, opt, out, stats, n_threads)
               : render_impl<double>(tree, rays, nullptr, opt, out, stats, n_threads);
}

// volume_render_image, rt_kernel.cu:1038-1057 (cam->c2w is a host pointer here)
int oracle_volume_render_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                               const SvoxRenderOptions* opt, void* out, SvoxMarchStats* stats,
                               int32_t n_threads) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!cam || !cam->c2w || !out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? render_impl<float>(tree, nullptr, cam, opt, out, stats, n_threads)
               : render_impl<double>(tree, nullptr, cam, opt, out, stats, n_threads);
}

// volume_render_backward, rt_kernel.cu:1059-1083
int oracle_volume_render_backward(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays,
                                  const SvoxRenderOptions* opt, const void* grad_output,
                                  void* grad_data_out, int32_t accumulate, SvoxMarchStats* stats,
                                  int32_t n_threads, int32_t exact_sum, void* slack_out) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!rays || !grad_output || !grad_data_out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? render_backward_impl<float>(tree, rays, nullptr, opt, grad_output, grad_data_out,
                                             accumulate, stats, n_threads, exact_sum, slack_out)
               : render_backward_impl<double>(tree, rays, nullptr, opt, grad_output, grad_data_out,
                                              accumulate, stats, n_threads, exact_sum, slack_out);
}

// volume_render_image_backward, rt_kernel.cu:1085-1109
int oracle_volume_render_image_backward(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                                        const SvoxRenderOptions* opt, const void* grad_output,
                                        void* grad_data_out, int32_t accumulate,
                                        SvoxMarchStats* stats, int32_t n_threads, int32_t exact_sum,
                                        void* slack_out) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!cam || !cam->c2w || !grad_output || !grad_data_out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? render_backward_impl<float>(tree, nullptr, cam, opt, grad_output, grad_data_out,
                                             accumulate, stats, n_threads, exact_sum, slack_out)
               : render_backward_impl<double>(tree, nullptr, cam, opt, grad_output, grad_data_out,
                                              accumulate, stats, n_threads, exact_sum, slack_out);
}

// se_grad, rt_kernel.cu:1111-1139: color_ref and color_out are (B, C); grad and hessdiag have the
// shape of tree.data and are zero-filled here.
int oracle_se_grad(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, const SvoxRenderOptions* opt,
                   const void* color_ref, void* color_out, void* grad_out, void* hessdiag_out,
                   int32_t n_threads, int32_t exact_sum, void* grad_slack_out, void* hess_slack_out) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!rays || !color_ref || !color_out || !grad_out || !hessdiag_out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? se_grad_impl<float>(tree, rays, nullptr, opt, color_ref, color_out, grad_out, hessdiag_out, n_threads, exact_sum,
                                     grad_slack_out, hess_slack_out)
               : se_grad_impl<double>(tree, rays, nullptr, opt, color_ref, color_out, grad_out, hessdiag_out, n_threads, exact_sum,
                                     grad_slack_out, hess_slack_out);
}

// se_grad_persp, rt_kernel.cu:1141-1173: color_ref and color_out are (H, W, C)
int oracle_se_grad_image(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                         const SvoxRenderOptions* opt, const void* color_ref, void* color_out,
                         void* grad_out, void* hessdiag_out, int32_t n_threads, int32_t exact_sum,
                         void* grad_slack_out, void* hess_slack_out) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    if (!cam || !cam->c2w || !color_ref || !color_out || !grad_out || !hessdiag_out) return SVOX_ERR_NULL_POINTER;
    return tree->dtype == SVOX_F32
               ? se_grad_impl<float>(tree, nullptr, cam, opt, color_ref, color_out, grad_out, hessdiag_out, n_threads, exact_sum,
                                     grad_slack_out, hess_slack_out)
               : se_grad_impl<double>(tree, nullptr, cam, opt, color_ref, color_out, grad_out, hessdiag_out, n_threads, exact_sum,
                                     grad_slack_out, hess_slack_out);
}

// grid_weight_render, rt_kernel.cu:1174-1203.  data, grid_weight_out and grid_hit_out are
// (reso, reso, reso); offset and scaling are 3 scalars each.
int oracle_grid_weight_render(const void* data, int32_t reso, int32_t dtype,
                              const SvoxCameraSpec* cam, const SvoxRenderOptions* opt,
                              const void* offset, const void* scaling, void* grid_weight_out,
                              void* grid_hit_out) {
    if (!data || !cam || !cam->c2w || !opt || !offset || !scaling || !grid_weight_out || !grid_hit_out)
        return SVOX_ERR_NULL_POINTER;
    if (reso < 1 || reso > 1290) return SVOX_ERR_BAD_SHAPE;   // int32 cell ids
    return dtype == SVOX_F32
               ? grid_weight_impl<float>(data, reso, cam, opt, offset, scaling, grid_weight_out, grid_hit_out)
               : grid_weight_impl<double>(data, reso, cam, opt, offset, scaling, grid_weight_out, grid_hit_out);
}

// The rays the image kernels trace, after cam2world / NDC / world->tree: origins, dirs, vdirs are
// (H*W, 3) of tree->dtype.  Lets tests pin rt_kernel.cu:758-796 on their own.
int oracle_image_rays(const SvoxTreeSpec* tree, const SvoxCameraSpec* cam,
                      const SvoxRenderOptions* opt, void* origins, void* dirs, void* vdirs) {
    if (!tree || !cam || !cam->c2w || !opt) return SVOX_ERR_NULL_POINTER;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const TreeView<T> tr = make_view<T>(tree);
        const int64_t n = (int64_t)cam->width * cam->height;
        for (int64_t p = 0; p < n; ++p)
            pixel_ray(tr, *cam, *opt, p, (T*)origins + p * 3, (T*)dirs + p * 3, (T*)vdirs + p * 3);
        return (int)SVOX_OK;
    };
    return tree->dtype == SVOX_F32 ? run(float()) : run(double());
}

// The leaf sequence of one ray of a batch: up to `max_visits` rows of
// (packed leaf id, t, delta_t, sigma); returns the number of visits (or a negative status).
int64_t oracle_trace_visits(const SvoxTreeSpec* tree, const SvoxRaysSpec* rays, int64_t ray_index,
                            const SvoxRenderOptions* opt, int64_t* leaf_out, double* t_out,
                            double* delta_out, double* sigma_out, int64_t max_visits) {
    const int rc = check_render_args(tree, opt);
    if (rc) return rc;
    std::vector<LeafVisit> visits;
    const int od = oracle_out_data_dim(opt->format, opt->basis_dim, tree->data_dim);
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const TreeView<T> tr = make_view<T>(tree);
        T origin[3], dir[3], vdir[3], out[SVOX_MAX_OUT_DIM];
        batch_ray(tr, *rays, ray_index, origin, dir, vdir);
        trace_ray(tr, *opt, origin, dir, vdir, od, out, (Counters*)nullptr, &visits);
    };
    if (tree->dtype == SVOX_F32)
        run(float());
    else
        run(double());
    const int64_t n = (int64_t)visits.size();
    for (int64_t i = 0; i < n && i < max_visits; ++i) {
        if (leaf_out) leaf_out[i] = visits[i].leaf;
        if (t_out) t_out[i] = visits[i].t;
        if (delta_out) delta_out[i] = visits[i].delta_t;
        if (sigma_out) sigma_out[i] = visits[i].sigma;
    }
    return n;
}

}  // extern "C"
