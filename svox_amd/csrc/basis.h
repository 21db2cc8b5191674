// basis.h -- view-dependent basis functions (reference: maybe_precalc_basis,
// svox/csrc/rt_kernel.cu:111-187; constants :53-83).
#pragma once

#include "fpmath.h"
#include "../../include/svox_hip.h"

namespace svox {

// Real spherical harmonics up to degree 4 in the reference's order and sign convention
// (out[1] = -C1*y, out[2] = C1*z, out[3] = -C1*x).  The direction is used as given, not
// normalised.  Constants are single precision as in the reference's tables; integer literals take
// the scalar type; `2.0 * zz - xx - yy` is evaluated in double.  basis_dim outside {1,4,9,16,25}
// fills only out[0], as the reference's fall-through switch does.
template <typename T>
__device__ __forceinline__ void sh_basis(int basis_dim, const T* dir, T* out) {
    const T C0 = (T)0.28209479177387814f;
    const T C1 = (T)0.4886025119029199f;
    out[0] = C0;
    const T x = dir[0], y = dir[1], z = dir[2];
    const T xx = x * x, yy = y * y, zz = z * z;
    const T xy = x * y, yz = y * z, xz = x * z;
    if (basis_dim == 25) {
        out[16] = (T)2.5033429417967046f * xy * (xx - yy);
        out[17] = (T)-1.7701307697799304f * yz * fma_(T(3), xx, -yy);
        out[18] = (T)0.9461746957575601f * xy * fma_(T(7), zz, T(-1));
        out[19] = (T)-0.6690465435572892f * yz * fma_(T(7), zz, T(-3));
        out[20] = (T)0.10578554691520431f * fma_(zz, fma_(T(35), zz, T(-30)), T(3));
        out[21] = (T)-0.6690465435572892f * xz * fma_(T(7), zz, T(-3));
        out[22] = (T)0.47308734787878004f * (xx - yy) * fma_(T(7), zz, T(-1));
        out[23] = (T)-1.7701307697799304f * xz * fma_(T(-3), yy, xx);
        out[24] = (T)0.6258357354491761f *
                  fma_(xx, fma_(T(-3), yy, xx), -(yy * fma_(T(3), xx, -yy)));
    }
    if (basis_dim == 25 || basis_dim == 16) {
        out[9] = (T)-0.5900435899266435f * y * fma_(T(3), xx, -yy);
        out[10] = (T)2.890611442640554f * xy * z;
        out[11] = (T)-0.4570457994644658f * y * (fma_(T(4), zz, -xx) - yy);
        out[12] = (T)0.3731763325901154f * z * fma_(T(-3), yy, fma_(T(2), zz, -(T(3) * xx)));
        out[13] = (T)-0.4570457994644658f * x * (fma_(T(4), zz, -xx) - yy);
        out[14] = (T)1.445305721320277f * z * (xx - yy);
        out[15] = (T)-0.5900435899266435f * x * fma_(T(-3), yy, xx);
    }
    if (basis_dim == 25 || basis_dim == 16 || basis_dim == 9) {
        out[4] = (T)1.0925484305920792f * xy;
        out[5] = (T)-1.0925484305920792f * yz;
        out[6] = (T)((double)0.31539156525252005f *
                     (__builtin_fma(2.0, (double)zz, -(double)xx) - (double)yy));
        out[7] = (T)-1.0925484305920792f * xz;
        out[8] = (T)0.5462742152960396f * (xx - yy);
    }
    if (basis_dim == 25 || basis_dim == 16 || basis_dim == 9 || basis_dim == 4) {
        out[1] = -C1 * y;
        out[2] = C1 * z;
        out[3] = -C1 * x;
    }
}

// Any format.  `extra` is the (basis_dim, extra_cols) table of lobes for SG ([lambda, mu]) and
// ASG ([lambda_x, lambda_y, x-axis, y-axis, z-axis]).
template <typename T>
__device__ __forceinline__ void precalc_basis(int format, int basis_dim, const T* extra,
                                              int extra_cols, const T* dir, T* out) {
    if (format == SVOX_FORMAT_SH) {
        sh_basis<T>(basis_dim, dir, out);
    } else if (format == SVOX_FORMAT_SG) {
        for (int i = 0; i < basis_dim; ++i) {
            const T* p = extra + (int64_t)i * extra_cols;
            out[i] = exp_sp<T>(p[0] * (dot3(dir, p + 1) - T(1))) / (T)basis_dim;
        }
    } else if (format == SVOX_FORMAT_ASG) {
        for (int i = 0; i < basis_dim; ++i) {
            const T* p = extra + (int64_t)i * extra_cols;
            const T S = dot3(dir, p + 8);
            const T dx = dot3(dir, p + 2);
            const T dy = dot3(dir, p + 5);
            const T arg = fma_(-p[0] * dx, dx, -((p[1] * dy) * dy));
            out[i] = S * exp_sp<T>(arg) / (T)basis_dim;
        }
    }
}

}  // namespace svox
