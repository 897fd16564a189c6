// tg_components.hip -- host-side scalar hooks: barycentric coordinates and the
// perspective-weighted interpolation with their hand-derived backward formulas.
//
// The reference exports these from its extension as CPU functions so that its
// component tests can gradcheck them (src/trigrad/tests.cu:43-76 around
// util.h:232-250, 299-355, 395-455).  They run on the host, take host pointers
// and mirror the arithmetic the backward kernels use on the device.
#include <cfloat>
#include <cmath>
#include <limits>

#include "../../include/trigrad_hip.h"

namespace {

using real = tg_real;  // the scalar type of the build

constexpr real kTiny = std::numeric_limits<real>::min();  // util.h:24

inline real cross2(real ax, real ay, real bx, real by) { return ax * by - ay * bx; }  // util.h:384-388

inline void bary_of(const real *v0, const real *v1, const real *v2, const real *p, real out[3]) {
    const real T = cross2(v1[0] - v0[0], v1[1] - v0[1], v2[0] - v0[0], v2[1] - v0[1]);
    out[0] = cross2(v1[0] - p[0], v1[1] - p[1], v2[0] - p[0], v2[1] - p[1]) / T;
    out[1] = cross2(v2[0] - p[0], v2[1] - p[1], v0[0] - p[0], v0[1] - p[1]) / T;
    out[2] = cross2(v0[0] - p[0], v0[1] - p[1], v1[0] - p[0], v1[1] - p[1]) / T;
}

}  // namespace

// util.h:395-403 barycentric(v0, v1, v2, p) -> 3 coordinates.
extern "C" void tg_barycentric(const real *v0, const real *v1, const real *v2, const real *p, real *out) {
    bary_of(v0, v1, v2, p, out);
}

// util.h:405-455 barycentric_backward: grads (4 x 2, rows v0, v1, v2, p) of sum(g * bary).
extern "C" void tg_barycentric_backward(const real *g, const real *a, const real *b, const real *c, const real *p,
                                        real *grads) {
    real l[3];
    bary_of(a, b, c, p, l);
    const real ax = a[0], ay = a[1], bx = b[0], by = b[1], cx = c[0], cy = c[1], px = p[0], py = p[1];
    const real d = ax * (by - cy) + bx * (-ay + cy) + cx * (ay - by);
    if (std::fabs(d) < kTiny) {
        for (int i = 0; i < 8; i++) grads[i] = 0.0f;
        return;
    }
    // J[row][axis][k] = d bary_k / d row.axis
    const real J[4][2][3] = {
        {{l[0] * (-by + cy) / d, (-cy - l[1] * (by - cy) + py) / d, (by - l[2] * (by - cy) - py) / d},
         {l[0] * (bx - cx) / d, (cx + l[1] * (bx - cx) - px) / d, (-bx + l[2] * (bx - cx) + px) / d}},
        {{(cy + l[0] * (ay - cy) - py) / d, l[1] * (ay - cy) / d, (-ay + l[2] * (ay - cy) + py) / d},
         {(-cx - l[0] * (ax - cx) + px) / d, l[1] * (-ax + cx) / d, (ax - l[2] * (ax - cx) - px) / d}},
        {{(-by - l[0] * (ay - by) + py) / d, (ay - l[1] * (ay - by) - py) / d, l[2] * (-ay + by) / d},
         {(bx + l[0] * (ax - bx) - px) / d, (-ax + l[1] * (ax - bx) + px) / d, l[2] * (ax - bx) / d}},
        {{(by - cy) / d, (-ay + cy) / d, (ay - by) / d}, {(-bx + cx) / d, (ax - cx) / d, (-ax + bx) / d}},
    };
    for (int r = 0; r < 4; r++)
        for (int ax_ = 0; ax_ < 2; ax_++) grads[2 * r + ax_] = g[0] * J[r][ax_][0] + g[1] * J[r][ax_][1] + g[2] * J[r][ax_][2];
}

// util.h:245-250 scalar interpolate3 with weights.
extern "C" real tg_interpolate3_scalar(const real *bary, real a, real b, real c, const real *w) {
    const real denom = bary[0] * w[0] + bary[1] * w[1] + bary[2] * w[2];
    return (bary[0] * a * w[0] + bary[1] * b * w[1] + bary[2] * c * w[2]) / denom;
}

// util.h:299-317.  Outputs: grad_bary[3], grad_values[3] (a, b, c), grad_w[3].
extern "C" void tg_interpolate3_scalar_backward(real g, const real *bary, real a, real b, real c, const real *w,
                                                real *grad_bary, real *grad_values, real *grad_w) {
    const real v[3] = {a, b, c};
    const real nom = (bary[0] * w[0] * v[0] + bary[1] * w[1] * v[1]) + bary[2] * w[2] * v[2];
    const real denom = (bary[0] * w[0] + bary[1] * w[1]) + bary[2] * w[2];
    if (denom * denom < kTiny) {
        for (int k = 0; k < 3; k++) grad_bary[k] = grad_values[k] = grad_w[k] = 0.0f;
        return;
    }
    const real inv2 = 1.0f / (denom * denom);
    for (int k = 0; k < 3; k++) {
        grad_bary[k] = g * ((v[k] * w[k] * denom - nom * w[k]) * inv2);
        grad_values[k] = g * bary[k] * w[k] / denom;
        grad_w[k] = g * (bary[k] * v[k] * denom - nom * bary[k]) * inv2;
    }
}

// util.h:232-237 vector interpolate3 with weights (3 components).
extern "C" void tg_interpolate3_vector(const real *bary, const real *a, const real *b, const real *c, const real *w,
                                       real *out) {
    const real denom = bary[0] * w[0] + bary[1] * w[1] + bary[2] * w[2];
    for (int k = 0; k < 3; k++) out[k] = (bary[0] * a[k] * w[0] + bary[1] * b[k] * w[1] + bary[2] * c[k] * w[2]) / denom;
}

// util.h:319-355.  Outputs: grad_bary[3], grad_a[3], grad_b[3], grad_c[3], grad_w[3].
extern "C" void tg_interpolate3_vector_backward(const real *g, const real *bary, const real *a, const real *b,
                                                const real *c, const real *w, real *grad_bary, real *grad_a,
                                                real *grad_b, real *grad_c, real *grad_w) {
    const real *v[3] = {a, b, c};
    real nom[3];
    for (int k = 0; k < 3; k++) nom[k] = (bary[0] * w[0] * a[k] + bary[1] * w[1] * b[k]) + bary[2] * w[2] * c[k];
    const real denom = bary[0] * w[0] + bary[1] * w[1] + bary[2] * w[2];
    if (denom * denom < kTiny) {
        for (int k = 0; k < 3; k++) grad_bary[k] = grad_a[k] = grad_b[k] = grad_c[k] = grad_w[k] = 0.0f;
        return;
    }
    const real inv2 = (real)(1.0 / (double)(denom * denom));
    for (int i = 0; i < 3; i++) {
        real dfb[3], dfw[3];
        for (int k = 0; k < 3; k++) {
            dfb[k] = w[i] * (v[i][k] * denom - nom[k]) * inv2;
            dfw[k] = (bary[i] * v[i][k] * denom - nom[k] * bary[i]) * inv2;
        }
        grad_bary[i] = (g[0] * dfb[0] + g[1] * dfb[1]) + g[2] * dfb[2];
        grad_w[i] = (g[0] * dfw[0] + g[1] * dfw[1]) + g[2] * dfw[2];
    }
    const real scale[3] = {bary[0] * w[0] / denom, bary[1] * w[1] / denom, bary[2] * w[2] / denom};
    for (int k = 0; k < 3; k++) {
        grad_a[k] = g[k] * scale[0];
        grad_b[k] = g[k] * scale[1];
        grad_c[k] = g[k] * scale[2];
    }
}
