// Device-side scalar math of the splat path (gfx950). Compiled with -ffp-contract=off: positions,
// depths and sizes feed integer decisions (pixel, layer, sort key), so every expression below is
// evaluated exactly in the order written, with IEEE single-precision operations.
//
// Reference lines restated here (paths relative to the reference checkout):
//   softplus / derivative     src/lib/rendering/RenderForward.cu:154-159, RenderBackward.cu:71-83
//   layer factor              src/lib/rendering/PointBlending.h:81-149
//   bilinear weights          src/lib/rendering/PointBlending.h:211-264
//   pinhole projection        src/lib/rendering/PointRendererHelper.h:232-253, RenderForward.cu:69-76,302-303
//   projection backward       src/lib/rendering/PointRendererHelper.h:434-494
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#pragma clang fp contract(off)

namespace trips
{
constexpr float kAlphaDestCutoff = 0.001f;  // ALPHA_DEST_CUTOFF, RenderForward.cu:907

// exp / log evaluated in double and rounded once, so that results do not depend on a libm's float path
__device__ __forceinline__ float exp_rn(float x) { return (float)exp((double)x); }
__device__ __forceinline__ float log_rn(float x) { return (float)log((double)x); }

__device__ __forceinline__ float softplus(float x)
{
    if (x > 20.f) return x;
    return log_rn(1.f + exp_rn(x));
}

__device__ __forceinline__ float softplus_backward(float y)
{
    if (y > 20.f) return 1.f;
    float z = exp_rn(y);
    return z / (z + 1.f);
}

// both at once, with the one exponential that they share (same bits as the two functions above)
__device__ __forceinline__ float softplus_and_derivative(float x, float* derivative)
{
    if (x > 20.f)
    {
        *derivative = 1.f;
        return x;
    }
    const float z = exp_rn(x);
    *derivative   = z / (z + 1.f);
    return log_rn(1.f + z);
}

// floor(log2 s), ceil(log2 s) for finite s > 0 from the bit pattern (exact; the reference rounds log2f first)
__device__ __forceinline__ void log2_floor_ceil(float s, int& lo, int& hi)
{
    uint32_t u   = __float_as_uint(s);
    int e        = int((u >> 23) & 0xff);
    uint32_t man = u & 0x7fffffu;
    if (e == 0)
    {
        lo = -127;
        hi = -126;
        return;
    }
    lo = e - 127;
    hi = lo + (man != 0 ? 1 : 0);
}

// compute_point_size_fac (PointBlending.h:81-149) for s > 1 and more than one layer, the branch that interpolates
// between two layers; written with selects only. (The other branch, 0.75 exp(s - 1) + 0.25 for a point that lands
// in layer 0 only, is evaluated once per point by encode_size_field below.)
// Between two layers the reference divides by 2^higher - 2^lower, which is 2^lower whenever the two differ (then
// neither is clamped): multiplying by 2^-lower instead gives the same bits, the scaling being exact.
__device__ __forceinline__ float layer_factor_interpolated(float s, int layer, int max_layers, float* grad)
{
    int lo, hi;
    log2_floor_ceil(s, lo, hi);  // lo >= 0 as s > 1
    const int layer_lower = min(lo, max_layers - 1), layer_higher = min(hi, max_layers - 1);
    const float l_l = __uint_as_float((uint32_t)(127 + layer_lower) << 23);  // 2^lower
    const float inv = __uint_as_float((uint32_t)(127 - layer_lower) << 23);  // 2^-lower
    float f         = (s - l_l) * inv;
    float J         = inv;
    if (layer == layer_lower)
    {
        f = 1.f - f;
        J = -J;
    }
    if (layer_lower == layer_higher)
    {
        f = 1.f;
        J = 1.f;
    }
    if (layer < layer_lower)
    {
        f = 1.f;
        J = 0.f;
    }
    if (grad) *grad = J;
    return f;
}

// The "small point" branch of the layer factor (layer_higher == 0, i.e. size <= 1 pixel or a single layer) is the
// only one that needs exp(), and it does not depend on the layer (such a point lands in layer 0 only). The
// projection kernel evaluates it once per point and stores it NEGATED in the size slot of the per-point record;
// the blend and the backward then read the factor instead of re-evaluating a double-precision exp per list entry.
__device__ __forceinline__ float encode_size_field(float size_px, int max_layers)
{
    const bool small_branch = !(size_px > 1.f) || max_layers == 1;
    return small_branch ? -(0.75f * exp_rn(size_px - 1.f) + 0.25f) : size_px;
}

// layer factor from the encoded size field
__device__ __forceinline__ float layer_factor_encoded(float field, int layer, int max_layers)
{
    if (field < 0.f) return -field;
    return layer_factor_interpolated(field, layer, max_layers, nullptr);
}

// same with the reference's gradient; true_size is the un-encoded projected size
__device__ __forceinline__ float layer_factor_encoded_grad(float field, float true_size, int layer, int max_layers,
                                                           float* grad)
{
    if (field < 0.f)
    {
        *grad = 0.27591f * true_size;
        return -field;
    }
    return layer_factor_interpolated(field, layer, max_layers, grad);
}

// alpha of a list entry (r0: the first four floats of its point's blend record) at pixel (gx, gy) of `layer`
// (RenderForward.cu:875-899: bilinear weight x confidence x layer factor)
__device__ __forceinline__ float entry_alpha(const float4& r0, int layer, int num_layers, int gx, int gy)
{
    const float m  = __uint_as_float((uint32_t)(127 - layer) << 23);  // 2^-layer
    const float ux = r0.x * m, uy = r0.y * m;
    float w        = (1.f - fabsf(ux - float(gx))) * (1.f - fabsf(uy - float(gy)));
    if (fabsf(ux - float(gx)) > 1.f || fabsf(uy - float(gy)) > 1.f) w = 0.f;
    float a = w * r0.w;
    a *= layer_factor_encoded(r0.z, layer, num_layers);
    return a;
}

struct Pose
{
    float qx, qy, qz, qw, tx, ty, tz;
};

// Sophus::SE3d memory (quaternion xyzw, translation, pad) cast to float (RenderConstants.h:88)
__device__ __forceinline__ Pose load_pose(const double* p)
{
    Pose P;
    P.qx = (float)p[0];
    P.qy = (float)p[1];
    P.qz = (float)p[2];
    P.qw = (float)p[3];
    P.tx = (float)p[4];
    P.ty = (float)p[5];
    P.tz = (float)p[6];
    return P;
}

// SE3f * point; rotation in the form of Eigen's QuaternionBase::_transformVector
__device__ __forceinline__ void transform_point(const Pose& V, float px, float py, float pz, float out[3])
{
    float ux = V.qy * pz - V.qz * py;
    float uy = V.qz * px - V.qx * pz;
    float uz = V.qx * py - V.qy * px;
    ux += ux;
    uy += uy;
    uz += uz;
    float cx = V.qy * uz - V.qz * uy;
    float cy = V.qz * ux - V.qx * uz;
    float cz = V.qx * uy - V.qy * ux;
    out[0]   = (px + V.qw * ux + cx) + V.tx;
    out[1]   = (py + V.qw * uy + cy) + V.ty;
    out[2]   = (pz + V.qw * uz + cz) + V.tz;
}

// Eigen's QuaternionBase::toRotationMatrix, row-major
__device__ __forceinline__ void rotation_matrix(const Pose& V, float R[9])
{
    float tx = 2.f * V.qx, ty = 2.f * V.qy, tz = 2.f * V.qz;
    float twx = tx * V.qw, twy = ty * V.qw, twz = tz * V.qw;
    float txx = tx * V.qx, txy = ty * V.qx, txz = tz * V.qx;
    float tyy = ty * V.qy, tyz = tz * V.qy, tzz = tz * V.qz;
    R[0]      = 1.f - (tyy + tzz);
    R[1]      = txy - twz;
    R[2]      = txz + twy;
    R[3]      = txy + twz;
    R[4]      = 1.f - (txx + tzz);
    R[5]      = tyz - twx;
    R[6]      = txz - twy;
    R[7]      = tyz + twx;
    R[8]      = 1.f - (txx + tyy);
}

// 8-parameter distortion (k1..k6 rational radial, p1 p2 tangential) of Saiga's distortNormalizedPoint,
// sentinel (100000,100000) beyond the cut-off radius. Jp: 2x2 row-major, Jd: 2x8 row-major; may be nullptr.
__device__ __forceinline__ void distort(float x, float y, const float* c, float cutoff, float& xd, float& yd,
                                        float* Jp, float* Jd)
{
    float k1 = c[0], k2 = c[1], k3 = c[2], k4 = c[3], k5 = c[4], k6 = c[5], p1 = c[6], p2 = c[7];
    float x2 = x * x, y2 = y * y;
    float r2 = x2 + y2, _2xy = 2.f * x * y;
    float r4 = r2 * r2, r6 = r4 * r2;
    float U   = 1.f + k1 * r2 + k2 * r4 + k3 * r6;
    float Vv  = 1.f + k4 * r2 + k5 * r4 + k6 * r6;
    float iV  = 1.f / Vv;
    float rad = U * iV;
    float tX  = p1 * _2xy + p2 * (r2 + 2.f * x2);
    float tY  = p1 * (r2 + 2.f * y2) + p2 * _2xy;
    xd        = x * rad + tX;
    yd        = y * rad + tY;
    if (Jp)
    {
        float dU   = k1 + 2.f * k2 * r2 + 3.f * k3 * r4;
        float dV   = k4 + 2.f * k5 * r2 + 3.f * k6 * r4;
        float drad = (dU * Vv - U * dV) * iV * iV;
        Jp[0]      = rad + x * drad * 2.f * x + (2.f * p1 * y + 6.f * p2 * x);
        Jp[1]      = x * drad * 2.f * y + (2.f * p1 * x + 2.f * p2 * y);
        Jp[2]      = y * drad * 2.f * x + (2.f * p1 * x + 2.f * p2 * y);
        Jp[3]      = rad + y * drad * 2.f * y + (6.f * p1 * y + 2.f * p2 * x);
    }
    if (Jd)
    {
        float uv2 = U * iV * iV;
        Jd[0]     = x * r2 * iV;
        Jd[1]     = x * r4 * iV;
        Jd[2]     = x * r6 * iV;
        Jd[3]     = -x * uv2 * r2;
        Jd[4]     = -x * uv2 * r4;
        Jd[5]     = -x * uv2 * r6;
        Jd[6]     = _2xy;
        Jd[7]     = r2 + 2.f * x2;
        Jd[8]     = y * r2 * iV;
        Jd[9]     = y * r4 * iV;
        Jd[10]    = y * r6 * iV;
        Jd[11]    = -y * uv2 * r2;
        Jd[12]    = -y * uv2 * r4;
        Jd[13]    = -y * uv2 * r6;
        Jd[14]    = r2 + 2.f * y2;
        Jd[15]    = _2xy;
    }
    if (r2 > cutoff * cutoff)
    {
        xd = 100000.f;
        yd = 100000.f;
        if (Jp) Jp[0] = Jp[1] = Jp[2] = Jp[3] = 0.f;
        if (Jd)
            for (int i = 0; i < 16; ++i) Jd[i] = 0.f;
    }
}

// Camera constants of one view, gathered once per thread from uniform memory.
struct Camera
{
    Pose V;
    float fx, fy, cx, cy, s;
    float dist[8];
    bool no_distortion;            // all of dist[] are zero (wave-uniform: the forward then skips the rational model)
    float cfx, cfy, ccx, ccy, cs;  // crop transform
    float r00, r01, r10, r11;      // crop rotation
    float centre_x, centre_y;      // float(w/2), float(h/2), integer division
    float dist_cutoff;
};

struct Projected
{
    float ipx, ipy, z, scale;  // scale = K.fx * crop.fx (divide by z after multiplying with a radius)
    float vx, vy, vz;          // view-space point
};

__device__ __forceinline__ Projected project(const Camera& cam, float px, float py, float pz)
{
    float view[3];
    transform_point(cam.V, px, py, pz, view);
    float z  = fmaxf(view[2], 0.f);
    float iz = 1.f / view[2];
    float nx = view[0] * iz, ny = view[1] * iz;
    float dx, dy;
    if (cam.no_distortion)
    {
        // all eight coefficients are zero: the model is x * (1 / 1) + 0 in float arithmetic, which is x + 0 (the
        // addition turns a negative zero into a positive one, as the full expression does); the cut-off stays
        dx = nx + 0.f;
        dy = ny + 0.f;
        if (nx * nx + ny * ny > cam.dist_cutoff * cam.dist_cutoff) dx = dy = 100000.f;
    }
    else
        distort(nx, ny, cam.dist, cam.dist_cutoff, dx, dy, nullptr, nullptr);
    if (dx == 100000.f) z = 0.f;
    float ix = cam.fx * dx + cam.s * dy + cam.cx;
    float iy = cam.fy * dy + cam.cy;
    float jx = cam.cfx * ix + cam.cs * iy + cam.ccx;
    float jy = cam.cfy * iy + cam.ccy;
    jx -= cam.centre_x;
    jy -= cam.centre_y;
    float rx = cam.r00 * jx + cam.r01 * jy;
    float ry = cam.r10 * jx + cam.r11 * jy;
    Projected P;
    P.ipx   = rx + cam.centre_x;
    P.ipy   = ry + cam.centre_y;
    P.z     = z;
    P.scale = cam.fx * cam.cfx;
    P.vx    = view[0];
    P.vy    = view[1];
    P.vz    = view[2];
    return P;
}

// image-space gradient (g0,g1) -> point (3), pose (6), K (5), distortion (8); view-space point given
__device__ __forceinline__ void project_backward(const Camera& cam, const float R[9], float vx, float vy, float vz,
                                                 float g0, float g1, float g_point[3], float g_pose[6], float g_k[5],
                                                 float g_dis[8], bool want_intrinsics)
{
    float iz = 1.f / vz, iz2 = 1.f / (vz * vz);
    float nx = vx * iz, ny = vy * iz;
    float Jp[4], Jd[16];
    float dx, dy;
    distort(nx, ny, cam.dist, cam.dist_cutoff, dx, dy, Jp, Jd);  // a pointer chosen at run time would put the arrays in scratch memory
    float gr0 = cam.r00 * g0 + cam.r10 * g1;
    float gr1 = cam.r01 * g0 + cam.r11 * g1;
    float a   = cam.cfx * gr0;
    float b   = cam.cs * gr0 + cam.cfy * gr1;
    float k0  = cam.fx * a;
    float k1  = cam.s * a + cam.fy * b;
    float d0  = Jp[0] * k0 + Jp[2] * k1;
    float d1  = Jp[1] * k0 + Jp[3] * k1;
    float v0  = iz * d0;
    float v1  = iz * d1;
    float v2  = (-vx * iz2) * d0 + (-vy * iz2) * d1;
    g_point[0] = R[0] * v0 + R[3] * v1 + R[6] * v2;
    g_point[1] = R[1] * v0 + R[4] * v1 + R[7] * v2;
    g_point[2] = R[2] * v0 + R[5] * v1 + R[8] * v2;
    g_pose[0]  = v0;
    g_pose[1]  = v1;
    g_pose[2]  = v2;
    g_pose[3]  = vy * v2 - vz * v1;
    g_pose[4]  = vz * v0 - vx * v2;
    g_pose[5]  = vx * v1 - vy * v0;
    if (want_intrinsics)
    {
        g_k[0] = dx * a;
        g_k[1] = dy * b;
        g_k[2] = a;
        g_k[3] = b;
        g_k[4] = dy * a;
        for (int i = 0; i < 8; ++i) g_dis[i] = Jd[i] * k0 + Jd[8 + i] * k1;
    }
}

// saturating float -> int (what v_cvt_i32_f32 does); NaN -> 0
__device__ __forceinline__ int trunc_sat(float v)
{
    if (!(v == v)) return 0;
    if (v >= 2147483648.f) return 2147483647;
    if (v <= -2147483648.f) return -2147483647 - 1;
    return (int)v;
}

}  // namespace trips
