/*
 * trips_oracle.cpp -- CPU oracle of the TRIPS trilinear point-splat path.
 *
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may load it. It restates, in plain loops, what the reference's CUDA path computes;
 * each function names the reference lines it follows (paths relative to the reference checkout).
 *
 * Build: g++ -O3 -march=native -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off matters: positions, depths and sizes feed integer decisions (pixel, layer,
 * sort key), so the operation order written here is the contract the device kernels repeat.
 *
 * Deliberate positions on ambiguities of the reference (none can be settled by running it):
 *  - sort order: ascending 64-bit key (depth bits << 32 | point id); the reference compares depth
 *    only (RenderForward.cu:464-467) and leaves ties to atomic slot order.
 *  - floor/ceil of log2(size) are taken from the float's exponent/mantissa (exact), where the
 *    reference rounds log2f() first (RenderForward.cu:345, PointBlending.h:83-90); they differ only
 *    for sizes a few ulp above a power of two.
 *  - expf/logf are evaluated in double and rounded once, so CPU and GPU agree bit for bit.
 *  - empty pixel = background * 1; every pixel is written exactly once (reference: RenderForward.cu:1002-1003
 *    reads a neighbour lane for empty lists and re-writes stale pixels at the queue tail).
 *  - backward decodes pixels with the forward's layer sizes (reference halves with floor,
 *    RenderBackward.cu:112-130, which disagrees with PointRenderer.cu:385-388 for odd sizes).
 *  - distortNormalizedPoint, TransformPoint, DivideByZ and normalizedToImage live in the un-vendored
 *    Saiga submodule; they are restated from their call sites and the published model
 *    (k1..k6 rational radial + p1,p2 tangential). Non-zero distortion is PARITY UNPINNED; with zero
 *    coefficients the model is the identity in float arithmetic.
 *
 * What pins the oracle is listed per test in tests/test_oracle_*.py (closed forms, brute force,
 * finite differences in f64, torch-CPU autograd, torch.optim.Adam, scipy expm).
 */
#include "trips_oracle.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <omp.h>
#include <vector>

namespace
{
constexpr float kAlphaDestCutoff = 0.001f;  // ALPHA_DEST_CUTOFF, RenderForward.cu:907

inline uint32_t f2u(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}

// float -> int conversion that saturates like the GPU's cvt instruction instead of being undefined
inline int trunc_sat(float v)
{
    if (!(v == v)) return 0;
    if (v >= 2147483648.f) return 2147483647;
    if (v <= -2147483648.f) return -2147483647 - 1;
    return (int)v;
}

// expf / logf evaluated in double, rounded once to float.
inline float exp_rn(float x) { return (float)std::exp((double)x); }
inline float log_rn(float x) { return (float)std::log((double)x); }

// _softplus, RenderForward.cu:154-159 (beta = 1, threshold = 20)
inline float softplus(float x)
{
    if (x > 20.f) return x;
    return log_rn(1.f + exp_rn(x));
}

// _softplus_backwards, RenderBackward.cu:71-83
inline float softplus_backward(float y)
{
    if (y > 20.f) return 1.f;
    float z = exp_rn(y);
    return z / (z + 1.f);
}

// floor(log2 s) and ceil(log2 s) for finite s > 0, from the bit pattern.
inline void log2_floor_ceil(float s, int& lo, int& hi)
{
    uint32_t u   = f2u(s);
    int e        = int((u >> 23) & 0xff);
    uint32_t man = u & 0x7fffffu;
    if (e == 0)
    {
        // subnormal: far below 1, callers only ask for s > 1
        lo = -127;
        hi = -126;
        return;
    }
    lo = e - 127;
    hi = lo + (man != 0 ? 1 : 0);
}

// compute_point_size_fac, PointBlending.h:81-149
inline float layer_factor(float s, int layer, int max_layers, float* grad)
{
    int layer_lower = 0, layer_higher = 0;
    if (s > 1.f)
    {
        int lo, hi;
        log2_floor_ceil(s, lo, hi);
        layer_lower  = std::min(std::max(0, lo), max_layers - 1);
        layer_higher = std::min(std::max(0, hi), max_layers - 1);
    }
    if (layer < layer_lower)
    {
        if (grad) *grad = 0.f;
        return 1.f;
    }
    float f = 1.f;
    if (layer_higher == 0)
    {
        // small point (PointBlending.h:99-107); the gradient is the reference's constant, not d/ds
        f = 0.75f * exp_rn(s - 1.f) + 0.25f;
        if (grad) *grad = 0.27591f * s;
    }
    else if (layer_lower == layer_higher)
    {
        if (grad) *grad = 1.f;
    }
    else
    {
        float l_l = float(1 << layer_lower);
        float l_h = float(1 << layer_higher);
        f         = (s - l_l) / (l_h - l_l);
        if (layer == layer_lower) f = 1.f - f;
        if (grad)
        {
            float J = 1.f / (l_h - l_l);
            if (layer == layer_lower) J = -J;
            *grad = J;
        }
        if (layer_lower == max_layers - 1)
        {
            f = 1.f;
            if (grad) *grad = 1.f;
        }
    }
    return f;
}

struct Pose
{
    float qx, qy, qz, qw, tx, ty, tz;
};

// Sophus::SE3d -> SE3f cast (RenderConstants.h:88); memory = quaternion xyzw, translation, pad
inline Pose load_pose(const double* p)
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

// GetPointWoNormal (NeuralPointCloudCuda.h:240-273): xyz of the point, plus view b's displacement when the scene
// optimises one (PointRenderer.cu:703-713); .w is the drop-out radius
struct PointPos
{
    float v[4];
    operator const float*() const { return v; }
};
inline PointPos load_point(const TripsSplatIn* in, int N, int b, int pid)
{
    PointPos p;
    const float* src = in->position + 4 * int64_t(pid);
    for (int k = 0; k < 4; ++k) p.v[k] = src[k];
    if (in->displacement)
    {
        const float* dsp = in->displacement + (int64_t(b) * N + pid) * 3;
        for (int k = 0; k < 3; ++k) p.v[k] += dsp[k];
    }
    return p;
}

// SE3f * point. Rotation as Eigen's QuaternionBase::_transformVector does it:
//   uv = 2 * (q.vec x v);  v' = v + w * uv + q.vec x uv
inline void transform_point(const Pose& V, const float p[3], float out[3])
{
    float ux = V.qy * p[2] - V.qz * p[1];
    float uy = V.qz * p[0] - V.qx * p[2];
    float uz = V.qx * p[1] - V.qy * p[0];
    ux += ux;
    uy += uy;
    uz += uz;
    float cx = V.qy * uz - V.qz * uy;
    float cy = V.qz * ux - V.qx * uz;
    float cz = V.qx * uy - V.qy * ux;
    out[0]   = (p[0] + V.qw * ux + cx) + V.tx;
    out[1]   = (p[1] + V.qw * uy + cy) + V.ty;
    out[2]   = (p[2] + V.qw * uz + cz) + V.tz;
}

// Eigen's QuaternionBase::toRotationMatrix, row-major R[9]
inline void rotation_matrix(const Pose& V, float R[9])
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

struct Distorted
{
    float x, y;
    bool cut;
};

// distortNormalizedPoint (Saiga, un-vendored): 8-parameter model k1..k6, p1, p2; returns the sentinel
// (100000, 100000) beyond the cut-off radius (checked by PointRendererHelper.h:246-249).
// Optional Jacobians: Jp = d(xd,yd)/d(x,y) row-major 2x2, Jd = d(xd,yd)/d(coeffs) row-major 2x8.
inline Distorted distort(float x, float y, const float* c, float cutoff, float* Jp, float* Jd)
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
    Distorted d;
    d.x   = x * rad + tX;
    d.y   = y * rad + tY;
    d.cut = false;
    if (Jp)
    {
        float dU   = k1 + 2.f * k2 * r2 + 3.f * k3 * r4;
        float dV   = k4 + 2.f * k5 * r2 + 3.f * k6 * r4;
        float drad = (dU * Vv - U * dV) * iV * iV;  // d rad / d r2
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
        d.x   = 100000.f;
        d.y   = 100000.f;
        d.cut = true;
        if (Jp) Jp[0] = Jp[1] = Jp[2] = Jp[3] = 0.f;
        if (Jd)
            for (int i = 0; i < 16; ++i) Jd[i] = 0.f;
    }
    return d;
}

struct Projected
{
    float ipx, ipy, z, scale;  // scale = K.fx * crop.fx / z
};

// ProjectPointPinholeWoNormal (PointRendererHelper.h:232-253) + crop transform and rotation
// (RenderForward.cu:302-303, rotateCropAroundCenter :69-76)
inline Projected project(const Pose& V, const float* intr, const TripsView& cam, float dist_cutoff, const float p[3])
{
    float view[3];
    transform_point(V, p, view);
    float z  = std::fmax(view[2], 0.f);
    float iz = 1.f / view[2];  // DivideByZ
    float nx = view[0] * iz, ny = view[1] * iz;
    Distorted d = distort(nx, ny, intr + 5, dist_cutoff, nullptr, nullptr);
    if (d.x == 100000.f) z = 0.f;
    float fx = intr[0], fy = intr[1], cx = intr[2], cy = intr[3], s = intr[4];
    float ix = fx * d.x + s * d.y + cx;  // IntrinsicsPinhole::normalizedToImage
    float iy = fy * d.y + cy;
    const float* c = cam.crop_transform;
    float jx       = c[0] * ix + c[4] * iy + c[2];
    float jy       = c[1] * iy + c[3];
    float ccx = float(cam.w / 2), ccy = float(cam.h / 2);  // integer division, RenderForward.cu:303
    jx -= ccx;
    jy -= ccy;
    float rx = cam.crop_rotation[0] * jx + cam.crop_rotation[1] * jy;
    float ry = cam.crop_rotation[2] * jx + cam.crop_rotation[3] * jy;
    Projected P;
    P.ipx   = rx + ccx;
    P.ipy   = ry + ccy;
    P.z     = z;
    P.scale = fx * c[0];  // divided by z by the caller after multiplying with radius / size
    return P;
}

void layer_sizes(const TripsSplatDesc& d, int32_t* w, int32_t* h)
{
    int cw = d.views[0].w, ch = d.views[0].h;
    for (int l = 0; l < d.num_layers; ++l)
    {
        w[l] = cw;
        h[l] = ch;
        if (!d.floor_layer_sizes)
        {
            // PointRenderer.cu:385-389
            ch = (int)std::ceil(float(ch) / 2.f);
            cw = (int)std::ceil(float(cw) / 2.f);
        }
        else
        {
            ch = ch / 2;
            cw = cw / 2;
        }
    }
}

struct PointRec
{
    float ipx, ipy, size_px, depth;
    int tex, max_layer;
};

inline float bilinear_wo_index(float ux, float uy, int gx, int gy)
{
    // compute_blending_fac_wo_index, PointBlending.h:211-214
    return (1.f - std::fabs(ux - float(gx))) * (1.f - std::fabs(uy - float(gy)));
}

// compute_blending_fac with Jacobian (PointBlending.h:216-257); blend[4], J row-major 4x2
inline void blending_fac(float ux, float uy, float blend[4], float J[8])
{
    float sx = ux - std::floor(ux), sy = uy - std::floor(uy);
    blend[0] = (1.f - sx) * (1.f - sy);
    blend[1] = sx * (1.f - sy);
    blend[2] = (1.f - sx) * sy;
    blend[3] = sx * sy;
    J[0]     = sy - 1.f;
    J[1]     = sx - 1.f;
    J[2]     = 1.f - sy;
    J[3]     = -sx;
    J[4]     = -sy;
    J[5]     = 1.f - sx;
    J[6]     = sy;
    J[7]     = sx;
}

// blend_fac_index, PointBlending.h:259-264
inline int blend_index(float ux, float uy, float gx, float gy)
{
    int x_i = gx < ux ? 0 : 1;
    int y_i = gy < uy ? 0 : 2;
    return y_i + x_i;
}

int validate(const TripsSplatDesc* d)
{
    if (!d) return TRIPS_ERR_INVALID_ARG;
    if (d->num_layers < 1 || d->num_layers > TRIPS_MAX_LAYERS) return TRIPS_ERR_INVALID_ARG;
    if (d->list_depth != 8 && d->list_depth != 16) return TRIPS_ERR_INVALID_ARG;
    if (d->num_views < 1 || d->num_views > TRIPS_MAX_VIEWS) return TRIPS_ERR_INVALID_ARG;
    if (d->num_channels < 1 || d->num_channels > 16) return TRIPS_ERR_INVALID_ARG;
    if (d->num_points < 0) return TRIPS_ERR_INVALID_ARG;
    return TRIPS_OK;
}

}  // namespace

extern "C" {

int oracle_num_threads(void) { return omp_get_max_threads(); }
void oracle_set_num_threads(int n) { omp_set_num_threads(n); }

float oracle_softplus(float x) { return softplus(x); }
float oracle_softplus_backward(float x) { return softplus_backward(x); }
float oracle_layer_factor(float s, int layer, int L, float* grad) { return layer_factor(s, layer, L, grad); }
void oracle_log2_floor_ceil(float s, int* lo, int* hi) { log2_floor_ceil(s, *lo, *hi); }

void oracle_project_point(const double* pose, const float* intr, const TripsView* view, float dist_cutoff,
                          const float* xyz, float* out4)
{
    Pose V      = load_pose(pose);
    Projected P = project(V, intr, *view, dist_cutoff, xyz);
    out4[0]     = P.ipx;
    out4[1]     = P.ipy;
    out4[2]     = P.z;
    out4[3]     = P.scale / P.z;
}

// ProjectPointPinholeBackward, PointRendererHelper.h:434-494.
// TransformPoint's Jacobians (Saiga, un-vendored) restated as J_point = R, J_pose = [I, -skew(view)]
// (left perturbation exp(tau) * V, translation first), DivideByZ's as [[iz,0,-x iz^2],[0,iz,-y iz^2]].
void oracle_project_point_backward(const double* pose, const float* intr, const TripsView* view, float dist_cutoff,
                                   const float* xyz, const float* grad2, float* g_point, float* g_pose, float* g_k,
                                   float* g_dis)
{
    for (int i = 0; i < 3; ++i) g_point[i] = 0.f;
    for (int i = 0; i < 6; ++i) g_pose[i] = 0.f;
    for (int i = 0; i < 5; ++i) g_k[i] = 0.f;
    for (int i = 0; i < 8; ++i) g_dis[i] = 0.f;
    Pose V = load_pose(pose);
    float vp[3];
    transform_point(V, xyz, vp);
    float z = vp[2];
    if (z <= 0) return;
    float R[9];
    rotation_matrix(V, R);
    float iz = 1.f / z, iz2 = 1.f / (z * z);
    float nx = vp[0] * iz, ny = vp[1] * iz;
    float Jp[4], Jd[16];
    Distorted d = distort(nx, ny, intr + 5, dist_cutoff, Jp, Jd);
    float fx = intr[0], fy = intr[1], s = intr[4];
    const float* c = view->crop_transform;
    // grad through crop rotation (J = rotation, transposed), crop K, K
    float gr0 = view->crop_rotation[0] * grad2[0] + view->crop_rotation[2] * grad2[1];
    float gr1 = view->crop_rotation[1] * grad2[0] + view->crop_rotation[3] * grad2[1];
    float a   = c[0] * gr0;              // J_p_K2^T = [[cfx,0],[cs,cfy]]
    float b   = c[4] * gr0 + c[1] * gr1;
    float k0  = fx * a;                  // J_p_K1^T * (a,b)
    float k1  = s * a + fy * b;
    float d0  = Jp[0] * k0 + Jp[2] * k1;  // J_p_dis^T
    float d1  = Jp[1] * k0 + Jp[3] * k1;
    float v0  = iz * d0;                  // J_p_div^T
    float v1  = iz * d1;
    float v2  = (-vp[0] * iz2) * d0 + (-vp[1] * iz2) * d1;
    g_point[0] = R[0] * v0 + R[3] * v1 + R[6] * v2;  // R^T
    g_point[1] = R[1] * v0 + R[4] * v1 + R[7] * v2;
    g_point[2] = R[2] * v0 + R[5] * v1 + R[8] * v2;
    g_pose[0]  = v0;
    g_pose[1]  = v1;
    g_pose[2]  = v2;
    g_pose[3]  = vp[1] * v2 - vp[2] * v1;  // (-skew(view))^T g = view x g
    g_pose[4]  = vp[2] * v0 - vp[0] * v2;
    g_pose[5]  = vp[0] * v1 - vp[1] * v0;
    g_k[0]     = d.x * a;  // J_k_K1^T: rows [x,0,1,0,y], [0,y,0,1,0]
    g_k[1]     = d.y * b;
    g_k[2]     = a;
    g_k[3]     = b;
    g_k[4]     = d.y * a;
    for (int i = 0; i < 8; ++i) g_dis[i] = Jd[i] * k0 + Jd[8 + i] * k1;
}

int oracle_layer_sizes(const TripsSplatDesc* desc, int32_t* w, int32_t* h)
{
    if (int e = validate(desc)) return e;
    layer_sizes(*desc, w, h);
    return TRIPS_OK;
}

/*
 * Forward. Follows, per view (RenderFast16, RenderForward.cu:1065-1394):
 *   CountAndCollectTiled  :168-366   projection, validity, layer selection, per-pixel counts
 *   scan section          :1155-1232 exclusive scan of the counts, layers concatenated
 *   SplattingPass         :368-436   64-bit keys (depth bits, point id) into the pixel lists
 *   FastSortFusedNew      :474-1059  K nearest per pixel, ascending; blend :820-1048
 */
int oracle_splat_forward(const TripsSplatDesc* desc, const TripsSplatIn* in, const OracleForwardOut* out)
{
    if (int e = validate(desc)) return e;
    if (!in || !out) return TRIPS_ERR_INVALID_ARG;
    const TripsSplatDesc& d = *desc;
    const int N = d.num_points, L = d.num_layers, K = d.list_depth, C = d.num_channels, B = d.num_views;
    int32_t lw[TRIPS_MAX_LAYERS], lh[TRIPS_MAX_LAYERS];
    layer_sizes(d, lw, lh);
    int64_t pix_off[TRIPS_MAX_LAYERS + 1];
    pix_off[0] = 0;
    for (int l = 0; l < L; ++l) pix_off[l + 1] = pix_off[l] + int64_t(lw[l]) * lh[l];
    const int64_t P = pix_off[L];

    std::vector<PointRec> rec(N);
    std::vector<int32_t> counts(P), cursor(P);
    std::vector<int64_t> offsets(P + 1);
    std::vector<uint64_t> keys;

    for (int b = 0; b < B; ++b)
    {
        const TripsView& cam = d.views[b];
        if (cam.camera_model_type != 0) return TRIPS_ERR_UNSUPPORTED;
        const Pose V      = load_pose(in->poses_se3 + 8 * cam.image_index);
        const float* intr = in->intrinsics + 13 * cam.camera_index;
        const float* drop = (d.train && in->dropout) ? in->dropout + int64_t(b) * N : nullptr;
        std::fill(counts.begin(), counts.end(), 0);
        int64_t n_valid = 0;

        // ---- CountAndCollectTiled ----
#pragma omp parallel for schedule(static) reduction(+ : n_valid)
        for (int pid = 0; pid < N; ++pid)
        {
            PointRec r;
            r.ipx = r.ipy = 0.f;
            r.size_px     = 0.f;
            r.depth       = -1.f;
            r.tex         = in->index[pid];
            r.max_layer   = 0;
            rec[pid]      = r;
            // a descriptor column outside the table: the reference would read past it; the build leaves the point out
            if ((unsigned)r.tex >= (unsigned)d.num_texels) continue;
            if (d.viewer_only)
            {
                // discard_point_for_confidence, RenderForward.cu:122-130
                if (in->confidence[r.tex] < d.stability_cutoff_value) continue;
            }
            if (drop && drop[pid] == 1.f) continue;
            float size         = softplus(in->point_size[pid]);
            const PointPos pos = load_point(in, N, b, pid);
            float drop_radius  = pos.v[3];
            Projected pr       = project(V, intr, cam, d.dist_cutoff, pos);
            float z            = pr.z;
            float radius_px    = pr.scale * drop_radius / z;
            float size_px      = pr.scale * size / z;
            float ipx = pr.ipx, ipy = pr.ipy;
            // valid_point, RenderForward.cu:212-218 (radius truncated to int by the lambda's signature)
            auto valid = [&](float x, float y, int layer, float radius) {
                if (z <= 0) return false;
                if (!(x >= 0) || x >= float(lw[layer] - 1) || !(y >= 0) || y >= float(lh[layer] - 1)) return false;
                if (d.drop_out_points_by_radius && float(trunc_sat(radius)) < d.drop_out_radius_threshold) return false;
                return true;
            };
            if (!valid(ipx, ipy, 0, radius_px)) continue;
            r.depth   = z;
            r.ipx     = ipx;
            r.ipy     = ipy;
            r.size_px = size_px;
            int layer_higher = 0;
            if (size_px > 1.f)
            {
                int lo, hi;
                log2_floor_ceil(size_px, lo, hi);
                layer_higher = std::min(hi, L - 1);  // RenderForward.cu:345
            }
            int layer = 0;
            for (; layer < layer_higher + 1; ++layer, ipx *= 0.5f, ipy *= 0.5f, radius_px *= 0.5f)
            {
                int px = (int)std::floor(ipx), py = (int)std::floor(ipy);
                if (!valid(float(px), float(py), layer, radius_px)) break;
                for (int i = 0; i < 4; ++i)
                {
                    int64_t pix = pix_off[layer] + int64_t(py + i / 2) * lw[layer] + (px + i % 2);
#pragma omp atomic
                    counts[pix] += 1;
                }
            }
            r.max_layer = layer;
            rec[pid]    = r;
            n_valid += 1;
        }

        // ---- scan: all layers concatenated == scanned_counts[l] + layer_lengths[l] (RenderForward.cu:408-410) ----
        offsets[0] = 0;
        for (int64_t p = 0; p < P; ++p) offsets[p + 1] = offsets[p] + counts[p];
        const int64_t E = offsets[P];
        keys.resize(E);
        for (int64_t p = 0; p < P; ++p) cursor[p] = 0;

        // ---- SplattingPass ----
#pragma omp parallel for schedule(static)
        for (int pid = 0; pid < N; ++pid)
        {
            const PointRec& r = rec[pid];
            if (!(r.depth > 0)) continue;
            uint64_t key = (uint64_t(f2u(r.depth)) << 32) | uint32_t(pid);  // __hiloint2double(bits(z), pid)
            float ipx = r.ipx, ipy = r.ipy;
            for (int layer = 0; layer < r.max_layer; ++layer)
            {
                int px = (int)std::floor(ipx), py = (int)std::floor(ipy);
                for (int sub = 0; sub < 4; ++sub)
                {
                    int64_t pix = pix_off[layer] + int64_t(py + sub / 2) * lw[layer] + (px + sub % 2);
                    int slot;
#pragma omp atomic capture
                    slot = cursor[pix]++;
                    keys[offsets[pix] + slot] = key;
                }
                ipx *= 0.5f;
                ipy *= 0.5f;
            }
        }

        // ---- FastSortFusedNew: top-K by key, blend ----
        int64_t n_retained = 0;
#pragma omp parallel for schedule(dynamic, 256) reduction(+ : n_retained)
        for (int64_t pix = 0; pix < P; ++pix)
        {
            int layer = 0;
            while (pix >= pix_off[layer + 1]) ++layer;
            int64_t local = pix - pix_off[layer];
            int gx = int(local % lw[layer]), gy = int(local / lw[layer]);
            uint64_t* kb = keys.data() + offsets[pix];
            int len      = counts[pix];
            int n        = std::min(len, K);
            if (len > K)
                std::partial_sort(kb, kb + K, kb + len);
            else
                std::sort(kb, kb + len);

            float color[16], alpha[16], contrib[16][16];
            float alpha_dest[16];
            int ret = 0;
            // transmittance chain: lane j holds prod_{k<j} (1 - alpha_k), zeroed below the cut-off
            float T = 1.f;
            for (int j = 0; j < n; ++j)
            {
                int pid           = int(uint32_t(kb[j] & 0xffffffffu));
                const PointRec& r = rec[pid];
                float m           = 1.f / float(1 << layer);
                float ux = r.ipx * m, uy = r.ipy * m;
                float w = bilinear_wo_index(ux, uy, gx, gy);
                if (std::fabs(ux - float(gx)) > 1.f || std::fabs(uy - float(gy)) > 1.f) w = 0.f;
                float a = w * in->confidence[r.tex];
                a *= layer_factor(r.size_px, layer, L, nullptr);
                alpha[j]      = a;
                float Tc      = (T >= kAlphaDestCutoff) ? T : 0.f;
                alpha_dest[j] = Tc;
                for (int c = 0; c < C; ++c) contrib[j][c] = Tc * a * in->texture[int64_t(c) * d.num_texels + r.tex];
                // entries the backward will walk: the leading run with transmittance >= cut-off (the reference's
                // backward stops at the first unsaved slot, RenderBackward.cu:205-210)
                if (Tc >= kAlphaDestCutoff && ret == j) ret = j + 1;
                T = T * (1.f - a);
            }
            for (int j = n; j < 16; ++j)
                for (int c = 0; c < C; ++c) contrib[j][c] = 0.f;
            // butterfly sum over the 16 lanes of a list (RenderForward.cu:983-994)
            for (int c = 0; c < C; ++c)
            {
                float v[16];
                for (int j = 0; j < 16; ++j) v[j] = contrib[j][c];
                for (int off = 1; off < 16; off *= 2)
                    for (int j = 0; j < 16; j += 2 * off) v[j] = v[j] + v[j + off];
                color[c] = v[0];
            }
            // background (RenderForward.cu:1002-1022); empty list -> weight 1
            float bgw = 1.f;
            if (n > 0)
            {
                if (d.background_mode == TRIPS_BG_REFERENCE)
                    bgw = alpha_dest[n - 1];
                else
                    bgw = T;  // prod over all n retained candidates
            }
            if (bgw >= kAlphaDestCutoff)
                for (int c = 0; c < C; ++c) color[c] += in->background[c] * (bgw * 1.f);

            for (int c = 0; c < C; ++c)
            {
                int64_t o;
                if (d.layout == TRIPS_LAYOUT_CHW)
                    o = ((int64_t(b) * C + c) * lh[layer] + gy) * lw[layer] + gx;
                else
                    o = ((int64_t(b) * lh[layer] + gy) * lw[layer] + gx) * C + c;
                out->image[layer][o] = color[c];
            }
            n_retained += ret;
            int64_t vp = int64_t(b) * P + pix;
            if (out->lengths) out->lengths[vp] = len;
            if (out->retained) out->retained[vp] = ret;
            if (out->lists)
                for (int j = 0; j < K; ++j) out->lists[vp * K + j] = j < n ? int(uint32_t(kb[j] & 0xffffffffu)) : -1;
            if (out->alpha)
                for (int j = 0; j < K; ++j) out->alpha[vp * K + j] = j < ret ? alpha[j] : -1.f;
        }

        if (out->counters)
        {
            out->counters[4 * b + 0] = n_valid;
            out->counters[4 * b + 1] = E;
            out->counters[4 * b + 2] = n_retained;
            out->counters[4 * b + 3] = P;
        }
        for (int pid = 0; pid < N; ++pid)
        {
            int64_t vp = int64_t(b) * N + pid;
            if (out->ip)
            {
                out->ip[2 * vp]     = rec[pid].ipx;
                out->ip[2 * vp + 1] = rec[pid].ipy;
            }
            if (out->depth) out->depth[vp] = rec[pid].depth;
            if (out->size_px) out->size_px[vp] = rec[pid].size_px;
            if (out->max_layer) out->max_layer[vp] = rec[pid].max_layer;
        }
    }
    return TRIPS_OK;
}

/*
 * Backward: BlendBackwardsBilinearTiled, RenderBackward.cu:90-618, one pixel list at a time.
 * The saved per-entry record of the reference {tex, pid, alpha, ip_l, blend_index, size_px}
 * (RenderForward.cu:957-979) is re-derived from fwd->lists / fwd->alpha and the same projection.
 */
int oracle_splat_backward(const TripsSplatDesc* desc, const TripsSplatIn* in, const OracleForwardOut* fwd,
                          const float* const grad_image[TRIPS_MAX_LAYERS], const TripsSplatGrads* g)
{
    if (int e = validate(desc)) return e;
    if (!in || !fwd || !g || !fwd->lists || !fwd->alpha || !fwd->retained) return TRIPS_ERR_INVALID_ARG;
    if (!g->d_texture || !g->d_confidence || !g->d_background) return TRIPS_ERR_INVALID_ARG;
    const TripsSplatDesc& d = *desc;
    const int N = d.num_points, L = d.num_layers, K = d.list_depth, C = d.num_channels, B = d.num_views;
    int32_t lw[TRIPS_MAX_LAYERS], lh[TRIPS_MAX_LAYERS];
    layer_sizes(d, lw, lh);
    int64_t pix_off[TRIPS_MAX_LAYERS + 1];
    pix_off[0] = 0;
    for (int l = 0; l < L; ++l) pix_off[l + 1] = pix_off[l] + int64_t(lw[l]) * lh[l];
    const int64_t P = pix_off[L];

    std::vector<PointRec> rec(N);
    for (int b = 0; b < B; ++b)
    {
        const TripsView& cam = d.views[b];
        const double* pose   = in->poses_se3 + 8 * cam.image_index;
        const Pose V         = load_pose(pose);
        const float* intr    = in->intrinsics + 13 * cam.camera_index;
#pragma omp parallel for schedule(static)
        for (int pid = 0; pid < N; ++pid)
        {
            const PointPos pos = load_point(in, N, b, pid);
            Projected pr       = project(V, intr, cam, d.dist_cutoff, pos);
            PointRec r;
            r.ipx       = pr.ipx;
            r.ipy       = pr.ipy;
            r.depth     = pr.z;
            r.size_px   = pr.scale * softplus(in->point_size[pid]) / pr.z;
            r.tex       = in->index[pid];
            r.max_layer = 0;
            rec[pid]    = r;
        }

        double acc_pose[6] = {0}, acc_k[5] = {0}, acc_dis[8] = {0}, acc_bg[16] = {0};
#pragma omp parallel
        {
            double t_pose[6] = {0}, t_k[5] = {0}, t_dis[8] = {0}, t_bg[16] = {0};
#pragma omp for schedule(dynamic, 256)
            for (int64_t pix = 0; pix < P; ++pix)
            {
                int layer = 0;
                while (pix >= pix_off[layer + 1]) ++layer;
                int64_t local = pix - pix_off[layer];
                int gx = int(local % lw[layer]), gy = int(local / lw[layer]);
                const int64_t vp     = int64_t(b) * P + pix;
                const int32_t* list  = fwd->lists + vp * K;
                const float* salpha  = fwd->alpha + vp * K;
                float grad_in[16];
                for (int c = 0; c < C; ++c)
                {
                    int64_t o;
                    if (d.layout == TRIPS_LAYOUT_CHW)
                        o = ((int64_t(b) * C + c) * lh[layer] + gy) * lw[layer] + gx;
                    else
                        o = ((int64_t(b) * lh[layer] + gy) * lw[layer] + gx) * C + c;
                    grad_in[c] = grad_image[layer][o];
                }

                // ---- compositing part, RenderBackward.cu:189-309 ----
                float conf_gradients[16];
                for (int i = 0; i < K; ++i) conf_gradients[i] = 0.f;
                int index_in_list = 0;
                float alpha_dest  = 1.f;
                do
                {
                    bool is_foreground = true;
                    float alpha_val    = (index_in_list >= K) ? -1.f : salpha[index_in_list];
                    if (alpha_val == -1.f)
                    {
                        is_foreground = false;
                        alpha_val     = 1.f;
                    }
                    int tex = 0;
                    if (is_foreground) tex = rec[list[index_in_list]].tex;
                    float colors[16];
                    for (int c = 0; c < C; ++c)
                        colors[c] = is_foreground ? in->texture[int64_t(c) * d.num_texels + tex] : in->background[c];
                    float g_alpha = 0.f;
                    for (int c = 0; c < C; ++c)
                    {
                        float gg = alpha_dest * alpha_val * grad_in[c];
                        if (is_foreground)
                        {
                            float* dst = g->d_texture + int64_t(c) * d.num_texels + tex;
#pragma omp atomic
                            *dst += gg;
                        }
                        else
                            t_bg[c] += (double)gg;
                        g_alpha += colors[c] * grad_in[c];
                    }
                    g_alpha *= alpha_dest;
                    if (is_foreground) conf_gradients[index_in_list] += g_alpha;
                    for (int j = 0; j < index_in_list; ++j)
                    {
                        float alpha_val_iter = salpha[j];
                        float g_iter         = 0.f;
                        for (int c = 0; c < C; ++c)
                        {
                            const float epsilon = 1e-9f;
                            float dem           = 1.f / (1.f - alpha_val_iter + epsilon);
                            float g_alpha_iter  = (grad_in[c] * colors[c] * alpha_dest * alpha_val * dem);
                            g_iter -= g_alpha_iter;
                        }
                        conf_gradients[j] += g_iter;
                    }
                    alpha_dest = (1.f - alpha_val) * alpha_dest;  // compute_new_alphadest, PointBlending.h:339-352
                    if (!is_foreground) break;
                    ++index_in_list;
                } while (index_in_list < K + 1 && alpha_dest >= 0.001);

                // ---- geometric part, RenderBackward.cu:311-538 ----
                for (int i = 0; i < index_in_list; ++i)
                {
                    int pid           = list[i];
                    const PointRec& r = rec[pid];
                    float m           = 1.f / float(1 << layer);
                    float ux = r.ipx * m, uy = r.ipy * m;
                    int bi           = blend_index(ux, uy, float(gx), float(gy));
                    float grad_alpha = conf_gradients[i];
                    float blend[4], J[8];
                    blending_fac(ux, uy, blend, J);
                    if (std::fabs(ux - float(gx)) > 1.f || std::fabs(uy - float(gy)) > 1.f)
                        for (int q = 0; q < 4; ++q) blend[q] *= 0.f;
                    float confidence_val = in->confidence[r.tex];
                    float lfac = 1.f, J_lf = 0.f;
                    if (g->d_point_size) lfac = layer_factor(r.size_px, layer, L, &J_lf);
                    {
                        float gc   = blend[bi] * lfac * grad_alpha;
                        float* dst = g->d_confidence + r.tex;
#pragma omp atomic
                        *dst += gc;
                    }
                    float grad_blend_single = confidence_val * lfac * grad_alpha;
                    float dR_dp[2]          = {J[2 * bi] * grad_blend_single, J[2 * bi + 1] * grad_blend_single};
                    const PointPos pos      = load_point(in, N, b, pid);
                    float g_point[3], g_pose[6], g_k[5], g_dis[8];
                    oracle_project_point_backward(pose, intr, &cam, d.dist_cutoff, pos, dR_dp, g_point, g_pose, g_k,
                                                  g_dis);
                    if (g->d_point_size)
                    {
                        float J_softmax_proj = intr[0] * cam.crop_transform[0] / r.depth;  // g_layer, :463
                        float J_softmax_ps   = softplus_backward(in->point_size[pid]);
                        float grad_layer_ps  = J_softmax_ps * J_softmax_proj * J_lf * grad_alpha;
                        float grad_layer     = blend[bi] * confidence_val * grad_layer_ps;
                        float* dst           = g->d_point_size + pid;
#pragma omp atomic
                        *dst += grad_layer;
                    }
                    if (g->d_position)
                        for (int k = 0; k < 3; ++k)
                        {
                            float* dst = g->d_position + 4 * int64_t(pid) + k;
#pragma omp atomic
                            *dst += g_point[k];
                        }
                    if (g->d_pose)
                        for (int k = 0; k < 6; ++k) t_pose[k] += (double)g_pose[k];
                    if (g->d_intrinsics)
                    {
                        for (int k = 0; k < 5; ++k) t_k[k] += (double)g_k[k];
                        for (int k = 0; k < 8; ++k) t_dis[k] += (double)g_dis[k];
                    }
                }
            }
#pragma omp critical
            {
                for (int k = 0; k < 6; ++k) acc_pose[k] += t_pose[k];
                for (int k = 0; k < 5; ++k) acc_k[k] += t_k[k];
                for (int k = 0; k < 8; ++k) acc_dis[k] += t_dis[k];
                for (int c = 0; c < C; ++c) acc_bg[c] += t_bg[c];
            }
        }
        // block-level write-back, RenderBackward.cu:587-617
        if (g->d_pose)
            for (int k = 0; k < 6; ++k) g->d_pose[6 * cam.image_index + k] += acc_pose[k];
        if (g->d_intrinsics)
        {
            for (int k = 0; k < 5; ++k) g->d_intrinsics[13 * cam.camera_index + k] += (float)acc_k[k];
            for (int k = 0; k < 8; ++k) g->d_intrinsics[13 * cam.camera_index + 5 + k] += (float)acc_dis[k];
        }
        for (int c = 0; c < C; ++c) g->d_background[c] += (float)acc_bg[c];
    }
    return TRIPS_OK;
}

/* adam_step, MyAdam.cu:41-88 (weight_decay :28-34, clamp :35-39) */
int oracle_adam_step(const TripsAdamTensor* tensors, int n_tensors)
{
    if (!tensors || n_tensors < 0) return TRIPS_ERR_INVALID_ARG;
    for (int t = 0; t < n_tensors; ++t)
    {
        const TripsAdamTensor& T = tensors[t];
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < T.n; ++i)
        {
            float gradient, weight_fp;
            if (T.dtype == TRIPS_DTYPE_F64)
            {
                gradient  = (float)((const double*)T.grads)[i] / T.loss_scale;
                weight_fp = (float)((double*)T.weights)[i];
            }
            else
            {
                gradient  = ((const float*)T.grads)[i] / T.loss_scale;
                weight_fp = ((float*)T.weights)[i];
            }
            if (gradient == 0.f) continue;
            const float gradient_sq   = gradient * gradient;
            float first_moment        = T.first_moment[i] = T.beta1 * T.first_moment[i] + (1 - T.beta1) * gradient;
            const float second_moment = T.second_moment[i] =
                T.beta2 * T.second_moment[i] + (1 - T.beta2) * gradient_sq;
            uint32_t current_step;
            if (T.steps_dtype == TRIPS_STEPS_I32)
                current_step = (uint32_t)(((int32_t*)T.steps)[i] += 1);
            else
                current_step = (uint32_t)(((int64_t*)T.steps)[i] += 1);
            float learning_rate         = T.lr;
            learning_rate *= std::sqrt(1 - std::pow(T.beta2, (float)current_step)) /
                             (1 - std::pow(T.beta1, (float)current_step));
            const float effective_learning_rate = std::fmin(
                std::fmax(learning_rate / (std::sqrt(second_moment) + T.eps), T.lower_lr_bound), T.upper_lr_bound);
            const float rel            = T.relative_weight_decay * learning_rate;
            const float ab             = T.absolute_weight_decay * learning_rate;
            const float decayed_weight = (1 - rel) * weight_fp - std::copysign(ab, weight_fp);
            float new_weight           = decayed_weight - effective_learning_rate * first_moment;
            if (T.weight_clipping_magnitude != 0.0f)
            {
                float lo = -T.weight_clipping_magnitude, hi = T.weight_clipping_magnitude;
                new_weight = new_weight < lo ? lo : (hi < new_weight ? hi : new_weight);
            }
            if (T.dtype == TRIPS_DTYPE_F64)
                ((double*)T.weights)[i] = new_weight;
            else
                ((float*)T.weights)[i] = new_weight;
        }
    }
    return TRIPS_OK;
}

/*
 * ApplyTangent, PointRenderer.cu:1428-1447: pose <- se3_exp(t with t[3:6] *= 0.1) * pose, t <- 0.
 * Sophus (un-vendored) restated: SO3::exp through the half-angle quaternion, SE3::exp with
 * V = I + (1-cos)/th^2 W + (th-sin)/th^3 W^2, product q1*q2 with Sophus' first-order renormalisation.
 */
int oracle_apply_tangent(double* tangent, double* poses, int n)
{
    for (int i = 0; i < n; ++i)
    {
        double* t = tangent + 6 * i;
        double* p = poses + 8 * i;
        double u[3] = {t[0], t[1], t[2]};
        double w[3] = {t[3] * 0.1, t[4] * 0.1, t[5] * 0.1};
        double th2  = w[0] * w[0] + w[1] * w[1] + w[2] * w[2];
        double th   = std::sqrt(th2);
        double imag, real;
        if (th < 1e-10)
        {
            double th4 = th2 * th2;
            imag       = 0.5 - th2 / 48.0 + th4 / 3840.0;
            real       = 1.0 - th2 / 8.0 + th4 / 384.0;
        }
        else
        {
            imag = std::sin(0.5 * th) / th;
            real = std::cos(0.5 * th);
        }
        double q1[4] = {imag * w[0], imag * w[1], imag * w[2], real};  // xyzw
        // V * u
        double W[9]  = {0, -w[2], w[1], w[2], 0, -w[0], -w[1], w[0], 0};
        double W2[9];
        for (int r = 0; r < 3; ++r)
            for (int c = 0; c < 3; ++c)
            {
                double s = 0;
                for (int k = 0; k < 3; ++k) s += W[3 * r + k] * W[3 * k + c];
                W2[3 * r + c] = s;
            }
        double Vm[9];
        if (th < 1e-10)
        {
            // V = so3.matrix()
            double x = q1[0], y = q1[1], z = q1[2], ww = q1[3];
            double R[9] = {1 - 2 * (y * y + z * z), 2 * (x * y - z * ww),     2 * (x * z + y * ww),
                           2 * (x * y + z * ww),     1 - 2 * (x * x + z * z), 2 * (y * z - x * ww),
                           2 * (x * z - y * ww),     2 * (y * z + x * ww),     1 - 2 * (x * x + y * y)};
            for (int k = 0; k < 9; ++k) Vm[k] = R[k];
        }
        else
        {
            double a = (1 - std::cos(th)) / th2, bq = (th - std::sin(th)) / (th2 * th);
            for (int k = 0; k < 9; ++k) Vm[k] = (k % 4 == 0 ? 1.0 : 0.0) + a * W[k] + bq * W2[k];
        }
        double t1[3];
        for (int r = 0; r < 3; ++r) t1[r] = Vm[3 * r] * u[0] + Vm[3 * r + 1] * u[1] + Vm[3 * r + 2] * u[2];
        // q = q1 * q2
        double x2 = p[0], y2 = p[1], z2 = p[2], w2 = p[3];
        double x1 = q1[0], y1 = q1[1], z1 = q1[2], w1 = q1[3];
        double q[4] = {w1 * x2 + x1 * w2 + y1 * z2 - z1 * y2, w1 * y2 - x1 * z2 + y1 * w2 + z1 * x2,
                       w1 * z2 + x1 * y2 - y1 * x2 + z1 * w2, w1 * w2 - x1 * x2 - y1 * y2 - z1 * z2};
        double sn = q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3];
        if (sn != 1.0)
        {
            double sc = 2.0 / (1.0 + sn);
            for (int k = 0; k < 4; ++k) q[k] *= sc;
        }
        // t = t1 + R1 * t2
        double R1[9] = {1 - 2 * (y1 * y1 + z1 * z1), 2 * (x1 * y1 - z1 * w1),     2 * (x1 * z1 + y1 * w1),
                        2 * (x1 * y1 + z1 * w1),     1 - 2 * (x1 * x1 + z1 * z1), 2 * (y1 * z1 - x1 * w1),
                        2 * (x1 * z1 - y1 * w1),     2 * (y1 * z1 + x1 * w1),     1 - 2 * (x1 * x1 + y1 * y1)};
        double tn[3];
        for (int r = 0; r < 3; ++r) tn[r] = t1[r] + R1[3 * r] * p[4] + R1[3 * r + 1] * p[5] + R1[3 * r + 2] * p[6];
        for (int k = 0; k < 4; ++k) p[k] = q[k];
        for (int k = 0; k < 3; ++k) p[4 + k] = tn[k];
        for (int k = 0; k < 6; ++k) t[k] = 0.0;
    }
    return TRIPS_OK;
}

}  // extern "C"
