/*
 * adop_oracle.cpp — CPU restatement of ADOP's one-pixel point rasterizer.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker for the HIP path, never the product: only tests, the smoke check and the
 * benchmark's cpu_baseline leg may build or call it.  It follows the reference line by line (citations are
 * paths inside the darglein/ADOP source tree) in single-threaded fp32 with -ffp-contract=off; an optional
 * OpenMP build of the same loops is used only for CPU-baseline timing.
 *
 * Third-party arithmetic: the reference calls into darglein/saiga (git submodule External/saiga, absent from
 * the reference tree, pinned commit unknown) and Sophus/Eigen.  The functions below restate their published
 * definitions; where the exact saiga source could not be consulted the behaviour is DEFINED here:
 *   - TransformPoint / DivideByZ / distortNormalizedPoint (OpenCV rational-tangential, k1..k6,p1,p2) /
 *     IntrinsicsPinhole::{normalizedToImage,scale,unproject2} / ProjectOCam (Scaramuzza world2cam polynomial)
 *     / Pack,UnpackNormal10Bit / undistortNormalizedPointSimple / ImageView::{inImage2,distanceFromEdge}
 *     : "defined, not verified against saiga" -> parity with saiga itself is UNPINNED.  What IS pinned (see
 *     tests/test_oracle_*.py): closed forms, finite-difference checks of every Jacobian, brute force.
 *   - Sophus SE3d -> SE3f cast normalises the float quaternion; SO3 * v is Eigen's Quaternion::_transformVector.
 *   - atan / atan2 / acos are evaluated with the fixed polynomials below (not libm) so that any other
 *     implementation using only IEEE + - * / sqrt reproduces them bit for bit.
 */
#include "../include/adop_raster.h"

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#    include <omp.h>
#endif

namespace
{
struct V2
{
    float x, y;
};
struct V3
{
    float x, y, z;
};

// ------------------------------------------------------------------------------------------------
// scalar helpers
// ------------------------------------------------------------------------------------------------

inline uint32_t float_bits(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float bits_float(uint32_t u)
{
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// __float2int_rn (PointRenderer.cu:266): round to nearest even, saturating, NaN -> 0.
inline int f2i_rn(float f)
{
    if (f != f) return 0;
    float r = std::nearbyintf(f);
    if (r >= 2147483648.f) return 2147483647;
    if (r <= -2147483648.f) return (-2147483647 - 1);
    return (int)r;
}

// IEEE half -> float (exact).
inline float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1Fu;
    uint32_t man  = h & 0x3FFu;
    uint32_t out;
    if (exp == 0)
    {
        if (man == 0)
            out = sign;
        else
        {
            int e = -1;
            do
            {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            out = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    }
    else if (exp == 31)
        out = sign | 0x7F800000u | (man << 13);
    else
        out = sign | ((exp + 112u) << 23) | (man << 13);
    return bits_float(out);
}

// Fixed-polynomial arctangent family (Cephes single-precision kernels), + - * / sqrt only.
const float kPi     = 3.14159265358979323846f;
const float kHalfPi = 1.57079632679489661923f;
const float kQuartPi = 0.78539816339744830962f;

inline float o_atanf(float xx)
{
    float x    = xx < 0 ? -xx : xx;
    float y;
    if (x > 2.414213562373095f)
    {
        y = kHalfPi;
        x = -(1.0f / x);
    }
    else if (x > 0.4142135623730950f)
    {
        y = kQuartPi;
        x = (x - 1.0f) / (x + 1.0f);
    }
    else
        y = 0.0f;
    float z = x * x;
    float p = (((8.05374449538e-2f * z - 1.38776856032e-1f) * z + 1.99777106478e-1f) * z - 3.33329491539e-1f);
    y       = y + (p * z * x + x);
    return xx < 0 ? -y : y;
}

inline float o_atan2f(float y, float x)
{
    if (x == 0.0f)
    {
        if (y > 0.0f) return kHalfPi;
        if (y < 0.0f) return -kHalfPi;
        return 0.0f;
    }
    float a = o_atanf(y / x);
    if (x < 0.0f) return (y < 0.0f) ? a - kPi : a + kPi;
    return a;
}

inline float o_asinf(float xx)
{
    float a    = xx < 0 ? -xx : xx;
    if (a > 1.0f) a = 1.0f;
    bool flag = a > 0.5f;
    float z, x;
    if (flag)
    {
        z = 0.5f * (1.0f - a);
        x = std::sqrt(z);
    }
    else
    {
        x = a;
        z = x * x;
    }
    float p = ((((4.2163199048e-2f * z + 2.4181311049e-2f) * z + 4.5470025998e-2f) * z + 7.4953002686e-2f) * z +
               1.6666752422e-1f);
    float r = p * z * x + x;
    if (flag)
    {
        r = r + r;
        r = kHalfPi - r;
    }
    return xx < 0 ? -r : r;
}

inline float o_acosf(float x)
{
    if (x < -0.5f) return kPi - 2.0f * o_asinf(std::sqrt(0.5f * (1.0f + x)));
    if (x > 0.5f) return 2.0f * o_asinf(std::sqrt(0.5f * (1.0f - x)));
    return kHalfPi - o_asinf(x);
}

// sine and cosine of an angle in [-pi/2, pi/2] (Cephes single-precision kernels on [-pi/4, pi/4], the rest through
// the complementary angle), + - * only.
inline void o_sincosf(float theta, float* s_out, float* c_out)
{
    float a    = theta < 0 ? -theta : theta;
    bool compl_ = a > kQuartPi;
    float x    = compl_ ? kHalfPi - a : a;
    float z    = x * x;
    float sn   = ((-1.9515295891e-4f * z + 8.3321608736e-3f) * z - 1.6666654611e-1f) * z * x + x;
    float cs   = ((2.443315711809948e-5f * z - 1.388731625493765e-3f) * z + 4.166664568298827e-2f) * z * z +
               (1.0f - 0.5f * z);
    float s = compl_ ? cs : sn;
    float c = compl_ ? sn : cs;
    *s_out  = theta < 0 ? -s : s;
    *c_out  = c;
}

// ------------------------------------------------------------------------------------------------
// geometry (saiga / Sophus / Eigen restatements)
// ------------------------------------------------------------------------------------------------

inline V3 cross(V3 a, V3 b)
{
    return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
inline float dot(V3 a, V3 b)
{
    return (a.x * b.x + a.y * b.y) + a.z * b.z;
}

struct Pose
{
    float qx, qy, qz, qw;
    float tx, ty, tz;
};

// d_render_params.Pose(): SE3d row -> SE3f (PointRenderer.cu:73).  Sophus' cast builds the float SO3 from
// the cast quaternion, which normalises it.
Pose load_pose(const double* p)
{
    Pose P;
    float x = (float)p[0], y = (float)p[1], z = (float)p[2], w = (float)p[3];
    float n = std::sqrt(((x * x + y * y) + z * z) + w * w);
    P.qx    = x / n;
    P.qy    = y / n;
    P.qz    = z / n;
    P.qw    = w / n;
    P.tx    = (float)p[4];
    P.ty    = (float)p[5];
    P.tz    = (float)p[6];
    return P;
}

// Eigen::Quaternion::_transformVector: uv = 2 * (q.vec x v); v + w*uv + q.vec x uv
inline V3 rotate(const Pose& P, V3 v)
{
    V3 q  = {P.qx, P.qy, P.qz};
    V3 uv = cross(q, v);
    uv.x += uv.x;
    uv.y += uv.y;
    uv.z += uv.z;
    V3 c = cross(q, uv);
    return {(v.x + P.qw * uv.x) + c.x, (v.y + P.qw * uv.y) + c.y, (v.z + P.qw * uv.z) + c.z};
}
inline V3 rotate_inv(const Pose& P, V3 v)
{
    Pose C = P;
    C.qx   = -P.qx;
    C.qy   = -P.qy;
    C.qz   = -P.qz;
    return rotate(C, v);
}
// TransformPoint (PointRendererHelper.h:55): V * p
inline V3 transform_point(const Pose& P, V3 p)
{
    V3 r = rotate(P, p);
    return {r.x + P.tx, r.y + P.ty, r.z + P.tz};
}

struct Pinhole
{
    float fx, fy, cx, cy, s;
};
struct Distortion
{
    float k1, k2, k3, k4, k5, k6, p1, p2;
};

// IntrinsicsPinhole::normalizedToImage
inline V2 k_apply(const Pinhole& K, V2 p)
{
    return {(K.fx * p.x + K.s * p.y) + K.cx, K.fy * p.y + K.cy};
}
// IntrinsicsPinhole::scale: every coefficient multiplied
inline Pinhole k_scale(const Pinhole& K, float f)
{
    return {K.fx * f, K.fy * f, K.cx * f, K.cy * f, K.s * f};
}
// IntrinsicsPinhole::unproject2
inline V2 k_unproject2(const Pinhole& K, V2 ip)
{
    float y = (ip.y - K.cy) / K.fy;
    float x = ((ip.x - K.cx) - K.s * y) / K.fx;
    return {x, y};
}

// distortNormalizedPoint: OpenCV rational + tangential model with a radius cutoff.  Beyond the cutoff
// the sentinel (100000,100000) is returned (tested at PointRendererHelper.h:74).
// J_point (2x2 row-major) and J_dist (2x8 row-major, order k1..k6,p1,p2) are optional.
V2 distort(V2 p, const Distortion& D, float max_r, float* Jp, float* Jd)
{
    float x = p.x, y = p.y;
    float x2 = x * x, y2 = y * y;
    float r2  = x2 + y2;
    float xy2 = 2.0f * x * y;
    float r4  = r2 * r2;
    float r6  = r2 * r4;

    float U    = 1.0f + D.k1 * r2 + D.k2 * r4 + D.k3 * r6;
    float Vv   = 1.0f + D.k4 * r2 + D.k5 * r4 + D.k6 * r6;
    float iV   = 1.0f / Vv;
    float rad  = U * iV;
    float tx   = D.p1 * xy2 + D.p2 * (r2 + 2.0f * x2);
    float ty   = D.p1 * (r2 + 2.0f * y2) + D.p2 * xy2;
    V2 out     = {x * rad + tx, y * rad + ty};

    if (Jp)
    {
        float dU  = D.k1 + 2.0f * D.k2 * r2 + 3.0f * D.k3 * r4;  // dU/dr2
        float dV  = D.k4 + 2.0f * D.k5 * r2 + 3.0f * D.k6 * r4;
        float dr  = (dU * Vv - U * dV) * iV * iV;                // d rad / d r2
        float drx = dr * 2.0f * x, dry = dr * 2.0f * y;
        Jp[0]     = rad + x * drx + D.p1 * 2.0f * y + D.p2 * 6.0f * x;
        Jp[1]     = x * dry + D.p1 * 2.0f * x + D.p2 * 2.0f * y;
        Jp[2]     = y * drx + D.p1 * 2.0f * x + D.p2 * 2.0f * y;
        Jp[3]     = rad + y * dry + D.p1 * 6.0f * y + D.p2 * 2.0f * x;
    }
    if (Jd)
    {
        float a = -U * iV * iV;
        float cu[3] = {r2 * iV, r4 * iV, r6 * iV};
        float cv[3] = {r2 * a, r4 * a, r6 * a};
        for (int i = 0; i < 3; ++i)
        {
            Jd[i]         = x * cu[i];
            Jd[3 + i]     = x * cv[i];
            Jd[8 + i]     = y * cu[i];
            Jd[8 + 3 + i] = y * cv[i];
        }
        Jd[6]     = xy2;
        Jd[7]     = r2 + 2.0f * x2;
        Jd[8 + 6] = r2 + 2.0f * y2;
        Jd[8 + 7] = xy2;
    }
    if (r2 > max_r * max_r)
    {
        out.x = 100000.f;
        out.y = 100000.f;
    }
    return out;
}

// undistortNormalizedPointSimple: OpenCV's fixed-point iteration, 5 rounds.
V2 undistort_simple(V2 p, const Distortion& D)
{
    float x0 = p.x, y0 = p.y, x = p.x, y = p.y;
    for (int it = 0; it < 5; ++it)
    {
        float r2     = x * x + y * y;
        float icdist = (1.0f + ((D.k6 * r2 + D.k5) * r2 + D.k4) * r2) / (1.0f + ((D.k3 * r2 + D.k2) * r2 + D.k1) * r2);
        float dx     = 2.0f * D.p1 * x * y + D.p2 * (r2 + 2.0f * x * x);
        float dy     = D.p1 * (r2 + 2.0f * y * y) + 2.0f * D.p2 * x * y;
        x            = (x0 - dx) * icdist;
        y            = (y0 - dy) * icdist;
    }
    return {x, y};
}

// UnpackNormal10Bit / PackNormal10Bit (NeuralPointCloudCuda.h:96, .cpp:31): 3 x 10 bit, x in bits 0..9.
V3 unpack_normal(int32_t enc)
{
    uint32_t e = (uint32_t)enc;
    float x    = (float)(e & 1023u), y = (float)((e >> 10) & 1023u), z = (float)((e >> 20) & 1023u);
    const float s = 2.0f / 1023.0f;
    return {x * s - 1.0f, y * s - 1.0f, z * s - 1.0f};
}
int32_t pack_normal(V3 n)
{
    auto q = [](float c)
    {
        int v = f2i_rn((c * 0.5f + 0.5f) * 1023.0f);
        return (uint32_t)(v < 0 ? 0 : (v > 1023 ? 1023 : v));
    };
    return (int32_t)(q(n.x) | (q(n.y) << 10) | (q(n.z) << 20));
}

// ProjectPointPinhole, PointRendererHelper.h:49-82
void project_pinhole(V3 p, V3 n, const Pose& V, const Pinhole& K, const Distortion& D, bool check_normal,
                     float dist_cutoff, V2* image_p, float* z_out)
{
    V3 view_p = transform_point(V, p);
    float z   = view_p.z;
    z         = std::fmax(z, 0.f);
    if (check_normal)
    {
        V3 view_n = rotate(V, n);
        if (dot(view_p, view_n) > 0) z = 0;
    }
    float iz  = 1.0f / view_p.z;  // DivideByZ
    V2 norm_p = {view_p.x * iz, view_p.y * iz};
    V2 dist_p = distort(norm_p, D, dist_cutoff, nullptr, nullptr);
    if (dist_p.x == 100000) z = 0;
    *image_p = k_apply(K, dist_p);
    *z_out   = z;
}

// ProjectOCam (saiga OCam.h), Scaramuzza world2cam with the camera looking along +z:
// theta = atan(-z / |xy|), rho = poly(theta), (u,v) = affine * rho * xy/|xy| + centre; returned depth is the
// Euclidean distance, 0 when theta exceeds the cutoff.  Jacobians: J_p 2x3, J_aff 2x5 (c,d,e,cx,cy).
void project_ocam_core(V3 p, const float* aff, const float* poly, int npoly, float cutoff, V2* uv, float* z_out,
                       float* Jp, float* Ja)
{
    float c = aff[0], d = aff[1], e = aff[2], cx = aff[3], cy = aff[4];
    float x = p.x, y = p.y, z = p.z;
    float r2   = x * x + y * y;
    float norm = std::sqrt(r2);
    float dist = std::sqrt(r2 + z * z);
    if (norm == 0.0f)
    {
        *uv    = {cx, cy};
        *z_out = z > 0 ? dist : 0.0f;
        if (Jp)
            for (int i = 0; i < 6; ++i) Jp[i] = 0;
        if (Ja)
        {
            for (int i = 0; i < 10; ++i) Ja[i] = 0;
            Ja[3] = 1;
            Ja[9] = 1;
        }
        return;
    }
    float theta = o_atanf(-z / norm);
    float rho   = poly[0];
    float drho  = 0;
    float t_i   = 1;
    for (int i = 1; i < npoly; ++i)
    {
        drho += (float)i * poly[i] * t_i;
        t_i *= theta;
        rho += t_i * poly[i];
    }
    float inv = 1.0f / norm;
    float cxn = x * inv, cyn = y * inv;
    float uu = cxn * rho, vv = cyn * rho;
    *uv    = {(uu * c + vv * d) + cx, (uu * e + vv) + cy};
    *z_out = theta > cutoff ? 0.0f : dist;

    if (Jp)
    {
        float d2  = r2 + z * z;
        float tx  = z * x / (norm * d2);
        float ty  = z * y / (norm * d2);
        float tz  = -norm / d2;
        float i3  = inv * inv * inv;
        float uux = rho * (inv - x * x * i3) + cxn * drho * tx;
        float uuy = rho * (-x * y * i3) + cxn * drho * ty;
        float uuz = cxn * drho * tz;
        float vvx = rho * (-x * y * i3) + cyn * drho * tx;
        float vvy = rho * (inv - y * y * i3) + cyn * drho * ty;
        float vvz = cyn * drho * tz;
        Jp[0]     = c * uux + d * vvx;
        Jp[1]     = c * uuy + d * vvy;
        Jp[2]     = c * uuz + d * vvz;
        Jp[3]     = e * uux + vvx;
        Jp[4]     = e * uuy + vvy;
        Jp[5]     = e * uuz + vvz;
    }
    if (Ja)
    {
        Ja[0] = uu; Ja[1] = vv; Ja[2] = 0;  Ja[3] = 1; Ja[4] = 0;
        Ja[5] = 0;  Ja[6] = 0;  Ja[7] = uu; Ja[8] = 0; Ja[9] = 1;
    }
}

// ProjectPointOcam, PointRendererHelper.h:85-106
void project_ocam(V3 p, V3 n, const Pose& V, const float* aff, const float* poly, int npoly, bool check_normal,
                  float dist_cutoff, V2* image_p, float* z_out)
{
    V3 view_p = transform_point(V, p);
    float z;
    project_ocam_core(view_p, aff, poly, npoly, dist_cutoff, image_p, &z, nullptr, nullptr);
    V3 view_n = rotate(V, n);
    if (check_normal & (dot(view_p, view_n) > 0)) z = 0;
    *z_out = z;
}

// Pixel of the uncropped OCam image -> unit ray in camera space: the inverse of project_ocam_core.  The reference
// has no such routine (its environment map asserts the pinhole model, EnvironmentMap.cu:129, and
// PointRendererHelper.h:85-106 is the forward direction only); DEFINED here: undo the affine map, then solve
// poly(theta) = rho with kOcamNewtonSteps Newton steps from the axis (theta = -pi/2), theta kept in [-pi/2, pi/2];
// the ray is (cos(theta) * (uu,vv)/rho, -sin(theta)), so that theta = atan(-z / |xy|) as in the forward direction.
// (Five steps: on fisheye polynomials with up to 5 % of higher-order terms the fourth step no longer changes the
// round trip project(unproject(pixel)) - pixel, which stays below 4e-4 pixels; tests/test_oracle_math.py.)
const int kOcamNewtonSteps = 5;
V3 ocam_unproject(const float* aff, const float* poly, int npoly, V2 ip)
{
    float c = aff[0], d = aff[1], e = aff[2], cx = aff[3], cy = aff[4];
    float px = ip.x - cx, py = ip.y - cy;
    float det = c - d * e;
    float uu  = (px - d * py) / det;
    float vv  = (c * py - e * px) / det;
    float rho = std::sqrt(uu * uu + vv * vv);
    float theta = -kHalfPi;
    for (int it = 0; it < kOcamNewtonSteps; ++it)
    {
        float r   = poly[0];
        float dr  = 0;
        float t_i = 1;
        for (int i = 1; i < npoly; ++i)
        {
            dr += (float)i * poly[i] * t_i;
            t_i *= theta;
            r += t_i * poly[i];
        }
        if (dr != 0) theta = theta - (r - rho) / dr;
        theta = std::fmin(std::fmax(theta, -kHalfPi), kHalfPi);
    }
    float sn, cs;
    o_sincosf(theta, &sn, &cs);
    float cxn = rho > 0 ? uu / rho : 0.f;
    float cyn = rho > 0 ? vv / rho : 0.f;
    return {cxn * cs, cyn * cs, -sn};
}

struct BackwardOut
{
    float g_point[3];
    float g_pose[6];
    float g_k[5];    // pinhole K or OCam affine
    float g_dis[8];  // pinhole only
};

// J_pose^T c  with J_pose = [I | -[view_p]x]  (TransformPoint, left perturbation exp(eps) * V,
// translation first): (c, view_p x c)
inline void pose_chain(V3 view_p, V3 c, float* g_pose)
{
    V3 r      = cross(view_p, c);
    g_pose[0] = c.x;
    g_pose[1] = c.y;
    g_pose[2] = c.z;
    g_pose[3] = r.x;
    g_pose[4] = r.y;
    g_pose[5] = r.z;
}

// ProjectPointPinholeBackward, PointRendererHelper.h:120-170
BackwardOut project_pinhole_backward(V3 p, V3 n, V2 grad, const Pose& V, const Pinhole& K, const Pinhole& crop,
                                     const Distortion& D, bool check_normal, float dist_cutoff)
{
    BackwardOut o;
    std::memset(&o, 0, sizeof(o));
    V3 view_p = transform_point(V, p);
    float z   = view_p.z;
    if (z <= 0) return o;
    if (check_normal)
    {
        V3 view_n = rotate(V, n);
        if (dot(view_p, view_n) > 0) return o;
    }
    float iz  = 1.0f / z;
    V2 norm_p = {view_p.x * iz, view_p.y * iz};
    float Jp[4], Jd[16];
    V2 dist_p = distort(norm_p, D, dist_cutoff, Jp, Jd);

    // J_crop^T grad ; J_K^T (.)
    V2 g2 = {crop.fx * grad.x, crop.s * grad.x + crop.fy * grad.y};
    V2 g1 = {K.fx * g2.x, K.s * g2.x + K.fy * g2.y};
    // J_dis^T
    V2 g0 = {Jp[0] * g1.x + Jp[2] * g1.y, Jp[1] * g1.x + Jp[3] * g1.y};
    // J_div^T
    V3 c = {g0.x * iz, g0.y * iz, (-(view_p.x * iz * iz)) * g0.x + (-(view_p.y * iz * iz)) * g0.y};

    V3 gp        = rotate_inv(V, c);  // J_point^T = R^T
    o.g_point[0] = gp.x;
    o.g_point[1] = gp.y;
    o.g_point[2] = gp.z;
    pose_chain(view_p, c, o.g_pose);

    // J_k^T g2, coefficient order fx,fy,cx,cy,s
    o.g_k[0] = dist_p.x * g2.x;
    o.g_k[1] = dist_p.y * g2.y;
    o.g_k[2] = g2.x;
    o.g_k[3] = g2.y;
    o.g_k[4] = dist_p.y * g2.x;
    for (int i = 0; i < 8; ++i) o.g_dis[i] = Jd[i] * g1.x + Jd[8 + i] * g1.y;
    return o;
}

// ProjectPointOcamBackward, PointRendererHelper.h:184-227
BackwardOut project_ocam_backward(V3 p, V3 n, V2 grad, const Pose& V, const Pinhole& crop, const float* aff,
                                  const float* poly, int npoly, bool check_normal, float dist_cutoff)
{
    BackwardOut o;
    std::memset(&o, 0, sizeof(o));
    V3 view_p = transform_point(V, p);
    V3 view_n = rotate(V, n);
    if (check_normal && dot(view_p, view_n) > 0) return o;
    float Jp[6], Ja[10];
    V2 uv;
    float z;
    project_ocam_core(view_p, aff, poly, npoly, dist_cutoff, &uv, &z, Jp, Ja);
    V2 g2 = {crop.fx * grad.x, crop.s * grad.x + crop.fy * grad.y};
    V3 c  = {Jp[0] * g2.x + Jp[3] * g2.y, Jp[1] * g2.x + Jp[4] * g2.y, Jp[2] * g2.x + Jp[5] * g2.y};
    V3 gp = rotate_inv(V, c);
    o.g_point[0] = gp.x;
    o.g_point[1] = gp.y;
    o.g_point[2] = gp.z;
    pose_chain(view_p, c, o.g_pose);
    for (int i = 0; i < 5; ++i) o.g_k[i] = Ja[i] * g2.x + Ja[5 + i] * g2.y;
    return o;
}

// ------------------------------------------------------------------------------------------------
// the render stage
// ------------------------------------------------------------------------------------------------

struct Cam
{
    Pose V;
    Pinhole K;
    Distortion D;
    const float* aff;
    const float* poly;
    int npoly;
    Pinhole crop;
    int model;
};

Cam make_cam(const adop_scene* s, const adop_view& v)
{
    Cam c;
    c.V              = load_pose(s->poses_se3 + 8 * (size_t)v.image_index);
    const float* ptr = s->intrinsics + (size_t)s->intrinsics_cols * v.camera_index;
    c.model          = v.camera_model_type;
    c.aff            = ptr;
    c.poly           = ptr + 5;
    c.npoly          = s->intrinsics_cols - 5;
    if (c.model == ADOP_CAMERA_PINHOLE_DISTORTION)
    {
        c.K = {ptr[0], ptr[1], ptr[2], ptr[3], ptr[4]};
        c.D = {ptr[5], ptr[6], ptr[7], ptr[8], ptr[9], ptr[10], ptr[11], ptr[12]};
    }
    else
    {
        c.K = {0, 0, 0, 0, 0};
        c.D = {0, 0, 0, 0, 0, 0, 0, 0};
    }
    c.crop = {v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy, v.crop_s};
    return c;
}

// DevicePointCloud::GetPoint, NeuralPointCloudCuda.h:82-103
inline void get_point(const adop_scene* s, int i, V3* pos, V3* nrm, float* radius)
{
    const float* p = s->position + 4 * (size_t)i;
    *pos           = {p[0], p[1], p[2]};
    *radius        = p[3];
    if (s->normal)
        *nrm = unpack_normal(s->normal[i]);
    else
        *nrm = {0, 0, 0};
}

inline float tex_fetch(const adop_scene* s, int c, int idx)
{
    size_t o = (size_t)c * s->num_texels + idx;
    if (s->texture_dtype == ADOP_TEXTURE_F16) return half_to_float(((const uint16_t*)s->texture)[o]);
    return ((const float*)s->texture)[o];
}

// Shared head of the three point kernels (PointRenderer.cu:227-256, 334-359, 409-438).
// Returns false when the point is culled (z == 0).
inline bool project_point(const adop_scene* s, const adop_render_params* rp, const Cam& cam, int w0, int i, V3* pos,
                          V3* nrm, V2* ip, float* z, float* radius_pixels)
{
    float r;
    get_point(s, i, pos, nrm, &r);
    V2 image_p;
    if (cam.model == ADOP_CAMERA_PINHOLE_DISTORTION)
    {
        project_pinhole(*pos, *nrm, cam.V, cam.K, cam.D, rp->check_normal != 0, rp->dist_cutoff, &image_p, z);
        *radius_pixels = cam.K.fx * cam.crop.fx * r / *z;
    }
    else
    {
        project_ocam(*pos, *nrm, cam.V, cam.aff, cam.poly, cam.npoly, rp->check_normal != 0, rp->dist_cutoff,
                     &image_p, z);
        *radius_pixels = (float)w0 * cam.crop.fx * r / *z;
    }
    if (*z == 0) return false;
    *ip = k_apply(cam.crop, image_p);
    return true;
}

inline bool in_image(const adop_layer& L, int y, int x)
{
    return x >= 0 && x < L.w && y >= 0 && y < L.h;
}
inline int distance_from_edge(const adop_layer& L, int y, int x)
{
    int a = x < (L.w - 1 - x) ? x : (L.w - 1 - x);
    int b = y < (L.h - 1 - y) ? y : (L.h - 1 - y);
    return a < b ? a : b;
}
inline size_t pix(const adop_layer& L, int b, int y, int x)
{
    return ((size_t)b * L.h + y) * L.w + x;
}
inline size_t pixc(const adop_layer& L, int C, int b, int c, int y, int x)
{
    return (((size_t)b * C + c) * L.h + y) * L.w + x;
}

const float kClearDepth = 100000.f;  // PointRenderer.cu:1045

}  // namespace

// ================================================================================================
// exported C entry points (called through ctypes by tests / bench cpu_baseline)
// ================================================================================================
extern "C"
{
// BlendPointCloudForward, PointRenderer.cu:1389-1531
int oracle_forward(const adop_scene* s, const adop_view* views, int B, const adop_render_params* rp,
                   const adop_forward_buffers* fb, adop_stats* stats)
{
    const int L = fb->num_layers;
    const int C = s->num_channels;
    const int N = rp->skip_points ? 0 : s->num_points;  // if (params.render_points), :1417,1433
    if (L < 1 || L > ADOP_MAX_LAYERS) return ADOP_UNSUPPORTED_LAYERS;
    if (stats) std::memset(stats, 0, sizeof(*stats));

    // InitializeData, :1039-1090
    for (int l = 0; l < L; ++l)
    {
        const adop_layer& Ly = fb->layers[l];
        size_t n             = (size_t)B * Ly.h * Ly.w;
        uint64_t clear       = ((uint64_t)float_bits(kClearDepth) << 32) | 0xFFFFFFFFull;
        for (size_t i = 0; i < n; ++i)
        {
            Ly.depth[i]  = kClearDepth;
            Ly.weight[i] = 0;
            if (Ly.depth_index) Ly.depth_index[i] = clear;
            if (Ly.mask) Ly.mask[i] = 0;
        }
        std::memset(Ly.out, 0, n * C * sizeof(float));
    }

    // DepthPrepassMulti, :203-301 (one pass per batch image, :1415-1425)
    for (int b = 0; b < B; ++b)
    {
        Cam cam = make_cam(s, views[b]);
#pragma omp parallel for schedule(static)
        for (int i = 0; i < N; ++i)
        {
            V3 pos, nrm;
            V2 ip;
            float z, radius_pixels;
            if (!project_point(s, rp, cam, fb->layers[0].w, i, &pos, &nrm, &ip, &z, &radius_pixels)) continue;
            for (int l = 0; l < L; ++l, radius_pixels *= 0.5f, ip.x *= 0.5f, ip.y *= 0.5f)
            {
                if (rp->drop_out_points_by_radius && radius_pixels < rp->drop_out_radius_threshold) break;
                int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                const adop_layer& Ly = fb->layers[l];
                if (!in_image(Ly, py, px)) continue;
                size_t o = pix(Ly, b, py, px);
                // atomicMin on the int bits of a positive float (:281,297)
                int32_t zi = (int32_t)float_bits(z);
#ifdef _OPENMP
                if (stats)
                {
#    pragma omp atomic
                    stats->visible[l]++;
                }
                int32_t* dst = (int32_t*)&Ly.depth[o];
                int32_t cur  = __atomic_load_n(dst, __ATOMIC_RELAXED);
                while (zi < cur && !__atomic_compare_exchange_n(dst, &cur, zi, true, __ATOMIC_RELAXED, __ATOMIC_RELAXED))
                {
                }
                if (Ly.depth_index)
                {
                    uint64_t pk   = ((uint64_t)float_bits(z) << 32) | (uint32_t)i;
                    uint64_t* d64 = &Ly.depth_index[o];
                    uint64_t c64  = __atomic_load_n(d64, __ATOMIC_RELAXED);
                    while (pk < c64 &&
                           !__atomic_compare_exchange_n(d64, &c64, pk, true, __ATOMIC_RELAXED, __ATOMIC_RELAXED))
                    {
                    }
                }
#else
                if (stats) stats->visible[l]++;
                if (Ly.depth_index)
                {
                    // legacy packed buffer, PackIndex (PointRendererHelper.h:30-34), min over every
                    // in-image point-level; no early-z here so the two buffers are computed independently
                    uint64_t pk = ((uint64_t)float_bits(z) << 32) | (uint32_t)i;
                    if (pk < Ly.depth_index[o]) Ly.depth_index[o] = pk;
                }
                if (z >= Ly.depth[o]) continue;  // early-z, :278
                int32_t* dst = (int32_t*)&Ly.depth[o];
                if (zi < *dst) *dst = zi;
#endif
            }
        }
    }

    // RenderForwardMulti, :303-393
    for (int b = 0; b < B; ++b)
    {
        Cam cam              = make_cam(s, views[b]);
        const float* dropout = fb->dropout_points ? fb->dropout_points + (size_t)b * N : nullptr;
#pragma omp parallel for schedule(static)
        for (int i = 0; i < N; ++i)
        {
            if (dropout && dropout[i] == 1) continue;  // :314-315
            V3 pos, nrm;
            V2 ip;
            float z, radius_pixels;
            if (!project_point(s, rp, cam, fb->layers[0].w, i, &pos, &nrm, &ip, &z, &radius_pixels)) continue;
            int texture_index = s->index[i];
            if (texture_index < 0 || texture_index >= s->num_texels)  // device assert :362
            {
                if (stats)
                {
#pragma omp atomic
                    stats->bad_index++;
                }
                continue;
            }
            for (int l = 0; l < L; ++l, radius_pixels *= 0.5f, ip.x *= 0.5f, ip.y *= 0.5f)
            {
                if (rp->drop_out_points_by_radius && radius_pixels < rp->drop_out_radius_threshold) break;
                int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                const adop_layer& Ly = fb->layers[l];
                if (!in_image(Ly, py, px)) continue;
                float image_depth = Ly.depth[pix(Ly, b, py, px)];
                if (z > image_depth * (rp->depth_accept + 1)) continue;  // :380
                for (int c = 0; c < C; ++c)
                {
                    float t  = tex_fetch(s, c, texture_index);
                    float* d = &Ly.out[pixc(Ly, C, b, c, py, px)];
#pragma omp atomic
                    *d += t;
                }
                float* wd = &Ly.weight[pix(Ly, b, py, px)];
#pragma omp atomic
                *wd += 1.f;
                if (stats)
                {
#pragma omp atomic
                    stats->accepted[l]++;
                }
            }
        }
    }

    // CombineAndFill (:726-754) and CreateMask (:828-847)
    for (int b = 0; b < B; ++b)
        for (int l = 0; l < L; ++l)
        {
            const adop_layer& Ly = fb->layers[l];
#pragma omp parallel for schedule(static)
            for (int y = 0; y < Ly.h; ++y)
                for (int x = 0; x < Ly.w; ++x)
                {
                    float cou = Ly.weight[pix(Ly, b, y, x)];
                    for (int c = 0; c < C; ++c)
                    {
                        float* o = &Ly.out[pixc(Ly, C, b, c, y, x)];
                        if (cou == 0)
                            *o = s->background_color[c];
                        else
                            *o /= cou;
                    }
                    if (rp->output_background_mask && Ly.mask)
                        Ly.mask[pix(Ly, b, y, x)] = (cou == 0) ? rp->output_background_mask_value : 1.f;
                }
        }
    return ADOP_OK;
}

// BlendPointCloudBackward, PointRenderer.cu:1549-1644.
// Sums that the reference forms with float/double atomics over many points (background, pose, intrinsics)
// are accumulated here in double and rounded once: the order-free value any atomic ordering approximates.
int oracle_backward(const adop_scene* s, const adop_view* views, int B, const adop_render_params* rp,
                    const adop_forward_buffers* fb, const adop_backward_buffers* gb, adop_stats* stats)
{
    const int L    = fb->num_layers;
    const int C    = s->num_channels;
    const int N    = s->num_points;
    const int cols = s->intrinsics_cols;
    if (L < 1 || L > ADOP_MAX_LAYERS) return ADOP_UNSUPPORTED_LAYERS;

    // Build(info,false): zeros (:922-949)
    std::memset(gb->grad_texture, 0, sizeof(float) * (size_t)C * s->num_texels);
    if (gb->grad_points)
    {
        std::memset(gb->grad_points, 0, sizeof(float) * 4 * (size_t)N);
        std::memset(gb->grad_points_count, 0, sizeof(float) * (size_t)N);
    }
    std::vector<double> acc_bg(C, 0.0);
    std::vector<double> acc_pose((size_t)6 * s->num_poses, 0.0), cnt_pose(s->num_poses, 0.0);
    std::vector<double> acc_intr((size_t)cols * s->num_cameras, 0.0), cnt_intr(s->num_cameras, 0.0);
    if (stats)
        for (int l = 0; l < ADOP_MAX_LAYERS; ++l) stats->spatial[l] = 0;

    // CombineAndFillBackward, :851-900
    for (int b = 0; b < B; ++b)
        for (int l = 0; l < L; ++l)
        {
            const adop_layer& Ly = fb->layers[l];
            for (int c = 0; c < C; ++c)
            {
                double a = 0;
#pragma omp parallel for reduction(+ : a) schedule(static)
                for (int y = 0; y < Ly.h; ++y)
                    for (int x = 0; x < Ly.w; ++x)
                        if (Ly.weight[pix(Ly, b, y, x)] == 0) a += gb->grad_out[l][pixc(Ly, C, b, c, y, x)];
                acc_bg[c] += a;
            }
        }
    for (int c = 0; c < C; ++c) gb->grad_background[c] = (float)acc_bg[c];

    // RenderBackward, :396-724
    for (int b = 0; b < B; ++b)
    {
        Cam cam              = make_cam(s, views[b]);
        const adop_view& vw  = views[b];
        const float* dropout = fb->dropout_points ? fb->dropout_points + (size_t)b * N : nullptr;
#pragma omp parallel
        {
        // per-thread partial sums (single-threaded build: the only copy)
        std::vector<double> l_pose(acc_pose.size(), 0.0), l_cnt_pose(cnt_pose.size(), 0.0);
        std::vector<double> l_intr(acc_intr.size(), 0.0), l_cnt_intr(cnt_intr.size(), 0.0);
        uint64_t l_spatial[ADOP_MAX_LAYERS] = {0, 0, 0, 0, 0};
#pragma omp for schedule(static)
        for (int i = 0; i < N; ++i)
        {
            bool drop_out = dropout && dropout[i] == 1;
            V3 pos, nrm;
            V2 ip;
            float z, radius_pixels;
            if (!project_point(s, rp, cam, fb->layers[0].w, i, &pos, &nrm, &ip, &z, &radius_pixels)) continue;
            int texture_index = s->index[i];
            if (texture_index < 0 || texture_index >= s->num_texels) continue;
            float scale = 1;
            for (int l = 0; l < ADOP_MAX_LAYERS;
                 ++l, scale *= 0.5f, radius_pixels *= 0.5f, ip.x *= 0.5f, ip.y *= 0.5f)
            {
                if (!(l < L)) continue;
                if (rp->drop_out_points_by_radius && radius_pixels < rp->drop_out_radius_threshold) continue;
                int px = f2i_rn(ip.x), py = f2i_rn(ip.y);
                const adop_layer& Ly = fb->layers[l];
                if (!in_image(Ly, py, px)) continue;
                float image_depth = Ly.depth[pix(Ly, b, py, px)];
                if (z > image_depth * (rp->depth_accept + 1)) break;  // :462 (break, not continue)
                float w          = Ly.weight[pix(Ly, b, py, px)];
                const float* gin = gb->grad_out[l];

                if (!drop_out)
                {
                    if (w == 0) continue;  // :473
                    float iw = 1.f / w;
                    for (int c = 0; c < C; ++c)
                    {
                        float g = iw * gin[pixc(Ly, C, b, c, py, px)];
                        float* gt = &gb->grad_texture[(size_t)c * s->num_texels + texture_index];
#pragma omp atomic
                        *gt += g;
                    }
                }

                bool point_grad = (rp->ghost_gradients && drop_out) | (!rp->ghost_gradients && !drop_out);
                if (!(point_grad && distance_from_edge(Ly, py, px) > 2)) continue;
                l_spatial[l]++;

                const int nx[4] = {px - 1, px + 1, px, px};
                const int ny[4] = {py, py, py - 1, py + 1};
                float Wn[4], Dn[4];
                for (int k = 0; k < 4; ++k)
                {
                    Wn[k] = Ly.weight[pix(Ly, b, ny[k], nx[k])];
                    Dn[k] = Ly.depth[pix(Ly, b, ny[k], nx[k])];
                }
                float dR_dpx = 0, dR_dpy = 0;
                for (int c = 0; c < C; ++c)
                {
                    float T_p = tex_fetch(s, c, texture_index);
                    float v[4];
                    for (int k = 0; k < 4; ++k)
                    {
                        float I_x = Ly.out[pixc(Ly, C, b, c, ny[k], nx[k])];
                        float G_x = gin[pixc(Ly, C, b, c, ny[k], nx[k])];
                        float dI;
                        if (rp->test_backward_mode == 4)
                        {
                            float W_x = Wn[k], D_x = Dn[k];
                            if (W_x == 0 || z * (rp->depth_accept + 1) < D_x)
                                dI = T_p - I_x;  // full override
                            else if (z > D_x * (rp->depth_accept + 1))
                                dI = 0;  // discard
                            else
                                dI = (W_x / (W_x + 1) * I_x + 1 / (W_x + 1) * T_p - I_x);  // blend
                        }
                        else
                            dI = T_p - I_x;
                        v[k] = dI * G_x;
                    }
                    float a0 = -v[0], a1 = v[1], b0 = -v[2], b1 = v[3];
                    dR_dpx += 0.5f * (a0 + a1);
                    dR_dpy += 0.5f * (b0 + b1);
                }
                V2 dR_dp      = {dR_dpx / (float)C, dR_dpy / (float)C};
                Pinhole crop2 = k_scale(cam.crop, scale * 1.f);  // :614-616

                BackwardOut bo;
                if (cam.model == ADOP_CAMERA_PINHOLE_DISTORTION)
                    bo = project_pinhole_backward(pos, nrm, dR_dp, cam.V, cam.K, crop2, cam.D, rp->check_normal != 0,
                                                  rp->dist_cutoff);
                else
                    bo = project_ocam_backward(pos, nrm, dR_dp, cam.V, crop2, cam.aff, cam.poly, cam.npoly,
                                               rp->check_normal != 0, rp->dist_cutoff);

                if (gb->grad_points)
                {
                    for (int k = 0; k < 3; ++k) gb->grad_points[4 * (size_t)i + k] += bo.g_point[k];
                    gb->grad_points_count[i] += 1;
                }
                if (gb->grad_pose)
                {
                    for (int k = 0; k < 6; ++k) l_pose[6 * (size_t)vw.image_index + k] += (double)bo.g_pose[k];
                    l_cnt_pose[vw.image_index] += 1;
                }
                if (gb->grad_intrinsics_count && gb->grad_intrinsics)
                {
                    double* gi = &l_intr[(size_t)cols * vw.camera_index];
                    if (cam.model == ADOP_CAMERA_PINHOLE_DISTORTION)
                    {
                        float k_factor = rp->K_gradient_factor;
                        // the damping factors are double literals in the reference (float *= double: the product is
                        // formed in double and rounded to float once), :653-673
                        bo.g_k[4] = (float)((double)bo.g_k[4] * 0.1);
                        bo.g_k[4] = (float)((double)bo.g_k[4] * 0);  // :653-654
                        for (int k = 0; k < 5; ++k) gi[k] += (double)(k_factor * bo.g_k[k]);
                        float df = rp->distortion_gradient_factor;
                        bo.g_dis[2] = (float)((double)bo.g_dis[2] * 0.25);
                        for (int k = 3; k < 8; ++k) bo.g_dis[k] = (float)((double)bo.g_dis[k] * 0.1);
                        for (int k = 0; k < 8; ++k) gi[5 + k] += (double)(df * bo.g_dis[k]);
                        l_cnt_intr[vw.camera_index] += 1.0 / 1024.0;  // :680-681
                    }
                    else
                    {
                        for (int k = 0; k < 5; ++k) gi[k] += (double)bo.g_k[k];
                        l_cnt_intr[vw.camera_index] += 1.0;  // :718
                    }
                }
            }
        }
#pragma omp critical
        {
            for (size_t k = 0; k < acc_pose.size(); ++k) acc_pose[k] += l_pose[k];
            for (size_t k = 0; k < cnt_pose.size(); ++k) cnt_pose[k] += l_cnt_pose[k];
            for (size_t k = 0; k < acc_intr.size(); ++k) acc_intr[k] += l_intr[k];
            for (size_t k = 0; k < cnt_intr.size(); ++k) cnt_intr[k] += l_cnt_intr[k];
            if (stats)
                for (int l = 0; l < ADOP_MAX_LAYERS; ++l) stats->spatial[l] += l_spatial[l];
        }
        }  // omp parallel
    }

    // NormalizeGradient, :1534-1547 and its three launches :1611-1636
    if (gb->grad_pose)
    {
        for (int f = 0; f < s->num_poses; ++f)
        {
            float c = (float)cnt_pose[f];
            gb->grad_pose_count[f] = c;
            for (int k = 0; k < 6; ++k)
            {
                double t = acc_pose[6 * (size_t)f + k];
                gb->grad_pose[6 * (size_t)f + k] = (c > 0) ? t / (double)c : t;
            }
        }
    }
    if (gb->grad_points)
    {
        if (rp->normalize_mode == 0)
        {
            // vec3 view of the [N,4] buffer (:1625): element t covers floats 3t..3t+2, divided by count[t]
            for (int t = 0; t < N; ++t)
            {
                float c = gb->grad_points_count[t];
                if (c > 0)
                    for (int k = 0; k < 3; ++k) gb->grad_points[3 * (size_t)t + k] /= c;
            }
        }
        else
        {
            for (int t = 0; t < N; ++t)
            {
                float c = gb->grad_points_count[t];
                if (c > 0)
                    for (int k = 0; k < 3; ++k) gb->grad_points[4 * (size_t)t + k] /= c;
            }
        }
    }
    if (gb->grad_intrinsics && gb->grad_intrinsics_count)
    {
        size_t total = (size_t)cols * s->num_cameras;
        for (size_t k = 0; k < total; ++k) gb->grad_intrinsics[k] = (float)acc_intr[k];
        for (int k = 0; k < s->num_cameras; ++k) gb->grad_intrinsics_count[k] = (float)cnt_intr[k];
        if (rp->normalize_mode == 0)
        {
            // always Vector<float,13> rows (:1633), whatever the real row width; stay inside the buffer
            for (int t = 0; t < s->num_cameras; ++t)
            {
                float c = gb->grad_intrinsics_count[t];
                if (c > 0)
                    for (int k = 0; k < 13; ++k)
                        if ((size_t)13 * t + k < total) gb->grad_intrinsics[(size_t)13 * t + k] /= c;
            }
        }
        else
        {
            for (int t = 0; t < s->num_cameras; ++t)
            {
                float c = gb->grad_intrinsics_count[t];
                if (c > 0)
                    for (int k = 0; k < cols; ++k) gb->grad_intrinsics[(size_t)cols * t + k] /= c;
            }
        }
    }
    return ADOP_OK;
}

// BuildSphericalUV + SphericalCoordinates (EnvironmentMap.cu:41-105) for one view at one level.
// uv_out [h,w,2]
void oracle_env_uv(const adop_scene* s, const adop_view* view, int level, int w, int h, float* uv_out)
{
    Cam cam    = make_cam(s, *view);
    float sc   = 1;
    for (int l = 0; l < level; ++l) sc /= 2;  // EnvironmentMap.cu:131,134
    Pinhole cr = k_scale(cam.crop, sc);
    // V.inverse(): rotation conj(q), translation -(R^T t)
    V3 t    = {cam.V.tx, cam.V.ty, cam.V.tz};
    V3 rt   = rotate_inv(cam.V, t);
    V3 tinv = {-rt.x, -rt.y, -rt.z};
    for (int gy = 0; gy < h; ++gy)
        for (int gx = 0; gx < w; ++gx)
        {
            V2 ip = {(float)gx, (float)gy};
            V3 inp;
            if (cam.model == ADOP_CAMERA_PINHOLE_DISTORTION)
            {
                V2 dist_p = k_unproject2(cam.K, k_unproject2(cr, ip));
                V2 np     = undistort_simple(dist_p, cam.D);
                inp       = {np.x, np.y, 1};
            }
            else  // OCam views (not in the reference: EnvironmentMap.cu:129 asserts pinhole)
                inp = ocam_unproject(cam.aff, cam.poly, cam.npoly, k_unproject2(cr, ip));
            V3 r      = rotate_inv(cam.V, inp);
            V3 wp     = {r.x + tinv.x, r.y + tinv.y, r.z + tinv.z};
            V3 d      = {wp.x - tinv.x, wp.y - tinv.y, wp.z - tinv.z};
            float n   = std::sqrt(dot(d, d));
            d         = {d.x / n, d.y / n, d.z / n};
            float phi = o_atan2f(-d.z, d.x);
            float x   = phi / (2.0f * kPi);
            x         = x - std::floor(x);  // fract
            float th  = o_acosf(d.y);
            float y   = 1 - th / kPi;
            uv_out[((size_t)gy * w + gx) * 2 + 0] = x * 2 - 1;
            uv_out[((size_t)gy * w + gx) * 2 + 1] = y * 2 - 1;
        }
}

// grid_sample(bilinear, border, align_corners=true) of tex [C,eh,ew] at uv [h,w,2] -> out [C,h,w]
void oracle_grid_sample(const float* tex, int C, int eh, int ew, const float* uv, int w, int h, float* out)
{
    for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
        {
            float u  = uv[((size_t)y * w + x) * 2 + 0];
            float v  = uv[((size_t)y * w + x) * 2 + 1];
            float fx = (u + 1) * 0.5f * (float)(ew - 1);
            float fy = (v + 1) * 0.5f * (float)(eh - 1);
            fx       = std::fmin(std::fmax(fx, 0.f), (float)(ew - 1));
            fy       = std::fmin(std::fmax(fy, 0.f), (float)(eh - 1));
            int x0 = (int)std::floor(fx), y0 = (int)std::floor(fy);
            int x1 = x0 + 1, y1 = y0 + 1;
            float ax = fx - (float)x0, ay = fy - (float)y0;
            float w00 = (1 - ax) * (1 - ay), w01 = ax * (1 - ay), w10 = (1 - ax) * ay, w11 = ax * ay;
            for (int c = 0; c < C; ++c)
            {
                const float* t = tex + (size_t)c * eh * ew;
                float a        = 0;
                a += t[(size_t)y0 * ew + x0] * w00;
                if (x1 < ew) a += t[(size_t)y0 * ew + x1] * w01;
                if (y1 < eh) a += t[(size_t)y1 * ew + x0] * w10;
                if (x1 < ew && y1 < eh) a += t[(size_t)y1 * ew + x1] * w11;
                out[((size_t)c * h + y) * w + x] = a;
            }
        }
}

// Sophus::se3_expd(t) * pose, tangent = 0 (ApplyTangent, PointRenderer.cu:1646-1657).  f64.
void oracle_apply_tangent(double* tangent, double* poses, int n)
{
    for (int i = 0; i < n; ++i)
    {
        double* t = tangent + 6 * (size_t)i;
        double* p = poses + 8 * (size_t)i;
        double ux = t[0], uy = t[1], uz = t[2], wx = t[3], wy = t[4], wz = t[5];
        double th2 = wx * wx + wy * wy + wz * wz;
        double th  = std::sqrt(th2);
        // SO3::exp -> quaternion
        double im, re;
        if (th < 1e-10)
        {
            double th4 = th2 * th2;
            im         = 0.5 - th2 / 48.0 + th4 / 3840.0;
            re         = 1.0 - th2 / 8.0 + th4 / 384.0;
        }
        else
        {
            im = std::sin(0.5 * th) / th;
            re = std::cos(0.5 * th);
        }
        double ex = im * wx, ey = im * wy, ez = im * wz, ew = re;
        // V * upsilon, V = I + (1-cos)/th^2 * W + (th - sin)/th^3 * W^2
        double a, bb;
        if (th < 1e-10)
        {
            a  = 0.5;
            bb = 1.0 / 6.0;
        }
        else
        {
            a  = (1.0 - std::cos(th)) / th2;
            bb = (th - std::sin(th)) / (th2 * th);
        }
        double c1x = wy * uz - wz * uy, c1y = wz * ux - wx * uz, c1z = wx * uy - wy * ux;          // w x u
        double c2x = wy * c1z - wz * c1y, c2y = wz * c1x - wx * c1z, c2z = wx * c1y - wy * c1x;    // w x (w x u)
        double etx = ux + a * c1x + bb * c2x, ety = uy + a * c1y + bb * c2y, etz = uz + a * c1z + bb * c2z;
        // compose: q' = e * q ; t' = e.R * t + et
        double qx = p[0], qy = p[1], qz = p[2], qw = p[3];
        double nx = ew * qx + ex * qw + ey * qz - ez * qy;
        double ny = ew * qy - ex * qz + ey * qw + ez * qx;
        double nz = ew * qz + ex * qy - ey * qx + ez * qw;
        double nw = ew * qw - ex * qx - ey * qy - ez * qz;
        double tx = p[4], ty = p[5], tz = p[6];
        double uvx = 2 * (ey * tz - ez * ty), uvy = 2 * (ez * tx - ex * tz), uvz = 2 * (ex * ty - ey * tx);
        double rx = tx + ew * uvx + (ey * uvz - ez * uvy);
        double ry = ty + ew * uvy + (ez * uvx - ex * uvz);
        double rz = tz + ew * uvz + (ex * uvy - ey * uvx);
        double qn = std::sqrt(nx * nx + ny * ny + nz * nz + nw * nw);
        p[0] = nx / qn;
        p[1] = ny / qn;
        p[2] = nz / qn;
        p[3] = nw / qn;
        p[4] = rx + etx;
        p[5] = ry + ety;
        p[6] = rz + etz;
        for (int k = 0; k < 6; ++k) t[k] = 0;
    }
}

// ---- unit-level entry points for the pinning tests -------------------------------------------------
float oracle_atanf(float x) { return o_atanf(x); }
float oracle_atan2f(float y, float x) { return o_atan2f(y, x); }
float oracle_acosf(float x) { return o_acosf(x); }
int oracle_f2i_rn(float x) { return f2i_rn(x); }
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }
int32_t oracle_pack_normal(float x, float y, float z) { return pack_normal({x, y, z}); }
void oracle_unpack_normal(int32_t enc, float* out)
{
    V3 n   = unpack_normal(enc);
    out[0] = n.x;
    out[1] = n.y;
    out[2] = n.z;
}
uint64_t oracle_pack_index(float depth, uint32_t index) { return ((uint64_t)float_bits(depth) << 32) | index; }

// pose8: SE3d row; intr: 13 floats; out: (u, v, z)
void oracle_project_pinhole(const float* p, const float* n, const double* pose8, const float* intr, int check_normal,
                            float dist_cutoff, float* out)
{
    Pose V       = load_pose(pose8);
    Pinhole K    = {intr[0], intr[1], intr[2], intr[3], intr[4]};
    Distortion D = {intr[5], intr[6], intr[7], intr[8], intr[9], intr[10], intr[11], intr[12]};
    V2 ip;
    float z;
    project_pinhole({p[0], p[1], p[2]}, {n[0], n[1], n[2]}, V, K, D, check_normal != 0, dist_cutoff, &ip, &z);
    out[0] = ip.x;
    out[1] = ip.y;
    out[2] = z;
}
void oracle_project_ocam(const float* p, const float* n, const double* pose8, const float* intr, int cols,
                         int check_normal, float dist_cutoff, float* out)
{
    Pose V = load_pose(pose8);
    V2 ip;
    float z;
    project_ocam({p[0], p[1], p[2]}, {n[0], n[1], n[2]}, V, intr, intr + 5, cols - 5, check_normal != 0, dist_cutoff,
                 &ip, &z);
    out[0] = ip.x;
    out[1] = ip.y;
    out[2] = z;
}
// out: g_point[3], g_pose[6], g_k[5], g_dis[8]  (22 floats)
void oracle_project_pinhole_backward(const float* p, const float* n, const float* grad, const double* pose8,
                                     const float* intr, const float* crop5, int check_normal, float dist_cutoff,
                                     float* out)
{
    Pose V       = load_pose(pose8);
    Pinhole K    = {intr[0], intr[1], intr[2], intr[3], intr[4]};
    Distortion D = {intr[5], intr[6], intr[7], intr[8], intr[9], intr[10], intr[11], intr[12]};
    Pinhole crop = {crop5[0], crop5[1], crop5[2], crop5[3], crop5[4]};
    BackwardOut o = project_pinhole_backward({p[0], p[1], p[2]}, {n[0], n[1], n[2]}, {grad[0], grad[1]}, V, K, crop, D,
                                             check_normal != 0, dist_cutoff);
    std::memcpy(out, &o, sizeof(o));
}
void oracle_project_ocam_backward(const float* p, const float* n, const float* grad, const double* pose8,
                                  const float* intr, int cols, const float* crop5, int check_normal,
                                  float dist_cutoff, float* out)
{
    Pose V        = load_pose(pose8);
    Pinhole crop  = {crop5[0], crop5[1], crop5[2], crop5[3], crop5[4]};
    BackwardOut o = project_ocam_backward({p[0], p[1], p[2]}, {n[0], n[1], n[2]}, {grad[0], grad[1]}, V, crop, intr,
                                          intr + 5, cols - 5, check_normal != 0, dist_cutoff);
    std::memcpy(out, &o, sizeof(o));
}
void oracle_distort(const float* p, const float* dist8, float max_r, float* out2, float* Jp4, float* Jd16)
{
    Distortion D = {dist8[0], dist8[1], dist8[2], dist8[3], dist8[4], dist8[5], dist8[6], dist8[7]};
    V2 r         = distort({p[0], p[1]}, D, max_r, Jp4, Jd16);
    out2[0]      = r.x;
    out2[1]      = r.y;
}
void oracle_undistort(const float* p, const float* dist8, float* out2)
{
    Distortion D = {dist8[0], dist8[1], dist8[2], dist8[3], dist8[4], dist8[5], dist8[6], dist8[7]};
    V2 r         = undistort_simple({p[0], p[1]}, D);
    out2[0]      = r.x;
    out2[1]      = r.y;
}
void oracle_sincosf(float theta, float* out2) { o_sincosf(theta, out2, out2 + 1); }
// intr: (c,d,e,cx,cy) + world2cam polynomial, cols floats; ip: pixel of the uncropped image; out: unit ray (camera)
void oracle_ocam_unproject(const float* intr, int cols, const float* ip, float* out3)
{
    V3 r    = ocam_unproject(intr, intr + 5, cols - 5, {ip[0], ip[1]});
    out3[0] = r.x;
    out3[1] = r.y;
    out3[2] = r.z;
}
// view-space point -> (u, v, z) through the OCam model alone (no pose, no normal test)
void oracle_ocam_core(const float* p, const float* intr, int cols, float cutoff, float* out3)
{
    V2 uv;
    float z;
    project_ocam_core({p[0], p[1], p[2]}, intr, intr + 5, cols - 5, cutoff, &uv, &z, nullptr, nullptr);
    out3[0] = uv.x;
    out3[1] = uv.y;
    out3[2] = z;
}
int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
}  // extern "C"
