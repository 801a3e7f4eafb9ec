// device_math.h — per-point camera arithmetic of the rasterizer kernels (gfx950 device code).
//
// Every function states the reference routine it stands for (paths inside the darglein/ADOP tree; the saiga
// routines are named by their call sites).  The operation ORDER written here is part of the contract: the file
// is compiled with -ffp-contract=off, IEEE division and square root, so depth bits and pixel coordinates are
// reproducible by any implementation that performs the same + - * / sqrt sequence.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#pragma clang fp contract(off)

namespace adop
{
struct V2
{
    float x, y;
};
struct V3
{
    float x, y, z;
};

// One view, prepared on the device from poses_se3 / intrinsics by prepare_views_kernel.
struct ViewConst
{
    float qx, qy, qz, qw;  // world->camera rotation (unit quaternion, float)
    float tx, ty, tz;
    float k[5];     // fx fy cx cy s
    float d[8];     // k1..k6 p1 p2
    float crop[5];  // crop_transform fx fy cx cy s
    int32_t w, h;
    int32_t image_index, camera_index;
    int32_t model;        // 0 pinhole+distortion, 1 OCam
    int32_t intr_offset;  // first float of this camera's row in `intrinsics`
    int32_t npoly;        // OCam: number of world2cam coefficients
    int32_t no_distortion;  // pinhole: all eight distortion coefficients are zero
};

__device__ __forceinline__ uint32_t f2u(float f)
{
    return __float_as_uint(f);
}

// __float2int_rn semantics (PointRenderer.cu:266): nearest-even, saturating, NaN -> 0.
// v_rndne_f32 + v_cvt_i32_f32: the conversion instruction itself saturates out-of-range values and turns NaN into 0
// (a C++ cast would be undefined there, and spelling the three cases out costs six more instructions per pixel
// coordinate in kernels that are bound by instruction issue).
__device__ __forceinline__ int f2i_rn(float f)
{
    const float r = rintf(f);
    int i;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(r));
    return i;
}

// Fixed-polynomial arctangent family (Cephes single precision), + - * / sqrt only.
#define ADOP_PI 3.14159265358979323846f
#define ADOP_HALF_PI 1.57079632679489661923f
#define ADOP_QUART_PI 0.78539816339744830962f

__device__ __forceinline__ float atan_poly(float xx)
{
    float x = xx < 0 ? -xx : xx;
    float y;
    if (x > 2.414213562373095f)
    {
        y = ADOP_HALF_PI;
        x = -(1.0f / x);
    }
    else if (x > 0.4142135623730950f)
    {
        y = ADOP_QUART_PI;
        x = (x - 1.0f) / (x + 1.0f);
    }
    else
        y = 0.0f;
    float z = x * x;
    float p = (((8.05374449538e-2f * z - 1.38776856032e-1f) * z + 1.99777106478e-1f) * z - 3.33329491539e-1f);
    y       = y + (p * z * x + x);
    return xx < 0 ? -y : y;
}

__device__ __forceinline__ float atan2_poly(float y, float x)
{
    if (x == 0.0f)
    {
        if (y > 0.0f) return ADOP_HALF_PI;
        if (y < 0.0f) return -ADOP_HALF_PI;
        return 0.0f;
    }
    float a = atan_poly(y / x);
    if (x < 0.0f) return (y < 0.0f) ? a - ADOP_PI : a + ADOP_PI;
    return a;
}

__device__ __forceinline__ float asin_poly(float xx)
{
    float a = xx < 0 ? -xx : xx;
    if (a > 1.0f) a = 1.0f;
    bool flag = a > 0.5f;
    float z, x;
    if (flag)
    {
        z = 0.5f * (1.0f - a);
        x = sqrtf(z);
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
        r = ADOP_HALF_PI - r;
    }
    return xx < 0 ? -r : r;
}

__device__ __forceinline__ float acos_poly(float x)
{
    if (x < -0.5f) return ADOP_PI - 2.0f * asin_poly(sqrtf(0.5f * (1.0f + x)));
    if (x > 0.5f) return 2.0f * asin_poly(sqrtf(0.5f * (1.0f - x)));
    return ADOP_HALF_PI - asin_poly(x);
}

// sine and cosine of an angle in [-pi/2, pi/2] (Cephes single-precision kernels on [-pi/4, pi/4], the rest through
// the complementary angle), + - * only.
__device__ __forceinline__ void sincos_poly(float theta, float* s_out, float* c_out)
{
    float a     = theta < 0 ? -theta : theta;
    bool compl_ = a > ADOP_QUART_PI;
    float x     = compl_ ? ADOP_HALF_PI - a : a;
    float z     = x * x;
    float sn    = ((-1.9515295891e-4f * z + 8.3321608736e-3f) * z - 1.6666654611e-1f) * z * x + x;
    float cs    = ((2.443315711809948e-5f * z - 1.388731625493765e-3f) * z + 4.166664568298827e-2f) * z * z +
               (1.0f - 0.5f * z);
    float s = compl_ ? cs : sn;
    float c = compl_ ? sn : cs;
    *s_out  = theta < 0 ? -s : s;
    *c_out  = c;
}

__device__ __forceinline__ V3 cross3(V3 a, V3 b)
{
    return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ __forceinline__ float dot3(V3 a, V3 b)
{
    return (a.x * b.x + a.y * b.y) + a.z * b.z;
}

// SO3f * v as Eigen evaluates it (Quaternion::_transformVector), used by Sophus for V.so3()*n and V*p
// (PointRendererHelper.h:55,63).
__device__ __forceinline__ V3 quat_rotate(float qx, float qy, float qz, float qw, V3 v)
{
    V3 q  = {qx, qy, qz};
    V3 uv = cross3(q, v);
    uv.x += uv.x;
    uv.y += uv.y;
    uv.z += uv.z;
    V3 c = cross3(q, uv);
    return {(v.x + qw * uv.x) + c.x, (v.y + qw * uv.y) + c.y, (v.z + qw * uv.z) + c.z};
}

// UnpackNormal10Bit (NeuralPointCloudCuda.h:96): three 10-bit fields, x in bits 0..9, mapped to [-1,1].
__device__ __forceinline__ V3 unpack_normal10(int32_t enc)
{
    uint32_t e    = (uint32_t)enc;
    const float s = 2.0f / 1023.0f;
    return {(float)(e & 1023u) * s - 1.0f, (float)((e >> 10) & 1023u) * s - 1.0f,
            (float)((e >> 20) & 1023u) * s - 1.0f};
}

// IntrinsicsPinhole::normalizedToImage
__device__ __forceinline__ V2 k_apply(const float* K, V2 p)
{
    return {(K[0] * p.x + K[4] * p.y) + K[2], K[1] * p.y + K[3]};
}

// distortNormalizedPoint (PointRendererHelper.h:72,151): OpenCV rational + tangential model, sentinel
// (100000,100000) beyond the cutoff radius.  Jp: 2x2, Jd: 2x8 (k1..k6,p1,p2), both row-major, optional.
template <bool WITH_J>
__device__ __forceinline__ V2 distort(V2 p, const float* D, float max_r, float* Jp, float* Jd)
{
    float k1 = D[0], k2 = D[1], k3 = D[2], k4 = D[3], k5 = D[4], k6 = D[5], p1 = D[6], p2 = D[7];
    float x = p.x, y = p.y;
    float x2 = x * x, y2 = y * y;
    float r2  = x2 + y2;
    float xy2 = 2.0f * x * y;
    float r4  = r2 * r2;
    float r6  = r2 * r4;
    float U   = 1.0f + k1 * r2 + k2 * r4 + k3 * r6;
    float Vv  = 1.0f + k4 * r2 + k5 * r4 + k6 * r6;
    float iV  = 1.0f / Vv;
    float rad = U * iV;
    float tx  = p1 * xy2 + p2 * (r2 + 2.0f * x2);
    float ty  = p1 * (r2 + 2.0f * y2) + p2 * xy2;
    V2 out    = {x * rad + tx, y * rad + ty};
    if (WITH_J)
    {
        float dU  = k1 + 2.0f * k2 * r2 + 3.0f * k3 * r4;
        float dV  = k4 + 2.0f * k5 * r2 + 3.0f * k6 * r4;
        float dr  = (dU * Vv - U * dV) * iV * iV;
        float drx = dr * 2.0f * x, dry = dr * 2.0f * y;
        Jp[0]     = rad + x * drx + p1 * 2.0f * y + p2 * 6.0f * x;
        Jp[1]     = x * dry + p1 * 2.0f * x + p2 * 2.0f * y;
        Jp[2]     = y * drx + p1 * 2.0f * x + p2 * 2.0f * y;
        Jp[3]     = rad + y * dry + p1 * 6.0f * y + p2 * 2.0f * x;
        float a   = -U * iV * iV;
        float cu0 = r2 * iV, cu1 = r4 * iV, cu2 = r6 * iV;
        float cv0 = r2 * a, cv1 = r4 * a, cv2 = r6 * a;
        Jd[0] = x * cu0; Jd[1] = x * cu1; Jd[2] = x * cu2;
        Jd[3] = x * cv0; Jd[4] = x * cv1; Jd[5] = x * cv2;
        Jd[6] = xy2;     Jd[7] = r2 + 2.0f * x2;
        Jd[8] = y * cu0; Jd[9] = y * cu1; Jd[10] = y * cu2;
        Jd[11] = y * cv0; Jd[12] = y * cv1; Jd[13] = y * cv2;
        Jd[14] = r2 + 2.0f * y2; Jd[15] = xy2;
    }
    if (r2 > max_r * max_r)
    {
        out.x = 100000.f;
        out.y = 100000.f;
    }
    return out;
}

// ProjectOCam (PointRendererHelper.h:95,211): Scaramuzza world2cam polynomial for a camera looking along +z.
template <bool WITH_J>
__device__ __forceinline__ void ocam_core(V3 p, const float* aff, const float* poly, int npoly, float cutoff, V2* uv,
                                          float* z_out, float* Jp, float* Ja)
{
    float c = aff[0], d = aff[1], e = aff[2], cx = aff[3], cy = aff[4];
    float x = p.x, y = p.y, z = p.z;
    float r2   = x * x + y * y;
    float norm = sqrtf(r2);
    float dist = sqrtf(r2 + z * z);
    if (norm == 0.0f)
    {
        *uv    = {cx, cy};
        *z_out = z > 0 ? dist : 0.0f;
        if (WITH_J)
        {
            for (int i = 0; i < 6; ++i) Jp[i] = 0;
            for (int i = 0; i < 10; ++i) Ja[i] = 0;
            Ja[3] = 1;
            Ja[9] = 1;
        }
        return;
    }
    float theta = atan_poly(-z / norm);
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
    if (WITH_J)
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
        Jp[0] = c * uux + d * vvx; Jp[1] = c * uuy + d * vvy; Jp[2] = c * uuz + d * vvz;
        Jp[3] = e * uux + vvx;     Jp[4] = e * uuy + vvy;     Jp[5] = e * uuz + vvz;
        Ja[0] = uu; Ja[1] = vv; Ja[2] = 0;  Ja[3] = 1; Ja[4] = 0;
        Ja[5] = 0;  Ja[6] = 0;  Ja[7] = uu; Ja[8] = 0; Ja[9] = 1;
    }
}

// Pixel of the uncropped OCam image -> unit ray in camera space, the inverse of ocam_core (the reference has none: its
// environment map asserts the pinhole model, EnvironmentMap.cu:129): undo the affine map, solve poly(theta) = rho with
// kOcamNewtonSteps Newton steps from the axis (theta = -pi/2), theta kept in [-pi/2, pi/2]; the ray is
// (cos(theta) * (uu,vv)/rho, -sin(theta)), so that theta = atan(-z / |xy|) as in the forward direction.
constexpr int kOcamNewtonSteps = 5;
__device__ __forceinline__ V3 ocam_unproject(const float* aff, const float* poly, int npoly, V2 ip)
{
    float c = aff[0], d = aff[1], e = aff[2], cx = aff[3], cy = aff[4];
    float px = ip.x - cx, py = ip.y - cy;
    float det   = c - d * e;
    float uu    = (px - d * py) / det;
    float vv    = (c * py - e * px) / det;
    float rho   = sqrtf(uu * uu + vv * vv);
    float theta = -ADOP_HALF_PI;
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
        theta = fminf(fmaxf(theta, -ADOP_HALF_PI), ADOP_HALF_PI);
    }
    float sn, cs;
    sincos_poly(theta, &sn, &cs);
    float cxn = rho > 0 ? uu / rho : 0.f;
    float cyn = rho > 0 ? vv / rho : 0.f;
    return {cxn * cs, cyn * cs, -sn};
}

// Head of the three reference point kernels (PointRenderer.cu:227-256, 334-359, 409-438), in two parts.
// First part, the same for every crop of one frame (pose and camera model): ProjectPointPinhole / ProjectPointOcam
// (PointRendererHelper.h:49-106) up to the point in the uncropped image.  Returns false when the point is culled
// (z == 0).
__device__ __forceinline__ bool project_frame(const ViewConst& vc, const float* __restrict__ intrinsics, V3 pos, V3 nrm,
                                              bool check_normal, float dist_cutoff, V2* image_p_out, float* z_out,
                                              V3* view_p_out)
{
    V3 r      = quat_rotate(vc.qx, vc.qy, vc.qz, vc.qw, pos);
    V3 view_p = {r.x + vc.tx, r.y + vc.ty, r.z + vc.tz};
    *view_p_out = view_p;
    V2 image_p = {0.f, 0.f};
    float z;
    if (vc.model == 0)
    {
        z = fmaxf(view_p.z, 0.f);
        if (check_normal)
        {
            V3 view_n = quat_rotate(vc.qx, vc.qy, vc.qz, vc.qw, nrm);
            if (dot3(view_p, view_n) > 0) z = 0;
        }
        // culled: nothing below can bring the point back; Morton-ordered clouds cull whole wavefronts here
        if (z == 0)
        {
            *z_out       = 0;
            *image_p_out = image_p;
            return false;
        }
        float iz  = 1.0f / view_p.z;
        V2 norm_p = {view_p.x * iz, view_p.y * iz};
        // A camera without distortion (the coefficients all zero): distortNormalizedPoint returns its argument, bit for
        // bit up to the sign of a zero, as long as r^6 is finite (0 * inf would make the polynomial NaN).  Taken when
        // that holds for every lane of the wavefront: a third of the projection's instructions.
        const float r2 = norm_p.x * norm_p.x + norm_p.y * norm_p.y;
        V2 dist_p;
        if (vc.no_distortion && __ballot(!(r2 < 1.0e12f)) == 0)
        {
            dist_p = norm_p;
            if (r2 > dist_cutoff * dist_cutoff) dist_p = {100000.f, 100000.f};
        }
        else
            dist_p = distort<false>(norm_p, vc.d, dist_cutoff, nullptr, nullptr);
        if (dist_p.x == 100000.f) z = 0;
        image_p = k_apply(vc.k, dist_p);
    }
    else
    {
        const float* row = intrinsics + vc.intr_offset;
        ocam_core<false>(view_p, row, row + 5, vc.npoly, dist_cutoff, &image_p, &z, nullptr, nullptr);
        V3 view_n = quat_rotate(vc.qx, vc.qy, vc.qz, vc.qw, nrm);
        if (check_normal & (dot3(view_p, view_n) > 0)) z = 0;
    }
    *z_out       = z;
    *image_p_out = image_p;
    return z != 0;
}

// Second part, per crop: the LOD radius in pixels and the crop transform of a point that project_frame kept.
__device__ __forceinline__ float crop_radius(const ViewConst& vc, float z, float radius, int w0)
{
    return (vc.model == 0 ? vc.k[0] : (float)w0) * vc.crop[0] * radius / z;
}

__device__ __forceinline__ void project_crop(const ViewConst& vc, V2 image_p, float z, float radius, int w0, V2* ip,
                                             float* radius_pixels)
{
    *radius_pixels = crop_radius(vc, z, radius, w0);
    *ip            = k_apply(vc.crop, image_p);
}

// A level-0 image point outside this box lands outside the image at every level: level l takes the pixel
// rint(ip * 0.5^l) (an exact scaling), which is inside only if -0.5 <= ip * 0.5^l <= w_l - 0.5.  The box is wider than
// that by a pixel of the coarsest level on every side; a NaN is never outside (its pixel is 0, as in the reference).
struct ImageBox
{
    float lo, hi_x, hi_y;
};

template <class LevelsT>
__device__ __forceinline__ ImageBox image_box(const LevelsT& lv)
{
    ImageBox box = {-(float)(1 << lv.num), 0.f, 0.f};
#pragma unroll
    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
        if (l < lv.num)
        {
            box.hi_x = fmaxf(box.hi_x, (float)(lv.l[l].w + 1) * (float)(1 << l));
            box.hi_y = fmaxf(box.hi_y, (float)(lv.l[l].h + 1) * (float)(1 << l));
        }
    return box;
}

__device__ __forceinline__ bool outside_every_level(const ImageBox& box, V2 ip)
{
    return ip.x < box.lo || ip.x > box.hi_x || ip.y < box.lo || ip.y > box.hi_y;
}

__device__ __forceinline__ bool project_point(const ViewConst& vc, const float* __restrict__ intrinsics, V3 pos,
                                              V3 nrm, float radius, bool check_normal, float dist_cutoff, int w0,
                                              V2* ip, float* z_out, float* radius_pixels, V3* view_p_out)
{
    V2 image_p;
    *radius_pixels = 0;
    if (!project_frame(vc, intrinsics, pos, nrm, check_normal, dist_cutoff, &image_p, z_out, view_p_out)) return false;
    project_crop(vc, image_p, *z_out, radius, w0, ip, radius_pixels);
    return true;
}

struct BackwardOut
{
    float g_point[3];
    float g_pose[6];
    float g_k[5];    // pinhole K (fx,fy,cx,cy,s) or OCam affine (c,d,e,cx,cy)
    float g_dis[8];  // pinhole distortion
};

// ProjectPointPinholeBackward / ProjectPointOcamBackward (PointRendererHelper.h:120-170, 184-227):
// J_point^T J_div^T J_dis^T J_K^T J_crop^T g.  The pose Jacobian is that of a left perturbation
// exp(eps)*V with translation first: J_pose = [I | -[V p]x], so J_pose^T c = (c, (V p) x c).
__device__ __forceinline__ void project_point_backward(const ViewConst& vc, const float* __restrict__ intrinsics,
                                                       V3 view_p, V2 grad, const float* crop, float dist_cutoff,
                                                       BackwardOut* o)
{
    V2 g2 = {crop[0] * grad.x, crop[4] * grad.x + crop[1] * grad.y};
    V3 c;
    if (vc.model == 0)
    {
        float iz  = 1.0f / view_p.z;
        V2 norm_p = {view_p.x * iz, view_p.y * iz};
        float Jp[4], Jd[16];
        V2 dist_p = distort<true>(norm_p, vc.d, dist_cutoff, Jp, Jd);
        V2 g1     = {vc.k[0] * g2.x, vc.k[4] * g2.x + vc.k[1] * g2.y};
        V2 g0     = {Jp[0] * g1.x + Jp[2] * g1.y, Jp[1] * g1.x + Jp[3] * g1.y};
        c         = {g0.x * iz, g0.y * iz, (-(view_p.x * iz * iz)) * g0.x + (-(view_p.y * iz * iz)) * g0.y};
        o->g_k[0] = dist_p.x * g2.x;
        o->g_k[1] = dist_p.y * g2.y;
        o->g_k[2] = g2.x;
        o->g_k[3] = g2.y;
        o->g_k[4] = dist_p.y * g2.x;
#pragma unroll
        for (int i = 0; i < 8; ++i) o->g_dis[i] = Jd[i] * g1.x + Jd[8 + i] * g1.y;
    }
    else
    {
        const float* row = intrinsics + vc.intr_offset;
        float Jp[6], Ja[10];
        V2 uv;
        float z;
        ocam_core<true>(view_p, row, row + 5, vc.npoly, dist_cutoff, &uv, &z, Jp, Ja);
        c = {Jp[0] * g2.x + Jp[3] * g2.y, Jp[1] * g2.x + Jp[4] * g2.y, Jp[2] * g2.x + Jp[5] * g2.y};
#pragma unroll
        for (int i = 0; i < 5; ++i) o->g_k[i] = Ja[i] * g2.x + Ja[5 + i] * g2.y;
#pragma unroll
        for (int i = 0; i < 8; ++i) o->g_dis[i] = 0;
    }
    V3 gp         = quat_rotate(-vc.qx, -vc.qy, -vc.qz, vc.qw, c);
    o->g_point[0] = gp.x;
    o->g_point[1] = gp.y;
    o->g_point[2] = gp.z;
    V3 rc         = cross3(view_p, c);
    o->g_pose[0]  = c.x;
    o->g_pose[1]  = c.y;
    o->g_pose[2]  = c.z;
    o->g_pose[3]  = rc.x;
    o->g_pose[4]  = rc.y;
    o->g_pose[5]  = rc.z;
}

}  // namespace adop
