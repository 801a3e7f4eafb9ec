// env_kernels.hip — environment-map kernels (EnvironmentMap.cu:41-157, RenderModule.cpp:106-127) and ApplyTangent.
#include "common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace adop
{
// ------------------------------------------------------------------------------------------------
// environment map (EnvironmentMap.cu:41-157) and its composition (RenderModule.cpp:106-127)
// ------------------------------------------------------------------------------------------------

__device__ __forceinline__ V2 k_unproject2(const float* K, V2 ip)
{
    float y = (ip.y - K[3]) / K[1];
    float x = ((ip.x - K[2]) - K[4] * y) / K[0];
    return {x, y};
}

// undistortNormalizedPointSimple: OpenCV fixed-point iteration, 5 rounds.
__device__ __forceinline__ V2 undistort_simple(V2 p, const float* D)
{
    float k1 = D[0], k2 = D[1], k3 = D[2], k4 = D[3], k5 = D[4], k6 = D[5], p1 = D[6], p2 = D[7];
    float x0 = p.x, y0 = p.y, x = p.x, y = p.y;
    for (int it = 0; it < 5; ++it)
    {
        float r2     = x * x + y * y;
        float icdist = (1.0f + ((k6 * r2 + k5) * r2 + k4) * r2) / (1.0f + ((k3 * r2 + k2) * r2 + k1) * r2);
        float dx     = 2.0f * p1 * x * y + p2 * (r2 + 2.0f * x * x);
        float dy     = p1 * (r2 + 2.0f * y * y) + 2.0f * p2 * x * y;
        x            = (x0 - dx) * icdist;
        y            = (y0 - dy) * icdist;
    }
    return {x, y};
}

// BuildSphericalUV + SphericalCoordinates for pixel (gx,gy) of a level whose crop is scaled by `sc`.
__device__ __forceinline__ V2 spherical_uv(const ViewConst& vc, const float* __restrict__ intrinsics, float sc, int gx,
                                           int gy)
{
    float cr[5] = {vc.crop[0] * sc, vc.crop[1] * sc, vc.crop[2] * sc, vc.crop[3] * sc, vc.crop[4] * sc};
    V3 t    = {vc.tx, vc.ty, vc.tz};
    V3 rt   = quat_rotate(-vc.qx, -vc.qy, -vc.qz, vc.qw, t);
    V3 tinv = {-rt.x, -rt.y, -rt.z};
    V2 ip   = {(float)gx, (float)gy};
    V3 inp;
    if (vc.model == 0)
    {
        V2 dist_p = k_unproject2(vc.k, k_unproject2(cr, ip));
        V2 np     = undistort_simple(dist_p, vc.d);
        inp       = {np.x, np.y, 1};
    }
    else
    {
        // OCam views (not in the reference, which asserts the pinhole model, EnvironmentMap.cu:129)
        const float* row = intrinsics + vc.intr_offset;
        inp              = ocam_unproject(row, row + 5, vc.npoly, k_unproject2(cr, ip));
    }
    V3 r      = quat_rotate(-vc.qx, -vc.qy, -vc.qz, vc.qw, inp);
    V3 wp     = {r.x + tinv.x, r.y + tinv.y, r.z + tinv.z};
    V3 d      = {wp.x - tinv.x, wp.y - tinv.y, wp.z - tinv.z};
    float n   = sqrtf(dot3(d, d));
    d         = {d.x / n, d.y / n, d.z / n};
    float phi = atan2_poly(-d.z, d.x);
    float x   = phi / (2.0f * ADOP_PI);
    x         = x - floorf(x);
    float th  = acos_poly(d.y);
    float y   = 1 - th / ADOP_PI;
    return {x * 2 - 1, y * 2 - 1};
}

struct Bilinear
{
    int x0, y0;
    float w00, w01, w10, w11;
    bool x1ok, y1ok;
};

// grid_sample(bilinear, padding border, align_corners=true) addressing
__device__ __forceinline__ Bilinear bilinear_setup(V2 uv, int ew, int eh)
{
    float fx = (uv.x + 1) * 0.5f * (float)(ew - 1);
    float fy = (uv.y + 1) * 0.5f * (float)(eh - 1);
    fx       = fminf(fmaxf(fx, 0.f), (float)(ew - 1));
    fy       = fminf(fmaxf(fy, 0.f), (float)(eh - 1));
    Bilinear s;
    s.x0     = (int)floorf(fx);
    s.y0     = (int)floorf(fy);
    float ax = fx - (float)s.x0, ay = fy - (float)s.y0;
    s.w00    = (1 - ax) * (1 - ay);
    s.w01    = ax * (1 - ay);
    s.w10    = (1 - ax) * ay;
    s.w11    = ax * ay;
    s.x1ok   = s.x0 + 1 < ew;
    s.y1ok   = s.y0 + 1 < eh;
    return s;
}


// Both kernels work on tiles of 16 x 16 pixels of one level of one view: workgroup -> (view, level, tile).
constexpr int kEnvTile = 16;
struct EnvTiles
{
    int prefix[ADOP_MAX_LAYERS + 1];  // tiles of the levels before l (one view)
    int tiles_x[ADOP_MAX_LAYERS];
};

struct EnvPixel
{
    int b, l, gx, gy;
    bool inside;
};

__device__ __forceinline__ EnvPixel env_pixel_of_thread(const Levels& lv, const EnvTiles& et)
{
    const int per_view = et.prefix[lv.num];
    EnvPixel e;
    e.b   = (int)blockIdx.x / per_view;
    int r = (int)blockIdx.x - e.b * per_view;
    e.l   = 0;
#pragma unroll
    for (int k = 1; k < ADOP_MAX_LAYERS; ++k)
        if (k < lv.num && r >= et.prefix[k]) e.l = k;
    r -= et.prefix[e.l];
    const int ty = r / et.tiles_x[e.l], tx = r - ty * et.tiles_x[e.l];
    e.gx     = tx * kEnvTile + ((int)threadIdx.x & (kEnvTile - 1));
    e.gy     = ty * kEnvTile + ((int)threadIdx.x >> 4);
    e.inside = e.gx < lv.l[e.l].w && e.gy < lv.l[e.l].h;
    return e;
}

// The view constants of the workgroup's view, computed by one thread (poses_se3 is f64, the intrinsics row up to 24
// floats: 256 threads each doing this for themselves cost more than the sampling).
__device__ __forceinline__ const ViewConst& env_view_const(ViewConst* s_vc, const ViewChunk& chunk, int b,
                                                           const double* __restrict__ poses,
                                                           const float* __restrict__ intrinsics, int cols)
{
    if (threadIdx.x == 0) *s_vc = make_view_const(chunk.v[b], poses, intrinsics, cols);
    __syncthreads();
    return *s_vc;
}

__global__ __launch_bounds__(kBlock) void env_sample_kernel(ViewChunk chunk, const double* __restrict__ poses,
                                                            const float* __restrict__ intrinsics, Levels lv,
                                                            EnvLevels ev, EnvTiles et, const float* __restrict__ tex,
                                                            int eh, int ew, int add_to_out, int cols)
{
    __shared__ ViewConst s_vc;
    const EnvPixel e    = env_pixel_of_thread(lv, et);
    const ViewConst& vc = env_view_const(&s_vc, chunk, e.b, poses, intrinsics, cols);
    if (!e.inside) return;
    const int l = e.l, b = e.b;
    const LevelArg& L = lv.l[l];
    const int p       = e.gy * L.w + e.gx;
    const size_t hw   = (size_t)L.w * L.h;
    float sc          = 1;
    for (int k = 0; k < l; ++k) sc /= 2;
    float bgw = 1.f;
    if (add_to_out && L.mask) bgw = 1.f - L.mask[(size_t)b * hw + p];
    if (add_to_out && bgw == 0.f)
    {
        // a rendered pixel: the composition does not sample it (and its uv is not written); out of place it is a copy
        if (add_to_out == 2)
            for (int c = 0; c < lv.C; ++c)
            {
                const size_t o = ((size_t)b * lv.C + c) * hw + p;
                ev.env[l][o]   = L.out[o];
            }
        else if (ev.env[l])
            for (int c = 0; c < lv.C; ++c) ev.env[l][((size_t)b * lv.C + c) * hw + p] = 0.f;
        return;
    }
    bool need = ev.uv[l] || ev.env[l] || add_to_out;
    if (!need) return;
    V2 uv = spherical_uv(vc, intrinsics, sc, e.gx, e.gy);
    if (ev.uv[l])
    {
        *(float2*)(ev.uv[l] + ((size_t)b * hw + p) * 2) = make_float2(uv.x, uv.y);
    }
    if (!ev.env[l] && !(add_to_out && bgw != 0.f)) return;
    Bilinear s = bilinear_setup(uv, ew, eh);
    for (int c = 0; c < lv.C; ++c)
    {
        const float* tc = tex + (size_t)c * eh * ew;
        float a         = 0;
        a += tc[(size_t)s.y0 * ew + s.x0] * s.w00;
        if (s.x1ok) a += tc[(size_t)s.y0 * ew + s.x0 + 1] * s.w01;
        if (s.y1ok) a += tc[(size_t)(s.y0 + 1) * ew + s.x0] * s.w10;
        if (s.x1ok && s.y1ok) a += tc[(size_t)(s.y0 + 1) * ew + s.x0 + 1] * s.w11;
        size_t o = ((size_t)b * lv.C + c) * hw + p;
        if (add_to_out == 2)
            ev.env[l][o] = L.out[o] + bgw * a;  // the composed image, out_l itself stays as the rasterizer left it
        else
        {
            if (ev.env[l]) ev.env[l][o] = a;
            if (add_to_out) L.out[o] = L.out[o] + bgw * a;
        }
    }
}

// Gradient of the texture.  The pixels of a tile land in a small window of the texture (a texel takes hundreds of
// contributions per call: 27 M empty pixels x 4 taps on 0.5 M texels in the 8-view fisheye configuration), so the
// workgroup first sums its contributions per texel in LDS and then issues one global float atomic per texel and channel
// it touched.  The LDS sums are 64-bit fixed point (32 fractional bits, integer LDS atomics: the native LDS float add
// is an order of magnitude slower, and the integer sum does not depend on the order of the additions); a contribution
// of magnitude >= 2^20, a non-finite one, and the tiles whose window does not fit (on the seam of the map, around its
// poles) go to global memory directly.
constexpr int kEnvAccEntries   = 4096;          // texels x channels of the LDS window (32 KB)
constexpr float kEnvFixedScale = 4294967296.f;  // 2^32
constexpr float kEnvFixedLimit = 1048576.f;     // 2^20: 1024 such terms stay inside 63 bits

__global__ __launch_bounds__(kBlock) void env_backward_kernel(ViewChunk chunk, const double* __restrict__ poses,
                                                              const float* __restrict__ intrinsics, Levels lv,
                                                              EnvLevels ev, EnvTiles et, float* __restrict__ genv, int eh,
                                                              int ew, int cols)
{
    __shared__ ViewConst s_vc;
    __shared__ unsigned long long s_acc[kEnvAccEntries];
    // window of the tile's active pixels in the texture: min / max of y0, of x0, and of x0 shifted by half the width
    // (modulo the width: a tile on the seam of the map is narrow there)
    __shared__ int s_box[6];
    if (threadIdx.x == 0)
    {
        s_box[0] = s_box[2] = s_box[4] = 0x7FFFFFFF;
        s_box[1] = s_box[3] = s_box[5] = -1;
    }
    const EnvPixel e    = env_pixel_of_thread(lv, et);
    const ViewConst& vc = env_view_const(&s_vc, chunk, e.b, poses, intrinsics, cols);  // (barrier: s_box is set)
    const int l = e.l, b = e.b, C = lv.C;
    const int half    = ew / 2;
    const LevelArg& L = lv.l[l];
    const int p       = e.gy * L.w + e.gx;
    const size_t hw   = (size_t)L.w * L.h;
    float sc          = 1;
    for (int k = 0; k < l; ++k) sc /= 2;
    float bgw = 0.f;
    if (e.inside) bgw = L.mask ? 1.f - L.mask[(size_t)b * hw + p] : 1.f;
    const bool active = e.inside && bgw != 0.f;
    Bilinear s;
    s.x0 = s.y0 = 0;
    s.w00 = s.w01 = s.w10 = s.w11 = 0.f;
    s.x1ok = s.y1ok = false;
    if (active)
    {
        V2 uv;
        if (ev.uv[l])  // kept from the forward call
        {
            const float2 t = *(const float2*)(ev.uv[l] + ((size_t)b * hw + p) * 2);
            uv             = {t.x, t.y};
        }
        else
            uv = spherical_uv(vc, intrinsics, sc, e.gx, e.gy);
        s = bilinear_setup(uv, ew, eh);
    }
    // (reduced inside the wavefront first: 64 lanes on one LDS address are served one after the other)
    {
        const int xs = s.x0 + half < ew ? s.x0 + half : s.x0 + half - ew;
        int lo[3] = {active ? s.y0 : 0x7FFFFFFF, active ? s.x0 : 0x7FFFFFFF, active ? xs : 0x7FFFFFFF};
        int hi[3] = {active ? s.y0 : -1, active ? s.x0 : -1, active ? xs : -1};
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
#pragma unroll
            for (int k = 0; k < 3; ++k)
            {
                lo[k] = min(lo[k], __shfl_xor(lo[k], off, 64));
                hi[k] = max(hi[k], __shfl_xor(hi[k], off, 64));
            }
        if ((threadIdx.x & 63) == 0 && hi[0] >= 0)
#pragma unroll
            for (int k = 0; k < 3; ++k)
            {
                atomicMin(&s_box[2 * k], lo[k]);
                atomicMax(&s_box[2 * k + 1], hi[k]);
            }
    }
    __syncthreads();
    if (s_box[1] < 0) return;  // no empty pixel in the tile (workgroup-uniform)
    // the narrower of the two windows; window column tx is texel column (bx + tx) (- half, modulo the width, if shifted)
    const bool shifted = s_box[5] - s_box[4] < s_box[3] - s_box[2];
    const int by = s_box[0], bx = shifted ? s_box[4] : s_box[2];
    const int bw = (shifted ? s_box[5] : s_box[3]) - bx + 2, bh = s_box[1] - by + 2;  // the taps reach one texel further
    const bool in_lds = (long long)bw * bh * C <= kEnvAccEntries;  // workgroup-uniform
    if (in_lds)
    {
        for (int k = threadIdx.x; k < bw * bh * C; k += kBlock) s_acc[k] = 0ull;
        __syncthreads();
    }
    if (active)
    {
        const int xs = s.x0 + half < ew ? s.x0 + half : s.x0 + half - ew;
        const int lx = (shifted ? xs : s.x0) - bx, ly = s.y0 - by;
        for (int c = 0; c < C; ++c)
        {
            const float g   = bgw * ev.gout[l][((size_t)b * C + c) * hw + p];
            float* tc       = genv + (size_t)c * eh * ew;
            const float v[4] = {g * s.w00, g * s.w01, g * s.w10, g * s.w11};
            const bool on[4] = {true, s.x1ok, s.y1ok, s.x1ok && s.y1ok};
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                if (!on[k]) continue;
                const int dx = k & 1, dy = k >> 1;
                if (in_lds && fabsf(v[k]) < kEnvFixedLimit)
                {
                    const long long q = __float2ll_rn(v[k] * kEnvFixedScale);
                    atomicAdd(&s_acc[((ly + dy) * bw + (lx + dx)) * C + c], (unsigned long long)q);
                }
                else
                    unsafeAtomicAdd(tc + (size_t)(s.y0 + dy) * ew + s.x0 + dx, v[k]);
            }
        }
    }
    if (!in_lds) return;
    __syncthreads();
    // flush: the texels of a window row are neighbours in memory (the texture is [C][eh][ew]) and neighbouring lanes
    // take them, so that a row costs one or two memory transactions, not one per texel
    for (int k = threadIdx.x; k < bw * bh * C; k += kBlock)
    {
        const int c = k / (bw * bh), t = k - c * (bw * bh);
        const int ty = t / bw, tx = t - ty * bw;
        const long long q = (long long)s_acc[(ty * bw + tx) * C + c];
        if (q != 0)
        {
            // (a window column / row past the border holds nothing: its taps were switched off)
            int x = bx + tx;
            if (shifted) x = x - half < 0 ? x - half + ew : x - half;
            unsafeAtomicAdd(genv + (size_t)c * eh * ew + (size_t)(by + ty) * ew + x,
                            (float)((double)q * (1.0 / 4294967296.0)));
        }
    }
}

// ApplyTangent (PointRenderer.cu:1646-1657): pose = Sophus::se3_expd(tangent) * pose; tangent = 0.  f64.
__global__ void apply_tangent_kernel(double* __restrict__ tangent, double* __restrict__ poses, int n)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    double* t = tangent + 6 * (size_t)i;
    double* p = poses + 8 * (size_t)i;
    double ux = t[0], uy = t[1], uz = t[2], wx = t[3], wy = t[4], wz = t[5];
    double th2 = wx * wx + wy * wy + wz * wz;
    double th  = sqrt(th2);
    double im, re, a, bb;
    if (th < 1e-10)
    {
        double th4 = th2 * th2;
        im         = 0.5 - th2 / 48.0 + th4 / 3840.0;
        re         = 1.0 - th2 / 8.0 + th4 / 384.0;
        a          = 0.5;
        bb         = 1.0 / 6.0;
    }
    else
    {
        im = sin(0.5 * th) / th;
        re = cos(0.5 * th);
        a  = (1.0 - cos(th)) / th2;
        bb = (th - sin(th)) / (th2 * th);
    }
    double ex = im * wx, ey = im * wy, ez = im * wz, ew = re;
    double c1x = wy * uz - wz * uy, c1y = wz * ux - wx * uz, c1z = wx * uy - wy * ux;
    double c2x = wy * c1z - wz * c1y, c2y = wz * c1x - wx * c1z, c2z = wx * c1y - wy * c1x;
    double etx = ux + a * c1x + bb * c2x, ety = uy + a * c1y + bb * c2y, etz = uz + a * c1z + bb * c2z;
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
    double qn = sqrt(nx * nx + ny * ny + nz * nz + nw * nw);
    p[0]      = nx / qn;
    p[1]      = ny / qn;
    p[2]      = nz / qn;
    p[3]      = nw / qn;
    p[4]      = rx + etx;
    p[5]      = ry + ety;
    p[6]      = rz + etz;
    for (int k = 0; k < 6; ++k) t[k] = 0;
}


static EnvTiles env_tiles(const Levels& lv)
{
    EnvTiles et;
    int acc = 0;
    for (int l = 0; l < ADOP_MAX_LAYERS; ++l)
    {
        et.prefix[l]  = acc;
        et.tiles_x[l] = 1;
        if (l < lv.num)
        {
            et.tiles_x[l] = (lv.l[l].w + kEnvTile - 1) / kEnvTile;
            acc += et.tiles_x[l] * ((lv.l[l].h + kEnvTile - 1) / kEnvTile);
        }
    }
    et.prefix[ADOP_MAX_LAYERS] = acc;
    for (int l = lv.num; l < ADOP_MAX_LAYERS; ++l) et.prefix[l] = acc;
    return et;
}

void launch_env_sample(const ViewChunk& chunk, const double* poses, const float* intrinsics, const Levels& lv,
                       const EnvLevels& ev, const float* tex, int eh, int ew, int add_to_out, int cols, hipStream_t st)
{
    static_assert(kEnvTile * kEnvTile == kBlock, "one thread per pixel of a tile");
    const EnvTiles et = env_tiles(lv);
    const int grid    = et.prefix[lv.num] * lv.B;
    if (grid > 0)
        hipLaunchKernelGGL(env_sample_kernel, dim3(grid), dim3(kBlock), 0, st, chunk, poses, intrinsics, lv, ev, et, tex,
                           eh, ew, add_to_out, cols);
}

void launch_env_backward(const ViewChunk& chunk, const double* poses, const float* intrinsics, const Levels& lv,
                         const EnvLevels& ev, float* genv, int eh, int ew, int cols, hipStream_t st)
{
    const EnvTiles et = env_tiles(lv);
    const int grid    = et.prefix[lv.num] * lv.B;
    if (grid > 0)
        hipLaunchKernelGGL(env_backward_kernel, dim3(grid), dim3(kBlock), 0, st, chunk, poses, intrinsics, lv, ev, et,
                           genv, eh, ew, cols);
}

void launch_apply_tangent(double* tangent, double* poses, int n, hipStream_t st)
{
    hipLaunchKernelGGL(apply_tangent_kernel, dim3((n + 127) / 128), dim3(128), 0, st, tangent, poses, n);
}

}  // namespace adop
