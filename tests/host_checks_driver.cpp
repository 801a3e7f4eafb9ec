// Host-side argument checks and workspace arithmetic of the C-ABI under AddressSanitizer / UBSan (CPU only, no GPU
// work: every call here either computes a size or is rejected before anything is launched).  Built and run by
// tests/test_sanitizers.py; prints one line per case, exits non-zero on a wrong status.  A sanitizer report aborts it.
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../include/adop_raster.h"

static int failures = 0;
#define EXPECT(cond, what)                                     \
    do                                                         \
    {                                                          \
        if (!(cond))                                           \
        {                                                      \
            printf("FAIL %s (%s)\n", what, #cond);             \
            ++failures;                                        \
        }                                                      \
        else                                                   \
            printf("ok   %s\n", what);                         \
    } while (0)

// pointers that are never dereferenced on the host: the calls below stop at the argument checks
static void* fake(size_t k)
{
    return (void*)(uintptr_t)(0x100000 * (k + 1));
}

static adop_scene make_scene(int n, int c, int cols)
{
    adop_scene s;
    memset(&s, 0, sizeof(s));
    s.position         = (const float*)fake(1);
    s.normal           = (const int32_t*)fake(2);
    s.index            = (const int32_t*)fake(3);
    s.num_points       = n;
    s.texture          = fake(4);
    s.num_channels     = c;
    s.num_texels       = n > 0 ? n : 1;
    s.background_color = (const float*)fake(5);
    s.poses_se3        = (const double*)fake(6);
    s.num_poses        = 4;
    s.intrinsics       = (const float*)fake(7);
    s.num_cameras      = 2;
    s.intrinsics_cols  = cols;
    return s;
}

static adop_forward_buffers make_buffers(int levels, int w, int h)
{
    adop_forward_buffers fb;
    memset(&fb, 0, sizeof(fb));
    fb.num_layers = levels;
    for (int l = 0; l < levels && l < ADOP_MAX_LAYERS; ++l)
    {
        fb.layers[l].w           = w;
        fb.layers[l].h           = h;
        fb.layers[l].depth_index = (uint64_t*)fake(10 + l);
        fb.layers[l].depth       = (float*)fake(20 + l);
        fb.layers[l].weight      = (float*)fake(30 + l);
        fb.layers[l].out         = (float*)fake(40 + l);
        w /= 2;
        h /= 2;
    }
    return fb;
}

static std::vector<adop_view> make_views(int B, int w, int h, int model)
{
    std::vector<adop_view> v((size_t)B);
    for (int b = 0; b < B; ++b)
    {
        memset(&v[b], 0, sizeof(adop_view));
        v[b].w                 = w;
        v[b].h                 = h;
        v[b].image_index       = b % 4;
        v[b].camera_index      = b % 2;
        v[b].camera_model_type = model;
        v[b].crop_fx = v[b].crop_fy = 1.f;
    }
    return v;
}

int main()
{
    adop_render_params rp;
    memset(&rp, 0, sizeof(rp));
    rp.depth_accept = 0.01f;

    // --- workspace sizes at the largest sizes the interface takes: no wrap-around, growing with every argument ---
    {
        adop_scene big = make_scene(1 << 30, 16, 13);
        size_t a       = adop_workspace_size(&big, 64, 5, 2200, 1500);
        // per point and view: 8 bytes of work queue, 16 of projected point, 4 of candidate list (the tile bins are left
        // out of a cloud this size: their entries could not address it)
        EXPECT(a > (size_t)28 * 64 * ((size_t)1 << 30), "workspace of 2^30 points x 64 views of 2200x1500x5 does not wrap");
        EXPECT(a == adop_workspace_size_for(&big, 64, 5, 2200, 1500, ADOP_WORKSPACE_NO_TILE_PATH), "no bins at 2^30 points");
        adop_scene binned = make_scene(1 << 27, 16, 13);
        size_t b          = adop_workspace_size(&binned, 8, 5, 2200, 1500);
        // with the bins: + a tile word and two entries of 16 bytes
        EXPECT(b > (size_t)(28 + 36) * 8 * ((size_t)1 << 27), "workspace of 2^27 points x 8 views holds the tile bins");
        EXPECT(adop_workspace_size_for(&binned, 8, 5, 2200, 1500, ADOP_WORKSPACE_NO_TILE_PATH) < b - (size_t)36 * 8 * ((size_t)1 << 27) + (64 << 20),
               "without the bins: 36 bytes per point and view less");
        EXPECT(adop_workspace_size_for(&binned, 8, 5, 2200, 1500, ADOP_WORKSPACE_POINT_CACHE_KEPT | ADOP_WORKSPACE_NO_TILE_PATH) <
                   (size_t)9 * 8 * ((size_t)1 << 27) + ((size_t)8 << 30),
               "with both flags: the work queue, the pixel arrays and little else");
        EXPECT(adop_workspace_size_for(&binned, 8, 5, 2200, 1500, 8u) == 0, "unknown workspace flag: 0");
        adop_scene mid = make_scene(1 << 30, 16, 13);
        EXPECT(adop_workspace_size(&mid, 63, 5, 2200, 1500) < a, "fewer views, smaller workspace");
        EXPECT(adop_workspace_size(&mid, 64, 4, 2200, 1500) < a, "fewer levels, smaller workspace");
        EXPECT(adop_workspace_size(&mid, 64, 5, 2199, 1500) < a, "smaller image, smaller workspace");
        adop_scene small = make_scene((1 << 30) - 1024, 16, 13);
        EXPECT(adop_workspace_size(&small, 64, 5, 2200, 1500) < a, "fewer points, smaller workspace");
        adop_scene maxi = make_scene(INT_MAX, 16, 24);
        size_t m        = adop_workspace_size(&maxi, 1024, 5, 32767, 32767);
        EXPECT(m > a, "INT_MAX points x 1024 views of 32767^2: still a size, larger than the last");
        EXPECT(adop_workspace_size(&big, 0, 5, 100, 100) == 0, "no views: 0");
        EXPECT(adop_workspace_size(&big, 1, 6, 100, 100) == 0, "six levels: 0");
        EXPECT(adop_workspace_size(&big, 1, 4, 0, 100) == 0, "empty image: 0");
        EXPECT(adop_workspace_size(nullptr, 1, 4, 100, 100) == 0, "no scene: 0");
        adop_scene neg = make_scene(-5, 4, 13);
        EXPECT(adop_workspace_size(&neg, 2, 4, 64, 64) > 0, "negative point count is sized like an empty cloud");
        EXPECT(adop_knn_workspace_size(INT_MAX) > (size_t)INT_MAX * 16, "knn workspace of INT_MAX points does not wrap");
        EXPECT(adop_knn_workspace_size(-1) == 0, "knn workspace of a negative count: 0");
        EXPECT(adop_frames_workspace_size(INT_MAX) > (size_t)INT_MAX * 100, "frame constants of INT_MAX frames do not wrap");
    }

    // --- argument checks of adop_forward / adop_backward with extreme and inconsistent values ---
    {
        adop_scene s             = make_scene(1 << 30, 16, 13);
        std::vector<adop_view> v = make_views(64, 2200, 1500, ADOP_CAMERA_PINHOLE_DISTORTION);
        adop_forward_buffers fb  = make_buffers(5, 2200, 1500);
        // all arguments valid, no workspace: the size check is the last thing before the first launch
        EXPECT(adop_forward(&s, v.data(), 64, &rp, &fb, nullptr, 0, nullptr, nullptr) == ADOP_WORKSPACE_TOO_SMALL,
               "2^30 points x 64 views: accepted up to the workspace check");
        EXPECT(adop_forward(&s, v.data(), 64, &rp, &fb, fake(50), 4096, nullptr, nullptr) == ADOP_WORKSPACE_TOO_SMALL,
               "a workspace of 4 KB is too small");
        s.num_points = (1 << 30) + 1;
        EXPECT(adop_forward(&s, v.data(), 64, &rp, &fb, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "more than 2^30 points");
        s.num_points = INT_MAX;
        EXPECT(adop_forward(&s, v.data(), 64, &rp, &fb, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "INT_MAX points");
        s.num_points = -1;
        EXPECT(adop_forward(&s, v.data(), 64, &rp, &fb, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "negative point count");
        s.num_points = 1000;
        // image sizes
        std::vector<adop_view> huge = make_views(2, INT_MAX, INT_MAX, ADOP_CAMERA_PINHOLE_DISTORTION);
        adop_forward_buffers fbh    = make_buffers(5, INT_MAX, INT_MAX);
        EXPECT(adop_forward(&s, huge.data(), 2, &rp, &fbh, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "INT_MAX x INT_MAX image");
        std::vector<adop_view> wide = make_views(8, 46340, 46340, ADOP_CAMERA_PINHOLE_DISTORTION);
        adop_forward_buffers fbw    = make_buffers(5, 46340, 46340);
        EXPECT(adop_forward(&s, wide.data(), 8, &rp, &fbw, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "46340^2 pixels x 8 views");
        std::vector<adop_view> many = make_views(100000, 512, 512, ADOP_CAMERA_PINHOLE_DISTORTION);
        adop_forward_buffers fbm    = make_buffers(4, 512, 512);
        EXPECT(adop_forward(&s, many.data(), 100000, &rp, &fbm, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "100000 views of 512^2: too many pixels");
        adop_forward_buffers fbn = make_buffers(4, -64, 64);
        std::vector<adop_view> nv = make_views(1, -64, 64, ADOP_CAMERA_PINHOLE_DISTORTION);
        EXPECT(adop_forward(&s, nv.data(), 1, &rp, &fbn, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "negative width");
        // levels
        adop_forward_buffers fb0 = make_buffers(0, 64, 64);
        std::vector<adop_view> v1 = make_views(1, 64, 64, ADOP_CAMERA_PINHOLE_DISTORTION);
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fb0, nullptr, 0, nullptr, nullptr) == ADOP_UNSUPPORTED_LAYERS, "zero levels");
        fb0.num_layers = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fb0, nullptr, 0, nullptr, nullptr) == ADOP_UNSUPPORTED_LAYERS, "INT_MAX levels");
        fb0.num_layers = INT_MIN;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fb0, nullptr, 0, nullptr, nullptr) == ADOP_UNSUPPORTED_LAYERS, "INT_MIN levels");
        adop_forward_buffers fb7 = make_buffers(5, 8, 8);  // 8,4,2,1,0: the last level is empty
        std::vector<adop_view> v8 = make_views(1, 8, 8, ADOP_CAMERA_PINHOLE_DISTORTION);
        EXPECT(adop_forward(&s, v8.data(), 1, &rp, &fb7, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "a level of size 0");
        // indices and counts
        adop_forward_buffers fbs = make_buffers(3, 64, 64);
        v1[0].image_index = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "image_index INT_MAX");
        v1[0].image_index  = 0;
        v1[0].camera_index = INT_MIN;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "camera_index INT_MIN");
        v1[0].camera_index      = 0;
        v1[0].camera_model_type = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "camera model INT_MAX");
        v1[0].camera_model_type = ADOP_CAMERA_PINHOLE_DISTORTION;
        EXPECT(adop_forward(&s, v1.data(), INT_MIN, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "INT_MIN views");
        s.num_channels = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "INT_MAX channels");
        s.num_channels    = 8;
        s.intrinsics_cols = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "INT_MAX intrinsics columns");
        s.intrinsics_cols = 13;
        rp.forward_path   = INT_MAX;
        EXPECT(adop_forward(&s, v1.data(), 1, &rp, &fbs, fake(60), (size_t)1 << 40, nullptr, nullptr) == ADOP_INVALID_ARG, "forward_path INT_MAX");
        rp.forward_path = 0;
        // backward: missing buffers
        adop_backward_buffers gb;
        memset(&gb, 0, sizeof(gb));
        EXPECT(adop_backward(&s, v1.data(), 1, &rp, &fbs, &gb, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "backward without gradient buffers");
        gb.grad_texture    = (float*)fake(70);
        gb.grad_background = (float*)fake(71);
        for (int l = 0; l < 3; ++l) gb.grad_out[l] = (const float*)fake(80 + l);
        gb.grad_points = (float*)fake(72);
        EXPECT(adop_backward(&s, v1.data(), 1, &rp, &fbs, &gb, nullptr, 0, nullptr, nullptr) == ADOP_INVALID_ARG, "grad_points without its count");
        gb.grad_points_count = (float*)fake(73);
        EXPECT(adop_backward(&s, v1.data(), 1, &rp, &fbs, &gb, nullptr, 0, nullptr, nullptr) == ADOP_WORKSPACE_TOO_SMALL, "backward accepted up to the workspace check");
        EXPECT(strlen(adop_last_error_string()) > 0, "the last error has a message");
    }

    // --- the other entry points: rejected before any launch ---
    {
        adop_scene s             = make_scene(1000, 4, 13);
        std::vector<adop_view> v = make_views(40, 64, 64, ADOP_CAMERA_PINHOLE_DISTORTION);
        adop_forward_buffers fb  = make_buffers(3, 64, 64);
        EXPECT(adop_env_sample(&s, v.data(), 40, (const float*)fake(90), 16, 32, &fb, nullptr, nullptr, 1, nullptr) == ADOP_INVALID_ARG, "environment map: more than 32 views");
        EXPECT(adop_env_sample(&s, v.data(), 1, (const float*)fake(90), 0, 32, &fb, nullptr, nullptr, 1, nullptr) == ADOP_INVALID_ARG, "environment map of height 0");
        EXPECT(adop_env_sample(&s, v.data(), 1, (const float*)fake(90), INT_MIN, INT_MIN, &fb, nullptr, nullptr, 1, nullptr) == ADOP_INVALID_ARG, "environment map of size INT_MIN");
        float box_lo[3] = {0, 0, 0}, box_hi[3] = {1, 1, 1};
        EXPECT(adop_knn_distance((const float*)fake(1), 1000, 0, box_lo, box_hi, (float*)fake(91), fake(92), (size_t)1 << 40, nullptr) == ADOP_INVALID_ARG, "neighbour rank 0");
        EXPECT(adop_knn_distance((const float*)fake(1), 1000, INT_MAX, box_lo, box_hi, (float*)fake(91), fake(92), (size_t)1 << 40, nullptr) == ADOP_INVALID_ARG, "neighbour rank INT_MAX");
        EXPECT(adop_knn_distance((const float*)fake(1), 4, 4, box_lo, box_hi, (float*)fake(91), fake(92), (size_t)1 << 40, nullptr) == ADOP_INVALID_ARG, "as many points as the rank");
        EXPECT(adop_knn_distance((const float*)fake(1), INT_MAX, 4, box_lo, box_hi, (float*)fake(91), fake(92), 1024, nullptr) == ADOP_WORKSPACE_TOO_SMALL, "INT_MAX points, small workspace");
        float inf_hi[3] = {1, 1.0e38f * 10.f, 1};
        EXPECT(adop_morton_codes((const float*)fake(1), 1000, box_lo, inf_hi, (uint64_t*)fake(93), nullptr) == ADOP_INVALID_ARG, "bounding box with an infinite side");
        float nan_lo[3] = {0, 0, 0};
        nan_lo[1]       = nan_lo[1] / nan_lo[1];
        EXPECT(adop_morton_codes((const float*)fake(1), 1000, nan_lo, box_hi, (uint64_t*)fake(93), nullptr) == ADOP_INVALID_ARG, "bounding box with a NaN corner");
        EXPECT(adop_close_points((const float*)fake(1), 1000, (const float*)fake(94), box_lo, box_hi, (int32_t*)fake(95), (uint32_t*)fake(96), INT_MAX, 0, fake(92), (size_t)1 << 40, nullptr) == ADOP_INVALID_ARG, "INT_MAX rounds");
        EXPECT(adop_point_distance_to_camera(&s, v.data(), INT_MIN, (float*)fake(97), fake(92), (size_t)1 << 40, nullptr) == ADOP_INVALID_ARG, "INT_MIN frames");
        EXPECT(adop_point_distance_to_camera_static(&s, v.data(), 40, nullptr, nullptr) == ADOP_INVALID_ARG, "no output buffer");
        std::vector<adop_view> lots = make_views(1025, 64, 64, ADOP_CAMERA_PINHOLE_DISTORTION);
        EXPECT(adop_point_distance_to_camera_static(&s, lots.data(), 1025, (float*)fake(97), nullptr) == ADOP_INVALID_ARG, "1025 frames for the static scratch array");
        EXPECT(adop_apply_tangent(nullptr, nullptr, 5, nullptr) == ADOP_INVALID_ARG, "ApplyTangent without buffers");
        EXPECT(adop_apply_tangent((double*)fake(98), (double*)fake(99), 0, nullptr) == ADOP_OK, "ApplyTangent of no poses");
    }
    printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
