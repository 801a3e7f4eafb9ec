"""Pins the camera arithmetic of the CPU checker without the reference (which cannot be built here):
closed forms, special cases of the published camera models, finite differences of every Jacobian, and library
routines (numpy / scipy) for what reduces to them.  A dropped term, a wrong sign or a transposed Jacobian fails
at least one of these.
"""
import ctypes as C

import numpy as np
import pytest
import scipy.linalg

from adop_amd import scenes


def f32(*v):
    return np.array(v, dtype=np.float32)


def ptr(a):
    return a.ctypes.data


IDENT_POSE = np.array([0, 0, 0, 1, 0, 0, 0, 0], dtype=np.float64)


def project_pinhole(L, p, n=(0, 0, -1), pose=IDENT_POSE, intr=None, check_normal=0, cutoff=1e4):
    p, n = f32(*p), f32(*n)
    pose = np.ascontiguousarray(pose, np.float64)
    out = np.zeros(3, np.float32)
    L.oracle_project_pinhole(ptr(p), ptr(n), ptr(pose), ptr(intr), check_normal, cutoff, ptr(out))
    return out


# --------------------------------------------------------------------------------------------------
# scalar helpers
# --------------------------------------------------------------------------------------------------

def test_atan_family_against_libm(oracle_mod):
    L = oracle_mod.lib()
    xs = np.concatenate([np.linspace(-50, 50, 4001), np.linspace(-1, 1, 2001), [1e-8, -1e-8, 1e6, -1e6, 0.0]])
    for x in xs.astype(np.float32):
        assert abs(L.oracle_atanf(float(x)) - np.arctan(np.float64(x))) < 4e-7
    for x in np.linspace(-1, 1, 4001).astype(np.float32):
        assert abs(L.oracle_acosf(float(x)) - np.arccos(np.float64(x))) < 6e-7
    g = scenes.rng(1)
    for y, x in g.standard_normal((3000, 2)).astype(np.float32):
        assert abs(L.oracle_atan2f(float(y), float(x)) - np.arctan2(np.float64(y), np.float64(x))) < 6e-7
    assert L.oracle_atan2f(1.0, 0.0) == pytest.approx(np.pi / 2)
    assert L.oracle_atan2f(-1.0, 0.0) == pytest.approx(-np.pi / 2)
    assert L.oracle_atan2f(0.0, -1.0) == pytest.approx(np.pi)


def test_round_to_nearest_even_and_saturation(oracle_mod):
    L = oracle_mod.lib()
    # __float2int_rn: ties to even
    for x, want in [(0.5, 0), (1.5, 2), (2.5, 2), (3.5, 4), (-0.5, 0), (-1.5, -2), (0.49999997, 0), (127.5, 128),
                    (128.5, 128), (-2.5, -2)]:
        assert L.oracle_f2i_rn(x) == want, x
    assert L.oracle_f2i_rn(float("nan")) == 0
    assert L.oracle_f2i_rn(float("inf")) == 2**31 - 1
    assert L.oracle_f2i_rn(-float("inf")) == -(2**31)
    assert L.oracle_f2i_rn(3e9) == 2**31 - 1


def test_pack_index_layout(oracle_mod):
    L = oracle_mod.lib()
    # depth bits in the high word, index in the low word; ordering by depth first, then index
    assert L.oracle_pack_index(1.0, 7) == (0x3F800000 << 32) | 7
    assert L.oracle_pack_index(100000.0, 0xFFFFFFFF) == (0x47C35000 << 32) | 0xFFFFFFFF
    assert L.oracle_pack_index(2.0, 0) > L.oracle_pack_index(1.9999999, 0xFFFFFFFF)
    assert L.oracle_pack_index(2.0, 5) < L.oracle_pack_index(2.0, 6)


def test_half_to_float_all_values(oracle_mod):
    L = oracle_mod.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    for i in range(0, 65536, 7):
        got = np.float32(L.oracle_half_to_float(int(h[i])))
        if np.isnan(want[i]):
            assert np.isnan(got)
        else:
            assert got == want[i], i
    for i in [0, 1, 0x3FF, 0x400, 0x7BFF, 0x7C00, 0x8000, 0x8001, 0xFBFF, 0xFC00]:
        assert np.float32(L.oracle_half_to_float(i)) == want[i]


def test_normal_packing(oracle_mod):
    L = oracle_mod.lib()
    g = scenes.rng(2)
    n = g.standard_normal((500, 3))
    n /= np.linalg.norm(n, axis=1, keepdims=True)
    out = np.zeros(3, np.float32)
    enc_np = scenes.pack_normals(n.astype(np.float32))
    for i, v in enumerate(n.astype(np.float32)):
        enc = L.oracle_pack_normal(float(v[0]), float(v[1]), float(v[2]))
        assert enc == enc_np[i]  # host generator and checker agree on the encoding
        L.oracle_unpack_normal(enc, ptr(out))
        assert np.abs(out - v).max() <= 1.0 / 1023 + 1e-6  # half a quantisation step of 2/1023
    # bit layout: x in bits 0..9, y 10..19, z 20..29
    assert L.oracle_pack_normal(1.0, -1.0, -1.0) == 1023
    assert L.oracle_pack_normal(-1.0, 1.0, -1.0) == 1023 << 10
    assert L.oracle_pack_normal(-1.0, -1.0, 1.0) == 1023 << 20


# --------------------------------------------------------------------------------------------------
# pinhole projection
# --------------------------------------------------------------------------------------------------

def test_pinhole_closed_form_no_distortion(oracle_mod):
    """zero distortion, identity pose: u = fx*x/z + s*y/z + cx, v = fy*y/z + cy, depth = z."""
    L = oracle_mod.lib()
    intr = scenes.pinhole_row(300.0, 310.0, 160.0, 120.0, 2.0)
    g = scenes.rng(3)
    for _ in range(200):
        p = g.uniform(-1, 1, 3)
        p[2] = g.uniform(0.5, 5)
        out = project_pinhole(L, p, intr=intr)
        u = 300.0 * p[0] / p[2] + 2.0 * p[1] / p[2] + 160.0
        v = 310.0 * p[1] / p[2] + 120.0
        assert out[0] == pytest.approx(u, rel=2e-6, abs=2e-4)
        assert out[1] == pytest.approx(v, rel=2e-6, abs=2e-4)
        assert out[2] == pytest.approx(p[2], rel=1e-6)


def test_config1_known_answer(oracle_mod):
    """camera at (0,0,-3) looking +z, fx=fy=256, c=128: the origin lands on pixel (128,128) with depth 3 and on
    (64,64), (32,32), (16,16) in the coarser levels."""
    hs = scenes.config1(n=1)
    hs.position[0] = [0, 0, 0, 0]
    hs.normal[0] = scenes.pack_normals(np.array([[0, 0, -1.0]], np.float32))[0]
    r = oracle_mod.forward(hs)
    for l, c in enumerate([128, 64, 32, 16]):
        assert r.weight[l][0, 0, c, c] == 1
        assert r.depth[l][0, 0, c, c] == np.float32(3.0)
        assert r.depth_index[l][0, 0, c, c] == (0x40400000 << 32) | 0
        assert r.weight[l].sum() == 1


def test_behind_camera_and_backface_are_culled(oracle_mod):
    L = oracle_mod.lib()
    intr = scenes.pinhole_row(100, 100, 50, 50)
    assert project_pinhole(L, (0, 0, -1), intr=intr)[2] == 0
    assert project_pinhole(L, (0, 0, 0), intr=intr)[2] == 0
    # normal pointing away from the camera (same direction as the view ray): culled only when check_normal
    assert project_pinhole(L, (0.1, 0, 2), n=(0, 0, 1), intr=intr, check_normal=1)[2] == 0
    assert project_pinhole(L, (0.1, 0, 2), n=(0, 0, 1), intr=intr, check_normal=0)[2] == 2
    assert project_pinhole(L, (0.1, 0, 2), n=(0, 0, -1), intr=intr, check_normal=1)[2] == 2


def test_pose_is_world_to_camera_quaternion_xyzw(oracle_mod):
    """V*p = R(q) p + t with q stored (x,y,z,w): checked against an independent rotation-matrix formula."""
    L = oracle_mod.lib()
    g = scenes.rng(4)
    intr = scenes.pinhole_row(1, 1, 0, 0)  # u = x/z, v = y/z
    for _ in range(50):
        q = g.standard_normal(4)
        q /= np.linalg.norm(q)
        t = g.uniform(-1, 1, 3) + [0, 0, 6]
        p = g.uniform(-1, 1, 3)
        pose = np.array([*q, *t, 0.0])
        vp = scenes.quaternion_to_rotation(q) @ p + t
        out = project_pinhole(L, p, pose=pose, intr=intr)
        assert out[0] == pytest.approx(vp[0] / vp[2], abs=3e-6)
        assert out[1] == pytest.approx(vp[1] / vp[2], abs=3e-6)
        assert out[2] == pytest.approx(vp[2], rel=2e-6)
    # an unnormalised stored quaternion is normalised by the float cast
    pose = np.array([0, 0, 0, 2.0, 0, 0, 1.0, 0])
    assert project_pinhole(L, (0.5, 0.25, 1.0), pose=pose, intr=intr)[:2] == pytest.approx([0.25, 0.125])


def distort(L, p, d, max_r=1e4, jac=False):
    p, d = f32(*p), f32(*d)
    out = np.zeros(2, np.float32)
    Jp, Jd = np.zeros(4, np.float32), np.zeros(16, np.float32)
    L.oracle_distort(ptr(p), ptr(d), max_r, ptr(out), ptr(Jp) if jac else None, ptr(Jd) if jac else None)
    return (out, Jp.reshape(2, 2), Jd.reshape(2, 8)) if jac else out


def test_distortion_special_cases_of_the_published_model(oracle_mod):
    """OpenCV rational model: x' = x*(1+k1 r2+k2 r4+k3 r6)/(1+k4 r2+k5 r4+k6 r6) + 2 p1 x y + p2 (r2 + 2 x^2),
    y' likewise with p1 (r2 + 2 y^2) + 2 p2 x y.  Each coefficient is isolated on an axis-aligned point."""
    L = oracle_mod.lib()
    x = 0.5
    r2 = x * x
    z8 = [0.0] * 8
    assert distort(L, (x, 0), z8) == pytest.approx([x, 0])
    for i, pw in enumerate([r2, r2**2, r2**3]):  # k1,k2,k3 numerator
        d = list(z8); d[i] = 0.3
        assert distort(L, (x, 0), d) == pytest.approx([x * (1 + 0.3 * pw), 0], rel=1e-6)
        assert distort(L, (0, x), d) == pytest.approx([0, x * (1 + 0.3 * pw)], rel=1e-6)
    for i, pw in enumerate([r2, r2**2, r2**3]):  # k4,k5,k6 denominator
        d = list(z8); d[3 + i] = 0.3
        assert distort(L, (x, 0), d) == pytest.approx([x / (1 + 0.3 * pw), 0], rel=1e-6)
    d = list(z8); d[6] = 0.1  # p1
    assert distort(L, (x, 0), d) == pytest.approx([x, 0.1 * r2], rel=1e-6)
    assert distort(L, (0, x), d) == pytest.approx([0, x + 0.1 * 3 * r2], rel=1e-6)
    d = list(z8); d[7] = 0.1  # p2
    assert distort(L, (x, 0), d) == pytest.approx([x + 0.1 * 3 * r2, 0], rel=1e-6)
    assert distort(L, (0, x), d) == pytest.approx([0.1 * r2, x], rel=1e-6)
    d = list(z8); d[6] = 0.1  # p1 cross term 2 p1 x y on the diagonal
    assert distort(L, (x, x), d)[0] == pytest.approx(x + 0.1 * 2 * x * x, rel=1e-6)
    # radius cutoff: sentinel 100000 beyond max_r (tested at PointRendererHelper.h:74)
    assert distort(L, (0.8, 0.7), z8, max_r=1.0)[0] == 100000
    assert distort(L, (0.6, 0.7), z8, max_r=1.0)[0] == pytest.approx(0.6)


def test_distortion_jacobians_by_finite_differences(oracle_mod):
    L = oracle_mod.lib()
    g = scenes.rng(5)
    for _ in range(20):
        p = g.uniform(-0.6, 0.6, 2)
        d = g.uniform(-0.05, 0.05, 8)
        _, Jp, Jd = distort(L, p, d, jac=True)
        # reference values: the same function evaluated in float32, central differences with a large step
        h = 1e-2
        for k in range(2):
            e = np.zeros(2); e[k] = h
            fd = (distort(L, p + e, d).astype(np.float64) - distort(L, p - e, d)) / (2 * h)
            assert Jp[:, k] == pytest.approx(fd, abs=2e-3)
        for k in range(8):
            e = np.zeros(8); e[k] = h
            fd = (distort(L, p, d + e).astype(np.float64) - distort(L, p, d - e)) / (2 * h)
            assert Jd[:, k] == pytest.approx(fd, abs=2e-3)


def test_undistort_inverts_distort(oracle_mod):
    L = oracle_mod.lib()
    g = scenes.rng(6)
    out = np.zeros(2, np.float32)
    for _ in range(50):
        p = g.uniform(-0.4, 0.4, 2).astype(np.float32)
        d = g.uniform(-0.02, 0.02, 8).astype(np.float32)
        q = distort(L, p, d)
        L.oracle_undistort(ptr(q), ptr(d), ptr(out))
        assert out == pytest.approx(p, abs=2e-5)


# --------------------------------------------------------------------------------------------------
# backward chain (pinhole): finite differences of the composed projection
# --------------------------------------------------------------------------------------------------

def _pix(L, p, pose, intr, crop):
    o = project_pinhole(L, p, pose=pose, intr=intr).astype(np.float64)
    return np.array([crop[0] * o[0] + crop[4] * o[1] + crop[2], crop[1] * o[1] + crop[3]])


def test_pinhole_backward_is_the_transposed_jacobian(oracle_mod):
    """g_point, g_pose (left perturbation exp(eps)*V, translation first), g_k (fx,fy,cx,cy,s) and g_dis (k1..k6,p1,p2)
    against central differences of pixel = crop(K(distort(divide(V p))))."""
    L = oracle_mod.lib()
    g = scenes.rng(7)
    for trial in range(8):
        q = g.standard_normal(4); q /= np.linalg.norm(q)
        pose = np.array([*q, *g.uniform(-0.3, 0.3, 2), 4.0, 0.0])
        p = g.uniform(-0.8, 0.8, 3)
        intr = scenes.pinhole_row(400, 420, 200, 150, 1.5, g.uniform(-0.03, 0.03, 8))
        crop = f32(1.3, 0.9, -20.0, 10.0, 0.2)
        grad = g.standard_normal(2).astype(np.float32)
        n = f32(0, 0, 0)
        out = np.zeros(22, np.float32)
        pf = p.astype(np.float32)
        L.oracle_project_pinhole_backward(ptr(pf), ptr(n), ptr(grad), ptr(pose), ptr(intr), ptr(crop), 0, 1e4, ptr(out))
        g_point, g_pose, g_k, g_dis = out[:3], out[3:9], out[9:14], out[14:22]
        gd = grad.astype(np.float64)

        def fd(fplus, fminus, h):
            return float(gd @ (fplus - fminus) / (2 * h))

        h = 2e-3
        for k in range(3):
            e = np.zeros(3); e[k] = h
            want = fd(_pix(L, pf + e, pose, intr, crop), _pix(L, pf - e, pose, intr, crop), h)
            assert g_point[k] == pytest.approx(want, rel=5e-3, abs=5e-2)
        for k in range(6):
            tp, tm = np.zeros((1, 6)), np.zeros((1, 6))
            tp[0, k], tm[0, k] = h, -h
            _, Pp = oracle_mod.apply_tangent(tp, pose[None])
            _, Pm = oracle_mod.apply_tangent(tm, pose[None])
            want = fd(_pix(L, pf, Pp[0], intr, crop), _pix(L, pf, Pm[0], intr, crop), h)
            assert g_pose[k] == pytest.approx(want, rel=5e-3, abs=8e-2), (trial, k)
        for k in range(5):
            hk = 0.5
            ip, im = intr.copy(), intr.copy()
            ip[k] += hk; im[k] -= hk
            want = fd(_pix(L, pf, pose, ip, crop), _pix(L, pf, pose, im, crop), hk)
            assert g_k[k] == pytest.approx(want, rel=5e-3, abs=2e-3)
        for k in range(8):
            hk = 1e-2
            ip, im = intr.copy(), intr.copy()
            ip[5 + k] += hk; im[5 + k] -= hk
            want = fd(_pix(L, pf, pose, ip, crop), _pix(L, pf, pose, im, crop), hk)
            assert g_dis[k] == pytest.approx(want, rel=1e-2, abs=5e-2)


# --------------------------------------------------------------------------------------------------
# OCam
# --------------------------------------------------------------------------------------------------

def project_ocam(L, p, intr, pose=IDENT_POSE, n=(0, 0, -1), check_normal=0, cutoff=1e4):
    p, n = f32(*p), f32(*n)
    pose = np.ascontiguousarray(pose, np.float64)
    out = np.zeros(3, np.float32)
    L.oracle_project_ocam(ptr(p), ptr(n), ptr(pose), ptr(intr), len(intr), check_normal, cutoff, ptr(out))
    return out


def test_ocam_constant_polynomial_maps_to_a_circle(oracle_mod):
    """world2cam polynomial {a0}: every point lands at distance a0 from the centre, in the direction of (x,y);
    returned depth is the Euclidean distance."""
    L = oracle_mod.lib()
    intr = f32(1, 0, 0, 320, 240, 150.0)
    g = scenes.rng(8)
    for _ in range(50):
        p = g.uniform(-1, 1, 3); p[2] = g.uniform(0.2, 3)
        o = project_ocam(L, p, intr)
        r = np.hypot(p[0], p[1])
        assert o[0] == pytest.approx(320 + 150 * p[0] / r, abs=1e-3)
        assert o[1] == pytest.approx(240 + 150 * p[1] / r, abs=1e-3)
        assert o[2] == pytest.approx(np.linalg.norm(p), rel=1e-6)


def test_ocam_equidistant_polynomial(oracle_mod):
    """rho = f*(theta + pi/2) with theta = atan(-z/|xy|) is the equidistant fisheye: pixel radius = f * angle
    between the ray and the optical axis (+z)."""
    L = oracle_mod.lib()
    f = 200.0
    intr = f32(1, 0, 0, 500, 400, f * np.pi / 2, f)
    g = scenes.rng(9)
    for _ in range(50):
        p = g.uniform(-1, 1, 3); p[2] = g.uniform(-0.2, 2)
        o = project_ocam(L, p, intr)
        angle = np.arccos(p[2] / np.linalg.norm(p))
        assert np.hypot(o[0] - 500, o[1] - 400) == pytest.approx(f * angle, abs=2e-3)
    # affine part: u = c*uu + d*vv + cx, v = e*uu + vv + cy
    intr2 = f32(1.1, 0.2, -0.3, 500, 400, f * np.pi / 2, f)
    p = (0.3, -0.2, 1.0)
    o1, o2 = project_ocam(L, p, intr), project_ocam(L, p, intr2)
    uu, vv = o1[0] - 500, o1[1] - 400
    assert o2[0] == pytest.approx(1.1 * uu + 0.2 * vv + 500, abs=1e-3)
    assert o2[1] == pytest.approx(-0.3 * uu + vv + 400, abs=1e-3)
    # theta cutoff: theta = atan(-z/|xy|) > cutoff  <=>  more than (90 deg + cutoff) off-axis -> culled
    cut = np.deg2rad(5.0)
    assert project_ocam(L, (1, 0, -np.tan(np.deg2rad(4.0))), intr, cutoff=cut)[2] > 0
    assert project_ocam(L, (1, 0, -np.tan(np.deg2rad(6.0))), intr, cutoff=cut)[2] == 0
    # on the axis the image point is the centre
    assert project_ocam(L, (0, 0, 2), intr)[:2] == pytest.approx([500, 400])


def test_sincos_polynomials_against_libm(oracle_mod):
    """The fixed sine / cosine polynomials of the OCam pixel-to-ray routine over their whole domain [-pi/2, pi/2]."""
    for t in np.concatenate([np.linspace(-np.pi / 2, np.pi / 2, 6001), [0.0, np.pi / 4, -np.pi / 4, 1e-9]]):
        t = np.float32(t)
        s, c = oracle_mod.sincos(t)
        assert abs(s - np.sin(np.float64(t))) < 2e-7 and abs(c - np.cos(np.float64(t))) < 2e-7, t
    assert oracle_mod.sincos(0.0) == (0.0, 1.0)


def test_ocam_unproject_equidistant_closed_form(oracle_mod):
    """rho = f*(theta + pi/2): a pixel at radius r from the centre, direction phi, comes from the ray
    (sin(a) cos(phi), sin(a) sin(phi), cos(a)) with a = r / f off the optical axis."""
    f = 200.0
    intr = f32(1, 0, 0, 500, 400, f * np.pi / 2, f)
    g = scenes.rng(31)
    for _ in range(200):
        a = g.uniform(0.01, np.deg2rad(100))
        phi = g.uniform(-np.pi, np.pi)
        ip = (500 + f * a * np.cos(phi), 400 + f * a * np.sin(phi))
        d = oracle_mod.ocam_unproject(intr, ip)
        want = (np.sin(a) * np.cos(phi), np.sin(a) * np.sin(phi), np.cos(a))
        assert d == pytest.approx(want, abs=3e-6)
        assert np.linalg.norm(d.astype(np.float64)) == pytest.approx(1.0, abs=1e-6)
    # the centre pixel is the optical axis
    assert oracle_mod.ocam_unproject(intr, (500, 400)) == pytest.approx([0, 0, 1], abs=1e-7)


def test_ocam_unproject_inverts_the_projection(oracle_mod):
    """project(unproject(pixel)) = pixel for a 5th-order polynomial with an affine part, over the image circle; and
    unproject(project(p)) is the direction of p."""
    g = scenes.rng(32)
    for seed in range(6):
        intr = scenes.ocam_row(1200, 900, seed=seed)
        intr[:3] = [1.0 + 0.02 * seed, 0.01 * seed, -0.015 * seed]
        if seed >= 4:
            intr[7:] *= 6.0  # six times the higher-order terms: the fixed number of Newton steps still converges
        r0 = oracle_mod.ocam_core(intr, (1e-6, 0, 1.0))  # radius the polynomial gives next to the axis
        r_min = abs(np.hypot(r0[0] - intr[3], r0[1] - intr[4])) + 2.0
        for _ in range(300):
            # a pixel on a ring the polynomial reaches (its value on the axis is not exactly 0)
            r = g.uniform(r_min, 600.0)
            phi = g.uniform(-np.pi, np.pi)
            ip = np.array([intr[3] + r * np.cos(phi), intr[4] + r * np.sin(phi)])
            d = oracle_mod.ocam_unproject(intr, ip)
            back = oracle_mod.ocam_core(intr, 3.7 * d)
            assert back[:2] == pytest.approx(ip, abs=2e-3), (seed, ip, d)
            assert back[2] == pytest.approx(3.7, rel=1e-6)
        for _ in range(100):
            p = g.uniform(-1, 1, 3)
            p[2] = g.uniform(0.0, 2.0)
            uvz = oracle_mod.ocam_core(intr, p)
            if np.hypot(uvz[0] - intr[3], uvz[1] - intr[4]) < r_min:
                continue
            d = oracle_mod.ocam_unproject(intr, uvz[:2])
            assert d == pytest.approx(p / np.linalg.norm(p), abs=2e-5)


def test_ocam_unproject_outside_the_polynomial_range(oracle_mod):
    """Pixels the polynomial does not reach take the ray at the nearest end of theta's range and stay finite."""
    f = 100.0
    intr = f32(1, 0, 0, 50, 50, f * np.pi / 2 + 5.0, f)  # rho(-pi/2) = 5: nothing projects inside 5 pixels
    assert oracle_mod.ocam_unproject(intr, (52, 50)) == pytest.approx([0, 0, 1], abs=1e-6)
    # far outside: theta stops at +pi/2, the ray points backwards along the axis
    d = oracle_mod.ocam_unproject(intr, (5000, 50))
    assert np.isfinite(d).all() and d == pytest.approx([0, 0, -1], abs=1e-6)


def test_ocam_backward_by_finite_differences(oracle_mod):
    L = oracle_mod.lib()
    g = scenes.rng(10)
    intr = scenes.ocam_row(800, 600, seed=3)
    crop = f32(1.2, 0.8, 5.0, -3.0, 0.1)
    for trial in range(6):
        q = g.standard_normal(4); q /= np.linalg.norm(q)
        pose = np.array([*q, *g.uniform(-0.2, 0.2, 2), 3.0, 0.0])
        pf = g.uniform(-0.8, 0.8, 3).astype(np.float32)
        grad = g.standard_normal(2).astype(np.float32)
        n = f32(0, 0, 0)
        out = np.zeros(22, np.float32)
        L.oracle_project_ocam_backward(ptr(pf), ptr(n), ptr(grad), ptr(pose), ptr(intr), len(intr), ptr(crop), 0, 1e4,
                                       ptr(out))
        gd = grad.astype(np.float64)

        def pix(p, P, I):
            o = project_ocam(L, p, I, pose=P).astype(np.float64)
            return np.array([crop[0] * o[0] + crop[4] * o[1] + crop[2], crop[1] * o[1] + crop[3]])

        h = 2e-3
        for k in range(3):
            e = np.zeros(3, np.float32); e[k] = h
            want = float(gd @ (pix(pf + e, pose, intr) - pix(pf - e, pose, intr)) / (2 * h))
            assert out[k] == pytest.approx(want, rel=1e-2, abs=5e-2)
        for k in range(6):
            tp, tm = np.zeros((1, 6)), np.zeros((1, 6))
            tp[0, k], tm[0, k] = h, -h
            _, Pp = oracle_mod.apply_tangent(tp, pose[None])
            _, Pm = oracle_mod.apply_tangent(tm, pose[None])
            want = float(gd @ (pix(pf, Pp[0], intr) - pix(pf, Pm[0], intr)) / (2 * h))
            assert out[3 + k] == pytest.approx(want, rel=1e-2, abs=8e-2)
        for k in range(5):
            hk = 1e-2 if k < 3 else 0.5
            ip, im = intr.copy(), intr.copy()
            ip[k] += hk; im[k] -= hk
            want = float(gd @ (pix(pf, pose, ip) - pix(pf, pose, im)) / (2 * hk))
            assert out[9 + k] == pytest.approx(want, rel=1e-2, abs=5e-2)


# --------------------------------------------------------------------------------------------------
# se3 exponential / ApplyTangent
# --------------------------------------------------------------------------------------------------

def _se3_matrix(pose8):
    T = np.eye(4)
    T[:3, :3] = scenes.quaternion_to_rotation(pose8[:4])
    T[:3, 3] = pose8[4:7]
    return T


def test_apply_tangent_is_left_multiplication_by_the_matrix_exponential(oracle_mod):
    """pose <- exp(twist) * pose with twist = (upsilon, omega): compared with scipy.linalg.expm of the 4x4 twist."""
    g = scenes.rng(11)
    for scale in [1e-12, 1e-3, 0.3, 2.0]:
        q = g.standard_normal(4); q /= np.linalg.norm(q)
        pose = np.array([[*q, *g.uniform(-2, 2, 3), 0.0]])
        t = (g.standard_normal((1, 6)) * scale)
        u, w = t[0, :3], t[0, 3:]
        X = np.zeros((4, 4))
        X[:3, :3] = [[0, -w[2], w[1]], [w[2], 0, -w[0]], [-w[1], w[0], 0]]
        X[:3, 3] = u
        want = scipy.linalg.expm(X) @ _se3_matrix(pose[0])
        t2, p2 = oracle_mod.apply_tangent(t, pose)
        assert np.all(t2 == 0)
        assert _se3_matrix(p2[0]) == pytest.approx(want, abs=1e-12)
        assert np.linalg.norm(p2[0, :4]) == pytest.approx(1.0, abs=1e-14)
