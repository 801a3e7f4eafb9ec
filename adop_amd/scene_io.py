"""The scene directory format of ADOP (scenes/README.md:57-95, data/SceneData.cpp:36-263) read into the tensors the
render stage consumes, and written back.

    dataset.ini           [SceneDatasetParams] camera_files, file_point_cloud, camera_type_int, ...
    camera<k>.ini         [SceneCameraParams] w, h, K (fx fy cx cy s), distortion (k1..k6 p1 p2), op (c d e cx cy),
                          poly_world2cam, ocam_cutoff
    point_cloud.ply       positions, normals (ascii or binary_little_endian)
    poses.txt             one line per image: qx qy qz qw tx ty tz, camera -> world
    images.txt, camera_indices.txt, masks.txt, exposure.txt, white_balance.txt   one line per image

The renderer works with the view transform: ``poses_se3`` holds the inverse of every pose as
(qx qy qz qw tx ty tz 0) in f64 (data/NeuralStructure.cpp:13-27), ``intrinsics`` one row (K | distortion) per pinhole
camera or (affine | world2cam polynomial) per OCam camera (data/NeuralStructure.cpp:63-130).
"""
import os
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import _capi

CAMERA_PINHOLE_DISTORTION = _capi.CAMERA_PINHOLE_DISTORTION
CAMERA_OCAM = _capi.CAMERA_OCAM


# ---------------------------------------------------------------------------------------------------
# ini files (saiga's: [Section], key = value, '#' starts a comment)
# ---------------------------------------------------------------------------------------------------
def read_ini(path):
    sections, cur = {}, None
    with open(path) as f:
        for raw in f:
            line = raw.split("#", 1)[0].strip()
            if not line:
                continue
            if line.startswith("[") and line.endswith("]"):
                cur = sections.setdefault(line[1:-1].strip(), {})
            elif "=" in line and cur is not None:
                k, v = line.split("=", 1)
                cur[k.strip()] = v.strip()
    return sections


def _floats(text):
    return [float(x) for x in text.split()]


def _fmt(values):
    return " ".join(f"{float(v):.15e}" for v in values)  # setprecision(15) << scientific, SceneData.h:169


def _bool(text):
    return text.strip().lower() in ("1", "true", "yes", "on")


def RenderParamsFromIni(path):
    """The [RenderParams] section of one of the reference's experiment files (configs/train_*.ini; RenderParams,
    Settings.h:22-52) -> (adop render params, dropout probability).  Keys the section does not hold keep the
    reference's defaults."""
    from . import scenes
    sec = read_ini(path).get("RenderParams", {})
    assert not _bool(sec.get("render_outliers", "false")), "the outlier cloud is a dead path in the reference"
    p = scenes.default_params(check_normal=1, ghost_gradients=0, drop_out_points_by_radius=1, depth_accept=0.01,
                              drop_out_radius_threshold=0.6, distortion_gradient_factor=0.005,
                              K_gradient_factor=0.5)  # the defaults of Settings.h:22-47
    for key in ("check_normal", "ghost_gradients", "drop_out_points_by_radius"):
        if key in sec:
            setattr(p, key, int(_bool(sec[key])))
    for key in ("drop_out_radius_threshold", "depth_accept", "distortion_gradient_factor", "K_gradient_factor"):
        if key in sec:
            setattr(p, key, float(sec[key]))
    if "test_backward_mode" in sec:
        p.test_backward_mode = int(sec["test_backward_mode"])
    if "render_points" in sec:
        p.skip_points = 0 if _bool(sec["render_points"]) else 1
    return p, float(sec.get("dropout", 0.25))


@dataclass
class SceneCameraParams:
    """data/SceneData.h:153-290"""
    w: int = 512
    h: int = 512
    K: np.ndarray = field(default_factory=lambda: np.array([1, 1, 0, 0, 0], np.float32))  # fx fy cx cy s
    distortion: np.ndarray = field(default_factory=lambda: np.zeros(8, np.float32))  # k1..k6 p1 p2
    ocam_affine: np.ndarray = field(default_factory=lambda: np.array([1, 0, 0, 0, 0], np.float64))  # c d e cx cy
    poly_world2cam: np.ndarray = field(default_factory=lambda: np.zeros(0, np.float64))
    poly_cam2world: np.ndarray = field(default_factory=lambda: np.zeros(0, np.float64))
    ocam_cutoff: float = 1.0

    @classmethod
    def load(cls, path):
        s = read_ini(path).get("SceneCameraParams", {})
        c = cls()
        c.w, c.h = int(s.get("w", c.w)), int(s.get("h", c.h))
        if "K" in s:
            k = _floats(s["K"])
            assert len(k) == 5, "K needs fx fy cx cy s"
            c.K = np.array(k, np.float64).astype(np.float32)  # parsed as double, stored as float (SceneData.h:187-193)
        if "distortion" in s:
            d = _floats(s["distortion"])
            assert len(d) == 8, "distortion needs 8 coefficients"
            c.distortion = np.array(d, np.float64).astype(np.float32)
        if "op" in s:
            a = _floats(s["op"])
            assert len(a) == 5, "op needs c d e cx cy"
            c.ocam_affine = np.array(a, np.float64)
        if "poly_world2cam" in s:
            c.poly_world2cam = np.array(_floats(s["poly_world2cam"]), np.float64)
        if "poly_cam2world" in s:
            c.poly_cam2world = np.array(_floats(s["poly_cam2world"]), np.float64)
        c.ocam_cutoff = float(s.get("ocam_cutoff", c.ocam_cutoff))
        return c

    def save(self, path):
        with open(path, "w") as f:
            f.write("[SceneCameraParams]\n")
            f.write(f"w = {self.w}\nh = {self.h}\n")
            f.write("# fx fy cx cy s\nK = " + _fmt(self.K) + "\n")
            f.write("# 8 paramter distortion model. see distortion.h\ndistortion = " + _fmt(self.distortion) + "\n")
            f.write("# c d e cx cy\nop = " + _fmt(self.ocam_affine) + "\n")
            f.write("poly_world2cam = " + _fmt(self.poly_world2cam) + "\n")
            f.write("poly_cam2world = " + _fmt(self.poly_cam2world) + "\n")
            f.write(f"ocam_cutoff = {self.ocam_cutoff:.9g}\n")


@dataclass
class SceneDatasetParams:
    """data/SceneData.h:91-150"""
    file_model: str = ""
    image_dir: str = "color/"
    mask_dir: str = "not set"
    camera_files: List[str] = field(default_factory=lambda: ["camera.ini"])
    file_point_cloud: str = "point_cloud.ply"
    file_point_cloud_compressed: str = "point_cloud.bin"
    camera_model: int = CAMERA_PINHOLE_DISTORTION
    znear: float = 0.1
    zfar: float = 1000.0
    render_scale: float = 1.0
    scene_exposure_value: float = 0.0
    scene_up_vector: np.ndarray = field(default_factory=lambda: np.array([0.0, 1.0, 0.0]))

    @classmethod
    def load(cls, path):
        s = read_ini(path).get("SceneDatasetParams", {})
        d = cls()
        for key in ("file_model", "image_dir", "mask_dir", "file_point_cloud", "file_point_cloud_compressed"):
            setattr(d, key, s.get(key, getattr(d, key)))
        if "camera_files" in s:
            d.camera_files = s["camera_files"].split()
        d.camera_model = int(s.get("camera_type_int", d.camera_model))
        for key in ("znear", "zfar", "render_scale", "scene_exposure_value"):
            setattr(d, key, float(s.get(key, getattr(d, key))))
        if "up_vector" in s:
            d.scene_up_vector = np.array(_floats(s["up_vector"]))
        return d

    def save(self, path):
        with open(path, "w") as f:
            f.write("[SceneDatasetParams]\n")
            f.write(f"file_model = {self.file_model}\nimage_dir = {self.image_dir}\nmask_dir = {self.mask_dir}\n")
            f.write("camera_files = " + " ".join(self.camera_files) + "\n")
            f.write(f"file_point_cloud = {self.file_point_cloud}\n")
            f.write(f"file_point_cloud_compressed = {self.file_point_cloud_compressed}\n")
            f.write(f"camera_type_int = {int(self.camera_model)}\n")
            f.write(f"znear = {self.znear:.9g}\nzfar = {self.zfar:.9g}\nrender_scale = {self.render_scale:.9g}\n")
            f.write(f"scene_exposure_value = {self.scene_exposure_value:.9g}\n")
            f.write("up_vector = " + _fmt(self.scene_up_vector) + "\n")


# ---------------------------------------------------------------------------------------------------
# poses
# ---------------------------------------------------------------------------------------------------
def quaternion_rotate(q, v):
    """Rotate v by the unit quaternion q = (x, y, z, w); f64."""
    x, y, z, w = q
    u = np.array([x, y, z])
    return v + 2.0 * np.cross(u, np.cross(u, v) + w * v)


def invert_pose(pose):
    """(qx qy qz qw tx ty tz) of the inverse transform; the quaternion is normalised first (Sophus does the same)."""
    q = np.asarray(pose[:4], np.float64)
    q = q / np.linalg.norm(q)
    qi = np.array([-q[0], -q[1], -q[2], q[3]])
    return np.concatenate([qi, -quaternion_rotate(qi, np.asarray(pose[4:7], np.float64))])


def read_poses(path):
    """poses.txt -> [F,7] f64, camera -> world (SceneData.cpp:127-143)."""
    rows = [_floats(line) for line in open(path) if line.strip()]
    assert all(len(r) == 7 for r in rows), "a pose line is qx qy qz qw tx ty tz"
    return np.array(rows, np.float64).reshape(-1, 7)


def _read_lines(path):
    return [line.rstrip("\r\n") for line in open(path)] if os.path.exists(path) else []


# ---------------------------------------------------------------------------------------------------
# point_cloud.ply
# ---------------------------------------------------------------------------------------------------
_PLY_TYPES = {"char": "i1", "uchar": "u1", "short": "i2", "ushort": "u2", "int": "i4", "uint": "u4", "float": "f4",
              "double": "f8", "int8": "i1", "uint8": "u1", "int16": "i2", "uint16": "u2", "int32": "i4", "uint32": "u4",
              "float32": "f4", "float64": "f8"}


def read_ply(path):
    """Vertex list of a PLY file -> dict of arrays: 'position' [N,3] f32, 'normal' [N,3] f32 or None, 'color' [N,3]
    f32 in [0,1] or None.  ascii and binary_little_endian; elements after the vertices are ignored."""
    with open(path, "rb") as f:
        assert f.readline().strip() == b"ply", "not a PLY file"
        fmt, props, count, in_vertex = None, [], 0, False
        while True:
            line = f.readline()
            assert line, "PLY header without end_header"
            tok = line.decode("ascii", "replace").split()
            if not tok:
                continue
            if tok[0] == "format":
                fmt = tok[1]
            elif tok[0] == "element":
                in_vertex = tok[1] == "vertex"
                if in_vertex:
                    count = int(tok[2])
            elif tok[0] == "property" and in_vertex:
                assert tok[1] != "list", "list property in the vertex element"
                props.append((tok[2], _PLY_TYPES[tok[1]]))
            elif tok[0] == "end_header":
                break
        assert fmt in ("ascii", "binary_little_endian"), f"unsupported PLY format {fmt}"
        dt = np.dtype([(n, "<" + t) for n, t in props])
        if fmt == "ascii":
            rows = [f.readline().split() for _ in range(count)]
            v = np.zeros(count, dt)
            for j, (n, _) in enumerate(props):
                v[n] = [float(r[j]) for r in rows]
        else:
            v = np.frombuffer(f.read(dt.itemsize * count), dt, count)
    names = set(dt.names)

    def cols(keys, scale=None):
        if not set(keys) <= names:
            return None
        a = np.stack([v[k].astype(np.float32) for k in keys], 1)
        if scale is not None and v[keys[0]].dtype.kind == "u":
            a = a / np.float32(scale)
        return a

    return {"position": cols(("x", "y", "z")), "normal": cols(("nx", "ny", "nz")),
            "color": cols(("red", "green", "blue"), 255.0)}


def write_ply(path, position, normal=None, color=None):
    """binary_little_endian PLY with x y z [nx ny nz] [red green blue]."""
    n = len(position)
    fields = [("x", "<f4"), ("y", "<f4"), ("z", "<f4")]
    if normal is not None:
        fields += [("nx", "<f4"), ("ny", "<f4"), ("nz", "<f4")]
    if color is not None:
        fields += [("red", "u1"), ("green", "u1"), ("blue", "u1")]
    v = np.zeros(n, np.dtype(fields))
    for j, k in enumerate("xyz"):
        v[k] = position[:, j]
    if normal is not None:
        for j, k in enumerate(("nx", "ny", "nz")):
            v[k] = normal[:, j]
    if color is not None:
        for j, k in enumerate(("red", "green", "blue")):
            v[k] = np.clip(np.rint(color[:, j] * 255.0), 0, 255)
    names = {"<f4": "float", "u1": "uchar"}
    with open(path, "wb") as f:
        f.write(b"ply\nformat binary_little_endian 1.0\n")
        f.write(f"element vertex {n}\n".encode())
        for name, t in fields:
            f.write(f"property {names[t]} {name}\n".encode())
        f.write(b"end_header\n")
        f.write(v.tobytes())


# ---------------------------------------------------------------------------------------------------
# the scene
# ---------------------------------------------------------------------------------------------------
@dataclass
class FrameData:
    """data/SceneData.h FrameData: one image of the scene."""
    image_index: int = 0
    camera_index: int = 0
    pose: np.ndarray = field(default_factory=lambda: np.array([0, 0, 0, 1, 0, 0, 0], np.float64))  # camera -> world
    exposure_value: float = 0.0
    white_balance: np.ndarray = field(default_factory=lambda: np.ones(3, np.float32))
    target_file: str = ""
    mask_file: str = ""
    w: int = 0
    h: int = 0


@dataclass
class SceneData:
    scene_path: str = ""
    dataset_params: SceneDatasetParams = field(default_factory=SceneDatasetParams)
    scene_cameras: List[SceneCameraParams] = field(default_factory=list)
    frames: List[FrameData] = field(default_factory=list)
    point_position: Optional[np.ndarray] = None  # [N,3] f32
    point_normal: Optional[np.ndarray] = None
    point_color: Optional[np.ndarray] = None

    @classmethod
    def load(cls, scene_path, load_points=True):
        """SceneData::SceneData(path) (SceneData.cpp:36-263) without the preprocessing of a new cloud."""
        sd = cls(scene_path=os.path.abspath(scene_path))
        ini = os.path.join(sd.scene_path, "dataset.ini")
        assert os.path.exists(ini), "dataset.ini is required"
        sd.dataset_params = SceneDatasetParams.load(ini)
        for name in sd.dataset_params.camera_files:
            file_ini = os.path.join(sd.scene_path, name)
            assert os.path.exists(file_ini), f"camera file {name} is missing"
            sd.scene_cameras.append(SceneCameraParams.load(file_ini))
        assert sd.scene_cameras, "a scene needs a camera"
        p = lambda name: os.path.join(sd.scene_path, name)
        assert os.path.exists(p("poses.txt")), "the pose file is required"
        poses = read_poses(p("poses.txt"))
        images, masks = _read_lines(p("images.txt")), _read_lines(p("masks.txt"))
        exposures = [float(x.split()[0]) for x in _read_lines(p("exposure.txt")) if x.strip()]
        wbs = [_floats(x) for x in _read_lines(p("white_balance.txt")) if x.strip()]
        cams = [int(x) for x in _read_lines(p("camera_indices.txt")) if x.strip()]
        n = max(len(images), len(poses))
        for name, lst in (("poses", poses), ("images", images), ("masks", masks), ("exposure", exposures),
                          ("white_balance", wbs), ("camera_indices", cams)):
            assert len(lst) in (0, n), f"{name}: {len(lst)} entries for {n} frames"
        for i in range(n):
            fd = FrameData(image_index=i, camera_index=cams[i] if cams else 0)
            if len(poses):
                fd.pose = poses[i]
            if exposures:
                fd.exposure_value = exposures[i]
            if wbs:
                fd.white_balance = np.array(wbs[i], np.float32)
            if images:
                fd.target_file = images[i]
            if masks:
                fd.mask_file = masks[i]
            cam = sd.scene_cameras[fd.camera_index]
            fd.w, fd.h = cam.w, cam.h
            sd.frames.append(fd)
        ply = p(sd.dataset_params.file_point_cloud)
        if load_points and os.path.exists(ply):
            pc = read_ply(ply)
            sd.point_position, sd.point_normal, sd.point_color = pc["position"], pc["normal"], pc["color"]
        return sd

    def save(self, scene_path):
        """SceneData::Save: the text files and the PLY cloud."""
        os.makedirs(scene_path, exist_ok=True)
        p = lambda name: os.path.join(scene_path, name)
        self.dataset_params.save(p("dataset.ini"))
        assert len(self.dataset_params.camera_files) == len(self.scene_cameras)
        for name, cam in zip(self.dataset_params.camera_files, self.scene_cameras):
            cam.save(p(name))
        with open(p("poses.txt"), "w") as f:
            for fd in self.frames:
                f.write(" ".join(f"{x:.17g}" for x in fd.pose) + "\n")
        with open(p("camera_indices.txt"), "w") as f:
            f.writelines(f"{fd.camera_index}\n" for fd in self.frames)
        if any(fd.target_file for fd in self.frames):
            with open(p("images.txt"), "w") as f:
                f.writelines(fd.target_file + "\n" for fd in self.frames)
        if any(fd.mask_file for fd in self.frames):
            with open(p("masks.txt"), "w") as f:
                f.writelines(fd.mask_file + "\n" for fd in self.frames)
        with open(p("exposure.txt"), "w") as f:
            f.writelines(f"{fd.exposure_value:.9g}\n" for fd in self.frames)
        if self.point_position is not None:
            write_ply(p(self.dataset_params.file_point_cloud), self.point_position, self.point_normal, self.point_color)

    # -- tensors of the render stage ---------------------------------------------------------------------------
    def poses_se3(self):
        """[F,8] f64: the view transform (inverse pose) of every frame, last element padding
        (PoseModuleImpl, NeuralStructure.cpp:13-27)."""
        out = np.zeros((len(self.frames), 8), np.float64)
        for i, fd in enumerate(self.frames):
            out[i, :7] = invert_pose(fd.pose)
        return out

    def intrinsics(self):
        """[K,13] f32 (K | distortion) for pinhole cameras, [K,5+P] (affine | world2cam) for OCam
        (IntrinsicsModuleImpl, NeuralStructure.cpp:63-130)."""
        if self.dataset_params.camera_model == CAMERA_OCAM:
            rows = [np.concatenate([c.ocam_affine, c.poly_world2cam]) for c in self.scene_cameras]
            assert len({len(r) for r in rows}) == 1, "OCam cameras of a scene share the polynomial degree"
            return np.array(rows, np.float64).astype(np.float32)
        return np.array([np.concatenate([c.K, c.distortion]) for c in self.scene_cameras], np.float32)

    def view(self, frame, scale=1.0):
        """ReducedImageInfo of a frame rendered at ``scale`` of its resolution with the matching crop transform."""
        fd = self.frames[frame]
        v = _capi.View()
        v.w, v.h = int(fd.w * scale), int(fd.h * scale)
        v.image_index, v.camera_index = fd.image_index, fd.camera_index
        v.camera_model_type = int(self.dataset_params.camera_model)
        v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy, v.crop_s = scale, scale, 0.0, 0.0, 0.0
        return v

    def host_scene(self, frames, texture, background=None, num_layers=4, params=None, radius=None, scale=1.0):
        """The inputs of one render call for the given frames: positions (x, y, z, radius), packed normals, one
        texel per point, the scene's poses and intrinsics."""
        from . import scenes
        assert self.point_position is not None, "the scene has no point cloud"
        n = len(self.point_position)
        pos = np.zeros((n, 4), np.float32)
        pos[:, :3] = self.point_position
        if radius is not None:
            pos[:, 3] = radius
        texture = np.asarray(texture)
        assert texture.ndim == 2 and texture.shape[1] == n, "one texel per point: texture is [C,N]"
        if params is None:
            params = scenes.default_params(check_normal=1 if self.point_normal is not None else 0)
        return scenes.HostScene(
            position=pos, normal=scenes.pack_normals(self.point_normal) if self.point_normal is not None else None,
            index=np.arange(n, dtype=np.int32), texture=texture,
            background=np.zeros(texture.shape[0], np.float32) if background is None else background,
            poses_se3=self.poses_se3(), intrinsics=self.intrinsics(), views=[self.view(f, scale) for f in frames],
            params=params, num_layers=num_layers, name=os.path.basename(self.scene_path))


# ---------------------------------------------------------------------------------------------------
# training crops
# ---------------------------------------------------------------------------------------------------
def RandomImageCrop(n, tries_per_crop, image_size_input, image_size_crop, prefer_border, random_translation,
                    min_max_zoom=(1.0, 1.0), generator=None):
    """Crop transforms for ``n`` training crops of one image -> [n,5] f32 rows (fx fy cx cy s) with fx = fy = zoom,
    s = 0: crop pixel = zoom * image pixel + (cx, cy), the matrix the rasterizer applies after the camera intrinsics
    (Dataset.cpp:140-160).  The arguments are those of saiga's RandomImageCrop, whose source is not part of the
    reference; the sampling law is this module's own:

      * zoom uniform in ``min_max_zoom``;
      * the crop window lies inside the zoomed image where that is larger than the crop (otherwise it is centred);
        without ``random_translation`` it is centred; with ``prefer_border`` the offset is drawn from a range a
        quarter crop wider on either side and clamped, which puts more windows against the image border;
      * of ``tries_per_crop`` candidates the one whose centre is farthest from the crops already chosen is kept.
    """
    g = generator if generator is not None else np.random.default_rng()
    size_in = np.asarray(image_size_input, np.float64)
    size_crop = np.asarray(image_size_crop, np.float64)
    chosen, centres = [], []
    for _ in range(n):
        best, best_centre, best_dis = None, None, -1.0
        for _ in range(max(1, tries_per_crop)):
            zoom = float(g.uniform(min_max_zoom[0], min_max_zoom[1]))
            room = size_in * zoom - size_crop  # free play of the window inside the zoomed image
            if random_translation:
                margin = 0.25 * size_crop if prefer_border else 0.0
                t = g.uniform(np.minimum(0.0, room) - margin, np.maximum(0.0, room) + margin)
                t = np.where(room > 0, np.clip(t, 0.0, np.maximum(room, 0.0)), 0.5 * room)
            else:
                t = 0.5 * room
            centre = (t + 0.5 * size_crop) / zoom  # in pixels of the input image
            dis = min((float(np.linalg.norm(centre - c)) for c in centres), default=0.0)
            if dis > best_dis:
                best, best_centre, best_dis = (zoom, zoom, -t[0], -t[1], 0.0), centre, dis
        chosen.append(best)
        centres.append(best_centre)
    return np.array(chosen, np.float32).reshape(n, 5)


class SceneDataTrainSampler:
    """The geometry side of SceneDataTrainSampler (Dataset.cpp:37-227): for a frame, ``inner_batch_size`` views of
    ``crop_size`` with random crop transforms (``down_scale``) or the full image.  Target images, uv images and
    masks belong to the loss and are not produced here."""

    def __init__(self, scene, indices, down_scale, crop_size, inner_batch_size, seed=0):
        self.scene, self.indices, self.down_scale = scene, list(indices), bool(down_scale)
        self.inner_batch_size = int(inner_batch_size)
        self.image_size_input = [(c.w, c.h) for c in scene.scene_cameras]
        if down_scale:
            assert crop_size[0] > 0
        self.image_size_crop = [tuple(crop_size) if down_scale else (c.w, c.h) for c in scene.scene_cameras]
        # Dataset.h:54-60
        self.random_translation, self.prefere_border, self.inner_sample_size = True, True, 1
        self.min_max_zoom = (0.75, 1.5)
        self.generator = np.random.default_rng(seed)

    def __len__(self):
        return len(self.indices)

    def Get(self, index):
        """-> (views, zoom): ``inner_batch_size`` adop views of frame ``indices[index]`` and the zoom of each."""
        actual = self.indices[index]
        fd = self.scene.frames[actual]
        cam = fd.camera_index
        w, h = self.image_size_crop[cam]
        rows = np.tile(np.float32([1, 1, 0, 0, 0]), (self.inner_batch_size, 1))
        if self.down_scale:
            rows = RandomImageCrop(self.inner_batch_size, self.inner_sample_size, self.image_size_input[cam],
                                   self.image_size_crop[cam], self.prefere_border, self.random_translation,
                                   self.min_max_zoom, self.generator)
        views = []
        for r in rows:
            v = _capi.View()
            v.w, v.h = int(w), int(h)
            v.image_index, v.camera_index = actual, cam
            v.camera_model_type = int(self.scene.dataset_params.camera_model)
            v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy, v.crop_s = [float(x) for x in r]
            views.append(v)
        return views, rows[:, 0].copy()
