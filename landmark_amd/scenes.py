"""Seeded synthetic GridNeRF scenes and pinhole cameras.

The generators draw tensors in the order the reference model constructs them
(app/models/gridnerf_sequential.py:676-718: density planes/lines per dimension and
level, then appearance planes/lines, then `basis_mat`, then the colour network's
three `Linear`s with PyTorch's default init, app/models/mlp_render_fea.py:30-41), so a
seed fully determines a scene.  Cameras follow the reference's blender convention
(app/tools/dataloader/ray_utils.py:492-531): pixel (i, j) at integer coordinates,
direction ((i-W/2)/f, -(j-H/2)/f, -1) rotated by the camera-to-world matrix, not
normalised.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch

from .params import MAT_MODE, VEC_MODE, GridNeRFParams


def _linear_init(out_f: int, in_f: int, bias: bool, gen_device="cpu"):
    lin = torch.nn.Linear(in_f, out_f, bias=bias)
    w = lin.weight.detach().clone()
    b = lin.bias.detach().clone() if bias else None
    return w, b


def mlp_in_dim(app_dim: int, view_pe: int, fea_pe: int) -> int:
    # app/models/mlp_render_fea.py:24
    return 2 * max(view_pe, 0) * 3 + 2 * fea_pe * app_dim + 3 * (view_pe > -1) + app_dim


def make_params(
    seed: int = 0,
    aabb: Sequence[Sequence[float]] = ((-1, -1, -1), (1, 1, 1)),
    gridSize: Sequence[int] = (256, 256, 256),
    ndims: int = 3,
    resMode: Sequence[int] = (1,),
    density_n_comp: int = 16,
    app_n_comp: int = 48,
    scale: float = 0.1,
    device: str = "cpu",
    dtype: torch.dtype = torch.float32,
    bias_enable: bool = True,
    feature_init: str = "normal",
    encode_app: bool = False,
    nonlinear_density: bool = False,
    n_images: int = 16,
    plane_division: Sequence[int] = None,
    **cfg,
) -> GridNeRFParams:
    """Random-init model.  On `device="cpu"` the global torch RNG is seeded and used
    exactly like the reference constructor does; on a GPU device the planes are drawn
    with a device generator (large scenes) and the small dense layers on the host."""
    torch.manual_seed(seed)
    gen = None
    if device != "cpu":
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)

    def draw(shape):
        if feature_init == "normal":
            t = scale * torch.randn(shape, device=device, generator=gen) if gen else scale * torch.randn(shape)
        elif feature_init == "uniform":
            t = (torch.rand(shape, device=device, generator=gen) if gen else torch.rand(shape)) * 2 - 1
        else:
            raise ValueError(feature_init)
        return t.to(dtype)

    def one_svd(n_comp):
        planes, lines = [], []
        for i in range(ndims):
            m0, m1 = MAT_MODE[i]
            v = VEC_MODE[i]
            for r in resMode:
                if plane_division is None:
                    planes.append(draw((1, n_comp, gridSize[m1] * r, gridSize[m0] * r)))
                    lines.append(draw((1, n_comp, gridSize[v] * r, 1)))
                else:  # block-stacked layout; gridSize is the size of one block
                    B = plane_division[0] * plane_division[1]
                    planes.append(draw((1, n_comp, B, gridSize[m1] * r, gridSize[m0] * r)))
                    lines.append(draw((1, n_comp, gridSize[v] * r, B)))
        return planes, lines

    dp, dl = one_svd(density_n_comp)
    ap, al = one_svd(app_n_comp)
    app_dim = cfg.pop("app_dim", 27)
    view_pe = cfg.pop("view_pe", 2)
    fea_pe = cfg.pop("fea_pe", 2)
    featureC = cfg.pop("featureC", 128)
    basis, _ = _linear_init(app_dim, app_n_comp * ndims * len(resMode), bias=False)
    basis_den = emb = None
    if nonlinear_density:
        basis_den, _ = _linear_init(1, density_n_comp * ndims * len(resMode), bias=False)
    if encode_app:
        emb = torch.randn(n_images, 48)  # torch.nn.Embedding default init
    in_c = mlp_in_dim(app_dim, view_pe, fea_pe) + (48 if encode_app else 0)
    w1, b1 = _linear_init(featureC, in_c, bias_enable)
    w2, b2 = _linear_init(featureC, featureC, bias_enable)
    w3, b3 = _linear_init(3, featureC, bias_enable)
    if bias_enable:
        b3 = torch.zeros_like(b3)  # mlp_render_fea.py:42-43
    mv = lambda t: None if t is None else t.to(device)
    return GridNeRFParams(
        aabb=torch.tensor(aabb, dtype=torch.float32, device=device),
        gridSize=list(gridSize),
        density_plane=dp,
        density_line=dl,
        app_plane=ap,
        app_line=al,
        basis_mat=mv(basis),
        mlp_w=[mv(w1), mv(w2), mv(w3)],
        mlp_b=[mv(b1), mv(b2), mv(b3)],
        ndims=ndims,
        resMode=list(resMode),
        app_dim=app_dim,
        view_pe=view_pe,
        fea_pe=fea_pe,
        featureC=featureC,
        encode_app=encode_app,
        embedding_app=mv(emb),
        nonlinear_density=nonlinear_density,
        basis_den=mv(basis_den),
        plane_division=None if plane_division is None else list(plane_division),
        **cfg,
    )


# --------------------------------------------------------------------------------------
# occupancy volumes
# --------------------------------------------------------------------------------------
def blob_occupancy(dims=(256, 256, 256), n_blobs=64, target=0.30, seed=0, device="cpu") -> torch.Tensor:
    """[D,H,W] float {0,1} volume: a sum of seeded Gaussian blobs thresholded so that
    about `target` of the voxels are occupied.  Stored as float like the reference
    (app/models/alpha_mask.py:23, gridnerf_sequential.py:234-241)."""
    g = torch.Generator().manual_seed(seed)
    c = torch.rand(n_blobs, 3, generator=g) * 1.6 - 0.8
    s = torch.rand(n_blobs, generator=g) * 0.20 + 0.08
    c, s = c.to(device), s.to(device)
    D, H, W = dims
    zs = torch.linspace(-1, 1, D, device=device)
    ys = torch.linspace(-1, 1, H, device=device)
    xs = torch.linspace(-1, 1, W, device=device)
    field = torch.zeros(D, H, W, device=device)
    for i in range(n_blobs):
        ex = torch.exp(-((xs - c[i, 0]) ** 2) / (2 * s[i] ** 2))
        ey = torch.exp(-((ys - c[i, 1]) ** 2) / (2 * s[i] ** 2))
        ez = torch.exp(-((zs - c[i, 2]) ** 2) / (2 * s[i] ** 2))
        field += ez[:, None, None] * ey[None, :, None] * ex[None, None, :]
    flat = field.flatten()
    sub = flat[:: max(1, flat.numel() // 1_000_000)]
    thr = torch.quantile(sub.float().cpu(), 1.0 - target).item()
    return (field > thr).float()


def heightfield_occupancy(dims=(64, 512, 512), target=0.15, seed=0, device="cpu") -> torch.Tensor:
    """[D,H,W] float {0,1}: building-like columns rising from the floor (z index 0);
    column heights are drawn per 16x16-voxel lot so that about `target` of the voxels
    are occupied."""
    g = torch.Generator().manual_seed(seed)
    D, H, W = dims
    lots_h, lots_w = (H + 15) // 16, (W + 15) // 16
    built = (torch.rand(lots_h, lots_w, generator=g) < 0.55).float()
    height = torch.rand(lots_h, lots_w, generator=g) * built * (2.0 * target / 0.55)
    height = height.clamp(max=1.0)
    height = height.repeat_interleave(16, 0)[:H].repeat_interleave(16, 1)[:, :W].to(device)
    z = (torch.arange(D, device=device).float() + 0.5) / D
    return (z[:, None, None] < height[None]).float()


# --------------------------------------------------------------------------------------
# cameras
# --------------------------------------------------------------------------------------
def look_at_pose(eye: Sequence[float], target: Sequence[float] = (0.0, 0.0, 0.0), up=(0.0, 0.0, 1.0)) -> torch.Tensor:
    """[3,4] camera-to-world matrix; the camera looks down its own -z axis with +y up
    (blender / OpenGL convention used by ray_utils.py:492-531)."""
    eye_t = torch.tensor(eye, dtype=torch.float64)
    fwd = torch.tensor(target, dtype=torch.float64) - eye_t
    fwd = fwd / fwd.norm()
    upv = torch.tensor(up, dtype=torch.float64)
    right = torch.linalg.cross(fwd, upv)
    right = right / right.norm()
    cam_up = torch.linalg.cross(right, fwd)
    c2w = torch.stack([right, cam_up, -fwd, eye_t], dim=1)
    return c2w.float()


def sphere_pose(radius: float, seed: int, elev_range=(25.0, 65.0)) -> torch.Tensor:
    """Seeded pose on a sphere of `radius`, above the scene, looking at the origin."""
    g = torch.Generator().manual_seed(seed)
    az = torch.rand(1, generator=g).item() * 2 * math.pi
    el = math.radians(elev_range[0] + torch.rand(1, generator=g).item() * (elev_range[1] - elev_range[0]))
    eye = (radius * math.cos(el) * math.cos(az), radius * math.cos(el) * math.sin(az), radius * math.sin(el))
    return look_at_pose(eye)


def orbit_pose(radius: float, height: float, frame: int, n_frames: int = 120, target=(0.0, 0.0, 0.0)) -> torch.Tensor:
    az = 2 * math.pi * frame / n_frames
    return look_at_pose((radius * math.cos(az), radius * math.sin(az), height), target)


def pinhole_rays(H: int, W: int, focal: float, c2w: torch.Tensor, device="cpu") -> torch.Tensor:
    """[H*W, 6] rays (origin, direction), row-major pixels.
    ray_utils.py:505-531 (`get_ray_directions_blender` + `get_rays_with_directions`)."""
    c2w = c2w.to(device)
    j, i = torch.meshgrid(
        torch.arange(H, dtype=torch.float32, device=device),
        torch.arange(W, dtype=torch.float32, device=device),
        indexing="ij",
    )
    dirs = torch.stack([(i - W / 2) / focal, -(j - H / 2) / focal, -torch.ones_like(i)], -1)
    rays_d = dirs @ c2w[:3, :3].T
    rays_o = c2w[:3, 3].expand(rays_d.shape)
    return torch.cat([rays_o.reshape(-1, 3), rays_d.reshape(-1, 3)], 1).contiguous()


# --------------------------------------------------------------------------------------
# the five benchmark configurations
# --------------------------------------------------------------------------------------
def c1_scene(dense: bool = False, sampling_opt: int = 1, device="cpu", grid=256, step_ratio: float = 2.0) -> GridNeRFParams:
    """Tiny full render: 3 planes 256^2 + 3 lines 256, 16/48 ch fp32, seed 0.
    `dense=True` uses density_shift 0 so that the colour network actually runs
    (with the stated init and shift -10 every weight is far below 1e-3).
    `sampling_opt=1`: 128 samples between near and the box floor (hull sampler); `sampling_opt=0`: equal steps of
    `step_ratio` grid cells from the slab entry (gridnerf_sequential.py:158-164, 260-281): with 128 steps the
    reference's default ratio 0.5 covers half a scene unit behind the entry point, 3.47 the whole diagonal of the
    box (and makes nSamples 128)."""
    return make_params(
        seed=0,
        gridSize=(grid, grid, grid),
        ndims=3,
        resMode=(1,),
        device=device,
        near_far=[0.5, 4.5],
        density_shift=0.0 if dense else -10.0,
        sampling_opt=sampling_opt,
        n_importance=128,
        step_ratio=step_ratio,
    )


def c1_rays(H=400, W=400, seed=0, device="cpu") -> torch.Tensor:
    focal = 0.5 * W / math.tan(math.radians(25.0))
    return pinhole_rays(H, W, focal, sphere_pose(2.5, seed), device=device)


def c4_scene(P: int = 3, base: int = 1024, device="cuda", density_shift: float = 0.0, alpha_dims=(256, 256, 256), **kw):
    """Full-frame multi-resolution model: levels base, 2*base, 4*base; 16 + 48 ch fp32,
    N(0, 0.1); occupancy from 64 seeded Gaussian blobs at about 30 %."""
    cfg = dict(sampling_opt=1, n_importance=128)
    cfg.update(kw)
    p = make_params(
        seed=4,
        gridSize=(base, base, base),
        ndims=P,
        resMode=(1, 2, 4),
        device=device,
        near_far=[0.5, 6.0],
        density_shift=density_shift,
        **cfg,
    )
    p.alpha_volume = blob_occupancy(alpha_dims, 64, 0.30, seed=4, device=device)
    p.alpha_aabb = p.aabb.clone()
    p.alpha_mask_filter_thre = 0.0
    return p


def c4_rays(H=1080, W=1920, frame=0, device="cuda") -> torch.Tensor:
    focal = 1483.6378 * (W / 1920.0)  # dist_render/ddp_infer/nerf_inferer.py:404
    return pinhole_rays(H, W, focal, orbit_pose(2.6, 1.9, frame), device=device)


def production_scene(base: int = 1024, step_ratio: float = 0.5, device="cuda", density_shift: float = 0.0):
    """The shape most of the reference's run configurations use (confs/*.txt): one plane orientation
    (ndims 1) at three levels, the equal-step AABB sampler (sampling_opt 0) with step_ratio grid cells per
    step (app/tools/config_parser.py:153-155: 0.5, i.e. several thousand samples per ray, nearly all of them
    culled by the occupancy volume), the appearance embedding, the density projection and biases in the
    colour network.  Tables, occupancy volume and camera are those of the full-frame multi-resolution scene."""
    p = c4_scene(P=1, base=base, device=device, density_shift=density_shift, sampling_opt=0, step_ratio=step_ratio,
                 encode_app=True, nonlinear_density=True)
    p.basis_den = p.basis_den.abs()  # keep relu(basis_den(.)) from zeroing half of the volume
    return p


def c5_scene(res: int = 8192, device="cuda", density_shift: float = 0.0):
    """One GPU's share of a plane-parallel city block: one level of `res`^2 planes,
    16 + 48 ch stored in fp16, AABB flattened to z in [-0.1, 0.1]."""
    p = make_params(
        seed=5,
        aabb=((-1, -1, -0.1), (1, 1, 0.1)),
        gridSize=(res, res, res),
        ndims=3,
        resMode=(1,),
        device=device,
        dtype=torch.float16,
        near_far=[0.2, 4.0],
        density_shift=density_shift,
        sampling_opt=1,
        n_importance=256,
    )
    p.alpha_volume = heightfield_occupancy((64, 512, 512), 0.15, seed=5, device=device)
    p.alpha_aabb = p.aabb.clone()
    return p


def c5_rays(H=2160, W=3840, device="cuda") -> torch.Tensor:
    focal = 1483.6378 * (W / 1920.0)
    el = math.radians(30.0)
    eye = (-1.2 * math.cos(el), 0.0, 1.2 * math.sin(el) - 0.1)
    return pinhole_rays(H, W, focal, look_at_pose(eye, (0.3, 0.0, -0.1)), device=device)
