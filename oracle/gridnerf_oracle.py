"""CPU oracle for the GridNeRF render path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module: it exists so that tests,
the smoke check and the benchmark's CPU-baseline leg can compare the HIP path
with an independent restatement of the reference's PyTorch arithmetic.  Every
function names the reference lines it follows (paths relative to the reference
checkout).  The arithmetic itself lives in PyTorch (`F.grid_sample`,
`torch.cumprod`, `F.softplus`, `F.linear`, `torch.linspace`, boolean-mask
indexing), so the oracle issues the same ATen calls in the same order with the
same operand dtypes: that is what makes the geometry / occupancy decisions
reproducible bit for bit.

How each function is pinned (tests/test_oracle_*.py):
  sample_ray_aabb / sample_ray_within_hull   closed forms + brute force
  sample_alpha                               scalar trilinear loop, volume invariants
  sample_and_cull                            the reference's own sub-results in the golden vectors (inside-box mask
                                             and occupancy lookups of every sample); used by render_chunk
  normalize_coord                            AABB corners -> +-1
  density_feature / app_feature              scalar bilinear loop, affine planes,
                                             texel-centre queries, one-hot column order
  feature2density                            library softplus / relu
  raw2alpha                                  double-loop volume rendering, closed forms
  positional_encoding                        math.sin / math.cos, index order
  mlp_render                                 fp64 numpy matmul chain
  compute_alpha / get_dense_alpha /          golden vectors (tests/golden/alphamask_*.npz) written from
  update_alpha_mask                          the reference's getDenseAlpha / updateAlphaMask
  assign_blocks_to_samples + stacked lookup  golden vectors (tests/golden/stacked_*.npz) written from the
                                             reference's GridNeRFBranchParallel.forward; block index and
                                             block-relative coordinates against a plain loop
  render_chunk (composition order)           golden vectors written by
                                             tests/golden/make_golden.py from the
                                             reference's own forward
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F

MAT_MODE = [[0, 1], [0, 2], [1, 2]]  # app/models/gridnerf_sequential.py:106
VEC_MODE = [2, 1, 0]  # app/models/gridnerf_sequential.py:107


# --------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------
def sample_ray_aabb(p, rays_o, rays_d, N_samples=-1):
    """Equal-step samples from the slab entry point (sampling_opt=0, eval mode).

    Follows app/models/gridnerf_sequential.py:260-281 with is_train=False.
    Returns (pts [N,S,3], z [N,S], inside [N,S] bool).
    """
    S = N_samples if N_samples > 0 else p.nSamples
    near, far = p.near_far
    vec = torch.where(rays_d == 0, torch.full_like(rays_d, 1e-6), rays_d)
    rate_a = (p.aabb[1] - rays_o) / vec
    rate_b = (p.aabb[0] - rays_o) / vec
    t_min = torch.minimum(rate_a, rate_b).amax(-1).clamp(min=near, max=far)
    rng = torch.arange(S)[None].float()
    step = p.stepSize * rng.to(rays_o.device)
    z = t_min[..., None] + step
    pts = rays_o[..., None, :] + rays_d[..., None, :] * z[..., None]
    outside = ((p.aabb[0] > pts) | (pts > p.aabb[1])).any(dim=-1)
    return pts, z, ~outside


def sample_ray_within_hull(p, rays_o, rays_d, N_samples):
    """Samples between `near` and the ray's hit with the AABB floor (sampling_opt=1).

    Follows app/models/gridnerf_sequential.py:298-319 with is_train=False.
    """
    near, far = p.near_far
    o_z = rays_o[:, -1:] - p.aabb[0, 2].item()
    d_z = rays_d[:, -1:]
    far = -(o_z / d_z)
    far[rays_d[:, 2] >= 0] = p.near_far[-1]
    t_vals = torch.linspace(0.0, 1.0, steps=N_samples, device=rays_o.device)
    z = near * (1.0 - t_vals) + far * t_vals
    pts = rays_o[..., None, :] + rays_d[..., None, :] * z[..., :, None]
    outside = ((p.aabb[0] > pts) | (pts > p.aabb[1])).any(dim=-1)
    return pts, z, ~outside


# --------------------------------------------------------------------------------------
# occupancy volume
# --------------------------------------------------------------------------------------
def sample_alpha(alpha_volume, alpha_aabb, pts):
    """Trilinear lookup in the occupancy volume, app/models/alpha_mask.py:16-59.

    `alpha_volume` is [D,H,W]; pts are world-space [M,3] (x->W, y->H, z->D).
    """
    size = alpha_aabb[1] - alpha_aabb[0]
    inv = 1.0 / size * 2
    c = (pts - alpha_aabb[0]) * inv - 1
    vol = alpha_volume.view(1, 1, *alpha_volume.shape[-3:])
    return F.grid_sample(vol, c.view(1, -1, 1, 1, 3), align_corners=True).view(-1)


def normalize_coord(p, pts):
    """app/models/gridnerf_sequential.py:203-204."""
    return (pts - p.aabb[0]) * p.invaabbSize - 1


# --------------------------------------------------------------------------------------
# plane / line features
# --------------------------------------------------------------------------------------
def assign_blocks_to_samples(p, xyz):
    """Normalised [M,3] -> xyzb [M,4] for a block-stacked model: x, y relative to the sample's
    block of the plane_division grid, z unchanged, b the block index mapped to [-1,1]
    (app/models/gridnerf_parallel.py:279-338, the path taken with ckpt_type "full")."""
    d0, d1 = p.plane_division
    width, height = 2 / d0, 2 / d1
    out = torch.zeros(*xyz.shape[:-1], 4, device=xyz.device)
    out[..., :3] = xyz
    out[..., :2] += 1
    out[..., 0] /= width
    out[..., 1] /= height
    out[..., 3] = torch.floor(out[..., 0]) * d1 + torch.floor(out[..., 1])
    out[..., :3] = xyz
    b = out[..., 3]
    lo = torch.stack([-1 + (b // d1) * width, -1 + (b % d1) * height], dim=-1)
    hi = torch.stack([-1 + (b // d1 + 1) * width, -1 + (b % d1 + 1) * height], dim=-1)
    out[..., :2] = (out[..., :2] - lo) * 2 / (hi - lo) - 1
    out[..., 3] = -1 + 2 * b / (d0 * d1 - 1)
    return out


def _coords(p, xyz):
    """Grid-sample coordinate tensors, app/models/gridnerf_sequential.py:790-795; for xyzb
    input (block-stacked planes [1,C,B,h,w], lines [1,C,L,B]) the plane lookup is trilinear over
    (x, y, b) and the line lookup bilinear over (b, z), app/models/gridnerf_branch_parallel.py:182-193."""
    n = p.ndims
    if xyz.shape[-1] == 4:
        cp = torch.stack([xyz[..., [*MAT_MODE[i], MAT_MODE[i][1] + 2]] for i in range(n)]).view(n, 1, -1, 1, 3)
        cl = torch.stack([xyz[..., [VEC_MODE[i] + 1, VEC_MODE[i]]] for i in range(n)]).view(n, -1, 1, 2)
        return cp, cl
    cp = torch.stack([xyz[..., MAT_MODE[i]] for i in range(n)]).view(n, -1, 1, 2)
    cl = torch.stack([xyz[..., VEC_MODE[i]] for i in range(n)])
    cl = torch.stack((torch.zeros_like(cl), cl), dim=-1).view(n, -1, 1, 2)
    return cp, cl


def _f32(t):
    # fp16 plane storage is interpolated in fp32
    # (app/models/gridnerf_tensor_parallel.py:74-81,180-181).
    return t if t.dtype == torch.float32 else t.float()


def density_feature(p, xyz):
    """Sum over planes and channels of plane*line, or relu(basis_den(products)) when
    nonlinear_density is set; gridnerf_sequential.py:790-827 (return_feat=False).
    xyz is normalised [M,3]."""
    cp, cl = _coords(p, xyz)
    L = len(p.resMode)
    out = torch.zeros((xyz.shape[0],), device=xyz.device)
    pcs, lcs = [], []
    for k in range(len(p.density_plane)):
        d = k // L
        pc = F.grid_sample(_f32(p.density_plane[k]), cp[[d]], align_corners=True).view(-1, xyz.shape[0])
        lc = F.grid_sample(_f32(p.density_line[k]), cl[[d]], align_corners=True).view(-1, xyz.shape[0])
        pcs.append(pc)
        lcs.append(lc)
        out = out + torch.sum(pc * lc, dim=0)
    if getattr(p, "nonlinear_density", False):
        out = F.relu(F.linear((torch.cat(pcs) * torch.cat(lcs)).T, p.basis_den))[..., 0]
    return out


def app_products(p, xyz):
    """[M, P*L*C_a] plane*line products; column = plane index major, channel minor
    (gridnerf_sequential.py:846-864)."""
    cp, cl = _coords(p, xyz)
    L = len(p.resMode)
    pcs, lcs = [], []
    for k in range(len(p.app_plane)):
        d = k // L
        pcs.append(F.grid_sample(_f32(p.app_plane[k]), cp[[d]], align_corners=True).view(-1, xyz.shape[0]))
        lcs.append(F.grid_sample(_f32(p.app_line[k]), cl[[d]], align_corners=True).view(-1, xyz.shape[0]))
    return (torch.cat(pcs) * torch.cat(lcs)).T


def app_feature(p, xyz):
    """basis_mat(products), gridnerf_sequential.py:871 (Linear without bias, :678)."""
    return F.linear(app_products(p, xyz), p.basis_mat)


def feature2density(p, f):
    """gridnerf_sequential.py:396-399."""
    if p.fea2denseAct == "softplus":
        return F.softplus(f + p.density_shift)
    if p.fea2denseAct == "relu":
        return F.relu(f)
    raise ValueError(p.fea2denseAct)


# --------------------------------------------------------------------------------------
# occupancy volume from the density field
# --------------------------------------------------------------------------------------
def compute_alpha(p, xyz_locs, length):
    """Alpha of a segment of `length` at world points [M,3], gridnerf_sequential.py:401-427."""
    if p.alpha_volume is not None:
        on = sample_alpha(p.alpha_volume, p.alpha_aabb, xyz_locs) > 0
    else:
        on = torch.ones_like(xyz_locs[:, 0], dtype=torch.bool)
    sigma = torch.zeros(xyz_locs.shape[:-1])
    if on.any():
        sigma[on] = feature2density(p, density_feature(p, normalize_coord(p, xyz_locs[on])))
    return 1 - torch.exp(-sigma * length)


def get_dense_alpha(p, gridSize=None):
    """(alpha [gx,gy,gz], dense_xyz [gx,gy,gz,3]) on the lattice of the AABB, gridnerf_sequential.py:321-349."""
    gs = list(p.gridSize if gridSize is None else gridSize)
    samples = torch.stack(torch.meshgrid(*[torch.linspace(0, 1, g) for g in gs], indexing="ij"), -1)
    dense_xyz = p.aabb[0] * (1 - samples) + p.aabb[1] * samples
    alpha = torch.zeros_like(dense_xyz[..., 0])
    for i in range(gs[0]):
        alpha[i] = compute_alpha(p, dense_xyz[i].view(-1, 3), p.stepSize).view(gs[1], gs[2])
    return alpha, dense_xyz


def update_alpha_mask(p, gridSize=(200, 200, 200), increase_alpha_thresh=0):
    """(new_aabb [2,3], volume [gz,gy,gx]) of gridnerf_sequential.py:351-384; the new mask's box is p.aabb."""
    gs = list(gridSize)
    alpha, dense_xyz = get_dense_alpha(p, gs)
    dense_xyz = dense_xyz.transpose(0, 2).contiguous()
    alpha = alpha.clamp(0, 1).transpose(0, 2).contiguous()[None, None]
    alpha = F.max_pool3d(alpha, kernel_size=3, padding=1, stride=1).view(gs[::-1])
    thres = p.alphaMask_thres * (10**increase_alpha_thresh)
    alpha[alpha >= thres] = 1
    alpha[alpha < thres] = 0
    valid = dense_xyz[alpha > 0.5]
    return torch.stack((valid.amin(0), valid.amax(0))), alpha


# --------------------------------------------------------------------------------------
# compositing
# --------------------------------------------------------------------------------------
def raw2alpha(sigma, dist):
    """app/tools/utils.py:51-64. Returns (alpha, weights, T_last)."""
    alpha = 1.0 - torch.exp(-sigma * dist)
    T = torch.cumprod(
        torch.cat([torch.ones(alpha.shape[0], 1, device=alpha.device), 1.0 - alpha + 1e-10], -1), -1
    )
    return alpha, alpha * T[:, :-1], T[:, -1:]


# --------------------------------------------------------------------------------------
# colour network
# --------------------------------------------------------------------------------------
def positional_encoding(x, freqs):
    """app/tools/utils.py:42-48."""
    bands = 2 ** torch.arange(freqs, dtype=torch.float, device=x.device)
    q = (x[..., None] * bands).reshape(x.shape[:-1] + (freqs * x.shape[-1],))
    return torch.cat([torch.sin(q), torch.cos(q)], dim=-1)


def mlp_input(p, viewdirs, feats, latent=None):
    """Row layout of the network input, app/models/mlp_render_fea.py:55-65:
    [feat | latent (encode_app) | view | PE(feat) | PE(view)]."""
    parts = [feats, latent] if (getattr(p, "encode_app", False) and latent is not None) else [feats]
    if p.view_pe > -1:
        parts.append(viewdirs)
    if p.fea_pe > 0:
        parts.append(positional_encoding(feats, p.fea_pe))
    if p.view_pe > 0:
        parts.append(positional_encoding(viewdirs, p.view_pe))
    return torch.cat(parts, dim=-1)


def mlp_render(p, viewdirs, feats, latent=None):
    """app/models/mlp_render_fea.py:30-41,66-68: Linear-ReLU-Linear-ReLU-Linear-sigmoid."""
    h = mlp_input(p, viewdirs, feats, latent)
    h = F.relu(F.linear(h, p.mlp_w[0], p.mlp_b[0]))
    h = F.relu(F.linear(h, p.mlp_w[1], p.mlp_b[1]))
    h = F.linear(h, p.mlp_w[2], p.mlp_b[2])
    return torch.sigmoid(h)


# --------------------------------------------------------------------------------------
# whole chunk
# --------------------------------------------------------------------------------------
@torch.no_grad()
def sample_and_cull(p, rays_chunk, N_samples=-1):
    """The head of GridBaseSequential.forward: the sampler, then the occupancy lookup on the
    un-normalised points of the samples inside the box, ANDed into the mask with the reference's
    update idiom (gridnerf_sequential.py:451-465 for sampling_opt=0, :528-541 for sampling_opt=1).
    Returns (xyz [N,S,3] un-normalised, z [N,S], ray_valid [N,S] bool).  Needs the occupancy volume
    and the box only, no feature table."""
    rays_o = rays_chunk[:, :3]
    viewdirs = rays_chunk[:, 3:6]
    if p.sampling_opt:
        xyz, z, ray_valid = sample_ray_within_hull(p, rays_o, viewdirs, p.n_importance)
    else:
        xyz, z, ray_valid = sample_ray_aabb(p, rays_o, viewdirs, N_samples)
    if p.alpha_volume is not None:
        alphas = sample_alpha(p.alpha_volume, p.alpha_aabb, xyz[ray_valid])
        keep = alphas > p.alpha_mask_filter_thre
        ray_invalid = ~ray_valid
        ray_invalid[ray_valid] |= ~keep
        ray_valid = ~ray_invalid
    return xyz, z, ray_valid


@torch.no_grad()
def render_chunk(p, rays_chunk, white_bg=True, N_samples=-1, return_aux=False, app_code=None):
    """GridBaseSequential.forward with is_train=False,
    app/models/gridnerf_sequential.py:448-504 (sampling_opt=0) and :523-576
    (sampling_opt=1); the two branches differ only in the sampler."""
    viewdirs = rays_chunk[:, 3:6]
    xyz, z, ray_valid = sample_and_cull(p, rays_chunk, N_samples)
    dists = torch.cat((z[:, 1:] - z[:, :-1], torch.zeros_like(z[:, :1])), dim=-1)
    viewdirs = viewdirs.view(-1, 1, 3).expand(xyz.shape)

    sigma = torch.zeros(xyz.shape[:-1], device=xyz.device)
    rgb = torch.zeros((*xyz.shape[:2], 3), device=xyz.device)
    if ray_valid.any():
        xyz = normalize_coord(p, xyz)
        if getattr(p, "plane_division", None):
            # gridnerf_parallel.py:765-771, 918-924: valid samples get block-relative coordinates
            xyzb = torch.zeros(*xyz.shape[:-1], 4, device=xyz.device)
            xyzb[..., :3] = xyz
            xyzb.masked_scatter_(ray_valid.unsqueeze(-1).expand(-1, -1, 4), assign_blocks_to_samples(p, xyz[ray_valid]))
            xyz = xyzb
        sigma[ray_valid] = feature2density(p, density_feature(p, xyz[ray_valid]))

    _, weight, _ = raw2alpha(sigma, dists * p.distance_scale)
    app_mask = weight > p.rayMarch_weight_thres
    if app_mask.any():
        feats = app_feature(p, xyz[app_mask])
        latent = None
        if getattr(p, "encode_app", False) and app_code is not None:
            # compute_app_latent, gridnerf_sequential.py:429-437: one embedding row for every sample
            idx = torch.ones(feats.shape[0], dtype=torch.long, device=feats.device) * torch.as_tensor(app_code).long()
            latent = F.embedding(idx, p.embedding_app)
        rgb[app_mask] = mlp_render(p, viewdirs[app_mask], feats, latent)

    acc = torch.sum(weight, -1)
    rgb_map = torch.sum(weight[..., None] * rgb, -2)
    if white_bg:
        rgb_map = rgb_map + (1.0 - acc[..., None])
    rgb_map = rgb_map.clamp(0, 1)
    depth_map = torch.sum(weight * z, -1)
    out = {"rgb_map": rgb_map, "depth_map": depth_map}
    if return_aux:
        out.update(
            {
                "ray_valid": ray_valid,
                "z_vals": z,
                "sigma": sigma,
                "weight": weight,
                "app_mask": app_mask,
                "acc_map": acc,
                "rgb": rgb,
            }
        )
    return out


def renderer_fn(
    rays, model, chunk=4096, N_samples=-1, white_bg=True, is_train=False, device="cpu", idxs=None, app_code=None
) -> Tuple[Dict[str, torch.Tensor], dict]:
    """Chunk loop, app/tools/render_utils.py:15-63, driving `render_chunk` on `model`
    (a parameter object).  `is_train` and `idxs` are accepted and must be off."""
    assert not is_train and idxs is None
    acc: Dict[str, list] = {}
    n = rays.shape[0]
    for i in range(n // chunk + int(n % chunk > 0)):
        ret = render_chunk(model, rays[i * chunk : (i + 1) * chunk].to(device), white_bg=white_bg, N_samples=N_samples, app_code=app_code)
        for k, v in ret.items():
            acc.setdefault(k, []).append(v)
    return {k: torch.cat(v, 0) for k, v in acc.items()}, {}


def to_fp16_features(p):
    """Parameter object with planes and lines stored in fp16 (interpolated in fp32)."""
    import copy

    q = copy.copy(p)
    q.density_plane = [t.half() for t in p.density_plane]
    q.density_line = [t.half() for t in p.density_line]
    q.app_plane = [t.half() for t in p.app_plane]
    q.app_line = [t.half() for t in p.app_line]
    return q


# --------------------------------------------------------------------------------------
# either side of the path in the serving loop
# --------------------------------------------------------------------------------------
def generate_rays(single_pose, H, W, focal=None):
    """dist_render/dataset/utils.py:57-113 on the CPU: two arange tables, z = -1,
    directions @ pose[:3,:3].T, origin = pose[:3,3].  Pinned by its closed form
    ((i - W/2)/f, -(j - H/2)/f, -1) rotated by the pose."""
    pose = torch.as_tensor(single_pose, dtype=torch.float32)
    if focal is None:
        focal = float(pose[-1, -1])
    cx, cy = W / 2, H / 2
    d = torch.empty((3, H, W), dtype=torch.float32)
    d[0] = torch.arange(-cx / focal, (W - cx - 1e-5) / focal, 1 / focal, dtype=torch.float32).view(1, W)
    d[1] = torch.arange(cy / focal, (cy - H + 1e-5) / focal, -1 / focal, dtype=torch.float32).view(H, 1)
    d[2] = -1
    d = d.permute(1, 2, 0)
    rays_d = d @ pose[:3, :3].T
    rays_o = pose[:3, 3].expand(rays_d.shape)
    return torch.cat([rays_o.reshape(-1, 3), rays_d.reshape(-1, 3)], 1)


def postprocess_rgba8(rgb_map, H, W):
    """dist_render/ddp_infer/nerf_inferer.py:366-370."""
    r = rgb_map.reshape(H, W, 3) * 255
    r = torch.cat([r, torch.ones((H, W, 1)) * 255], dim=-1)
    return r.byte()
