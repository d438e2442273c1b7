"""GPU parity tests: the HIP path through the C-ABI against the CPU oracle.

Bars: sample masks, sample counts and valid-sample indices
bit-exact; depths of the samples bit-exact; rgb / depth within 1e-4 absolute with fp32
tables and an fp32 colour network, 1e-2 with fp16 tables or a 16-bit colour network.
The appearance mask (weight > 1e-3) derives from floats that are summed in a different
order than ATen does, so it may flip for weights within rounding of the threshold; such
samples are excluded by an explicit band and counted.
"""
import ctypes as C

import pytest
import torch

from landmark_amd import scenes
from oracle import gridnerf_oracle as O
from tests.helpers import alphamask_names, golden_names, load_golden, stacked_names

pytestmark = pytest.mark.gpu

RGB_TOL_F32 = 1e-4
RGB_TOL_16 = 1e-2


def _model(p, **kw):
    from landmark_amd.model import GridNeRFHIP

    return GridNeRFHIP(p, **kw)


def _scene(seed=3, grid=(9, 11, 13), opt=1, S=64, with_mask=True, thre=0.0, shift=0.0, boost=6.0, **kw):
    p = scenes.make_params(seed=seed, gridSize=grid, near_far=[0.5, 4.5], n_importance=S, sampling_opt=opt,
                           density_shift=shift, **kw)
    for t in p.density_plane:
        t.mul_(boost)
    if with_mask:
        p.alpha_volume = scenes.blob_occupancy((grid[2], grid[1], grid[0]), 6, 0.45, seed=seed)
        p.alpha_aabb = p.aabb + torch.tensor([[0.01, 0.0, -0.02], [0.0, 0.05, 0.0]])
        p.alpha_mask_filter_thre = thre
    return p


# ------------------------------------------------------------------------------------ part 1
@pytest.mark.parametrize("name", golden_names())
def test_sample_cull_golden(gpu_lib, name):
    p, d, cfg = load_golden(name)
    ref = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], return_aux=True, app_code=cfg.get("app_code"))
    out = _model(p).sample_cull(d["rays"], N_samples=cfg["N_samples"])
    assert torch.equal(out["z_vals"].cpu(), ref["z_vals"])
    assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])
    assert out["n_valid"] == int(ref["ray_valid"].sum())
    assert torch.equal(out["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])


@pytest.mark.parametrize("opt,S,thre", [(1, 64, 0.0), (1, 128, 0.5), (1, 100, 0.98), (0, 50, 0.0), (0, 77, 0.5)])
def test_sample_cull_random_scene_bit_exact(gpu_lib, opt, S, thre):
    p = _scene(opt=opt, S=S, thre=thre, step_ratio=0.4)
    rays = scenes.pinhole_rays(96, 96, 80.0, scenes.sphere_pose(2.5, 5))
    ref = O.render_chunk(p, rays, N_samples=S, return_aux=True)
    out = _model(p).sample_cull(rays, N_samples=S)
    assert 0 < int(ref["ray_valid"].sum()) < ref["ray_valid"].numel()
    assert torch.equal(out["z_vals"].cpu(), ref["z_vals"])
    assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])
    assert torch.equal(out["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])


@pytest.mark.parametrize("opt,S,thre,mask,occ", [
    (1, 64, 0.0, True, "auto"), (1, 128, 0.0, True, "auto"), (1, 256, 0.0, True, "auto"), (1, 128, 0.5, True, "auto"),
    (1, 128, 0.0, True, "f32"), (1, 128, 0.0, False, "auto"), (0, 64, 0.0, True, "auto"), (0, 128, 0.98, True, "u8"),
])
def test_sample_cull_ray_per_lane_kernel(gpu_lib, opt, S, thre, mask, occ):
    """S = 64, 128, 256 without depths takes the kernel with one lane per (ray, bitmap word): same masks, same
    list, same counts as the oracle and as the sample-per-lane kernel (taken when depths are asked for)."""
    p = _scene(opt=opt, S=S, thre=thre, with_mask=mask, step_ratio=0.4)
    rays = scenes.pinhole_rays(101, 77, 80.0, scenes.sphere_pose(2.5, 5))  # 7777 rays: ragged last workgroup
    ref = O.render_chunk(p, rays, N_samples=S, return_aux=True)
    m = _model(p, occupancy=occ)
    a = m.sample_cull(rays, N_samples=S, want_z=False)
    b = m.sample_cull(rays, N_samples=S, want_z=True)
    assert 0 < int(ref["ray_valid"].sum()) < ref["ray_valid"].numel()
    assert torch.equal(a["ray_valid"].cpu(), ref["ray_valid"])
    assert torch.equal(a["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])
    assert a["n_valid"] == b["n_valid"] and torch.equal(a["bitmap"], b["bitmap"]) and torch.equal(a["word_prefix"], b["word_prefix"])


@pytest.mark.parametrize("opt,S", [(0, 128), (1, 128), (1, 256)])
def test_cull_rays_along_box_faces(gpu_lib, opt, S):
    """Rays that run in a face of the box, one float above and below it, and through its edges and corners: whole
    words of samples sit exactly on the boundary of the box test, where the kernel's segment shortcut must stay
    on the safe side."""
    p = _scene(opt=opt, S=S, with_mask=False, step_ratio=0.05)
    lo, hi = p.aabb[0], p.aabb[1]
    up = lambda x: torch.nextafter(torch.tensor(x), torch.tensor(10.0)).item()
    dn = lambda x: torch.nextafter(torch.tensor(x), torch.tensor(-10.0)).item()
    rays = []
    for ax in range(3):
        for face in (lo[ax].item(), hi[ax].item()):
            for c in (face, up(face), dn(face)):
                for sgn in (1.0, -1.0):
                    o = [0.1, -0.2, 1.9]
                    d = [0.3 * sgn, 0.2, -1.0]
                    if ax == 2:
                        o, d = [-1.7, 0.05, c], [1.0, 0.1 * sgn, 0.0]
                    else:
                        o[ax], d[ax] = c, 0.0
                    rays.append(o + d)
    rays.append([lo[0].item(), lo[1].item(), 1.9, 0.0, 0.0, -1.0])  # down a vertical edge
    rays.append([-1.8, -1.8, 1.8, 1.0, 1.0, -1.0])  # through two corners
    rays = torch.tensor(rays, dtype=torch.float32)
    ref = O.render_chunk(p, rays, N_samples=S, return_aux=True)
    out = _model(p).sample_cull(rays, N_samples=S, want_z=False)
    assert ref["ray_valid"].any() and not ref["ray_valid"].all()
    assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])
    res, _ = _model(p)(rays, N_samples=S)  # the one-launch cull of the whole-chunk render takes the same decisions
    assert (res["depth_map"].cpu() - ref["depth_map"]).abs().max().item() <= RGB_TOL_F32


def test_occupancy_lookup_on_voxel_centres(gpu_lib):
    """Sample points that fall exactly on voxel centres and faces of the occupancy grid (zero upper weights):
    the positive-lookup shortcut must agree with the summed lookup."""
    p = _scene(with_mask=False, S=64, opt=0, step_ratio=1.0, grid=(9, 9, 9))
    p.aabb = torch.tensor([[-1.0, -1.0, -1.0], [1.0, 1.0, 1.0]])
    g = torch.Generator().manual_seed(5)
    p.alpha_volume = (torch.rand(9, 9, 9, generator=g) < 0.3).float()
    p.alpha_aabb = p.aabb.clone()
    # axis-parallel rays through lattice lines: x, y on voxel centres, z stepping by exactly one voxel (0.25)
    xs = torch.linspace(-1, 1, 9)
    o = torch.stack(torch.meshgrid(xs, xs, indexing="ij"), -1).reshape(-1, 2)
    rays = torch.cat([o, torch.full((81, 1), -1.5), torch.zeros(81, 2), torch.ones(81, 1)], 1)
    p.near_far = [0.5, 4.0]
    S = 64
    ref = O.render_chunk(p, rays, N_samples=S, return_aux=True)
    assert 0 < int(ref["ray_valid"].sum())
    for occ in ("auto", "f32"):
        out = _model(p, occupancy=occ).sample_cull(rays, N_samples=S, want_z=False)
        assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])


@pytest.mark.parametrize("occupancy", ["f32", "u8", "cells"])
def test_occupancy_storages_agree_bit_for_bit(gpu_lib, occupancy):
    p = _scene(S=128, thre=0.5)
    rays = scenes.pinhole_rays(96, 96, 80.0, scenes.sphere_pose(2.5, 5))
    ref = O.render_chunk(p, rays, return_aux=True)
    for thre in (0.0, 0.5, 0.98):
        p.alpha_mask_filter_thre = thre
        ref = O.render_chunk(p, rays, return_aux=True)
        m = _model(p, occupancy=occupancy)
        assert m._vol_dtype == {"f32": 0, "u8": 2, "cells": 3}[occupancy]
        out = m.sample_cull(rays)
        assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])


def test_non_binary_occupancy_falls_back_to_float(gpu_lib):
    p = _scene(S=64, thre=0.2)
    g = torch.Generator().manual_seed(3)
    p.alpha_volume = torch.rand(p.alpha_volume.shape, generator=g)  # arbitrary float volume
    rays = scenes.pinhole_rays(64, 64, 50.0, scenes.sphere_pose(2.5, 5))
    ref = O.render_chunk(p, rays, return_aux=True)
    m = _model(p)
    assert m._vol_dtype == 0
    assert torch.equal(m.sample_cull(rays)["ray_valid"].cpu(), ref["ray_valid"])


def test_sample_cull_edge_cases(gpu_lib):
    p = _scene(with_mask=False, S=64)
    m = _model(p)
    # empty chunk
    out = m.sample_cull(torch.zeros(0, 6))
    assert out["n_valid"] == 0
    # every ray misses the box -> empty list
    rays = torch.tensor([[5.0, 5.0, 5.0, 0.0, 0.0, 1.0]]).repeat(70, 1)
    out = m.sample_cull(rays)
    assert out["n_valid"] == 0 and not out["ray_valid"].any()
    # one ray, ragged tail (N*S not a multiple of a 4096-sample workgroup)
    rays = scenes.pinhole_rays(3, 1, 4.0, scenes.sphere_pose(2.5, 1))
    ref = O.render_chunk(p, rays, return_aux=True)
    out = m.sample_cull(rays)
    assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])
    # all-ones occupancy keeps every in-box sample, all-zeros none
    p.alpha_volume, p.alpha_aabb = torch.ones(4, 4, 4), p.aabb.clone()
    assert _model(p).sample_cull(rays)["n_valid"] == int(ref["ray_valid"].sum())
    p.alpha_volume = torch.zeros(4, 4, 4)
    assert _model(p).sample_cull(rays)["n_valid"] == 0


@pytest.mark.parametrize("opt,S,mask", [(1, 128, True), (0, 100, True), (1, 64, False), (0, 200, False)])
def test_non_finite_rays_do_not_disturb_their_neighbours(gpu_lib, opt, S, mask):
    """Rays with NaN or infinite components (a degenerate pose, a normalised zero vector) and rays along the axes
    (zero direction components: the sampler's 1e-6 substitute) sit between ordinary rays of a chunk.  Every
    address the kernels form stays inside the tables whatever the coordinates, and the ordinary rays come out as
    they do without the others, bit for bit."""
    p = _scene(opt=opt, S=S, with_mask=mask, step_ratio=0.3)
    m = _model(p, mlp_precision="f16x2")
    good = scenes.pinhole_rays(48, 40, 42.0, scenes.sphere_pose(2.5, 9))
    nan, inf = float("nan"), float("inf")
    odd = torch.tensor([
        [nan, 0.0, 0.0, 0.0, 0.0, -1.0], [0.0, 0.0, 2.0, nan, nan, nan], [nan] * 6,
        [inf, 0.0, 0.0, 0.0, 0.0, -1.0], [0.0, 0.0, 2.0, inf, 0.0, -1.0], [0.0, 0.0, -inf, 0.0, 0.0, 1.0],
        [0.0, 0.0, 2.0, 0.0, 0.0, 0.0], [0.1, -0.2, 2.0, 0.0, 0.0, -1.0], [2.0, 0.1, 0.0, -1.0, 0.0, 0.0],
        [0.0, 0.0, 2.0, 0.0, 0.0, -1e30], [1e30, 1e30, 1e30, -1.0, -1.0, -1.0], [0.0, 0.0, 2.0, 1e-30, 0.0, -1e-30],
    ])
    mixed = good.clone()
    where = torch.arange(odd.shape[0]) * 157 + 3
    mixed[where] = odd
    keep = torch.ones(good.shape[0], dtype=torch.bool)
    keep[where] = False
    want = m(good, N_samples=S)[0]
    got = m(mixed, N_samples=S)[0]
    assert torch.equal(got["rgb_map"].cpu()[keep], want["rgb_map"].cpu()[keep])
    assert torch.equal(got["depth_map"].cpu()[keep], want["depth_map"].cpu()[keep])
    # the axis-parallel rays are ordinary input for the reference: against the oracle
    axis = odd[7:9]
    ref = O.render_chunk(p, axis, N_samples=S)
    out = m(axis, N_samples=S)[0]
    assert (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item() <= RGB_TOL_F32
    assert (out["depth_map"].cpu() - ref["depth_map"]).abs().max().item() <= RGB_TOL_F32


# ------------------------------------------------------------------------------------ part 2
@pytest.mark.parametrize("ndims,res,dn,an", [(3, (1,), 16, 48), (1, (1, 2, 4), 16, 48), (3, (1, 2), 64, 64), (2, (1,), 8, 16)])
def test_gather_matches_grid_sample(gpu_lib, ndims, res, dn, an):
    p = scenes.make_params(seed=7, gridSize=(13, 9, 11), ndims=ndims, resMode=res, density_n_comp=dn, app_n_comp=an,
                           feature_init="uniform")
    g = torch.Generator().manual_seed(8)
    xyz = torch.rand(5000, 3, generator=g) * 2.2 - 1.1  # a band outside [-1,1] exercises zero padding
    xyz[:8] = torch.tensor([[-1.0, -1, -1], [1, 1, 1], [1, -1, 0], [0, 0, 0], [-1, 1, 1], [0.5, 1, -1], [1, 0.25, 1], [-1, -1, 1]])
    m = _model(p)
    ref_d = O.density_feature(p, xyz)
    assert torch.allclose(m.compute_densityfeature(xyz).cpu(), ref_d, atol=2e-5 * max(1, dn // 16 * len(res) * ndims))
    ref_a = O.app_products(p, xyz)
    got_a = m.app_products(xyz).cpu()
    assert got_a.shape == ref_a.shape
    assert torch.allclose(got_a, ref_a, atol=2e-6)


@pytest.mark.parametrize("an,dtype,M", [(8, torch.float32, 3), (24, torch.float32, 1001), (72, torch.float32, 257),
                                        (72, torch.float16, 530), (40, torch.float16, 77), (64, torch.float16, 15),
                                        (48, torch.float32, 16), (80, torch.float32, 4099)])
def test_app_products_other_widths_and_counts(gpu_lib, an, dtype, M):
    """The stage-level appearance gather writes a wave's sixteen samples through an LDS tile (planes of up to 64
    channels) or directly (wider planes): channel counts on both sides of that limit and off the multiples of 16 (six
    planes, so that their sum stays a multiple of 16 as basis_mat's packing asks), row
    counts that leave a wave partly filled or a workgroup with idle waves."""
    p = scenes.make_params(seed=11, gridSize=(9, 14, 6), ndims=3, resMode=(1, 2), density_n_comp=8, app_n_comp=an,
                           feature_init="uniform", dtype=dtype)
    g = torch.Generator().manual_seed(12)
    xyz = torch.rand(M, 3, generator=g) * 2.1 - 1.05
    got = _model(p).app_products(xyz).cpu()
    ref = O.app_products(p, xyz)
    assert got.shape == ref.shape == (M, 6 * an)
    assert torch.allclose(got, ref, atol=2e-6)


def test_gather_fp16_tables(gpu_lib):
    p = scenes.make_params(seed=9, gridSize=(17, 12, 10), ndims=3, resMode=(1, 2), density_n_comp=16, app_n_comp=48,
                           dtype=torch.float16)
    g = torch.Generator().manual_seed(8)
    xyz = torch.rand(4000, 3, generator=g) * 2 - 1
    m = _model(p)
    # the oracle interpolates the same fp16 values in fp32, so only summation order differs
    assert torch.allclose(m.compute_densityfeature(xyz).cpu(), O.density_feature(p, xyz), atol=2e-5)
    assert torch.allclose(m.app_products(xyz).cpu(), O.app_products(p, xyz), atol=2e-6)


def test_gather_closed_forms(gpu_lib):
    p = scenes.make_params(seed=1, gridSize=(7, 5, 9), density_n_comp=16, app_n_comp=48, ndims=3, resMode=(1, 2))
    for k, pl in enumerate(p.density_plane):
        H, W = pl.shape[-2:]
        ys, xs = torch.meshgrid(torch.linspace(-1, 1, H), torch.linspace(-1, 1, W), indexing="ij")
        pl.zero_()
        pl[0, 3] = (0.3 + 0.1 * k) * xs + (-0.2 + 0.05 * k) * ys + 0.7
        p.density_line[k].fill_(1.0)
    g = torch.Generator().manual_seed(2)
    xyz = torch.rand(300, 3, generator=g) * 2 - 1
    exp = torch.zeros(300)
    for k in range(6):
        m0, m1 = O.MAT_MODE[k // 2]
        exp += (0.3 + 0.1 * k) * xyz[:, m0] + (-0.2 + 0.05 * k) * xyz[:, m1] + 0.7
    assert torch.allclose(_model(p).compute_densityfeature(xyz).cpu(), exp, atol=1e-5)


# ------------------------------------------------------------------------------------ part 3
@pytest.mark.parametrize("prec,tol", [("f32", 2e-6), ("f16x2", 3e-6), ("f16", 4e-3), ("bf16", 3e-2)])
def test_colour_network(gpu_lib, prec, tol):
    p = scenes.make_params(seed=5, gridSize=(4, 4, 4), density_n_comp=4, app_n_comp=48)
    g = torch.Generator().manual_seed(6)
    for M in (1, 31, 32, 33, 4097):
        feats, view = torch.randn(M, 27, generator=g), torch.randn(M, 3, generator=g)
        got = _model(p).render_module(view, feats, precision=prec).cpu()
        ref = O.mlp_render(p, view, feats)
        assert (got - ref).abs().max().item() < tol, (M, prec)


@pytest.mark.parametrize("prec,tol", [("f16", 4e-3), ("bf16", 3e-2)])
@pytest.mark.parametrize("shift", [0, 1, 2, 3])
def test_colour_network_staged_inputs(gpu_lib, prec, tol, shift):
    """The 16-bit modes copy a tile's feature rows into LDS with 16-byte transfers, or 4-byte ones when the feature
    array does not start on a 16-byte boundary (here: a view that starts `shift` floats into its storage), and a
    workgroup's waves take tiles from a shared counter: row counts around whole tiles, around one round of tiles over
    all workgroups and above it, every row checked."""
    p = scenes.make_params(seed=5, gridSize=(4, 4, 4), density_n_comp=4, app_n_comp=48)
    m = _model(p)
    g = torch.Generator().manual_seed(16 + shift)
    for M in (63, 64, 65, 127, 8 * 256 * 64 - 1, 8 * 256 * 64 + 129):
        store = torch.randn(M * 27 + shift, generator=g).to("cuda")
        feats = store[shift:].view(M, 27)
        assert feats.data_ptr() % 16 == (4 * shift) % 16
        view = torch.randn(M, 3, generator=g)
        got = m.render_module(view, feats, precision=prec).cpu()
        ref = O.mlp_render(p, view, feats.cpu())
        assert (got - ref).abs().max().item() < tol, (M, prec, shift)


@pytest.mark.parametrize("prec", ["f32", "f16x2"])
def test_colour_network_large_arguments(gpu_lib, prec):
    """Features far outside the fast sine / cosine reduction's range (|x| > 8192) take the library routines: the
    encoding stays float-accurate.  Weights are scaled down so that the raw features do not saturate the network.
    The split-fp16 mode carries features as two halves, so its inputs must stay below the fp16 maximum (65504)."""
    p = scenes.make_params(seed=5, gridSize=(4, 4, 4), density_n_comp=4, app_n_comp=48)
    # the columns of the raw features and view direction: scaled down, or switched off where such small weights
    # would be fp16 subnormals; the large arguments then act through the sine / cosine columns alone
    p.mlp_w[0][:, :30] *= 1e-5 if prec == "f32" else 0.0
    g = torch.Generator().manual_seed(8)
    feats, view = torch.randn(257, 27, generator=g), torch.randn(257, 3, generator=g)
    if prec == "f32":
        feats[::3] *= 3.0e4
        feats[1::7] *= 2.0e6
    else:
        feats[::3] = (feats[::3] * 1.5e4).clamp(-6.0e4, 6.0e4)
    view[::5] *= 1.0e4
    got = _model(p).render_module(view, feats, precision=prec).cpu()
    ref = O.mlp_render(p, view, feats)
    assert (got - ref).abs().max().item() < 2e-5


@pytest.mark.parametrize("prec,tol", [("f32", 2e-6), ("f16x2", 3e-6), ("f16", 2e-3)])
def test_basis_projection(gpu_lib, prec, tol):
    p = scenes.make_params(seed=5, gridSize=(4, 4, 4), density_n_comp=4, app_n_comp=48, ndims=3, resMode=(1, 2))
    g = torch.Generator().manual_seed(6)
    prod = torch.randn(1000, 288, generator=g)
    got = _model(p).basis(prod, precision=prec).cpu()
    assert (got - O.F.linear(prod, p.basis_mat)).abs().max().item() < tol
    onehot = torch.zeros(3, 288)
    onehot[0, 5], onehot[1, 48 + 7], onehot[2, 287] = 1, 1, 1
    got = _model(p).basis(onehot, precision="f32").cpu()
    assert torch.allclose(got, p.basis_mat[:, [5, 55, 287]].T, atol=1e-7)


# ------------------------------------------------------------------------------------ part 4
def test_weights_against_raw2alpha(gpu_lib):
    p = _scene(S=128, thre=0.0)
    rays = scenes.pinhole_rays(64, 64, 60.0, scenes.sphere_pose(2.5, 5))
    ref = O.render_chunk(p, rays, return_aux=True)
    m = _model(p)
    cull = m.sample_cull(rays)
    sigma = m.density_valid(cull)
    assert torch.allclose(sigma.cpu(), ref["sigma"][ref["ray_valid"]], atol=2e-5, rtol=1e-5)
    w = m.weights(cull, sigma)
    assert torch.allclose(w["weight"].cpu(), ref["weight"], atol=1e-5)
    assert torch.allclose(w["acc_map"].cpu(), ref["acc_map"], atol=1e-5)
    assert torch.allclose(w["depth_map"].cpu(), ref["depth_map"], atol=2e-5)
    band = (ref["weight"] - p.rayMarch_weight_thres).abs() < 1e-6
    assert torch.equal(w["app_mask"].cpu() | band, ref["app_mask"] | band)
    assert w["n_app"] == int(w["app_mask"].sum()) == int(w["app_cnt"].sum())
    # the compact weights are the dense ones at the valid samples
    assert torch.equal(w["w_valid"], w["weight"].reshape(-1)[cull["valid_idx"]])
    # a ray's slots are contiguous, in sample order, and hold exactly its masked samples with their weights
    flat = w["app_mask"].reshape(-1).nonzero()[:, 0]
    order = torch.argsort(w["app_idx"])
    assert torch.equal(w["app_idx"][order], flat)
    assert torch.equal(w["app_w"][order], w["weight"].reshape(-1)[flat])
    S = cull["S"]
    for r in w["app_cnt"].nonzero()[:50, 0].tolist():
        first, n = int(w["app_first"][r]), int(w["app_cnt"][r])
        seg = w["app_idx"][first : first + n]
        assert torch.equal(seg, w["app_mask"][r].nonzero()[:, 0] + r * S)


@pytest.mark.parametrize("white_bg", [True, False])
def test_colour_sum_stage(gpu_lib, white_bg):
    """lm_composite_rgb alone: per-ray sum of weight * rgb over the appearance list, white background before the
    clamp, against the dense tensor expression of the reference (rgb zero outside the mask)."""
    p = _scene(S=128, thre=0.0)
    rays = scenes.pinhole_rays(64, 64, 60.0, scenes.sphere_pose(2.5, 5))
    m = _model(p)
    cull = m.sample_cull(rays)
    w = m.weights(cull, m.density_valid(cull))
    assert w["n_app"] > 1000
    g = torch.Generator(device="cuda").manual_seed(3)
    rgb = torch.rand((w["n_app"], 3), device="cuda", generator=g) * 1.6 - 0.2  # sums that reach past both clamp limits
    got = m.composite_rgb(w, rgb, white_bg=white_bg)
    N, S = rays.shape[0], cull["S"]
    dense = torch.zeros((N * S, 3), device="cuda", dtype=torch.float64)
    dense[w["app_idx"]] = rgb.double()
    exp = (w["weight"].double()[..., None] * dense.view(N, S, 3)).sum(1)
    if white_bg:
        exp = exp + (1.0 - w["acc_map"].double()[:, None])
    exp = exp.clamp(0, 1)
    assert (got.double() - exp).abs().max().item() <= 2e-6
    assert bool((got == 0).any()) or bool((got == 1).any())  # the clamp was reached
    empty = w["app_cnt"] == 0
    assert bool(empty.any())
    if white_bg:
        assert torch.equal(got[empty], (1.0 - w["acc_map"][empty])[:, None].expand(-1, 3).clamp(0, 1))
    else:
        assert bool((got[empty] == 0).all())


@pytest.mark.parametrize("prec,tol", [("f32", 5e-6), ("f16x2", 5e-6), ("f16", 5e-3), ("bf16", 4e-2)])
def test_fused_appearance_features(gpu_lib, prec, tol):
    """gather + basis_mat over the appearance list against the oracle's compute_appfeature"""
    p = _scene(S=64, resMode=(1, 2), thre=0.0)
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 5))
    m = _model(p, mlp_precision=prec)
    cull = m.sample_cull(rays)
    w = m.weights(cull, m.density_valid(cull))
    assert w["n_app"] > 100
    feat = m.app_features_list(cull, w).cpu()
    pts, _, _ = O.sample_ray_within_hull(p, rays[:, :3], rays[:, 3:6], 64)
    xyz = O.normalize_coord(p, pts).reshape(-1, 3)[w["app_idx"].cpu()]
    ref = O.app_feature(p, xyz)
    assert (feat - ref).abs().max().item() < tol


# ------------------------------------------------------------------------------------ whole path
def _check_render(p, rays, tol, S=-1, white_bg=True, **kw):
    ref = O.render_chunk(p, rays, white_bg=white_bg, N_samples=S, return_aux=True)
    out, extra = _model(p, **kw)(rays, white_bg=white_bg, N_samples=S)
    assert extra == {} and set(out) == {"rgb_map", "depth_map"}
    # rays holding a sample whose weight sits within rounding of the threshold may differ by that sample
    band = ((ref["weight"] - p.rayMarch_weight_thres).abs() < 2e-7).any(-1)
    ok = ~band
    d_rgb = (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max(-1).values
    d_dep = (out["depth_map"].cpu() - ref["depth_map"]).abs()
    assert d_rgb[ok].max().item() <= tol, f"rgb max diff {d_rgb[ok].max().item()}"
    assert d_dep[ok].max().item() <= tol, f"depth max diff {d_dep[ok].max().item()}"
    assert int(band.sum()) <= max(3, ref["weight"].numel() // 10000)  # about 4e-5 of the samples sit in the band
    if band.any():
        assert d_rgb[band].max().item() <= 2e-3
    return ref, out


@pytest.mark.parametrize("an,dn,dtype,tol", [(24, 8, torch.float32, RGB_TOL_F32), (40, 12, torch.float32, RGB_TOL_F32),
                                             (80, 16, torch.float32, RGB_TOL_F32), (24, 8, torch.float16, 1e-2)])
def test_render_other_channel_counts(gpu_lib, an, dn, dtype, tol):
    """Appearance planes whose channel count is not 16, 32, 48 or 64 leave the fused gather: the render forms the
    plane x line product matrix in memory and projects it with basis_mat in a second kernel.  Same picture."""
    p = _scene(seed=21, S=96, shift=0.0, ndims=3, resMode=(1, 2), app_n_comp=an, density_n_comp=dn, dtype=dtype)
    rays = scenes.pinhole_rays(48, 40, 42.0, scenes.sphere_pose(2.5, 4))
    ref, _ = _check_render(p, rays, tol, S=96)
    assert ref["app_mask"].any()


@pytest.mark.parametrize("name", golden_names())
def test_render_golden_vectors(gpu_lib, name):
    p, d, cfg = load_golden(name)
    code = cfg.get("app_code")
    out, _ = _model(p)(d["rays"], app_code=code, white_bg=True, N_samples=cfg["N_samples"])
    assert (out["rgb_map"].cpu() - d["rgb_map"]).abs().max().item() <= RGB_TOL_F32
    assert (out["depth_map"].cpu() - d["depth_map"]).abs().max().item() <= RGB_TOL_F32
    out, _ = _model(p)(d["rays"], app_code=code, white_bg=False, N_samples=cfg["N_samples"])
    assert (out["rgb_map"].cpu() - d["rgb_map_black"]).abs().max().item() <= RGB_TOL_F32


@pytest.mark.parametrize("opt,act,shift,res,ndims", [(1, "softplus", 0.0, (1,), 3), (1, "relu", -10.0, (1, 2, 4), 1), (0, "softplus", -1.0, (1, 2), 3)])
def test_render_random_scenes(gpu_lib, opt, act, shift, res, ndims):
    p = _scene(opt=opt, S=128, shift=shift, fea2denseAct=act, resMode=res, ndims=ndims, step_ratio=0.3, thre=0.0)
    rays = scenes.pinhole_rays(80, 80, 70.0, scenes.sphere_pose(2.5, 9))
    ref, _ = _check_render(p, rays, RGB_TOL_F32, S=128)
    assert ref["app_mask"].any(), "scene must exercise the colour network"


@pytest.mark.parametrize("opt,S,step", [(1, 192, 0.08), (1, 320, 0.08), (0, 448, 0.08), (1, 100, 0.08), (1, 600, 0.08),
                                        (0, 1100, 0.08), (0, 3544, 0.004), (0, 4500, 0.0031)])
def test_render_other_sample_counts(gpu_lib, opt, S, step):
    """Sample counts other than 64 and 128 take the cull that walks a ray's bitmap words in one lane, or, for a
    chunk as small as this one, in 2, 4, 8 or 16 lanes (3, 5, 7, 2, 10 and 18 words per ray here; 56 words at the
    reference's default step, and 71: beyond the 64 words a ray's word mask can describe, so every word is walked).
    The last two use a step that spreads the samples over the whole box, so that late words hold valid samples."""
    p = _scene(opt=opt, S=S, shift=0.0, step_ratio=step, thre=0.0)
    rays = scenes.pinhole_rays(40, 40, 34.0, scenes.sphere_pose(2.5, 9))
    ref, _ = _check_render(p, rays, RGB_TOL_F32, S=S)
    assert ref["app_mask"].any()
    if S > 1100:
        last = ref["ray_valid"].reshape(rays.shape[0], S)[:, S - S // 4:].any()
        assert last, "valid samples in the last quarter of the rays"
    if S > 1100:
        # the same rays often enough for the quad-per-ray march (chunks above 12 288 rays)
        m = _model(p, mlp_precision="f16x2")
        small = m(rays, N_samples=S)[0]
        many = m(rays.repeat(8, 1), N_samples=S)[0]
        assert torch.equal(many["rgb_map"][-rays.shape[0]:], small["rgb_map"])
        assert torch.equal(many["depth_map"][-rays.shape[0]:], small["depth_map"])


def test_render_configuration_sweep(gpu_lib):
    """Forty seeded random configurations (sampler, sample count, levels, plane orientations, table storage,
    activation, occupancy threshold, ragged ray counts) against the oracle: the combinations the fixed cases leave out."""
    import random

    rnd = random.Random(1234)
    for it in range(40):
        opt = rnd.choice([0, 1])
        S = rnd.choice([16, 37, 64, 100, 128, 200, 256, 330])
        res = rnd.choice([(1,), (1, 2), (1, 2, 4)])
        ndims = rnd.choice([1, 2, 3])
        fp16 = rnd.random() < 0.35
        act = rnd.choice(["softplus", "relu"])
        shift = rnd.choice([0.0, -1.0])
        thre = rnd.choice([0.0, 0.0, 0.5])
        mask = rnd.random() < 0.8
        w, h, cut, seed = rnd.randint(3, 70), rnd.randint(3, 70), rnd.randint(0, 5), rnd.randint(0, 1000)
        p = _scene(seed=seed, opt=opt, S=S, thre=thre, shift=shift, with_mask=mask, resMode=res, ndims=ndims,
                   fea2denseAct=act, step_ratio=0.25 if opt == 0 else 2.0)
        if fp16:
            p = O.to_fp16_features(p)
        rays = scenes.pinhole_rays(w, h, 0.8 * max(w, h), scenes.sphere_pose(2.5, seed % 17))[cut:]
        try:
            _, out = _check_render(p, rays, RGB_TOL_16 if fp16 else RGB_TOL_F32, S=S if opt == 0 else -1, mlp_precision="f16x2")
            # the same rays repeated until the chunk takes the large-chunk kernels (a quad per ray in the march, a lane
            # per word or ray in the cull) instead of the small-chunk ones: identical bits for the first copy
            reps = 13000 // rays.shape[0] + 1
            big, _ = _model(p, mlp_precision="f16x2")(rays.repeat(reps, 1), N_samples=S if opt == 0 else -1)
            n = rays.shape[0]
            assert torch.equal(big["rgb_map"][:n], out["rgb_map"]) and torch.equal(big["depth_map"][:n], out["depth_map"])
            assert torch.equal(big["rgb_map"][-n:], out["rgb_map"])
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: opt {opt} S {S} res {res} ndims {ndims} fp16 {fp16} act {act} "
                                 f"shift {shift} thre {thre} mask {mask} {w}x{h} cut {cut} seed {seed}: {e}") from e


def test_appearance_embedding_and_density_projection(gpu_lib):
    """encode_app (latent folded into the first layer's bias, switched per call) and
    nonlinear_density against the oracle."""
    p = _scene(S=64, resMode=(1, 2), encode_app=True, nonlinear_density=True, fea2denseAct="relu", boost=3.0)
    p.basis_den.abs_()
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 5))
    m = _model(p)
    outs = {}
    for code in (0, 7, 0):  # switching back and forth must re-fold the bias
        ref = O.render_chunk(p, rays, app_code=code, return_aux=True)
        assert ref["app_mask"].any()
        out, _ = m(rays, app_code=torch.tensor(code))
        band = ((ref["weight"] - 1e-3).abs() < 2e-7).any(-1)
        assert (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max(-1).values[~band].max().item() <= RGB_TOL_F32
        assert (out["depth_map"].cpu() - ref["depth_map"]).abs()[~band].max().item() <= RGB_TOL_F32
        outs.setdefault(code, []).append(out["rgb_map"])
    assert torch.equal(outs[0][0], outs[0][1]) and not torch.equal(outs[0][0], outs[7][0])
    g = torch.Generator().manual_seed(1)
    xyz = torch.rand(3000, 3, generator=g) * 2 - 1
    assert torch.allclose(m.compute_densityfeature(xyz).cpu(), O.density_feature(p, xyz), atol=2e-5)
    with pytest.raises(ValueError):
        m(rays)  # a model with an embedding needs the code
    with pytest.raises(NotImplementedError):
        _model(_scene(S=64))(rays, app_code=1)


def _oracle_in_chunks(p, rays, S=-1, chunk=16384):
    """render_chunk over slices of the rays: rgb, depth, masks and depths of every ray, the rays that hold a weight
    within rounding of the appearance threshold, and the number of appearance samples."""
    keep = {k: [] for k in ("rgb_map", "depth_map", "ray_valid", "z_vals", "band")}
    n_app = 0
    for i in range(0, rays.shape[0], chunk):
        r = O.render_chunk(p, rays[i:i + chunk], N_samples=S, return_aux=True)
        r["band"] = ((r["weight"] - p.rayMarch_weight_thres).abs() < 2e-7).any(-1)
        n_app += int(r["app_mask"].sum())
        for k in keep:
            keep[k].append(r[k])
    out = {k: torch.cat(v) for k, v in keep.items()}
    out["n_app"] = n_app
    return out


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("opt,step_ratio", [(1, 2.0), (0, 0.5), (0, 3.47)])
def test_render_c1_tiny_config(gpu_lib, opt, step_ratio, dense):
    """The tiny full-render configuration at its full 400 x 400 image, 128 samples per ray, both samplers: the hull
    sampler (sampling_opt 1, n_importance 128) and the equal-step sampler (sampling_opt 0, N_samples 128) with the
    reference's default step_ratio 0.5 (128 steps reach half a scene unit behind the entry point) and with 3.47
    (the steps span the box diagonal).  Each with the stated init (shift -10: every weight is below the appearance
    threshold, the image is background) and the dense variant (shift 0) that runs every stage.  Masks, indices and
    depths bit-exact, rgb / depth within 1e-4."""
    rays = scenes.c1_rays(400, 400)
    p = scenes.c1_scene(dense=dense, sampling_opt=opt, step_ratio=step_ratio)
    assert p.alpha_volume is None and rays.shape[0] == 160000
    ref = _oracle_in_chunks(p, rays, S=128)
    assert (ref["n_app"] > 0) == dense and 0 < int(ref["ray_valid"].sum()) < ref["ray_valid"].numel()
    m = _model(p)
    cull = m.sample_cull(rays, N_samples=128)
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"])
    assert torch.equal(cull["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])
    assert torch.equal(cull["z_vals"].cpu(), ref["z_vals"])
    out, _ = m(rays, N_samples=128)
    assert m.last_counts()["n_valid"] == int(ref["ray_valid"].sum())
    # rays holding a sample whose weight is within 2e-7 of the appearance threshold may differ by that sample
    ok = ~ref["band"]
    assert int(ref["band"].sum()) <= max(3, ref["ray_valid"].numel() // 10000)
    d_rgb = (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max(-1).values
    assert d_rgb[ok].max().item() <= RGB_TOL_F32
    assert (out["depth_map"].cpu() - ref["depth_map"]).abs()[ok].max().item() <= RGB_TOL_F32
    if ref["band"].any():
        assert d_rgb[ref["band"]].max().item() <= 2e-3
    if not dense:
        # no sample reaches the colour network: every pixel is the grey 1 - acc of the white background
        assert bool((out["rgb_map"][:, 0] == out["rgb_map"][:, 1]).all()) and bool((out["rgb_map"][:, 0] == out["rgb_map"][:, 2]).all())


def test_render_16bit_network_and_fp16_tables(gpu_lib):
    p = _scene(S=64)
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 5))
    _check_render(p, rays, RGB_TOL_F32, mlp_precision="f16x2")
    _check_render(p, rays, RGB_TOL_16, mlp_precision="f16")
    _check_render(p, rays, 3e-2, mlp_precision="bf16")
    _check_render(O.to_fp16_features(p), rays, RGB_TOL_16)


def test_chunk_drivers(gpu_lib):
    from landmark_amd.render import MultiBlockParallelHIP, renderer_fn

    p = _scene(S=64)
    rays = scenes.pinhole_rays(40, 40, 40.0, scenes.sphere_pose(2.5, 5))
    m = _model(p)
    full, _ = m(rays)
    for chunk, exact in ((1, True), (333, True), (333, False), (4096, False)):
        ret, extra = renderer_fn(rays, m, chunk=chunk, device="cuda", exact_chunk=exact)
        assert extra == {} and set(ret) == {"rgb_map", "depth_map"}
        # rays are independent: any chunking gives identical bits
        assert torch.equal(ret["rgb_map"], full["rgb_map"]) and torch.equal(ret["depth_map"], full["depth_map"])
    # the library's own choice of chunk: everything at once here, bounded by the workspace budget and by
    # 32-bit sample indices; a single call larger than that is split inside forward
    assert m.preferred_chunk(rays.shape[0]) == rays.shape[0] and m.preferred_chunk(1 << 30) == 1 << 20
    small = _model(p, capacity="worst")
    small.workspace_budget = 5000 * small.lib.lm_render_workspace_bytes(C.byref(small._model_struct(64, True)), 1 << 16) // (1 << 16)
    more = scenes.pinhole_rays(80, 80, 80.0, scenes.sphere_pose(2.5, 5))
    assert 4096 <= small.preferred_chunk(more.shape[0]) < more.shape[0]
    split, _ = small(more)
    whole, _ = m(more)
    assert torch.equal(split["rgb_map"], whole["rgb_map"]) and torch.equal(split["depth_map"], whole["depth_map"])
    fused = MultiBlockParallelHIP()
    fused.allocate_tensors(m, 512)
    ret = fused.forward(rays[:512].cuda(), app_code=None, white_bg=True)
    assert torch.equal(ret["rgb_map"], full["rgb_map"][:512])
    with pytest.raises(NotImplementedError):
        m(rays, is_train=True)


@pytest.mark.parametrize("opt,S", [(1, 128), (0, 200)])
def test_workspace_capacity_overflow_is_reported_and_repeatable(gpu_lib, opt, S):
    """A workspace below the worst case: rays whose samples do not fit are dropped and counted, the counters still
    report what would have fit, and the repeat with those capacities equals the worst-case render bit for bit."""
    from landmark_amd import _lib as L

    p = _scene(opt=opt, S=S, thre=0.0, step_ratio=0.3)
    rays = scenes.pinhole_rays(100, 90, 85.0, scenes.sphere_pose(2.5, 9)).cuda()
    N = rays.shape[0]
    m = _model(p, capacity="worst")
    full, _ = m(rays, N_samples=S)
    want = m.last_counts()
    assert want["overflow"] == 0 and want["n_app"] > 1000

    def render(caps):
        st = L.LmModel.from_buffer_copy(m._model_struct(S, True))
        st.cap_valid, st.cap_app = caps
        need = m.lib.lm_render_workspace_bytes(C.byref(st), N)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        rgb, dep = torch.empty((N, 3), device="cuda"), torch.empty((N,), device="cuda")
        cnt = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device="cuda")
        L.check(m.lib.lm_render(C.byref(st), rays.data_ptr(), N, ws.data_ptr(), need, rgb.data_ptr(), dep.data_ptr(), cnt.data_ptr(),
                                L.current_stream()), "lm_render")
        torch.cuda.synchronize()
        c = cnt.cpu().long() & 0xFFFFFFFF
        return rgb, dep, int(c[L.LM_STAT_N_VALID]), int(c[L.LM_STAT_N_APP]), int(c[L.LM_STAT_OVERFLOW]), need

    worst_bytes = m.lib.lm_render_workspace_bytes(C.byref(m._model_struct(S, True)), N)
    # room for a third of the valid samples: rays are dropped, the valid count is still the whole chunk's
    rgb, dep, nv, na, over, need = render((want["n_valid"] // 3, want["n_app"]))
    assert over > 0 and nv == want["n_valid"] and na < want["n_app"] and need < worst_bytes
    kept = (rgb == full["rgb_map"]).all(-1) & (dep == full["depth_map"])
    dropped = ~kept
    assert int(dropped.sum()) <= over and bool((rgb[dropped] == 1.0).all()) and bool((dep[dropped] == 0.0).all())
    # room for half of the appearance samples: those rays keep their depth and show the background
    rgb, dep, nv, na, over, _ = render((want["n_valid"], want["n_app"] // 2))
    assert over > 0 and nv == want["n_valid"] and na == want["n_app"]
    assert torch.equal(dep, full["depth_map"]) and not torch.equal(rgb, full["rgb_map"])
    # exactly enough room: nothing dropped, identical bits
    rgb, dep, nv, na, over, _ = render((want["n_valid"], want["n_app"]))
    assert over == 0 and torch.equal(rgb, full["rgb_map"]) and torch.equal(dep, full["depth_map"])
    # the wrapper's adaptive sizing: starts too small, reads the counters, repeats the chunk, remembers
    a = _model(p)
    a.small_workspace = 0  # chunks this small would otherwise get the worst case
    a.samples_per_ray = [0.2 * want["n_valid"] / N, 0.2 * want["n_app"] / N]
    assert a.capacities(N, S)[0] * 4 < want["n_valid"] * 4 and a.capacities(N, S) != (0, 0)
    out, _ = a(rays, N_samples=S)
    assert torch.equal(out["rgb_map"], full["rgb_map"]) and torch.equal(out["depth_map"], full["depth_map"])
    assert a.samples_per_ray[0] * N >= want["n_valid"] and a.samples_per_ray[1] * N >= want["n_app"]
    assert a.last_counts()["overflow"] == 0
    out2, _ = a(rays, N_samples=S)  # now sized right the first time
    assert torch.equal(out2["rgb_map"], full["rgb_map"])


@pytest.mark.parametrize("opt,S,term,fp16,div", [(1, 128, 0.0, False, None), (1, 128, 1e-4, False, None), (0, 200, 1e-4, False, None),
                                                  (1, 64, 0.0, True, None), (0, 330, 0.0, False, None), (1, 128, 1e-4, False, (2, 3))])
def test_both_march_kernels_give_the_same_bits(gpu_lib, opt, S, term, fp16, div):
    """Chunks of up to 12288 rays march with a wave per ray, larger ones with a quad per ray: the same operations in
    the same order, so a ray's result does not depend on the size of the chunk it arrives in (early termination,
    word masks of long rays, fp16 tables and block-stacked tables included)."""
    from landmark_amd.render import renderer_fn

    if div is None:
        p = _scene(opt=opt, S=S, thre=0.0, step_ratio=0.2, resMode=(1, 2))
    else:
        p = scenes.make_params(seed=11, gridSize=(10, 9, 12), near_far=[0.5, 4.5], n_importance=S, sampling_opt=opt,
                               density_shift=0.0, resMode=(1, 2), ndims=1, plane_division=div)
        for t in p.density_plane:
            t.mul_(8.0)
    if fp16:
        p = O.to_fp16_features(p)
    rays = scenes.pinhole_rays(200, 150, 170.0, scenes.sphere_pose(2.5, 9)).cuda()  # 30000 rays: one quad-march chunk
    m = _model(p, term_eps=term, mlp_precision="f16x2")
    whole, _ = renderer_fn(rays, m, chunk=1 << 20, N_samples=S, device="cuda")
    parts, _ = renderer_fn(rays, m, chunk=7001, N_samples=S, device="cuda", exact_chunk=True)  # five wave-march chunks
    assert float(whole["rgb_map"].min()) < 0.9
    assert torch.equal(whole["depth_map"], parts["depth_map"])
    assert torch.equal(whole["rgb_map"], parts["rgb_map"])
    ref = O.render_chunk(p, rays[:3000].cpu(), N_samples=S, return_aux=True)
    band = ((ref["weight"] - 1e-3).abs() < 2e-7).any(-1)
    tol = (RGB_TOL_16 if fp16 else RGB_TOL_F32) + term * 4.5
    assert (parts["rgb_map"][:3000].cpu() - ref["rgb_map"]).abs().max(-1).values[~band].max().item() <= tol
    assert (parts["depth_map"][:3000].cpu() - ref["depth_map"]).abs()[~band].max().item() <= tol


@pytest.mark.parametrize("S,width", [(128, 96), (64, 40), (100, 96), (128, 50)])
def test_row_length_hint_changes_nothing(gpu_lib, S, width):
    """ray_row only changes the order in which rays are visited (8 x 8 pixel tiles): bit-identical output, for
    chunks that start mid-row and end mid-band, sample counts with and without the one-launch cull, and a row
    length that is not a multiple of 8 (ignored)."""
    p = _scene(opt=1, S=S, thre=0.0)
    rays = scenes.pinhole_rays(width, 61, 70.0, scenes.sphere_pose(2.5, 9))[37:]
    m = _model(p)
    a, _ = m(rays)
    m.ray_row_length = width
    b, _ = m(rays)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])
    assert a["rgb_map"].min() < 0.99


@pytest.mark.parametrize("fp16_tables,res", [(False, (1,)), (True, (1,)), (True, (1, 2))])
def test_early_termination_bounds(gpu_lib, fp16_tables, res):
    """Rays stop up to three samples late (four are gathered per round); fp32 planes, three and six narrow fp16 planes."""
    p = _scene(S=128, resMode=res)
    if fp16_tables:
        p = O.to_fp16_features(p)
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 5))
    exact, _ = _model(p)(rays)
    term, _ = _model(p, term_eps=1e-4)(rays)
    ref = O.render_chunk(p, rays)
    assert (exact["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item() <= (RGB_TOL_16 if fp16_tables else RGB_TOL_F32)
    # all samples after T < 1e-4 have weight < 1e-4 < threshold: colour unchanged up to the white
    # background term (<= 1e-4); depth loses at most T * z_far
    assert (term["rgb_map"] - exact["rgb_map"]).abs().max().item() <= 1e-4
    assert (term["depth_map"] - exact["depth_map"]).abs().max().item() <= 1e-4 * 4.5 * 1.5


@pytest.mark.parametrize("prec", ["f32", "f16x2"])
def test_termination_at_the_benchmark_rule_keeps_the_parity_bar(gpu_lib, prec):
    """bench.py stops a ray at T < 1e-4 / far, chosen so that neither rgb (<= eps with a white background) nor depth
    (<= eps * far) can move by more than the fp32 bar: rendered with that value the picture still meets the bar against
    the oracle, which never stops a ray, and the appearance samples are the same ones."""
    p = _scene(S=128, resMode=(1, 2))
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 5))
    eps = 1e-4 / float(p.near_far[1])
    m = _model(p, term_eps=eps, mlp_precision=prec)
    got, _ = m(rays)
    ref = O.render_chunk(p, rays)
    assert (got["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item() <= RGB_TOL_F32
    assert (got["depth_map"].cpu() - ref["depth_map"]).abs().max().item() <= RGB_TOL_F32
    n_app = m.last_counts()["n_app"]
    m0 = _model(p, mlp_precision=prec)
    exact, _ = m0(rays)
    assert n_app == m0.last_counts()["n_app"] > 0
    assert (got["rgb_map"] - exact["rgb_map"]).abs().max().item() <= eps + 1e-6


def test_ray_generation_and_rgba8(gpu_lib):
    from landmark_amd.render import generate_rays, postprocess_rgba8

    pose = torch.cat([scenes.orbit_pose(2.6, 1.9, 7), torch.tensor([[0.0], [0.0], [1483.6378]])], 1)
    for H, W in ((1080, 1920), (7, 5)):
        got = generate_rays(pose, H, W).cpu()
        ref = O.generate_rays(pose, H, W)
        assert torch.equal(got[:, :3], ref[:, :3])
        assert (got[:, 3:] - ref[:, 3:]).abs().max().item() <= 2e-7  # three-term dot product, order / fma differ
    g = torch.Generator().manual_seed(0)
    rgb = torch.rand(480 * 640, 3, generator=g)
    rgb[:4] = torch.tensor([[0.0, 1.0, 0.5], [0.999, 0.0039, 0.00392157], [1.0, 1.0, 1.0], [0.0, 0.0, 0.0]])
    assert torch.equal(postprocess_rgba8(rgb.cuda(), 480, 640).cpu(), O.postprocess_rgba8(rgb, 480, 640))


def test_render_frame_from_pose(gpu_lib):
    """Pose -> RGBA8 image in one call: equals rays from the pose, the chunked render and the byte conversion done
    step by step with the oracle, up to one grey level where a channel sits on a rounding boundary."""
    from landmark_amd.render import render_frame

    p = _scene(S=64, thre=0.0)
    H, W, focal = 72, 96, 90.0
    pose = torch.cat([scenes.orbit_pose(2.6, 1.9, 3), torch.tensor([[0.0], [0.0], [focal]])], 1)
    m = _model(p, mlp_precision="f16x2")
    img, dep = render_frame(m, pose, H, W, chunk=20 * W, depth=True)
    assert img.shape == (H, W, 4) and img.dtype == torch.uint8 and m.ray_row_length == 0
    ref = O.render_chunk(p, O.generate_rays(pose, H, W))
    want = O.postprocess_rgba8(ref["rgb_map"], H, W)
    diff = (img.cpu().int() - want.int()).abs()
    assert diff.max().item() <= 1 and (diff > 0).float().mean().item() < 0.01
    assert (dep.cpu().reshape(-1) - ref["depth_map"]).abs().max().item() <= 2 * RGB_TOL_F32
    assert want[..., :3].min() < 250  # the scene is visible
    # the pinned device-to-host step of the serving loop
    from landmark_amd.render import pinned_image
    host = pinned_image(H, W)
    render_frame(m, pose, H, W, chunk=20 * W, host_image=host)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(host, img.cpu())
    with pytest.raises(ValueError):
        render_frame(m, pose, H, W, host_image=torch.empty((H, W, 4), dtype=torch.uint8))
    # chunks dealt to one, two (the default) or three streams: the same bits
    for n in (1, 3):
        img_n, dep_n = render_frame(m, pose, H, W, chunk=20 * W, depth=True, streams=n)
        assert torch.equal(img_n, img) and torch.equal(dep_n, dep)
    # a workspace sized far too small, on a frame large enough to pass the floors of the adaptive sizing: the chunks
    # of both streams overflow, are repeated after the streams join, and the frame comes out as on a worst-case
    # workspace; the model remembers the room it needed
    H2, W2 = 144, 192
    pose2 = torch.cat([scenes.orbit_pose(2.6, 1.9, 3), torch.tensor([[0.0], [0.0], [2 * focal]])], 1)
    img_w, dep_w = render_frame(_model(p, mlp_precision="f16x2", capacity="worst"), pose2, H2, W2, chunk=72 * W2, depth=True)
    tight = _model(p, mlp_precision="f16x2")
    tight.small_workspace = 0
    tight.samples_per_ray = [0.5, 0.05]
    img_t, dep_t = render_frame(tight, pose2, H2, W2, chunk=72 * W2, depth=True)
    assert torch.equal(img_t, img_w) and torch.equal(dep_t, dep_w)
    assert tight.samples_per_ray[0] > 0.5 and tight.samples_per_ray[1] > 0.05
    before = list(tight.samples_per_ray)
    img_t, _ = render_frame(tight, pose2, H2, W2, chunk=72 * W2, depth=True)
    assert torch.equal(img_t, img_w) and tight.samples_per_ray == before


# ------------------------------------------------------------------------------------ occupancy volume from the model
ALPHA_TOL = 2e-6  # alpha lies in [0, 1]


def _pooled_max(alpha):
    a = alpha.clamp(0, 1).transpose(0, 2).contiguous()[None, None]
    return torch.nn.functional.max_pool3d(a, kernel_size=3, padding=1, stride=1)[0, 0]


def _check_mask_update(p, gs, inc, want_volume=None, want_aabb=None):
    ref_aabb, ref_vol = O.update_alpha_mask(p, gs, inc)
    if want_volume is not None:
        assert torch.equal(ref_vol, want_volume) and torch.equal(ref_aabb, want_aabb)
    m = _model(p)
    new_aabb = m.updateAlphaMask(gs, inc)
    vol = m.alphaMask.alpha_volume[0, 0].cpu()
    assert tuple(vol.shape) == tuple(gs[::-1]) and torch.equal(m.alphaMask.aabb.cpu(), p.aabb)
    # a voxel whose pooled alpha sits within rounding of the threshold may flip
    thres = p.alphaMask_thres * 10**inc
    band = (_pooled_max(O.get_dense_alpha(p, gs)[0]) - thres).abs() < 5e-7  # 1 - exp(-x) near 1e-3: a few ulp of 1.0
    assert torch.equal(vol[~band], ref_vol[~band])
    assert int(band.sum()) <= max(2, vol.numel() // 1000)
    if not band.any():
        assert torch.equal(new_aabb.cpu(), ref_aabb)
    return m, vol, new_aabb


@pytest.mark.parametrize("name", alphamask_names())
def test_dense_alpha_and_mask_update_golden(gpu_lib, name):
    p, d, cfg = load_golden(name, kind="alphamask")
    m = _model(p)
    alpha, xyz = m.getDenseAlpha()
    assert torch.equal(xyz.cpu(), d["dense_xyz"])
    assert (alpha.cpu() - d["dense_alpha"]).abs().max().item() <= ALPHA_TOL
    alpha, _ = m.getDenseAlpha(cfg["gs"])
    assert (alpha.cpu() - d["dense_alpha_gs"]).abs().max().item() <= ALPHA_TOL
    _check_mask_update(p, cfg["gs"], cfg["inc"], d["new_volume"], d["new_aabb"])


@pytest.mark.parametrize("act,shift,res,with_mask", [("softplus", -6.0, (1,), False), ("relu", -10.0, (1, 2), True)])
def test_mask_update_random_scene_then_render(gpu_lib, act, shift, res, with_mask):
    p = _scene(grid=(17, 19, 15), S=64, shift=shift, fea2denseAct=act, resMode=res, with_mask=with_mask, boost=40.0)
    # density confined to a slab so that the rebuilt volume is neither empty nor full
    for k, ln in enumerate(p.density_line):
        c = torch.linspace(-1, 1, ln.shape[2])
        ln.mul_(((c > -0.5) & (c < 0.3)).float()[None, None, :, None])
    gs = [40, 36, 44]
    m, vol, new_aabb = _check_mask_update(p, gs, 0)
    assert 0 < int(vol.sum()) < vol.numel()
    # the model now culls with the rebuilt volume
    p2 = p.to("cpu")
    p2.alpha_volume, p2.alpha_aabb = vol, p.aabb
    rays = scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.5, 4))
    ref = O.render_chunk(p2, rays, return_aux=True)
    out = m.sample_cull(rays)
    assert torch.equal(out["ray_valid"].cpu(), ref["ray_valid"])
    res_, _ = m(rays)
    assert (res_["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item() <= RGB_TOL_F32


# ------------------------------------------------------------------------------------ block-stacked models
@pytest.mark.parametrize("name", stacked_names())
def test_stacked_model_golden(gpu_lib, name):
    p, d, cfg = load_golden(name, kind="stacked")
    code = cfg.get("app_code")
    m = _model(p)
    ref = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], app_code=code, return_aux=True)
    cull = m.sample_cull(d["rays"], N_samples=cfg["N_samples"])
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"])
    # densities of the valid samples through the stage entry point
    sigma = m.density_valid(cull)
    assert (sigma.cpu() - ref["sigma"][ref["ray_valid"]]).abs().max().item() <= 1e-5 * max(1.0, ref["sigma"].max().item())
    for white, key in ((True, "rgb_map"), (False, "rgb_map_black")):
        out, _ = m(d["rays"], app_code=code, white_bg=white, N_samples=cfg["N_samples"])
        assert (out["rgb_map"].cpu() - d[key]).abs().max().item() <= RGB_TOL_F32
        assert (out["depth_map"].cpu() - d["depth_map"]).abs().max().item() <= RGB_TOL_F32


@pytest.mark.parametrize("div,res,prec", [((2, 3), (1,), "f32"), ((4, 2), (1, 2), "f16x2"), ((3, 3), (1, 2, 4), "f16x2")])
def test_stacked_model_random_scene(gpu_lib, div, res, prec):
    p = scenes.make_params(seed=11, gridSize=(10, 9, 12), near_far=[0.5, 4.5], n_importance=96, sampling_opt=1,
                           density_shift=0.0, resMode=res, ndims=1, plane_division=div)
    for t in p.density_plane:
        t.mul_(8.0)
    rays = scenes.pinhole_rays(72, 72, 60.0, scenes.sphere_pose(2.5, 7))
    ref = O.render_chunk(p, rays, return_aux=True)
    assert ref["app_mask"].any()
    out, _ = _model(p, mlp_precision=prec)(rays)
    band = ((ref["weight"] - p.rayMarch_weight_thres).abs() < 2e-7).any(-1)
    assert (out["rgb_map"].cpu() - ref["rgb_map"])[~band].abs().max().item() <= RGB_TOL_F32
    assert (out["depth_map"].cpu() - ref["depth_map"])[~band].abs().max().item() <= RGB_TOL_F32
    assert int(band.sum()) <= max(2, rays.shape[0] // 500)


def test_stacked_model_single_block_is_refused(gpu_lib):
    """plane_division (1, 1): the reference's block coordinate is 0 / 0 there (its render is NaN, and so is the
    oracle's); the wrapper and the C ABI refuse it instead of inventing a result."""
    from landmark_amd import _lib as L

    p = scenes.make_params(seed=11, gridSize=(10, 9, 12), near_far=[0.5, 4.5], n_importance=32, sampling_opt=1,
                           density_shift=0.0, ndims=1, plane_division=(1, 1))
    rays = scenes.pinhole_rays(8, 8, 7.0, scenes.sphere_pose(2.5, 7))
    assert torch.isnan(O.render_chunk(p, rays)["rgb_map"]).any()
    with pytest.raises(L.LandmarkError, match="one block"):
        _model(p)
    p2 = scenes.make_params(seed=11, gridSize=(10, 9, 12), near_far=[0.5, 4.5], n_importance=32, sampling_opt=1,
                            density_shift=0.0, ndims=1, plane_division=(2, 1))
    m = _model(p2)
    g = m._geom(32)
    g.div0 = g.div1 = 1
    cnt = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device="cuda")
    rc = m.lib.lm_sample_cull(C.byref(g), rays.cuda().data_ptr(), rays.shape[0], cnt.data_ptr(), cnt.data_ptr(), None,
                              cnt.data_ptr(), None, cnt.data_ptr(), L.current_stream())
    assert rc == -2 and b"1 x 1" in m.lib.lm_last_error()


@pytest.mark.parametrize("div", [(2, 3), (5, 4), (7, 1)])
def test_block_assignment_is_bit_faithful(gpu_lib, div):
    """Planes that are constant inside a block and differ between blocks (relu activation, one channel set): the density
    of a sample then names the block it was assigned to, exactly, for every valid sample including those next to block
    borders; a second model with planes linear in the block-relative x pins those coordinates to float accuracy."""
    B = div[0] * div[1]
    p = scenes.make_params(seed=2, gridSize=(6, 5, 7), near_far=[0.5, 4.5], n_importance=128, sampling_opt=1,
                           density_shift=0.0, resMode=(1,), ndims=1, plane_division=div, fea2denseAct="relu")
    ids = torch.arange(1, B + 1, dtype=torch.float32)
    p.density_plane[0].zero_()
    p.density_plane[0][0, 0] = ids.view(B, 1, 1).expand(B, 5, 6)
    p.density_line[0].zero_()
    p.density_line[0][0, 0] = 1.0
    rays = scenes.pinhole_rays(64, 64, 50.0, scenes.sphere_pose(2.5, 3))
    ref = O.render_chunk(p, rays, return_aux=True)
    m = _model(p)
    cull = m.sample_cull(rays)
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"])
    sig = m.density_valid(cull).cpu()
    want = ref["sigma"][ref["ray_valid"]]
    assert len(set(want.round().tolist())) == B  # every block is hit
    # the reference interpolates over the block axis with a coordinate that is an integer up to rounding
    assert (sig - want).abs().max().item() <= 1e-5 * B
    assert torch.equal(sig.round(), want.round())
    # block-relative x: plane value = column index inside the block
    p.density_plane[0][0, 0] = torch.arange(6, dtype=torch.float32).view(1, 1, 6).expand(B, 5, 6)
    ref = O.render_chunk(p, rays, return_aux=True)
    sig = _model(p).density_valid(cull).cpu()
    assert (sig - ref["sigma"][ref["ray_valid"]]).abs().max().item() <= 2e-5


def test_stacked_checkpoint_round_trip(gpu_lib, tmp_path):
    from landmark_amd import checkpoint

    p, d, cfg = load_golden(stacked_names()[0], kind="stacked")
    path = str(tmp_path / "x-merged-stack.th")
    checkpoint.save_checkpoint(p, path)
    q = checkpoint.load_checkpoint(path, resMode=cfg["resMode"], ndims=1, sampling_opt=cfg["sampling_opt"],
                                   n_importance=cfg["n_importance"], alpha_mask_filter_thre=cfg["thre"])
    assert q.plane_division == cfg["plane_division"] and q.density_plane[0].dim() == 5
    out, _ = _model(q)(d["rays"], N_samples=cfg["N_samples"])
    assert (out["rgb_map"].cpu() - d["rgb_map"]).abs().max().item() <= RGB_TOL_F32
