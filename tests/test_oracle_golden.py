"""The oracle against the golden vectors written from the reference's own forward
(tests/golden/make_golden.py).  Same ATen calls on the same CPU => exact equality is
expected for everything, and required for the geometry / mask outputs."""
import pytest
import torch

from oracle import gridnerf_oracle as O
from tests.helpers import alphamask_names, golden_names, load_golden, stacked_names

NAMES = golden_names()


def test_fixtures_present():
    assert len(NAMES) >= 6


@pytest.mark.parametrize("name", NAMES)
def test_forward_matches_reference(name):
    p, d, cfg = load_golden(name)
    out = O.render_chunk(p, d["rays"], white_bg=True, N_samples=cfg["N_samples"], app_code=cfg.get("app_code"))
    assert torch.equal(out["rgb_map"], d["rgb_map"])
    assert torch.equal(out["depth_map"], d["depth_map"])
    out_b = O.render_chunk(p, d["rays"], white_bg=False, N_samples=cfg["N_samples"], app_code=cfg.get("app_code"))
    assert torch.equal(out_b["rgb_map"], d["rgb_map_black"])


@pytest.mark.parametrize("name", NAMES)
def test_subfunctions_match_reference(name):
    p, d, cfg = load_golden(name)
    o, v = d["rays"][:, :3], d["rays"][:, 3:6]
    if cfg["sampling_opt"]:
        pts, z, inside = O.sample_ray_within_hull(p, o, v, cfg["n_importance"])
    else:
        pts, z, inside = O.sample_ray_aabb(p, o, v, cfg["N_samples"])
        assert p.nSamples == cfg["nSamples"]
        assert float(p.stepSize) == pytest.approx(cfg["stepSize"], rel=1e-6)
    assert torch.equal(pts, d["sub_pts"]) and torch.equal(z, d["sub_z"])
    assert torch.equal(inside, d["sub_inside"].bool())
    q = O.normalize_coord(p, pts).reshape(-1, 3)
    assert torch.equal(O.density_feature(p, q), d["sub_density_feature"])
    feats = O.app_feature(p, q)
    assert torch.equal(feats, d["sub_app_feature"])
    vd = d["rays"][:, None, 3:6].expand(pts.shape).reshape(-1, 3)
    latent = None
    if cfg.get("encode_app"):
        latent = p.embedding_app[cfg["app_code"]][None].expand(feats.shape[0], 48)
    assert torch.equal(O.mlp_render(p, vd, feats, latent), d["sub_rgb"])
    sig = O.feature2density(p, d["sub_density_feature"]).view(z.shape)
    dists = torch.cat((z[:, 1:] - z[:, :-1], torch.zeros_like(z[:, :1])), dim=-1)
    a, w, t = O.raw2alpha(sig, dists * p.distance_scale)
    assert torch.equal(a, d["sub_alpha"]) and torch.equal(w, d["sub_weight"]) and torch.equal(t, d["sub_t_last"])
    assert torch.equal(O.positional_encoding(feats[:5], 2), d["sub_pe"])
    if p.alpha_volume is not None:
        assert torch.equal(O.sample_alpha(p.alpha_volume, p.alpha_aabb, pts.reshape(-1, 3)), d["sub_alpha_lookup"])


@pytest.mark.parametrize("name", NAMES)
def test_sample_mask_matches_reference_subresults(name):
    """sample_and_cull's mask = the reference's inside-box mask AND its occupancy lookups above the threshold
    (both stored in the fixture for every sample), and its depths are the reference sampler's."""
    p, d, cfg = load_golden(name)
    xyz, z, valid = O.sample_and_cull(p, d["rays"], cfg["N_samples"])
    want = d["sub_inside"].bool()
    if p.alpha_volume is not None:
        want = want & (d["sub_alpha_lookup"].view(want.shape) > p.alpha_mask_filter_thre)
    assert torch.equal(valid, want) and torch.equal(z, d["sub_z"]) and torch.equal(xyz, d["sub_pts"])
    aux = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], app_code=cfg.get("app_code"), return_aux=True)
    assert torch.equal(aux["ray_valid"], valid)


def test_fixture_masks_are_discriminating():
    """In several fixtures the occupancy volume removes samples that are inside the box, and keeps others."""
    culling = 0
    for name in NAMES:
        p, d, cfg = load_golden(name)
        if p.alpha_volume is None:
            continue
        inside = d["sub_inside"].bool()
        keep = d["sub_alpha_lookup"].view(inside.shape) > p.alpha_mask_filter_thre
        culling += int(bool((inside & ~keep).any()) and bool((inside & keep).any()))
    assert culling >= 3


def test_chunk_driver_is_chunk_invariant():
    p, d, cfg = load_golden("hull_softplus_L1")
    full = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"])
    for chunk in (1, 7, 16, 4096):
        ret, extra = O.renderer_fn(d["rays"], p, chunk=chunk, N_samples=cfg["N_samples"])
        assert extra == {} and set(ret) == {"rgb_map", "depth_map"}
        # rays are independent; ATen's GEMM blocking depends on the row count, so the
        # colour network may differ in the last bits between chunkings
        assert torch.allclose(ret["rgb_map"], full["rgb_map"], atol=1e-6, rtol=0)
        assert torch.equal(ret["depth_map"], full["depth_map"])


@pytest.mark.parametrize("name", alphamask_names())
def test_alpha_mask_update_matches_reference(name):
    """getDenseAlpha / updateAlphaMask of the reference (tests/golden/alphamask_*.npz)."""
    p, d, cfg = load_golden(name, kind="alphamask")
    assert float(p.stepSize) == pytest.approx(cfg["stepSize"], rel=1e-6)
    alpha, xyz = O.get_dense_alpha(p)
    assert torch.equal(xyz, d["dense_xyz"]) and torch.equal(alpha, d["dense_alpha"])
    alpha_gs, _ = O.get_dense_alpha(p, cfg["gs"])
    assert torch.equal(alpha_gs, d["dense_alpha_gs"])
    new_aabb, vol = O.update_alpha_mask(p, cfg["gs"], cfg["inc"])
    assert torch.equal(vol, d["new_volume"]) and torch.equal(new_aabb, d["new_aabb"])
    assert torch.equal(d["new_mask_aabb"], p.aabb)
    # the fixture is discriminating: some but not all voxels are set, and the box is tight on every axis
    assert 0 < int(vol.sum()) < vol.numel()
    assert bool((new_aabb[0] > p.aabb[0]).any()) and bool((new_aabb[1] < p.aabb[1]).any())


def test_alpha_mask_pool_brute_force():
    """update_alpha_mask's pooling against a plain triple loop on a random lattice."""
    p, d, cfg = load_golden(alphamask_names()[0], kind="alphamask")
    gs = [5, 4, 6]
    alpha, xyz = O.get_dense_alpha(p, gs)
    new_aabb, vol = O.update_alpha_mask(p, gs, 0)
    a = alpha.clamp(0, 1)
    lo, hi = [None] * 3, [None] * 3
    for x in range(gs[0]):
        for y in range(gs[1]):
            for z in range(gs[2]):
                m = max(
                    float(a[xx, yy, zz])
                    for xx in range(max(x - 1, 0), min(x + 2, gs[0]))
                    for yy in range(max(y - 1, 0), min(y + 2, gs[1]))
                    for zz in range(max(z - 1, 0), min(z + 2, gs[2]))
                )
                want = 1.0 if m >= p.alphaMask_thres else 0.0
                assert float(vol[z, y, x]) == want
                if want:
                    for k, v in enumerate(xyz[x, y, z].tolist()):
                        lo[k] = v if lo[k] is None else min(lo[k], v)
                        hi[k] = v if hi[k] is None else max(hi[k], v)
    assert new_aabb[0].tolist() == lo and new_aabb[1].tolist() == hi


@pytest.mark.parametrize("name", stacked_names())
def test_stacked_model_matches_reference(name):
    """Block-stacked planes rendered on one device (tests/golden/stacked_*.npz, written from
    GridNeRFBranchParallel.forward with ckpt_type "full")."""
    p, d, cfg = load_golden(name, kind="stacked")
    code = cfg.get("app_code")
    out = O.render_chunk(p, d["rays"], white_bg=True, N_samples=cfg["N_samples"], app_code=code, return_aux=True)
    assert torch.equal(out["rgb_map"], d["rgb_map"]) and torch.equal(out["depth_map"], d["depth_map"])
    out_b = O.render_chunk(p, d["rays"], white_bg=False, N_samples=cfg["N_samples"], app_code=code)
    assert torch.equal(out_b["rgb_map"], d["rgb_map_black"])
    assert out["app_mask"].any()
    xyzb = O.assign_blocks_to_samples(p, d["sub_xyz"])
    assert torch.equal(xyzb, d["sub_xyzb"])
    assert torch.equal(O.density_feature(p, xyzb), d["sub_density_feature"])
    assert torch.equal(O.app_feature(p, xyzb), d["sub_app_feature"])


def test_block_assignment_plain_loop():
    """Block index and block-relative coordinates against scalar arithmetic in float64."""
    p, d, cfg = load_golden(stacked_names()[0], kind="stacked")
    d0, d1 = cfg["plane_division"]
    g = torch.Generator().manual_seed(3)
    xyz = torch.rand(500, 3, generator=g) * 1.98 - 0.99
    out = O.assign_blocks_to_samples(p, xyz)
    for (x, y, z), (lx, ly, lz, b) in zip(xyz.double().tolist(), out.double().tolist()):
        bx, by = int((x + 1) / (2 / d0)), int((y + 1) / (2 / d1))
        assert round((b + 1) / 2 * (d0 * d1 - 1)) == bx * d1 + by
        assert lz == z
        assert abs(lx - (((x + 1) - bx * 2 / d0) * d0 - 1)) < 1e-5 and abs(ly - (((y + 1) - by * 2 / d1) * d1 - 1)) < 1e-5
