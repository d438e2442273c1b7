"""GPU tests at the benchmark configurations' full sizes, through properties that do not
need the CPU oracle on the whole input: closed forms, sortedness / counting identities,
chunk invariance, plus an oracle spot check on a thin slice."""
import pytest
import torch

from landmark_amd import scenes
from oracle import gridnerf_oracle as O

pytestmark = pytest.mark.gpu


def _model(p, **kw):
    from landmark_amd.model import GridNeRFHIP

    return GridNeRFHIP(p, **kw)


def test_isolated_gather_full_size_closed_form(gpu_lib):
    """3 planes 2048^2 x 64 ch fp32, 2^24 uniform queries: affine planes and unit lines must
    reproduce the affine function (bilinear interpolation is exact on it)."""
    dev, res, C = "cuda", 2048, 64
    p = scenes.make_params(seed=2, gridSize=(res, res, res), ndims=3, resMode=(1,), density_n_comp=C, app_n_comp=16,
                           device=dev, feature_init="uniform")
    g = torch.Generator(device=dev).manual_seed(5)
    coef = torch.rand(3, C, 3, device=dev, generator=g) - 0.5
    lin = torch.linspace(-1, 1, res, device=dev)
    for k in range(3):
        a, b, c = coef[k, :, 0], coef[k, :, 1], coef[k, :, 2]
        p.density_plane[k] = (a[:, None, None] * lin[None, None, :] + b[:, None, None] * lin[None, :, None] + c[:, None, None])[None].contiguous()
        p.density_line[k] = torch.ones(1, C, res, 1, device=dev)
    m = _model(p, release_source=True)
    M = 1 << 24
    xyz = torch.rand(M, 3, device=dev, generator=g) * 2 - 1
    got = m.compute_densityfeature(xyz)
    exp = torch.zeros(M, device=dev, dtype=torch.float64)
    for k in range(3):
        m0, m1 = O.MAT_MODE[k]
        s = coef[k].double().sum(0)
        exp += s[0] * xyz[:, m0].double() + s[1] * xyz[:, m1].double() + s[2]
    err = (got.double() - exp).abs().max().item()
    assert err < 2e-4, err  # 192 fp32 terms of magnitude <= 1


@pytest.fixture(scope="module")
def frame():
    p = scenes.c4_scene(P=3, base=1024, device="cuda", density_shift=0.0)
    rays = scenes.c4_rays(1080, 1920, device="cuda")
    m = _model(p, mlp_precision="f16x2")
    return p, rays, m


def test_full_frame_compaction_identities(gpu_lib, frame):
    p, rays, m = frame
    out = m.sample_cull(rays, want_z=False)
    idx = out["valid_idx"]
    n = out["n_valid"]
    assert 0 < n < rays.shape[0] * 128
    assert n == int(out["ray_valid"].sum())  # count = popcount of the bitmap
    assert bool((idx[1:] > idx[:-1]).all())  # strictly ascending = stable order, no duplicates
    assert bool(out["ray_valid"].reshape(-1)[idx].all())  # every listed sample is marked valid
    # word prefixes are the exclusive scan of the per-word popcounts
    pop = out["ray_valid"].reshape(-1, 64).sum(1)
    assert torch.equal(out["word_prefix"].long() & 0xFFFFFFFF, torch.cumsum(pop, 0) - pop)


def test_full_frame_chunk_invariance_and_background(gpu_lib, frame):
    from landmark_amd.render import renderer_fn

    p, rays, m = frame
    a, _ = renderer_fn(rays, m, chunk=262144, device="cuda")
    b, _ = renderer_fn(rays, m, chunk=100003, device="cuda")
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])
    assert float(a["rgb_map"].min()) >= 0.0 and float(a["rgb_map"].max()) <= 1.0
    black, _ = renderer_fn(rays, m, chunk=262144, white_bg=False, device="cuda")
    # white background adds (1 - acc) >= 0 to every channel before the clamp; depth does not depend on it
    assert bool((a["rgb_map"] >= black["rgb_map"] - 1e-6).all())
    assert torch.equal(a["depth_map"], black["depth_map"])
    # rays that hit nothing are exactly white / black with zero depth
    empty = (a["depth_map"] == 0)
    assert bool(empty.any()) and bool((a["rgb_map"][empty] == 1.0).all()) and bool((black["rgb_map"][empty] == 0.0).all())


def test_full_frame_oracle_spot_check(gpu_lib, frame):
    p, rays, m = frame
    out, _ = m(rays[: 1920 * 540 + 960][-4096:])  # 4096 rays around the image centre
    sub = rays[: 1920 * 540 + 960][-4096:].cpu()
    ref = O.render_chunk(p.to("cpu"), sub, return_aux=True)
    band = ((ref["weight"] - 1e-3).abs() < 2e-7).any(-1)
    assert ref["app_mask"].any()
    d_rgb = (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max(-1).values
    d_dep = (out["depth_map"].cpu() - ref["depth_map"]).abs()
    assert d_rgb[~band].max().item() <= 1e-4 and d_dep[~band].max().item() <= 1e-4
