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


@pytest.mark.parametrize("prec,tol", [("f16", 4e-3), ("f16x2", 3e-6)])
def test_isolated_colour_network_full_size(gpu_lib, prec, tol):
    """2^23 rows (27 features ~ N(0,1), unit view directions) through the fused network: a strided sample against
    the oracle, and row independence at full size (a reversed copy of the input gives the reversed output, bit for bit:
    rows meet other rows in a wave tile, a different lane and a different workgroup)."""
    dev = "cuda"
    p = scenes.make_params(seed=3, gridSize=(8, 8, 8), density_n_comp=4, app_n_comp=48)
    m = _model(p, mlp_precision=prec)
    M = 1 << 23
    g = torch.Generator(device=dev).manual_seed(3)
    feat = torch.randn((M, 27), device=dev, generator=g)
    view = torch.nn.functional.normalize(torch.randn((M, 3), device=dev, generator=g), dim=-1)
    out = m.render_module(view, feat)
    assert out.shape == (M, 3) and float(out.min()) >= 0.0 and float(out.max()) <= 1.0
    idx = torch.arange(0, M, 127, device=dev)[: 1 << 16]
    ref = O.mlp_render(p, view[idx].cpu(), feat[idx].cpu())
    assert (out[idx].cpu() - ref).abs().max().item() <= tol
    back = m.render_module(view.flip(0).contiguous(), feat.flip(0).contiguous())
    assert torch.equal(back.flip(0), out)


def test_largest_chunk_the_abi_admits(gpu_lib):
    """One lm_render call of 2^25 - 1 rays x 128 samples (N*S = 2^32 - 128, the last sample index a chunk may have):
    a 1024 x 512 image repeated 64 times.  Every copy must equal the first bit for bit (sample and slot indices
    near 2^32 behave like those near 0), the first must equal the same image rendered on its own, and one ray more
    is refused."""
    from landmark_amd import _lib as L
    from tests.test_gpu_parity import _scene

    dev = "cuda"
    p = _scene(opt=1, S=128, grid=(33, 37, 41), step_ratio=2.0)
    m = _model(p, mlp_precision="f16x2")
    tile = scenes.pinhole_rays(1024, 512, 900.0, scenes.sphere_pose(2.5, 5)).to(dev)
    T = tile.shape[0]
    N = (1 << 25) - 1
    rays = tile.repeat(64, 1)[:N].contiguous()
    alone = m(tile)[0]
    one = m.last_counts()
    assert one["n_valid"] > T and one["n_app"] > T // 4
    m.samples_per_ray = [1.3 * one["n_valid"] / T, 1.3 * one["n_app"] / T]
    rgb = torch.full((N, 3), -1.0, device=dev)
    depth = torch.full((N,), -1.0, device=dev)
    m.render_into(rays, rgb, depth)
    c = m.last_counts()
    assert c["overflow"] == 0
    assert 63 * one["n_valid"] <= c["n_valid"] <= 64 * one["n_valid"] and 63 * one["n_app"] <= c["n_app"] <= 64 * one["n_app"]
    assert torch.equal(rgb[:T], alone["rgb_map"]) and torch.equal(depth[:T], alone["depth_map"])
    for k in (1, 31, 62):
        assert torch.equal(rgb[k * T:(k + 1) * T], rgb[:T]) and torch.equal(depth[k * T:(k + 1) * T], depth[:T])
    assert torch.equal(rgb[63 * T:], rgb[:T - 1]) and torch.equal(depth[63 * T:], depth[:T - 1])
    del rgb, depth
    more = torch.cat([rays, tile[:1]])
    with pytest.raises(L.LandmarkError, match="32-bit"):
        m.render_into(more, torch.empty((N + 1, 3), device=dev), torch.empty((N + 1,), device=dev))


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


def _frame_sample(rays, H=1080, W=1920):
    """Rays of the 1080p frame for the oracle: 4096 around the image centre, and a strided sample of the whole
    frame (every `stride`-th pixel, a stride coprime to the row length so that all columns are visited)."""
    centre = torch.arange(W * (H // 2) + W // 2 - 4096, W * (H // 2) + W // 2)
    return centre, torch.arange(0, H * W, 37), torch.arange(0, H * W, 521)


def test_full_frame_sample_masks_bit_exact(gpu_lib, frame):
    """The decisions the benchmark frame is culled with, on the frame's own 256^3 occupancy volume and 1080p
    camera: valid mask, ascending valid-sample indices and sample depths equal the oracle's bit for bit on 60 000
    rays spread over the whole frame, and the whole-chunk render counts exactly the oracle's valid samples."""
    import copy

    p, rays, m = frame
    centre, dense, _ = _frame_sample(rays)
    idx = torch.unique(torch.cat([centre, dense]))
    sub = rays[idx.cuda()].contiguous()
    q = copy.copy(p)  # the mask needs the box, the sampler settings and the occupancy volume only
    q.aabb, q.alpha_volume, q.alpha_aabb = p.aabb.cpu(), p.alpha_volume.cpu(), p.alpha_aabb.cpu()
    _, z, valid = O.sample_and_cull(q, sub.cpu())
    frac = valid.float().mean().item()
    assert 0.02 < frac < 0.5 and bool(valid.any(-1).any()) and not bool(valid.any(-1).all())
    cull = m.sample_cull(sub)
    assert torch.equal(cull["ray_valid"].cpu(), valid)
    assert torch.equal(cull["valid_idx"].cpu(), valid.reshape(-1).nonzero()[:, 0])
    assert torch.equal(cull["z_vals"].cpu(), z)
    assert cull["n_valid"] == int(valid.sum())
    # lm_render's own cull (a lane per ray and bitmap word, no index list) on the same rays
    rgb = torch.empty((sub.shape[0], 3), device="cuda")
    dep = torch.empty((sub.shape[0],), device="cuda")
    m.samples_per_ray[0] = max(m.samples_per_ray[0], 1.3 * int(valid.sum()) / sub.shape[0])
    m.render_into(sub, rgb, dep)
    c = m.last_counts()
    assert c["n_valid"] == int(valid.sum()) and c["overflow"] == 0
    # rays without a valid sample are background: exactly white, depth 0
    empty = ~valid.any(-1)
    assert bool((rgb.cpu()[empty] == 1.0).all()) and bool((dep.cpu()[empty] == 0.0).all())


def test_production_shape_full_size_against_oracle(gpu_lib):
    """The shape most of the reference's run configurations use (one orientation at three levels, the equal-step
    AABB sampler at its default of half a grid cell per step = 3544 samples per ray, appearance embedding, density
    projection) on the benchmark frame's occupancy volume and camera, where the coarse occupancy level acts on every
    ray: masks, index list and depths of 8 000 rays spread over the frame equal the oracle's bit for bit, the
    whole-chunk render counts the oracle's valid and appearance samples, and its pixels meet the fp32 bar."""
    p = scenes.production_scene(base=1024, step_ratio=0.5, device="cuda")
    rays = scenes.c4_rays(1080, 1920, device="cuda")
    m = _model(p, mlp_precision="f16x2")
    assert m._samples_for(-1) == 3544 and m._coarse_can_act(3544)
    idx = torch.arange(0, 1080 * 1920, 257)
    sub = rays[idx.cuda()].contiguous()
    ref = O.render_chunk(p.to("cpu"), sub.cpu(), return_aux=True, app_code=3)
    valid = ref["ray_valid"]
    assert 0.001 < valid.float().mean().item() < 0.5
    cull = m.sample_cull(sub)
    assert torch.equal(cull["ray_valid"].cpu(), valid)
    assert torch.equal(cull["valid_idx"].cpu(), valid.reshape(-1).nonzero()[:, 0])
    assert torch.equal(cull["z_vals"].cpu(), ref["z_vals"])
    out, _ = m(sub, app_code=3)
    c = m.last_counts()
    band = ((ref["weight"] - p.rayMarch_weight_thres).abs() < 2e-7).any(-1)
    assert c["n_valid"] == int(valid.sum()) and c["overflow"] == 0
    assert abs(c["n_app"] - int(ref["app_mask"].sum())) <= int(band.sum())
    ok = ~band
    assert (out["rgb_map"].cpu() - ref["rgb_map"])[ok].abs().max().item() <= 1e-4
    assert (out["depth_map"].cpu() - ref["depth_map"])[ok].abs().max().item() <= 1e-4
    off = _model(p, mlp_precision="f16x2", coarse_occupancy=False)
    plain, _ = off(sub, app_code=3)
    assert torch.equal(plain["rgb_map"], out["rgb_map"]) and torch.equal(plain["depth_map"], out["depth_map"])


def test_full_frame_oracle_spot_check(gpu_lib, frame):
    """rgb / depth of the frame's centre block and of a strided sample of the whole frame against the oracle, with
    the masks of the same rays (the oracle's full render needs the 17 GB of tables on the host)."""
    p, rays, m = frame
    centre, _, sparse = _frame_sample(rays)
    idx = torch.unique(torch.cat([centre, sparse]))
    sub = rays[idx.cuda()].contiguous()
    out, _ = m(sub)
    n_valid = m.last_counts()["n_valid"]
    ref = O.render_chunk(p.to("cpu"), sub.cpu(), return_aux=True)
    cull = m.sample_cull(sub)
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"]) and n_valid == int(ref["ray_valid"].sum())
    assert torch.equal(cull["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])
    assert torch.equal(cull["z_vals"].cpu(), ref["z_vals"])
    band = ((ref["weight"] - 1e-3).abs() < 2e-7).any(-1)
    assert ref["app_mask"].any() and int(band.sum()) <= 2
    d_rgb = (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max(-1).values
    d_dep = (out["depth_map"].cpu() - ref["depth_map"]).abs()
    assert d_rgb[~band].max().item() <= 1e-4 and d_dep[~band].max().item() <= 1e-4


# ---------------------------------------------------------------------------------------------
# Fifth benchmark configuration: one GPU's share of a plane-parallel 4K city block.  Planes 8192^2 x
# (16 + 48) channels stored as fp16 and interpolated in fp32 (the reference's half storage,
# app/models/gridnerf_tensor_parallel.py:74-81, 180-181), AABB flattened to z in [-0.1, 0.1], a
# 512 x 512 x 64 heightfield occupancy, 256 samples per ray, aerial camera at 30 degrees pitch.
# ---------------------------------------------------------------------------------------------
def _c5_sample(rays, H=2160, W=3840):
    """A few thousand rays of the 4K frame: a block at the image centre, whole-image strided samples,
    and the rows where the view crosses the far and near rims of the slab (the silhouette)."""
    centre = ((torch.arange(H // 2 - 16, H // 2 + 16)[:, None]) * W + torch.arange(W // 2 - 32, W // 2 + 32)[None]).reshape(-1)
    strided = torch.arange(0, H * W, 4099)
    rim = torch.cat([(torch.tensor(r) * W + torch.arange(0, W, 7)) for r in (0, 40, 120, 300, H - 300, H - 1)])
    idx = torch.unique(torch.cat([centre, strided, rim]))
    return idx, rays[idx.to(rays.device)]


def test_city_block_reduced_resolution_against_oracle(gpu_lib):
    """Same structure at 1024^2 tables (the oracle finishes in seconds): fp16 tables, flattened AABB, the
    512 x 512 x 64 heightfield mask, S = 256, the 4K camera.  Masks bit-exact, rgb / depth within 1e-2."""
    p = scenes.c5_scene(res=1024, device="cpu")
    rays_all = scenes.c5_rays(2160, 3840, device="cpu")
    idx, rays = _c5_sample(rays_all)
    assert p.density_plane[0].dtype == torch.float16 and p.n_importance == 256 and p.alpha_volume.shape == (64, 512, 512)
    ref = O.render_chunk(p, rays, return_aux=True)
    assert ref["app_mask"].any() and 0 < int(ref["ray_valid"].sum()) < ref["ray_valid"].numel()
    m = _model(p, mlp_precision="f16")
    cull = m.sample_cull(rays)
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"])
    assert torch.equal(cull["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])
    assert torch.equal(cull["z_vals"].cpu(), ref["z_vals"])
    for prec in ("f16", "f16x2"):
        out, _ = _model(p, mlp_precision=prec)(rays)
        d_rgb = (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item()
        d_dep = (out["depth_map"].cpu() - ref["depth_map"]).abs().max().item()
        assert d_rgb <= 1e-2 and d_dep <= 1e-2, (prec, d_rgb, d_dep)
    # the AABB sampler (sampling_opt 0) on the same tables and mask, 256 steps from the slab entry
    p.sampling_opt, p.step_ratio = 0, 5.0
    ref = O.render_chunk(p, rays, N_samples=256, return_aux=True)
    assert ref["app_mask"].any()
    m = _model(p, mlp_precision="f16")
    cull = m.sample_cull(rays, N_samples=256)
    assert torch.equal(cull["ray_valid"].cpu(), ref["ray_valid"])
    out, _ = m(rays, N_samples=256)
    assert (out["rgb_map"].cpu() - ref["rgb_map"]).abs().max().item() <= 1e-2
    assert (out["depth_map"].cpu() - ref["depth_map"]).abs().max().item() <= 1e-2


@pytest.fixture(scope="module")
def city():
    free, _ = torch.cuda.mem_get_info()
    if free < 120 << 30:
        pytest.skip(f"the 25.8 GB fp16 tables, their source copy and a 1 M-ray workspace need 120 GB; {free >> 30} GB free")
    p = scenes.c5_scene(res=8192, device="cuda")
    m = _model(p, mlp_precision="f16")
    rays = scenes.c5_rays(2160, 3840, device="cuda")
    return p, rays, m


def test_city_block_full_size_compaction_identities(gpu_lib, city):
    p, rays, m = city
    assert sum(t.numel() * t.element_size() for t in m._tables) > 25.7e9
    chunk = rays[3840 * 540 : 3840 * 540 + (1 << 20)]  # one 1 M-ray chunk across the middle of the frame
    out = m.sample_cull(chunk, want_z=False)
    idx, n = out["valid_idx"], out["n_valid"]
    assert 0 < n < chunk.shape[0] * 256
    assert n == int(out["ray_valid"].sum())
    assert bool((idx[1:] > idx[:-1]).all())
    assert bool(out["ray_valid"].reshape(-1)[idx].all())
    pop = out["ray_valid"].reshape(-1, 64).sum(1)
    assert torch.equal(out["word_prefix"].long() & 0xFFFFFFFF, torch.cumsum(pop, 0) - pop)
    # the whole-chunk render's own cull (one lane per ray walking four words) counts the same samples
    rgb = torch.empty((chunk.shape[0], 3), device="cuda")
    dep = torch.empty((chunk.shape[0],), device="cuda")
    m.render_into(chunk, rgb, dep)
    assert m.last_counts()["n_valid"] == n


def test_city_block_full_size_chunk_invariance_and_background(gpu_lib, city):
    from landmark_amd.render import renderer_fn

    p, rays, m = city
    a, _ = renderer_fn(rays, m, chunk=1 << 19, device="cuda", exact_chunk=True)
    b, _ = renderer_fn(rays, m, chunk=300007, device="cuda", exact_chunk=True)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])
    assert float(a["rgb_map"].min()) >= 0.0 and float(a["rgb_map"].max()) <= 1.0
    black, _ = renderer_fn(rays, m, chunk=1 << 19, white_bg=False, device="cuda", exact_chunk=True)
    assert bool((a["rgb_map"] >= black["rgb_map"] - 1e-6).all())
    assert torch.equal(a["depth_map"], black["depth_map"])
    empty = a["depth_map"] == 0
    assert bool(empty.any()) and not bool(empty.all())
    assert bool((a["rgb_map"][empty] == 1.0).all()) and bool((black["rgb_map"][empty] == 0.0).all())
    assert float(a["rgb_map"][~empty].min()) < 0.99  # the colour network contributes


def test_city_block_full_size_oracle_spot_check(gpu_lib, city):
    """A few hundred rays of the full-size scene against the oracle's operation sequence run by PyTorch's own
    GPU kernels on the same device tensors (the 25.8 GB tables would take minutes on the host; the
    reduced-resolution test above holds the bit-exact comparison with the CPU oracle)."""
    p, rays, m = city
    idx = torch.cat([torch.arange(3840 * 1080 + 1900, 3840 * 1080 + 2028), torch.arange(0, 2160 * 3840, 65537)])
    sub = rays[idx.cuda()]
    ref = O.render_chunk(p, sub, return_aux=True)
    assert ref["app_mask"].any() and not ref["ray_valid"].all()
    out, _ = m(sub)
    assert (out["rgb_map"] - ref["rgb_map"]).abs().max().item() <= 1e-2
    assert (out["depth_map"] - ref["depth_map"]).abs().max().item() <= 1e-2
    cull = m.sample_cull(sub, want_z=False)
    # PyTorch's GPU kernels may contract or reorder what its CPU kernels round separately: decisions of samples
    # within rounding of a boundary may differ from the device oracle (they are bit-exact against the CPU oracle)
    assert int((cull["ray_valid"] != ref["ray_valid"]).sum()) <= max(2, ref["ray_valid"].numel() // 20000)
