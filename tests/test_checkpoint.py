"""Checkpoint format round trip (the reference's save/load layout,
app/models/gridnerf_sequential.py:171-242) and what the loader infers from it."""
import numpy as np
import pytest
import torch

from landmark_amd import checkpoint as CK
from landmark_amd import scenes
from oracle import gridnerf_oracle as O


def _scene(**kw):
    p = scenes.make_params(seed=4, gridSize=(6, 7, 5), ndims=3, resMode=(1, 2), near_far=[0.4, 4.0], n_importance=24,
                           density_shift=0.0, **kw)
    for t in p.density_plane:
        t.mul_(8.0)
    p.alpha_volume = scenes.blob_occupancy((5, 7, 6), 4, 0.5, seed=2)
    p.alpha_aabb = p.aabb.clone()
    return p


@pytest.mark.parametrize("extra", [{}, {"encode_app": True, "nonlinear_density": True}])
def test_round_trip_preserves_the_render(tmp_path, extra):
    p = _scene(**extra)
    path = str(tmp_path / "model.th")
    CK.save_checkpoint(p, path)
    raw = torch.load(path, weights_only=False)
    assert set(raw) == {"kwargs", "state_dict", "alphaMask.shape", "alphaMask.mask", "alphaMask.aabb"}
    assert raw["alphaMask.mask"].dtype == np.uint8 and tuple(raw["alphaMask.shape"]) == (1, 1, 5, 7, 6)
    assert "density_plane.5" in raw["state_dict"] and "renderModule.mlp.4.bias" in raw["state_dict"]
    with pytest.raises(ValueError, match="sampling_opt"):
        CK.load_checkpoint(path)  # a single-model file does not record the sampler
    q = CK.load_checkpoint(path, sampling_opt=1, n_importance=24)  # ndims and the levels are read from the file
    assert q.ndims == 3 and q.resMode == [1, 2] and q.encode_app == bool(extra) and q.nonlinear_density == bool(extra)
    assert torch.equal(q.alpha_volume, p.alpha_volume)
    rays = scenes.pinhole_rays(12, 12, 10.0, scenes.sphere_pose(2.5, 1))
    code = 2 if extra else None
    a = O.render_chunk(p, rays, app_code=code)
    b = O.render_chunk(q, rays, app_code=code)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])


def test_loader_rejects_inconsistent_or_stacked_layouts():
    ck = CK.checkpoint_from_params(_scene())
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2, 4, 8], sampling_opt=1)  # 6 planes do not split into 4 levels
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2], ndims=2, sampling_opt=1)
    with pytest.raises(ValueError, match="ndims"):
        # read as one orientation with six levels, the XZ and YZ planes would pass for levels of the XY plane
        CK.params_from_checkpoint(ck, ndims=1, resMode=[1, 2, 4, 8, 16, 32], sampling_opt=1)
    legacy = {"kwargs": {k: v for k, v in ck["kwargs"].items() if k != "density_n_comp"}, "state_dict": ck["state_dict"]}
    with pytest.raises(ValueError, match="wrong ndims"):  # a file without the list: the plane sizes still tell
        CK.params_from_checkpoint(legacy, ndims=1, resMode=[1, 2, 4, 8, 16, 32], sampling_opt=1)
    ck["state_dict"]["density_plane.0"] = ck["state_dict"]["density_plane.0"][:, :, None]  # [1,C,B,h,w]
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2], sampling_opt=1)  # stacked planes without a plane division


def test_common_reference_layout_is_not_misread():
    """One orientation with three levels (ndims 1, resMode [1,2,4]: most of the reference's confs): the three
    planes must load as levels of the XY plane, not as XY, XZ, YZ of a one-level model."""
    p = scenes.make_params(seed=8, gridSize=(6, 7, 5), ndims=1, resMode=(1, 2, 4), near_far=[0.4, 4.0], sampling_opt=0,
                           step_ratio=0.3, density_shift=0.0)
    ck = CK.checkpoint_from_params(p)
    assert ck["kwargs"]["density_n_comp"] == [16]
    q = CK.params_from_checkpoint(ck, sampling_opt=0)
    assert q.ndims == 1 and q.resMode == [1, 2, 4] and q.sampling_opt == 0
    rays = scenes.pinhole_rays(8, 8, 7.0, scenes.sphere_pose(2.5, 1))
    a, b = O.render_chunk(p, rays), O.render_chunk(q, rays)
    assert torch.equal(a["rgb_map"], b["rgb_map"])


def test_block_stacked_round_trip(tmp_path):
    """The "-merged-stack" layout: 5-D planes, lines with a block axis, plane_division in kwargs["args"];
    state-dict names may carry the wrappers' ".module" / ".params" infixes."""
    p = scenes.make_params(seed=6, gridSize=(5, 4, 6), ndims=1, resMode=(1, 2), near_far=[0.4, 4.0], n_importance=20,
                           density_shift=0.0, plane_division=(2, 3))
    for t in p.density_plane:
        t.mul_(8.0)
    ck = CK.checkpoint_from_params(p)
    assert ck["state_dict"]["density_plane.1"].shape == (1, 16, 6, 8, 10) and ck["state_dict"]["app_line.0"].shape == (1, 48, 6, 6)
    ck["state_dict"] = {k.replace("_plane.", "_plane.module.params.").replace("_line.", "_line.params."): v
                        for k, v in ck["state_dict"].items()}
    path = str(tmp_path / "x-merged-stack.th")
    torch.save(ck, path)
    q = CK.load_checkpoint(path)  # a merged checkpoint carries its run configuration
    assert q.plane_division == [2, 3] and q.ndims == 1 and q.resMode == [1, 2] and q.n_importance == 20 and q.sampling_opt == 1
    rays = scenes.pinhole_rays(10, 10, 8.0, scenes.sphere_pose(2.5, 1))
    a, b = O.render_chunk(p, rays), O.render_chunk(q, rays)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and a["rgb_map"].min() < 0.99
    with pytest.raises(ValueError):
        CK.load_checkpoint(path, resMode=[1, 2], plane_division=[2, 2])  # 4 blocks, the file holds 6


# ---- files written by the reference's own save / merge_ckpts (tests/golden/make_golden.py --only=checkpoint) ----
def _reference_file(name):
    import json
    import os

    from tests.helpers import GOLDEN_DIR

    z = np.load(os.path.join(GOLDEN_DIR, f"ckpt_{name}.npz"))
    cfg = json.loads(bytes(z["cfg_json"]).decode())
    data = {k: torch.from_numpy(z[k]) for k in z.files if k != "cfg_json"}
    path = os.path.join(GOLDEN_DIR, f"ckpt_{name}" + ("-merged-stack.th" if cfg["stacked"] else ".th"))
    return path, data, cfg


def test_reference_written_single_model_file():
    """GridBaseSequential.save output: kwargs with a tensor aabb and density_n_comp sliced to ndims, a 5-D
    alphaMask.shape, no bias tensors (bias_enable 0), embedding_app and basis_den in the state dict."""
    path, d, cfg = _reference_file("aabb_relu_L3_P1_production")
    p = CK.load_checkpoint(path, sampling_opt=cfg["sampling_opt"], alpha_mask_filter_thre=cfg["alpha_mask_filter_thre"])  # weights-only load
    assert p.ndims == 1 and p.resMode == [1, 2, 4] and len(p.density_plane) == 3
    assert p.mlp_b == [None, None, None] and p.encode_app and p.nonlinear_density
    assert p.alpha_volume.shape == (5, 7, 6) and p.nSamples == cfg["nSamples"]
    ref = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], app_code=cfg["app_code"], return_aux=True)
    assert ref["app_mask"].any()
    assert torch.equal(ref["rgb_map"], d["rgb_map"]) and torch.equal(ref["depth_map"], d["depth_map"])
    black = O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], app_code=cfg["app_code"], white_bg=False)
    assert torch.equal(black["rgb_map"], d["rgb_map_black"])
    # the layout the loader must not fall for: the same planes read as XY, XZ, YZ of a one-level model
    with pytest.raises(ValueError):
        CK.load_checkpoint(path, sampling_opt=0, ndims=3, resMode=[1])


def test_reference_written_merged_stack_file():
    """merge_ckpts output: 5-D planes, lines with a block axis, kwargs["args"] = the run's arguments as a dict,
    kwargs["device"], a gridShape entry; everything the render needs is read from the file."""
    path, d, cfg = _reference_file("hull_softplus_div2x3")
    p = CK.load_checkpoint(path)
    assert p.plane_division == cfg["plane_division"] and p.ndims == 1 and p.resMode == cfg["resMode"]
    assert p.sampling_opt == 1 and p.n_importance == cfg["n_importance"] and p.density_plane[0].dim() == 5
    assert p.alpha_volume is not None
    ref = O.render_chunk(p, d["rays"], return_aux=True)
    assert ref["app_mask"].any()
    assert (ref["rgb_map"] - d["rgb_map"]).abs().max().item() <= 1e-6
    assert (ref["depth_map"] - d["depth_map"]).abs().max().item() <= 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["aabb_relu_L3_P1_production", "hull_softplus_div2x3"])
def test_reference_written_files_render_on_the_gpu(gpu_lib, name):
    from landmark_amd.model import GridNeRFHIP

    path, d, cfg = _reference_file(name)
    extra = {} if cfg["stacked"] else {"sampling_opt": cfg["sampling_opt"], "alpha_mask_filter_thre": cfg["alpha_mask_filter_thre"]}
    m = GridNeRFHIP(CK.load_checkpoint(path, **extra))
    out, _ = m(d["rays"], app_code=cfg["app_code"], N_samples=cfg["N_samples"])
    assert (out["rgb_map"].cpu() - d["rgb_map"]).abs().max().item() <= 1e-4
    assert (out["depth_map"].cpu() - d["depth_map"]).abs().max().item() <= 1e-4
    out, _ = m(d["rays"], app_code=cfg["app_code"], N_samples=cfg["N_samples"], white_bg=False)
    assert (out["rgb_map"].cpu() - d["rgb_map_black"]).abs().max().item() <= 1e-4


@pytest.mark.gpu
def test_model_save_writes_the_mask_it_holds(gpu_lib, tmp_path):
    """GridNeRFHIP.save after updateAlphaMask: the file carries the rebuilt occupancy volume (packed bits, 5-D shape,
    its box) in the reference's layout (gridnerf_sequential.py:209-223), loads with the weights-only loader, and a
    model built from it renders what the saving model renders, bit for bit."""
    from landmark_amd import scenes
    from landmark_amd.model import GridNeRFHIP

    p = scenes.make_params(seed=21, gridSize=(9, 11, 13), near_far=[0.5, 4.5], n_importance=64, sampling_opt=1,
                           density_shift=-6.0, step_ratio=0.5, resMode=(1, 2))
    for t in p.density_plane:
        t.mul_(8.0)
    m = GridNeRFHIP(p)
    assert m.alphaMask is None
    m.updateAlphaMask(gridSize=(14, 12, 10))
    vol = m.alphaMask.alpha_volume
    assert 0 < int(vol.sum()) < vol.numel()
    path = str(tmp_path / "saved.th")
    m.save(path)
    raw = torch.load(path, map_location="cpu", weights_only=False)
    assert tuple(raw["alphaMask.shape"]) == (1, 1, 10, 12, 14) and raw["alphaMask.mask"].dtype == np.uint8
    assert set(raw) == {"kwargs", "state_dict", "alphaMask.shape", "alphaMask.mask", "alphaMask.aabb"}
    q = CK.load_checkpoint(path, sampling_opt=1, n_importance=64)
    assert torch.equal(q.alpha_volume, vol.reshape(10, 12, 14).cpu()) and torch.equal(q.alpha_aabb, m.alphaMask.aabb.cpu())
    rays = scenes.pinhole_rays(40, 40, 40.0, scenes.sphere_pose(2.5, 5))
    a, _ = m(rays)
    b, _ = GridNeRFHIP(q)(rays)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])
    released = GridNeRFHIP(scenes.make_params(seed=21, gridSize=(9, 11, 13)), release_source=True)
    with pytest.raises(Exception, match="released"):
        released.save(path)


@pytest.mark.gpu
def test_fp16_matrix_modes_refuse_tables_beyond_their_range(gpu_lib):
    """f16 / f16x2 carry plane x line products as fp16: tables whose products can pass 65504 are refused for those
    modes at construction (and when the mode is switched), not rendered to inf; bf16 and f32 take them."""
    from landmark_amd import _lib as L
    from landmark_amd import scenes
    from landmark_amd.model import GridNeRFHIP

    p = scenes.make_params(seed=22, gridSize=(9, 11, 13), near_far=[0.5, 4.5], n_importance=64, density_shift=0.0)
    ok = GridNeRFHIP(p, mlp_precision="f16x2")
    assert 0 < ok.fp16_range_bounds()["product"] < 1.0
    p.app_plane[1] = p.app_plane[1] * 3000.0
    p.app_line[1] = p.app_line[1] * 3000.0
    for prec in ("f16", "f16x2"):
        with pytest.raises(L.LandmarkError, match="fp16 range"):
            GridNeRFHIP(p, mlp_precision=prec)
    wide = GridNeRFHIP(p, mlp_precision="bf16")
    rays = scenes.pinhole_rays(24, 24, 24.0, scenes.sphere_pose(2.5, 5))
    assert bool(torch.isfinite(wide(rays)[0]["rgb_map"]).all())
    wide.mlp_precision = "f16"
    with pytest.raises(L.LandmarkError, match="fp16 range"):
        wide(rays)
    assert GridNeRFHIP(p, mlp_precision="f16", check_fp16_range=False) is not None
