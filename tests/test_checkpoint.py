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
    assert raw["alphaMask.mask"].dtype == np.uint8 and tuple(raw["alphaMask.shape"]) == (5, 7, 6)
    assert "density_plane.5" in raw["state_dict"] and "renderModule.mlp.4.bias" in raw["state_dict"]
    q = CK.load_checkpoint(path, resMode=[1, 2], n_importance=24)
    assert q.ndims == 3 and q.encode_app == bool(extra) and q.nonlinear_density == bool(extra)
    assert torch.equal(q.alpha_volume, p.alpha_volume)
    rays = scenes.pinhole_rays(12, 12, 10.0, scenes.sphere_pose(2.5, 1))
    code = 2 if extra else None
    a = O.render_chunk(p, rays, app_code=code)
    b = O.render_chunk(q, rays, app_code=code)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and torch.equal(a["depth_map"], b["depth_map"])


def test_loader_rejects_inconsistent_or_stacked_layouts():
    ck = CK.checkpoint_from_params(_scene())
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2, 4, 8])  # 6 planes do not split into 4 levels
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2], ndims=2)
    ck["state_dict"]["density_plane.0"] = ck["state_dict"]["density_plane.0"][:, :, None]  # [1,C,B,h,w]
    with pytest.raises(ValueError):
        CK.params_from_checkpoint(ck, resMode=[1, 2])  # stacked planes without a plane division


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
    q = CK.load_checkpoint(path, resMode=[1, 2], n_importance=20)
    assert q.plane_division == [2, 3] and q.ndims == 1
    rays = scenes.pinhole_rays(10, 10, 8.0, scenes.sphere_pose(2.5, 1))
    a, b = O.render_chunk(p, rays), O.render_chunk(q, rays)
    assert torch.equal(a["rgb_map"], b["rgb_map"]) and a["rgb_map"].min() < 0.99
    with pytest.raises(ValueError):
        CK.load_checkpoint(path, resMode=[1, 2], plane_division=[2, 2])  # 4 blocks, the file holds 6
