"""The drop-in binding: wrapping the object the reference's callers hold.

`from_reference_model` / `MultiBlockParallelHIP.allocate_tensors` receive the reference's loaded model
(app/tools/render_utils.py:452-463; dist_render/ddp_infer/inferer_impl.py:354-362 passes it to
allocate_tensors).  The tests build a stand-in with the reference's attribute names from golden fixtures
(single models and block-stacked ones) and check the field mapping against the fixture's render: on the CPU
through the oracle, on the GPU through the wrapped model."""
import pytest
import torch

from oracle import gridnerf_oracle as O
from tests.helpers import golden_names, load_golden, reference_model_stub, stacked_names

CASES = [("forward", n) for n in golden_names()] + [("stacked", n) for n in stacked_names()]


@pytest.mark.parametrize("kind,name", CASES)
def test_field_mapping_reproduces_the_fixture(kind, name):
    from landmark_amd.model import params_from_reference_model

    p, d, cfg = load_golden(name, kind)
    stub = reference_model_stub(p, args_as_dict=(kind == "stacked"))
    q = params_from_reference_model(stub)
    assert q.plane_division == p.plane_division and q.ndims == p.ndims and q.resMode == list(p.resMode)
    assert q.sampling_opt == p.sampling_opt and q.alpha_mask_filter_thre == p.alpha_mask_filter_thre
    assert (q.alpha_volume is None) == (p.alpha_volume is None)
    if q.alpha_volume is not None:
        assert q.alpha_volume.dim() == 3
    out = O.render_chunk(q, d["rays"], N_samples=cfg["N_samples"], app_code=cfg.get("app_code"))
    assert torch.equal(out["rgb_map"], O.render_chunk(p, d["rays"], N_samples=cfg["N_samples"], app_code=cfg.get("app_code"))["rgb_map"])
    assert (out["rgb_map"] - d["rgb_map"]).abs().max().item() <= 1e-6
    assert (out["depth_map"] - d["depth_map"]).abs().max().item() <= 1e-6


def test_stacked_model_without_plane_division_is_refused():
    from landmark_amd._lib import LandmarkError
    from landmark_amd.model import params_from_reference_model

    p, _, _ = load_golden(stacked_names()[0], "stacked")
    stub = reference_model_stub(p)
    del stub.args.plane_division
    with pytest.raises(LandmarkError, match="plane_division"):
        params_from_reference_model(stub)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,name", CASES)
def test_wrapped_reference_model_renders_the_fixture(gpu_lib, kind, name):
    from landmark_amd.model import GridNeRFHIP, from_reference_model
    from landmark_amd.render import MultiBlockParallelHIP

    p, d, cfg = load_golden(name, kind)
    stub = reference_model_stub(p, args_as_dict=(kind == "stacked"))
    code = cfg.get("app_code")
    direct, _ = GridNeRFHIP(p)(d["rays"], app_code=code, N_samples=cfg["N_samples"])
    wrapped = from_reference_model(stub, device="cuda")
    out, _ = wrapped(d["rays"], app_code=code, N_samples=cfg["N_samples"])
    assert torch.equal(out["rgb_map"], direct["rgb_map"]) and torch.equal(out["depth_map"], direct["depth_map"])
    assert (out["rgb_map"].cpu() - d["rgb_map"]).abs().max().item() <= 1e-4
    assert (out["depth_map"].cpu() - d["depth_map"]).abs().max().item() <= 1e-4
    # the fused-path convention: allocate_tensors receives the reference's model object and wraps it itself
    if cfg["sampling_opt"] == 1 or cfg["N_samples"] in (-1, None):
        fused = MultiBlockParallelHIP(device="cuda")
        hip = fused.allocate_tensors(stub, d["rays"].shape[0])
        assert isinstance(hip, GridNeRFHIP)
        ret = fused.forward(d["rays"].cuda(), app_code=code, white_bg=True)
        assert set(ret) == {"rgb_map", "depth_map"}
        assert torch.equal(ret["rgb_map"], direct["rgb_map"])
    # the occupancy threshold is a live attribute like the reference's
    if p.alpha_volume is not None:
        wrapped.alpha_mask_filter_thre = 2.0  # nothing passes
        none, _ = wrapped(d["rays"], app_code=code, N_samples=cfg["N_samples"])
        assert bool((none["rgb_map"] == 1.0).all()) and bool((none["depth_map"] == 0.0).all())
