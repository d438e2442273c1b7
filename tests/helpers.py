"""Shared test helpers: golden-fixture loading and small scene builders."""
import glob
import json
import os

import numpy as np
import torch

from landmark_amd.params import GridNeRFParams

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden_names():
    return sorted(os.path.basename(p)[len("forward_") : -len(".npz")] for p in glob.glob(os.path.join(GOLDEN_DIR, "forward_*.npz")))


def alphamask_names():
    return sorted(os.path.basename(p)[len("alphamask_") : -len(".npz")] for p in glob.glob(os.path.join(GOLDEN_DIR, "alphamask_*.npz")))


def stacked_names():
    return sorted(os.path.basename(p)[len("stacked_") : -len(".npz")] for p in glob.glob(os.path.join(GOLDEN_DIR, "stacked_*.npz")))


def load_golden(name, kind="forward"):
    """(params, data dict of tensors, cfg) for one fixture written by golden/make_golden.py."""
    z = np.load(os.path.join(GOLDEN_DIR, f"{kind}_{name}.npz"))
    cfg = json.loads(bytes(z["cfg_json"]).decode())
    data = {k: torch.from_numpy(z[k]) for k in z.files if k != "cfg_json"}
    n = cfg["ndims"] * len(cfg["resMode"])
    sd = {k[3:]: v for k, v in data.items() if k.startswith("sd.")}
    has_bias = "renderModule.mlp.0.bias" in sd
    p = GridNeRFParams(
        aabb=data["aabb"],
        gridSize=cfg["grid"],
        density_plane=[sd[f"density_plane.{k}"] for k in range(n)],
        density_line=[sd[f"density_line.{k}"] for k in range(n)],
        app_plane=[sd[f"app_plane.{k}"] for k in range(n)],
        app_line=[sd[f"app_line.{k}"] for k in range(n)],
        basis_mat=sd["basis_mat.weight"],
        mlp_w=[sd[f"renderModule.mlp.{i}.weight"] for i in (0, 2, 4)],
        mlp_b=[sd[f"renderModule.mlp.{i}.bias"] if has_bias else None for i in (0, 2, 4)],
        ndims=cfg["ndims"],
        resMode=cfg["resMode"],
        near_far=cfg["near_far"],
        density_shift=cfg["density_shift"],
        distance_scale=25.0,
        rayMarch_weight_thres=1e-3,
        fea2denseAct=cfg["fea2denseAct"],
        step_ratio=cfg["step_ratio"],
        sampling_opt=cfg.get("sampling_opt", 1),
        n_importance=cfg.get("n_importance", 16),
        alpha_volume=data.get("alpha_volume"),
        alpha_aabb=data.get("alpha_aabb"),
        alpha_mask_filter_thre=cfg.get("thre", 0.0),
        alphaMask_thres=cfg.get("alphaMask_thres", 0.001),
        encode_app=cfg.get("encode_app", False),
        embedding_app=sd.get("embedding_app.weight"),
        nonlinear_density=cfg.get("nonlinear_density", False),
        basis_den=sd.get("basis_den.weight"),
        plane_division=cfg.get("plane_division"),
    )
    return p, data, cfg


def reference_model_stub(p: GridNeRFParams, args_as_dict=False):
    """An object carrying exactly the attributes a loaded reference model has (GridBaseSequential.__init__ and
    GridNeRF.init_svd_volume, app/models/gridnerf_sequential.py:46-132, 669-683; AlphaGridMask,
    app/models/alpha_mask.py:16-26; MLPRender_Fea.mlp, app/models/mlp_render_fea.py:30-41): module containers
    for the networks, tensors for the tables, the run's arguments under `.args`.  The reference itself is
    not imported."""
    from types import SimpleNamespace

    import torch.nn as nn

    def linear(w, b):
        lin = nn.Linear(w.shape[1], w.shape[0], bias=b is not None)
        with torch.no_grad():
            lin.weight.copy_(w)
            if b is not None:
                lin.bias.copy_(b)
        return lin

    mlp = nn.Sequential(linear(p.mlp_w[0], p.mlp_b[0]), nn.ReLU(inplace=True), linear(p.mlp_w[1], p.mlp_b[1]),
                        nn.ReLU(inplace=True), linear(p.mlp_w[2], p.mlp_b[2]))
    args = dict(
        distributed=False, run_nerf=False, nonlinear_density=p.nonlinear_density, ndims=p.ndims, resMode=list(p.resMode),
        sampling_opt=p.sampling_opt, bias_enable=int(p.mlp_b[0] is not None), encode_app=p.encode_app,
        n_importance=p.n_importance, alpha_mask_filter_thre=p.alpha_mask_filter_thre, ckpt=None, device="cpu",
    )
    if p.plane_division is not None:
        args["plane_division"] = list(p.plane_division)
    m = SimpleNamespace(
        aabb=p.aabb.clone(), gridSize=torch.tensor(p.gridSize), device="cpu",
        density_plane=nn.ParameterList([nn.Parameter(t.clone()) for t in p.density_plane]),
        density_line=nn.ParameterList([nn.Parameter(t.clone()) for t in p.density_line]),
        app_plane=nn.ParameterList([nn.Parameter(t.clone()) for t in p.app_plane]),
        app_line=nn.ParameterList([nn.Parameter(t.clone()) for t in p.app_line]),
        basis_mat=linear(p.basis_mat, None), renderModule=SimpleNamespace(mlp=mlp),
        ndims=p.ndims, resMode=list(p.resMode), near_far=list(p.near_far), density_shift=p.density_shift,
        distance_scale=p.distance_scale, rayMarch_weight_thres=p.rayMarch_weight_thres, fea2denseAct=p.fea2denseAct,
        step_ratio=p.step_ratio, sampling_opt=p.sampling_opt, n_importance=p.n_importance, view_pe=p.view_pe, fea_pe=p.fea_pe,
        pos_pe=6, app_dim=p.app_dim, featureC=p.featureC, alpha_mask_filter_thre=p.alpha_mask_filter_thre,
        alphaMask_thres=p.alphaMask_thres, nonlinear_density=p.nonlinear_density, run_nerf=False, alphaMask=None,
        args=args if args_as_dict else SimpleNamespace(**args),
    )
    if p.alpha_volume is not None:
        m.alphaMask = SimpleNamespace(alpha_volume=p.alpha_volume.clone().view(1, 1, *p.alpha_volume.shape[-3:]),
                                      aabb=p.alpha_aabb.clone(), device="cpu")
    if p.nonlinear_density:
        m.basis_den = linear(p.basis_den, None)
    if p.encode_app:
        m.embedding_app = nn.Embedding(p.embedding_app.shape[0], p.embedding_app.shape[1])
        with torch.no_grad():
            m.embedding_app.weight.copy_(p.embedding_app)
    return m
