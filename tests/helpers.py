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
