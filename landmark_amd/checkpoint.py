"""Read and write the reference's single-model checkpoint format.

Format (GridBaseSequential.save / load, app/models/gridnerf_sequential.py:209-242):
    {"kwargs": get_kwargs() (:171-189), "state_dict": model.state_dict(),
     "alphaMask.shape": tuple, "alphaMask.mask": np.packbits(bool volume), "alphaMask.aabb": tensor}
State-dict names: density_plane.{k}, density_line.{k}, app_plane.{k}, app_line.{k} with
k = dim * len(resMode) + level; basis_mat.weight; renderModule.mlp.{0,2,4}.{weight,bias};
optional basis_den.weight (nonlinear_density) and embedding_app.weight (encode_app).
What is not stored in the file (ndims / resMode split of the plane count, sampler choice,
n_importance, alpha_mask_filter_thre) comes from the run configuration and is passed in.
The block-stacked "-merged-stack" layout of the branch-parallel trainer
(app/models/gridnerf_branch_parallel.py:465-527: planes [1,C,B,h,w], lines [1,C,L,B], B =
plane_division[0] * plane_division[1], kwargs["args"] = the run's arguments as a dict) is read
too; plane_division comes from that dict or from the caller.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch

from .params import GridNeRFParams


def params_from_checkpoint(
    ckpt: dict,
    resMode: Optional[Sequence[int]] = None,
    ndims: Optional[int] = None,
    sampling_opt: int = 1,
    n_importance: int = 128,
    alpha_mask_filter_thre: float = 0.0,
    near_far: Optional[Sequence[float]] = None,
    plane_division: Optional[Sequence[int]] = None,
) -> GridNeRFParams:
    kw, sd = ckpt["kwargs"], ckpt["state_dict"]
    sd = {k.replace(".module", "").replace(".params", ""): v for k, v in sd.items()}  # DDP / wrapper prefixes
    n = len([k for k in sd if k.startswith("density_plane.")])
    if n == 0:
        raise ValueError("checkpoint holds no density_plane.* tensors (a stacked multi-block checkpoint?)")
    resMode = list(resMode) if resMode is not None else [1]
    if ndims is None:
        if n % len(resMode):
            raise ValueError(f"{n} planes cannot be split into levels {resMode}")
        ndims = n // len(resMode)
    if ndims * len(resMode) != n:
        raise ValueError(f"ndims {ndims} x levels {len(resMode)} != {n} planes in the checkpoint")
    stacked = sd["density_plane.0"].dim() == 5  # "-merged-stack" layout, gridnerf_branch_parallel.py:465-527
    if stacked:
        if plane_division is None:
            saved = kw.get("args")
            plane_division = saved.get("plane_division") if isinstance(saved, dict) else None
        if plane_division is None:
            raise ValueError("block-stacked planes ([1,C,B,h,w]): plane_division is needed")
        B = int(plane_division[0]) * int(plane_division[1])
        for k in range(n):
            if sd[f"density_plane.{k}"].dim() != 5 or sd[f"density_plane.{k}"].shape[2] != B or sd[f"density_line.{k}"].shape[-1] != B:
                raise ValueError(f"plane {k} does not hold {B} blocks")
    else:
        plane_division = None
    has_bias = "renderModule.mlp.0.bias" in sd
    vol = aabb_m = None
    if "alphaMask.aabb" in ckpt:
        shape = tuple(int(x) for x in ckpt["alphaMask.shape"])
        bits = np.unpackbits(np.asarray(ckpt["alphaMask.mask"]))[: int(np.prod(shape))].reshape(shape)
        vol = torch.from_numpy(bits).float().reshape(shape[-3:])
        aabb_m = torch.as_tensor(ckpt["alphaMask.aabb"]).float().cpu()
    return GridNeRFParams(
        aabb=torch.as_tensor(kw["aabb"]).float().cpu(),
        gridSize=[int(x) for x in kw["gridSize"]],
        density_plane=[sd[f"density_plane.{k}"] for k in range(n)],
        density_line=[sd[f"density_line.{k}"] for k in range(n)],
        app_plane=[sd[f"app_plane.{k}"] for k in range(n)],
        app_line=[sd[f"app_line.{k}"] for k in range(n)],
        basis_mat=sd["basis_mat.weight"],
        mlp_w=[sd[f"renderModule.mlp.{i}.weight"] for i in (0, 2, 4)],
        mlp_b=[sd[f"renderModule.mlp.{i}.bias"] if has_bias else None for i in (0, 2, 4)],
        ndims=ndims,
        resMode=resMode,
        near_far=[float(x) for x in (near_far if near_far is not None else kw["near_far"])],
        density_shift=float(kw["density_shift"]),
        distance_scale=float(kw["distance_scale"]),
        rayMarch_weight_thres=float(kw["rayMarch_weight_thres"]),
        fea2denseAct=kw["fea2denseAct"],
        step_ratio=float(kw["step_ratio"]),
        sampling_opt=sampling_opt,
        n_importance=n_importance,
        view_pe=int(kw["view_pe"]),
        fea_pe=int(kw["fea_pe"]),
        app_dim=int(kw["app_dim"]),
        featureC=int(kw["featureC"]),
        alpha_volume=vol,
        alpha_aabb=aabb_m,
        alpha_mask_filter_thre=alpha_mask_filter_thre,
        alphaMask_thres=float(kw.get("alphaMask_thres", 0.001)),
        encode_app="embedding_app.weight" in sd,
        embedding_app=sd.get("embedding_app.weight"),
        nonlinear_density="basis_den.weight" in sd,
        basis_den=sd.get("basis_den.weight"),
        plane_division=None if plane_division is None else [int(v) for v in plane_division],
    )


def checkpoint_from_params(p: GridNeRFParams) -> dict:
    """The dictionary GridBaseSequential.save would write for this model."""
    sd = {}
    for k in range(len(p.density_plane)):
        sd[f"density_plane.{k}"] = p.density_plane[k].cpu()
        sd[f"density_line.{k}"] = p.density_line[k].cpu()
    for k in range(len(p.app_plane)):
        sd[f"app_plane.{k}"] = p.app_plane[k].cpu()
        sd[f"app_line.{k}"] = p.app_line[k].cpu()
    sd["basis_mat.weight"] = p.basis_mat.cpu()
    if p.nonlinear_density:
        sd["basis_den.weight"] = p.basis_den.cpu()
    if p.encode_app:
        sd["embedding_app.weight"] = p.embedding_app.cpu()
    for i, j in enumerate((0, 2, 4)):
        sd[f"renderModule.mlp.{j}.weight"] = p.mlp_w[i].cpu()
        if p.mlp_b[i] is not None:
            sd[f"renderModule.mlp.{j}.bias"] = p.mlp_b[i].cpu()
    n_ch = lambda planes: [int(planes[d * len(p.resMode)].shape[1]) for d in range(p.ndims)]
    kwargs = {
        "aabb": p.aabb.cpu(), "gridSize": list(p.gridSize), "density_n_comp": n_ch(p.density_plane),
        "appearance_n_comp": n_ch(p.app_plane), "app_dim": p.app_dim, "density_shift": p.density_shift,
        "alphaMask_thres": p.alphaMask_thres, "distance_scale": p.distance_scale, "rayMarch_weight_thres": p.rayMarch_weight_thres,
        "fea2denseAct": p.fea2denseAct, "near_far": list(p.near_far), "step_ratio": p.step_ratio, "pos_pe": 6,
        "view_pe": p.view_pe, "fea_pe": p.fea_pe, "featureC": p.featureC,
    }
    if p.plane_division is not None:
        kwargs["args"] = {"plane_division": list(p.plane_division)}
    ckpt = {"kwargs": kwargs, "state_dict": sd}
    if p.alpha_volume is not None:
        vol = p.alpha_volume.bool().cpu().numpy()
        ckpt["alphaMask.shape"] = vol.shape
        ckpt["alphaMask.mask"] = np.packbits(vol.reshape(-1))
        ckpt["alphaMask.aabb"] = p.alpha_aabb.cpu()
    return ckpt


def save_checkpoint(p: GridNeRFParams, path: str) -> None:
    torch.save(checkpoint_from_params(p), path)


def load_checkpoint(path: str, trusted: bool = False, **config) -> GridNeRFParams:
    """Load a checkpoint file.  By default only tensors, plain containers and numpy arrays are
    unpickled (`weights_only=True`); `trusted=True` falls back to full unpickling for files
    whose origin the caller vouches for."""
    if trusted:
        ckpt = torch.load(path, map_location="cpu", weights_only=False)
    else:
        import numpy.core.multiarray as ncm

        safe = [ncm._reconstruct, np.ndarray, np.dtype, type(np.dtype(np.uint8))]
        with torch.serialization.safe_globals(safe):
            ckpt = torch.load(path, map_location="cpu", weights_only=True)
    return params_from_checkpoint(ckpt, **config)
