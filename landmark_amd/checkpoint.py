"""Read and write the reference's single-model checkpoint format.

Format (GridBaseSequential.save / load, app/models/gridnerf_sequential.py:209-242):
    {"kwargs": get_kwargs() (:171-189), "state_dict": model.state_dict(),
     "alphaMask.shape": tuple, "alphaMask.mask": np.packbits(bool volume), "alphaMask.aabb": tensor}
State-dict names: density_plane.{k}, density_line.{k}, app_plane.{k}, app_line.{k} with
k = dim * len(resMode) + level; basis_mat.weight; renderModule.mlp.{0,2,4}.{weight,bias};
optional basis_den.weight (nonlinear_density) and embedding_app.weight (encode_app).
The split of the plane count into ndims x levels is read from the file (kwargs["density_n_comp"] has
ndims entries; plane sizes give the levels); the sampler choice, n_importance and
alpha_mask_filter_thre are run configuration: a merged checkpoint stores it in kwargs["args"], for a
single-model file the caller passes it.
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


def _saved_args(kw) -> dict:
    """The run arguments a merged checkpoint stores (`kwargs["args"] = vars(args)`,
    gridnerf_branch_parallel.py:520-521), else nothing."""
    saved = kw.get("args")
    if isinstance(saved, dict):
        return saved
    return dict(vars(saved)) if hasattr(saved, "__dict__") else {}


def params_from_checkpoint(
    ckpt: dict,
    resMode: Optional[Sequence[int]] = None,
    ndims: Optional[int] = None,
    sampling_opt: Optional[int] = None,
    n_importance: Optional[int] = None,
    alpha_mask_filter_thre: Optional[float] = None,
    near_far: Optional[Sequence[float]] = None,
    plane_division: Optional[Sequence[int]] = None,
) -> GridNeRFParams:
    """Arguments left at None are taken from the file where it holds them: `ndims` is the length of
    kwargs["density_n_comp"] (the reference slices that list to ndims, gridnerf_sequential.py:88), the
    number of levels follows from the plane count, and a merged checkpoint carries the whole run
    configuration in kwargs["args"].  What a single-model file does not record (`sampling_opt`, default
    off in the reference's configuration but on in a few of its confs) must be given."""
    kw, sd = ckpt["kwargs"], ckpt["state_dict"]
    sd = {k.replace(".module", "").replace(".params", ""): v for k, v in sd.items()}  # DDP / wrapper prefixes
    saved = _saved_args(kw)
    n = len([k for k in sd if k.startswith("density_plane.")])
    if n == 0:
        raise ValueError("checkpoint holds no density_plane.* tensors")
    if ndims is None:
        ndims = saved.get("ndims")
    if ndims is None and "density_n_comp" in kw:
        ndims = len(kw["density_n_comp"])
    if resMode is None:
        resMode = saved.get("resMode")
    if ndims is None:
        if resMode is None:
            raise ValueError("neither ndims nor resMode is given and the checkpoint records neither")
        ndims = n // len(resMode)
    ndims = int(ndims)
    if "density_n_comp" in kw and len(kw["density_n_comp"]) != ndims:
        raise ValueError(f"ndims = {ndims}, but the checkpoint was saved by a model with ndims = {len(kw['density_n_comp'])} "
                         "(its density_n_comp list)")
    if ndims < 1 or n % ndims:
        raise ValueError(f"{n} planes cannot belong to ndims = {ndims}")
    levels = n // ndims
    stacked = sd["density_plane.0"].dim() == 5  # "-merged-stack" layout, gridnerf_branch_parallel.py:465-527
    if resMode is None:
        # level j of a dimension is the base grid times resMode[j] (gridnerf_sequential.py:700-716)
        w0 = sd["density_plane.0"].shape[-1]
        resMode = [max(1, round(sd[f"density_plane.{j}"].shape[-1] / w0)) for j in range(levels)]
    resMode = [int(r) for r in resMode]
    if len(resMode) != levels:
        raise ValueError(f"ndims {ndims} x levels {len(resMode)} != {n} planes in the checkpoint")
    # plane k = dimension k // levels at level k % levels: its size must be the level's multiple of the first
    for d in range(ndims):
        base = sd[f"density_plane.{d * levels}"].shape[-2:]
        for j in range(levels):
            for name in ("density_plane", "app_plane"):
                got = tuple(sd[f"{name}.{d * levels + j}"].shape[-2:])
                want = tuple(int(round(b * resMode[j] / resMode[0])) for b in base)
                if any(abs(g - w) > 1 for g, w in zip(got, want)):
                    raise ValueError(f"{name}.{d * levels + j} is {got[1]}x{got[0]}, expected {want[1]}x{want[0]} for ndims "
                                     f"{ndims}, resMode {resMode}: wrong ndims / resMode for this checkpoint?")
    if sampling_opt is None:
        sampling_opt = saved.get("sampling_opt")
    if sampling_opt is None:
        raise ValueError("sampling_opt is not recorded in this checkpoint: pass sampling_opt=0 (sample_ray, the reference's "
                         "default) or 1 (sample_ray_within_hull) as the run configuration sets it")
    if n_importance is None:
        n_importance = saved.get("n_importance", 128)  # config_parser.py:38-43
    if alpha_mask_filter_thre is None:
        alpha_mask_filter_thre = saved.get("alpha_mask_filter_thre", 0.0)  # config_parser.py:263-265
    if stacked:
        if plane_division is None:
            plane_division = saved.get("plane_division")
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
        shape = tuple(int(x) for x in ckpt["alphaMask.shape"])  # [1,1,D,H,W] in the reference's files
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
        sampling_opt=int(sampling_opt),
        n_importance=int(n_importance),
        view_pe=int(kw["view_pe"]),
        fea_pe=int(kw["fea_pe"]),
        app_dim=int(kw["app_dim"]),
        featureC=int(kw["featureC"]),
        alpha_volume=vol,
        alpha_aabb=aabb_m,
        alpha_mask_filter_thre=float(alpha_mask_filter_thre),
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
        # merge_ckpts stores the run's arguments as a dict (gridnerf_branch_parallel.py:520-521)
        kwargs["args"] = {
            "plane_division": list(p.plane_division), "ndims": p.ndims, "resMode": list(p.resMode),
            "sampling_opt": p.sampling_opt, "n_importance": p.n_importance,
            "alpha_mask_filter_thre": p.alpha_mask_filter_thre, "encode_app": p.encode_app,
            "nonlinear_density": p.nonlinear_density, "bias_enable": int(p.mlp_b[0] is not None),
        }
        kwargs["device"] = "cpu"
    ckpt = {"kwargs": kwargs, "state_dict": sd}
    if p.alpha_volume is not None:
        vol = p.alpha_volume.bool().cpu().numpy()
        vol = vol.reshape((1, 1) + vol.shape[-3:])  # AlphaGridMask keeps [1,1,D,H,W] (alpha_mask.py:23)
        ckpt["alphaMask.shape"] = vol.shape
        ckpt["alphaMask.mask"] = np.packbits(vol.reshape(-1))
        ckpt["alphaMask.aabb"] = p.alpha_aabb.cpu()
    return ckpt


def save_checkpoint(p: GridNeRFParams, path: str) -> None:
    torch.save(checkpoint_from_params(p), path)


def _numpy_globals():
    """What a pickled numpy array names (the packed occupancy bits): `_reconstruct`, `ndarray`, `dtype` and the
    dtype's class.  A file written under numpy 1.x spells the module `numpy.core.multiarray`, one written under
    numpy 2.x `numpy._core.multiarray`; both are allowed under both names."""
    import importlib

    rec = None
    for mod in ("numpy._core.multiarray", "numpy.core.multiarray"):
        try:
            rec = importlib.import_module(mod)._reconstruct
            break
        except Exception:  # noqa: BLE001 - the spelling this numpy does not have
            continue
    safe = [np.ndarray, np.dtype, type(np.dtype(np.uint8))]
    if rec is not None:
        safe += [rec, (rec, "numpy.core.multiarray._reconstruct"), (rec, "numpy._core.multiarray._reconstruct")]
    return safe


def load_checkpoint(path: str, trusted: bool = False, **config) -> GridNeRFParams:
    """Load a checkpoint file.  By default only tensors, plain containers and numpy arrays are
    unpickled (`weights_only=True`); `trusted=True` falls back to full unpickling for files
    whose origin the caller vouches for."""
    if trusted:
        ckpt = torch.load(path, map_location="cpu", weights_only=False)
    else:
        with torch.serialization.safe_globals(_numpy_globals()):
            ckpt = torch.load(path, map_location="cpu", weights_only=True)
    return params_from_checkpoint(ckpt, **config)
