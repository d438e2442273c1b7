"""ctypes binding of liblandmark_hip.so (include/landmark_hip.h).

The library is the product; there is no fallback.  `load()` raises if the shared
object has not been built (python -m landmark_amd.build, or __graft_entry__.build()).
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(HERE, "liblandmark_hip.so")

LM_MAX_PLANES = 12
LM_STATIC_WORKSPACE_BYTES = 80 << 20
LM_N_STAGES = 6
STAGE_NAMES = ["cull", "density_march", "app_list", "app_gather", "colour", "composite"]
LM_ABI_VERSION = 4  # include/landmark_hip.h
LM_STAT_N_VALID, LM_STAT_N_APP, LM_STAT_N_MARCHED, LM_STAT_OVERFLOW, LM_STAT_BINS, LM_STAT_QUEUE, LM_STAT_WORDS = 0, 1, 2, 3, 4, 8, 16
LM_F32, LM_F16, LM_U8, LM_CELLS = 0, 1, 2, 3
LM_SAMPLER_AABB, LM_SAMPLER_HULL = 0, 1
LM_ACT_SOFTPLUS, LM_ACT_RELU = 0, 1
LM_MLP_F32, LM_MLP_F16, LM_MLP_BF16, LM_MLP_F16X2 = 0, 1, 2, 3
MLP_PREC = {"f32": LM_MLP_F32, "fp32": LM_MLP_F32, "f16": LM_MLP_F16, "fp16": LM_MLP_F16, "bf16": LM_MLP_BF16, "f16x2": LM_MLP_F16X2}


class LmPlane(C.Structure):
    _fields_ = [
        ("plane", C.c_void_p), ("line", C.c_void_p),
        ("H", C.c_int32), ("W", C.c_int32), ("Len", C.c_int32), ("C", C.c_int32),
        ("ax0", C.c_int32), ("ax1", C.c_int32), ("axl", C.c_int32), ("dtype", C.c_int32),
    ]


class LmGeom(C.Structure):
    _fields_ = [
        ("sampler", C.c_int32), ("S", C.c_int32), ("aabb", C.c_float * 6), ("near_", C.c_float), ("far_", C.c_float),
        ("tab_a", C.c_void_p), ("tab_t", C.c_void_p), ("inv_aabb", C.c_float * 3),
        ("vol", C.c_void_p), ("vd", C.c_int32), ("vh", C.c_int32), ("vw", C.c_int32), ("vol_dtype", C.c_int32),
        ("vol_aabb_min", C.c_float * 3), ("vol_inv", C.c_float * 3), ("vol_thre", C.c_float),
        ("div0", C.c_int32), ("div1", C.c_int32), ("blk_w", C.c_float), ("blk_h", C.c_float),
        ("vol_coarse", C.c_void_p),
    ]


class LmModel(C.Structure):
    _fields_ = [
        ("geom", LmGeom), ("n_planes", C.c_int32),
        ("density", LmPlane * LM_MAX_PLANES), ("app", LmPlane * LM_MAX_PLANES),
        ("density_basis", C.c_void_p), ("act", C.c_int32), ("density_shift", C.c_float), ("distance_scale", C.c_float), ("weight_thres", C.c_float),
        ("mlp_prec", C.c_int32), ("mlp_packed", C.c_void_p), ("white_bg", C.c_int32), ("term_eps", C.c_float),
        ("ray_row", C.c_int32), ("reserved_", C.c_int32), ("cap_valid", C.c_int64), ("cap_app", C.c_int64),
        ("events", C.c_void_p * (LM_N_STAGES + 1)),
    ]


# name -> (restype, argtypes); every symbol include/landmark_hip.h declares
_P, _I32, _I64, _F, _SZ = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t
SYMBOLS = {
    "lm_abi_version": (C.c_int, []),
    "lm_last_error": (C.c_char_p, []),
    "lm_relayout_nchw_to_hwc": (C.c_int, [_P, _P, _I32, _I32, _I32, _I32, _P]),
    "lm_pack_occupancy": (C.c_int, [_P, _I32, _I32, _I32, _P, _P, _P]),
    "lm_occupancy_coarse_bytes": (_SZ, [_I32, _I32, _I32]),
    "lm_pack_occupancy_coarse": (C.c_int, [_P, _I32, _I32, _I32, _P, _P]),
    "lm_dense_alpha": (C.c_int, [C.POINTER(LmModel), _P, _P, _P, _I32, _I32, _I32, _F, _P, _P]),
    "lm_alpha_mask_pool": (C.c_int, [_P, _I32, _I32, _I32, _F, _P, _P, _P, _P]),
    "lm_sample_cull_scratch_bytes": (_SZ, [_I64, _I32]),
    "lm_sample_cull": (C.c_int, [C.POINTER(LmGeom), _P, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "lm_gather_density_xyz": (C.c_int, [C.POINTER(LmPlane), _I32, _P, _P, _I64, _P, _P]),
    "lm_gather_app_xyz": (C.c_int, [C.POINTER(LmPlane), _I32, _P, _I64, _P, _P]),
    "lm_mlp_packed_bytes": (_SZ, [_I32, _I32]),
    "lm_mlp_pack": (C.c_int, [_I32, _I32, _P, _P, _P, _P, _P, _P, _P, _P]),
    "lm_mlp_bias1_offset": (_SZ, [_I32, _I32]),
    "lm_mlp_pack_bias1": (C.c_int, [_P, _P]),
    "lm_mlp": (C.c_int, [_I32, _P, _I32, _P, _P, _I64, _P, _P]),
    "lm_basis": (C.c_int, [_I32, _P, _I32, _P, _I64, _P, _P]),
    "lm_weights": (C.c_int, [C.POINTER(LmGeom), _P, _I64, _P, _P, _P, _F, _F, _F, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "lm_composite_rgb": (C.c_int, [_I64, _P, _P, _P, _P, _P, _I32, _P, _P]),
    "lm_render_workspace_bytes": (_SZ, [C.POINTER(LmModel), _I64]),
    "lm_app_features": (C.c_int, [C.POINTER(LmModel), _P, _P, _P, _P, _P]),
    "lm_render": (C.c_int, [C.POINTER(LmModel), _P, _I64, _P, _SZ, _P, _P, _P, _P]),
    "lm_render_static": (C.c_int, [C.POINTER(LmModel), _P, _I64, _P, _P, _P, _P]),
    "lm_generate_rays": (C.c_int, [_P, _P, _P, _I32, _I32, _P, _P]),
    "lm_rgba8": (C.c_int, [_P, _I64, _P, _P]),
    "lm_density_valid": (C.c_int, [C.POINTER(LmModel), _P, _P, _P, _P, _P]),
    "lm_app_products": (C.c_int, [C.POINTER(LmModel), _P, _P, _P, _P, _P]),
}


class LandmarkError(RuntimeError):
    pass


_lib = None


def load() -> C.CDLL:
    """Load the C-ABI library; raise loudly when it is missing or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise LandmarkError(
            f"{SO_PATH} is not built: run `python -m landmark_amd.build` (hipcc, gfx950). "
            "There is no CPU or PyTorch fallback for the render path."
        )
    lib = C.CDLL(SO_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the header and the library disagree
        fn.restype, fn.argtypes = res, args
    if lib.lm_abi_version() != LM_ABI_VERSION:
        raise LandmarkError(f"ABI version mismatch: library reports {lib.lm_abi_version()}")
    _lib = lib
    return lib


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = load().lm_last_error().decode(errors="replace")
        raise LandmarkError(f"{what or 'landmark_hip'} failed ({rc}): {msg}")


def ptr(t) -> int:
    """Device (or host) address of a torch tensor, or None."""
    return None if t is None else t.data_ptr()


def current_stream() -> int:
    import torch

    return torch.cuda.current_stream().cuda_stream
