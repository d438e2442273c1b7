"""ctypes binding of oracle/scalar_ref.c.  TEST INFRASTRUCTURE ONLY (see that file)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libscalar_ref.so")

MAT_MODE = [[0, 1], [0, 2], [1, 2]]
VEC_MODE = [2, 1, 0]


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "scalar_ref.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "_build/libscalar_ref.so"], stdout=subprocess.DEVNULL)
    return _SO


class Geom(C.Structure):
    _fields_ = [
        ("sampling_opt", C.c_int), ("S", C.c_int), ("aabb", C.c_float * 6), ("near", C.c_float), ("far", C.c_float),
        ("tab_a", C.POINTER(C.c_float)), ("tab_t", C.POINTER(C.c_float)), ("inv_aabb", C.c_float * 3),
        ("vol", C.POINTER(C.c_float)), ("vd", C.c_int), ("vh", C.c_int), ("vw", C.c_int),
        ("vol_aabb_min", C.c_float * 3), ("vol_inv", C.c_float * 3), ("vol_thre", C.c_float),
    ]


class Plane(C.Structure):
    _fields_ = [
        ("plane", C.POINTER(C.c_float)), ("line", C.POINTER(C.c_float)),
        ("C", C.c_int), ("H", C.c_int), ("W", C.c_int), ("Len", C.c_int),
        ("ax0", C.c_int), ("ax1", C.c_int), ("axl", C.c_int),
    ]


class Model(C.Structure):
    _fields_ = [
        ("geom", Geom), ("n_planes", C.c_int), ("density", C.POINTER(Plane)), ("app", C.POINTER(Plane)),
        ("app_dim", C.c_int), ("basis", C.POINTER(C.c_float)),
        ("view_pe", C.c_int), ("fea_pe", C.c_int), ("hidden", C.c_int),
        ("w1", C.POINTER(C.c_float)), ("b1", C.POINTER(C.c_float)), ("w2", C.POINTER(C.c_float)),
        ("b2", C.POINTER(C.c_float)), ("w3", C.POINTER(C.c_float)), ("b3", C.POINTER(C.c_float)),
        ("softplus", C.c_int), ("density_shift", C.c_float), ("distance_scale", C.c_float),
        ("weight_thres", C.c_float), ("white_bg", C.c_int),
        ("basis_den", C.POINTER(C.c_float)), ("latent", C.POINTER(C.c_float)), ("latent_dim", C.c_int),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.lmref_sample_cull.restype = C.c_long
        _lib.lmref_bilinear.restype = C.c_float
        _lib.lmref_linear.restype = C.c_float
        _lib.lmref_alpha_lookup.restype = C.c_float
    return _lib


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def sampler_tables(p, S):
    """The two per-sample tables the samplers need, computed with torch itself so that
    they hold exactly what the reference's tensors hold
    (gridnerf_sequential.py:268-273 and :303-304)."""
    if p.sampling_opt:
        t = torch.linspace(0.0, 1.0, steps=S)
        a = p.near_far[0] * (1.0 - t)
    else:
        t = torch.zeros(S)
        a = p.stepSize.cpu() * torch.arange(S)[None].float()[0]
    return a.contiguous().numpy().copy(), t.contiguous().numpy().copy()


class ScalarModel:
    """Keeps the numpy buffers alive behind a `Model` struct built from a parameter object."""

    def __init__(self, p, N_samples=-1, white_bg=True, app_code=None):
        self.keep = []
        if p.sampling_opt:
            S = p.n_importance
        else:
            S = N_samples if N_samples > 0 else p.nSamples
        self.S = S
        g = Geom()
        g.sampling_opt, g.S = int(bool(p.sampling_opt)), S
        g.aabb[:] = p.aabb.reshape(-1).tolist()
        near32 = torch.tensor(p.near_far[0], dtype=torch.float32).item()
        far32 = torch.tensor(p.near_far[1], dtype=torch.float32).item()
        g.near, g.far = near32, far32
        a, t = sampler_tables(p, S)
        self.keep += [a, t]
        g.tab_a, g.tab_t = _fp(a), _fp(t)
        g.inv_aabb[:] = p.invaabbSize.tolist()
        if p.alpha_volume is not None:
            vol = np.ascontiguousarray(p.alpha_volume.float().numpy())
            self.keep.append(vol)
            g.vol = _fp(vol)
            g.vd, g.vh, g.vw = vol.shape[-3:]
            g.vol_aabb_min[:] = p.alpha_aabb[0].tolist()
            g.vol_inv[:] = (1.0 / (p.alpha_aabb[1] - p.alpha_aabb[0]) * 2).tolist()
            g.vol_thre = torch.tensor(p.alpha_mask_filter_thre, dtype=torch.float32).item()
        self.geom = g
        n = len(p.density_plane)
        L = len(p.resMode)

        def planes(pl, ln):
            arr = (Plane * n)()
            for k in range(n):
                d = k // L
                a_ = np.ascontiguousarray(pl[k][0].float().numpy())
                b_ = np.ascontiguousarray(ln[k][0, :, :, 0].float().numpy())
                self.keep += [a_, b_]
                arr[k].plane, arr[k].line = _fp(a_), _fp(b_)
                arr[k].C, arr[k].H, arr[k].W = a_.shape
                arr[k].Len = b_.shape[1]
                arr[k].ax0, arr[k].ax1 = MAT_MODE[d]
                arr[k].axl = VEC_MODE[d]
            return arr

        m = Model()
        m.geom = g
        m.n_planes = n
        self.dens, self.app = planes(p.density_plane, p.density_line), planes(p.app_plane, p.app_line)
        m.density, m.app = self.dens, self.app
        m.app_dim = p.app_dim

        def f(t_):
            if t_ is None:
                return None
            a_ = np.ascontiguousarray(t_.float().numpy())
            self.keep.append(a_)
            return _fp(a_)

        m.basis = f(p.basis_mat)
        m.view_pe, m.fea_pe, m.hidden = p.view_pe, p.fea_pe, p.featureC
        m.w1, m.b1, m.w2, m.b2, m.w3, m.b3 = (
            f(p.mlp_w[0]), f(p.mlp_b[0]), f(p.mlp_w[1]), f(p.mlp_b[1]), f(p.mlp_w[2]), f(p.mlp_b[2])
        )
        m.softplus = int(p.fea2denseAct == "softplus")
        m.density_shift, m.distance_scale = p.density_shift, p.distance_scale
        m.weight_thres = p.rayMarch_weight_thres
        m.white_bg = int(white_bg)
        if getattr(p, "nonlinear_density", False):
            m.basis_den = f(p.basis_den.reshape(-1))
        if getattr(p, "encode_app", False) and app_code is not None:
            m.latent = f(p.embedding_app[int(app_code)])
            m.latent_dim = p.embedding_app.shape[1]
        self.model = m

    def sample_cull(self, rays):
        r = np.ascontiguousarray(rays.numpy(), dtype=np.float32)
        N = r.shape[0]
        valid = np.zeros(N * self.S, np.uint8)
        z = np.zeros(N * self.S, np.float32)
        cnt = lib().lmref_sample_cull(C.byref(self.geom), _fp(r), C.c_long(N), valid.ctypes.data_as(C.c_void_p), _fp(z))
        return torch.from_numpy(valid.reshape(N, self.S)).bool(), torch.from_numpy(z.reshape(N, self.S)), int(cnt)

    def render(self, rays):
        r = np.ascontiguousarray(rays.numpy(), dtype=np.float32)
        N, S = r.shape[0], self.S
        rgb = np.zeros((N, 3), np.float32)
        depth = np.zeros(N, np.float32)
        valid = np.zeros(N * S, np.uint8)
        sigma = np.zeros(N * S, np.float32)
        weight = np.zeros(N * S, np.float32)
        app = np.zeros(N * S, np.uint8)
        lib().lmref_render(
            C.byref(self.model), _fp(r), C.c_long(N), _fp(rgb), _fp(depth),
            valid.ctypes.data_as(C.c_void_p), _fp(sigma), _fp(weight), app.ctypes.data_as(C.c_void_p),
        )
        t = torch.from_numpy
        return {
            "rgb_map": t(rgb), "depth_map": t(depth), "ray_valid": t(valid.reshape(N, S)).bool(),
            "sigma": t(sigma.reshape(N, S)), "weight": t(weight.reshape(N, S)), "app_mask": t(app.reshape(N, S)).bool(),
        }
