"""Host-side mirror of the reference's render model on top of the C-ABI library.

`GridNeRFHIP` keeps the call signature and the attributes callers read from the
reference's `GridNeRF` in render mode (app/models/gridnerf_sequential.py:439-447 for
`forward`; `run_nerf`, `alphaMask`, `aabb`, `n_importance`, `near_far`,
`distance_scale`, `rayMarch_weight_thres`, `alpha_mask_filter_thre` as read by
app/tools/render_utils.py:208 and dist_render/kernel/cuda_render_extend.py:43-159).
PyTorch is used for device memory and streams only; every computation of the render
path is a HIP kernel reached through ctypes.  There is no fallback: without the built
library, or without a GPU, construction raises.
"""
from __future__ import annotations

import ctypes as C
from types import SimpleNamespace
from typing import Dict, Optional, Tuple

import numpy as np
import torch

from . import _lib as L
from .params import MAT_MODE, VEC_MODE, GridNeRFParams


def _sampler_tables(p: GridNeRFParams, S: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-sample tables of the two samplers, evaluated with the same PyTorch CPU ops the
    reference uses (gridnerf_sequential.py:268-273 and :303-304) so that they hold the
    same bits: hull -> (near*(1-t), t) with t = linspace(0,1,S); aabb -> (stepSize*arange, 0)."""
    if p.sampling_opt:
        t = torch.linspace(0.0, 1.0, steps=S)
        a = p.near_far[0] * (1.0 - t)
    else:
        t = torch.zeros(S)
        a = (p.stepSize.cpu() * torch.arange(S)[None].float())[0]
    return a.contiguous(), t.contiguous()


class GridNeRFHIP:
    """Render-only GridNeRF on one MI355X."""

    def __init__(
        self,
        params: GridNeRFParams,
        device: str = "cuda",
        mlp_precision: str = "f32",
        term_eps: float = 0.0,
        release_source: bool = False,
        occupancy: str = "auto",  # auto | cells | u8 | f32: storage of the occupancy volume
        coarse_occupancy: bool = True,  # a coarse level over the cell table: empty runs of samples are skipped
        capacity: str = "adaptive",  # adaptive | worst: how the render workspace is sized (see `capacities`)
        check_fp16_range: bool = True,  # refuse f16 / f16x2 for tables whose products can leave the fp16 range
    ):
        if not torch.cuda.is_available():
            raise L.LandmarkError("GridNeRFHIP needs a GPU; there is no CPU path")
        self.lib = L.load()
        self.device = torch.device(device)
        self.p = params
        self.mlp_precision = mlp_precision
        self.term_eps = float(term_eps)
        if capacity not in ("adaptive", "worst"):
            raise ValueError(f"capacity {capacity!r}")
        self.capacity = capacity
        # [valid, appearance] samples per ray the workspace is sized for (chunk average); grows on overflow
        self.samples_per_ray = [32.0, 12.0]
        # set by callers that render images: rays arrive row by row, this many per row (0 = unknown); lets the
        # kernels visit rays in 8 x 8 pixel tiles.  Results do not depend on it.
        self.ray_row_length = 0
        if params.app_dim != 27 or params.view_pe != 2 or params.fea_pe != 2 or params.featureC != 128:
            raise L.LandmarkError("colour network shape must be app_dim 27, view_pe = fea_pe = 2, featureC 128")
        if params.fea2denseAct not in ("softplus", "relu"):
            raise L.LandmarkError(f"fea2denseAct {params.fea2denseAct!r}")
        # --- attributes the reference's callers read
        self.run_nerf = False
        self.aabb = params.aabb.to(self.device)
        self.n_importance = params.n_importance
        self.near_far = list(params.near_far)
        self.distance_scale = params.distance_scale
        self.rayMarch_weight_thres = params.rayMarch_weight_thres
        self._alpha_mask_filter_thre = float(params.alpha_mask_filter_thre)
        self.sampling_opt = params.sampling_opt
        self.ndims, self.resMode = params.ndims, list(params.resMode)
        self.nSamples = params.nSamples
        self.alphaMask_thres = params.alphaMask_thres
        self.gridSize = list(params.gridSize)
        self.stepSize = params.stepSize
        self._occupancy = occupancy
        self._coarse_occupancy = bool(coarse_occupancy)
        self._geom_cache: Dict[int, Tuple[L.LmGeom, tuple]] = {}
        self._struct_cache: Dict[tuple, L.LmModel] = {}
        self._need_cache: Dict[tuple, int] = {}
        self._set_alpha_mask(params.alpha_volume, params.alpha_aabb)
        # --- channel-last tables
        self.plane_division = None if params.plane_division is None else [int(v) for v in params.plane_division]
        self._n_blocks = 0
        if self.plane_division is not None:
            if params.ndims != 1:
                raise L.LandmarkError("a block-stacked model has ndims = 1 (XY planes, z lines)")
            self._n_blocks = self.plane_division[0] * self.plane_division[1]
            if self._n_blocks == 1:
                # the reference's block coordinate 2 b / (B - 1) - 1 is 0 / 0 for one block (gridnerf_parallel.py:333-335)
                raise L.LandmarkError("plane_division [1, 1]: one block is the plain layout; squeeze the block axis "
                                      "(planes [1,C,h,w], lines [1,C,L,1]) and pass plane_division=None")
        self._tables = []  # keep device tensors alive
        self._density = self._relayout_set(params.density_plane, params.density_line)
        self._app = self._relayout_set(params.app_plane, params.app_line)
        self.K_app = sum(pl.C for pl in self._app)
        if release_source:
            params.density_plane, params.density_line, params.app_plane, params.app_line = [], [], [], []
        # --- density projection (nonlinear_density)
        self._den_w = None
        if params.nonlinear_density:
            self._den_w = params.basis_den.detach().to(self.device, torch.float32).reshape(-1).contiguous()
            if self._den_w.numel() != sum(pl.C for pl in self._density):
                raise L.LandmarkError("basis_den width does not match the density planes")
        # --- colour network; with encode_app the 48 latent columns of the first layer fold into its bias
        self.encode_app = bool(params.encode_app)
        self._latent_dim = 0
        if self.encode_app:
            self._latent_dim = params.embedding_app.shape[1]
            self.embedding_app = params.embedding_app.detach().float().cpu()
            w1 = params.mlp_w[0].detach().float().cpu()
            self._w1_latent = w1[:, 27 : 27 + self._latent_dim].contiguous()  # [128, 48]
            self._w1_plain = torch.cat([w1[:, :27], w1[:, 27 + self._latent_dim :]], 1).contiguous()  # [128, 150]
        self._packed = {}
        self._bias_code = {}
        self.check_fp16_range = bool(check_fp16_range)
        self._fp16_bounds = None
        self._pack_mlp(mlp_precision)
        # --- workspace cache (per-S geometry is cached in _geom_cache)
        self._ws = {}  # workspace per slot (one slot per stream that renders concurrently)
        self._side_streams = []
        self._slot_counters = []
        with torch.inference_mode(False):
            self.counters = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device=self.device)  # copied into per call

    @property
    def alpha_mask_filter_thre(self) -> float:
        """Occupancy lookups must exceed this to keep a sample (gridnerf_sequential.py:131, 463)."""
        return self._alpha_mask_filter_thre

    @alpha_mask_filter_thre.setter
    def alpha_mask_filter_thre(self, value) -> None:
        self._alpha_mask_filter_thre = float(value)
        self._invalidate()  # the cached geometry holds the threshold

    def _invalidate(self) -> None:
        """Drop everything derived from the geometry (after the occupancy volume or its threshold changed)."""
        self._geom_cache.clear()
        self._struct_cache.clear()
        self._need_cache.clear()

    # ------------------------------------------------------------------ construction helpers
    def _set_alpha_mask(self, volume, aabb):
        """Install an occupancy volume [D,H,W] (AlphaGridMask, app/models/alpha_mask.py:16-26) or none."""
        self._invalidate()
        self.alphaMask = None
        self._vol, self._vol_store, self._vol_dtype, self._alpha_aabb = None, None, L.LM_F32, None
        self._vol_coarse = None
        if volume is None:
            return
        vol = volume.to(self.device, torch.float32).contiguous()
        self._alpha_aabb = aabb.detach().to(torch.float32).cpu()
        self.alphaMask = SimpleNamespace(alpha_volume=vol.view(1, 1, *vol.shape[-3:]), aabb=aabb.to(self.device))
        self._vol = self._vol_store = self.alphaMask.alpha_volume
        if self._occupancy in ("auto", "cells", "u8"):
            D, H, W = self._vol.shape[-3:]
            cells = torch.empty((D + 1) * (H + 1) * (W + 1), dtype=torch.uint8, device=self.device)
            flag = torch.zeros(1, dtype=torch.int32, device=self.device)
            L.check(self.lib.lm_pack_occupancy(self._vol.data_ptr(), D, H, W, cells.data_ptr(), flag.data_ptr(), L.current_stream()), "lm_pack_occupancy")
            if self._occupancy != "u8" and int(flag.item()) == 0:
                # a 0/1 mask (what the reference stores): one byte per trilinear cell, one load per sample
                self._vol_dtype, self._vol_store = L.LM_CELLS, cells
                if self._coarse_occupancy:
                    coarse = torch.empty(self.lib.lm_occupancy_coarse_bytes(D, H, W), dtype=torch.uint8, device=self.device)
                    L.check(self.lib.lm_pack_occupancy_coarse(cells.data_ptr(), D, H, W, coarse.data_ptr(), L.current_stream()), "lm_pack_occupancy_coarse")
                    self._vol_coarse = coarse
            else:
                as_u8 = self._vol.clamp(0, 255).to(torch.uint8)
                if bool((as_u8.float() == self._vol).all()):
                    self._vol_dtype, self._vol_store = L.LM_U8, as_u8.contiguous()

    def _relayout(self, t: torch.Tensor) -> torch.Tensor:
        """[1,C,H,W] -> device [H,W,C] through lm_relayout_nchw_to_hwc."""
        src = t.to(self.device).contiguous()
        _, Cc, H, W = src.shape
        dst = torch.empty((H, W, Cc), dtype=src.dtype, device=self.device)
        dt = L.LM_F32 if src.dtype == torch.float32 else L.LM_F16
        L.check(self.lib.lm_relayout_nchw_to_hwc(src.data_ptr(), dst.data_ptr(), Cc, H, W, dt, L.current_stream()), "relayout")
        torch.cuda.current_stream().synchronize()  # src may be a temporary
        return dst

    def _relayout_set(self, planes, lines):
        out = []
        L_ = len(self.resMode)
        if len(planes) > L.LM_MAX_PLANES:
            raise L.LandmarkError(f"{len(planes)} planes > LM_MAX_PLANES")
        for k, (pl, ln) in enumerate(zip(planes, lines)):
            if pl.dtype not in (torch.float32, torch.float16):
                raise L.LandmarkError(f"plane dtype {pl.dtype}")
            s = L.LmPlane()
            if self._n_blocks:
                # block-stacked: [1,C,B,h,w] -> [B][h][w][C], [1,C,Len,B] -> [Len][B][C]
                if pl.dim() != 5 or pl.shape[2] != self._n_blocks or ln.shape[-1] != self._n_blocks:
                    raise L.LandmarkError(f"plane {k}: shapes {tuple(pl.shape)}, {tuple(ln.shape)} do not hold {self._n_blocks} blocks")
                _, Cc, B, h, w = pl.shape
                P, Ln = self._relayout(pl.reshape(1, Cc, B * h, w)), self._relayout(ln)
                s.H, s.W, s.C = h, w, Cc
            else:
                if pl.dim() != 4:
                    raise L.LandmarkError(f"plane {k} has shape {tuple(pl.shape)}: block-stacked planes need plane_division")
                P, Ln = self._relayout(pl), self._relayout(ln)
                s.H, s.W, s.C = P.shape
            self._tables += [P, Ln]
            d = k // L_
            s.plane, s.line = P.data_ptr(), Ln.data_ptr()
            s.Len = Ln.shape[0]
            s.ax0, s.ax1 = MAT_MODE[d]
            s.axl = VEC_MODE[d]
            s.dtype = L.LM_F32 if P.dtype == torch.float32 else L.LM_F16
            out.append(s)
        return out

    FP16_MAX = 65504.0

    def fp16_range_bounds(self) -> Dict[str, float]:
        """Upper bounds of the magnitudes the fp16 matrix modes (f16, f16x2) carry as fp16 numbers: the plane x line
        products of the appearance tables (max |plane_k| * max |line_k| over the planes) and the 27 features behind
        basis_mat (row sums of |basis_mat| weighted with the per-plane product bounds).  One pass over the tables,
        cached."""
        if self._fp16_bounds is None:
            per_plane = []
            for k in range(len(self._app)):
                P, Ln = self._tables[2 * (len(self._density) + k)], self._tables[2 * (len(self._density) + k) + 1]
                (p_lo, p_hi), (l_lo, l_hi) = torch.aminmax(P), torch.aminmax(Ln)  # no temporary of the table's size
                per_plane.append(max(-float(p_lo), float(p_hi)) * max(-float(l_lo), float(l_hi)))
            basis = self.p.basis_mat.detach().float().abs().cpu()
            col = torch.cat([torch.full((pl.C,), b) for pl, b in zip(self._app, per_plane)])
            self._fp16_bounds = {"product": max(per_plane), "feature": float((basis * col[None]).sum(1).max())}
        return self._fp16_bounds

    def _check_fp16_range(self, precision: str) -> None:
        """The fp16 matrix modes turn a product beyond 65504 into inf without any status.  Refuse them for tables whose
        plane x line products can get there; warn when only the (looser) bound of the projected features does."""
        if precision not in ("f16", "fp16", "f16x2") or not self.check_fp16_range:
            return
        b = self.fp16_range_bounds()
        if not b["product"] < self.FP16_MAX:
            raise L.LandmarkError(
                f"mlp_precision={precision!r}: plane x line products of the appearance tables can reach {b['product']:.3g}, "
                f"beyond the fp16 range (65504); use mlp_precision='bf16' or 'f32' (or check_fp16_range=False to override)")
        if not b["feature"] < self.FP16_MAX:
            import warnings

            warnings.warn(f"mlp_precision={precision!r}: the bound of the projected appearance features is {b['feature']:.3g}, "
                          "beyond the fp16 range (65504); results turn inf if a feature really gets there", RuntimeWarning)

    def _pack_mlp(self, precision: str):
        if precision in self._packed:
            return self._packed[precision]
        self._check_fp16_range(precision)
        prec = L.MLP_PREC[precision]
        p = self.p
        K = self.K_app
        n = self.lib.lm_mlp_packed_bytes(prec, K)
        if n == 0:
            raise L.LandmarkError(self.lib.lm_last_error().decode())
        host = np.zeros(n, dtype=np.uint8)
        keep = []

        def f(t):
            if t is None:
                return None
            a = np.ascontiguousarray(t.detach().float().cpu().numpy())
            keep.append(a)
            return a.ctypes.data

        w1 = self._w1_plain if self.encode_app else p.mlp_w[0]
        if tuple(w1.shape) != (128, 150):
            raise L.LandmarkError(f"first colour layer has shape {tuple(w1.shape)}, expected (128, 150)")
        L.check(
            self.lib.lm_mlp_pack(
                prec, K, f(p.basis_mat), f(w1), f(p.mlp_b[0]), f(p.mlp_w[1]), f(p.mlp_b[1]),
                f(p.mlp_w[2]), f(p.mlp_b[2]), host.ctypes.data,
            ),
            "lm_mlp_pack",
        )
        with torch.inference_mode(False):
            # updated in place per app_code later on: must not become an inference tensor when the first call
            # comes from inside torch.inference_mode() (as the serving engine's does)
            dev = torch.from_numpy(host).to(self.device)
        self._packed[precision] = (prec, dev)
        return self._packed[precision]

    def _set_app_code(self, precision: str, app_code):
        """Fold embedding_app[app_code] into the packed first-layer bias (512 bytes, stream ordered)."""
        if not self.encode_app:
            if app_code is not None:
                raise NotImplementedError("app_code given but the model has no appearance embedding (encode_app)")
            return
        if app_code is None:
            raise ValueError("this model was trained with encode_app: forward needs app_code")
        code = int(app_code)
        prec, packed = self._pack_mlp(precision)
        if self._bias_code.get(precision) == code:
            return
        b1 = self.p.mlp_b[0]
        b1 = torch.zeros(128) if b1 is None else b1.detach().float().cpu()
        eff = (b1 + self._w1_latent @ self.embedding_app[code]).contiguous().numpy()
        out = np.zeros(128, dtype=np.float32)
        L.check(self.lib.lm_mlp_pack_bias1(eff.ctypes.data, out.ctypes.data), "lm_mlp_pack_bias1")
        off = self.lib.lm_mlp_bias1_offset(prec, self.K_app)
        packed[off : off + 512].copy_(torch.from_numpy(out.view(np.uint8)), non_blocking=False)
        self._bias_code[precision] = code

    def _geom(self, S: int) -> L.LmGeom:
        if S in self._geom_cache:
            return self._geom_cache[S][0]
        p = self.p
        a, t = _sampler_tables(p, S)
        a_d, t_d = a.to(self.device), t.to(self.device)
        g = L.LmGeom()
        g.sampler = L.LM_SAMPLER_HULL if p.sampling_opt else L.LM_SAMPLER_AABB
        g.S = S
        g.aabb[:] = p.aabb.detach().cpu().reshape(-1).tolist()
        g.near_ = torch.tensor(p.near_far[0], dtype=torch.float32).item()
        g.far_ = torch.tensor(p.near_far[1], dtype=torch.float32).item()
        g.tab_a, g.tab_t = a_d.data_ptr(), t_d.data_ptr()
        g.inv_aabb[:] = p.invaabbSize.detach().cpu().tolist()
        if self._vol is not None:
            g.vol = self._vol_store.data_ptr()
            g.vol_dtype = self._vol_dtype
            if self._vol_coarse is not None and self._coarse_can_act(S):
                g.vol_coarse = self._vol_coarse.data_ptr()
            g.vd, g.vh, g.vw = self._vol.shape[-3:]
            ab = self._alpha_aabb
            g.vol_aabb_min[:] = ab[0].tolist()
            g.vol_inv[:] = (1.0 / (ab[1] - ab[0]) * 2).tolist()
            g.vol_thre = torch.tensor(self._alpha_mask_filter_thre, dtype=torch.float32).item()
        if self._n_blocks:
            g.div0, g.div1 = self.plane_division
            # the reference divides float tensors by the Python floats 2/div (gridnerf_parallel.py:304-311)
            g.blk_w = torch.tensor(2 / g.div0, dtype=torch.float32).item()
            g.blk_h = torch.tensor(2 / g.div1, dtype=torch.float32).item()
        self._geom_cache[S] = (g, (a_d, t_d))
        return g

    def _coarse_can_act(self, S: int) -> bool:
        """The coarse occupancy level answers for runs of 16 samples that span at most two blocks of 8 cells per axis:
        it is handed to the kernels when neighbouring samples are at most about a cell apart (the equal-step sampler's
        step, or the hull sampler's longest spacing (far - near) / (S - 1)), and left out where it could only cost."""
        p = self.p
        ab = self._alpha_aabb
        cell = float(((ab[1] - ab[0]) / torch.tensor([float(d - 1) for d in self._vol.shape[-3:]][::-1]).clamp(min=1.0)).min())
        if p.sampling_opt == 0:
            spacing = float(torch.as_tensor(p.stepSize).item())
        else:
            spacing = (float(p.near_far[1]) - float(p.near_far[0])) / max(S - 1, 1)
        return spacing <= 1.25 * cell

    def _model_struct(self, S: int, white_bg: bool, caps: Tuple[int, int] = (0, 0)) -> L.LmModel:
        """The lm_model of a render with S samples per ray and workspace capacities `caps` (valid samples,
        appearance samples; 0 = worst case), built once per distinct setting and reused (a caller that keeps
        small chunks pays for launches only); never carries event handles."""
        key = (int(S), bool(white_bg), self.mlp_precision, float(self.term_eps), int(self.ray_row_length), caps)
        m = self._struct_cache.get(key)
        if m is None:
            if len(self._struct_cache) > 64:
                self._struct_cache.clear()
            m = self._struct_cache[key] = self._build_model_struct(S, white_bg)
            m.cap_valid, m.cap_app = int(caps[0]), int(caps[1])
        return m

    def _build_model_struct(self, S: int, white_bg: bool) -> L.LmModel:
        m = L.LmModel()
        m.geom = self._geom(S)
        m.n_planes = len(self._density)
        for k in range(len(self._density)):
            m.density[k] = self._density[k]
            m.app[k] = self._app[k]
        m.density_basis = None if self._den_w is None else self._den_w.data_ptr()
        m.act = L.LM_ACT_SOFTPLUS if self.p.fea2denseAct == "softplus" else L.LM_ACT_RELU
        m.density_shift = self.p.density_shift
        m.distance_scale = self.p.distance_scale
        m.weight_thres = self.p.rayMarch_weight_thres
        prec, packed = self._pack_mlp(self.mlp_precision)
        m.mlp_prec, m.mlp_packed = prec, packed.data_ptr()
        m.white_bg = int(bool(white_bg))
        m.term_eps = self.term_eps
        m.ray_row = int(self.ray_row_length)
        return m

    def _samples_for(self, N_samples: int) -> int:
        if self.p.sampling_opt:
            return int(self.p.n_importance)
        return int(N_samples) if N_samples > 0 else int(self.nSamples)

    # ------------------------------------------------------------------ workspace
    def capacities(self, n_rays: int, S: int) -> Tuple[int, int]:
        """Room (valid samples, appearance samples) the workspace of an n_rays chunk is given.  With
        `capacity="worst"` both are 0 = the worst case, which cannot overflow (every sample valid, every ray with
        min(S, 1 / weight threshold) appearance samples: 132 bytes per ray and sample).  Otherwise they follow
        `samples_per_ray` = [valid, appearance] samples per ray averaged over a chunk, which starts from a guess
        and is raised whenever a render reports an overflow (`forward` and `render_frame` repeat such a chunk)."""
        if self.capacity == "worst":
            return (0, 0)
        total = int(n_rays) * int(S)
        if total * 132 <= self.small_workspace:
            # a small chunk: the worst case costs little memory, and without the check for an overflow
            # consecutive calls need no host synchronisation between them
            return (0, 0)
        per_ray_app = min(int(S), int(1.001 / self.p.rayMarch_weight_thres) + 2) if self.p.rayMarch_weight_thres > 0 else int(S)
        want_valid = max(1 << 16, int(self.samples_per_ray[0] * n_rays) + 1)
        want_app = max(1 << 14, int(self.samples_per_ray[1] * n_rays) + 1)
        cap_valid = 0 if want_valid >= total else want_valid
        cap_app = 0 if want_app >= int(n_rays) * per_ray_app else want_app
        return (cap_valid, cap_app)

    def _grow_capacity(self, n_rays: int, n_valid: int, n_app: int, valid_overflowed: bool) -> None:
        """Raise samples_per_ray so that a chunk like the one that reported these counts fits, with a quarter to spare.
        After a valid-sample overflow the appearance count is only a lower bound: double it as well."""
        v = 1.25 * n_valid / max(n_rays, 1)
        a = 1.25 * n_app / max(n_rays, 1)
        if valid_overflowed:
            a = max(a, 2.0 * self.samples_per_ray[1])
        self.samples_per_ray = [max(self.samples_per_ray[0], v), max(self.samples_per_ray[1], a)]

    def workspace(self, n_rays: int, S: int, slot: int = 0, caps: Optional[Tuple[int, int]] = None) -> torch.Tensor:
        """Device workspace for chunks of up to n_rays rays; grown on demand and reused
        (the role of allocate_tensors, dist_render/kernel/cuda_render_extend.py:35-159).
        Renders that run concurrently on different streams take different slots."""
        caps = self.capacities(n_rays, S) if caps is None else caps
        key = (int(n_rays), int(S), self.mlp_precision, caps)
        need = self._need_cache.get(key)
        if need is None:
            m = self._model_struct(S, True, caps)
            need = self.lib.lm_render_workspace_bytes(C.byref(m), n_rays)
            if need == 0:
                raise L.LandmarkError(self.lib.lm_last_error().decode())
            if len(self._need_cache) > 256:
                self._need_cache.clear()
            self._need_cache[key] = need
        ws = self._ws.get(slot)
        if ws is None or ws.numel() < need:
            self._ws[slot] = None
            ws = self._ws[slot] = torch.empty(need, dtype=torch.uint8, device=self.device)
        return ws

    # bytes of workspace a render may take when the library picks the chunk size itself
    workspace_budget = 24 << 30
    # chunks whose worst-case workspace stays below this are always given the worst case
    small_workspace = 256 << 20

    def preferred_chunk(self, n_rays: int, N_samples: int = -1, lanes: int = 1) -> int:
        """Rays per lm_render call when the caller leaves the choice to the library: up to 2^20
        (large launches are what keeps the GPU busy: a 1080p frame in 4096-ray chunks takes 14
        times as long as in two chunks), as many as `workspace_budget` and 32-bit sample indices allow.
        `lanes`: streams the chunks will be dealt to; each owns a workspace, so the budget is shared among them."""
        S = self._samples_for(N_samples)
        probe = 1 << 16
        m = self._model_struct(S, True, self.capacities(probe, S))
        per_ray = self.lib.lm_render_workspace_bytes(C.byref(m), probe) / probe
        fit = int(self.workspace_budget / max(int(lanes), 1) / max(per_ray, 1.0))
        cap = min(1 << 20, ((1 << 32) - 1) // S, max(fit, 4096))
        return max(1, min(int(n_rays), cap))

    def slot_counters(self, slot: int) -> torch.Tensor:
        """The counter block lm_render uses for a slot (slot 0: self.counters)."""
        if slot == 0:
            return self.counters
        while len(self._slot_counters) < slot:
            self._slot_counters.append(torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device=self.device))
        return self._slot_counters[slot - 1]

    def side_streams(self, n: int):
        """n extra streams (default priority) for renders that overlap with the current stream's."""
        while len(self._side_streams) < n:
            self._side_streams.append(torch.cuda.Stream(device=self.device))
        return self._side_streams[:n]

    # ------------------------------------------------------------------ reference interface
    def eval(self):
        return self

    def to(self, device):
        return self

    @torch.no_grad()
    def forward(self, rays_chunk, app_code=None, white_bg=True, is_train=False, N_samples=-1, idxs_chunk=None,
                chunk=None, streams=2):
        """GridBaseSequential.forward in render mode -> ({"rgb_map","depth_map"}, {}).  Two arguments the reference
        does not have: `chunk` = rays per lm_render call (default: as many as one launch and the workspace budget
        take) and `streams` = how many streams the chunks of this call are dealt to (see render_chunks; a call that is
        one chunk stays on the current stream)."""
        if is_train:
            raise NotImplementedError("training is outside this render path (is_train must be False)")
        if idxs_chunk is not None:
            raise NotImplementedError("per-ray image indices (idxs_chunk) are a training input")
        self._set_app_code(self.mlp_precision, app_code)
        rays = rays_chunk.to(self.device, torch.float32).contiguous()
        if rays.dim() != 2 or rays.shape[1] != 6:
            raise ValueError(f"rays_chunk must be [N,6], got {tuple(rays.shape)}")
        N = rays.shape[0]
        rgb = torch.empty((N, 3), dtype=torch.float32, device=self.device)
        depth = torch.empty((N,), dtype=torch.float32, device=self.device)
        if N:
            # a call of any size: split where one launch cannot take it
            step = self.preferred_chunk(N, N_samples, lanes=streams) if chunk is None else max(1, int(chunk))
            self.render_chunks(rays, rgb, depth, step, white_bg=white_bg, N_samples=N_samples, streams=streams)
        return {"rgb_map": rgb, "depth_map": depth}, {}

    def render_chunks(self, rays, rgb, depth, step, white_bg=True, N_samples=-1, streams=1) -> int:
        """Render rays[N,6] into rgb[N,3] / depth[N] in chunks of `step` rays, the chunks dealt in turn to `streams`
        streams: the current one and side streams of the same priority, each with a workspace and a counter block
        of its own, so that the compute-bound stages of one chunk run under the memory-bound stages of another (and
        small chunks, which cannot fill the GPU, run side by side).  The current stream continues after all of
        them; chunks whose workspace overflowed are then repeated (finish_chunks).  Returns the number of chunks."""
        N = rays.shape[0]
        S = self._samples_for(N_samples)
        if step * S >= 2**32:
            raise L.LandmarkError(f"{step} rays x {S} samples do not fit 32-bit sample indices; use smaller chunks")
        starts = list(range(0, N, step))
        if not starts:
            return 0
        current = torch.cuda.current_stream(self.device)
        side = self.side_streams(min(int(streams), len(starts)) - 1) if streams > 1 and len(starts) > 1 else []
        counters = torch.zeros((len(starts), L.LM_STAT_WORDS), dtype=torch.int32, device=self.device)  # a block per chunk
        if side:
            ready = torch.cuda.Event()
            ready.record(current)
            for s in side:
                s.wait_event(ready)
        lanes = [current] + side
        done = []
        for i, start in enumerate(starts):
            sl = slice(start, min(start + step, N))
            with torch.cuda.stream(lanes[i % len(lanes)]):
                caps = self.render_into(rays[sl], rgb[sl], depth[sl], white_bg=white_bg, N_samples=N_samples,
                                        slot=i % len(lanes), counters=counters[i])
            done.append((sl, counters[i], caps))
        for s in side:
            current.wait_stream(s)
        self.finish_chunks(done, rays, rgb, depth, white_bg=white_bg, N_samples=N_samples)
        self.counters.copy_(counters[len(starts) - 1])
        return len(starts)

    __call__ = forward

    def finish_chunks(self, chunks, rays, rgb, depth, white_bg=True, N_samples=-1) -> int:
        """Chunks rendered with a workspace below the worst case may have dropped rays: read their counter blocks
        (one small copy, the call's one host synchronisation), raise the capacity to what the counters ask for and
        render the affected chunks again until none overflows.  `chunks`: (slice of the ray array, the counter
        block its render wrote, the capacities render_into returned for it).  Returns the number of repeated
        renders; nothing to do with capacity="worst"."""
        # chunks rendered on a worst-case workspace cannot have overflowed: no need to look (or to synchronise).
        # The capacities are the ones each render was launched with: an earlier chunk of the same call may have
        # raised samples_per_ray since.
        pending = [(sl, c, caps) for sl, c, caps in chunks if caps != (0, 0)]
        if not pending:
            return 0
        repeats = 0
        for _ in range(6):
            host = torch.stack([c for _, c, _ in pending]).cpu().long() & 0xFFFFFFFF
            again = []
            for (sl, cnt, caps), row in zip(pending, host):
                if int(row[L.LM_STAT_OVERFLOW]) == 0:
                    continue
                n = sl.stop - sl.start
                valid_over = caps[0] != 0 and int(row[L.LM_STAT_N_VALID]) > caps[0]
                self._grow_capacity(n, int(row[L.LM_STAT_N_VALID]), int(row[L.LM_STAT_N_APP]), valid_over)
                again.append((sl, cnt))
            if not again:
                return repeats
            pending = []
            for sl, cnt in again:
                caps = self.render_into(rays[sl], rgb[sl], depth[sl], white_bg=white_bg, N_samples=N_samples, counters=cnt)
                pending.append((sl, cnt, caps))
                repeats += 1
        raise L.LandmarkError("workspace capacity still overflows after six repeats")

    def render_into(self, rays, rgb, depth, white_bg=True, N_samples=-1, counters=None, events=None, slot=0):
        """lm_render on device tensors the caller owns.  `counters`: int32[LM_STAT_WORDS] device tensor
        receiving the chunk's sample counts; `events`: 7 recorded torch.cuda.Event objects
        (enable_timing=True) re-recorded around the stages on the current stream.  Calls that may
        run at the same time (different streams) must use different slots: a slot owns a workspace
        and a counter block.  The workspace has the room `capacities` gives it: unless that is the worst
        case, counters[LM_STAT_OVERFLOW] tells whether rays were dropped (see finish_chunks).  Returns the capacities
        (valid samples, appearance samples; (0, 0) = worst case) the render was launched with."""
        N = rays.shape[0]
        if N == 0:
            return (0, 0)
        S = self._samples_for(N_samples)
        caps = self.capacities(N, S)
        ws = self.workspace(N, S, slot, caps)
        m = self._model_struct(S, white_bg, caps)
        if events is not None:
            m = L.LmModel.from_buffer_copy(m)  # the cached struct stays free of event handles
            for i, e in enumerate(events):
                m.events[i] = e.cuda_event
        cnt = self.slot_counters(slot) if counters is None else counters
        L.check(
            self.lib.lm_render(
                C.byref(m), rays.data_ptr(), N, ws.data_ptr(), ws.numel(), rgb.data_ptr(), depth.data_ptr(),
                cnt.data_ptr(), L.current_stream(),
            ),
            "lm_render",
        )
        return caps

    # ------------------------------------------------------------------ occupancy volume from the model
    @torch.no_grad()
    def getDenseAlpha(self, gridSize=None):
        """Alpha of one step at the lattice points of the AABB -> (alpha [gx,gy,gz], dense_xyz [gx,gy,gz,3])
        (gridnerf_sequential.py:321-349)."""
        if self._n_blocks:
            raise NotImplementedError("getDenseAlpha of a block-stacked model (per-block, training only in the reference)")
        gs = [int(v) for v in (self.gridSize if gridSize is None else gridSize)]
        lin = [torch.linspace(0, 1, g).to(self.device) for g in gs]
        samples = torch.stack(torch.meshgrid(*lin, indexing="ij"), -1)
        dense_xyz = self.aabb[0] * (1 - samples) + self.aabb[1] * samples
        alpha = torch.empty(gs, dtype=torch.float32, device=self.device)
        m = self._model_struct(self._samples_for(-1), True)
        length = torch.as_tensor(self.stepSize, dtype=torch.float32).item()
        L.check(
            self.lib.lm_dense_alpha(C.byref(m), lin[0].data_ptr(), lin[1].data_ptr(), lin[2].data_ptr(), gs[0], gs[1], gs[2],
                                    length, alpha.data_ptr(), L.current_stream()),
            "lm_dense_alpha",
        )
        torch.cuda.current_stream().synchronize()  # the tables are temporaries
        return alpha, dense_xyz

    @torch.no_grad()
    def updateAlphaMask(self, gridSize=(200, 200, 200), increase_alpha_thresh=0):
        """Rebuild the occupancy volume from the density field and return the tight AABB of what is occupied
        (gridnerf_sequential.py:351-384)."""
        gs = [int(v) for v in gridSize]
        alpha, _ = self.getDenseAlpha(gs)
        thres = torch.tensor(self.alphaMask_thres * (10**increase_alpha_thresh), dtype=torch.float32).item()
        volume = torch.empty(gs[::-1], dtype=torch.float32, device=self.device)
        box = torch.empty(6, dtype=torch.int32, device=self.device)
        count = torch.empty(1, dtype=torch.int64, device=self.device)
        L.check(
            self.lib.lm_alpha_mask_pool(alpha.data_ptr(), gs[0], gs[1], gs[2], thres, volume.data_ptr(), box.data_ptr(),
                                        count.data_ptr(), L.current_stream()),
            "lm_alpha_mask_pool",
        )
        self._set_alpha_mask(volume, self.aabb)
        b = box.cpu().tolist()
        if int(count.item()) == 0:
            raise L.LandmarkError("updateAlphaMask: no voxel reaches the threshold")
        a0, a1 = self.aabb[0].cpu(), self.aabb[1].cpu()
        lin = [torch.linspace(0, 1, g) for g in gs]
        lo = torch.stack([a0[d] * (1 - lin[d][b[d]]) + a1[d] * lin[d][b[d]] for d in range(3)])
        hi = torch.stack([a0[d] * (1 - lin[d][b[3 + d]]) + a1[d] * lin[d][b[3 + d]] for d in range(3)])
        total = gs[0] * gs[1] * gs[2]
        self.alpha_rest_percent = int(count.item()) / total * 100
        return torch.stack((lo, hi)).to(self.device)

    def save(self, path) -> None:
        """Write the model in the reference's checkpoint format (GridBaseSequential.save,
        gridnerf_sequential.py:209-223): kwargs, state dict and the occupancy volume the model holds NOW, i.e. the
        one updateAlphaMask built if it was called, packed to bits with its box.  Needs the source tensors
        (not available after release_source=True)."""
        import copy

        from .checkpoint import save_checkpoint

        if not self.p.density_plane:
            raise L.LandmarkError("save: the source tables were released (release_source=True)")
        q = copy.copy(self.p)
        if self.alphaMask is None:
            q.alpha_volume, q.alpha_aabb = None, None
        else:
            q.alpha_volume = self.alphaMask.alpha_volume.reshape(self.alphaMask.alpha_volume.shape[-3:]).cpu()
            q.alpha_aabb = self.alphaMask.aabb.detach().float().cpu()
        q.alpha_mask_filter_thre = self._alpha_mask_filter_thre
        save_checkpoint(q, path)

    def last_counts(self) -> Dict[str, int]:
        """Valid / appearance sample counts of the last chunk (synchronises)."""
        c = self.counters.cpu()
        return {"n_valid": int(c[L.LM_STAT_N_VALID]) & 0xFFFFFFFF, "n_app": int(c[L.LM_STAT_N_APP]) & 0xFFFFFFFF,
                "overflow": int(c[L.LM_STAT_OVERFLOW]) & 0xFFFFFFFF}

    # ------------------------------------------------------------------ stage entry points
    @torch.no_grad()
    def sample_cull(self, rays, N_samples=-1, want_z=True):
        """Part 1 alone: valid mask [N,S], ascending valid flat indices, depths."""
        rays = rays.to(self.device, torch.float32).contiguous()
        N, S = rays.shape[0], self._samples_for(N_samples)
        total = N * S
        n_words = (total + 63) // 64
        bitmap = torch.zeros(max(n_words, 1), dtype=torch.int64, device=self.device)
        prefix = torch.zeros(max(n_words, 1), dtype=torch.int32, device=self.device)
        idx = torch.empty(max(total, 1), dtype=torch.int32, device=self.device)
        z = torch.empty((N, S), dtype=torch.float32, device=self.device) if want_z else None
        scratch = torch.empty(max(self.lib.lm_sample_cull_scratch_bytes(N, S), 256), dtype=torch.uint8, device=self.device)
        cnt = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device=self.device)
        g = self._geom(S)
        L.check(
            self.lib.lm_sample_cull(
                C.byref(g), rays.data_ptr(), N, bitmap.data_ptr(), prefix.data_ptr(), idx.data_ptr(), cnt.data_ptr(),
                L.ptr(z), scratch.data_ptr(), L.current_stream(),
            ),
            "lm_sample_cull",
        )
        n_valid = int(cnt[L.LM_STAT_N_VALID].item()) & 0xFFFFFFFF
        bits = (bitmap[:, None] >> torch.arange(64, device=self.device)) & 1
        mask = bits.reshape(-1)[:total].bool().view(N, S)
        return {
            "ray_valid": mask, "valid_idx": idx[:n_valid].long() & 0xFFFFFFFF, "n_valid": n_valid, "z_vals": z,
            "bitmap": bitmap, "word_prefix": prefix, "counters": cnt, "valid_idx_raw": idx, "rays": rays, "S": S,
        }

    def _plane_array(self, planes):
        arr = (L.LmPlane * len(planes))()
        for k, s in enumerate(planes):
            arr[k] = s
        return arr

    @torch.no_grad()
    def compute_densityfeature(self, xyz_sampled):
        """GridNeRF.compute_densityfeature on normalised coordinates [M,3] -> [M]."""
        xyz = xyz_sampled.to(self.device, torch.float32).contiguous()
        M = xyz.shape[0]
        out = torch.empty(M, dtype=torch.float32, device=self.device)
        arr = self._plane_array(self._density)
        L.check(self.lib.lm_gather_density_xyz(arr, len(self._density), L.ptr(self._den_w), xyz.data_ptr(), M, out.data_ptr(), L.current_stream()), "lm_gather_density_xyz")
        return out

    @torch.no_grad()
    def app_products(self, xyz_sampled):
        """plane*line products [M, P*L*C_a] (compute_appfeature before basis_mat)."""
        xyz = xyz_sampled.to(self.device, torch.float32).contiguous()
        M = xyz.shape[0]
        out = torch.empty((M, self.K_app), dtype=torch.float32, device=self.device)
        arr = self._plane_array(self._app)
        L.check(self.lib.lm_gather_app_xyz(arr, len(self._app), xyz.data_ptr(), M, out.data_ptr(), L.current_stream()), "lm_gather_app_xyz")
        return out

    @torch.no_grad()
    def basis(self, products, precision=None):
        prec, packed = self._pack_mlp(precision or self.mlp_precision)
        products = products.to(self.device, torch.float32).contiguous()
        M = products.shape[0]
        out = torch.empty((M, 27), dtype=torch.float32, device=self.device)
        L.check(self.lib.lm_basis(prec, packed.data_ptr(), self.K_app, products.data_ptr(), M, out.data_ptr(), L.current_stream()), "lm_basis")
        return out

    @torch.no_grad()
    def compute_appfeature(self, xyz_sampled, precision=None):
        """GridNeRF.compute_appfeature: basis_mat(products) -> [M,27]."""
        return self.basis(self.app_products(xyz_sampled), precision)

    @torch.no_grad()
    def render_module(self, viewdirs, features, precision=None, app_code=None):
        """MLPRender_Fea.forward(viewdirs, features[, latent of app_code]) -> rgb [M,3]."""
        self._set_app_code(precision or self.mlp_precision, app_code)
        prec, packed = self._pack_mlp(precision or self.mlp_precision)
        feat = features.to(self.device, torch.float32).contiguous()
        view = viewdirs.to(self.device, torch.float32).contiguous()
        M = feat.shape[0]
        out = torch.empty((M, 3), dtype=torch.float32, device=self.device)
        L.check(self.lib.lm_mlp(prec, packed.data_ptr(), self.K_app, feat.data_ptr(), view.data_ptr(), M, out.data_ptr(), L.current_stream()), "lm_mlp")
        return out

    renderModule = render_module

    @torch.no_grad()
    def density_valid(self, cull, white_bg=True):
        """sigma of the valid samples of a `sample_cull` result, in list order."""
        m = self._model_struct(cull["S"], white_bg)
        sigma = torch.zeros(max(cull["n_valid"], 1), dtype=torch.float32, device=self.device)
        L.check(
            self.lib.lm_density_valid(C.byref(m), cull["rays"].data_ptr(), cull["valid_idx_raw"].data_ptr(), cull["counters"].data_ptr(), sigma.data_ptr(), L.current_stream()),
            "lm_density_valid",
        )
        return sigma[: cull["n_valid"]]

    @torch.no_grad()
    def weights(self, cull, sigma, term_eps=None):
        """Part 4 on a `sample_cull` result: dense weights, appearance list and mask, acc, depth."""
        rays, S = cull["rays"], cull["S"]
        N = rays.shape[0]
        dev = self.device
        weight = torch.zeros((N, S), dtype=torch.float32, device=dev)
        w_valid = torch.zeros(max(cull["n_valid"], 1), dtype=torch.float32, device=dev)
        app_first = torch.zeros(N, dtype=torch.int32, device=dev)
        app_cnt = torch.zeros(N, dtype=torch.int32, device=dev)
        app_idx = torch.zeros(max(N * S, 1), dtype=torch.int32, device=dev)
        app_w = torch.zeros(max(N * S, 1), dtype=torch.float32, device=dev)
        acc = torch.zeros(N, dtype=torch.float32, device=dev)
        depth = torch.zeros(N, dtype=torch.float32, device=dev)
        cnt = cull["counters"].clone()
        cnt[L.LM_STAT_N_APP] = 0
        sig = sigma if sigma.numel() else torch.zeros(1, device=dev)
        g = self._geom(S)
        L.check(
            self.lib.lm_weights(
                C.byref(g), rays.data_ptr(), N, cull["bitmap"].data_ptr(), cull["word_prefix"].data_ptr(), sig.data_ptr(),
                self.p.distance_scale, self.p.rayMarch_weight_thres, self.term_eps if term_eps is None else term_eps,
                w_valid.data_ptr(), weight.data_ptr(), app_first.data_ptr(), app_cnt.data_ptr(), app_idx.data_ptr(),
                app_w.data_ptr(), acc.data_ptr(), depth.data_ptr(), cnt.data_ptr(), L.current_stream(),
            ),
            "lm_weights",
        )
        n_app = int(cnt[L.LM_STAT_N_APP].item()) & 0xFFFFFFFF
        idx = app_idx[:n_app].long() & 0xFFFFFFFF
        app_mask = torch.zeros(N * S, dtype=torch.bool, device=dev)
        app_mask[idx] = True
        return {
            "weight": weight, "app_mask": app_mask.view(N, S), "acc_map": acc, "depth_map": depth, "n_app": n_app,
            "app_idx": idx, "app_w": app_w[:n_app], "app_first": app_first.long(), "app_cnt": app_cnt.long(),
            "w_valid": w_valid[: cull["n_valid"]], "counters": cnt, "app_idx_raw": app_idx,
        }

    @torch.no_grad()
    def composite_rgb(self, wres, rgb, white_bg=True):
        """The per-ray colour sum over the appearance list of a `weights` result; rgb is [n_app,3] in list order."""
        N = wres["acc_map"].shape[0]
        rgb = rgb.to(self.device, torch.float32).contiguous()
        first = wres["app_first"].to(torch.int32).contiguous()
        cnt = wres["app_cnt"].to(torch.int32).contiguous()
        out = torch.empty((N, 3), dtype=torch.float32, device=self.device)
        L.check(
            self.lib.lm_composite_rgb(N, first.data_ptr(), cnt.data_ptr(), wres["app_w"].contiguous().data_ptr(), rgb.data_ptr(),
                                      wres["acc_map"].data_ptr(), int(bool(white_bg)), out.data_ptr(), L.current_stream()),
            "lm_composite_rgb",
        )
        return out

    @torch.no_grad()
    def app_features_list(self, cull, wres, precision=None):
        """Fused gather + basis_mat over the appearance list of a `weights` result -> [n_app,27]."""
        old = self.mlp_precision
        self.mlp_precision = precision or old
        try:
            m = self._model_struct(cull["S"], True)
            feat = torch.zeros((max(wres["n_app"], 1), 27), dtype=torch.float32, device=self.device)
            L.check(
                self.lib.lm_app_features(C.byref(m), cull["rays"].data_ptr(), wres["app_idx_raw"].data_ptr(),
                                         wres["counters"].data_ptr(), feat.data_ptr(), L.current_stream()),
                "lm_app_features",
            )
        finally:
            self.mlp_precision = old
        return feat[: wres["n_app"]]


def params_from_reference_model(model) -> GridNeRFParams:
    """The parameter container of an object that carries the reference model's attributes: a loaded `GridNeRF`
    (gridnerf_sequential.py:46-132, 661-747) or the block-stacked `GridNeRFBranchParallel` a "-merged-stack"
    checkpoint loads into (planes [1,C,B,h,w], `model.args.plane_division`, gridnerf_parallel.py:299-335).
    Reads attributes only; the reference is not imported."""
    args = getattr(model, "args", None)

    def arg(name, default=None):
        # values the reference keeps on the model where it has them, else in its run arguments
        # (an ArgsConfig / namespace, or the dict a merged checkpoint stores)
        if hasattr(model, name):
            return getattr(model, name)
        if isinstance(args, dict):
            return args.get(name, default)
        return getattr(args, name, default)

    lin = [model.renderModule.mlp[i] for i in (0, 2, 4)]
    am = getattr(model, "alphaMask", None)
    planes = [t.detach() for t in model.density_plane]
    division = None
    if planes[0].dim() == 5:
        division = arg("plane_division")
        if division is None:
            raise L.LandmarkError("block-stacked planes ([1,C,B,h,w]) but the model's args hold no plane_division")
        division = [int(v) for v in division]
    grid = model.gridSize
    encode_app = bool(arg("encode_app", False))
    nonlinear = bool(arg("nonlinear_density", False))
    res_mode = arg("resMode")
    vol = None
    if am is not None:
        vol = am.alpha_volume.detach()
        vol = vol.reshape(vol.shape[-3:])  # the reference keeps [1,1,D,H,W] (alpha_mask.py:23)
    return GridNeRFParams(
        aabb=torch.as_tensor(model.aabb).detach().float().cpu(),
        gridSize=[int(x) for x in (grid.tolist() if torch.is_tensor(grid) else grid)],
        density_plane=planes,
        density_line=[t.detach() for t in model.density_line],
        app_plane=[t.detach() for t in model.app_plane],
        app_line=[t.detach() for t in model.app_line],
        basis_mat=model.basis_mat.weight.detach(),
        mlp_w=[l.weight.detach() for l in lin],
        mlp_b=[None if l.bias is None else l.bias.detach() for l in lin],
        ndims=int(model.ndims),
        resMode=[1] if res_mode is None else [int(r) for r in res_mode],
        near_far=[float(x) for x in model.near_far],
        density_shift=float(model.density_shift),
        distance_scale=float(model.distance_scale),
        rayMarch_weight_thres=float(model.rayMarch_weight_thres),
        fea2denseAct=model.fea2denseAct,
        step_ratio=float(model.step_ratio),
        sampling_opt=int(arg("sampling_opt", 0)),
        n_importance=int(arg("n_importance", 128)),
        view_pe=int(model.view_pe),
        fea_pe=int(model.fea_pe),
        app_dim=int(model.app_dim),
        featureC=int(model.featureC),
        alpha_volume=vol,
        alpha_aabb=None if am is None else torch.as_tensor(am.aabb).detach().float().cpu(),
        alpha_mask_filter_thre=float(arg("alpha_mask_filter_thre", 0.0)),
        alphaMask_thres=float(arg("alphaMask_thres", 0.001)),
        encode_app=encode_app,
        embedding_app=model.embedding_app.weight.detach() if encode_app else None,
        nonlinear_density=nonlinear,
        basis_den=model.basis_den.weight.detach() if nonlinear else None,
        plane_division=division,
    )


def from_reference_model(model, **kw) -> GridNeRFHIP:
    """Wrap an object with the reference model's attributes (see params_from_reference_model);
    keyword arguments go to GridNeRFHIP (device, mlp_precision, term_eps, ...)."""
    if isinstance(model, GridNeRFHIP):
        return model
    return GridNeRFHIP(params_from_reference_model(model), **kw)
