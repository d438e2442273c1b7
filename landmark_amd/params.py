"""Plain parameter container for one GridNeRF render model.

Field names and defaults follow the reference model's constructor and config
(app/models/gridnerf_sequential.py:46-132, app/tools/config_parser.py:24-80):
the tensors are the ones the reference keeps in its state dict
(`density_plane.{k}`, `density_line.{k}`, `app_plane.{k}`, `app_line.{k}`,
`basis_mat.weight`, `renderModule.mlp.{0,2,4}.{weight,bias}`) in the reference's
NCHW layout; the HIP model re-lays them out when it is built from this object.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch

MAT_MODE = [[0, 1], [0, 2], [1, 2]]  # gridnerf_sequential.py:106
VEC_MODE = [2, 1, 0]  # gridnerf_sequential.py:107


@dataclass
class GridNeRFParams:
    aabb: torch.Tensor  # [2,3] fp32
    gridSize: List[int]  # [3] base resolution (x, y, z)
    density_plane: List[torch.Tensor]  # P*L x [1,C_d,H,W]
    density_line: List[torch.Tensor]  # P*L x [1,C_d,Len,1]
    app_plane: List[torch.Tensor]  # P*L x [1,C_a,H,W]
    app_line: List[torch.Tensor]  # P*L x [1,C_a,Len,1]
    basis_mat: torch.Tensor  # [app_dim, P*L*C_a]  (Linear weight, no bias)
    mlp_w: List[torch.Tensor]  # 3 x Linear weight [out,in]
    mlp_b: List[Optional[torch.Tensor]]  # 3 x bias or None (bias_enable)
    ndims: int = 3
    resMode: List[int] = field(default_factory=lambda: [1])
    near_far: List[float] = field(default_factory=lambda: [2.0, 6.0])
    density_shift: float = -10.0
    distance_scale: float = 25.0
    rayMarch_weight_thres: float = 1e-3
    fea2denseAct: str = "softplus"
    step_ratio: float = 2.0
    sampling_opt: int = 1
    n_importance: int = 128
    view_pe: int = 2
    fea_pe: int = 2
    app_dim: int = 27
    featureC: int = 128
    # occupancy volume ("alpha mask"), app/models/alpha_mask.py
    alpha_volume: Optional[torch.Tensor] = None  # [D,H,W] float {0,1}
    alpha_aabb: Optional[torch.Tensor] = None  # [2,3]
    alpha_mask_filter_thre: float = 0.0
    alphaMask_thres: float = 0.001  # threshold updateAlphaMask applies (gridnerf_sequential.py:57, 366-367)
    # per-image appearance embedding (args.encode_app, gridnerf_sequential.py:681-682): the
    # first Linear then takes 27 + 48 + 3 + 108 + 12 = 198 inputs (mlp_render_fea.py:23-24)
    encode_app: bool = False
    embedding_app: Optional[torch.Tensor] = None  # [n_images, 48]
    # density through a learned projection (args.nonlinear_density, gridnerf_sequential.py:679-680, 819-822)
    nonlinear_density: bool = False
    basis_den: Optional[torch.Tensor] = None  # [1, P*L*C_d]
    # block-stacked model ("-merged-stack" checkpoint, gridnerf_branch_parallel.py:465-527): planes are
    # [1,C,B,h,w], lines [1,C,L,B], B = plane_division[0] * plane_division[1] blocks of the XY extent
    plane_division: Optional[List[int]] = None

    # ---- derived quantities, gridnerf_sequential.py:149-164 -------------------------
    @property
    def aabbSize(self) -> torch.Tensor:
        return self.aabb[1] - self.aabb[0]

    @property
    def invaabbSize(self) -> torch.Tensor:
        return 2.0 / self.aabbSize

    @property
    def stepSize(self) -> torch.Tensor:
        gs = torch.tensor(self.gridSize, device=self.aabb.device)
        units = self.aabbSize / (gs - 1)
        return torch.mean(units) * self.step_ratio

    @property
    def nSamples(self) -> int:
        diag = torch.sqrt(torch.sum(torch.square(self.aabbSize)))
        return int((diag / self.stepSize).item()) + 1

    @property
    def n_levels(self) -> int:
        return len(self.resMode)

    def to(self, device) -> "GridNeRFParams":
        def mv(t):
            return None if t is None else t.to(device)

        return GridNeRFParams(
            aabb=mv(self.aabb),
            gridSize=list(self.gridSize),
            density_plane=[mv(t) for t in self.density_plane],
            density_line=[mv(t) for t in self.density_line],
            app_plane=[mv(t) for t in self.app_plane],
            app_line=[mv(t) for t in self.app_line],
            basis_mat=mv(self.basis_mat),
            mlp_w=[mv(t) for t in self.mlp_w],
            mlp_b=[mv(t) for t in self.mlp_b],
            ndims=self.ndims,
            resMode=list(self.resMode),
            near_far=list(self.near_far),
            density_shift=self.density_shift,
            distance_scale=self.distance_scale,
            rayMarch_weight_thres=self.rayMarch_weight_thres,
            fea2denseAct=self.fea2denseAct,
            step_ratio=self.step_ratio,
            sampling_opt=self.sampling_opt,
            n_importance=self.n_importance,
            view_pe=self.view_pe,
            fea_pe=self.fea_pe,
            app_dim=self.app_dim,
            featureC=self.featureC,
            alpha_volume=mv(self.alpha_volume),
            alpha_aabb=mv(self.alpha_aabb),
            alpha_mask_filter_thre=self.alpha_mask_filter_thre,
            alphaMask_thres=self.alphaMask_thres,
            encode_app=self.encode_app,
            embedding_app=mv(self.embedding_app),
            nonlinear_density=self.nonlinear_density,
            basis_den=mv(self.basis_den),
            plane_division=None if self.plane_division is None else list(self.plane_division),
        )
