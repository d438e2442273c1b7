"""The coarse level over the occupancy cell table lets the culling kernels reject runs of samples in empty space without
visiting them.  It must never change a decision: sample masks with and without it are compared bit for bit, and against
the oracle (AlphaGridMask.sample_alpha > 0 inside the box: app/models/alpha_mask.py:35-59,
app/models/gridnerf_sequential.py:528-541), at the step sizes where it acts (half a grid cell per sample, the reference's
default: app/models/gridnerf_sequential.py:244-281) and where it cannot."""
import ctypes as C

import pytest
import torch

from landmark_amd import _lib as L
from landmark_amd import scenes
from oracle import gridnerf_oracle as O

pytestmark = pytest.mark.gpu


def _model(p, **kw):
    from landmark_amd.model import GridNeRFHIP

    return GridNeRFHIP(p, **kw)


def _scene(grid, opt, S, step_ratio, target, seed=4):
    p = scenes.make_params(seed=seed, gridSize=grid, near_far=[0.4, 5.0], n_importance=S, sampling_opt=opt, step_ratio=step_ratio)
    p.alpha_volume = scenes.blob_occupancy((grid[2], grid[1], grid[0]), 5, target, seed=seed)
    p.alpha_aabb = p.aabb + torch.tensor([[0.01, 0.0, -0.02], [0.0, 0.03, 0.0]])
    p.alpha_mask_filter_thre = 0.0
    return p


def _odd_rays():
    """Rays a camera does not produce: axis parallel, starting inside the box, grazing a face, NaN and infinite ones."""
    r = torch.tensor([
        [0.0, 0.0, 3.0, 0.0, 0.0, -1.0], [0.2, -3.0, 0.1, 0.0, 1.0, 0.0], [-3.0, 0.3, 0.2, 1.0, 0.0, 0.0],
        [0.1, 0.1, 0.1, 0.3, 0.4, -0.866], [0.0, 0.0, 0.0, 0.0, 0.0, 1.0], [1.0, 1.0, 3.0, 0.0, 0.0, -1.0],
        [float("nan"), 0.0, 3.0, 0.0, 0.0, -1.0], [0.0, 0.0, 3.0, float("nan"), 0.0, -1.0],
        [0.0, 0.0, 3.0, 0.0, float("inf"), -1.0], [float("inf"), 0.0, 3.0, 0.0, 0.0, -1.0],
        [0.0, 0.0, 3.0, 0.0, 0.0, 0.0], [5.0, 5.0, 5.0, 0.577, 0.577, 0.577],
    ])
    return r


def test_coarse_table_is_the_pooled_cell_table(gpu_lib):
    D, H, W = 37, 50, 66
    vol = scenes.blob_occupancy((D, H, W), 4, 0.08, seed=2).to("cuda").float().contiguous()
    cells = torch.empty((D + 1) * (H + 1) * (W + 1), dtype=torch.uint8, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    lib = L.load()
    L.check(lib.lm_pack_occupancy(vol.data_ptr(), D, H, W, cells.data_ptr(), flag.data_ptr(), None), "pack")
    n = lib.lm_occupancy_coarse_bytes(D, H, W)
    nz, ny, nx = (D + 8) // 8, (H + 8) // 8, (W + 8) // 8
    assert n == 2 * nz * ny * nx
    coarse = torch.full((n,), 7, dtype=torch.uint8, device="cuda")
    L.check(lib.lm_pack_occupancy_coarse(cells.data_ptr(), D, H, W, coarse.data_ptr(), None), "coarse")
    torch.cuda.synchronize()
    c = (cells.view(D + 1, H + 1, W + 1) != 0).float()[None, None]
    blocks = torch.nn.functional.max_pool3d(c, 8, 8, ceil_mode=True)
    assert blocks.shape[-3:] == (nz, ny, nx)
    padded = torch.nn.functional.pad(blocks, (0, 1, 0, 1, 0, 1))
    dil = torch.nn.functional.max_pool3d(padded, 2, 1)
    assert torch.equal(coarse[: n // 2].view(nz, ny, nx).float(), dil[0, 0])
    assert 0.0 < float(dil.mean()) < 1.0, "the table separates empty from occupied space"


@pytest.mark.parametrize("grid,opt,S,step,target", [
    ((72, 80, 96), 0, -1, 0.5, 0.06),    # the reference's default step: quarters of a bitmap word fit two coarse blocks
    ((72, 80, 96), 0, -1, 0.25, 0.06),   # finer: whole words do
    ((72, 80, 96), 0, -1, 3.0, 0.06),    # coarse steps: the coarse level cannot act, the decisions still agree
    ((72, 80, 96), 1, 128, 2.0, 0.06),   # hull sampler, two words per ray
    ((72, 80, 96), 1, 700, 2.0, 0.2),    # hull sampler, fine steps
    ((8, 8, 8), 0, -1, 0.5, 0.3),        # a table of one coarse block per axis and a half
    ((130, 120, 129), 0, -1, 0.5, 0.02),
])
def test_sample_masks_are_the_same_with_and_without_the_coarse_level(gpu_lib, grid, opt, S, step, target):
    p = _scene(grid, opt, 128 if S < 0 else S, step, target)
    if S < 0:
        S = int(p.nSamples)
    rays = torch.cat([scenes.pinhole_rays(48, 48, 40.0, scenes.sphere_pose(2.6, 3)), _odd_rays(),
                      scenes.pinhole_rays(24, 24, 12.0, scenes.look_at_pose((0.2, 0.1, 0.3), (1.0, 0.5, -0.2)))])
    with_c = _model(p).sample_cull(rays, N_samples=S)
    without = _model(p, coarse_occupancy=False).sample_cull(rays, N_samples=S)
    assert torch.equal(with_c["ray_valid"], without["ray_valid"])
    assert torch.equal(with_c["valid_idx"], without["valid_idx"])
    assert with_c["n_valid"] == without["n_valid"]
    ref = O.render_chunk(p, rays, N_samples=S, return_aux=True)
    assert torch.equal(with_c["ray_valid"].cpu(), ref["ray_valid"])
    n = int(ref["ray_valid"].sum())
    assert 0 < n < ref["ray_valid"].numel() // 4
    # the whole-chunk render takes the other culling kernels: same counters, same picture
    m1, m0 = _model(p, mlp_precision="f32"), _model(p, mlp_precision="f32", coarse_occupancy=False)
    a, b = m1(rays, N_samples=S)[0], m0(rays, N_samples=S)[0]
    assert torch.equal(a["rgb_map"].nan_to_num(7.0), b["rgb_map"].nan_to_num(7.0))
    assert torch.equal(a["depth_map"].nan_to_num(7.0), b["depth_map"].nan_to_num(7.0))
