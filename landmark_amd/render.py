"""Chunk drivers with the reference's call signatures.

`renderer_fn` mirrors app/tools/render_utils.py:15-63 (also the shape of
AbstractDDPInfererImpl.renderer_fn, dist_render/ddp_infer/inferer_impl.py:95-120):
split the rays into chunks, call the model on each, concatenate per key.
`MultiBlockParallelHIP` mirrors the two-call convention of the reference's fused path
(dist_render/kernel/cuda_render_extend.py:35, 350): `allocate_tensors(model, N_rays)`
once, then `forward(rays_chunk, app_code=None, white_bg=True) -> dict`.
"""
from __future__ import annotations

import torch


def renderer_fn(rays, gridnerf, chunk=4096, N_samples=-1, white_bg=True, is_train=False, device="cuda", idxs=None,
                app_code=None):
    """Returns ({"rgb_map": [N,3], "depth_map": [N]}, {}).  `app_code` (dist_render's
    per-frame appearance code, inferer_impl.py:144-145) is forwarded when given."""
    extra_kw = {} if app_code is None else {"app_code": app_code}
    all_ret = {}
    extra_loss = {}
    n_all = rays.shape[0]
    for ci in range(n_all // chunk + int(n_all % chunk > 0)):
        rays_chunk = rays[ci * chunk : (ci + 1) * chunk].to(device)
        if idxs is not None:
            idxs_chunk = idxs[ci * chunk : (ci + 1) * chunk].to(device)
            ret, extra_loss = gridnerf(rays_chunk, is_train=is_train, white_bg=white_bg, N_samples=N_samples, idxs_chunk=idxs_chunk)
        else:
            ret, extra_loss = gridnerf(rays_chunk, is_train=is_train, white_bg=white_bg, N_samples=N_samples, **extra_kw)
        for k in ret:
            all_ret.setdefault(k, []).append(ret[k])
    all_ret = {k: torch.cat(v, 0) for k, v in all_ret.items()}
    return all_ret, extra_loss


class MultiBlockParallelHIP:
    """Pre-sized workspace + forward, the calling convention dist_render's inferer installs
    with set_forward_func (dist_render/ddp_infer/inferer_impl.py:351-366)."""

    def __init__(self):
        self._tensorf = None

    def allocate_tensors(self, tensorf, N_rays):
        self._tensorf = tensorf
        S = tensorf._samples_for(-1)
        tensorf.workspace(int(N_rays), S)

    def forward(self, rays_chunk, app_code=None, white_bg=True):
        if self._tensorf is None:
            raise RuntimeError("allocate_tensors(model, N_rays) must be called first")
        ret, _ = self._tensorf(rays_chunk, app_code=app_code, white_bg=white_bg, is_train=False)
        return ret

    __call__ = forward
