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
                app_code=None, exact_chunk=False):
    """Returns ({"rgb_map": [N,3], "depth_map": [N]}, {}).  `app_code` (dist_render's
    per-frame appearance code, inferer_impl.py:144-145) is forwarded when given.
    Rays are independent, so the result does not depend on how they are cut into chunks (bit for
    bit); `chunk` bounds memory in the reference and is a lower bound here: a model that offers
    `preferred_chunk` gets launches of that size (up to 2^20 rays within its workspace budget)
    unless exact_chunk=True asks for the reference's slicing."""
    extra_kw = {} if app_code is None else {"app_code": app_code}
    all_ret = {}
    extra_loss = {}
    n_all = rays.shape[0]
    chunk = int(chunk)
    if not exact_chunk and idxs is None and n_all > chunk and hasattr(gridnerf, "preferred_chunk"):
        chunk = max(chunk, gridnerf.preferred_chunk(n_all, N_samples))
    if exact_chunk and idxs is None and not is_train and hasattr(gridnerf, "render_chunks"):
        # the reference's slicing, but one call: outputs allocated once, the chunks dealt to four streams (a chunk
        # of a few thousand rays cannot fill the GPU, four of them side by side come closer)
        return gridnerf(rays.to(device), is_train=False, white_bg=white_bg, N_samples=N_samples, chunk=chunk, streams=4,
                        **extra_kw)
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

    def __init__(self, **model_kw):
        """Keyword arguments (device, mlp_precision, term_eps, ...) are used when allocate_tensors has to
        wrap a reference model itself."""
        self._tensorf = None
        self._model_kw = model_kw

    def allocate_tensors(self, tensorf, N_rays):
        """`tensorf` is what dist_render's inferer passes: its loaded reference model, single or block-stacked
        (inferer_impl.py:354-362), which is wrapped here; an already wrapped GridNeRFHIP is taken as it is."""
        from .model import from_reference_model

        self._tensorf = from_reference_model(tensorf, **self._model_kw)
        S = self._tensorf._samples_for(-1)
        self._tensorf.workspace(int(N_rays), S)
        return self._tensorf

    def forward(self, rays_chunk, app_code=None, white_bg=True):
        if self._tensorf is None:
            raise RuntimeError("allocate_tensors(model, N_rays) must be called first")
        ret, _ = self._tensorf(rays_chunk, app_code=app_code, white_bg=white_bg, is_train=False)
        return ret

    __call__ = forward


def ray_direction_tables(H, W, focal):
    """The two torch.arange tables of get_ray_directions_blender_faster
    (dist_render/dataset/utils.py:57-72), evaluated on the host."""
    cx, cy = W / 2, H / 2
    dx = torch.arange(-cx / focal, (W - cx - 1e-5) / focal, 1 / focal, dtype=torch.float32)
    dy = torch.arange(cy / focal, (cy - H + 1e-5) / focal, -1 / focal, dtype=torch.float32)
    if dx.numel() != W or dy.numel() != H:
        raise ValueError(f"direction tables have {dx.numel()}x{dy.numel()} entries for a {W}x{H} image")
    return dx, dy


def generate_rays(single_pose, H, W, focal=None, device="cuda"):
    """[H*W, 6] rays on the GPU from a [3,4+] pose; `focal` defaults to pose[-1,-1]
    (generate_rays, dist_render/dataset/utils.py:92-113)."""
    from . import _lib as L

    pose = torch.as_tensor(single_pose, dtype=torch.float32).cpu()
    if focal is None:
        focal = float(pose[-1, -1])
    dx, dy = ray_direction_tables(int(H), int(W), float(focal))
    dx, dy = dx.to(device), dy.to(device)
    p34 = pose[:3, :4].contiguous().numpy()
    rays = torch.empty((int(H) * int(W), 6), dtype=torch.float32, device=device)
    L.check(L.load().lm_generate_rays(dx.data_ptr(), dy.data_ptr(), p34.ctypes.data, int(H), int(W), rays.data_ptr(), L.current_stream()), "lm_generate_rays")
    return rays


def pinned_image(H, W):
    """Page-locked host buffer for one [H,W,4] uint8 frame (allocated pinned; reuse it across frames)."""
    return torch.empty((int(H), int(W), 4), dtype=torch.uint8, pin_memory=True)


def postprocess_rgba8(rgb_map, H, W, host_image=None):
    """[H,W,4] uint8 image (alpha 255) from rgb in [0,1]
    (model_infer_postprocess, dist_render/ddp_infer/nerf_inferer.py:366-370).  With `host_image` (from
    pinned_image) the frame is also copied there on the current stream without blocking, the reference's
    pinned device-to-host step (nerf_inferer.py:371-374); it is complete once the stream is synchronised."""
    from . import _lib as L

    rgb = rgb_map.contiguous()
    out = torch.empty((int(H), int(W), 4), dtype=torch.uint8, device=rgb.device)
    L.check(L.load().lm_rgba8(rgb.data_ptr(), rgb.shape[0], out.data_ptr(), L.current_stream()), "lm_rgba8")
    if host_image is not None:
        if not host_image.is_pinned() or host_image.shape != out.shape or host_image.dtype != torch.uint8:
            raise ValueError("host_image must be a pinned uint8 tensor of shape [H,W,4]")
        host_image.copy_(out, non_blocking=True)
    return out


@torch.no_grad()
def render_frame(gridnerf, single_pose, H, W, focal=None, chunk=1 << 19, app_code=None, white_bg=True, depth=False,
                 streams=2, host_image=None):
    """Pose -> [H,W,4] uint8 image on the GPU: rays from the pose, the render in chunks, the RGBA8 conversion
    (the per-frame sequence of dist_render's inferer: generate_rays, renderer_fn, model_infer_postprocess;
    dist_render/ddp_infer/inferer_impl.py:143-170, nerf_inferer.py:345-378).  Rays are produced row by row, so the
    model is told the row length and chunks are cut at whole bands of 8 rows; nothing leaves the device.
    The chunks are dealt to `streams` streams (the current one and side streams of the same priority, a workspace
    each), so the compute-bound stages of one chunk run under the memory-bound stages of another; the current
    stream continues after all of them.  Half-million-ray chunks on two streams measured best for a 1080p frame
    (0.2 ms less than two chunks of a million, 0.8 ms less than one stream).  With depth=True also returns the [H,W] depth map; with `host_image`
    (pinned_image) the frame is also copied to the host without blocking."""
    H, W = int(H), int(W)
    rays = generate_rays(single_pose, H, W, focal, device=gridnerf.device)
    N = H * W
    S = gridnerf._samples_for(-1)
    while chunk * S >= 2**32:
        chunk //= 2
    if W % 8 == 0:
        chunk = max(8 * W, int(chunk) // (8 * W) * (8 * W))
    rgb = torch.empty((N, 3), dtype=torch.float32, device=gridnerf.device)
    dep = torch.empty((N,), dtype=torch.float32, device=gridnerf.device)
    gridnerf._set_app_code(gridnerf.mlp_precision, app_code)
    saved = gridnerf.ray_row_length
    gridnerf.ray_row_length = W if W % 8 == 0 else 0
    try:
        gridnerf.render_chunks(rays, rgb, dep, chunk, white_bg=white_bg, streams=streams)
    finally:
        gridnerf.ray_row_length = saved
    image = postprocess_rgba8(rgb, H, W, host_image)
    return (image, dep.view(H, W)) if depth else image
