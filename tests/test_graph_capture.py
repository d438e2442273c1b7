"""The whole-chunk render recorded into a HIP graph and replayed.

lm_render and lm_render_static only launch kernels on the stream they are given (counters and bitmaps are cleared
by fill kernels, not by memset nodes) and look device facts up once per device, so after one eager call both can be
recorded by stream capture.  The test records each into a graph, replays it on changing inputs with eager renders
in between, and compares every replay with the eager result bit for bit."""
import ctypes as C

import pytest
import torch

from landmark_amd import _lib as L
from landmark_amd import scenes

pytestmark = pytest.mark.gpu


def _scene(S, opt, seed=11):
    p = scenes.make_params(seed=seed, gridSize=(9, 11, 13), near_far=[0.5, 4.5], n_importance=S, sampling_opt=opt,
                           density_shift=0.0, step_ratio=0.3, resMode=(1, 2))
    for t in p.density_plane:
        t.mul_(6.0)
    p.alpha_volume = scenes.blob_occupancy((13, 11, 9), 6, 0.45, seed=seed)
    p.alpha_aabb = p.aabb.clone()
    return p


@pytest.mark.parametrize("static", [False, True])
@pytest.mark.parametrize("opt,S", [(1, 128), (0, 100)])
def test_render_recorded_into_a_graph(gpu_lib, static, opt, S):
    from landmark_amd.model import GridNeRFHIP

    dev = "cuda"
    model = GridNeRFHIP(_scene(S, opt), mlp_precision="f16x2", capacity="worst")
    lib = model.lib
    poses = [scenes.pinhole_rays(60, 50, 52.0, scenes.sphere_pose(2.5, k)).to(dev) for k in (9, 3, 14)]
    N = poses[0].shape[0]
    m = model._model_struct(S, True)
    ws = model.workspace(N, S)

    def launch(rays, rgb, depth, cnt):
        if static:
            rc = lib.lm_render_static(C.byref(m), rays.data_ptr(), N, rgb.data_ptr(), depth.data_ptr(), cnt.data_ptr(),
                                      L.current_stream())
        else:
            rc = lib.lm_render(C.byref(m), rays.data_ptr(), N, ws.data_ptr(), ws.numel(), rgb.data_ptr(), depth.data_ptr(),
                               cnt.data_ptr(), L.current_stream())
        L.check(rc, "render")

    def eager(rays):
        rgb = torch.full((N, 3), -1.0, device=dev)
        depth = torch.full((N,), -1.0, device=dev)
        cnt = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device=dev)
        launch(rays, rgb, depth, cnt)
        torch.cuda.synchronize()
        return rgb, depth, cnt[:4].clone()

    want = [eager(r) for r in poses]  # also the first call on this device: set-up happens here, outside the capture
    assert all(int(w[2][L.LM_STAT_N_APP]) > 100 for w in want)
    rays = poses[0].clone()
    rgb = torch.full((N, 3), -1.0, device=dev)
    depth = torch.full((N,), -1.0, device=dev)
    cnt = torch.zeros(L.LM_STAT_WORDS, dtype=torch.int32, device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(rays, rgb, depth, cnt)
    for k in (0, 1, 2, 1, 0):
        rays.copy_(poses[k])
        rgb.fill_(-1.0)
        depth.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(rgb, want[k][0]) and torch.equal(depth, want[k][1]) and torch.equal(cnt[:4], want[k][2]), k
        again = eager(poses[(k + 1) % 3])  # the program's own eager work between replays
        assert torch.equal(again[0], want[(k + 1) % 3][0])
