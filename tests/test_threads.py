"""The calling convention of the reference's serving engine: the model is called from a pipeline worker thread,
inside torch.inference_mode() and possibly under a stream of its own (dist_render/ddp_infer/inferer_impl.py:95-120,
dist_render/runner/pipe_runner/easy_pipeline/worker.py:38-46).  The library promises that calls from different
threads do not interact unless they share buffers; these tests run it that way."""
import threading

import pytest
import torch

from landmark_amd import scenes

pytestmark = pytest.mark.gpu


def _scene(seed, S=128, opt=1):
    p = scenes.make_params(seed=seed, gridSize=(17, 19, 23), near_far=[0.5, 4.5], n_importance=S, sampling_opt=opt,
                           density_shift=0.0, step_ratio=0.3, resMode=(1, 2))
    for t in p.density_plane:
        t.mul_(6.0)
    p.alpha_volume = scenes.blob_occupancy((23, 19, 17), 6, 0.45, seed=seed)
    p.alpha_aabb = p.aabb.clone()
    return p


def _run_threads(workers):
    errors = []

    def guard(fn):
        def run():
            try:
                fn()
            except BaseException as e:  # noqa: BLE001 - reported by the main thread
                errors.append(e)
        return run

    threads = [threading.Thread(target=guard(w)) for w in workers]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    if errors:
        raise errors[0]


def test_two_worker_threads_own_models_own_streams(gpu_lib):
    """Two threads, each with its own model, its own current stream and inference mode, rendering repeatedly at the
    same time (one of them with the white background off and a smaller chunk): every result equals the
    single-threaded render of the same model bit for bit."""
    from landmark_amd.model import GridNeRFHIP

    rays = [scenes.pinhole_rays(96, 80, 80.0, scenes.sphere_pose(2.5, 9)).cuda(),
            scenes.pinhole_rays(70, 110, 75.0, scenes.sphere_pose(2.4, 4)).cuda()]
    models = [GridNeRFHIP(_scene(11), mlp_precision="f16x2"), GridNeRFHIP(_scene(12, S=100, opt=0), mlp_precision="f32")]
    kw = [dict(white_bg=True, app_code=None), dict(white_bg=False, app_code=None, N_samples=100)]
    want = [m(r, **k)[0] for m, r, k in zip(models, rays, kw)]
    assert all(int(m.last_counts()["n_app"]) > 0 for m in models)
    torch.cuda.synchronize()
    got = [[], []]
    start = threading.Barrier(2)

    def worker(i):
        def run():
            stream = torch.cuda.Stream()
            start.wait(timeout=60)
            with torch.inference_mode(), torch.cuda.stream(stream):
                for rep in range(6):
                    out = models[i](rays[i], **kw[i])  # the engine's call: gridnerf(rays_chunk, white_bg=..., app_code=...)
                    ret = out[0] if isinstance(out, tuple) else out
                    got[i].append((ret["rgb_map"], ret["depth_map"]))
                stream.synchronize()
        return run

    _run_threads([worker(0), worker(1)])
    for i in range(2):
        assert len(got[i]) == 6
        for rgb, dep in got[i]:
            assert torch.equal(rgb, want[i]["rgb_map"]) and torch.equal(dep, want[i]["depth_map"])


def test_two_worker_threads_share_one_model_through_slots(gpu_lib):
    """One model, two threads, each rendering its half of the rays into the shared outputs through a workspace slot
    and counter block of its own (render_into(..., slot=)) on its own stream: the halves equal the single-threaded
    render bit for bit, whichever thread runs first."""
    from landmark_amd.model import GridNeRFHIP

    m = GridNeRFHIP(_scene(13), mlp_precision="f16x2", capacity="worst")
    rays = scenes.pinhole_rays(120, 100, 95.0, scenes.sphere_pose(2.5, 2)).cuda()
    N = rays.shape[0]
    want, _ = m(rays)
    torch.cuda.synchronize()
    halves = [slice(0, N // 2 + 77), slice(N // 2 + 77, N)]
    start = threading.Barrier(2)
    for rep in range(3):
        rgb = torch.full((N, 3), -1.0, device="cuda")
        dep = torch.full((N,), -1.0, device="cuda")
        torch.cuda.synchronize()

        def worker(i):
            def run():
                stream = torch.cuda.Stream()
                start.wait(timeout=60)
                with torch.inference_mode(), torch.cuda.stream(stream):
                    for _ in range(4):
                        m.render_into(rays[halves[i]], rgb[halves[i]], dep[halves[i]], white_bg=True, slot=i)
                    stream.synchronize()
            return run

        _run_threads([worker(0), worker(1)])
        assert torch.equal(rgb, want["rgb_map"]) and torch.equal(dep, want["depth_map"])


def test_forward_on_a_non_default_stream(gpu_lib):
    """forward under `with torch.cuda.stream(s)` (no default-stream ordering to lean on): inputs produced on that
    stream just before the call, several chunks dealt to side streams, result read after synchronising s only."""
    from landmark_amd.model import GridNeRFHIP

    m = GridNeRFHIP(_scene(14), mlp_precision="f16x2")
    base = scenes.pinhole_rays(90, 90, 85.0, scenes.sphere_pose(2.5, 6)).cuda()
    want, _ = m(base)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s), torch.inference_mode():
        rays = base.clone() * 1.0  # produced on s: the render must be ordered behind it
        out, _ = m(rays, chunk=1000, streams=3)
        s.synchronize()
        assert torch.equal(out["rgb_map"], want["rgb_map"]) and torch.equal(out["depth_map"], want["depth_map"])
