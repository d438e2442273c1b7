#!/usr/bin/env python3
"""Benchmark of the MI355X GridNeRF render path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c1|c2|c3|c5] ...

A step is one pass of the render path over one synthetic frame (or one batch of the
isolated-kernel workloads).  Inputs are resident in HBM before the timed region.  One
JSON line is printed: whole-frame throughput in Mrays/s (`value`), the per-stage kernel
times measured with HIP events inside the timed region, the roofline figure of the
dominant kernel, and the CPU oracle timed on this box's host cores on a bounded sample
of the same workload.

Default workload (the fourth benchmark configuration): a full 1920x1080 frame of a multi-resolution GridNeRF
(levels 1024^2/2048^2/4096^2, 16 + 48 channels fp32, 256^3 occupancy at ~30 %, 128
samples per ray).  The density shift is 0 so that every stage does work (with the stated
N(0, 0.1) init and shift -10 every weight stays below the 1e-3 threshold and the colour
network never runs; `--density-shift -10` reproduces that case).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0, "bf16": 2500.0, "f16x2": 2500.0}
MLP_FLOP_PER_ROW = 2 * (150 * 128 + 128 * 128 + 128 * 3)
PROFILE_DIR = os.path.join(ROOT, "profiles")


def measured_traffic(workload, chunk, mlp, term, kernel):
    """HBM-side bytes per launch of `kernel` as the rocprofv3 counter runs summarised under profiles/ measured
    them, or None.  A summary carries one line per kernel of the form
        bench-traffic: workload=<name> chunk=<rays> mlp=<mode> term_eps=<auto|value> kernel=<k> fetch_bytes=<n> write_bytes=<n>
    (FETCH_SIZE and WRITE_SIZE per dispatch, scaled by the factors a copy of known size gave in the same runs).
    Returns (bytes, "file:line") for the first line that names this exact configuration."""
    if not os.path.isdir(PROFILE_DIR):
        return None
    for fn in sorted(os.listdir(PROFILE_DIR)):
        if not fn.endswith(".txt"):
            continue
        with open(os.path.join(PROFILE_DIR, fn)) as f:
            for ln, line in enumerate(f, 1):
                if not line.startswith("bench-traffic:"):
                    continue
                kv = dict(tok.split("=", 1) for tok in line.split()[1:] if "=" in tok)
                if (kv.get("workload") == workload and kv.get("chunk") == str(chunk) and kv.get("mlp") == mlp
                        and kv.get("term_eps") == term and kv.get("kernel") == kernel):
                    return float(kv["fetch_bytes"]) + float(kv["write_bytes"]), f"profiles/{fn}:{ln}"
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def plane_bytes_per_sample(planes):
    return sum(4 * pl.C * (4 if pl.dtype == 0 else 2) for pl in planes)


# ----------------------------------------------------------------------------------------
def frame_chunks(model, N, S, W, want, row_hint=True):
    """Rays per lm_render call: as asked, within 32-bit sample indices, whole bands of 8 image rows when the
    rays are an image's pixels (the library then visits them in 8 x 8 tiles)."""
    chunk = min(want, N)
    while chunk * S >= 2**32:
        chunk //= 2
    model.ray_row_length = 0
    if row_hint and W % 8 == 0:
        model.ray_row_length = W
        chunk = max(8 * W, chunk // (8 * W) * (8 * W))
    return chunk


def time_frames(model, rays, rgb, depth, chunk, steps, warmup, counters=None, events=None):
    """ms per frame over `steps` frames on the current stream (wall clock between two synchronisations)."""
    N = rays.shape[0]
    n_chunks = (N + chunk - 1) // chunk

    def frame(ev=None):
        for ci in range(n_chunks):
            sl = slice(ci * chunk, min((ci + 1) * chunk, N))
            model.render_into(rays[sl], rgb[sl], depth[sl], white_bg=True, counters=None if counters is None else counters[ci],
                              events=None if ev is None else ev[ci])

    for _ in range(warmup):
        frame()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        frame(None if events is None else events[k])
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def bench_frame(args, workload):
    from landmark_amd import _lib as L
    from landmark_amd import scenes
    from landmark_amd.model import GridNeRFHIP

    dev = "cuda:0"
    t0 = time.time()
    app_code = None
    if workload == "c4":
        p = scenes.c4_scene(P=args.planes, base=args.base, device=dev, density_shift=args.density_shift)
        H, W = args.height, args.width
        rays = scenes.c4_rays(H, W, frame=args.frame, device=dev)
        name = f"c4_1080p_multires_P{args.planes}_base{args.base}_shift{args.density_shift:g}"
    elif workload == "prod":
        p = scenes.production_scene(base=args.base, step_ratio=args.step_ratio, device=dev, density_shift=args.density_shift)
        H, W = args.height, args.width
        rays = scenes.c4_rays(H, W, frame=args.frame, device=dev)
        name = f"prod_1080p_aabb_sampler_P1_L3_base{args.base}_step{args.step_ratio:g}_encodeapp_nonlinear"
        app_code = 3
    elif workload == "c1":
        # sampling_opt 0: 3.47 grid cells per step make nSamples 128 and the steps span the box diagonal
        p = scenes.c1_scene(dense=args.density_shift == 0.0, device=dev, sampling_opt=args.sampling_opt, step_ratio=3.47 if args.sampling_opt == 0 else 2.0)
        H, W = 400, 400
        rays = scenes.c1_rays(H, W, device=dev)
        name = f"c1_tiny_400x400_shift{args.density_shift:g}_{'hull' if args.sampling_opt else 'aabb_step3.47'}_S128"
    elif workload == "c5":
        p = scenes.c5_scene(res=args.base * 8, device=dev, density_shift=args.density_shift)
        H, W = 2160, 3840
        rays = scenes.c5_rays(H, W, device=dev)
        name = f"c5_4k_cityblock_res{args.base * 8}"
    else:
        raise ValueError(workload)
    if args.mlp == "auto":
        args.mlp = "f16" if p.app_plane[0].dtype == torch.float16 else "f16x2"
    term_auto = args.term_eps == "auto"
    term_eps = 1e-4 / float(p.near_far[1]) if term_auto else float(args.term_eps)
    args.term_eps = term_eps
    model = GridNeRFHIP(p, device=dev, mlp_precision=args.mlp, term_eps=term_eps, capacity=args.capacity)
    model._set_app_code(args.mlp, app_code)
    torch.cuda.synchronize()
    log(f"[bench] scene {name} built in {time.time() - t0:.1f}s; tables "
        f"{sum(t.numel() * t.element_size() for t in model._tables) / 1e9:.2f} GB")
    N = rays.shape[0]
    S = model._samples_for(-1)
    chunk = frame_chunks(model, N, S, W, args.chunk, not args.no_row_hint)
    n_chunks = (N + chunk - 1) // chunk
    rgb = torch.empty((N, 3), device=dev)
    depth = torch.empty((N,), device=dev)
    counters = torch.zeros((n_chunks, L.LM_STAT_WORDS), dtype=torch.int32, device=dev)
    # one untimed frame sizes the workspace: the library starts from a guess of the samples per ray, reads the
    # counters and repeats chunks that did not fit (GridNeRFHIP.finish_chunks); the timed frames then run on a
    # workspace of fixed size, and the overflow counter is checked again after them
    done = []
    for ci in range(n_chunks):
        sl = slice(ci * chunk, min((ci + 1) * chunk, N))
        caps = model.render_into(rays[sl], rgb[sl], depth[sl], white_bg=True, counters=counters[ci])
        done.append((sl, counters[ci], caps))
    repeats = model.finish_chunks(done, rays, rgb, depth, white_bg=True)
    ws = model.workspace(chunk, S)
    log(f"[bench] workspace {ws.numel() / 1e9:.2f} GB for chunks of {chunk} rays ({repeats} chunk renders repeated while sizing it; "
        f"samples per ray it holds: valid {model.samples_per_ray[0]:.1f}, appearance {model.samples_per_ray[1]:.1f})")
    n_ev = L.LM_N_STAGES + 1
    events = [[[torch.cuda.Event(enable_timing=True) for _ in range(n_ev)] for _ in range(n_chunks)] for _ in range(args.steps)]
    for per_step in events:
        for per_chunk in per_step:
            for e in per_chunk:
                e.record()  # creates the underlying hipEvent handle

    # ---- the timed region: inputs resident, `steps` frames on one stream
    ms_step = time_frames(model, rays, rgb, depth, chunk, args.steps, args.warmup, counters, events)

    def frame_plain():
        for ci in range(n_chunks):
            sl = slice(ci * chunk, min((ci + 1) * chunk, N))
            model.render_into(rays[sl], rgb[sl], depth[sl], white_bg=True, counters=counters[ci])

    # the same frames when the boundary hands over host buffers: rays from pinned host memory, rgb and depth back to
    # it, copies and kernels on the one stream (reported beside the metric, never as the metric)
    ms_host_io = None
    if args.host_io:
        rays_h = torch.empty(rays.shape, dtype=rays.dtype, pin_memory=True).copy_(rays)
        rgb_h = torch.empty(rgb.shape, dtype=rgb.dtype, pin_memory=True)
        depth_h = torch.empty(depth.shape, dtype=depth.dtype, pin_memory=True)
        rays_d = torch.empty_like(rays)

        def frame_io():
            for ci in range(n_chunks):
                sl = slice(ci * chunk, min((ci + 1) * chunk, N))
                rays_d[sl].copy_(rays_h[sl], non_blocking=True)
                model.render_into(rays_d[sl], rgb[sl], depth[sl], white_bg=True, counters=counters[ci])
                rgb_h[sl].copy_(rgb[sl], non_blocking=True)
                depth_h[sl].copy_(depth[sl], non_blocking=True)

        frame_io()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            frame_io()
        torch.cuda.synchronize()
        ms_host_io = (time.perf_counter() - t0) / args.steps * 1e3
        assert torch.equal(rgb_h, rgb.cpu())

    # the same frames with the chunks dealt to two streams (a workspace each): the compute-bound stages of one
    # chunk run under the memory-bound stages of the other (reported beside the metric)
    ms_two = None
    if args.streams > 1 and n_chunks > 1:
        streams = [torch.cuda.Stream() for _ in range(args.streams)]
        slot_counters = torch.zeros((n_chunks, L.LM_STAT_WORDS), dtype=torch.int32, device=dev)
        rgb2, depth2 = torch.empty_like(rgb), torch.empty_like(depth)

        def frame_streams():
            for ci in range(n_chunks):
                sl = slice(ci * chunk, min((ci + 1) * chunk, N))
                with torch.cuda.stream(streams[ci % args.streams]):
                    model.render_into(rays[sl], rgb2[sl], depth2[sl], white_bg=True, counters=slot_counters[ci],
                                      slot=ci % args.streams)

        torch.cuda.synchronize()
        frame_streams()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            frame_streams()
        torch.cuda.synchronize()
        ms_two = (time.perf_counter() - t0) / args.steps * 1e3
        assert torch.equal(rgb2, rgb) and torch.equal(depth2, depth)
        del rgb2, depth2

    cnt = counters.cpu().long() & 0xFFFFFFFF
    n_valid, n_app = int(cnt[:, L.LM_STAT_N_VALID].sum()), int(cnt[:, L.LM_STAT_N_APP].sum())
    n_marched = int(cnt[:, L.LM_STAT_N_MARCHED].sum())
    overflow = int(cnt[:, L.LM_STAT_OVERFLOW].sum())
    if overflow:
        raise RuntimeError(f"{overflow} rays did not fit the workspace capacity: the timed frames are incomplete")
    stage_ms = [0.0] * L.LM_N_STAGES  # per frame, averaged over steps
    for per_step in events:
        for per_chunk in per_step:
            for s in range(L.LM_N_STAGES):
                stage_ms[s] += per_chunk[s].elapsed_time(per_chunk[s + 1])
    stage_ms = [x / args.steps for x in stage_ms]
    launches = n_chunks  # one launch of each stage kernel per chunk
    dens_B = plane_bytes_per_sample(model._density) + 4  # + weight out
    app_B = plane_bytes_per_sample(model._app) + 4 + 27 * 4  # + index in, projected features out
    basis_flop = 2 * model.K_app * 27  # basis_mat runs inside the appearance gather
    stages = {}
    for i, nm in enumerate(L.STAGE_NAMES):
        stages[nm] = {"ms_per_frame": round(stage_ms[i], 4)}
    # GB/s figures of the gathers are in gather-convention bytes: every corner load of every sample, no reuse
    stages["density_march"].update(bytes_per_sample=dens_B, samples=n_marched,
                                   convention_GBps=round(n_marched * dens_B / max(stage_ms[1], 1e-9) / 1e6, 1))
    stages["app_gather"].update(bytes_per_sample=app_B, samples=n_app,
                                convention_GBps=round(n_app * app_B / max(stage_ms[3], 1e-9) / 1e6, 1),
                                basis_TFLOPs=round(n_app * basis_flop / max(stage_ms[3], 1e-9) / 1e9, 2))
    stages["colour"].update(rows=n_app, TFLOPs=round(n_app * MLP_FLOP_PER_ROW / max(stage_ms[4], 1e-9) / 1e9, 2),
                            frac_of_mfma_peak=round(n_app * MLP_FLOP_PER_ROW / max(stage_ms[4], 1e-9) / 1e9 / MFMA_PEAK_TFLOPS[args.mlp], 4))
    # occupancy lookups: 1 byte per sample from the cell table (8 x 4 bytes with a float volume), upper bound
    # every sample; 1 bit per sample and 24 bytes per ray besides
    cull_B = (1 if model._vol_dtype == L.LM_CELLS else 32 if model._vol is not None else 0) + 0.125
    stages["cull"].update(bytes_per_sample=cull_B, Gsamples_per_s=round(N * S / (stage_ms[0] * 1e-3) / 1e9, 1),
                          GBps=round((N * S * cull_B + N * 24) / (stage_ms[0] * 1e-3) / 1e9, 1))
    stages["composite"].update(GBps=round((n_app * 16 + N * 32) / max(stage_ms[5], 1e-9) / 1e6, 1))  # w + rgb per slot; first, count, acc in and rgb out per ray
    stages["app_list"].update(GBps=round((n_marched * 4 + N * S / 8 + n_app * 8 + N * 16) / (stage_ms[2] * 1e-3) / 1e9, 1))

    # dominant kernel -> roofline object
    cand = {"density_march": stage_ms[1], "app_gather": stage_ms[3], "colour": stage_ms[4]}
    dom = max(cand, key=cand.get)
    avg_ms = cand[dom] / launches
    if dom == "colour":
        ach = stages["colour"]["TFLOPs"]
        peak = MFMA_PEAK_TFLOPS[args.mlp]
        roof = {"kernel": "k_mlp", "bound": "mfma", "achieved": ach, "peak": peak, "unit": "TFLOP/s",
                "frac": round(ach / peak, 4), "traffic": None}
    else:
        kernel = "k_march" if dom == "density_march" else "k_app_feat"
        conv = stages[dom]["convention_GBps"]
        found = measured_traffic(name, chunk, args.mlp, "auto" if term_auto else f"{term_eps:g}", kernel) \
            if int(model.ray_row_length) == W else None
        roof = {"kernel": kernel, "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "convention": "gather, no reuse: every corner load of every sample counted, line tables excluded",
                "convention_bytes_per_launch": round(stages[dom]["samples"] * stages[dom]["bytes_per_sample"] / launches),
                "convention_GBps": conv}
        if found:
            # bytes the launch moved past the L2 (rocprofv3 counters, summarised under profiles/) / its duration here
            roof["traffic"], roof["traffic_source"] = found
            roof["achieved"] = round(found[0] / (avg_ms * 1e-3) / 1e9, 1)
            roof["frac"] = round(roof["achieved"] / HBM_PEAK_GBS, 4)
            roof["basis"] = "counter-derived HBM-side bytes per launch / launch duration measured in this run"
        else:
            # no counter figure for this configuration: the convention rate is an upper bound of the HBM rate (texels
            # shared by neighbouring samples are counted once per sample), so it is no fraction of the peak
            roof["traffic"] = None
            roof["achieved"] = conv
            roof["frac"] = None
            roof["basis"] = "gather-convention bytes / launch duration (no counter run covers this configuration)"
    roof["avg_launch_ms"] = round(avg_ms, 4)
    roof["launches_per_frame"] = launches

    cpu, parity = cpu_baseline_frame(args, model, p, rays, rgb, depth, H, W, app_code)
    mrays = N / (ms_step * 1e-3) / 1e6
    out = {
        "metric": "render_throughput", "value": round(mrays, 3), "unit": "Mrays/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": ("f16" if p.app_plane[0].dtype == torch.float16 else "f32") + ("" if args.mlp == "f32" else f"+{args.mlp}-mlp"),
        "data": "synthetic",
        "config": {"workload": name, "rays": N, "samples_per_ray": S, "chunk_rays": chunk, "ray_row_hint": int(model.ray_row_length), "mlp": args.mlp,
                   "term_eps": args.term_eps, "valid_samples": n_valid, "marched_samples": n_marched, "app_samples": n_app,
                   "workspace_GB": round(ws.numel() / 1e9, 3)},
        "frames_per_s": round(1e3 / ms_step, 3), "mpixel_per_s": round(mrays, 3),
        "stages": stages, "roofline": roof, "cpu_baseline": cpu, "parity": parity,
    }
    if ms_host_io is not None:
        out["ms_per_step_host_buffers"] = round(ms_host_io, 4)
    if ms_two is not None:
        out["ms_per_step_streams"] = {"streams": args.streams, "ms": round(ms_two, 4)}
    if workload == "c4" and not args.no_extra:
        # the same frame in two more settings, timed in this run after the region above (never `value`):
        # the reference-semantics mode (fp32 matrix products, no early termination) and the one-orientation model
        steps = max(3, args.steps // 2)

        def timed_complete(mod, ck, what):
            """ms per frame of `mod`, after a sizing frame and with the overflow counters checked after the timed ones."""
            nck = (N + ck - 1) // ck
            cn = torch.zeros((nck, L.LM_STAT_WORDS), dtype=torch.int32, device=dev)
            sized = []
            for ci in range(nck):
                sl = slice(ci * ck, min((ci + 1) * ck, N))
                caps = mod.render_into(rays[sl], rgb[sl], depth[sl], white_bg=True, counters=cn[ci])
                sized.append((sl, cn[ci], caps))
            mod.finish_chunks(sized, rays, rgb, depth, white_bg=True)
            ms = time_frames(mod, rays, rgb, depth, ck, steps, 2, cn)
            dropped = int((cn[:, L.LM_STAT_OVERFLOW].cpu().long() & 0xFFFFFFFF).sum())
            if dropped:
                raise RuntimeError(f"{what}: {dropped} rays did not fit the workspace capacity: the timed frames are incomplete")
            return round(ms, 4)

        model.mlp_precision, model.term_eps = "f32", 0.0
        out["ms_per_step_exact"] = {"mlp": "f32", "term_eps": 0.0, "ms": timed_complete(model, chunk, "exact mode")}
        del model
        torch.cuda.empty_cache()
        if args.planes != 1:
            p1 = scenes.c4_scene(P=1, base=args.base, device=dev, density_shift=args.density_shift)
            m1 = GridNeRFHIP(p1, device=dev, mlp_precision=args.mlp, term_eps=term_eps, release_source=True)
            c1 = frame_chunks(m1, N, S, W, args.chunk, not args.no_row_hint)
            out["ms_per_step_P1"] = {"workload": f"c4_1080p_multires_P1_base{args.base}_shift{args.density_shift:g}",
                                     "ms": timed_complete(m1, c1, "one-orientation model")}
            del m1, p1
            torch.cuda.empty_cache()
        # the shape most of the reference's run configurations use (one orientation, three levels, equal-step AABB
        # sampler, appearance embedding, basis_den) on the same tables, mask and camera, at two and at half a grid cell
        # per step (the reference's default); `--workload prod` times it stage by stage
        out["ms_per_step_production_shape"] = {}
        for step_ratio in (2.0, 0.5):
            pp = scenes.production_scene(base=args.base, step_ratio=step_ratio, device=dev, density_shift=args.density_shift)
            mp = GridNeRFHIP(pp, device=dev, mlp_precision=args.mlp, term_eps=1e-4 / float(pp.near_far[1]), release_source=True)
            mp._set_app_code(args.mlp, 3)
            Sp = mp._samples_for(-1)
            cp = frame_chunks(mp, N, Sp, W, args.chunk, not args.no_row_hint)
            steps = 3
            out["ms_per_step_production_shape"][f"step_ratio_{step_ratio:g}"] = {
                "samples_per_ray": Sp, "ms": timed_complete(mp, cp, f"production shape, step ratio {step_ratio:g}")}
            del mp, pp
            torch.cuda.empty_cache()
    return out


def cpu_baseline_frame(args, model, p, rays, rgb, depth, H, W, app_code=None):
    """The CPU oracle on a bounded sample of the frame (evenly spaced scan-lines), timed as the CPU baseline, and the
    parity of the frame just rendered against it: sample-mask mismatches, valid-index and depth-table equality,
    sample counts of the library's own counters, and the two maxima."""
    if args.no_cpu:
        return None, None
    from landmark_amd import _lib as L
    from oracle import gridnerf_oracle as O

    S = p.n_importance if p.sampling_opt else p.nSamples
    rows = max(1, min(H, args.cpu_rows * 128 // max(S, 128)))  # about the same number of samples whatever the sampler
    ys = torch.linspace(0, H - 1, rows).long().unique()
    idx = (ys[:, None] * W + torch.arange(W)[None]).reshape(-1)
    t0 = time.time()
    pc = p.to("cpu")
    log(f"[bench] cpu copy of the model {time.time() - t0:.1f}s")
    r_dev = rays[idx.to(rays.device)].contiguous()
    r = r_dev.cpu()
    torch.set_num_threads(os.cpu_count() if args.cpu_threads <= 0 else args.cpu_threads)
    kw = {} if app_code is None else {"app_code": app_code}
    ref = {k: [] for k in ("rgb_map", "depth_map", "ray_valid", "z_vals", "band")}
    n_app_ref, dt = 0, 0.0
    for i in range(0, r.shape[0], 8192):  # the reference's chunk loop (app/tools/render_utils.py:15-63), chunk 8192
        t0 = time.perf_counter()
        ret = O.render_chunk(pc, r[i:i + 8192], white_bg=True, return_aux=True, **kw)
        dt += time.perf_counter() - t0  # only the render counts as the baseline, not the bookkeeping below
        ret["band"] = ((ret["weight"] - p.rayMarch_weight_thres).abs() < 2e-7).any(-1)
        n_app_ref += int(ret["app_mask"].sum())
        for k in ref:
            ref[k].append(ret[k])
    ref = {k: torch.cat(v) for k, v in ref.items()}
    cpu = {"value": round(r.shape[0] / dt / 1e6, 5), "unit": "Mrays/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"{len(ys)} evenly spaced scan-lines ({r.shape[0]} rays) of the same frame, PyTorch oracle, "
                     f"chunk 8192, {dt:.1f}s"}
    # ---- parity of this run's frame (untimed): decisions bit for bit, rgb / depth maxima
    got_rgb, got_dep = rgb[idx.to(rgb.device)].cpu(), depth[idx.to(rgb.device)].cpu()
    d_rgb = (got_rgb - ref["rgb_map"]).abs().max(-1).values
    d_dep = (got_dep - ref["depth_map"]).abs()
    cull = model.sample_cull(r_dev)
    mism = int((cull["ray_valid"].cpu() != ref["ray_valid"]).sum())
    idx_equal = torch.equal(cull["valid_idx"].cpu(), ref["ray_valid"].reshape(-1).nonzero()[:, 0])
    z_mism = int((cull["z_vals"].cpu() != ref["z_vals"]).sum())
    del cull
    # the whole-chunk render of the same rays on their own: its counters against the oracle's counts, and its
    # pixels against the frame's (rays are independent: the same bits whatever chunk a ray arrives in)
    sub, _ = model(r_dev, white_bg=True, **kw)
    cnt = model.last_counts()
    ok = ~ref["band"]
    parity = {
        "rays_checked": int(r.shape[0]), "samples_checked": int(ref["ray_valid"].numel()),
        "mask_mismatches": mism, "valid_idx_equal": bool(idx_equal), "z_mismatches": z_mism,
        "valid_samples": {"oracle": int(ref["ray_valid"].sum()), "lm_render_counter": cnt["n_valid"]},
        "app_samples": {"oracle": n_app_ref, "lm_render_counter": cnt["n_app"]},
        "app_mask_band_rays": int(ref["band"].sum()),
        "max_abs_rgb": d_rgb.max().item(), "max_abs_depth": d_dep.max().item(),
        "max_abs_rgb_outside_band": d_rgb[ok].max().item(), "max_abs_depth_outside_band": d_dep[ok].max().item(),
        "chunk_invariant": bool(torch.equal(sub["rgb_map"].cpu(), got_rgb) and torch.equal(sub["depth_map"].cpu(), got_dep)),
        "note": "mask = AABB and occupancy decisions of every sample of the checked rays (lm_sample_cull vs oracle); band = rays "
                "holding a weight within 2e-7 of the appearance threshold, whose appearance mask may legitimately differ",
    }
    return cpu, parity


# ----------------------------------------------------------------------------------------
def bench_gather(args):
    """Second benchmark configuration: isolated plane/line gather, 3 planes 2048^2 x 64 ch fp32, 2^24 queries.
    Density form (default): sum over planes and channels -> [M].  Appearance form (--app-mode): the products
    themselves -> [M, 3*64]."""
    from landmark_amd import scenes
    from landmark_amd.model import GridNeRFHIP

    dev = "cuda:0"
    res = args.base * 2
    app = bool(args.app_mode)
    p = scenes.make_params(seed=2, gridSize=(res, res, res), ndims=3, resMode=(1,), density_n_comp=4 if app else 64,
                           app_n_comp=64 if app else 16, device=dev, feature_init="uniform")
    model = GridNeRFHIP(p, device=dev, release_source=True)
    M = args.queries
    g = torch.Generator(device=dev).manual_seed(2)
    xyz = torch.rand((M, 3), device=dev, generator=g) * 2 - 1
    if args.coherent:
        xyz = xyz[torch.argsort((xyz[:, 0] * 64).floor() * 4096 + (xyz[:, 1] * 64).floor())]
    run = model.app_products if app else model.compute_densityfeature
    out = run(xyz)
    for _ in range(args.warmup):
        out = run(xyz)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for k in range(args.steps):
        out = run(xyz)
        ev[k + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ker_ms = sum(ev[k].elapsed_time(ev[k + 1]) for k in range(args.steps)) / args.steps
    planes = model._app if app else model._density
    Bq = plane_bytes_per_sample(planes) + 12 + (4 * model.K_app if app else 4)
    gbs = M * Bq / (ker_ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import gridnerf_oracle as O

        n = 1 << (18 if app else 20)
        pc, sub = p.to("cpu"), xyz[:n].cpu()
        t0 = time.perf_counter()
        ref = O.app_products(pc, sub) if app else O.density_feature(pc, sub)
        cdt = time.perf_counter() - t0
        err = (out[:n].cpu() - ref).abs().max().item()
        cpu = {"value": round(sub.shape[0] / cdt / 1e6, 4), "unit": "Mqueries/s", "cores": torch.get_num_threads(),
               "kind": "port", "sample": f"first {n} queries, F.grid_sample oracle, {cdt:.1f}s, max|diff| {err:.2e}"}
    return {
        "metric": "gather_throughput", "value": round(M / (dt / args.steps) / 1e6, 2), "unit": "Mqueries/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"c2_gather_3x{res}^2x64ch_{M}q_{'coherent' if args.coherent else 'random'}_{'app' if app else 'density'}"},
        "roofline": {"kernel": "k_app_xyz" if app else "k_density_xyz", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     # sorted queries share texels: their algorithmic rate is cache-served and no fraction of the peak
                     "unit": "GB/s", "frac": None if args.coherent else round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "avg_launch_ms": round(ker_ms, 4), "bytes_per_query": Bq},
        "cpu_baseline": cpu,
    }


def bench_mlp(args):
    """Third benchmark configuration: isolated colour network on 2^23 rows."""
    from landmark_amd import scenes
    from landmark_amd.model import GridNeRFHIP

    dev = "cuda:0"
    p = scenes.make_params(seed=3, gridSize=(8, 8, 8), density_n_comp=4, app_n_comp=48)
    prec = args.mlp = "f16" if args.mlp == "auto" else args.mlp  # the isolated network is quoted with fp16 weights
    model = GridNeRFHIP(p, device=dev, mlp_precision=prec)
    M = args.rows
    g = torch.Generator(device=dev).manual_seed(3)
    feat = torch.randn((M, 27), device=dev, generator=g)
    view = torch.nn.functional.normalize(torch.randn((M, 3), device=dev, generator=g), dim=-1)
    for _ in range(args.warmup):
        out = model.render_module(view, feat)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for k in range(args.steps):
        out = model.render_module(view, feat)
        ev[k + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ker_ms = sum(ev[k].elapsed_time(ev[k + 1]) for k in range(args.steps)) / args.steps
    tf = M * MLP_FLOP_PER_ROW / (ker_ms * 1e-3) / 1e12
    # The same launch with a memory-bound kernel (1 GiB elementwise add) before each one, timed alone: back to back the
    # matrix pipes hold the chip at its power limit and the clock falls; in a frame the network follows the gathers.
    pad = torch.zeros(1 << 28, device=dev)
    e0 = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    e1 = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    for k in range(args.steps):
        pad.add_(1.0)
        e0[k].record()
        out = model.render_module(view, feat)
        e1[k].record()
    torch.cuda.synchronize()
    mixed_ms = sum(a.elapsed_time(b) for a, b in zip(e0, e1)) / args.steps
    del pad
    cpu = None
    if not args.no_cpu:
        from oracle import gridnerf_oracle as O

        n = 1 << 20
        t0 = time.perf_counter()
        ref = O.mlp_render(p, view[:n].cpu(), feat[:n].cpu())
        cdt = time.perf_counter() - t0
        err = (out[:n].cpu() - ref).abs().max().item()
        cpu = {"value": round(n / cdt / 1e6, 4), "unit": "Mrows/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"first 2^20 rows, PyTorch oracle, {cdt:.1f}s, max|diff| {err:.2e}"}
    return {
        "metric": "mlp_throughput", "value": round(M / (dt / args.steps) / 1e6, 2), "unit": "Mrows/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": prec, "data": "synthetic",
        "config": {"workload": f"c3_mlp_{M}rows_{prec}"},
        "roofline": {"kernel": "k_mlp_feat", "bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_PEAK_TFLOPS[prec],
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS[prec], 4), "traffic": None,
                     "avg_launch_ms": round(ker_ms, 4)},
        "ms_per_launch_after_memory_bound_kernel": round(mixed_ms, 4),
        "frac_after_memory_bound_kernel": round(M * MLP_FLOP_PER_ROW / (mixed_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS[prec], 4),
        "cpu_baseline": cpu,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--streams", type=int, default=2, help="also time the frame with its chunks dealt to this many streams")
    ap.add_argument("--workload", default="c4", choices=["c1", "c2", "c3", "c4", "c5", "prod"],
                    help="c4 (default): 1080p frame of the multi-resolution model; prod: the same frame with the reference's "
                         "production shape (one orientation, AABB sampler, embedding, density projection)")
    ap.add_argument("--step-ratio", type=float, default=0.5, help="prod: grid cells per sampling step (the reference's default)")
    ap.add_argument("--capacity", default="adaptive", choices=["adaptive", "worst"],
                    help="render workspace: sized from the samples per ray a first frame reports, or for the worst case")
    ap.add_argument("--no-extra", action="store_true", help="c4: skip the exact-mode and one-orientation timings after the timed region")
    ap.add_argument("--planes", type=int, default=3, help="ndims of the c4 model (3 = XY,XZ,YZ; 1 = XY only)")
    ap.add_argument("--base", type=int, default=1024, help="base plane resolution of c4 (levels x1,x2,x4)")
    ap.add_argument("--height", type=int, default=1080)
    ap.add_argument("--width", type=int, default=1920)
    ap.add_argument("--frame", type=int, default=0)
    ap.add_argument("--density-shift", type=float, default=0.0)
    ap.add_argument("--mlp", default="auto", choices=["auto", "f32", "f16x2", "f16", "bf16"],
                    help="arithmetic of the colour network; auto = f16x2 (1e-4 class) with fp32 tables, f16 (1e-2 class) "
                         "where the tables are fp16 already")
    ap.add_argument("--term-eps", default="auto",
                    help="ray termination threshold on the transmittance; 'auto' = 1e-4 / far, the largest value that "
                         "keeps rgb and depth within 1e-4 of the unterminated render; 0 = never terminate")
    ap.add_argument("--chunk", type=int, default=1048576)
    ap.add_argument("--queries", type=int, default=1 << 24)
    ap.add_argument("--rows", type=int, default=1 << 23)
    ap.add_argument("--coherent", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=270)
    ap.add_argument("--cpu-threads", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--host-io", action="store_true", help="also time the frame with rays and results in pinned host memory")
    ap.add_argument("--no-row-hint", action="store_true", help="do not tell the library that rays are image rows")
    ap.add_argument("--calib", action="store_true", help="accepted and ignored: the copy and streaming yardsticks run every time")
    ap.add_argument("--app-mode", action="store_true", help="c2: the appearance form of the gather ([M, 3*64] products out)")
    ap.add_argument("--sampling-opt", type=int, default=1, choices=[0, 1],
                    help="c1: 1 = hull sampler (n_importance 128), 0 = equal-step sampler, 128 steps of 3.47 grid cells")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build renders on one GPU; rays are independent, so more GPUs would each take a slice of "
              "the pixel array, but nothing here launches a second rank. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    # yardsticks of this box's memory system, measured in every run (a fraction of a second): a plain 1 GiB device
    # copy and an elementwise add (1 GiB in, 1 GiB out), bytes read + written per second
    a = torch.ones(1 << 28, device="cuda:0")
    b = torch.empty_like(a)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rates = []
    for op in (lambda: b.copy_(a), lambda: torch.add(a, 1.0, out=b)):
        op()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(20):
            op()
        e1.record()
        torch.cuda.synchronize()
        rates.append(20 * 2 * a.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9)
    copy_rate, stream_rate = rates
    log(f"[bench] 1 GiB device copy {copy_rate:.0f} GB/s, elementwise add {stream_rate:.0f} GB/s (read + write)")
    del a, b
    torch.cuda.empty_cache()
    if args.workload == "c2":
        out = bench_gather(args)
    elif args.workload == "c3":
        out = bench_mlp(args)
    else:
        out = bench_frame(args, args.workload)
    out["hbm_copy_GBps"] = round(copy_rate, 1)
    out["hbm_stream_GBps"] = round(stream_rate, 1)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
