"""Forward-render throughput of the tile renderer on one MI355X.

A step is one full forward render of one camera pose through the scene module's public call
(`scene(rays_o, rays_d, score_threshold=, view_matrix=, proj_matrix=)`): sparse tile binning, tile-list
validation, per-tile depth sort and the render kernel.  The workload is the 200k-primitive, 1200x680
synthetic scene (seed 0) seen from 32 seeded poses; scene and rays are resident in HBM before the clock
starts.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK = {"f32": 157.3, "bf16": 2500.0}          # MI355X dense peaks, TFLOP/s
HBM_PEAK_GBS = 8000.0
PROFILES = os.path.join(ROOT, "profiles")


def measured_traffic(kernel: str, workload: str, ms_per_launch: float):
    """HBM bytes per launch of `kernel` from the committed hardware-counter profile profiles/<kernel>_<workload>.txt
    (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE, each scaled by what the counter reads for a device copy of
    known size; the file states the commands).  The profile carries the kernel's average duration when the counters
    were taken: if this run's duration differs from it by more than 15 % (boxes of this pool run one build up to 9 %
    apart), the kernel is no longer the one that was profiled and no traffic figure is reported.
    -> (bytes or None, note)"""
    import re
    path = os.path.join(PROFILES, f"{kernel}_{workload}.txt")
    if not os.path.exists(path):
        return None, f"no profile {os.path.basename(path)}"
    text = open(path).read()
    got = {k: re.search(rf"^bench\.{k}\s*=\s*([0-9.eE+]+)", text, flags=re.M) for k in ("traffic_bytes", "kernel_avg_us")}
    if not all(got.values()):
        return None, f"{os.path.basename(path)} holds no bench.traffic_bytes / bench.kernel_avg_us lines"
    traffic, avg_us = float(got["traffic_bytes"].group(1)), float(got["kernel_avg_us"].group(1))
    if abs(ms_per_launch * 1e3 - avg_us) > 0.15 * avg_us:
        return None, (f"profiled kernel took {avg_us:.1f} us, this run {ms_per_launch * 1e3:.1f} us: "
                      f"{os.path.basename(path)} is stale")
    return int(traffic), f"profiles/{os.path.basename(path)} (kernel {avg_us:.1f} us when profiled)"


def dense_culling_cpu_torch(positions, log_scales, view, proj, W, H, tile, thr):
    """The reference's culling as it writes it -- a dense [tiles x primitives] overlap matrix turned into a tile-major
    list (scannet/cumodel.py:994-1070) -- evaluated with CPU torch.  Measurement aid of the cpu_baseline leg only:
    the renderer itself never bins this way.  -> (seconds, number of tile-primitive pairs)"""
    import torch
    t0 = time.perf_counter()
    with torch.no_grad():
        n = positions.shape[0]
        homogeneous = torch.cat([positions, positions.new_ones(n, 1)], dim=1)
        in_view = homogeneous @ view.T
        z = in_view[:, 2]
        visible = z > 1e-3
        largest_axis = log_scales.exp().amax(dim=1)
        focal = 0.5 * (proj[0, 0] * W / 2.0 + proj[1, 1] * H / 2.0)
        reach = largest_axis * torch.sqrt(-2.0 * torch.log(torch.tensor(float(thr)))) / (z + 1e-8) * focal
        clip = in_view @ proj.T
        w = clip[:, 3:4]
        w = w + 1e-6 * (w == 0)
        ndc = clip[:, :3] / w
        cx, cy = (ndc[:, 0] + 1) * 0.5 * W, (ndc[:, 1] + 1) * 0.5 * H
        ntx, nty = (W + tile - 1) // tile, (H + tile - 1) // tile
        tiles = torch.arange(ntx * nty)
        left, top = ((tiles % ntx) * tile)[:, None], ((tiles // ntx) * tile)[:, None]
        touches = ((cx - reach)[None] < left + tile) & ((cx + reach)[None] > left) \
            & ((cy - reach)[None] < top + tile) & ((cy + reach)[None] > top) & visible[None]
        pairs = touches.nonzero()
        order = torch.argsort(pairs[:, 0])
        pairs = pairs[order]
        offsets = torch.zeros(ntx * nty + 1, dtype=torch.long)
        which, how_many = torch.unique_consecutive(pairs[:, 0], return_counts=True)
        offsets.scatter_add_(0, which + 1, how_many)
        offsets = offsets.cumsum(0).to(torch.int32)
        listed = pairs[:, 1].to(torch.int32)
    return time.perf_counter() - t0, int(listed.numel())


def train_steps(args, scene, frames, proj, thr, W, H, sc, dev):
    """One training step = scene(...) under autograd -> L1 loss against a fixed image -> backward (records
    forward, reverse compositing, grouped weight gradients in IEEE f32) -> Adam step on every parameter."""
    import torch
    scene.train()
    scene.render_precision = "f32"
    params = [scene.positions, scene.log_scales, scene.quats, scene.W1, scene.b1, scene.W2, scene.b2, scene.W3, scene.b3]
    opt = torch.optim.Adam(params, lr=1e-4, fused=True)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    target = torch.rand(W * H, 3, device=dev, generator=gen)

    feature_dim = 0 if scene.feat_attr is None else int(scene.feat_attr.shape[-1])
    feature_target = None
    if feature_dim:
        # record-based step with the streamed feature loss against a quarter-resolution target
        params.append(scene.feat_attr)
        opt = torch.optim.Adam(params, lr=1e-4, fused=True)
        feature_target = (torch.randn(H // 4, W // 4, feature_dim, device=dev, generator=gen) * 0.05).half()

    def step(i):
        ro, rd, views, _ = frames[i % len(frames)]
        opt.zero_grad(set_to_none=True)
        if feature_target is None:
            rgb = scene(ro, rd, score_threshold=thr, view_matrix=views[0], proj_matrix=proj)
            loss = (rgb - target).abs().mean()
        elif args.dense_feature_loss:
            # the reference's "legacy" training backend: dense feature image under autograd, resampled by torch
            rgb, feat = scene(ro, rd, score_threshold=thr, view_matrix=views[0], proj_matrix=proj, return_feature=True)
            low = torch.nn.functional.interpolate(feat.view(H, W, feature_dim).permute(2, 0, 1).unsqueeze(0),
                                                  size=(H // 4, W // 4), mode="bilinear", align_corners=False)
            feature_loss = (low.squeeze(0).permute(1, 2, 0) - feature_target.float()).abs().mean()
            loss = (rgb - target).abs().mean() + 0.5 * feature_loss
        else:
            rgb, feature_loss = scene(ro, rd, score_threshold=thr, view_matrix=views[0], proj_matrix=proj,
                                      return_feature=True, feature_target=feature_target)
            loss = (rgb - target).abs().mean() + 0.5 * feature_loss
        loss.backward()
        opt.step()
        return loss

    steps, warmup = min(args.steps, 24), min(args.warmup, 4)
    wake_until = time.perf_counter() + args.wake_seconds     # untimed, as in the render loop of main()
    i = 0
    while time.perf_counter() < wake_until:
        step(i)
        i += 1
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        loss = step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    print(json.dumps({
        "metric": ("training_steps_per_sec_1200x680_200k_primitives" if not feature_dim else
                   f"feature_training_steps_per_sec_{args.workload}"), "value": round(steps / elapsed, 3),
        "unit": "steps/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(1000.0 * elapsed / steps, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "primitives": sc.n, "width": W, "height": H, "tile": 8, "threshold": thr,
                   "poses": len(frames), "loss": ("L1 against a fixed random image" if not feature_dim else
                            "L1 image loss + L1 of the dense feature image, resampled by torch, against a "
                            "quarter-resolution target" if args.dense_feature_loss else
                            "L1 image loss + streamed feature L1 against a quarter-resolution fp16 target"),
                   "feature_channels": feature_dim,
                   "mlp_gradient_precision": ("f32" if not feature_dim or args.dense_feature_loss else
                                                                               os.environ.get("MLPSP_CSR_MLP_PRECISION", "float16")),
                   "optimizer": "Adam (fused), all parameter tensors",
                   "entry": "NeuralPrimitiveSceneTileCUDA.forward + backward"},
        "final_loss": round(float(loss.detach()), 6)}))
    return 0


class Workload:
    """One of synthetic.CONFIGS on the device: the scene module, its camera frames and the call that renders one."""

    def __init__(self, name, precision, poses, dev):
        import numpy as np
        import torch

        from mlp_splatting_amd import ops, synthetic as syn
        from mlp_splatting_amd.cumodel import NeuralPrimitiveSceneTileCUDA

        self.name, self.dev = name, dev
        self.feature_dim = int(syn.CONFIGS[name]["feature_dim"])
        self.sc, self.cfg = syn.scene_for_config(name, with_features=False)
        sc, cfg = self.sc, self.cfg
        self.W, self.H, self.f, self.thr = cfg["width"], cfg["height"], cfg["focal"], cfg["threshold"]
        self.precision = precision if sc.hidden == 32 else "f32"   # the matrix-core render exists for the released width
        self.mosaic = name.startswith("cfg4")

        def t(a):
            return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

        scene = NeuralPrimitiveSceneTileCUDA(num_primitives=sc.n, hidden_dim=sc.hidden, feature_dim_low=self.feature_dim)
        scene.load_state_dict({"positions": torch.from_numpy(sc.positions), "log_scales": torch.from_numpy(sc.log_scales),
                               "quats": torch.from_numpy(sc.quats), "W1": torch.from_numpy(sc.W1),
                               "b1": torch.from_numpy(sc.b1), "W2": torch.from_numpy(sc.W2), "b2": torch.from_numpy(sc.b2),
                               "W3": torch.from_numpy(sc.W3), "b3": torch.from_numpy(sc.b3)}, strict=False)
        scene = scene.to(dev).eval()
        if self.feature_dim:
            # feat_attr [N,4,C] ~ N(0, 0.05), drawn on the device (1.6 GB at 200k x 4 x 512)
            gen = torch.Generator(device=dev)
            gen.manual_seed(0)
            with torch.no_grad():
                scene.feat_attr.copy_(torch.randn(scene.feat_attr.shape, device=dev, generator=gen) * 0.05)
        scene.set_image_size(self.W, self.H)
        scene.render_precision = self.precision
        self.scene = scene
        self.proj = t(syn.projection_matrix(self.f, self.W, self.H))
        cams = syn.random_poses(poses, 0)
        frames, self.skipped_poses = [], 0
        if self.mosaic:
            # four views of (W/2) x (H/2) per call; tile t renders view tile_view_ids[t]
            for g0 in range(0, len(cams) - 3, 4):
                ro, rd, tv, views = syn.mosaic_frame(self.W // 2, self.H // 2, self.f, cams[g0:g0 + 4])
                frames.append((t(ro), t(rd), t(views), t(tv)))
        else:
            for c2w in cams:
                ro, rd = syn.pinhole_rays(self.W, self.H, self.f, c2w)
                frames.append((t(ro), t(rd), t(syn.view_matrix(c2w))[None], None))
            # A pose whose fullest tile exceeds the 1,536-candidate capacity is an error of the path, not a frame
            # (the reference raises, and so does this build); the headline scene was constructed so that all 32 poses
            # fit, the literally specified smaller scenes were not.  Such poses are left out and counted.
            fitting = []
            with torch.no_grad():
                for frame in frames:
                    longest = ops.bin_legacy(scene.positions.detach(), scene.log_scales.detach(), frame[2].cpu(),
                                             self.proj.cpu(), self.W, self.H, int(scene.tile_size), self.thr, None,
                                             with_longest=True)[2]
                    if int(longest) <= scene._ensure_tile_ext().max_tile_prims:
                        fitting.append(frame)
            self.skipped_poses = len(frames) - len(fitting)
            frames = fitting
        self.frames = frames
        # the 4x4 view matrix a caller of forward() holds (one tensor per pose, made once)
        self.view_of = [None if f[3] is not None else f[2][0] for f in frames]

    def render(self, i):
        import torch
        ro, rd, views, tv = self.frames[i % len(self.frames)]
        scene = self.scene
        with torch.inference_mode():
            if tv is not None:
                cand, off = scene.build_tilecenter_culling_from_tile_views(tv, views, self.proj, self.thr)
                return scene(ro, rd, score_threshold=self.thr, culled_prim_indices=cand, tile_offsets=off)
            out = scene(ro, rd, score_threshold=self.thr, view_matrix=self.view_of[i % len(self.frames)],
                        proj_matrix=self.proj, return_feature=bool(self.feature_dim))
            return out[0] if self.feature_dim else out

    def timed(self, steps, warmup, wake_seconds, min_seconds):
        """-> (frames/s, seconds, frames timed).  Untimed first: `wake_seconds` of the same frames (a box whose GPU
        has idled while the scene was built on the host takes a few hundred milliseconds of work to reach its
        sustained clocks: the first process on a fresh box timed 1.5 ms per frame in this loop and 1.1 ms in the
        latency loop right after it; a second process 1.1 ms in both), then `warmup` frames.  The timed region is
        whole passes of `steps` frames until `min_seconds` have gone by."""
        import torch
        wake_until = time.perf_counter() + wake_seconds
        i = 0
        while time.perf_counter() < wake_until:
            self.render(i)
            i += 1
        for i in range(warmup):
            self.render(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        timed_steps = 0
        while True:
            for i in range(steps):
                self.render(timed_steps + i)
            timed_steps += steps
            # (checked on the host clock without a synchronisation: the queue is a few frames deep at most)
            if time.perf_counter() - t0 >= min_seconds:
                break
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        return timed_steps / elapsed, elapsed, timed_steps

    def timed_in_flight(self, in_flight, frames_per_call, min_seconds):
        """Frames per second through ``render_frames``: the same frames, `frames_per_call` cameras handed over per
        call and `in_flight` of them queued on the device at once (the images are those of ``render``; the tests
        compare them).  One untimed call, then whole calls for at least `min_seconds`.  None for a workload whose
        lists are handed in by the caller (the mosaic)."""
        import torch
        if self.mosaic:
            return None
        n = len(self.frames)
        feature = bool(self.feature_dim)

        def call(first):
            batch = [(self.frames[i % n][0], self.frames[i % n][1], self.view_of[i % n], self.proj)
                     for i in range(first, first + frames_per_call)]
            with torch.inference_mode():
                self.scene.render_frames(batch, self.thr, return_feature=feature, frames_in_flight=in_flight)
        call(0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = 0
        while time.perf_counter() - t0 < min_seconds:
            call(done)
            done += frames_per_call
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        return {"value": round(done / elapsed, 1), "unit": "frames/s", "ms_per_frame": round(elapsed / done * 1e3, 4),
                "frames_in_flight": in_flight, "frames_per_call": frames_per_call, "frames": done,
                "entry": "NeuralPrimitiveSceneTileCUDA.render_frames"}

    def probe_stages(self, n_probe=8):
        """The stages of a frame one by one, with HIP events on the launch stream around each as a frame queues it
        (no work counters and no read-back inside a bracket), and the render launch once more, untimed, for its
        work counters.  Means over the first `n_probe` frames -> dict."""
        import torch

        from mlp_splatting_amd import ops
        scene, dev, W, H, thr, precision = self.scene, self.dev, self.W, self.H, self.thr, self.precision
        freq, att = scene._frequency_tables(dev)
        quats = torch.nn.functional.normalize(scene.quats.detach(), dim=-1).contiguous()
        weights = [p.detach().contiguous() for p in (scene.W1, scene.b1, scene.W2, scene.b2, scene.W3, scene.b3)]
        packed = ops.pack_mfma_weights(*weights, bf16=True) if precision == "bf16" else None
        feat = scene.feat_attr.detach() if self.feature_dim and precision == "bf16" else None
        packed_feat = ops.pack_mfma_feat(feat)[0] if feat is not None else None
        n_probe = min(len(self.frames), n_probe)
        acc, held = {}, {}
        # two passes over the same poses: the first only warms the allocator (a first-time tensor size inside
        # the event brackets would be timed as kernel time), the second is measured
        for i in list(range(n_probe)) * 2:
            if i == 0:
                acc = dict(bin_ms=0.0, prologue_ms=0.0, sort_ms=0.0, render_ms=0.0, product_ms=0.0, hits=0, proc=0,
                           hit_waves=0, cand=0)
            ro, rd_raw, views, tv = self.frames[i]
            rd = torch.nn.functional.normalize(rd_raw, dim=-1).contiguous()
            e = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
            flags = torch.zeros(16, dtype=torch.int32, device=dev)     # (a queued frame finds its flag words clear)
            rec = ops.prepare_primitives(scene.positions.detach(), scene.log_scales.detach(), quats)
            cand, off = ops.bin_legacy(scene.positions.detach(), scene.log_scales.detach(), views, self.proj, W, H, 8, thr,
                                       tile_view_ids=tv)
            n_cand = int(cand.numel())
            # the binning as a frame queues it: no host synchronisation, candidate buffer sized beforehand
            # (a frame on the matrix cores takes its lists in per-tile segments: level 2 in one launch)
            segments = tv is None and precision == "bf16"
            ends = None
            e[0].record()
            if segments:
                # (the buffers handed on from frame to frame, as a queued frame of the scene module does)
                cand, off, ends, _ = ops.bin_segments_async(scene.positions.detach(), scene.log_scales.detach(), views[0],
                                                            self.proj, W, H, 8, thr, reuse=held)
            else:
                ops.bin_legacy_async(scene.positions.detach(), scene.log_scales.detach(), views, self.proj, W, H, 8, thr,
                                     cand.numel(), tile_view_ids=tv)
            e[1].record()
            pyramids = None
            if tv is None:
                # unit directions and the tiles' ray pyramids in one launch, as a frame of the scene module queues them
                # (lists handed in by a caller, the mosaic's, are rendered with torch's unit directions)
                rd, pyramids, _ = ops.frame_prologue(ro, rd_raw, W, H)
            e[2].record()
            order, _ = ops.sort_tiles(ro, rd, rec, cand, off, W, H, 8, 8, cull_threshold=thr, tile_pyramids=pyramids,
                                      tile_ends=ends, ids_ascend=tv is None)     # (as a queued frame sorts its own lists)
            e[3].record()
            counters = torch.zeros(4, dtype=torch.int64, device=dev)
            if feat is not None:
                # render with coefficient records, then the feature product, as two calls
                marks = {2: e[4], 3: e[5]}
                ops.render_tilecenter_mfma_feat(ro, rd, rec, order, off, freq, att, *weights, feat,
                                                float(scene.feature_gating_beta), float(scene.feature_gating_temp), W, H,
                                                thr, bf16=True, packed=packed, packed_feat=packed_feat, check=False,
                                                stages=lambda k: marks[k].record() if k in marks else None,
                                                tile_ends=ends)
            elif precision == "bf16":
                ops.render_tilecenter_mfma(ro, rd, rec, order, off, freq, att, *weights, W, H, thr, bf16=True,
                                           packed=packed, check=False, status=flags, status_is_clear=tv is None,
                                           tile_ends=ends)
                e[4].record()
            else:
                ops.render_tilecenter_f32(ro, rd, rec, order, off, freq, att, *weights, W, H, 8, 8, thr)
                e[4].record()
            torch.cuda.synchronize()
            # the same render launch once more, untimed, for its work counters (their atomics are not part of a frame)
            if precision == "bf16":
                ops.render_tilecenter_mfma(ro, rd, rec, order, off, freq, att, *weights, W, H, thr, bf16=True,
                                           counters=counters, packed=packed, tile_ends=ends)
            else:
                ops.render_tilecenter_f32(ro, rd, rec, order, off, freq, att, *weights, W, H, 8, 8, thr, counters=counters)
            torch.cuda.synchronize()
            acc["bin_ms"] += e[0].elapsed_time(e[1])
            acc["prologue_ms"] += e[1].elapsed_time(e[2])
            acc["sort_ms"] += e[2].elapsed_time(e[3])
            acc["render_ms"] += e[3].elapsed_time(e[4])
            if feat is not None:
                acc["product_ms"] += e[4].elapsed_time(e[5])
            c = counters.cpu().numpy()
            acc["hits"] += int(c[3])
            acc["proc"] += int(c[1])
            acc["hit_waves"] += int(c[2])
            acc["cand"] += n_cand
        out = {k: v / n_probe for k, v in acc.items()}
        out["n_probe"] = n_probe
        return out


def other_workload(name, args, dev):
    """A short leg of another configuration of the same scene family, outside the headline's timed region: one
    untimed pose cycle, then whole cycles for at least 0.25 s, and the per-launch figures of its dominant kernels
    (the reference's benchmark also reports RGB and RGB + feature in one run, tools/benchmark_inference.py:264-313)."""
    import gc

    import torch
    wl = Workload(name, "bf16", args.poses, dev)
    if not wl.frames:
        return {"skipped": "every pose exceeds the tile candidate capacity"}
    cycle = len(wl.frames)
    fps, elapsed, steps = wl.timed(cycle, cycle, 0.0, 0.25)
    st = wl.probe_stages(min(4, cycle))
    flops_per_hit = 2 * (72 * 32 + 32 * 32 + 4 * 32)
    render_s = st["render_ms"] * 1e-3
    tflops = flops_per_hit * st["hits"] / render_s / 1e12
    kernel = "render_tilecenter_mfma"
    traffic, note = measured_traffic(kernel, name, st["render_ms"])
    out = {"fps": round(fps, 2), "ms_per_step": round(1e3 * elapsed / steps, 4), "steps": steps, "dtype": wl.precision,
           "views_per_call": 4 if wl.mosaic else 1, "feature_channels": wl.feature_dim, "poses": cycle,
           "stages": {k: round(st[k], 4) for k in ("bin_ms", "prologue_ms", "sort_ms", "render_ms") +
                      (("product_ms",) if wl.feature_dim else ())},
           "hits_per_launch": int(st["hits"]), "hit_wavefronts_per_launch": int(st["hit_waves"])}
    if not wl.mosaic and not args.no_frames_in_flight:
        out["two_frames_in_flight"] = wl.timed_in_flight(2, 8 if wl.feature_dim else cycle, 0.25)
    if wl.mosaic:
        # 17 of a tile's 64 pixels hit per step here: the launch is bound by the weight blocks it streams, one
        # 7,808-byte block per (tile, primitive) that hits, plus 40 bytes per pixel
        bytes_alg = 7808.0 * st["hit_waves"] + 40.0 * wl.W * wl.H
        gbs = bytes_alg / render_s / 1e9
        out["roofline"] = {"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(gbs / HBM_PEAK_GBS, 5), "traffic": traffic, "traffic_source": note,
                           "ms_per_launch": round(st["render_ms"], 4), "mfma_tflops": round(tflops, 1),
                           "mfma_frac": round(tflops / PEAK["bf16"], 5)}
    else:
        out["roofline"] = {"kernel": kernel, "bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK["bf16"],
                           "unit": "TFLOP/s", "frac": round(tflops / PEAK["bf16"], 5), "traffic": traffic,
                           "traffic_source": note, "ms_per_launch": round(st["render_ms"], 4)}
    if wl.feature_dim:
        # feature product: the f32 image written once + the fp16 coefficient records (64 pixels x 8 bytes per hit step)
        bytes_alg = 4.0 * wl.W * wl.H * wl.feature_dim + 512.0 * st["hit_waves"]
        gbs = bytes_alg / (st["product_ms"] * 1e-3) / 1e9
        ptraffic, pnote = measured_traffic("feat_gemm", name, st["product_ms"])
        out["feature_product"] = {"kernel": "feat_gemm", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                                  "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 5), "traffic": ptraffic,
                                  "traffic_source": pnote, "ms_per_launch": round(st["product_ms"], 4)}
    del wl
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=96)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--workload", default="cfg3_200k_1200x680")
    ap.add_argument("--precision", choices=["f32", "bf16"], default=None,
                    help="MLP arithmetic of the render kernel (default: bf16 matrix cores when built, else f32)")
    ap.add_argument("--poses", type=int, default=32)
    ap.add_argument("--dense-feature-loss", action="store_true",
                    help="with --train on a feature workload: the dense feature image under autograd (the reference's "
                         "legacy training backend) instead of the record-based streamed loss")
    ap.add_argument("--train", action="store_true",
                    help="time full training steps instead (f32 render with autograd, L1 image loss, backward through "
                         "the record pipeline, Adam on all nine parameter tensors); prints its own JSON line")
    ap.add_argument("--wake-seconds", type=float, default=1.0,
                    help="untimed rendering before the warm-up steps, to bring an idle GPU to its sustained clocks")
    ap.add_argument("--min-seconds", type=float, default=0.5,
                    help="the timed region is extended, in whole passes of --steps, until it lasts at least this long; "
                         "the JSON line reports the steps actually timed")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short legs of the feature (cfg5) and mosaic (cfg4) configurations that the default "
                         "run of the headline workload appends under other_workloads")
    ap.add_argument("--no-frames-in-flight", action="store_true",
                    help="skip the leg that renders the same frames with two in flight (render_frames): under a kernel "
                         "trace its overlapping launches would blur the per-kernel durations")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run 4 plain device copies of 1 GiB, the known-size kernel that hardware counter "
                         "readings of a profiled run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (each GPU box has one GPU); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from mlp_splatting_amd import _lib, ops

    _lib.load()
    dev = torch.device("cuda", int(os.environ.get("LOCAL_RANK", "0")))
    torch.cuda.set_device(dev)
    precision = args.precision or ("bf16" if hasattr(ops, "render_tilecenter_mfma") else "f32")

    wl = Workload(args.workload, precision, args.poses, dev)
    if precision == "bf16" and wl.precision != "bf16":
        if args.precision == "bf16":
            print(f"--precision bf16 needs the 72->32->32->4 MLP; {args.workload} has hidden width {wl.sc.hidden}", file=sys.stderr)
            return 2
        precision = "f32"
    sc, cfg, scene, frames, proj = wl.sc, wl.cfg, wl.scene, wl.frames, wl.proj
    W, H, thr, feature_dim, mosaic, skipped_poses = wl.W, wl.H, wl.thr, wl.feature_dim, wl.mosaic, wl.skipped_poses
    if not frames:
        print(f"{args.workload}: every pose exceeds the tile candidate capacity", file=sys.stderr)
        return 2

    if args.train:
        return train_steps(args, scene, frames, proj, thr, W, H, sc, dev)

    render = wl.render
    fps, elapsed, timed_steps = wl.timed(args.steps, args.warmup, args.wake_seconds, args.min_seconds)

    # per-frame latency distribution, the way tools/benchmark_inference.py:121-149 times a frame: a
    # synchronise on both sides of every call (so nothing overlaps between frames, unlike the loop above)
    lat = []
    for i in range(min(args.steps, 3 * len(frames))):
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        render(i)
        torch.cuda.synchronize()
        lat.append((time.perf_counter() - t1) * 1e3)
    from mlp_splatting_amd.harness import timing_stats
    latency = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in timing_stats(lat).items()}
    latency["frames"] = latency.pop("samples")

    # ---- the same frames with two in flight (frame k+1 queued on a second stream before the host waits for frame k):
    # reported beside the headline, which stays the frame-after-frame call of the reference's interface
    in_flight = None
    if precision == "bf16" and not args.no_frames_in_flight:
        # (a feature frame's result holds a 1.67 GB image: eight cameras per call there)
        in_flight = wl.timed_in_flight(2, 8 if feature_dim else len(frames), args.min_seconds)

    # ---- the stages of a frame alone: HIP events on the stream they are launched on, and the render's work counters
    st = wl.probe_stages(8)
    n_probe = st["n_probe"]
    kernel_ms, sort_ms, bin_ms = st["render_ms"] * n_probe, st["sort_ms"] * n_probe, st["bin_ms"] * n_probe
    hits, proc, hit_waves, cand_total = (int(st[k] * n_probe) for k in ("hits", "proc", "hit_waves", "cand"))
    freq, att = scene._frequency_tables(dev)
    quats = torch.nn.functional.normalize(scene.quats.detach(), dim=-1).contiguous()
    # what the matrix cores sustain on this box with nothing else in the way
    mfma_probe = None
    if precision == "bf16":
        sink = torch.zeros(1, device=dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        lib = _lib.load()
        stream = torch.cuda.current_stream(dev).cuda_stream
        lib.mlpsp_probe_mfma_bf16(200, sink.data_ptr(), stream)
        e0.record()
        probe_flops = lib.mlpsp_probe_mfma_bf16(4000, sink.data_ptr(), stream)
        e1.record()
        torch.cuda.synchronize()
        mfma_probe = round(probe_flops / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
    # how matrix-core, vector and transcendental instructions share a SIMD's issue time at the render kernel's
    # occupancy (four wavefronts per SIMD): core clocks per instruction and SIMD for each mix (mlpsp_probe_issue)
    import ctypes
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    sink = torch.zeros(1, device=dev)
    probe_out = torch.zeros(4096 * 3, dtype=torch.int64, device=dev)
    per_batch = {1: ("mfma", 16), 2: ("valu", 128), 3: ("trans", 128), 4: ("mfma", 16)}

    def issue(roles):
        arr = (ctypes.c_int32 * 4)(*roles)
        lib.mlpsp_probe_issue(arr, 1500, probe_out.data_ptr(), sink.data_ptr(), stream)
        torch.cuda.synchronize()
        rec = probe_out.cpu().numpy().reshape(4096, 3)
        role_of = (rec[:, 2] & 0xffffffff).astype(int)
        out_clk = {}
        for role in sorted(set(roles) - {0}):
            sel = role_of == role
            clocks_per_batch_simd = rec[sel, 1].mean() / (rec[sel, 0].mean() * roles.count(role))
            out_clk[role] = clocks_per_batch_simd / per_batch[role][1]
        return out_clk
    issue((1, 1, 1, 1))                                         # (clock ramp)
    alone = {**issue((1, 1, 1, 1)), **issue((2, 2, 2, 2)), **issue((3, 3, 3, 3))}
    mixed_wave = issue((4, 4, 4, 4))[4]                         # clocks per (MFMA + 8 FMA), every wavefront doing both
    across = issue((1, 2, 1, 2))                                # two MFMA wavefronts and two FMA wavefronts per SIMD
    issue_probe = {"waves_per_simd": 4,
                   "clk_per_mfma_32x32x16": round(alone[1], 2), "clk_per_valu_fma": round(alone[2], 2),
                   "clk_per_transcendental": round(alone[3], 2),
                   "same_wave_mfma_plus_8_fma_clk": round(mixed_wave, 2),
                   "same_wave_if_serial_clk": round(alone[1] + 8 * alone[2], 2),
                   "across_waves_clk_per_mfma": round(across[1], 2), "across_waves_clk_per_fma": round(across[2], 2),
                   "across_waves_fma_issued_per_mfma": round(across[1] / across[2], 2)}
    flops_per_hit = 2 * (72 * sc.hidden + sc.hidden * sc.hidden + 4 * sc.hidden)
    achieved_tflops = flops_per_hit * hits / (kernel_ms * 1e-3) / 1e12
    # sort kernel: 8 compulsory bytes per candidate (4 id in, 4 id out) + the 64-byte record of every primitive
    # once (the per-candidate geometry gathers are served by L2)
    sort_gbs = (8.0 * cand_total + 64.0 * sc.n * n_probe) / (sort_ms * 1e-3) / 1e9
    # binning: 24 bytes per primitive in, 4 per candidate and per tile out
    T_tiles = ((W + 7) // 8) * ((H + 7) // 8)
    bin_gbs = (24.0 * sc.n * n_probe + 4.0 * cand_total + 4.0 * (T_tiles + 1) * n_probe) / (bin_ms * 1e-3) / 1e9

    render_kernel = "render_tilecenter_" + ("mfma" if precision == "bf16" else "f32")
    traffic, traffic_note = measured_traffic(render_kernel, args.workload, kernel_ms / n_probe)
    sort_traffic, sort_note = measured_traffic("sort_tiles", args.workload, sort_ms / n_probe)
    # the sort by the accounting of the hot-path scope table: 4 B id in + 40 B gathered geometry + 4 B id out per
    # candidate (next to the kernel's own compulsory bytes above, in which every 64-byte record counts once)
    sort_gbs_per_candidate = 48.0 * cand_total / (sort_ms * 1e-3) / 1e9
    out = {
        "metric": ("forward_render_frames_per_sec_1200x680_200k_primitives" if args.workload.startswith("cfg3")
                   else f"forward_render_frames_per_sec_{args.workload}"),
        "value": round(fps, 3), "unit": "frames/s", "n_gpus": 1, "steps": timed_steps, "warmup": args.warmup,
        "wake_seconds": args.wake_seconds, "steps_per_pass": args.steps, "min_seconds": args.min_seconds,
        "ms_per_step": round(1000.0 * elapsed / timed_steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": precision, "data": "synthetic",
        "config": {"workload": args.workload, "primitives": sc.n, "width": W, "height": H, "tile": 8,
                   "threshold": thr, "poses": len(frames), "poses_over_capacity_left_out": skipped_poses,
                   "log_scale_mean": cfg["log_scale_mean"],
                   "mlp": f"72-{sc.hidden}-{sc.hidden}-4", "feature_channels": feature_dim,
                   "views_per_call": 4 if mosaic else 1, "entry": "NeuralPrimitiveSceneTileCUDA.forward"},
        "mpix_per_sec": round(fps * W * H / 1e6, 2), "latency": latency, "two_frames_in_flight": in_flight,
        "roofline": {"bound": "mfma", "kernel": "render_tilecenter_" + ("mfma" if precision == "bf16" else "f32"),
                     "achieved": round(achieved_tflops, 3), "peak": PEAK[precision], "unit": "TFLOP/s",
                     "frac": round(achieved_tflops / PEAK[precision], 5),
                     "traffic": traffic, "traffic_source": traffic_note,
                     "ms_per_launch": round(kernel_ms / n_probe, 4), "hits_per_launch": hits // n_probe,
                     "tile_primitives_per_launch": proc // n_probe,
                     "hit_wavefronts_per_launch": hit_waves // n_probe, "flops_per_hit": flops_per_hit,
                     "measured_mfma_peak": mfma_probe, "issue_probe": issue_probe},
        "stages": {"bin_ms": round(bin_ms / n_probe, 4), "prologue_ms": round(st["prologue_ms"], 4),
                   "sort_ms": round(sort_ms / n_probe, 4), "render_ms": round(kernel_ms / n_probe, 4),
                   "sort_hbm": {"bound": "hbm", "achieved": round(sort_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": round(sort_gbs / HBM_PEAK_GBS, 5),
                                "achieved_at_48B_per_candidate": round(sort_gbs_per_candidate, 1),
                                "frac_at_48B_per_candidate": round(sort_gbs_per_candidate / HBM_PEAK_GBS, 5),
                                "traffic": sort_traffic, "traffic_source": sort_note},
                   "bin_hbm": {"bound": "hbm", "achieved": round(bin_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                               "frac": round(bin_gbs / HBM_PEAK_GBS, 5)},
                   "candidates_per_launch": cand_total // n_probe},
    }

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if not args.no_cpu_baseline:
        # the CPU restatement of the same algorithm, on this host's cores: full frames of pose 0, median of the runs
        import oracle
        ro, rd_raw, views, tv = frames[0]
        rd = torch.nn.functional.normalize(rd_raw, dim=-1).cpu().numpy()
        ro_np = ro.cpu().numpy()
        fkw = {}
        if feature_dim:            # (the 1.6 GB attribute download is not part of the CPU figure)
            fkw = dict(feat_attr=scene.feat_attr.detach().cpu().numpy(), beta=float(scene.feature_gating_beta),
                       temp=float(scene.feature_gating_temp))
        views_np, proj_np = views.cpu().numpy(), proj.cpu().numpy()
        tv_np = None if tv is None else tv.cpu().numpy()
        runs, budget_s, res = [], 30.0, None
        while len(runs) < 3 and (not runs or sum(runs) + runs[-1] <= budget_s):
            tc = time.perf_counter()
            cand, off = oracle.bin_legacy(sc.positions, sc.log_scales, views_np, proj_np, W, H, 8, thr, tile_view_ids=tv_np)
            res = oracle.render_tilecenter(ro_np, rd, sc.positions, sc.log_scales, quats.cpu().numpy(), cand, off,
                                           freq.cpu().numpy(), att.cpu().numpy(), *sc.mlp(), W, H, 8, 8, thr, **fkw)
            runs.append(time.perf_counter() - tc)
        cpu_s = float(np.median(runs))
        gpu_rgb = render(0).cpu().numpy()
        out["cpu_baseline"] = {"value": round(1.0 / cpu_s, 4), "unit": "frames/s", "cores": oracle.num_threads(),
                               "kind": "port",
                               "sample": f"median of {len(runs)} full frame(s) (pose 0) of the same workload: binning + "
                               "per-tile sort + f32 render" + (" with the feature channel" if feature_dim else "") +
                               ", OpenMP over tiles",
                               "ms_per_frame": round(cpu_s * 1e3, 1), "runs_ms": [round(r * 1e3, 1) for r in runs],
                               "gpu_vs_cpu_image_max_abs": float(np.abs(gpu_rgb - res["rgb"]).max())}
        if sc.n * T_tiles <= 300_000_000 and tv is None:
            # the reference's own culling expression (dense [tiles x primitives] booleans), once, with CPU torch:
            # the part of its path that is PyTorch and therefore runs on a CPU at all
            torch.set_num_threads(oracle.num_threads())
            dense_s, dense_pairs = dense_culling_cpu_torch(torch.from_numpy(sc.positions), torch.from_numpy(sc.log_scales),
                                                           torch.from_numpy(views_np[0]), torch.from_numpy(proj_np), W, H,
                                                           8, thr)
            out["cpu_baseline"]["reference_culling"] = {
                "kind": "reference culling expression, CPU torch", "ms": round(dense_s * 1e3, 1), "pairs": dense_pairs,
                "pairs_of_this_build": int(cand.size), "threads": torch.get_num_threads(),
                "sample": "one evaluation of scannet/cumodel.py:994-1070 restated with torch on the CPU (dense overlap "
                          "matrix, nonzero, argsort, offsets), pose 0"}
        else:
            out["cpu_baseline"]["reference_culling"] = {
                "kind": "reference culling expression, CPU torch", "ms": None,
                "skipped": (f"tiles x primitives = {sc.n * T_tiles:.3g}: the dense overlap matrix is timed only up to 3e8 "
                            "elements and for one view (run --workload cfg1_5k_160x120 or cfg2_50k_640x480)")}
    # ---- short legs of the feature and the mosaic configuration (the headline fields above are not touched)
    if args.workload.startswith("cfg3") and precision == "bf16" and not args.no_other_workloads:
        del wl, scene, frames, render
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        out["other_workloads"] = {name: other_workload(name, args, dev)
                                  for name in ("cfg5_200k_feat512", "cfg4_200k_mosaic4")}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
