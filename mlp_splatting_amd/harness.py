"""What the reference's evaluation and benchmark scripts do around a render call, for callers that do not go
through those scripts (scannet/eval_rgb_psnr.py:443-493, tools/benchmark_inference.py:85-149, 287-311): one timed
view, the statistics of a series of timings, PSNR per view and over all views, and the check that the render with
the feature channel produces the RGB of the render without it."""
from __future__ import annotations

import math
import time

import numpy as np
import torch


def timing_stats(values_ms):
    """mean / median / 95th percentile / sample standard deviation / coefficient of variation / rates
    (tools/benchmark_inference.py:85-99: ``std`` with ddof = 1, zero for a single sample)."""
    samples = np.asarray(list(values_ms), dtype=np.float64)
    if samples.size == 0:
        raise ValueError("timing_stats needs at least one sample")
    mean, median = float(samples.mean()), float(np.median(samples))
    std = float(samples.std(ddof=1)) if samples.size > 1 else 0.0
    return {"samples": int(samples.size), "mean_ms": mean, "median_ms": median,
            "p95_ms": float(np.percentile(samples, 95)), "std_ms": std,
            "coefficient_of_variation": std / mean if mean else 0.0,
            "fps_from_mean": 1000.0 / mean if mean else float("inf"),
            "fps_from_median": 1000.0 / median if median else float("inf")}


def quality(predictions, targets):
    """PSNR of images in [0, 1]: per view, their mean and median, and the PSNR of the error pooled over all views
    (tools/benchmark_inference.py:102-118); a view that matches exactly counts as +inf."""
    predictions, targets = list(predictions), list(targets)
    if len(predictions) != len(targets) or not predictions:
        raise ValueError("quality needs as many predictions as targets, and at least one")
    per_view, squared_sum, values = [], 0.0, 0
    for prediction, target in zip(predictions, targets):
        squared = (prediction.double() - target.double()).square()
        mse = float(squared.mean())
        per_view.append(-10.0 * math.log10(mse) if mse else float("inf"))
        squared_sum += float(squared.sum())
        values += squared.numel()
    pooled = squared_sum / values
    return {"mean_psnr_db": float(np.mean(per_view)), "median_psnr_db": float(np.median(per_view)),
            "global_psnr_db": -10.0 * math.log10(pooled) if pooled else float("inf"), "per_view_psnr_db": per_view}


def render_view(scene, rays_o, rays_d, view_matrix, proj_matrix, width, height, threshold, return_feature=False):
    """One view the way the reference's harness renders and times it (tools/benchmark_inference.py:121-149):
    ``set_image_size``, a synchronise on both sides, an event pair and the wall clock around the call under
    ``torch.inference_mode()`` -> (rgb [H, W, 3] clamped to [0, 1], wall ms, device ms, feature shape or None)."""
    scene.set_image_size(int(width), int(height))
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    wall = time.perf_counter()
    start.record()
    with torch.inference_mode():
        out = scene(rays_o, rays_d, score_threshold=threshold, view_matrix=view_matrix, proj_matrix=proj_matrix,
                    return_feature=return_feature)
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall) * 1000.0
    feature_shape = None
    if return_feature:
        out, feature = out
        feature_shape = list(feature.shape)
        del feature
    return out.view(int(height), int(width), 3).clamp(0.0, 1.0), wall_ms, float(start.elapsed_time(end)), feature_shape


def rgb_parity_with_features(scene, rays_o, rays_d, view_matrix, proj_matrix, width, height, threshold):
    """Largest absolute difference between the RGB of the render with the feature channel and of the render
    without it (the parity block of tools/benchmark_inference.py:287-311)."""
    plain = render_view(scene, rays_o, rays_d, view_matrix, proj_matrix, width, height, threshold, False)[0]
    joint = render_view(scene, rays_o, rays_d, view_matrix, proj_matrix, width, height, threshold, True)[0]
    return float((plain - joint).abs().max())
