"""The workload the headline figure is quoted on, built in one place so that the benchmark and the parity test
that checks it run the same model on the same frame.

BASELINE configuration 3: int8 CenterPoint-shaped backbone, seeded synthetic 250 k-point frame; per-channel
weight ranges from the seeded fp16 weights; per-tensor activation ranges = the 99.99th percentile of
|activation| over 4 seeded calibration frames (seeds 101 .. 104), the activations taken from the fp16 HIP engine.
"""
from __future__ import annotations

import zlib
from typing import Callable, Sequence, Tuple

import numpy as np

from . import graphs, synth
from .calibrate import calibrate_amax, gpu_runner

GRID_ZYX = (41, 1440, 1440)
FRAME_SEED = 0
CALIBRATION_SEEDS = (101, 102, 103, 104)
OUTPUT_BOUND = 400000    # above every stage of the synthetic frame (322,224 rows at most): nothing is truncated

Voxelizer = Callable[[np.ndarray], Tuple[np.ndarray, np.ndarray]]   # points -> (features fp16 [N,5], indices zyx [N,4])


def headline_points(n_points: int = 250000) -> np.ndarray:
    return synth.lidar_frame(seed=FRAME_SEED, n_points=n_points)


def headline_model(precision: str, voxelize: Voxelizer, output_bound: int = OUTPUT_BOUND, n_points: int = 250000,
                   calibration_frames: Sequence[Tuple[np.ndarray, np.ndarray]] = ()):
    """The CenterPoint-shaped graph (seed 0); for int8 annotated with the CenterPoint exporter's precision plan and
    ranges calibrated on the four seeded frames (or on calibration_frames when given)."""
    graph, tags = graphs.centerpoint_scn(seed=0, output_bound=output_bound)
    if precision == "int8":
        frames = list(calibration_frames) or [voxelize(synth.lidar_frame(seed=s, n_points=n_points))
                                              for s in CALIBRATION_SEEDS]
        amax = calibrate_amax(graph, frames, GRID_ZYX, gpu_runner)
        graphs.apply_int8_plan(graph, tags, amax, "centerpoint")
    return graph


def bev_checksum(bev: np.ndarray) -> int:
    """CRC-32 of the dense output's bytes: equal checksums = the same bits."""
    return int(zlib.crc32(np.ascontiguousarray(bev).view(np.uint8).tobytes()))
