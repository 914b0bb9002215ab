"""Copies the reference's own input DATA files into small compressed fixtures.

Only data is read (no reference code is imported or executed):
  libraries/3DSparseConvolution/workspace/centerpoint/in_features.torch.fp16.tensor   79,745 x 5 fp16
  libraries/3DSparseConvolution/workspace/centerpoint/in_indices_zyx.torch.int32.tensor 79,745 x 4 int32
  libraries/3DSparseConvolution/workspace/bevfusion/infer.xyz.{voxels,coors}          17,748 voxels
  libraries/3DSparseConvolution/workspace/ff9eff4389a740848f9a56ad749a4ae8.bin        271,156 x 5 fp16 points
Run from the repository root: python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
from lidar_ai_solution_amd import tensor  # noqa: E402

W = "/root/reference/libraries/3DSparseConvolution/workspace/"
OUT = os.path.dirname(os.path.abspath(__file__))

feat = tensor.load(W + "centerpoint/in_features.torch.fp16.tensor")
idx = tensor.load(W + "centerpoint/in_indices_zyx.torch.int32.tensor")
np.savez_compressed(os.path.join(OUT, "centerpoint_input.npz"), features=feat, indices_zyx=idx)

bf = tensor.load(W + "bevfusion/infer.xyz.voxels")
bc = tensor.load(W + "bevfusion/infer.xyz.coors")
np.savez_compressed(os.path.join(OUT, "bevfusion_input.npz"), features=bf, indices_xyz=bc)

pts = np.fromfile(W + "ff9eff4389a740848f9a56ad749a4ae8.bin", dtype=np.float16).reshape(-1, 5)
np.savez_compressed(os.path.join(OUT, "nuscenes_frame.npz"), points=pts)
print(feat.shape, idx.shape, bf.shape, bc.shape, pts.shape)
