"""Host-side Python mirror of the reference's SCN interfaces, over the C ABI of libscn_hip.so.

  Engine            spconv::Engine + load_engine_from_onnx + EngineBuilder
                    (`libspconv/include/spconv/engine.hpp:55-167`, `src/onnx-parser.hpp:32-40`)
  SCNModel          pyscn.SCNModel(onnx, precision).forward(features, indices, grid, stream)
                    (`libraries/3DSparseConvolution/src/pyscn.cpp:47-140`)
  Voxelization      bevfusion::lidar::Voxelization (`CUDA-BEVFusion/src/bevfusion/lidar-voxelization.hpp:42-72`)
  LidarSCN          bevfusion::lidar::SCN: points -> voxelize -> engine -> BEV tensor
                    (`CUDA-BEVFusion/src/bevfusion/lidar-scn.cpp:34-50`)

PyTorch is used only to own device memory and streams.  There is no CPU path: every call goes to
the HIP library and fails loudly when it is missing.
"""
from __future__ import annotations

import ctypes as C
import os
import tempfile
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import capi
from .onnx_dialect import Graph, save as save_onnx

PRECISION = {"fp16": capi.PRECISION_FP16, "float16": capi.PRECISION_FP16, "int8": capi.PRECISION_INT8}


def _stream_ptr(stream) -> C.c_void_p:
    if stream is None:
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if hasattr(stream, "cuda_stream"):
        return C.c_void_p(stream.cuda_stream)
    return C.c_void_p(int(stream))


def _prec(p) -> int:
    return PRECISION[p.lower()] if isinstance(p, str) else int(p)


class TensorView:
    """A device tensor owned by the engine (valid until the next forward / engine destruction)."""

    def __init__(self, v: capi.TensorView):
        self.name = v.name.decode() if v.name else ""
        self.ptr = v.features_dev
        self.dtype = v.dtype
        self.shape = [int(v.shape[i]) for i in range(v.ndim)]
        self.indices_ptr = v.indices_dev
        self.num_ptr = v.num_dev
        self.grid_size = [int(x) for x in v.grid_size]
        self.dynamic_range = float(v.dynamic_range)  # int8 tensors: amax; value = q * (amax / 127)
        self.scale = float(np.float32(v.dynamic_range) / np.float32(127.0))
        self.dense = v.indices_dev is None

    def _copy(self, ptr, shape, tdtype):
        import torch
        out = torch.empty(shape, dtype=tdtype, device="cuda")
        if out.numel():
            torch.cuda.synchronize()
            hip = capi.hip_runtime()
            hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
            rc = hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(ptr), out.numel() * out.element_size(), 3)
            if rc != 0:
                raise RuntimeError(f"hipMemcpy failed ({rc})")
        return out

    def num_rows(self) -> int:
        import torch
        if self.dense:
            return self.shape[0]
        return int(self._copy(self.num_ptr, (1,), torch.int32).cpu().numpy().view(np.uint32)[0])

    def torch(self):
        """A copy as a torch tensor: dense -> its shape; sparse -> (features [n, ld], indices [n, 4])."""
        import torch
        tdt = {capi.DTYPE_FP16: torch.float16, capi.DTYPE_INT8: torch.int8, capi.DTYPE_FP32: torch.float32,
               capi.DTYPE_INT32: torch.int32}[self.dtype]
        if self.dense:
            return self._copy(self.ptr, self.shape, tdt)
        n = self.num_rows()
        feats = self._copy(self.ptr, (n, self.shape[1]), tdt)
        idx = self._copy(self.indices_ptr, (n, 4), torch.int32)
        return feats, idx


class Engine:
    """An SCN engine built from an ONNX file, or from an in-memory Graph through the builder calls."""

    def __init__(self, handle):
        if not handle:
            raise RuntimeError("engine creation failed: " + capi.lib().scn_last_error().decode())
        self._h = handle
        self._keep = None

    @classmethod
    def from_onnx(cls, path: str, precision="fp16", sortmask=False, enable_blackwell=False, with_auxiliary_stream=False,
                  fixed_launch_points: int = 10000, stream=None, keep_all: bool = False,
                  precision_overrides=(), tensor_ranges=None, tile_plans: bool = False) -> "Engine":
        """spconv::load_engine_from_onnx.  Raises instead of returning nullptr on failure.

        precision_overrides: (selector, by_optype, precision, output_precision) tuples applied to the
        nodes' precisions before the engine is planned -- the older interface's set_node_precision_byname /
        set_node_precision_byoptype + reconfigure; precision None leaves the model's value.
        tensor_ranges: {tensor name: calibrated |max|} (see collect_amax); replaces the dynamic ranges of the
        model's convolutions and Adds.
        sortmask is the reference's hint (the engine re-orders rows only where that is faster: at present nowhere);
        tile_plans runs every narrow layer on a sorted tile plan regardless."""
        flags = (capi.BUILD_SORTMASK if sortmask else 0) | (capi.BUILD_AUX_STREAM if with_auxiliary_stream else 0) | \
                (capi.BUILD_KEEP_ALL if keep_all else 0) | (capi.BUILD_TILE_PLANS if tile_plans else 0)
        n = len(precision_overrides)
        arr = (capi.PrecisionOverride * max(n, 1))()
        for i, (sel, by_optype, prec, out_prec) in enumerate(precision_overrides):
            arr[i].selector = sel.encode()
            arr[i].by_optype = int(bool(by_optype))
            arr[i].precision = _prec(prec) if prec is not None else 0
            arr[i].output_precision = _prec(out_prec) if out_prec is not None else 0
        ranges = list((tensor_ranges or {}).items())
        rarr = (capi.TensorAmax * max(len(ranges), 1))()
        for i, (name, amax) in enumerate(ranges):
            rarr[i].tensor = name.encode()
            rarr[i].amax = float(amax)
        opt = capi.LoadOptions(C.cast(arr, C.c_void_p) if n else None, n,
                               C.cast(rarr, C.c_void_p) if ranges else None, len(ranges))
        h = capi.lib().scn_engine_create_from_onnx_ex(path.encode(), _prec(precision), flags, fixed_launch_points,
                                                      C.byref(opt), _stream_ptr(stream) if stream is not None else None)
        return cls(h)

    @classmethod
    def from_graph(cls, graph: Graph, precision="fp16", keep_all: bool = False,
                   with_auxiliary_stream: bool = False, sortmask: bool = False, tile_plans: bool = False) -> "Engine":
        """Drives the EngineBuilder calls (push_input / push_sparse_conv / ... / build) node by node,
        the way `onnx-parser.cpp:116-230` does."""
        L = capi.lib()
        b = L.scn_builder_create()
        try:
            tmap: Dict[str, int] = {}
            for name in graph.inputs:
                tmap[name] = L.scn_builder_push_input(b, name.encode())
            for n in graph.nodes:
                a = n.attrs
                pr = lambda key: capi.PRECISION_INT8 if a.get(key, "") == "int8" else capi.PRECISION_FP16  # noqa: E731
                if n.op_type == "SparseConvolution":
                    w = np.ascontiguousarray(graph.initializers[n.inputs[1]], np.float16)
                    bias = np.ascontiguousarray(graph.initializers[n.inputs[2]], np.float16)
                    wr = np.ascontiguousarray(a.get("weight_dynamic_ranges", []), np.float32)
                    out = L.scn_builder_push_sparse_conv(
                        b, n.name.encode(), tmap[n.inputs[0]], w.ctypes.data_as(C.c_void_p), capi.i5(*w.shape),
                        wr.ctypes.data_as(C.c_void_p) if wr.size else None, int(wr.size),
                        bias.ctypes.data_as(C.c_void_p), int(bias.size), str(a.get("activation", "")).encode(),
                        capi.i3(*a["kernel_size"]), capi.i3(*a.get("stride", [1, 1, 1])),
                        capi.i3(*a.get("padding", [0, 0, 0])), capi.i3(*a.get("dilation", [1, 1, 1])),
                        float(a.get("input_dynamic_range", 0.0)), int(a.get("subm", 0)),
                        int(a.get("output_bound", 150000)), 10000, str(a.get("rulebook", "")).encode(),
                        pr("precision"), pr("output_precision"), n.outputs[0].encode(), int(a.get("inverse", 0)))
                elif n.op_type in ("Add", "QuantAdd"):
                    out = L.scn_builder_push_add(b, n.name.encode(), tmap[n.inputs[0]], tmap[n.inputs[1]],
                                                 float(a.get("input0_dynamic_range", 0.0)),
                                                 float(a.get("input1_dynamic_range", 0.0)), n.outputs[0].encode(),
                                                 pr("precision"), pr("output_precision"), 10000)
                elif n.op_type == "Relu":
                    out = L.scn_builder_push_relu(b, n.name.encode(), tmap[n.inputs[0]], n.outputs[0].encode())
                elif n.op_type == "ScatterDense":
                    oshape = (C.c_int * len(a["output_shape"]))(*[int(v) for v in a["output_shape"]])
                    layout = {"NCHW32": 2, "NHWzC": 3}.get(a.get("output_layout", ""), 1)
                    out = L.scn_builder_push_dense(b, n.name.encode(), tmap[n.inputs[0]], str(a.get("format", "")).encode(),
                                                   n.outputs[0].encode(), capi.i3(*a["input_spatial_shape"]), oshape,
                                                   len(a["output_shape"]), layout, float(a.get("input_dynamic_range", 0.0)), 0)
                elif n.op_type in ("Reshape", "Transpose"):
                    dims = (C.c_int64 * len(a["dims"]))(*[int(v) for v in a["dims"]])
                    fn = L.scn_builder_push_reshape if n.op_type == "Reshape" else L.scn_builder_push_transpose
                    out = fn(b, n.name.encode(), tmap[n.inputs[0]], dims, len(a["dims"]), n.outputs[0].encode())
                else:
                    raise RuntimeError(f"Unsupport operator [{n.op_type}]")
                if out < 0:
                    raise RuntimeError(f"builder rejected node {n.name}: " + L.scn_last_error().decode())
                tmap[n.outputs[0]] = out
            for name in graph.outputs:
                capi.check(L.scn_builder_push_output(b, tmap[name]))
            flags = (capi.BUILD_KEEP_ALL if keep_all else 0) | (capi.BUILD_AUX_STREAM if with_auxiliary_stream else 0) | \
                    (capi.BUILD_SORTMASK if sortmask else 0) | (capi.BUILD_TILE_PLANS if tile_plans else 0)
            h = L.scn_builder_build(b, _prec(precision), flags, None)
        finally:
            L.scn_builder_destroy(b)
        return cls(h)

    def close(self):
        if getattr(self, "_h", None):
            capi.lib().scn_engine_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    # --- spconv::Engine surface
    def num_input(self) -> int:
        return capi.lib().scn_engine_num_input(self._h)

    def num_output(self) -> int:
        return capi.lib().scn_engine_num_output(self._h)

    def set_input(self, features, indices, grid_size: Sequence[int], num: Optional[int] = None):
        """features: fp16 cuda tensor [N, C]; indices: int32 cuda tensor [N, 4]; both are aliased, not copied."""
        n = int(features.shape[0] if num is None else num)
        self._keep = (features, indices)
        capi.check(capi.lib().scn_engine_set_input(self._h, 0, C.c_void_p(features.data_ptr()), n, int(features.shape[1]),
                                                   C.c_void_p(indices.data_ptr()), capi.i3(*[int(g) for g in grid_size])))

    def set_input_ptr(self, features_ptr: int, n: int, channels: int, indices_ptr: int, grid_size: Sequence[int]):
        capi.check(capi.lib().scn_engine_set_input(self._h, 0, C.c_void_p(features_ptr), n, channels,
                                                   C.c_void_p(indices_ptr), capi.i3(*[int(g) for g in grid_size])))

    def set_dds_num_of_points_pointer(self, n_dev):
        """n_dev: cuda int32/uint32 tensor with one element holding the real number of rows, or None."""
        self._keep_dds = n_dev
        capi.check(capi.lib().scn_engine_set_num_points_device_ptr(
            self._h, 0, C.c_void_p(n_dev.data_ptr()) if n_dev is not None else None))

    def forward(self, stream=None):
        capi.check(capi.lib().scn_engine_forward(self._h, _stream_ptr(stream)))

    def collect_amax(self, stream=None) -> Dict[str, float]:
        """max |value| of every sparse tensor the engine holds after a forward (all of them with keep_all)."""
        cap = 4096
        arr = (capi.TensorAmax * cap)()
        n = capi.lib().scn_engine_collect_amax(self._h, _stream_ptr(stream), C.cast(arr, C.c_void_p), cap)
        if n < 0:
            raise RuntimeError("collect_amax failed: " + capi.lib().scn_last_error().decode())
        return {arr[i].tensor.decode(): float(arr[i].amax) for i in range(n)}

    def output(self, index: int = 0) -> TensorView:
        v = capi.TensorView()
        capi.check(capi.lib().scn_engine_output(self._h, index, C.byref(v)))
        return TensorView(v)

    def tensor(self, name: str):
        """(view, accumulator pointer or None) of any kept tensor."""
        v = capi.TensorView()
        acc = C.c_void_p()
        capi.check(capi.lib().scn_engine_tensor(self._h, name.encode(), C.byref(v), C.byref(acc)))
        return TensorView(v), acc.value

    def set_profiling(self, enabled: bool):
        capi.check(capi.lib().scn_engine_set_profiling(self._h, int(enabled)))

    def step_times(self):
        """[(label, kind, ms)] of the last forward (profiling must be enabled)."""
        L = capi.lib()
        out = []
        for i in range(L.scn_engine_num_nodes(self._h)):
            name, kind, ms = C.c_char_p(), C.c_char_p(), C.c_float()
            capi.check(L.scn_engine_node_info(self._h, i, C.byref(name), C.byref(kind), C.byref(ms)))
            out.append((name.value.decode(), kind.value.decode(), float(ms.value)))
        return out


class SCNModel:
    """`pyscn.SCNModel`: numpy in, numpy out (`libraries/3DSparseConvolution/src/pyscn.cpp:47-125`)."""

    def __init__(self, onnx: str, precision: str = "fp16"):
        self.engine = Engine.from_onnx(onnx, precision)

    def forward(self, features: np.ndarray, indices: np.ndarray, grid_size: Sequence[int], stream=None):
        import torch
        f = torch.from_numpy(np.ascontiguousarray(features, np.float16).view(np.int16)).cuda().view(torch.float16)
        i = torch.from_numpy(np.ascontiguousarray(indices, np.int32)).cuda()
        self.engine.set_input(f, i, grid_size)
        self.engine.forward(stream)
        out = self.engine.output(0)
        if out.dense:
            return out.torch().cpu().numpy(), None
        feats, idx = out.torch()
        return feats.cpu().numpy(), idx.cpu().numpy()


class Voxelization:
    """`bevfusion::lidar::Voxelization`: fp16 points on the device -> mean voxel features + indices."""

    def __init__(self, min_range, max_range, voxel_size, grid_size=None, num_feature=5, max_voxels=160000,
                 max_points_per_voxel=10, max_points=300000):
        p = capi.VoxelizationParam()
        p.min_range[:] = [float(v) for v in min_range]
        p.max_range[:] = [float(v) for v in max_range]
        p.voxel_size[:] = [float(v) for v in voxel_size]
        if grid_size is None:  # VoxelizationParameter::compute_grid_size
            grid_size = [int(round((float(max_range[a]) - float(min_range[a])) / float(voxel_size[a]))) for a in range(3)]
        p.grid_size[:] = [int(v) for v in grid_size]
        p.num_feature, p.max_voxels, p.max_points_per_voxel, p.max_points = num_feature, max_voxels, max_points_per_voxel, max_points
        self.param = p
        self._h = capi.lib().scn_voxelizer_create(C.byref(p))
        if not self._h:
            raise RuntimeError("voxelizer creation failed: " + capi.lib().scn_last_error().decode())
        self.order = capi.ORDER_XYZ

    def close(self):
        if getattr(self, "_h", None):
            capi.lib().scn_voxelizer_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def forward(self, points, num_points: Optional[int] = None, stream=None, order: str = "xyz"):
        self.order = capi.ORDER_ZYX if order.lower() == "zyx" else capi.ORDER_XYZ
        n = int(points.shape[0] if num_points is None else num_points)
        self._keep = points
        import torch
        if points.dtype not in (torch.float16, torch.float32):
            raise ValueError("points must be a float16 or float32 device tensor")
        dtype = capi.DTYPE_FP32 if points.dtype == torch.float32 else capi.DTYPE_FP16
        capi.check(capi.lib().scn_voxelizer_forward_points(self._h, C.c_void_p(points.data_ptr()), dtype, n, self.order,
                                                           _stream_ptr(stream)))

    def num_voxels(self, stream=None) -> int:
        return int(capi.lib().scn_voxelizer_num_voxels(self._h, _stream_ptr(stream)))

    def num_voxels_dev_ptr(self) -> int:
        return capi.lib().scn_voxelizer_num_voxels_dev(self._h)

    def voxel_dim(self) -> int:
        return self.param.num_feature

    def indices_dim(self) -> int:
        return 4

    def grid_size(self) -> List[int]:
        g = capi.i3()
        capi.lib().scn_voxelizer_grid_size(self._h, self.order, g)
        return [int(v) for v in g]

    def features_ptr(self) -> int:
        return capi.lib().scn_voxelizer_features(self._h)

    def indices_ptr(self) -> int:
        return capi.lib().scn_voxelizer_indices(self._h)


class LidarSCN:
    """`bevfusion::lidar::SCN`: one call from points to the BEV feature map.

    Unlike the reference glue, which reads the voxel count back to the host between voxelization and
    the engine, the count stays on the device: the engine takes max_voxels as the row bound and the
    voxelizer's device counter as the real number of rows, so a frame needs no host synchronisation.
    """

    def __init__(self, model, voxelization: Voxelization, order: str = "xyz", precision: str = "fp16"):
        self.voxelization = voxelization
        self.order = order
        if isinstance(model, Graph):
            fd, path = tempfile.mkstemp(suffix=".scn.onnx")
            os.close(fd)
            try:
                save_onnx(model, path)
                self.engine = Engine.from_onnx(path, precision)
            finally:
                os.unlink(path)
        else:
            self.engine = Engine.from_onnx(model, precision)
        self._bound = False

    def forward(self, points, num_points: Optional[int] = None, stream=None) -> TensorView:
        v = self.voxelization
        v.forward(points, num_points, stream, self.order)
        if not self._bound:
            self.engine.set_input_ptr(v.features_ptr(), v.param.max_voxels, v.voxel_dim(), v.indices_ptr(), v.grid_size())
            capi.check(capi.lib().scn_engine_set_num_points_device_ptr(self.engine._h, 0, C.c_void_p(v.num_voxels_dev_ptr())))
            self._bound = True
        self.engine.forward(stream)
        return self.engine.output(0)

    def shape(self) -> List[int]:
        return self.engine.output(0).shape
