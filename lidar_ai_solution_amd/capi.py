"""ctypes declarations of the C ABI in include/scn_c_api.h.

The shared library is required: importing `lib()` raises when libscn_hip.so has not been built;
there is no CPU fallback of any kind.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libscn_hip.so")

OK = 0
PRECISION_FP16, PRECISION_INT8 = 1, 2
DTYPE_INT32, DTYPE_FP16, DTYPE_FP32, DTYPE_INT8 = 1, 2, 3, 7
ORDER_XYZ, ORDER_ZYX = 1, 2
BUILD_SORTMASK, BUILD_AUX_STREAM, BUILD_KEEP_ALL, BUILD_TILE_PLANS = 1, 4, 256, 512

vp = C.c_void_p
u32 = C.c_uint32
i3 = C.c_int * 3
i5 = C.c_int * 5


class PrecisionOverride(C.Structure):
    _fields_ = [("selector", C.c_char_p), ("by_optype", C.c_int), ("precision", C.c_int), ("output_precision", C.c_int)]


class TensorAmax(C.Structure):
    _fields_ = [("tensor", C.c_char_p), ("amax", C.c_float)]


class LoadOptions(C.Structure):
    _fields_ = [("overrides", C.c_void_p), ("n_overrides", C.c_int), ("ranges", C.c_void_p), ("n_ranges", C.c_int)]


class VoxelizationParam(C.Structure):
    _fields_ = [("min_range", C.c_float * 3), ("max_range", C.c_float * 3), ("voxel_size", C.c_float * 3),
                ("grid_size", C.c_int * 3), ("num_feature", C.c_int), ("max_voxels", C.c_int),
                ("max_points_per_voxel", C.c_int), ("max_points", C.c_int)]


class ConvIO(C.Structure):
    _fields_ = [("x_dev", vp), ("x_ld", u32), ("x_dynamic_range", C.c_float), ("relu", C.c_int), ("out_dtype", C.c_int),
                ("out_dynamic_range", C.c_float), ("out_dev", vp), ("out_ld", u32), ("acc_dev", vp), ("res_dev", vp),
                ("res_dtype", C.c_int), ("res_dynamic_range", C.c_float), ("res_ld", u32), ("mid_dtype", C.c_int),
                ("mid_dynamic_range", C.c_float), ("a_requant_range", C.c_float), ("b_requant_range", C.c_float),
                ("relu_after_add", C.c_int), ("fixed_launch_points", u32)]


class TensorView(C.Structure):
    _fields_ = [("name", C.c_char_p), ("features_dev", vp), ("dtype", C.c_int), ("ndim", C.c_int),
                ("shape", C.c_int64 * 8), ("indices_dev", vp), ("num_dev", vp), ("grid_size", C.c_int * 3),
                ("dynamic_range", C.c_float)]


LOG_CALLBACK = C.CFUNCTYPE(None, C.c_char_p, C.c_int, C.c_char_p, C.c_int, vp)

_SIGNATURES = {
    "scn_version": (C.c_int, []),
    "scn_last_error": (C.c_char_p, []),
    "scn_device_bytes_in_use": (C.c_size_t, []),
    "scn_set_log_level": (None, [C.c_int]),
    "scn_get_log_level": (C.c_int, []),
    "scn_set_debug_sync": (None, [C.c_int]),
    "scn_get_debug_sync": (C.c_int, []),
    "scn_set_log_callback": (None, [LOG_CALLBACK, vp]),
    "scn_log": (None, [C.c_char_p, C.c_int, C.c_int, C.c_char_p]),
    "scn_memset_async": (C.c_int, [vp, C.c_ubyte, C.c_size_t, vp]),
    "scn_hash_u64": (C.c_uint64, [C.c_uint64]),
    "scn_hash_capacity_for": (C.c_size_t, [u32]),
    "scn_hash_build": (C.c_int, [vp, C.c_size_t, vp, u32, vp, i3, vp]),
    "scn_hash_query": (C.c_int, [vp, C.c_size_t, vp, u32, i3, vp, vp]),
    "scn_voxelizer_create": (vp, [C.POINTER(VoxelizationParam)]),
    "scn_voxelizer_destroy": (None, [vp]),
    "scn_voxelizer_forward": (C.c_int, [vp, vp, u32, C.c_int, vp]),
    "scn_voxelizer_forward_points": (C.c_int, [vp, vp, C.c_int, u32, C.c_int, vp]),
    "scn_voxelizer_features": (vp, [vp]),
    "scn_voxelizer_indices": (vp, [vp]),
    "scn_voxelizer_num_voxels_dev": (vp, [vp]),
    "scn_voxelizer_points_per_voxel": (vp, [vp]),
    "scn_voxelizer_num_voxels": (u32, [vp, vp]),
    "scn_voxelizer_grid_size": (None, [vp, C.c_int, i3]),
    "scn_rulebook_create": (vp, [u32, u32, C.c_int]),
    "scn_rulebook_destroy": (None, [vp]),
    "scn_rulebook_build_subm": (C.c_int, [vp, vp, u32, vp, i3, i3, i3, vp]),
    "scn_rulebook_build_sparse": (C.c_int, [vp, vp, u32, vp, i3, i3, i3, i3, i3, vp]),
    "scn_rulebook_build_inverse": (C.c_int, [vp, vp, vp, vp]),
    "scn_rulebook_build_plan": (C.c_int, [vp, C.c_int, vp]),
    "scn_rulebook_plan": (C.c_int, [vp, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp)]),
    "scn_rulebook_nbr": (vp, [vp]),
    "scn_rulebook_nbr_ld": (u32, [vp]),
    "scn_rulebook_out_indices": (vp, [vp]),
    "scn_rulebook_num_out_dev": (vp, [vp]),
    "scn_rulebook_num_out_total_dev": (vp, [vp]),
    "scn_rulebook_out_grid": (None, [vp, i3]),
    "scn_rulebook_pairs": (C.c_int, [vp, vp, vp, vp, C.c_uint64, vp]),
    "scn_conv_create": (vp, [vp, i5, vp, vp, C.c_int]),
    "scn_conv_destroy": (None, [vp]),
    "scn_conv_forward": (C.c_int, [vp, vp, C.POINTER(ConvIO), vp]),
    "scn_convert_rows": (C.c_int, [vp, C.c_int, u32, u32, C.c_float, vp, C.c_int, u32, u32, C.c_float, C.c_int, u32, vp, vp]),
    "scn_add_relu": (C.c_int, [vp, C.c_int, C.c_float, C.c_float, vp, C.c_int, C.c_float, C.c_float, vp, C.c_int,
                               C.c_float, C.c_int, u32, u32, vp, vp]),
    "scn_scatter_dense": (C.c_int, [vp, C.c_int, C.c_float, u32, u32, vp, u32, vp, i5, vp, vp, vp]),
    "scn_scatter_dense_layout": (C.c_int, [vp, C.c_int, C.c_float, u32, u32, vp, u32, vp, i5, vp, C.c_int, C.c_int,
                                           C.c_int, C.c_float, vp, vp]),
    "scn_scatter_dense_map_cells": (C.c_size_t, [i5, vp]),
    "scn_scatter_dense_with_map": (C.c_int, [vp, C.c_int, C.c_float, u32, u32, vp, u32, vp, i5, vp, vp, vp, vp]),
    "scn_scatter_dense_noalloc_max_cells": (C.c_size_t, []),
    "scn_scatter_dense_noalloc": (C.c_int, [vp, C.c_int, C.c_float, u32, u32, vp, u32, vp, i5, vp, vp, vp]),
    "scn_builder_create": (vp, []),
    "scn_builder_destroy": (None, [vp]),
    "scn_builder_push_input": (C.c_int, [vp, C.c_char_p]),
    "scn_builder_push_sparse_conv": (C.c_int, [vp, C.c_char_p, C.c_int, vp, i5, vp, C.c_int, vp, C.c_int, C.c_char_p,
                                               i3, i3, i3, i3, C.c_float, C.c_int, u32, u32, C.c_char_p, C.c_int,
                                               C.c_int, C.c_char_p, C.c_int]),
    "scn_builder_push_add": (C.c_int, [vp, C.c_char_p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_char_p, C.c_int,
                                       C.c_int, u32]),
    "scn_builder_push_relu": (C.c_int, [vp, C.c_char_p, C.c_int, C.c_char_p]),
    "scn_builder_push_dense": (C.c_int, [vp, C.c_char_p, C.c_int, C.c_char_p, C.c_char_p, i3, vp, C.c_int, C.c_int,
                                         C.c_float, u32]),
    "scn_builder_push_reshape": (C.c_int, [vp, C.c_char_p, C.c_int, vp, C.c_int, C.c_char_p]),
    "scn_builder_push_transpose": (C.c_int, [vp, C.c_char_p, C.c_int, vp, C.c_int, C.c_char_p]),
    "scn_builder_push_output": (C.c_int, [vp, C.c_int]),
    "scn_builder_build": (vp, [vp, C.c_int, C.c_uint, vp]),
    "scn_engine_create_from_onnx": (vp, [C.c_char_p, C.c_int, C.c_uint, C.c_uint, vp]),
    "scn_engine_create_from_onnx_ex": (vp, [C.c_char_p, C.c_int, C.c_uint, C.c_uint, vp, vp]),
    "scn_engine_create_from_onnx_memory": (vp, [vp, C.c_size_t, C.c_int, C.c_uint, C.c_uint, vp, vp]),
    "scn_engine_collect_amax": (C.c_int, [vp, vp, vp, C.c_int]),
    "scn_engine_destroy": (None, [vp]),
    "scn_engine_num_input": (C.c_int, [vp]),
    "scn_engine_num_output": (C.c_int, [vp]),
    "scn_engine_set_input": (C.c_int, [vp, C.c_int, vp, u32, u32, vp, i3]),
    "scn_engine_set_num_points_device_ptr": (C.c_int, [vp, C.c_int, vp]),
    "scn_engine_prepare": (C.c_int, [vp, i3]),
    "scn_engine_forward": (C.c_int, [vp, vp]),
    "scn_engine_output": (C.c_int, [vp, C.c_int, C.POINTER(TensorView)]),
    "scn_engine_tensor": (C.c_int, [vp, C.c_char_p, C.POINTER(TensorView), C.POINTER(vp)]),
    "scn_engine_set_profiling": (C.c_int, [vp, C.c_int]),
    "scn_engine_num_nodes": (C.c_int, [vp]),
    "scn_engine_node_info": (C.c_int, [vp, C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(C.c_float)]),
}

_lib = None
_hip = None


def hip_runtime():
    """The HIP runtime shared by this process, loaded with RTLD_GLOBAL before libscn_hip.so.

    libscn_hip.so has no DT_NEEDED entry for libamdhip64: when PyTorch is importable its bundled
    runtime is used (so torch streams and device pointers are valid inside the library), otherwise
    the ROCm installation's.
    """
    global _hip
    if _hip is None:
        candidates = []
        try:
            import torch  # noqa: F401  (its runtime must be the one in use when torch tensors are passed in)
            candidates.append(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
        except Exception:
            pass
        candidates += [os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "libamdhip64.so"), "libamdhip64.so"]
        err = None
        for c in candidates:
            if os.path.isabs(c) and not os.path.exists(c):
                continue
            try:
                _hip = C.CDLL(c, mode=C.RTLD_GLOBAL)
                break
            except OSError as e:  # pragma: no cover
                err = e
        if _hip is None:
            raise RuntimeError(f"no HIP runtime found ({err})")
    return _hip


def declared_symbols():
    return sorted(_SIGNATURES)


def lib():
    """The loaded library.  Raises if it has not been built (python -m lidar_ai_solution_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m lidar_ai_solution_amd.build` "
                               "(there is no fallback path)")
        hip_runtime()
        handle = C.CDLL(LIB_PATH)
        missing = []
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError:
                missing.append(name)
                continue
            fn.restype = res
            fn.argtypes = args
        if missing and not os.environ.get("SCN_PARTIAL_LIB"):
            raise RuntimeError(f"{LIB_PATH} does not export {missing}: rebuild it")
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != OK:
        raise RuntimeError(f"libscn_hip error {rc}: {lib().scn_last_error().decode()}")
