"""Exporter-side transformations of a model before it is written in the ONNX dialect.

The reference's exporters trace a trained PyTorch/spconv module; what they do to the weights and
attributes on the way out is restated here on plain numpy arrays and on `onnx_dialect.Graph`:

* `fuse_bn_weights`   BatchNorm1d folded into the preceding sparse convolution
                      (`CUDA-BEVFusion/qat/lean/funcs.py:54-73`, same rule in
                      `CUDA-CenterPoint/qat/onnx_export/funcs.py`);
* `invert_graph`      index order xyz -> zyx (or back): the spatial axes of every kernel and attribute
                      reversed (`CUDA-BEVFusion/qat/lean/exptool.py:332-343`), the dense tail rewritten
                      as the inverted forward hook does (`exptool.py:284-291`);
* `invert_indices`    the matching change of the coordinate columns (`exptool.py:348`).
"""
from __future__ import annotations

import copy
from typing import Optional, Sequence

import numpy as np

from .onnx_dialect import Graph, Node


def fuse_bn_weights(conv_w: np.ndarray, conv_b: Optional[np.ndarray], bn_mean: np.ndarray, bn_var: np.ndarray,
                    bn_eps: float, bn_weight: Optional[np.ndarray] = None, bn_bias: Optional[np.ndarray] = None):
    """Fold y = gamma * (conv(x) + b - mean) / sqrt(var + eps) + beta into the convolution.

    conv_w is `[Cout, K0, K1, K2, Cin]` (any number of kernel axes); returns (weight, bias) in fp32,
    weight in the same layout.  Missing conv bias / BN affine terms count as 0 / 1 / 0.
    """
    w = np.asarray(conv_w, np.float32)
    cout = w.shape[0]
    mean = np.asarray(bn_mean, np.float32)
    var = np.asarray(bn_var, np.float32)
    b = np.zeros(cout, np.float32) if conv_b is None else np.asarray(conv_b, np.float32)
    gamma = np.ones(cout, np.float32) if bn_weight is None else np.asarray(bn_weight, np.float32)
    beta = np.zeros(cout, np.float32) if bn_bias is None else np.asarray(bn_bias, np.float32)
    rstd = (1.0 / np.sqrt(var + np.float32(bn_eps))).astype(np.float32)
    scale = gamma * rstd
    w_fused = w * scale.reshape((cout,) + (1,) * (w.ndim - 1))
    b_fused = (b - mean) * rstd * gamma + beta
    return w_fused.astype(np.float32), b_fused.astype(np.float32)


_SPATIAL_ATTRS = ("kernel_size", "stride", "padding", "dilation", "output_padding")


def invert_indices(indices: np.ndarray) -> np.ndarray:
    """`[N, 4]` (batch, a, b, c) -> (batch, c, b, a)."""
    return np.ascontiguousarray(np.asarray(indices)[:, [0, 3, 2, 1]])


def invert_graph(graph: Graph) -> Graph:
    """The same network for coordinates given in the reverse axis order.

    Convolutions: kernel `[Cout, K0, K1, K2, Cin]` -> `[Cout, K2, K1, K0, Cin]` and every per-axis
    attribute reversed.  ScatterDense: `input_spatial_shape` and the three spatial entries of
    `output_shape` reversed, `format` flipped between "xyz" and "zyx".  A Transpose that follows a
    ScatterDense permutes the reversed axes instead, so that the graph's dense outputs are unchanged:
    source axis s >= 2 of the old dense tensor is axis 6 - s of the new one.
    """
    g = copy.deepcopy(graph)
    dense_outputs = set()
    for n in g.nodes:
        if n.op_type == "SparseConvolution":
            w = g.initializers[n.inputs[1]]
            if w.ndim != 5:
                raise ValueError(f"{n.name}: expected a [Cout, K0, K1, K2, Cin] kernel, got {w.shape}")
            g.initializers[n.inputs[1]] = np.ascontiguousarray(w.transpose(0, 3, 2, 1, 4))
            for a in _SPATIAL_ATTRS:
                if a in n.attrs:
                    n.attrs[a] = list(n.attrs[a])[::-1]
        elif n.op_type == "ScatterDense":
            if "input_spatial_shape" in n.attrs:
                n.attrs["input_spatial_shape"] = list(n.attrs["input_spatial_shape"])[::-1]
            shape = list(n.attrs["output_shape"])
            if len(shape) != 5:
                raise ValueError(f"{n.name}: output_shape must be [N, C, d0, d1, d2]")
            n.attrs["output_shape"] = shape[:2] + shape[2:][::-1]
            fmt = n.attrs.get("format", "")
            if fmt in ("xyz", "zyx"):
                n.attrs["format"] = fmt[::-1]
            dense_outputs.add(n.outputs[0])
        elif n.op_type == "Transpose" and n.inputs[0] in dense_outputs:
            n.attrs["dims"] = [d if d < 2 else 6 - d for d in n.attrs["dims"]]
        elif n.op_type == "Reshape" and n.inputs[0] in dense_outputs:
            # A reshape straight after the scatter merges axes of the reversed tensor: make the old order
            # explicit first.  (The CenterPoint tail merges C with the leading spatial axis.)
            raise ValueError(f"{n.name}: a Reshape directly after ScatterDense cannot be inverted without a Transpose; "
                             "insert Transpose(dims=[0, 1, 2, 3, 4]) before it")
    return g


def insert_identity_transpose(graph: Graph) -> Graph:
    """Put an explicit identity Transpose between every ScatterDense and a Reshape that consumes it, so
    that `invert_graph` has an axis permutation to rewrite."""
    g = copy.deepcopy(graph)
    dense_outputs = {n.outputs[0] for n in g.nodes if n.op_type == "ScatterDense"}
    used = {t for n in g.nodes for t in list(n.inputs) + list(n.outputs)} | set(g.initializers)
    nodes = []
    k = 0
    for n in g.nodes:
        if n.op_type == "Reshape" and n.inputs[0] in dense_outputs:
            name = f"{n.inputs[0]}.t"
            while name in used:
                name += "_"
            used.add(name)
            nodes.append(Node("Transpose", f"transpose_id{k}", [n.inputs[0]], [name], {"dims": [0, 1, 2, 3, 4]}))
            k += 1
            n.inputs[0] = name
        nodes.append(n)
    g.nodes = nodes
    return g
