"""Builders of CenterPoint- and BEVFusion-shaped SCN graphs in the reference's ONNX dialect.

They play the role of the reference's exporters (which trace real checkpoints that are not
available offline): same node kinds, attribute names, tensor naming (decimal strings in creation
order), weight layout `[Cout, K0, K1, K2, Cin]` and precision plans, but with seeded random
weights.  Followed: `CUDA-CenterPoint/qat/onnx_export/exptool.py:115-262` (node attributes),
`CUDA-CenterPoint/qat/onnx_export/export-scn.py:52-68` (CenterPoint int8 plan),
`CUDA-BEVFusion/qat/export-scn.py:62-67` (BEVFusion int8 plan),
`CUDA-BEVFusion/qat/lean/exptool.py:269-294` (dense / permute / reshape tail).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .onnx_dialect import Graph, Node


class _Builder:
    def __init__(self, seed: int, weight_std: float = 0.02, output_bound: int = 200000):
        self.rng = np.random.default_rng(seed)
        self.std = weight_std
        self.output_bound = int(output_bound)
        self.nodes: List[Node] = []
        self.inits: Dict[str, np.ndarray] = {}
        self.next_tensor = 1
        self.nconv = 0
        self.nadd = 0
        self.nrelu = 0

    def tensor(self) -> str:
        t = str(self.next_tensor)
        self.next_tensor += 1
        return t

    def conv(self, x: str, cin: int, cout: int, ksize, stride=(1, 1, 1), padding=(0, 0, 0), subm=False,
             rulebook="", activation="ReLU", tag="", inverse=False) -> str:
        i = self.nconv
        self.nconv += 1
        w = (self.rng.standard_normal((cout, *ksize, cin)) * self.std).astype(np.float16)
        b = (self.rng.standard_normal((cout,)) * self.std).astype(np.float16)
        self.inits[f"spconv{i}.weight"] = w
        self.inits[f"spconv{i}.bias"] = b
        y = self.tensor()
        self.nodes.append(Node("SparseConvolution", f"conv{i}", [x, f"spconv{i}.weight", f"spconv{i}.bias"], [y], {
            "ndim": 3, "in_channels": cin, "out_channels": cout,
            "kernel_size": list(ksize), "stride": list(stride), "padding": list(padding), "dilation": [1, 1, 1],
            "output_bound": self.output_bound, "transposed": 0, "inverse": int(inverse), "groups": 1,
            "subm": int(subm), "rulebook": rulebook, "activation": activation, "tag": tag,
        }))
        return y

    def add(self, a: str, b: str, tag="") -> str:
        y = self.tensor()
        self.nodes.append(Node("Add", f"add{self.nadd}", [a, b], [y], {"tag": tag}))
        self.nadd += 1
        return y

    def relu(self, x: str) -> str:
        y = self.tensor()
        self.nodes.append(Node("Relu", f"relu{self.nrelu}", [x], [y], {}))
        self.nrelu += 1
        return y

    def block(self, x: str, c: int, key: str, tag: str) -> str:
        h = self.conv(x, c, c, (3, 3, 3), subm=True, rulebook=key, activation="ReLU", tag=tag + ".conv1")
        h = self.conv(h, c, c, (3, 3, 3), subm=True, rulebook=key, activation="None", tag=tag + ".conv2")
        h = self.add(h, x, tag=tag + ".quant_add")
        return self.relu(h)


def _strip_tags(nodes: List[Node]) -> Dict[str, str]:
    tags = {}
    for n in nodes:
        t = n.attrs.pop("tag", "")
        if t:
            tags[n.name] = t
    return tags


def centerpoint_scn(seed: int = 0, in_channels: int = 5, grid_zyx: Sequence[int] = (41, 1440, 1440),
                    channels: Sequence[int] = (16, 32, 64, 128), weight_std: float = 0.02,
                    output_bound: int = 200000) -> Tuple[Graph, Dict[str, str]]:
    """CenterPoint `SpMiddleResNetFHD`-shaped graph, zyx index order, all fp16.

    output_bound is the row capacity every convolution carries (the exporter's `output_bound` attribute,
    CUDA-CenterPoint/qat/onnx_export/exptool.py:178-205); the random weights do not depend on it.
    Returns the graph and a map node name -> module path (used by the precision plans).
    """
    b = _Builder(seed, weight_std, output_bound)
    c0, c1, c2, c3 = channels
    x = b.conv("0", in_channels, c0, (3, 3, 3), subm=True, rulebook="res0", tag="conv_input")
    x = b.block(x, c0, "res0", "conv1.0")
    x = b.block(x, c0, "res0", "conv1.1")
    x = b.conv(x, c0, c1, (3, 3, 3), (2, 2, 2), (1, 1, 1), tag="conv2.0")
    x = b.block(x, c1, "res1", "conv2.3")
    x = b.block(x, c1, "res1", "conv2.4")
    x = b.conv(x, c1, c2, (3, 3, 3), (2, 2, 2), (1, 1, 1), tag="conv3.0")
    x = b.block(x, c2, "res2", "conv3.3")
    x = b.block(x, c2, "res2", "conv3.4")
    x = b.conv(x, c2, c3, (3, 3, 3), (2, 2, 2), (0, 1, 1), tag="conv4.0")
    x = b.block(x, c3, "res3", "conv4.3")
    x = b.block(x, c3, "res3", "conv4.4")
    x = b.conv(x, c3, c3, (3, 1, 1), (2, 1, 1), (0, 0, 0), tag="extra_conv")
    g = list(grid_zyx)
    for k, s, p in (((3, 3, 3), (2, 2, 2), (1, 1, 1)),) * 2 + (((3, 3, 3), (2, 2, 2), (0, 1, 1)),
                                                                 ((3, 1, 1), (2, 1, 1), (0, 0, 0))):
        g = [(g[a] + 2 * p[a] - (k[a] - 1) - 1) // s[a] + 1 for a in range(3)]
    d = b.tensor()
    b.nodes.append(Node("ScatterDense", "scatter0", [x], [d], {
        "input_spatial_shape": g, "format": "zyx", "output_shape": [1, c3, *g]}))
    r = b.tensor()
    b.nodes.append(Node("Reshape", "reshape0", [d], [r], {"dims": [1, c3 * g[0], g[1], g[2]]}))
    tags = _strip_tags(b.nodes)
    return Graph(["0"], [r], b.nodes, b.inits), tags


def bevfusion_scn(seed: int = 0, in_channels: int = 5, grid_xyz: Sequence[int] = (1440, 1440, 41),
                  channels: Sequence[int] = (16, 32, 64, 128), weight_std: float = 0.02,
                  output_bound: int = 200000) -> Tuple[Graph, Dict[str, str]]:
    """BEVFusion lidar `SparseEncoder`-shaped graph, xyz index order, all fp16."""
    b = _Builder(seed, weight_std, output_bound)
    c0, c1, c2, c3 = channels
    x = b.conv("0", in_channels, c0, (3, 3, 3), subm=True, rulebook="subm1", tag="conv_input")
    g = list(grid_xyz)
    pads = ((1, 1, 1), (1, 1, 1), (1, 1, 0))
    cs = (c0, c1, c2, c3)
    for i in range(4):
        x = b.block(x, cs[i], f"subm{i + 1}", f"encoder_layers.{i}.0")
        x = b.block(x, cs[i], f"subm{i + 1}", f"encoder_layers.{i}.1")
        if i < 3:
            x = b.conv(x, cs[i], cs[i + 1], (3, 3, 3), (2, 2, 2), pads[i], rulebook=f"spconv{i + 2}",
                       tag=f"encoder_layers.{i}.2")
            g = [(g[a] + 2 * pads[i][a] - 2 - 1) // 2 + 1 for a in range(3)]
    x = b.conv(x, c3, c3, (1, 1, 3), (1, 1, 2), (0, 0, 0), rulebook="spconv_down2", tag="conv_out")
    g = [g[0], g[1], (g[2] - 2 - 1) // 2 + 1]
    d = b.tensor()
    b.nodes.append(Node("ScatterDense", "scatter0", [x], [d], {
        "input_spatial_shape": g, "format": "xyz", "output_shape": [1, c3, *g]}))
    t = b.tensor()
    b.nodes.append(Node("Transpose", "transpose0", [d], [t], {"dims": [0, 1, 4, 2, 3]}))
    r = b.tensor()
    b.nodes.append(Node("Reshape", "reshape0", [t], [r], {"dims": [1, c3 * g[2], g[0], g[1]]}))
    tags = _strip_tags(b.nodes)
    return Graph(["0"], [r], b.nodes, b.inits), tags


def single_subm_layer(seed: int = 0, cin: int = 16, cout: int = 16) -> Graph:
    """One SubMConv3d 3x3x3 layer with ReLU: the smallest graph of the dialect."""
    b = _Builder(seed)
    y = b.conv("0", cin, cout, (3, 3, 3), subm=True, rulebook="subm0")
    _strip_tags(b.nodes)
    return Graph(["0"], [y], b.nodes, b.inits)


def unet_scn(seed: int = 0, in_channels: int = 5, channels: Sequence[int] = (16, 32, 64), weight_std: float = 0.05
             ) -> Tuple[Graph, Dict[str, str]]:
    """Small encoder-decoder (two strided convolutions down, two SparseInverseConvolution nodes back up
    on the same rulebooks, skip connections by Add): the shape of spconv's segmentation networks, with a
    sparse graph output.  Exercises the `inverse` attribute of the dialect."""
    b = _Builder(seed, weight_std)
    c0, c1, c2 = channels
    x0 = b.conv("0", in_channels, c0, (3, 3, 3), subm=True, rulebook="s0", tag="enc0.in")
    x0 = b.block(x0, c0, "s0", "enc0.res")
    x1 = b.conv(x0, c0, c1, (3, 3, 3), (2, 2, 2), (1, 1, 1), rulebook="down1", tag="enc1.down")
    x1 = b.block(x1, c1, "s1", "enc1.res")
    x2 = b.conv(x1, c1, c2, (3, 3, 3), (2, 2, 2), (1, 1, 1), rulebook="down2", tag="enc2.down")
    x2 = b.block(x2, c2, "s2", "enc2.res")
    u1 = b.conv(x2, c2, c1, (3, 3, 3), (2, 2, 2), (1, 1, 1), rulebook="down2", activation="None", tag="dec1.up",
                inverse=True)
    u1 = b.relu(b.add(u1, x1, tag="dec1.skip"))
    u1 = b.block(u1, c1, "s1", "dec1.res")
    u0 = b.conv(u1, c1, c0, (3, 3, 3), (2, 2, 2), (1, 1, 1), rulebook="down1", activation="None", tag="dec0.up",
                inverse=True)
    u0 = b.relu(b.add(u0, x0, tag="dec0.skip"))
    tags = _strip_tags(b.nodes)
    return Graph(["0"], [u0], b.nodes, b.inits), tags


# --------------------------------------------------------------------------- int8 plans
def weight_dynamic_ranges(w: np.ndarray) -> List[float]:
    """Per-output-channel amax of `[Cout, K0, K1, K2, Cin]` fp16 weights (quantizer axis 0)."""
    return [float(v) for v in np.abs(w.astype(np.float32)).reshape(w.shape[0], -1).max(axis=1)]


def apply_int8_plan(graph: Graph, tags: Dict[str, str], tensor_amax: Dict[str, float], plan: str) -> Graph:
    """Annotate a graph with dynamic ranges and per-node precisions.

    tensor_amax maps a tensor name to the calibrated per-tensor amax of its values.  Conv nodes get
    `input_dynamic_range` = amax of their input; Add nodes get one shared range for both inputs
    (`exptool.py:226-227`): the larger of the two input amaxes.
    plan: "centerpoint", "bevfusion" or "all-int8" (every convolution and Add computes and stores int8).
    """
    fp16_compute: set = set()
    fp16_output: set = set()
    if plan == "centerpoint":
        fp16_compute = {"conv_input", "conv1.0.conv1", "conv1.0.conv2", "conv1.0.quant_add"}
        fp16_output = {"conv_input", "conv1.0.conv1", "conv1.0.conv2", "extra_conv"}
    elif plan == "bevfusion":
        fp16_compute = {"conv_input"}
        fp16_output = {"conv_out"}
    elif plan == "all-int8":
        pass
    else:
        raise ValueError(plan)
    for n in graph.nodes:
        tag = tags.get(n.name, "")
        if n.op_type == "SparseConvolution":
            n.attrs["input_dynamic_range"] = float(tensor_amax[n.inputs[0]])
            n.attrs["weight_dynamic_ranges"] = weight_dynamic_ranges(graph.initializers[n.inputs[1]])
        elif n.op_type == "Add":
            r = float(max(tensor_amax[n.inputs[0]], tensor_amax[n.inputs[1]]))
            n.attrs["input0_dynamic_range"] = r
            n.attrs["input1_dynamic_range"] = r
        else:
            continue
        n.attrs["precision"] = "fp16" if tag in fp16_compute else "int8"
        n.attrs["output_precision"] = "fp16" if tag in fp16_output else "int8"
    return graph


def percentile_amax(abs_values: np.ndarray, q: float = 99.99) -> float:
    """The calibration rule of the int8 configurations: the q-th percentile of |activation|."""
    if abs_values.size == 0:
        return 1.0
    v = float(np.percentile(abs_values.astype(np.float32), q))
    return v if v > 0 else 1.0
