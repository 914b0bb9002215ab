"""Post-training calibration of per-tensor activation ranges.

The reference calibrates with pytorch-quantization histograms
(`CUDA-CenterPoint/qat/tools/sparseconv_quantization.py:165-207`); the benchmark configurations of
this repository state a simpler rule instead: amax = the 99.99th percentile of |activation| over a
few calibration frames.  The activations come from a runner passed in by the caller: the fp16 HIP
engine with every tensor kept (`gpu_runner`), or any other function with the same signature.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, Sequence, Tuple

import numpy as np

from .graphs import percentile_amax
from .onnx_dialect import Graph

Runner = Callable[[Graph, np.ndarray, np.ndarray, Sequence[int]], Dict[str, np.ndarray]]


def sparse_tensor_names(graph: Graph):
    """Names of the tensors whose ranges the int8 plans need: the input and every conv/add/relu output."""
    names = list(graph.inputs)
    for n in graph.nodes:
        if n.op_type in ("SparseConvolution", "Add", "QuantAdd", "Relu"):
            names.append(n.outputs[0])
    return names


def calibrate_amax(graph: Graph, frames: Iterable[Tuple[np.ndarray, np.ndarray]], grid: Sequence[int], runner: Runner,
                   q: float = 99.99, max_samples_per_frame: int = 4_000_000, seed: int = 0) -> Dict[str, float]:
    """frames: iterable of (features fp16 [N,C], indices int32 [N,4])."""
    rng = np.random.default_rng(seed)
    pools: Dict[str, list] = {}
    for feats, idx in frames:
        acts = runner(graph, feats, idx, grid)
        for name, v in acts.items():
            a = np.abs(np.asarray(v, np.float32)).reshape(-1)
            if a.size > max_samples_per_frame:
                a = a[rng.choice(a.size, max_samples_per_frame, replace=False)]
            pools.setdefault(name, []).append(a)
    return {name: percentile_amax(np.concatenate(parts), q) for name, parts in pools.items()}


def gpu_runner(graph: Graph, feats: np.ndarray, idx: np.ndarray, grid: Sequence[int]) -> Dict[str, np.ndarray]:
    """Runs the fp16 HIP engine with every tensor kept and returns the sparse activations."""
    import torch
    from .scn import Engine
    eng = Engine.from_graph(graph, "fp16", keep_all=True)
    f = torch.from_numpy(np.ascontiguousarray(feats, np.float16).view(np.int16)).cuda().view(torch.float16)
    i = torch.from_numpy(np.ascontiguousarray(idx, np.int32)).cuda()
    eng.set_input(f, i, grid)
    eng.forward()
    torch.cuda.synchronize()
    out = {graph.inputs[0]: np.asarray(feats, np.float32)}
    for name in sparse_tensor_names(graph)[1:]:
        view, _ = eng.tensor(name)
        t, _ = view.torch()
        out[name] = t[:, :].float().cpu().numpy()
    eng.close()
    return out
