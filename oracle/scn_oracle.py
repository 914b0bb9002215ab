"""ctypes front end of the CPU oracle plus a node-by-node walk of an SCN graph.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg as the checker / timed baseline.  The product never imports this module.

The graph walk restates what the reference engine does with a loaded graph
(`libraries/3DSparseConvolution/src/onnx-parser.cpp:101-231` for the node semantics,
`libspconv/include/spconv/engine.hpp:96-167` for the builder arguments), one node at a time and
without any fusion, so that every intermediate tensor can be compared.

Precision rules stated by this build (the closed engine's are not recoverable):
  * engine precision fp16 makes every node fp16; with int8, a conv computes in int8 when its
    `precision` attribute is "int8" and it has an input range and per-channel weight ranges;
    an Add computes in int8 when `precision` is "int8" and both input ranges are set.
  * a tensor is stored int8 when its producer's `output_precision` is "int8" and some consumer
    fixes its dynamic range (amax): an int8 conv's `input_dynamic_range` first, else (through Relu)
    the next consumer, else an int8 Add's `inputK_dynamic_range`.
  * quantisation follows pytorch-quantization's fake-quant: q = clamp(rint(x * (127/amax)), +-127);
    the value of an int8 element is q * (amax/127); both factors are computed in fp32.
  * int8 conv: Wq from the per-channel weight ranges the same way, acc int32,
    y = acc * (s_x * s_w[c]) + bias (two fp32 roundings), ReLU, then int8 or fp16 store.
  * Add: value of an int8 operand is q * (amax(tensor)/127); one fp32 add; same stores.
  * SparseInverseConvolution (parity unpinned: no reference vector exists): the transposed convolution
    on the named strided rulebook, out[i] += W[k] x[o] for each of its pairs (i, o, k), kernel not
    flipped; pinned against torch's conv_transpose3d under that rule.
  * dense output forms (engine.hpp:26,114-123): NCHW32 / NHWzC are defined by their names over the
    [1, C * Z, H, W] view the exporters' tails build; an int8 dense output (the node carries
    input_dynamic_range) holds the fake-quantised fp32 value of every element at that range, and a tensor
    no convolution or Add reads is stored int8 with the dense node's range.  The closed engine's byte layout
    is not observable; the definitions are pinned element by element with explicit index arithmetic and an
    independent dense walk (tests/test_oracle_graph.py).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Dict, List, Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# SCN_ORACLE_LIB names another build of the same source (the sanitizer build of the Makefile's `sanitize` target)
_LIB_PATH = os.environ.get("SCN_ORACLE_LIB") or os.path.join(_HERE, "libscn_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "scn_oracle.cpp")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.scn_ref_hash.restype = C.c_uint64
        _lib.scn_ref_hash.argtypes = [C.c_uint64]
        _lib.scn_ref_half2float.restype = C.c_float
        _lib.scn_ref_half2float.argtypes = [C.c_uint16]
        _lib.scn_ref_float2half.restype = C.c_uint16
        _lib.scn_ref_float2half.argtypes = [C.c_float]
        _lib.scn_ref_rulebook_subm.restype = C.c_int64
        _lib.scn_ref_rulebook_sparse.restype = C.c_int64
        _lib.scn_ref_voxelize.restype = C.c_int
        _lib.scn_ref_num_threads.restype = C.c_int
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _i3(v):
    return (C.c_int * 3)(*[int(x) for x in v])


def _f3(v):
    return (C.c_float * 3)(*[float(x) for x in v])


def hash64(k: int) -> int:
    return int(lib().scn_ref_hash(C.c_uint64(k)))


def num_threads() -> int:
    return int(lib().scn_ref_num_threads())


def set_num_threads(n: int) -> None:
    lib().scn_ref_set_num_threads(C.c_int(n))


# ------------------------------------------------------------------------------- voxelization
def voxelize(points_f16: np.ndarray, min_range, max_range, voxel_size, grid_xyz, max_voxels=160000,
             max_points=10, order="zyx"):
    """Returns (features [nv, F] fp16, indices [nv, 4] int32, points_per_voxel [nv] int32).  Points are taken as
    fp16 unless the array is float32 (the raw sweep of CUDA-CenterPoint's preprocessing)."""
    f32 = np.asarray(points_f16).dtype == np.float32
    pts = np.ascontiguousarray(points_f16, dtype=np.float32 if f32 else np.float16)
    n, nf = pts.shape
    feats = np.zeros((max_voxels, nf), np.float16)
    idx = np.zeros((max_voxels, 4), np.int32)
    cnt = np.zeros((max_voxels,), np.int32)
    fn = lib().scn_ref_voxelize_f32 if f32 else lib().scn_ref_voxelize
    fn.restype = C.c_int
    nv = fn(_p(pts if f32 else pts.view(np.uint16)), C.c_int(n), C.c_int(nf), _f3(min_range), _f3(max_range),
            _f3(voxel_size), _i3(grid_xyz), C.c_int(max_voxels), C.c_int(max_points),
            C.c_int(2 if order == "zyx" else 1), _p(feats.view(np.uint16)), _p(idx), _p(cnt))
    return feats[:nv].copy(), idx[:nv].copy(), cnt[:nv].copy()


# ------------------------------------------------------------------------------- rulebooks
class Rulebook:
    """Pairs sorted by (offset, out, in).  offsets has kvol+1 entries."""

    def __init__(self, pair_in, pair_out, offsets, out_indices, out_grid, n_out, n_out_total=None):
        self.pair_in, self.pair_out, self.offsets = pair_in, pair_out, offsets
        self.out_indices, self.out_grid, self.n_out = out_indices, list(out_grid), int(n_out)
        self.n_out_total = int(n_out if n_out_total is None else n_out_total)

    @property
    def num_pairs(self) -> int:
        return int(self.offsets[-1])


def conv_out_size(in_size, ksize, stride, padding, dilation):
    out = (C.c_int * 3)()
    lib().scn_ref_conv_out_size(_i3(in_size), _i3(ksize), _i3(stride), _i3(padding), _i3(dilation), out)
    return [int(v) for v in out]


def rulebook_subm(indices: np.ndarray, grid, ksize, dilation=(1, 1, 1)) -> Rulebook:
    idx = np.ascontiguousarray(indices, dtype=np.int32)
    n = idx.shape[0]
    kvol = int(np.prod(ksize))
    cap = max(1, n * kvol)
    pin = np.empty(cap, np.int32)
    pout = np.empty(cap, np.int32)
    offs = np.zeros(kvol + 1, np.int64)
    npairs = lib().scn_ref_rulebook_subm(_p(idx), C.c_int(n), _i3(grid), _i3(ksize), _i3(dilation), _p(pin), _p(pout),
                                         _p(offs), C.c_int64(cap))
    assert npairs >= 0
    return Rulebook(pin[:npairs].copy(), pout[:npairs].copy(), offs, idx, grid, n)


def rulebook_sparse(indices: np.ndarray, grid, ksize, stride, padding, dilation=(1, 1, 1), max_out=200000) -> Rulebook:
    idx = np.ascontiguousarray(indices, dtype=np.int32)
    n = idx.shape[0]
    kvol = int(np.prod(ksize))
    cap = max(1, n * kvol)
    pin = np.empty(cap, np.int32)
    pout = np.empty(cap, np.int32)
    offs = np.zeros(kvol + 1, np.int64)
    oidx = np.zeros((max(1, max_out), 4), np.int32)
    ogrid = (C.c_int * 3)()
    n_out = C.c_int(0)
    n_tot = C.c_int(0)
    npairs = lib().scn_ref_rulebook_sparse(_p(idx), C.c_int(n), _i3(grid), _i3(ksize), _i3(stride), _i3(padding),
                                           _i3(dilation), C.c_int(max_out), _p(oidx), ogrid, C.byref(n_out),
                                           C.byref(n_tot), _p(pin), _p(pout), _p(offs), C.c_int64(cap))
    assert npairs >= 0
    return Rulebook(pin[:npairs].copy(), pout[:npairs].copy(), offs, oidx[:n_out.value].copy(),
                    [int(v) for v in ogrid], n_out.value, n_tot.value)


def rulebook_inverse(rb: Rulebook, in_indices: np.ndarray, in_grid) -> Rulebook:
    """Rulebook of a SparseInverseConvolution on the rulebook `rb` of a strided convolution whose input
    was (in_indices, in_grid): the same pairs with input and output swapped, so the outputs are that
    convolution's input rows; the kernel offset of a pair (and with it the weight slice) stays.
    (`inverse` argument of push_sparse_conv, libraries/3DSparseConvolution/libspconv/include/spconv/engine.hpp:139-156;
    the arithmetic behind it is not in the reference's sources: this rule is the transposed
    convolution, out[i] += W[k] x[o] for every pair (i, o, k) of the forward rulebook.)"""
    pin = np.empty_like(rb.pair_in)
    pout = np.empty_like(rb.pair_out)
    for k in range(len(rb.offsets) - 1):
        a, b = int(rb.offsets[k]), int(rb.offsets[k + 1])
        order = np.lexsort((rb.pair_out[a:b], rb.pair_in[a:b]))   # by new output (old input), then new input
        pin[a:b] = rb.pair_out[a:b][order]
        pout[a:b] = rb.pair_in[a:b][order]
    idx = np.ascontiguousarray(in_indices, np.int32)
    return Rulebook(pin, pout, rb.offsets.copy(), idx, list(in_grid), idx.shape[0])


# ------------------------------------------------------------------------------- conv + elementwise
def f32(v) -> np.float32:
    return np.float32(v)


def quantize_weights(w_f16: np.ndarray, ranges) -> Tuple[np.ndarray, np.ndarray]:
    """[Cout,K0,K1,K2,Cin] fp16 -> ([kvol][cout][cin] int8, s_w[cout] fp32)."""
    cout, cin = w_f16.shape[0], w_f16.shape[-1]
    s_w = (np.asarray(ranges, np.float32) / f32(127.0)).astype(np.float32)
    r_w = (f32(127.0) / np.asarray(ranges, np.float32)).astype(np.float32)
    w = w_f16.astype(np.float32).reshape(cout, -1, cin)
    q = np.rint(w * r_w[:, None, None])
    q = np.clip(q, -127, 127).astype(np.int8)
    return np.ascontiguousarray(q.transpose(1, 0, 2)), s_w


def conv_int8_acc(x_i8: np.ndarray, wq: np.ndarray, rb: Rulebook) -> np.ndarray:
    kvol, cout, cin = wq.shape
    x = np.ascontiguousarray(x_i8, np.int8)
    assert x.shape[1] == cin
    acc = np.empty((rb.n_out, cout), np.int32)
    lib().scn_ref_conv_int8_acc(_p(x), C.c_int(cin), _p(np.ascontiguousarray(wq)), C.c_int(cout), C.c_int(kvol),
                                _p(rb.pair_in), _p(rb.pair_out), _p(rb.offsets), _p(acc), C.c_int(rb.n_out))
    return acc


def conv_f32_acc(x_f32: np.ndarray, w_f32: np.ndarray, rb: Rulebook) -> np.ndarray:
    kvol, cout, cin = w_f32.shape
    x = np.ascontiguousarray(x_f32, np.float32)
    assert x.shape[1] == cin
    acc = np.empty((rb.n_out, cout), np.float32)
    lib().scn_ref_conv_f32_acc(_p(x), C.c_int(cin), _p(np.ascontiguousarray(w_f32, np.float32)), C.c_int(cout),
                               C.c_int(kvol), _p(rb.pair_in), _p(rb.pair_out), _p(rb.offsets), _p(acc),
                               C.c_int(rb.n_out))
    return acc


def epilogue(acc: np.ndarray, scale: Optional[np.ndarray], bias_f32: np.ndarray, relu: bool, out_int8: bool,
             out_range: float = 127.0) -> np.ndarray:
    n, cout = acc.shape
    out = np.empty((n, cout), np.int8 if out_int8 else np.float16)
    oi8 = _p(out) if out_int8 else None
    of16 = None if out_int8 else _p(out.view(np.uint16))
    bias = np.ascontiguousarray(bias_f32, np.float32)
    if acc.dtype == np.int32:
        lib().scn_ref_epilogue_int32(_p(np.ascontiguousarray(acc)), C.c_int64(n), C.c_int(cout),
                                     _p(np.ascontiguousarray(scale, np.float32)), _p(bias), C.c_int(int(relu)),
                                     C.c_float(out_range), oi8, of16)
    else:
        lib().scn_ref_epilogue_f32(_p(np.ascontiguousarray(acc, np.float32)), C.c_int64(n), C.c_int(cout), _p(bias),
                                   C.c_int(int(relu)), C.c_float(out_range), oi8, of16)
    return out


def quantize(x_f16: np.ndarray, rng: float) -> np.ndarray:
    x = np.ascontiguousarray(x_f16, np.float16)
    q = np.empty(x.shape, np.int8)
    lib().scn_ref_quantize(_p(x.view(np.uint16)), C.c_int64(x.size), C.c_float(rng), _p(q))
    return q


def quantize_f32(x_f32: np.ndarray, rng: float) -> np.ndarray:
    x = np.ascontiguousarray(x_f32, np.float32)
    q = np.empty(x.shape, np.int8)
    lib().scn_ref_quantize_f32(_p(x), C.c_int64(x.size), C.c_float(rng), _p(q))
    return q


def dequantize(q_i8: np.ndarray, rng: float) -> np.ndarray:
    q = np.ascontiguousarray(q_i8, np.int8)
    x = np.empty(q.shape, np.float16)
    lib().scn_ref_dequantize(_p(q), C.c_int64(q.size), C.c_float(rng), _p(x.view(np.uint16)))
    return x


def add(a: np.ndarray, a_range: float, b: np.ndarray, b_range: float, relu: bool, out_int8: bool,
        out_range: float = 127.0) -> np.ndarray:
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    out = np.empty(a.shape, np.int8 if out_int8 else np.float16)
    lib().scn_ref_add(_p(a) if a.dtype == np.int8 else None, _p(a.view(np.uint16)) if a.dtype == np.float16 else None,
                      C.c_float(a_range), _p(b) if b.dtype == np.int8 else None,
                      _p(b.view(np.uint16)) if b.dtype == np.float16 else None, C.c_float(b_range),
                      C.c_int64(a.size), C.c_int(int(relu)), C.c_float(out_range), _p(out) if out_int8 else None,
                      None if out_int8 else _p(out.view(np.uint16)))
    return out


def scatter_dense(feat: np.ndarray, indices: np.ndarray, dims) -> np.ndarray:
    feat = np.ascontiguousarray(feat)
    n, c = feat.shape
    dense = np.empty((1, c, int(dims[0]), int(dims[1]), int(dims[2])), feat.dtype)
    lib().scn_ref_scatter_dense(_p(feat), _p(np.ascontiguousarray(indices, np.int32)), C.c_int(n), C.c_int(c),
                                _i3(dims), C.c_int(feat.dtype.itemsize), _p(dense))
    return dense


def dense_to_layout(dense: np.ndarray, fmt: str, layout: str) -> np.ndarray:
    """[1, C, D0, D1, D2] -> the vectorised layouts of push_dense (engine.hpp:26): first the 4-D tensor
    [1, C * Z, H, W] the exporters' tails build (channel c * Z + z; z is the first spatial axis of "zyx" tensors,
    the last of "xyz" ones), then NCHW32 = [1, ceil(CZ / 32), H, W, 32] zero padded, NHWzC = [1, H, W, Z, C]."""
    if fmt == "xyz":
        dense = np.transpose(dense, (0, 1, 4, 2, 3))      # [1, C, Z, H, W]
    _, c, z, h, w = dense.shape
    if layout == "NHWzC":
        return np.ascontiguousarray(np.transpose(dense, (0, 3, 4, 2, 1)))
    if layout != "NCHW32":
        raise ValueError(layout)
    flat = np.ascontiguousarray(dense).reshape(1, c * z, h, w)
    groups = (c * z + 31) // 32
    pad = np.zeros((1, groups * 32, h, w), dense.dtype)
    pad[:, :c * z] = flat
    return np.ascontiguousarray(pad.reshape(1, groups, 32, h, w).transpose(0, 1, 3, 4, 2))


# ------------------------------------------------------------------------------- graph walk
class SparseT:
    """features (fp16, or int8 with its dynamic range `rng`), indices, grid."""

    def __init__(self, feat, rng, indices, grid):
        self.feat, self.rng, self.indices, self.grid = feat, rng, indices, list(grid)


def _consumers(graph):
    cons: Dict[str, List[Tuple[object, int]]] = {}
    for n in graph.nodes:
        for slot, t in enumerate(n.inputs):
            cons.setdefault(t, []).append((n, slot))
    return cons


def node_precisions(graph, engine_precision: str):
    """node name -> (compute, output) with values 'fp16' / 'int8' after the engine-level override."""
    out = {}
    for n in graph.nodes:
        comp = outp = "fp16"
        if engine_precision == "int8":
            if n.op_type == "SparseConvolution":
                cout = graph.initializers[n.inputs[1]].shape[0]
                ok = float(n.attrs.get("input_dynamic_range", 0.0)) > 0 and \
                    len(n.attrs.get("weight_dynamic_ranges", [])) == cout
                comp = "int8" if (n.attrs.get("precision", "") == "int8" and ok) else "fp16"
                outp = "int8" if n.attrs.get("output_precision", "") == "int8" else "fp16"
            elif n.op_type in ("Add", "QuantAdd"):
                ok = float(n.attrs.get("input0_dynamic_range", 0.0)) > 0 and \
                    float(n.attrs.get("input1_dynamic_range", 0.0)) > 0
                comp = "int8" if (n.attrs.get("precision", "") == "int8" and ok) else "fp16"
                outp = "int8" if n.attrs.get("output_precision", "") == "int8" else "fp16"
        out[n.name] = (comp, outp)
    return out


def tensor_ranges(graph, prec):
    """tensor name -> dynamic range (amax) fixed by its consumers (None when no consumer fixes one)."""
    cons = _consumers(graph)
    memo: Dict[str, Optional[np.float32]] = {}

    def req(t):
        if t in memo:
            return memo[t]
        memo[t] = None
        res = None
        cl = cons.get(t, [])
        for n, _ in cl:
            if n.op_type == "SparseConvolution" and prec[n.name][0] == "int8":
                res = f32(n.attrs["input_dynamic_range"])
                break
        if res is None:
            for n, _ in cl:
                if n.op_type == "Relu":
                    res = req(n.outputs[0])
                    if res is not None:
                        break
        if res is None:
            for n, slot in cl:
                if n.op_type in ("Add", "QuantAdd") and prec[n.name][0] == "int8":
                    res = f32(n.attrs[f"input{slot}_dynamic_range"])
                    break
        if res is None:
            for n, _ in cl:
                if n.op_type == "ScatterDense" and float(n.attrs.get("input_dynamic_range", 0.0)) > 0:
                    res = f32(n.attrs["input_dynamic_range"])
                    break
        memo[t] = res
        return res

    for n in graph.nodes:
        for t in n.outputs:
            req(t)
    return memo


def run_graph(graph, features_f16: np.ndarray, indices: np.ndarray, grid, precision: str = "fp16",
              record: Optional[dict] = None, override: Optional[dict] = None):
    """Walks the graph.  Returns {output name: ndarray (dense) or SparseT}.

    record, when given, receives per node name a dict with the rulebook, the accumulators (`acc`)
    and the stored output (`out`, plus its dynamic `range` for int8) of that node.
    override maps a tensor name to stored features that replace what the walk computed for that
    tensor (same dtype and shape).  Tests use it to re-base the walk on the device's own output of
    an fp16-computed node, whose summation order the oracle does not model, so that every int8 node
    downstream sees identical inputs and can be compared bit for bit.
    """
    prec = node_precisions(graph, precision)
    ranges = tensor_ranges(graph, prec)
    T: Dict[str, object] = {graph.inputs[0]: SparseT(np.ascontiguousarray(features_f16, np.float16), None,
                                                     np.ascontiguousarray(indices, np.int32), grid)}
    rb_cache: Dict[str, Rulebook] = {}

    def stored(out_prec, name):
        """(store int8?, dynamic range) for an output tensor."""
        if out_prec == "int8" and ranges.get(name) is not None:
            return True, float(ranges[name])
        return False, 127.0

    for n in graph.nodes:
        comp, outp = prec[n.name]
        rec = {} if record is not None else None
        if n.op_type == "SparseConvolution":
            x: SparseT = T[n.inputs[0]]
            a = n.attrs
            w = graph.initializers[n.inputs[1]]
            bias = graph.initializers[n.inputs[2]].astype(np.float32)
            ks, dil = a["kernel_size"], a.get("dilation", [1, 1, 1]) or [1, 1, 1]
            key = a.get("rulebook", "")
            if a.get("inverse", 0):
                fwd = rb_cache.get("conv:" + key)
                if fwd is None or not np.array_equal(fwd.out_indices, x.indices):
                    raise ValueError(f"node {n.name}: inverse convolution needs the rulebook '{key}' of an earlier "
                                     f"strided convolution whose output it runs on")
                rb = rb_cache.get("inv:" + key)
                if rb is None:
                    rb = rb_cache["inv:" + key] = rulebook_inverse(fwd, fwd.in_indices, fwd.in_grid)
            elif a.get("subm", 0):
                ck = "subm:" + key
                rb = rb_cache.get(ck) if key else None
                if rb is None:
                    rb = rulebook_subm(x.indices, x.grid, ks, dil)
                    if key:
                        rb_cache[ck] = rb
            else:
                ck = "conv:" + key
                rb = rb_cache.get(ck) if key else None
                if rb is None:
                    rb = rulebook_sparse(x.indices, x.grid, ks, a["stride"], a["padding"], dil,
                                         int(a.get("output_bound", 150000)))
                    rb.in_indices, rb.in_grid = x.indices, list(x.grid)
                    if key:
                        rb_cache[ck] = rb
            relu = a.get("activation", "") == "ReLU"
            o_i8, r_out = stored(outp, n.outputs[0])
            if comp == "int8":
                if x.feat.dtype == np.int8:
                    xq, x_rng = x.feat, f32(x.rng)
                else:
                    x_rng = f32(a["input_dynamic_range"])
                    xq = quantize(x.feat, float(x_rng))
                s_x = x_rng / f32(127.0)
                wq, s_w = quantize_weights(w, a["weight_dynamic_ranges"])
                acc = conv_int8_acc(xq, wq, rb)
                out = epilogue(acc, (s_x * s_w).astype(np.float32), bias, relu, o_i8, r_out)
            else:
                xf = x.feat if x.feat.dtype == np.float16 else dequantize(x.feat, float(x.rng))
                cout, cin = w.shape[0], w.shape[-1]
                wf = np.ascontiguousarray(w.astype(np.float32).reshape(cout, -1, cin).transpose(1, 0, 2))
                acc = conv_f32_acc(xf.astype(np.float32), wf, rb)
                out = epilogue(acc, None, bias, relu, o_i8, r_out)
            T[n.outputs[0]] = SparseT(out, r_out if o_i8 else None, rb.out_indices, rb.out_grid)
            if rec is not None:
                rec.update(rulebook=rb, acc=acc, out=out, range=r_out if o_i8 else None)
        elif n.op_type in ("Add", "QuantAdd"):
            A: SparseT = T[n.inputs[0]]
            B: SparseT = T[n.inputs[1]]
            fa, ra, fb, rb_ = A.feat, A.rng, B.feat, B.rng
            if comp == "int8":
                if fa.dtype == np.float16:
                    ra = float(f32(n.attrs["input0_dynamic_range"]))
                    fa = quantize(fa, ra)
                if fb.dtype == np.float16:
                    rb_ = float(f32(n.attrs["input1_dynamic_range"]))
                    fb = quantize(fb, rb_)
            o_i8, r_out = stored(outp, n.outputs[0])
            out = add(fa, ra or 127.0, fb, rb_ or 127.0, False, o_i8, r_out)
            T[n.outputs[0]] = SparseT(out, r_out if o_i8 else None, A.indices, A.grid)
            if rec is not None:
                rec.update(out=out, range=r_out if o_i8 else None)
        elif n.op_type == "Relu":
            X: SparseT = T[n.inputs[0]]
            out = np.maximum(X.feat, X.feat.dtype.type(0))
            T[n.outputs[0]] = SparseT(out, X.rng, X.indices, X.grid)
            if rec is not None:
                rec.update(out=out, range=X.rng)
        elif n.op_type == "ScatterDense":
            X = T[n.inputs[0]]
            oshape = [int(v) for v in n.attrs["output_shape"]]
            out_rng = float(n.attrs.get("input_dynamic_range", 0.0) or 0.0)
            layout = n.attrs.get("output_layout", "") or "NCHW"
            if out_rng > 0 and precision == "int8":
                # int8 dense output (push_dense's input_dynamic_range, engine.hpp:121): the fp32 value of every
                # element, quantised with the node's range
                val = X.feat.astype(np.float32) if X.feat.dtype == np.float16 else \
                    X.feat.astype(np.float32) * (f32(X.rng) / f32(127.0))
                dense = scatter_dense(quantize_f32(val, out_rng), X.indices, oshape[2:5])
            else:
                feat = X.feat if X.feat.dtype == np.float16 else dequantize(X.feat, float(X.rng))
                dense = scatter_dense(feat, X.indices, oshape[2:5])
            if layout != "NCHW":
                dense = dense_to_layout(dense, n.attrs.get("format", "zyx"), layout)
                T["__fixed_form__" + n.outputs[0]] = True
            T[n.outputs[0]] = dense
            if rec is not None:
                rec.update(out=dense)
        elif n.op_type in ("Reshape", "Transpose") and T.get("__fixed_form__" + n.inputs[0]):
            # a tensor in a vectorised layout already is the final tensor: the exporter's tail leaves it as it is
            T[n.outputs[0]] = T[n.inputs[0]]
            T["__fixed_form__" + n.outputs[0]] = True
            if rec is not None:
                rec.update(out=T[n.outputs[0]])
        elif n.op_type == "Reshape":
            T[n.outputs[0]] = np.ascontiguousarray(T[n.inputs[0]]).reshape([int(v) for v in n.attrs["dims"]])
            if rec is not None:
                rec.update(out=T[n.outputs[0]])
        elif n.op_type == "Transpose":
            T[n.outputs[0]] = np.ascontiguousarray(np.transpose(T[n.inputs[0]], [int(v) for v in n.attrs["dims"]]))
            if rec is not None:
                rec.update(out=T[n.outputs[0]])
        else:
            raise ValueError(f"Unsupport operator [{n.op_type}]")
        if override and n.outputs[0] in override and isinstance(T[n.outputs[0]], SparseT):
            t = T[n.outputs[0]]
            new = np.ascontiguousarray(override[n.outputs[0]])[:, :t.feat.shape[1]]
            assert new.dtype == t.feat.dtype and new.shape == t.feat.shape, n.name
            t.feat = new
            if rec is not None:
                rec["out"] = new
        if record is not None:
            record[n.name] = rec
    return {name: T[name] for name in graph.outputs}
