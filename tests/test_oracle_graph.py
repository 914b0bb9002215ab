"""Pins the oracle's graph walk (oracle/scn_oracle.py: run_graph, node_precisions, tensor_ranges) against an
independent walk written here from the exporters' rules, on dense grids.

What the oracle's walk decides and nothing else in the CPU suite checks: how the active set propagates
through SubM / strided / inverse convolutions, that rulebooks shared by key are the right ones, with which
dynamic range every int8 tensor is stored and with which one an Add reads each operand, where bias and
ReLU act, and the dense layout of the tail (ScatterDense, Transpose, Reshape).  The walk below shares no
code with it:

  * tensors are zero-filled dense grids [C, D0, D1, D2] plus an occupancy mask; a convolution is
    torch.nn.functional.conv3d / conv_transpose3d in float64 (exact for int8 codes: |sum| < 2^53),
    weights [Cout, K0, K1, K2, Cin] -> [Cout, Cin, K0, K1, K2], kernel not flipped; SubM keeps the mask,
    a strided convolution's mask is where the occupancy convolution is non-zero, an inverse one's is the
    mask of the strided convolution's input (spconv semantics the exporters trace:
    libraries/3DSparseConvolution/tool/centerpoint-export/exptool.py:69-135);
  * fake quantisation as in pytorch-quantization, which the exporter reads its ranges from
    (CUDA-CenterPoint/qat/tools/sparseconv_quantization.py:51-60,116-128): per-tensor activations,
    per-output-channel weights, code = clamp(rint(x * 127 / amax), +-127), value = code * amax / 127;
  * the dynamic range each tensor is stored with is found by pushing ranges from consumers to the tensors
    they read (the oracle pulls them from the producer's side);
  * tail: dense().view() of the CenterPoint exporter (exptool.py:159-183) and dense().permute().reshape()
    of the BEVFusion one (CUDA-BEVFusion/qat/lean/exptool.py:285-293), as numpy calls.

All-int8 plans must agree bit for bit; fp16 graphs within the tolerance stated in the GPU tests; a walk
that reads an Add operand with the Add's own range instead of the tensor's stored range must NOT agree.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from lidar_ai_solution_amd import graphs
from oracle import scn_oracle as O

F32 = np.float32
FP16_REL = 1e-2   # max-abs <= FP16_REL * max|reference| after the whole backbone
FP16_COS = 0.9999


# ------------------------------------------------------------------------------------------ inputs
def blob_voxels(seed, grid, n_blobs=14, per_blob=260, plane_axis=0, plane_at=6, plane_n=900):
    """A few thousand unique voxels: a sparse plane (rows whose neighbours all lie in one slice) plus
    dense blobs (rows with up to 27 neighbours), the two populations of a lidar frame."""
    rng = np.random.default_rng(seed)
    g = np.asarray(grid)
    cells = []
    for _ in range(n_blobs):
        c = rng.integers(0, g)
        d = np.rint(rng.normal(0, 2.2, size=(per_blob, 3))).astype(np.int64)
        cells.append(c + d)
    p = rng.integers(0, g, size=(plane_n, 3))
    p[:, plane_axis] = plane_at
    cells.append(p)
    cells = np.concatenate(cells)
    ok = np.all((cells >= 0) & (cells < g), axis=1)
    cells = np.unique(cells[ok], axis=0)          # ascending linear order
    idx = np.concatenate([np.zeros((len(cells), 1), np.int64), cells], axis=1).astype(np.int32)
    feats = rng.normal(0, 1.0, size=(len(cells), 5)).astype(np.float16)
    return feats, idx


# ------------------------------------------------------------------------------------------ the dense walk
class Dense:
    """val: float64 [C, D0, D1, D2]: int8 codes when rng is set, fp16-representable values otherwise."""

    def __init__(self, val, mask, rng=None):
        self.val, self.mask, self.rng = val, mask, rng


def _quant(y32, amax):
    r = F32(127.0) / F32(amax)
    return np.clip(np.rint(y32.astype(F32) * r), -127, 127)


def _store(y32, mask, int8_range):
    """fp32 values -> stored form, zero outside the active set."""
    if int8_range is not None:
        v = _quant(y32, int8_range).astype(np.float64)
    else:
        v = y32.astype(np.float16).astype(np.float64)
    return v * mask[None]


def _compute_kinds(graph, precision):
    kinds = {}
    for n in graph.nodes:
        comp = outp = "fp16"
        a = n.attrs
        if precision == "int8" and n.op_type == "SparseConvolution":
            cout = graph.initializers[n.inputs[1]].shape[0]
            if a.get("precision") == "int8" and a.get("input_dynamic_range", 0) > 0 and \
                    len(a.get("weight_dynamic_ranges", ())) == cout:
                comp = "int8"
            outp = "int8" if a.get("output_precision") == "int8" else "fp16"
        elif precision == "int8" and n.op_type == "Add":
            if a.get("precision") == "int8" and a.get("input0_dynamic_range", 0) > 0 and a.get("input1_dynamic_range", 0) > 0:
                comp = "int8"
            outp = "int8" if a.get("output_precision") == "int8" else "fp16"
        kinds[n.name] = (comp, outp)
    return kinds


def _pushed_ranges(graph, kinds):
    """Consumers push the range they read with onto the tensor: int8 convolutions first, then int8 Adds
    for tensors no convolution reads; a Relu hands its output's range to its input."""
    rng = {}
    relus = [n for n in graph.nodes if n.op_type == "Relu"]

    def through_relus():
        changed = True
        while changed:
            changed = False
            for n in relus:
                if n.outputs[0] in rng and n.inputs[0] not in rng:
                    rng[n.inputs[0]] = rng[n.outputs[0]]
                    changed = True

    for n in graph.nodes:
        if n.op_type == "SparseConvolution" and kinds[n.name][0] == "int8":
            rng.setdefault(n.inputs[0], F32(n.attrs["input_dynamic_range"]))
    through_relus()
    for n in graph.nodes:
        if n.op_type == "Add" and kinds[n.name][0] == "int8":
            for slot in (0, 1):
                rng.setdefault(n.inputs[slot], F32(n.attrs[f"input{slot}_dynamic_range"]))
    through_relus()
    for n in graph.nodes:   # an int8 dense output quantises with its own range a tensor nobody else fixed
        if n.op_type == "ScatterDense" and float(n.attrs.get("input_dynamic_range", 0.0) or 0.0) > 0:
            rng.setdefault(n.inputs[0], F32(n.attrs["input_dynamic_range"]))
    through_relus()
    return rng


def _conv3d(x, w, **kw):
    return F.conv3d(torch.from_numpy(x)[None], torch.from_numpy(w), **kw)[0].numpy()


def dense_walk(graph, feats, idx, grid, precision, record=None, rebase=None, add_reads_with_own_range=False):
    """Returns the graph outputs (numpy arrays for dense ones, Dense for sparse ones).  record receives
    the stored Dense of every node output.  rebase maps a tensor name to a Dense that replaces the walk's
    own result for it."""
    kinds = _compute_kinds(graph, precision)
    ranges = _pushed_ranges(graph, kinds)
    grid = tuple(int(v) for v in grid)
    x0 = np.zeros((feats.shape[1],) + grid)
    m0 = np.zeros(grid)
    x0[:, idx[:, 1], idx[:, 2], idx[:, 3]] = feats.astype(np.float64).T
    m0[idx[:, 1], idx[:, 2], idx[:, 3]] = 1.0
    T = {graph.inputs[0]: Dense(x0, m0)}
    strided_in = {}   # rulebook key -> (mask, grid) of the strided convolution's input
    fixed_form = set()

    def value(t: Dense):
        """fp32 value of every stored element."""
        if t.rng is None:
            return t.val.astype(F32)
        return t.val.astype(F32) * (F32(t.rng) / F32(127.0))

    for n in graph.nodes:
        a = n.attrs
        comp, outp = kinds[n.name]
        name = n.outputs[0]
        out_rng = ranges.get(name) if outp == "int8" else None
        if n.op_type == "SparseConvolution":
            x = T[n.inputs[0]]
            w16 = graph.initializers[n.inputs[1]]
            bias = graph.initializers[n.inputs[2]].astype(F32)
            ks = [int(v) for v in a["kernel_size"]]
            dil = [int(v) for v in (a.get("dilation") or [1, 1, 1])]
            st = [int(v) for v in a["stride"]]
            pd = [int(v) for v in a["padding"]]
            if comp == "int8":
                if x.rng is None:
                    x_rng = F32(a["input_dynamic_range"])
                    xin = _quant(x.val.astype(F32), x_rng).astype(np.float64)
                else:
                    x_rng, xin = F32(x.rng), x.val
                wr = np.asarray(a["weight_dynamic_ranges"], F32)
                wq = np.clip(np.rint(w16.astype(F32) * (F32(127.0) / wr)[:, None, None, None, None]), -127, 127)
                wk = wq.astype(np.float64)
                scale = ((x_rng / F32(127.0)) * (wr / F32(127.0))).astype(F32)
            else:
                xin = value(x).astype(np.float64)
                wk = w16.astype(np.float64)
                scale = None
            wk = np.ascontiguousarray(np.transpose(wk, (0, 4, 1, 2, 3)))   # [Cout, Cin, K0, K1, K2]
            if a.get("inverse", 0):
                in_mask, in_grid = strided_in[a["rulebook"]]
                opad = [in_grid[i] - ((x.mask.shape[i] - 1) * st[i] - 2 * pd[i] + dil[i] * (ks[i] - 1) + 1) for i in range(3)]
                acc = F.conv_transpose3d(torch.from_numpy(xin)[None],
                                         torch.from_numpy(np.ascontiguousarray(np.transpose(wk, (1, 0, 2, 3, 4)))),
                                         stride=st, padding=pd, output_padding=opad, dilation=dil)[0].numpy()
                mask = in_mask
            elif a.get("subm", 0):
                acc = _conv3d(xin, wk, padding=[(ks[i] // 2) * dil[i] for i in range(3)], dilation=dil)
                mask = x.mask
            else:
                acc = _conv3d(xin, wk, stride=st, padding=pd, dilation=dil)
                occ = _conv3d(x.mask[None], np.ones((1, 1, *ks)), stride=st, padding=pd, dilation=dil)[0]
                mask = (occ > 0).astype(np.float64)
                if a.get("rulebook"):
                    strided_in[a["rulebook"]] = (x.mask, x.mask.shape)
            y = acc.astype(F32)
            if scale is not None:
                y = y * scale[:, None, None, None]
            y = y + bias[:, None, None, None]
            if a.get("activation", "") == "ReLU":
                y = np.maximum(y, F32(0))
            T[name] = Dense(_store(y, mask, out_rng), mask, out_rng)
        elif n.op_type == "Add":
            ops = []
            for slot in (0, 1):
                t = T[n.inputs[slot]]
                own = F32(a.get(f"input{slot}_dynamic_range", 0.0))
                if t.rng is None and comp == "int8":
                    ops.append(_quant(t.val.astype(F32), own).astype(F32) * (own / F32(127.0)))
                elif t.rng is not None and add_reads_with_own_range and comp == "int8":
                    ops.append(t.val.astype(F32) * (own / F32(127.0)))
                else:
                    ops.append(value(t))
            y = ops[0] + ops[1]
            mask = T[n.inputs[0]].mask
            T[name] = Dense(_store(y, mask, out_rng), mask, out_rng)
        elif n.op_type == "Relu":
            t = T[n.inputs[0]]
            T[name] = Dense(np.maximum(t.val, 0.0), t.mask, t.rng)
        elif n.op_type == "ScatterDense":
            T[name], fixed = dense_tail(T[n.inputs[0]], n, precision)   # [1, C, D0, D1, D2], zero outside the mask
            if fixed:
                fixed_form.add(name)
        elif n.op_type in ("Reshape", "Transpose") and n.inputs[0] in fixed_form:
            T[name] = T[n.inputs[0]]          # a vectorised layout already is the final tensor
            fixed_form.add(name)
        elif n.op_type == "Reshape":
            T[name] = np.ascontiguousarray(T[n.inputs[0]]).reshape([int(v) for v in a["dims"]])
        elif n.op_type == "Transpose":
            T[name] = np.transpose(T[n.inputs[0]], [int(v) for v in a["dims"]])
        else:
            raise AssertionError(n.op_type)
        if rebase and name in rebase:
            T[name] = rebase[name]
        if record is not None:
            record[n.name] = T[name]
    return {o: T[o] for o in graph.outputs}


# ------------------------------------------------------------------------------------------ comparison helpers
def to_dense(t: O.SparseT):
    """The oracle's sparse tensor on a dense grid: (values float64 [C, *grid], mask)."""
    g = tuple(t.grid)
    v = np.zeros((t.feat.shape[1],) + g)
    m = np.zeros(g)
    i = t.indices
    v[:, i[:, 1], i[:, 2], i[:, 3]] = t.feat.astype(np.float64).T
    m[i[:, 1], i[:, 2], i[:, 3]] = 1.0
    return v, m


def rows_in_canonical_order(t: O.SparseT):
    i = t.indices.astype(np.int64)
    lin = (i[:, 1] * t.grid[1] + i[:, 2]) * t.grid[2] + i[:, 3]
    return np.all(np.diff(lin) > 0)


def calibrate(graph, feats, idx, grid):
    """Per-tensor |max| percentile from the dense walk in fp16 (the int8 configurations' rule)."""
    rec = {}
    dense_walk(graph, feats, idx, grid, "fp16", rec)
    amax = {graph.inputs[0]: graphs.percentile_amax(np.abs(feats.astype(F32)))}
    for n in graph.nodes:
        if n.op_type in ("SparseConvolution", "Add", "Relu"):
            t = rec[n.name]
            amax[n.outputs[0]] = graphs.percentile_amax(np.abs(t.val[:, t.mask > 0]).astype(F32))
    return amax


CP_GRID = (41, 64, 64)
BEV_GRID = (64, 64, 41)
CHANNELS = (16, 16, 32, 32)


def _cp(seed=3):
    feats, idx = blob_voxels(seed, CP_GRID, plane_axis=0, plane_at=6)
    return feats, idx, CP_GRID


def _bev(seed=4):
    feats, idx = blob_voxels(seed, BEV_GRID, plane_axis=2, plane_at=6)
    return feats, idx, BEV_GRID


def _graph(kind, seed, plan=None, data=None):
    make = {"centerpoint": graphs.centerpoint_scn, "bevfusion": graphs.bevfusion_scn}.get(kind)
    if kind == "centerpoint":
        g, tags = make(seed=seed, grid_zyx=CP_GRID, channels=CHANNELS, weight_std=0.08)
    elif kind == "bevfusion":
        g, tags = make(seed=seed, grid_xyz=BEV_GRID, channels=CHANNELS, weight_std=0.08)
    else:
        g, tags = graphs.unet_scn(seed=seed, channels=(16, 16, 32), weight_std=0.08)
    if plan:
        graphs.apply_int8_plan(g, tags, calibrate(g, *data), plan)
    return g


def _check_every_tensor(graph, precision, data, rebase_fp16=False):
    """Walks both ways and compares every node output.  Returns (#bit-exact int8 tensors, #fp16 tensors)."""
    feats, idx, grid = data
    rec_o = {}
    out_o = O.run_graph(graph, feats, idx, grid, precision, rec_o)
    kinds = _compute_kinds(graph, precision)
    assert kinds == O.node_precisions(graph, precision)
    rebase = None
    if rebase_fp16:
        # fp16-computed convolutions: the two walks sum in different orders (fp32 pair order against float64),
        # so the dense walk continues from the oracle's stored result of those nodes, after checking that its
        # own is within the fp16 tolerance of it
        own = {}
        dense_walk(graph, feats, idx, grid, precision, own)
        rebase = {}
        for n in graph.nodes:
            if n.op_type == "SparseConvolution" and kinds[n.name][0] == "fp16":
                t = T_of(rec_o, out_o, graph, n)
                v, m = to_dense(t)
                assert np.array_equal(m, own[n.name].mask), n.name
                ref = v * (1.0 if t.rng is None else t.rng / 127.0)
                mine = own[n.name].val * (1.0 if own[n.name].rng is None else float(own[n.name].rng) / 127.0)
                assert np.abs(mine - ref).max() <= FP16_REL * max(np.abs(ref).max(), 1e-6), n.name
                rebase[n.outputs[0]] = Dense(v, m, None if t.rng is None else F32(t.rng))
    rec_d = {}
    out_d = dense_walk(graph, feats, idx, grid, precision, rec_d, rebase=rebase)
    n_i8 = n_f16 = 0
    for n in graph.nodes:
        if n.op_type in ("SparseConvolution", "Add", "Relu"):
            t = T_of(rec_o, out_o, graph, n)
            d = rec_d[n.name]
            assert rows_in_canonical_order(t), n.name
            v, m = to_dense(t)
            assert np.array_equal(m, d.mask), f"active set of {n.name}"
            assert (t.rng is None) == (d.rng is None), f"storage type of {n.name}"
            if t.rng is not None:
                assert F32(t.rng) == F32(d.rng), f"dynamic range of {n.name}: {t.rng} vs {d.rng}"
                assert np.array_equal(v, d.val), f"int8 codes of {n.name}"
                n_i8 += 1
            elif precision == "int8" and not (n.op_type == "SparseConvolution" and kinds[n.name][0] == "fp16" and not rebase_fp16):
                # int8 arithmetic (or a rebased fp16 node) stored as fp16: no summation order is involved
                assert np.array_equal(v, d.val), f"fp16 values of {n.name}"
                n_f16 += 1
            else:
                assert np.abs(v - d.val).max() <= FP16_REL * max(np.abs(v).max(), 1e-6), f"fp16 values of {n.name}"
                n_f16 += 1
        else:
            assert np.array_equal(np.asarray(rec_o[n.name]["out"]).shape, np.asarray(rec_d[n.name]).shape), n.name
    return out_o, out_d, n_i8, n_f16


def T_of(rec_o, out_o, graph, n):
    """The oracle's SparseT for node n's output, rebuilt from its record (stored features + range) and the
    rulebook / input it was computed on."""
    r = rec_o[n.name]
    if n.op_type == "SparseConvolution":
        rb = r["rulebook"]
        return O.SparseT(r["out"], r["range"], rb.out_indices[:rb.n_out], rb.out_grid)
    # Add / Relu keep their first operand's coordinates: find them by walking up
    producer = {m.outputs[0]: m for m in graph.nodes}
    t = n.inputs[0]
    while producer[t].op_type != "SparseConvolution":
        t = producer[t].inputs[0]
    rb = rec_o[producer[t].name]["rulebook"]
    return O.SparseT(r["out"], r["range"], rb.out_indices[:rb.n_out], rb.out_grid)


# ------------------------------------------------------------------------------------------ tests
@pytest.mark.parametrize("kind,data_fn", [("centerpoint", _cp), ("bevfusion", _bev)])
def test_all_int8_walk_is_bit_exact_against_dense_walk(kind, data_fn):
    data = data_fn()
    assert 2500 < data[0].shape[0] < 8000
    g = _graph(kind, 11, "all-int8", data)
    out_o, out_d, n_i8, n_f16 = _check_every_tensor(g, "int8", data)
    assert n_i8 >= 29 and n_f16 == 1, (n_i8, n_f16)   # the last convolution's output has no quantising consumer
    name = g.outputs[0]
    assert out_o[name].shape == out_d[name].shape == (1, CHANNELS[3] * 2, 8, 8)
    assert np.array_equal(out_o[name].view(np.uint16), out_d[name].view(np.uint16))
    assert np.count_nonzero(out_d[name]) > 50


@pytest.mark.parametrize("kind,data_fn", [("centerpoint", _cp), ("bevfusion", _bev)])
def test_exporter_plans_bit_exact_downstream_of_the_fp16_nodes(kind, data_fn):
    """The reference's own precision plans (conv_input and, for CenterPoint, the first block in fp16;
    the last convolution's output in fp16)."""
    data = data_fn()
    g = _graph(kind, 12, kind, data)
    out_o, out_d, n_i8, n_f16 = _check_every_tensor(g, "int8", data, rebase_fp16=True)
    assert n_i8 >= (23 if kind == "centerpoint" else 28) and n_f16 >= (4 if kind == "centerpoint" else 1), (n_i8, n_f16)
    name = g.outputs[0]
    assert np.array_equal(out_o[name].view(np.uint16), out_d[name].view(np.uint16))


@pytest.mark.parametrize("kind,data_fn", [("centerpoint", _cp), ("bevfusion", _bev), ("unet", _cp)])
def test_fp16_walk_within_tolerance_of_dense_walk(kind, data_fn):
    data = data_fn()
    g = _graph(kind, 13)
    out_o, out_d, n_i8, n_f16 = _check_every_tensor(g, "fp16", data)
    assert n_i8 == 0 and n_f16 >= 20
    name = g.outputs[0]
    if kind == "unet":
        return
    a, b = out_o[name].astype(F32).ravel(), out_d[name].astype(F32).ravel()
    assert np.abs(a - b).max() <= FP16_REL * np.abs(b).max()
    assert np.dot(a, b) / (np.linalg.norm(a) * np.linalg.norm(b)) >= FP16_COS
    assert np.array_equal(a != 0, b != 0) or np.mean((a != 0) != (b != 0)) < 1e-3


def test_unet_with_inverse_convolutions_all_int8_bit_exact():
    data = _cp(5)
    g = _graph("unet", 14, "all-int8", data)
    out_o, out_d, n_i8, _ = _check_every_tensor(g, "int8", data)
    assert n_i8 >= 20
    t = out_o[g.outputs[0]]
    v, m = to_dense(t)
    d = out_d[g.outputs[0]]
    assert np.array_equal(m, d.mask) and np.array_equal(v, d.val) and t.rng is None and d.rng is None   # fp16: no consumer


def test_a_wrong_range_for_an_add_operand_is_caught():
    """Sensitivity of the comparison: a walk that reads the block input of an Add with the Add's own range
    (instead of the range the tensor is stored with, fixed by the convolution that also reads it) must
    differ from the oracle.  The calibrated plan gives the two different values for every block."""
    data = _cp()
    g = _graph("centerpoint", 11, "all-int8", data)
    adds = [n for n in g.nodes if n.op_type == "Add"]
    convs_in = {n.inputs[0]: n.attrs["input_dynamic_range"] for n in g.nodes if n.op_type == "SparseConvolution"}
    assert any(F32(convs_in[a.inputs[1]]) != F32(a.attrs["input1_dynamic_range"]) for a in adds if a.inputs[1] in convs_in)
    feats, idx, grid = data
    want = O.run_graph(g, feats, idx, grid, "int8")[g.outputs[0]]
    good = dense_walk(g, feats, idx, grid, "int8")[g.outputs[0]]
    bad = dense_walk(g, feats, idx, grid, "int8", add_reads_with_own_range=True)[g.outputs[0]]
    assert np.array_equal(want.view(np.uint16), good.view(np.uint16))
    assert not np.array_equal(want.view(np.uint16), bad.view(np.uint16))


def test_one_range_per_tensor_against_per_consumer_fake_quant():
    """How far the one-range-per-tensor rule is from per-consumer fake quantisation (the QAT graph, where the
    Add's quantiser re-quantises the block input with its own amax): the block input read by the Add differs
    by at most half a step of each of the two quantisers."""
    data = _cp()
    g = _graph("centerpoint", 11, "all-int8", data)
    feats, idx, grid = data
    rec = {}
    dense_walk(g, feats, idx, grid, "int8", rec)
    producer = {n.outputs[0]: n for n in g.nodes}
    worst = 0.0
    for n in g.nodes:
        if n.op_type != "Add":
            continue
        t = rec[producer[n.inputs[1]].name]
        own = F32(n.attrs["input1_dynamic_range"])
        stored = t.val.astype(F32) * (F32(t.rng) / F32(127.0))
        per_consumer = _quant(stored, own).astype(F32) * (own / F32(127.0))     # what fq(x, amax_add) would read
        step = max(float(own), float(t.rng)) / 127.0
        diff = float(np.abs(per_consumer - stored).max())
        assert diff <= 0.5 * float(own) / 127.0 + 1e-6
        worst = max(worst, diff / step)
    print(f"one range per tensor vs per-consumer fake-quant: worst difference {worst:.3f} quantisation steps")
    assert worst <= 0.5 + 1e-6


# ------------------------------------------------------------------------------------------ dense output forms
# push_dense's vectorised layouts and int8 output (engine.hpp:26,114-123; src/onnx-parser.cpp:196-203).  The
# definitions are closed forms over the [1, C * Z, H, W] tensor the exporters' tails build (channel c * Z + z:
# tool/centerpoint-export/exptool.py:159-183 for zyx, CUDA-BEVFusion/qat/lean/exptool.py:285-293 for xyz, whose
# dense tensor is [1, C, X, Y, Z] and whose H, W are X, Y).  They are written here element by element with
# explicit index arithmetic; nothing below calls numpy's transpose or reshape on the data.
def _view_axes(fmt, d0, d1, d2):
    """(Z, H, W) and a function (z, h, w) -> (i0, i1, i2) of the [1, C, D0, D1, D2] dense tensor."""
    if fmt == "zyx":
        return (d0, d1, d2), (lambda z, h, w: (z, h, w))
    return (d2, d0, d1), (lambda z, h, w: (h, w, z))


def layout_by_index_arithmetic(dense, fmt, layout, swap_z_and_c=False):
    _, C, d0, d1, d2 = dense.shape
    (Z, H, W), at = _view_axes(fmt, d0, d1, d2)
    if layout == "NCHW32":
        groups = (C * Z + 31) // 32
        flat = np.zeros(groups * H * W * 32, dense.dtype)
        shape = (1, groups, H, W, 32)
    elif layout == "NHWzC":
        flat = np.zeros(H * W * Z * C, dense.dtype)
        shape = (1, H, W, Z, C)
    else:
        flat = np.zeros(C * Z * H * W, dense.dtype)
        shape = (1, C * Z, H, W)
    for c in range(C):
        for z in range(Z):
            cz = c * Z + z
            for h in range(H):
                for w in range(W):
                    v = dense[(0, c) + at(z, h, w)]
                    if layout == "NCHW32":
                        flat[(((cz // 32) * H + h) * W + w) * 32 + cz % 32] = v
                    elif layout == "NHWzC":
                        flat[(((h * W + w) * C + c) * Z + z) if swap_z_and_c else (((h * W + w) * Z + z) * C + c)] = v
                    else:
                        flat[(cz * H + h) * W + w] = v
    return flat.reshape(shape)


@pytest.mark.parametrize("fmt", ["zyx", "xyz"])
def test_dense_to_layout_by_explicit_index_arithmetic(fmt):
    """Every element distinct, C * Z = 48 so that NCHW32 pads its second group with zeros."""
    C, Z, H, W = 24, 2, 5, 7
    dims = (Z, H, W) if fmt == "zyx" else (H, W, Z)
    dense = (np.arange(C * Z * H * W, dtype=np.int32) + 1).reshape(1, C, *dims).astype(np.float32).astype(np.float16)
    assert len(np.unique(dense)) == dense.size   # 1 .. 1680 are exact in fp16
    for layout in ("NCHW32", "NHWzC"):
        want = layout_by_index_arithmetic(dense, fmt, layout)
        got = O.dense_to_layout(dense, fmt, layout)
        assert got.shape == want.shape and np.array_equal(got, want), (fmt, layout)
    pad = O.dense_to_layout(dense, fmt, "NCHW32")
    assert pad.shape == (1, 2, H, W, 32) and np.count_nonzero(pad[0, 1, :, :, 16:]) == 0 and np.count_nonzero(pad) == dense.size
    # sensitivity: a definition with z and C swapped in NHWzC, or the other format's axis convention, is a different tensor
    assert not np.array_equal(layout_by_index_arithmetic(dense, fmt, "NHWzC", swap_z_and_c=True).ravel(),
                              O.dense_to_layout(dense, fmt, "NHWzC").ravel())
    other = "xyz" if fmt == "zyx" else "zyx"
    wrong_axes = np.ascontiguousarray(dense.reshape(1, C, *((H, W, Z) if fmt == "zyx" else (Z, H, W))))
    assert not np.array_equal(O.dense_to_layout(wrong_axes, other, "NCHW32").ravel(), pad.ravel())
    # the plain NCHW tail of the exporters, by the same arithmetic, against their own numpy calls
    tail = dense.reshape(1, C * Z, H, W) if fmt == "zyx" else np.transpose(dense, (0, 1, 4, 2, 3)).reshape(1, C * Z, H, W)
    assert np.array_equal(layout_by_index_arithmetic(dense, fmt, "NCHW"), tail)


def dense_tail(t: Dense, node, precision):
    """Independent restatement of a ScatterDense node: the fp32 value of every stored element as fp16, or, for an
    int8 output (the node carries input_dynamic_range and the engine runs int8), that value fake-quantised with
    the node's own range; zero outside the active set either way; then the layout by index arithmetic.
    Returns (tensor, True when it is in a vectorised layout that the Transpose / Reshape tail leaves alone)."""
    a = node.attrs
    val = t.val.astype(F32) if t.rng is None else t.val.astype(F32) * (F32(t.rng) / F32(127.0))
    out_rng = float(a.get("input_dynamic_range", 0.0) or 0.0)
    if out_rng > 0 and precision == "int8":
        dense = (_quant(val, out_rng) * t.mask[None]).astype(np.int8)[None]
    else:
        dense = val.astype(np.float16)[None]
    layout = a.get("output_layout", "") or "NCHW"
    if layout == "NCHW":
        return dense, False
    return layout_by_index_arithmetic(dense, a.get("format", "zyx"), layout), True


@pytest.mark.parametrize("kind,data_fn,layout,int8_out,plan", [
    ("centerpoint", _cp, "NCHW32", True, "all-int8"), ("centerpoint", _cp, "NCHW", True, "all-int8"),
    ("bevfusion", _bev, "NHWzC", False, "all-int8"), ("bevfusion", _bev, "NCHW32", True, "all-int8"),
    ("bevfusion", _bev, "NHWzC", True, "all-int8"), ("centerpoint", _cp, "NCHW32", False, "all-int8"),
    ("bevfusion", _bev, "NCHW", True, "bevfusion")])   # (last: the tensor in front of the dense node is stored fp16)
def test_dense_output_forms_of_the_graph_walk_against_dense_walk(kind, data_fn, layout, int8_out, plan):
    """run_graph's ScatterDense branch for int8 output and the vectorised layouts, and the rule that the tensor
    feeding an int8 dense node is stored int8 with that node's range when no other consumer fixes one, against
    the dense walk (ranges pushed from consumers, dense_tail, layouts by index arithmetic)."""
    data = data_fn()
    feats, idx, grid = data
    g = _graph(kind, 21, plan, data)
    sd = [n for n in g.nodes if n.op_type == "ScatterDense"][0]
    sd.attrs["output_layout"] = layout
    last_conv = [n for n in g.nodes if n.outputs[0] == sd.inputs[0]][0]
    if int8_out:
        # a range that clips some values, so that the clamp and the choice of range both show
        rec = {}
        dense_walk(g, feats, idx, grid, "int8", rec)
        t = rec[last_conv.name]
        sd.attrs["input_dynamic_range"] = float(0.6 * np.abs(t.val[:, t.mask > 0]).max())
    rec_o, rec_d = {}, {}
    got = O.run_graph(g, feats, idx, grid, "int8", rec_o)[g.outputs[0]]
    rebase = None
    if plan != "all-int8":
        # conv_input computes in fp16 (summation order): continue the dense walk from the oracle's result of it
        n0 = g.nodes[0]
        v, m = to_dense(T_of(rec_o, None, g, n0))
        rebase = {n0.outputs[0]: Dense(v, m, None if rec_o[n0.name]["range"] is None else F32(rec_o[n0.name]["range"]))}
    want = dense_walk(g, feats, idx, grid, "int8", rec_d, rebase=rebase)[g.outputs[0]]
    if int8_out and plan == "all-int8":
        assert F32(rec_o[last_conv.name]["range"]) == F32(rec_d[last_conv.name].rng) == F32(sd.attrs["input_dynamic_range"])
    else:   # stored fp16: by the plan, or because nothing downstream quantises
        assert rec_o[last_conv.name]["range"] is None and rec_d[last_conv.name].rng is None
    assert got.dtype == want.dtype == (np.int8 if int8_out else np.float16)
    c3, z = CHANNELS[3], 2
    expect = {"NCHW32": (1, (c3 * z + 31) // 32, 8, 8, 32), "NHWzC": (1, 8, 8, z, c3), "NCHW": (1, c3 * z, 8, 8)}[layout]
    assert got.shape == want.shape == expect, (got.shape, want.shape)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    assert np.count_nonzero(got) > 50
    if int8_out:
        assert np.abs(got).max() == 127 and np.mean(np.abs(got[got != 0]) == 127) < 0.5   # the range clips, not everywhere
        # sensitivity: quantising the dense output from the stored fp16-rounded value instead of from the int8 code's
        # value, or with the conv's weight range, is caught because the range differs from every other in the graph
        assert all(F32(n.attrs.get("input_dynamic_range", -1)) != F32(sd.attrs["input_dynamic_range"])
                   for n in g.nodes if n is not sd)
