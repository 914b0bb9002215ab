"""Tile plans (the reference loader's `sortmask` switch) and the tile-plan convolution kernel of the narrow
layers: the plan is what its definition says (masks, a permutation sorted by offset set inside 1024-row windows, the table in plan
order), and convolutions with a plan -- in row order and sorted -- give the bits of the plan-less kernels and of
the CPU oracle.  Needs a MI355X."""
import ctypes as C

import numpy as np
import pytest
import torch

from lidar_ai_solution_amd import capi, synth
from oracle import scn_oracle as O

pytestmark = pytest.mark.gpu

from tests.gpu_helpers import DEV, GpuConv, GpuRulebook, copy_from_ptr, to_dev, stream  # noqa: E402
from tests.test_gpu_stages import _weights, note  # noqa: E402

GRID = (41, 1440, 1440)


def _plan_of(rb, n, kvol):
    L = capi.lib()
    tm, pm, nb = C.c_void_p(), C.c_void_p(), C.c_void_p()
    capi.check(L.scn_rulebook_plan(rb.h, C.byref(tm), C.byref(pm), C.byref(nb)))
    pos = (n + 31) // 32 * 32
    tmask = copy_from_ptr(tm.value, (pos // 32,), np.uint32).cpu().numpy().view(np.uint32) if pos else np.zeros(0, np.uint32)
    perm = copy_from_ptr(pm.value, (pos,), np.uint32).cpu().numpy().view(np.uint32) if pm.value and pos else None
    ld = capi.lib().scn_rulebook_nbr_ld(rb.h)
    table = copy_from_ptr(nb.value, (kvol, ld), np.int32).cpu().numpy()[:, :pos] if nb.value and pos else None
    return tmask, perm, table


def _dense_table(ref_rb, n_out, kvol):
    t = np.full((kvol, n_out), -1, np.int32)
    for k in range(kvol):
        a, b = int(ref_rb.offsets[k]), int(ref_rb.offsets[k + 1])
        t[k, ref_rb.pair_out[a:b]] = ref_rb.pair_in[a:b]
    return t


@pytest.mark.parametrize("kind", ["subm", "strided"])
def test_plan_is_what_it_says(kind, centerpoint_input):
    _, idx_all = centerpoint_input
    idx = idx_all[:20011]
    n_in = idx.shape[0]
    L = capi.lib()
    if kind == "subm":
        ref = O.rulebook_subm(idx, GRID, (3, 3, 3))
        rb = GpuRulebook(n_in, n_in, 27)
        rb.build_subm(to_dev(idx), n_in, GRID, (3, 3, 3))
    else:
        ref = O.rulebook_sparse(idx, GRID, (3, 3, 3), (2, 2, 2), (1, 1, 1), max_out=200000)
        rb = GpuRulebook(n_in, 200000, 27)
        rb.build_sparse(to_dev(idx), n_in, GRID, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    n = ref.n_out
    table = _dense_table(ref, n, 27)
    masks = np.zeros(n, np.uint32)
    for k in range(27):
        masks |= (table[k] >= 0).astype(np.uint32) << np.uint32(k)
    pos = (n + 31) // 32 * 32
    padded = np.zeros(pos, np.uint32)
    padded[:n] = masks
    note(f"tile plan in row order, {kind} rulebook, {n} rows")
    capi.check(L.scn_rulebook_build_plan(rb.h, 0, stream()))
    tmask, perm, tab = _plan_of(rb, n, 27)
    assert perm is None and tab is None
    assert np.array_equal(tmask, np.bitwise_or.reduce(padded.reshape(-1, 32), axis=1))
    note(f"sorted tile plan, {kind} rulebook")
    capi.check(L.scn_rulebook_build_plan(rb.h, 1, stream()))
    tmask, perm, tab = _plan_of(rb, n, 27)
    # the definition: stable sort by offset set inside windows of 1024 consecutive rows
    order = np.concatenate([b + np.argsort(masks[b:b + 1024], kind="stable") for b in range(0, n, 1024)])
    assert np.all(order // 1024 == np.arange(n) // 1024)
    assert np.array_equal(perm[:n], order.astype(np.uint32))
    assert np.all(perm[n:] >= n)
    sorted_masks = np.zeros(pos, np.uint32)
    sorted_masks[:n] = masks[order]
    assert np.array_equal(tmask, np.bitwise_or.reduce(sorted_masks.reshape(-1, 32), axis=1))
    assert np.array_equal(tab[:, :n], table[:, order]) and np.all(tab[:, n:] == -1)
    slots_before = sum(bin(int(v)).count("1") for v in np.bitwise_or.reduce(padded.reshape(-1, 32), axis=1))
    slots_after = sum(bin(int(v)).count("1") for v in tmask)
    print(f"(tile, offset) slots with work: {slots_before} in row order, {slots_after} sorted, of {pos // 32 * 27}")
    assert slots_after < slots_before


# (Cin, Cout, strided, element type): every shape the tile-plan kernel is instantiated for
TILE_SHAPES = [(16, 16, False, "int8"), (32, 32, False, "int8"), (16, 32, True, "int8"), (32, 64, True, "int8"),
               (16, 64, False, "int8"), (5, 16, False, "fp16"), (16, 16, False, "fp16"), (16, 32, True, "fp16"),
               (32, 32, False, "fp16")]


@pytest.mark.parametrize("cin,cout,strided,el", TILE_SHAPES)
def test_conv_with_plan_equals_conv_without(cin, cout, strided, el, centerpoint_input):
    _, idx_all = centerpoint_input
    rng = np.random.default_rng(cin * 1000 + cout + strided)
    idx = idx_all[:30017]
    n_in = idx.shape[0]
    L = capi.lib()
    note(f"{el} conv {cin}->{cout} {'strided' if strided else 'subm'} on {n_in} fixture voxels: no plan / plan / sorted plan")
    if strided:
        ref_rb = O.rulebook_sparse(idx, GRID, (3, 3, 3), (2, 2, 2), (1, 1, 1), max_out=200000)
        rb = GpuRulebook(n_in, 200000, 27)
        rb.build_sparse(to_dev(idx), n_in, GRID, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    else:
        ref_rb = O.rulebook_subm(idx, GRID, (3, 3, 3))
        rb = GpuRulebook(n_in, n_in, 27)
        rb.build_subm(to_dev(idx), n_in, GRID, (3, 3, 3))
    n_out = ref_rb.n_out
    w, b, ranges = _weights(rng, cout, (3, 3, 3), cin)
    if el == "int8":
        x = rng.integers(-127, 128, (n_in, cin)).astype(np.int8)
        conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
        x_range, out_range = 3.9, 1.1
        wq, s_w = O.quantize_weights(w, ranges)
        acc_ref = O.conv_int8_acc(x, wq, ref_rb)
        scale = (np.float32(x_range) / np.float32(127) * s_w).astype(np.float32)
        want8 = O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range)
        want16 = O.epilogue(acc_ref, scale, b.astype(np.float32), False, False)
        res = rng.integers(-127, 128, (n_out, (cout + 15) // 16 * 16)).astype(np.int8)
        d_x, d_res = to_dev(x), to_dev(res)
        # the fused Conv + Add + ReLU of the un-fused oracle: int8 intermediate, int8 add, ReLU, int8 store
        mid = O.epilogue(acc_ref, scale, b.astype(np.float32), False, True, 1.7)
        want_fused = O.add(mid, 1.7, res[:, :cout], 2.2, True, True, out_range)
        results = []
        for plan in (None, 0, 1):
            if plan is not None:
                capi.check(L.scn_rulebook_build_plan(rb.h, plan, stream()))
            o8, acc = conv.forward(rb, d_x, n_out, x_range=x_range, relu=True, out_int8=True, out_range=out_range, want_acc=True)
            o8b, _ = conv.forward(rb, d_x, n_out, x_range=x_range, relu=True, out_int8=True, out_range=out_range)
            o16, _ = conv.forward(rb, d_x, n_out, x_range=x_range, relu=False, out_int8=False)
            fused, _ = conv.forward(rb, d_x, n_out, x_range=x_range, relu=False, out_int8=True, out_range=out_range,
                                    res=d_res, res_range=2.2, mid_int8=True, mid_range=1.7, relu2=True)
            results.append([t.cpu().numpy() for t in (o8, acc, o8b, o16, fused)])
        for k, r in enumerate(results):
            assert np.array_equal(r[1], acc_ref), f"accumulators, variant {k}"
            assert np.array_equal(r[0][:, :cout], want8) and np.array_equal(r[2][:, :cout], want8), f"int8 output, variant {k}"
            assert np.array_equal(r[3][:, :cout].view(np.uint16), want16.view(np.uint16)), f"fp16 output, variant {k}"
            assert np.array_equal(r[4][:, :cout], want_fused), f"fused residual against the un-fused oracle, variant {k}"
        assert np.count_nonzero(results[0][4]) > n_out
    else:
        cpad = 8 if cin == 5 else cin
        x = np.zeros((n_in, cpad), np.float16)
        x[:, :cin] = rng.standard_normal((n_in, cin)).astype(np.float16)
        conv = GpuConv(w, None, b, capi.PRECISION_FP16)
        wf = np.ascontiguousarray(w.astype(np.float32).reshape(cout, -1, cin).transpose(1, 0, 2))
        acc_ref = O.conv_f32_acc(np.ascontiguousarray(x[:, :cin]).astype(np.float32), wf, ref_rb)
        want = O.epilogue(acc_ref, None, b.astype(np.float32), True, False).astype(np.float32)
        res = rng.standard_normal((n_out, (cout + 15) // 16 * 16)).astype(np.float16)
        d_x, d_res = to_dev(x), to_dev(res)
        outs = []
        for plan in (None, 0, 1):
            if plan is not None:
                capi.check(L.scn_rulebook_build_plan(rb.h, plan, stream()))
            o, _ = conv.forward(rb, d_x, n_out, relu=True, out_int8=False)
            f, _ = conv.forward(rb, d_x, n_out, relu=False, out_int8=False, res=d_res, relu2=True)
            m, _ = conv.forward(rb, d_x, n_out, relu=False, out_int8=False)
            outs.append((o.cpu().numpy(), f.cpu().numpy(), m.cpu().numpy()))
        tol = 2e-3 * max(float(np.abs(want).max()), 1e-3)   # a few fp16 steps of the largest value: products are summed in fp32
        for k, (o, f, m) in enumerate(outs):
            assert np.abs(o[:, :cout].astype(np.float32) - want).max() <= tol, f"variant {k}"
            # fused fp16 Conv + Add + ReLU, exactly: the oracle's Add of the same kernel's un-fused fp16 result (same MFMA
            # sequence, no ReLU) and the residual
            want_f = O.add(np.ascontiguousarray(m[:, :cout]), 127.0, np.ascontiguousarray(res[:, :cout]), 127.0, True, False)
            assert np.array_equal(f[:, :cout].view(np.uint16), want_f.view(np.uint16)), f"fused fp16 residual, variant {k}"
        # the sorted plan and the plan in row order add a row's products in the same order
        assert np.array_equal(outs[1][0].view(np.uint16), outs[2][0].view(np.uint16))
        assert np.array_equal(outs[1][1].view(np.uint16), outs[2][1].view(np.uint16))
        if cin != 5:   # rows of more than 16 bytes: the same MFMA sequence as the plan-less kernel, zero steps left out
            assert np.array_equal(outs[0][0].view(np.uint16), outs[1][0].view(np.uint16))


def test_rebuilding_a_rulebook_drops_its_tile_plan():
    """A plan describes the table of one build: after the rulebook is built again on other coordinates (without a new
    plan) a convolution must not use the old masks, permutation or plan-order table."""
    rng = np.random.default_rng(9)
    L = capi.lib()
    grid = (8, 64, 64)
    idx_a = synth.uniform_voxels(6, 9000, grid)
    idx_b = synth.uniform_voxels(7, 7001, grid)
    w, b, ranges = _weights(rng, 32, (3, 3, 3), 32)
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    wq, s_w = O.quantize_weights(w, ranges)
    scale = (np.float32(2.0) / np.float32(127) * s_w).astype(np.float32)
    rb = GpuRulebook(9000, 9000, 27)
    for sorted_plan in (1, 0):
        note(f"build -> plan (sorted={sorted_plan}) -> build on other coordinates -> convolution")
        rb.build_subm(to_dev(idx_a), idx_a.shape[0], grid, (3, 3, 3))
        capi.check(L.scn_rulebook_build_plan(rb.h, sorted_plan, stream()))
        rb.build_subm(to_dev(idx_b), idx_b.shape[0], grid, (3, 3, 3))
        assert L.scn_rulebook_plan(rb.h, None, None, None) != 0      # no plan any more
        x = rng.integers(-127, 128, (idx_b.shape[0], 32)).astype(np.int8)
        want = O.epilogue(O.conv_int8_acc(x, wq, O.rulebook_subm(idx_b, grid, (3, 3, 3))), scale, b.astype(np.float32),
                          True, True, 1.5)
        out, _ = conv.forward(rb, to_dev(x), idx_b.shape[0], x_range=2.0, relu=True, out_int8=True, out_range=1.5)
        assert np.array_equal(out.cpu().numpy(), want)


def test_plan_with_device_side_count_and_empty_input():
    """Rows beyond the device-side count take no part: the plan built for a bound of 9,000 rows with 3,333 real ones
    gives the result of a 3,333-row rulebook; zero rows launch nothing that writes."""
    rng = np.random.default_rng(5)
    L = capi.lib()
    grid = (8, 64, 64)
    idx = synth.uniform_voxels(5, 9000, grid)
    k = 3333
    note("sorted tile plan under a device-side row count")
    ref_rb = O.rulebook_subm(idx[:k], grid, (3, 3, 3))
    w, b, ranges = _weights(rng, 32, (3, 3, 3), 32)
    x = rng.integers(-127, 128, (9000, 32)).astype(np.int8)
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x[:k], wq, ref_rb)
    want = O.epilogue(acc_ref, (np.float32(2.0) / np.float32(127) * s_w).astype(np.float32), b.astype(np.float32), True, True, 1.5)
    cnt = to_dev(np.array([k], np.uint32))
    rb = GpuRulebook(9000, 9000, 27)
    d_idx = to_dev(idx)
    rb.build_subm(d_idx, 9000, grid, (3, 3, 3), n_dev=cnt)
    capi.check(L.scn_rulebook_build_plan(rb.h, 1, stream()))
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    out, _ = conv.forward(rb, to_dev(x), 9000, x_range=2.0, relu=True, out_int8=True, out_range=1.5)
    got = out.cpu().numpy()
    assert np.array_equal(got[:k], want) and not got[k:].any()
    note("sorted tile plan of an empty rulebook")
    zero = to_dev(np.array([0], np.uint32))
    rb.build_subm(d_idx, 9000, grid, (3, 3, 3), n_dev=zero)
    capi.check(L.scn_rulebook_build_plan(rb.h, 1, stream()))
    out, _ = conv.forward(rb, to_dev(x), 9000, x_range=2.0, relu=True, out_int8=True, out_range=1.5)
    assert not out.cpu().numpy().any()


def test_engine_sortmask_gives_identical_results(centerpoint_input, bevfusion_input):
    """Engines built with tile plans (`sortmask` of load_engine_from_onnx / EngineBuilder::build is the hint; the
    plans themselves are switched on by SCN_BUILD_TILE_PLANS): the narrow layers run on sorted tile plans.
    Every kept tensor of the int8 CenterPoint-shaped engine and the BEV outputs of the fused int8 / fp16 engines,
    with and without an auxiliary stream, equal the plain engine's bit for bit; a second, smaller frame on the
    same engines too (no stale plan)."""
    from lidar_ai_solution_amd import graphs
    from lidar_ai_solution_amd.scn import Engine
    from tests.test_gpu_engine import _oracle_calibration, _run_engine, GRID_ZYX, GRID_XYZ
    feats, idx = centerpoint_input
    g16, tags = graphs.centerpoint_scn(seed=0)
    amax = _oracle_calibration(g16, feats, idx, GRID_ZYX)
    g8, tags8 = graphs.centerpoint_scn(seed=0)
    graphs.apply_int8_plan(g8, tags8, amax, "centerpoint")
    note("int8 engine, every tensor kept: sortmask vs plain")
    plain = Engine.from_graph(g8, "int8", keep_all=True)
    sort = Engine.from_graph(g8, "int8", keep_all=True, sortmask=True, tile_plans=True)
    _run_engine(plain, feats, idx, GRID_ZYX)
    _run_engine(sort, feats, idx, GRID_ZYX)
    checked = 0
    for n in g8.nodes:
        if n.op_type not in ("SparseConvolution", "Add", "Relu"):
            continue
        a, _ = plain.tensor(n.outputs[0])
        b, _ = sort.tensor(n.outputs[0])
        ta, _ = a.torch()
        tb, _ = b.torch()
        assert ta.dtype == tb.dtype and torch.equal(ta.view(torch.uint8), tb.view(torch.uint8)), n.name
        checked += 1
    assert checked >= 30
    for prec, graph in (("int8", g8), ("fp16", g16)):
        want_eng = Engine.from_graph(graph, prec)
        for aux in (False, True):
            note(f"fused {prec} engine with sortmask, auxiliary stream {aux}: two frames")
            eng = Engine.from_graph(graph, prec, sortmask=True, tile_plans=True, with_auxiliary_stream=aux)
            for rows in (feats.shape[0], 23456, feats.shape[0]):
                _run_engine(want_eng, feats[:rows], idx[:rows], GRID_ZYX)
                want = want_eng.output(0).torch().clone()
                _run_engine(eng, feats[:rows], idx[:rows], GRID_ZYX)
                got = eng.output(0).torch()
                assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (prec, aux, rows)
    note("BEVFusion-shaped int8 engine (xyz) with sortmask")
    bf, bi = bevfusion_input
    b16, bt = graphs.bevfusion_scn(seed=1)
    bamax = _oracle_calibration(b16, bf, bi, GRID_XYZ)
    b8, bt8 = graphs.bevfusion_scn(seed=1)
    graphs.apply_int8_plan(b8, bt8, bamax, "bevfusion")
    e0, e1 = Engine.from_graph(b8, "int8"), Engine.from_graph(b8, "int8", sortmask=True, tile_plans=True)
    _run_engine(e0, bf, bi, GRID_XYZ)
    _run_engine(e1, bf, bi, GRID_XYZ)
    assert torch.equal(e0.output(0).torch().view(torch.int16), e1.output(0).torch().view(torch.int16))
