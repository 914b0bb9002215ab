"""Parity of every HIP stage with the CPU oracle, through the C ABI.  Needs a MI355X."""
import ctypes as C
import json
import os

import numpy as np
import pytest
import torch

from lidar_ai_solution_amd import capi, synth
from oracle import scn_oracle as O

pytestmark = pytest.mark.gpu

from tests.gpu_helpers import DEV, GpuConv, GpuRulebook, copy_from_ptr, i3, ptr, read_u32, stream, to_dev  # noqa: E402

KNOWN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")))


def note(msg):
    print(f"[case] {msg}", flush=True)


# ----------------------------------------------------------------------------- hash
def test_hash_build_and_query(centerpoint_input):
    note("hash build/query on the 79,745-voxel fixture")
    L = capi.lib()
    _, idx = centerpoint_input
    assert L.scn_hash_u64(85017599) == O.hash64(85017599)
    n = idx.shape[0]
    cap = L.scn_hash_capacity_for(n)
    assert cap >= 2 * n and cap & (cap - 1) == 0
    table = torch.zeros(cap, dtype=torch.int64, device=DEV)
    d_idx = to_dev(idx)
    grid = (41, 1440, 1440)
    capi.check(L.scn_hash_build(ptr(table), cap, ptr(d_idx), n, None, i3(grid), stream()))
    rng = np.random.default_rng(0)
    q = idx[rng.permutation(n)[:5000]].copy()
    miss = q.copy()
    miss[:, 3] = (miss[:, 3] + 1) % 1440
    d = {tuple(r): i for i, r in enumerate(idx)}
    qq = np.concatenate([q, miss])
    rows = torch.zeros(qq.shape[0], dtype=torch.int32, device=DEV)
    d_qq = to_dev(qq)
    capi.check(L.scn_hash_query(ptr(table), cap, ptr(d_qq), qq.shape[0], i3(grid), ptr(rows), stream()))
    torch.cuda.synchronize()
    want = np.array([d.get(tuple(r), -1) for r in qq], np.int32)
    assert np.array_equal(rows.cpu().numpy(), want)
    # occupancy: every row landed in exactly one slot
    t = table.cpu().numpy().view(np.uint64)
    used = t != np.uint64(0xFFFFFFFFFFFFFFFF)
    assert int(used.sum()) == n
    assert np.array_equal(np.sort((t[used] & np.uint64(0xFFFFFFFF)).astype(np.int64)), np.arange(n))


# ----------------------------------------------------------------------------- rulebooks
STAGES = [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
          ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((3, 1, 1), (2, 1, 1), (0, 0, 0))]


def _check_pairs(rb_gpu, ref):
    pin, pout, offs = rb_gpu.pairs(max(ref.num_pairs, 1))
    assert np.array_equal(offs, ref.offsets)
    assert np.array_equal(pout, ref.pair_out)
    assert np.array_equal(pin, ref.pair_in)


def test_rulebooks_on_reference_fixture_all_stages(centerpoint_input):
    _, idx = centerpoint_input
    ka = KNOWN["centerpoint_fixture"]
    grid = [41, 1440, 1440]
    for s in range(4):
        n = idx.shape[0]
        note(f"rulebooks stage {s}: n={n} grid={grid}")
        d_idx = to_dev(idx)
        sub = GpuRulebook(n, n, 27)
        sub.build_subm(d_idx, n, grid, (3, 3, 3))
        ref = O.rulebook_subm(idx, grid, (3, 3, 3))
        assert ref.num_pairs == ka["subm_pairs"][s]
        _check_pairs(sub, ref)
        k, st, p = STAGES[s]
        sp = GpuRulebook(n, 200000, int(np.prod(k)))
        sp.build_sparse(d_idx, n, grid, k, st, p)
        ref2 = O.rulebook_sparse(idx, grid, k, st, p)
        assert sp.out_grid() == ref2.out_grid == ka["grids"][s + 1]
        assert sp.n_out() == ref2.n_out == ka["active"][s + 1]
        assert np.array_equal(sp.out_indices(), ref2.out_indices)
        _check_pairs(sp, ref2)
        idx, grid = ref2.out_indices, ref2.out_grid


def test_sparse_rulebook_truncation_empty_and_device_count():
    rng = np.random.default_rng(11)
    grid = (9, 40, 37)
    vol = int(np.prod(grid))
    lin = rng.choice(vol, 3000, replace=False)
    idx = np.zeros((3000, 4), np.int32)
    idx[:, 3] = lin % grid[2]; idx[:, 2] = (lin // grid[2]) % grid[1]; idx[:, 1] = lin // (grid[2] * grid[1])
    d_idx = to_dev(idx)
    note("sparse rulebook truncated to 500 outputs")
    rb = GpuRulebook(3000, 500, 27)
    rb.build_sparse(d_idx, 3000, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    ref = O.rulebook_sparse(idx, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1), max_out=500)
    assert rb.n_out() == 500 and rb.n_out_total() == ref.n_out_total
    assert np.array_equal(rb.out_indices(), ref.out_indices)
    _check_pairs(rb, ref)
    note("device-side row count smaller than the bound")
    n_dev = torch.tensor([1234], dtype=torch.int32, device=DEV)
    rb2 = GpuRulebook(3000, 3000, 27)
    rb2.build_sparse(d_idx, 3000, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1), n_dev=n_dev)
    ref2 = O.rulebook_sparse(idx[:1234], grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    assert rb2.n_out() == ref2.n_out
    assert np.array_equal(rb2.out_indices(), ref2.out_indices)
    _check_pairs(rb2, ref2)
    sub = GpuRulebook(3000, 3000, 27)
    sub.build_subm(d_idx, 3000, grid, (3, 3, 3), n_dev=n_dev)
    _check_pairs(sub, O.rulebook_subm(idx[:1234], grid, (3, 3, 3)))
    note("empty input")
    n0 = torch.tensor([0], dtype=torch.int32, device=DEV)
    rb3 = GpuRulebook(3000, 3000, 27)
    rb3.build_sparse(d_idx, 3000, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1), n_dev=n0)
    assert rb3.n_out() == 0
    pin, pout, offs = rb3.pairs(16)
    assert offs[-1] == 0
    note("dilated and non-cubic kernels")
    for ks, st, pd, dl in [((3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2)), ((1, 3, 3), (1, 2, 2), (0, 1, 1), (1, 1, 1)),
                           ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)), ((1, 1, 3), (1, 1, 2), (0, 0, 0), (1, 1, 1))]:
        r = GpuRulebook(3000, 3000 * 8, int(np.prod(ks)))
        r.build_sparse(d_idx, 3000, grid, ks, st, pd, dl)
        rr = O.rulebook_sparse(idx, grid, ks, st, pd, dl)
        assert r.n_out() == rr.n_out and np.array_equal(r.out_indices(), rr.out_indices)
        _check_pairs(r, rr)
    s2 = GpuRulebook(3000, 3000, 27)
    s2.build_subm(d_idx, 3000, grid, (3, 3, 3), (2, 2, 2))
    _check_pairs(s2, O.rulebook_subm(idx, grid, (3, 3, 3), (2, 2, 2)))


def test_row_lookup_of_canonical_and_caller_order_inputs_on_one_rulebook():
    """Rows in canonical order (strictly ascending linear index) are found by rank in an occupancy bitmap written
    without atomics, any other order through the coordinate hash; which of the two a build tries first follows what
    the previous build found.  One rulebook object sees both orders in turn (more than 16 builds, so that the periodic
    second look happens too) and near-misses of the order: a swapped pair, a row outside the
    grid, a device-side count that cuts the rows.  Every table must equal the oracle's."""
    rng = np.random.default_rng(5)
    grid = (7, 45, 70)
    vol = int(np.prod(grid))
    n = 2500

    def coords(lin):
        idx = np.zeros((lin.size, 4), np.int32)
        idx[:, 3] = lin % grid[2]; idx[:, 2] = (lin // grid[2]) % grid[1]; idx[:, 1] = lin // (grid[2] * grid[1])
        return idx

    lin_sorted = np.sort(rng.choice(vol, n, replace=False))
    cases = []
    for i in range(18):
        lin = np.sort(rng.choice(vol, n, replace=False))
        if i % 3 == 2:
            lin = rng.permutation(lin)
        cases.append((f"build {i}: {'caller' if i % 3 == 2 else 'canonical'} order", coords(lin), n))
    swapped = lin_sorted.copy(); swapped[[1200, 1201]] = swapped[[1201, 1200]]
    cases.append(("one swapped pair", coords(swapped), n))
    cases.append(("canonical again", coords(lin_sorted), n))
    cases.append(("device-side count 1000 of canonical rows", coords(lin_sorted), 1000))
    last_in_word = coords(lin_sorted[: n - 1])
    cases.append(("one row fewer", last_in_word, n - 1))
    sub = GpuRulebook(n, n, 27)
    sp = GpuRulebook(n, n * 8, 27)
    for label, idx, count in cases:
        note("row lookup: " + label)
        d_idx = to_dev(idx)
        n_dev = None if count == idx.shape[0] else torch.tensor([count], dtype=torch.int32, device=DEV)
        sub.build_subm(d_idx, idx.shape[0], grid, (3, 3, 3), n_dev=n_dev)
        _check_pairs(sub, O.rulebook_subm(idx[:count], grid, (3, 3, 3)))
        sp.build_sparse(d_idx, idx.shape[0], grid, (3, 3, 3), (2, 2, 2), (1, 1, 1), n_dev=n_dev)
        ref = O.rulebook_sparse(idx[:count], grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
        assert sp.n_out() == ref.n_out and np.array_equal(sp.out_indices(), ref.out_indices)
        _check_pairs(sp, ref)
    note("row lookup: one row outside the grid among canonical rows")
    # (what such a row itself pairs with is not defined; every other row must see the tensor without it)
    outside = coords(lin_sorted); outside[77, 3] = grid[2]
    sub.build_subm(to_dev(outside), n, grid, (3, 3, 3))
    pin, pout, offs = sub.pairs(27 * n)
    ref = O.rulebook_subm(np.delete(outside, 77, axis=0), grid, (3, 3, 3))
    shift = lambda r: r + (r >= 77)
    for k in range(27):
        got = {(int(a), int(b)) for a, b in zip(pin[offs[k]:offs[k + 1]], pout[offs[k]:offs[k + 1]]) if a != 77 and b != 77}
        want = {(int(shift(a)), int(shift(b))) for a, b in zip(ref.pair_in[ref.offsets[k]:ref.offsets[k + 1]],
                                                               ref.pair_out[ref.offsets[k]:ref.offsets[k + 1]])}
        assert got == want, k


# ----------------------------------------------------------------------------- convolution
def _weights(rng, cout, ks, cin, std=0.02):
    w = (rng.standard_normal((cout, *ks, cin)) * std).astype(np.float16)
    b = (rng.standard_normal(cout) * std).astype(np.float16)
    ranges = np.abs(w.astype(np.float32)).reshape(cout, -1).max(1)
    return w, b, ranges


def test_config1_single_int8_subm_layer():
    """One int8 SubMConv3d 3x3x3 16->16 on 20,000 uniform voxels: int32 accumulators and the int8
    requantised ReLU output are bit-exact."""
    note("config 1: int8 subm 16->16, 20000 voxels")
    rng = np.random.default_rng(0)
    grid = (41, 1440, 1440)
    idx = synth.uniform_voxels(0, 20000, grid)
    x = rng.integers(-127, 128, (20000, 16)).astype(np.int8)
    w, b, ranges = _weights(rng, 16, (3, 3, 3), 16)
    x_range = np.float32(0.05 * 127)  # a per-tensor activation scale of 0.05
    s_x = x_range / np.float32(127)
    ref_rb = O.rulebook_subm(idx, grid, (3, 3, 3))
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x, wq, ref_rb)
    scale = (s_x * s_w).astype(np.float32)
    y = np.maximum(acc_ref.astype(np.float32) * scale + b.astype(np.float32), 0)
    out_range = float(np.float32(np.percentile(y, 99.99)))  # output range fixed up front: 99.99th percentile
    out_ref = O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range)
    rb = GpuRulebook(20000, 20000, 27)
    rb.build_subm(to_dev(idx), 20000, grid, (3, 3, 3))
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    out, acc = conv.forward(rb, to_dev(x), 20000, x_range=float(x_range), relu=True, out_int8=True, out_range=out_range, want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(out.cpu().numpy(), out_ref)
    assert ref_rb.num_pairs >= 20000 and np.abs(out_ref).max() > 20


SHAPES = [(16, 16), (16, 32), (32, 32), (32, 64), (64, 64), (64, 128), (128, 128)]


@pytest.mark.parametrize("cin,cout", SHAPES)
def test_int8_conv_shapes_bit_exact(cin, cout, centerpoint_input):
    _, idx_all = centerpoint_input
    rng = np.random.default_rng(cin * 1000 + cout)
    idx = idx_all[:30000]
    n = idx.shape[0]
    grid = (41, 1440, 1440)
    subm = cin == cout
    note(f"int8 conv {cin}->{cout} {'subm' if subm else 'strided'} on {n} fixture voxels")
    x = rng.integers(-127, 128, (n, cin)).astype(np.int8)
    w, b, ranges = _weights(rng, cout, (3, 3, 3), cin)
    x_range, out_range = 3.9, 5.5
    s_x = np.float32(x_range) / np.float32(127)
    if subm:
        ref_rb = O.rulebook_subm(idx, grid, (3, 3, 3))
        rb = GpuRulebook(n, n, 27)
        rb.build_subm(to_dev(idx), n, grid, (3, 3, 3))
    else:
        ref_rb = O.rulebook_sparse(idx, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
        rb = GpuRulebook(n, 200000, 27)
        rb.build_sparse(to_dev(idx), n, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x, wq, ref_rb)
    scale = (s_x * s_w).astype(np.float32)
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    out, acc = conv.forward(rb, to_dev(x), ref_rb.n_out, x_range=x_range, relu=True, out_int8=True, out_range=out_range, want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(out.cpu().numpy(), O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range))
    out16, _ = conv.forward(rb, to_dev(x), ref_rb.n_out, x_range=x_range, relu=False, out_int8=False)
    ref16 = O.epilogue(acc_ref, scale, b.astype(np.float32), False, False)
    assert np.array_equal(out16.cpu().numpy().view(np.uint16), ref16.view(np.uint16))


@pytest.mark.parametrize("n", [10335, 30000, 66000, 75000, 84000, 93000, 101000])
def test_int8_conv_workgroup_heights(n):
    """128-channel layers pick their workgroup height (2, 4 or 8..12 waves of 32 rows) from the row count of
    the rulebook's previous build: every height, and the two-workgroups-per-CU case above 98,304 rows, gives
    the same bit-exact result.  Clustered coordinates so that most offsets have neighbours."""
    rng = np.random.default_rng(n)
    grid = (6, 300, 300) if n >= 60000 else (5, 100, 100) if n >= 20000 else (5, 60, 60)
    idx = synth.uniform_voxels(n, n, grid)
    note(f"int8 conv 128->128 subm, {n} voxels in {grid} (workgroup height from the row count)")
    x = rng.integers(-127, 128, (n, 128)).astype(np.int8)
    w, b, ranges = _weights(rng, 128, (3, 3, 3), 128)
    x_range, out_range = 3.9, 9.0
    ref_rb = O.rulebook_subm(idx, grid, (3, 3, 3))
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x, wq, ref_rb)
    scale = (np.float32(x_range) / np.float32(127) * s_w).astype(np.float32)
    rb = GpuRulebook(n, n, 27)
    d_idx = to_dev(idx)
    rb.build_subm(d_idx, n, grid, (3, 3, 3))
    torch.cuda.synchronize()
    rb.build_subm(d_idx, n, grid, (3, 3, 3))  # the second build finds the first one's row count on the host
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    out, acc = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=True, out_int8=True, out_range=out_range, want_acc=True)
    assert ref_rb.num_pairs > 3 * n
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(out.cpu().numpy(), O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range))


@pytest.mark.parametrize("cin,cout,ks", [(48, 96, (3, 3, 3)), (24, 40, (1, 3, 5)), (64, 32, (2, 2, 2)), (128, 64, (5, 3, 3)),
                                         (64, 64, (2, 2, 2)), (128, 128, (3, 1, 1)), (64, 128, (3, 3, 3)), (128, 128, (1, 1, 2))])
def test_int8_conv_padded_channels_and_kernel_shapes(cin, cout, ks, centerpoint_input):
    """Channel counts that are not powers of two (rows padded to 16-byte chunks, partial MFMA tiles), output
    rows that are not a multiple of 16 bytes (scalar store path), even and large kernel volumes."""
    _, idx_all = centerpoint_input
    rng = np.random.default_rng(cin * 100 + cout)
    idx = idx_all[:9000]
    n = idx.shape[0]
    grid = (41, 1440, 1440)
    kvol = ks[0] * ks[1] * ks[2]
    note(f"int8 conv {cin}->{cout} k={ks} on {n} fixture voxels")
    cpad = {48: 64, 24: 32}.get(cin, cin)  # the kernel's row stride: chunks per row rounded to a power of two
    x = np.zeros((n, cpad), np.int8)
    x[:, :cin] = rng.integers(-127, 128, (n, cin))
    w, b, ranges = _weights(rng, cout, ks, cin)
    x_range, out_range = 3.9, 5.5
    ref_rb = O.rulebook_subm(idx, grid, ks)
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(np.ascontiguousarray(x[:, :cin]), wq, ref_rb)
    scale = (np.float32(x_range) / np.float32(127) * s_w).astype(np.float32)
    rb = GpuRulebook(n, n, kvol)
    rb.build_subm(to_dev(idx), n, grid, ks)
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    want_acc = cout % 16 == 0
    out, acc = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=True, out_int8=True, out_range=out_range, want_acc=want_acc)
    if want_acc:
        assert np.array_equal(acc.cpu().numpy(), acc_ref)
    ref = O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range)
    assert np.array_equal(out.cpu().numpy()[:, :cout], ref)
    # a row stride that is not a multiple of 16 bytes takes the 4-byte store path
    out2, _ = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=True, out_int8=True, out_range=out_range,
                           out_ld=(cout + 15) // 16 * 16 + 4)
    assert np.array_equal(out2.cpu().numpy()[:, :cout], ref)


@pytest.mark.parametrize("cin,cout", [(5, 16), (16, 16), (32, 64), (128, 128)])
def test_fp16_conv_within_tolerance(cin, cout, centerpoint_input):
    """fp16 MFMA path: fp32 accumulation in hardware order.  Tolerance (stated): every accumulator
    within 2e-3 * (sum of |products|) + 1e-6 of the fp32 oracle; fp16 outputs within 1 ulp-ish
    (rtol 2e-3, atol 1e-3)."""
    feats, idx_all = centerpoint_input
    rng = np.random.default_rng(cin * 7 + cout)
    idx = idx_all[:30000]
    n = idx.shape[0]
    grid = (41, 1440, 1440)
    note(f"fp16 conv {cin}->{cout} on {n} fixture voxels")
    if cin == 5:
        x = feats[:n].astype(np.float16)
    else:
        x = rng.standard_normal((n, cin)).astype(np.float16)
    w, b, _ = _weights(rng, cout, (3, 3, 3), cin, std=0.05)
    ref_rb = O.rulebook_subm(idx, grid, (3, 3, 3))
    wf = np.ascontiguousarray(w.astype(np.float32).reshape(cout, 27, cin).transpose(1, 0, 2))
    acc_ref = O.conv_f32_acc(x.astype(np.float32), wf, ref_rb)
    mag = O.conv_f32_acc(np.abs(x.astype(np.float32)), np.abs(wf), ref_rb)
    rb = GpuRulebook(n, n, 27)
    rb.build_subm(to_dev(idx), n, grid, (3, 3, 3))
    conv = GpuConv(w, None, b, capi.PRECISION_FP16)
    cpad = 8 if cin == 5 else cin
    xp = np.zeros((n, cpad), np.float16)
    xp[:, :cin] = x
    out, acc = conv.forward(rb, to_dev(xp), n, relu=True, want_acc=True)
    acc = acc.cpu().numpy()
    assert np.all(np.abs(acc - acc_ref) <= 2e-3 * mag + 1e-6)
    ref = O.epilogue(acc_ref, None, b.astype(np.float32), True, False).astype(np.float32)
    assert np.allclose(out.cpu().numpy().astype(np.float32), ref, rtol=2e-3, atol=1e-3)


@pytest.mark.parametrize("channels,n_rows", [(32, 20000), (64, 9991), (128, 5003), (16, 4097)])
def test_fused_residual_epilogue_matches_unfused_oracle(channels, n_rows, centerpoint_input):
    """conv2 -> Add(identity) -> ReLU fused into one kernel equals the node-by-node oracle, for every tile
    width of the kernel (the residual is staged per tile from 64 channels up) and row counts that end inside a tile."""
    _, idx_all = centerpoint_input
    rng = np.random.default_rng(21)
    idx = idx_all[:n_rows]
    n = idx.shape[0]
    grid = (41, 1440, 1440)
    cin = cout = channels
    note(f"fused residual epilogue, {channels} channels, {n} rows")
    x = rng.integers(-127, 128, (n, cin)).astype(np.int8)
    ident = rng.integers(0, 128, (n, cout)).astype(np.int8)
    w, b, ranges = _weights(rng, cout, (3, 3, 3), cin)
    x_range, mid_range, res_range, out_range = 2.5, 4.4, 3.4, 6.3
    ref_rb = O.rulebook_subm(idx, grid, (3, 3, 3))
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x, wq, ref_rb)
    scale = ((np.float32(x_range) / np.float32(127)) * s_w).astype(np.float32)
    rb = GpuRulebook(n, n, 27)
    rb.build_subm(to_dev(idx), n, grid, (3, 3, 3))
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    note("int8 conv -> int8 add -> relu")
    mid = O.epilogue(acc_ref, scale, b.astype(np.float32), False, True, mid_range)
    want = O.add(mid, mid_range, ident, res_range, True, True, out_range)
    out, _ = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=False, out_int8=True, out_range=out_range,
                          res=to_dev(ident), res_range=res_range, mid_int8=True, mid_range=mid_range, relu2=True)
    assert np.array_equal(out.cpu().numpy(), want)
    note("the same with the convolution's own ReLU in front of the intermediate quantiser, no ReLU after the add")
    mid_r = O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, mid_range)
    want_r = O.add(mid_r, mid_range, ident, res_range, False, True, out_range)
    out_r, _ = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=True, out_int8=True, out_range=out_range,
                            res=to_dev(ident), res_range=res_range, mid_int8=True, mid_range=mid_range, relu2=False)
    assert np.array_equal(out_r.cpu().numpy(), want_r)
    note("fp16-stored conv output and fp16 identity, int8 add re-quantising both, int8 out")
    ident16 = (rng.standard_normal((n, cout)) * 2).astype(np.float16)
    mid16 = O.epilogue(acc_ref, scale, b.astype(np.float32), False, False)
    add_range = 5.1
    want2 = O.add(O.quantize(mid16, add_range), add_range, O.quantize(ident16, add_range), add_range, True, True, out_range)
    out2, _ = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=False, out_int8=True, out_range=out_range,
                           res=to_dev(ident16), mid_int8=False, a_rq=add_range, b_rq=add_range, relu2=True)
    assert np.array_equal(out2.cpu().numpy(), want2)
    note("fp16 add of fp16 operands, fp16 out")
    want3 = O.add(mid16, 127.0, ident16, 127.0, True, False)
    out3, _ = conv.forward(rb, to_dev(x), n, x_range=x_range, relu=False, out_int8=False,
                           res=to_dev(ident16), mid_int8=False, relu2=True)
    assert np.array_equal(out3.cpu().numpy().view(np.uint16), want3.view(np.uint16))


# ----------------------------------------------------------------------------- elementwise / dense
def test_convert_add_and_dense():
    L = capi.lib()
    rng = np.random.default_rng(31)
    n, c = 5000, 32
    note("quantise / dequantise / pad rows")
    x = (rng.standard_normal((n, 5)) * 20).astype(np.float16)
    s = 38.1  # dynamic range
    out = torch.zeros((n, 16), dtype=torch.int8, device=DEV)
    d_x = to_dev(x)
    capi.check(L.scn_convert_rows(ptr(d_x), capi.DTYPE_FP16, 5, 5, 0.0, ptr(out), capi.DTYPE_INT8, 16, 16, s, 0, n, None, stream()))
    torch.cuda.synchronize()
    want = np.zeros((n, 16), np.int8)
    want[:, :5] = O.quantize(x, s)
    assert np.array_equal(out.cpu().numpy(), want)
    q = rng.integers(-127, 128, (n, c)).astype(np.int8)
    out = torch.zeros((n, c), dtype=torch.float16, device=DEV)
    d_q = to_dev(q)
    capi.check(L.scn_convert_rows(ptr(d_q), capi.DTYPE_INT8, c, c, s, ptr(out), capi.DTYPE_FP16, c, c, 0.0, 0, n, None, stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), O.dequantize(q, s).view(np.uint16))
    padded = torch.full((n, 8), 7, dtype=torch.float16, device=DEV)
    capi.check(L.scn_convert_rows(ptr(d_x), capi.DTYPE_FP16, 5, 5, 0.0, ptr(padded), capi.DTYPE_FP16, 8, 8, 0.0, 0, n, None, stream()))
    torch.cuda.synchronize()
    pw = np.zeros((n, 8), np.float16); pw[:, :5] = x
    assert np.array_equal(padded.cpu().numpy().view(np.uint16), pw.view(np.uint16))
    note("add + relu, int8 and fp16 operands, device-side count")
    a = rng.integers(-127, 128, (n, c)).astype(np.int8)
    b = rng.integers(-127, 128, (n, c)).astype(np.int8)
    n_dev = torch.tensor([4321], dtype=torch.int32, device=DEV)
    out = torch.zeros((n, c), dtype=torch.int8, device=DEV)
    da, db = to_dev(a), to_dev(b)  # keep both alive: the caching allocator would hand b the memory of a
    capi.check(L.scn_add_relu(ptr(da), capi.DTYPE_INT8, 3.8, 0.0, ptr(db), capi.DTYPE_INT8, 2.5, 0.0, ptr(out),
                              capi.DTYPE_INT8, 5.1, 1, c, n, ptr(n_dev), stream()))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got[:4321], O.add(a[:4321], 3.8, b[:4321], 2.5, True, True, 5.1)) and not got[4321:].any()
    h1 = rng.standard_normal((n, c)).astype(np.float16); h2 = rng.standard_normal((n, c)).astype(np.float16)
    out = torch.zeros((n, c), dtype=torch.float16, device=DEV)
    d1, d2 = to_dev(h1), to_dev(h2)
    capi.check(L.scn_add_relu(ptr(d1), capi.DTYPE_FP16, 0.0, 0.0, ptr(d2), capi.DTYPE_FP16, 0.0, 0.0, ptr(out),
                              capi.DTYPE_FP16, 0.0, 0, c, n, None, stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), O.add(h1, 127.0, h2, 127.0, False, False).view(np.uint16))
    note("scatter dense, plain and with the fused transpose")
    dims = (2, 45, 37)
    lin = rng.choice(int(np.prod(dims)), 1500, replace=False)
    idx = np.zeros((1500, 4), np.int32)
    idx[:, 3] = lin % dims[2]; idx[:, 2] = (lin // dims[2]) % dims[1]; idx[:, 1] = lin // (dims[2] * dims[1])
    feat = rng.standard_normal((1500, 16)).astype(np.float16)
    dense_ref = O.scatter_dense(feat, idx, dims)
    shape = capi.i5(1, 16, *dims)
    out = torch.full((1, 16, *dims), 3, dtype=torch.float16, device=DEV)
    d_feat, d_idx = to_dev(feat), to_dev(idx)
    capi.check(L.scn_scatter_dense(ptr(d_feat), capi.DTYPE_FP16, 0.0, 16, 16, ptr(d_idx), 1500, None, shape, None, ptr(out), stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), dense_ref.view(np.uint16))
    perm = (0, 1, 4, 2, 3)
    out = torch.full((1, 16, dims[2], dims[0], dims[1]), 3, dtype=torch.float16, device=DEV)
    capi.check(L.scn_scatter_dense(ptr(d_feat), capi.DTYPE_FP16, 0.0, 16, 16, ptr(d_idx), 1500, None, shape,
                                   capi.i5(*perm), ptr(out), stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), np.ascontiguousarray(dense_ref.transpose(perm)).view(np.uint16))
    qf = rng.integers(-127, 128, (1500, 16)).astype(np.int8)
    out = torch.zeros((1, 16, *dims), dtype=torch.float16, device=DEV)
    d_qf = to_dev(qf)
    capi.check(L.scn_scatter_dense(ptr(d_qf), capi.DTYPE_INT8, 6.35, 16, 16, ptr(d_idx), 1500, None, shape, None, ptr(out), stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), O.scatter_dense(O.dequantize(qf, 6.35), idx, dims).view(np.uint16))


@pytest.mark.parametrize("cin,cout", [(32, 16), (128, 64)])
def test_inverse_rulebook_and_int8_conv(cin, cout, centerpoint_input):
    """SparseInverseConvolution: the swapped rulebook of a strided convolution (pairs identical to the
    oracle's, output rows = the forward convolution's input rows, also with a device-side input count)
    and an int8 convolution through it, bit-exact."""
    _, idx_all = centerpoint_input
    rng = np.random.default_rng(cin)
    n = 20000
    idx = idx_all[:n]
    grid = (41, 1440, 1440)
    ks, st, pad = (3, 3, 3), (2, 2, 2), (1, 1, 1)
    note(f"inverse rulebook of a stride-2 3x3x3 convolution on {n} fixture voxels, int8 conv {cin}->{cout}")
    ref_f = O.rulebook_sparse(idx, grid, ks, st, pad, max_out=n * 2)
    ref_i = O.rulebook_inverse(ref_f, idx, grid)
    d_idx = to_dev(idx)
    fwd = GpuRulebook(n, n * 2, 27)
    fwd.build_sparse(d_idx, n, grid, ks, st, pad)
    m = fwd.n_out()
    assert m == ref_f.n_out
    inv = GpuRulebook(n * 2, n, 27)
    inv.build_inverse(fwd)
    assert inv.n_out() == n
    pin, pout, offs = inv.pairs(ref_i.num_pairs + 16)
    assert np.array_equal(offs, ref_i.offsets) and np.array_equal(pin, ref_i.pair_in) and np.array_equal(pout, ref_i.pair_out)
    assert np.array_equal(inv.out_indices(), idx)
    x = rng.integers(-127, 128, (m, cin)).astype(np.int8)
    w, b, ranges = _weights(rng, cout, ks, cin)
    x_range, out_range = 4.2, 7.7
    wq, s_w = O.quantize_weights(w, ranges)
    acc_ref = O.conv_int8_acc(x, wq, ref_i)
    scale = (np.float32(x_range) / np.float32(127) * s_w).astype(np.float32)
    conv = GpuConv(w, ranges, b, capi.PRECISION_INT8)
    out, acc = conv.forward(inv, to_dev(x), n, x_range=x_range, relu=True, out_int8=True, out_range=out_range, want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(out.cpu().numpy(), O.epilogue(acc_ref, scale, b.astype(np.float32), True, True, out_range))
    note("device-side input count below the bound: rows past it neither appear as outputs nor as neighbours")
    k = n - 777
    cnt = to_dev(np.array([k], np.uint32))
    ref_f2 = O.rulebook_sparse(idx[:k], grid, ks, st, pad, max_out=n * 2)
    ref_i2 = O.rulebook_inverse(ref_f2, idx[:k], grid)
    fwd.build_sparse(d_idx, n, grid, ks, st, pad, n_dev=cnt)
    inv.build_inverse(fwd, n_in_dev=cnt)
    assert inv.n_out() == k
    pin, pout, offs = inv.pairs(ref_i2.num_pairs + 16)
    assert np.array_equal(offs, ref_i2.offsets) and np.array_equal(pin, ref_i2.pair_in) and np.array_equal(pout, ref_i2.pair_out)


def test_scatter_dense_with_row_map():
    """The dense-major variant (row map, no clear, whole 16-byte stores) against the oracle: fp16 and int8
    rows, channel counts that are not a multiple of 8, permuted spatial axes, a device-side row count, a
    map holding stale entries, and layouts that do not qualify (channel-last, odd plane)."""
    L = capi.lib()
    rng = np.random.default_rng(77)
    for dims, c, ld, n, perm in [((2, 44, 36), 16, 16, 1500, None), ((2, 44, 36), 16, 16, 1500, (0, 1, 4, 2, 3)),
                                 ((3, 40, 40), 20, 24, 2500, (0, 1, 2, 3, 4)), ((1, 64, 72), 128, 128, 4000, (0, 1, 3, 2, 4)),
                                 ((2, 44, 36), 16, 16, 1500, (0, 2, 3, 4, 1)), ((2, 45, 37), 16, 16, 1500, None),
                                 ((2, 44, 36), 16, 16, 0, None)]:
        note(f"scatter with map dims={dims} c={c} ld={ld} n={n} perm={perm}")
        cells = int(np.prod(dims))
        lin = rng.choice(cells, max(n, 1), replace=False)[:n]
        idx = np.zeros((n, 4), np.int32)
        idx[:, 3] = lin % dims[2]; idx[:, 2] = (lin // dims[2]) % dims[1]; idx[:, 1] = lin // (dims[2] * dims[1])
        shape = capi.i5(1, c, *dims)
        pm = capi.i5(*perm) if perm else None
        want_cells = L.scn_scatter_dense_map_cells(shape, pm)
        qualifies = cells % 8 == 0 and (perm is None or perm[1] == 1)
        assert want_cells == (cells if qualifies else 0)
        cell_map = torch.full((max(want_cells, 1),), 5, dtype=torch.int32, device=DEV)   # stale contents
        oshape = (1, c, *dims) if not perm else tuple((1, c, *dims)[a] for a in perm)
        for dtype in (capi.DTYPE_FP16, capi.DTYPE_INT8):
            if dtype == capi.DTYPE_FP16:
                feat = rng.standard_normal((n, ld)).astype(np.float16); ref_rows = feat[:, :c]; rng_ = 0.0
            else:
                feat = rng.integers(-127, 128, (n, ld)).astype(np.int8); ref_rows = O.dequantize(feat[:, :c], 6.35); rng_ = 6.35
            ref = O.scatter_dense(ref_rows, idx, dims)
            if perm: ref = np.ascontiguousarray(ref.transpose(perm))
            out = torch.full(oshape, 3, dtype=torch.float16, device=DEV)
            d_feat, d_idx = to_dev(feat), to_dev(idx)
            capi.check(L.scn_scatter_dense_with_map(ptr(d_feat) if n else None, dtype, rng_, c, ld, ptr(d_idx) if n else None,
                                                    n, None, shape, pm, ptr(out), ptr(cell_map) if want_cells else None, stream()))
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))
            if n:  # device-side count: only the first rows are scattered
                k = n // 3
                cnt = to_dev(np.array([k], np.uint32))
                ref = O.scatter_dense(ref_rows[:k], idx[:k], dims)
                if perm: ref = np.ascontiguousarray(ref.transpose(perm))
                out.fill_(7)
                capi.check(L.scn_scatter_dense_with_map(ptr(d_feat), dtype, rng_, c, ld, ptr(d_idx), n, ptr(cnt), shape, pm,
                                                        ptr(out), ptr(cell_map) if want_cells else None, stream()))
                torch.cuda.synchronize()
                assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("fmt", ["zyx", "xyz"])
def test_dense_output_layouts_and_int8(fmt):
    """push_dense's other output forms (engine.hpp:26,114-123): int8 output in the NCHW layout (with and without a
    Transpose), and NCHW32 / NHWzC of the [1, C * Z, H, W] view, fp16 and int8, against numpy reshapes of the
    oracle's NCHW tensor."""
    L = capi.lib()
    rng = np.random.default_rng(17)
    dims = (2, 36, 40) if fmt == "zyx" else (36, 40, 2)
    zaxis = 0 if fmt == "zyx" else 2
    n = 1500
    vol = int(np.prod(dims))
    lin = np.sort(rng.choice(vol, n, replace=False))
    idx = np.zeros((n, 4), np.int32)
    idx[:, 1], idx[:, 2], idx[:, 3] = lin // (dims[1] * dims[2]), (lin // dims[2]) % dims[1], lin % dims[2]
    d_idx = to_dev(idx)
    for c in (24, 128):      # 24 * 2 = 48 channels: NCHW32 pads the second group
        ld = (c + 15) // 16 * 16
        for in_dtype in (capi.DTYPE_INT8, capi.DTYPE_FP16):
            if in_dtype == capi.DTYPE_INT8:
                feat = np.zeros((n, ld), np.int8); feat[:, :c] = rng.integers(-127, 128, (n, c)); in_rng = 3.3
                val = feat[:, :c].astype(np.float32) * (np.float32(in_rng) / np.float32(127))
            else:
                feat = np.zeros((n, ld), np.float16); feat[:, :c] = rng.standard_normal((n, c)); in_rng = 0.0
                val = feat[:, :c].astype(np.float32)
            d_feat = to_dev(feat)
            for out_i8 in (False, True):
                out_rng = 2.9 if out_i8 else 0.0
                rows = O.quantize_f32(val, out_rng) if out_i8 else val.astype(np.float16)
                nchw = O.scatter_dense(rows, idx, dims)
                for layout, name in ((1, "NCHW"), (2, "NCHW32"), (3, "NHWzC")):
                    perms = [None, (0, 1, 4, 2, 3)] if layout == 1 else [None]
                    for perm in perms:
                        want = nchw if layout == 1 else O.dense_to_layout(nchw, fmt, name)
                        if perm:
                            want = np.ascontiguousarray(want.transpose(perm))
                        note(f"dense {name} perm={perm} fmt={fmt} C={c} in={in_dtype} int8 out={out_i8}: {want.shape}")
                        out = torch.full(want.shape, 3, dtype=torch.int8 if out_i8 else torch.float16, device=DEV)
                        capi.check(L.scn_scatter_dense_layout(ptr(d_feat), in_dtype, in_rng, c, ld, ptr(d_idx), n, None,
                                                              capi.i5(1, c, *dims), capi.i5(*perm) if perm else None, zaxis, layout,
                                                              capi.DTYPE_INT8 if out_i8 else capi.DTYPE_FP16, out_rng, ptr(out), stream()))
                        torch.cuda.synchronize()
                        got = out.cpu().numpy()
                        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
                        assert np.count_nonzero(got) > n


def test_memset_kernel_any_alignment_and_inside_a_graph():
    """scn_memset_async (Tensor::memset of the C++ header): byte ranges with unaligned heads and tails, and
    recorded into a HIP graph that is replayed with other work in between."""
    L = capi.lib()
    note("byte fill kernel: unaligned ranges, then graph replays")
    buf = torch.zeros(100003, dtype=torch.uint8, device=DEV)
    for off, n, v in ((0, 100003, 7), (1, 15, 9), (3, 4096 + 5, 250), (16, 64, 1), (17, 1, 33), (5, 0, 99)):
        buf.fill_(0)
        capi.check(L.scn_memset_async(C.c_void_p(buf.data_ptr() + off), v, n, stream()))
        torch.cuda.synchronize()
        want = np.zeros(100003, np.uint8)
        want[off:off + n] = v
        assert np.array_equal(buf.cpu().numpy(), want), (off, n, v)
    st = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        capi.check(L.scn_memset_async(C.c_void_p(buf.data_ptr() + 2), 5, 1001, C.c_void_p(st.cuda_stream)))
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=st):
        capi.check(L.scn_memset_async(C.c_void_p(buf.data_ptr() + 2), 5, 1001, C.c_void_p(st.cuda_stream)))
    for rep in range(3):
        buf.fill_(rep + 10)
        assert np.isfinite(torch.randn(1 << 18, device=DEV).sum().item())
        g.replay()
        torch.cuda.synchronize()
        want = np.full(100003, rep + 10, np.uint8)
        want[2:1003] = 5
        assert np.array_equal(buf.cpu().numpy(), want), rep


# ----------------------------------------------------------------------------- voxelization
def _voxelizer(max_voxels=160000, max_points=300000, per_voxel=10):
    p = capi.VoxelizationParam()
    p.min_range[:] = synth.MIN_RANGE; p.max_range[:] = synth.MAX_RANGE; p.voxel_size[:] = synth.VOXEL_SIZE
    p.grid_size[:] = synth.GRID_XYZ
    p.num_feature, p.max_voxels, p.max_points_per_voxel, p.max_points = 5, max_voxels, per_voxel, max_points
    h = capi.lib().scn_voxelizer_create(C.byref(p))
    assert h
    return h


def _run_voxelizer(h, pts, order, max_voxels):
    L = capi.lib()
    code = capi.ORDER_ZYX if order == "zyx" else capi.ORDER_XYZ
    d = to_dev(pts)
    if pts.dtype == np.float32:
        capi.check(L.scn_voxelizer_forward_points(h, ptr(d), capi.DTYPE_FP32, pts.shape[0], code, stream()))
    else:
        capi.check(L.scn_voxelizer_forward(h, ptr(d), pts.shape[0], code, stream()))
    nv = L.scn_voxelizer_num_voxels(h, stream())
    f = copy_from_ptr(L.scn_voxelizer_features(h), (nv, 5), np.float16).cpu().numpy()
    i = copy_from_ptr(L.scn_voxelizer_indices(h), (nv, 4), np.int32).cpu().numpy()
    c = copy_from_ptr(L.scn_voxelizer_points_per_voxel(h), (nv,), np.int32).cpu().numpy()
    return f, i, c


@pytest.mark.parametrize("order", ["zyx", "xyz"])
def test_voxelization_real_frame_bit_exact(order, nuscenes_frame):
    note(f"voxelization of the 271,156-point frame, order {order}")
    L = capi.lib()
    h = _voxelizer()
    try:
        f, i, c = _run_voxelizer(h, nuscenes_frame, order, 160000)
        rf, ri, rc = O.voxelize(nuscenes_frame, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
        assert f.shape[0] == KNOWN["nuscenes_frame"]["voxels"]
        assert np.array_equal(i, ri) and np.array_equal(c, rc)
        assert np.array_equal(f.view(np.uint16), rf.view(np.uint16))
        g = capi.i3()
        L.scn_voxelizer_grid_size(h, capi.ORDER_ZYX if order == "zyx" else capi.ORDER_XYZ, g)
        assert list(g) == ([41, 1440, 1440] if order == "zyx" else [1440, 1440, 41])
        note("second frame on the same object (state is cleared), then an empty frame")
        pts2 = synth.lidar_frame(3, 100000)
        f2, i2, c2 = _run_voxelizer(h, pts2, order, 160000)
        rf2, ri2, rc2 = O.voxelize(pts2, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
        assert np.array_equal(i2, ri2) and np.array_equal(c2, rc2) and np.array_equal(f2.view(np.uint16), rf2.view(np.uint16))
        f0, i0, _ = _run_voxelizer(h, pts2[:0], order, 160000)
        assert f0.shape[0] == 0
    finally:
        L.scn_voxelizer_destroy(h)


@pytest.mark.parametrize("order", ["zyx", "xyz"])
def test_voxelization_of_fp32_points_bit_exact(order, nuscenes_frame):
    """The raw fp32 sweep, as CUDA-CenterPoint's preprocessing takes it (PreProcessCuda::generateVoxels(const float*),
    src/preprocess.cpp:82, src/preprocess_kernels.cu:70-154): coordinates that no fp16 value represents, so that the
    range test, the cell index and the fp32 sums really run on the fp32 values."""
    rng = np.random.default_rng(9)
    pts = nuscenes_frame[:150000].astype(np.float32)
    pts[:, :3] += rng.uniform(-0.03, 0.03, (pts.shape[0], 3)).astype(np.float32)
    pts[:, 3] *= np.float32(1.0009765)
    assert not np.array_equal(pts, pts.astype(np.float16).astype(np.float32))
    note(f"voxelization of {pts.shape[0]} fp32 points, order {order}")
    L = capi.lib()
    h = _voxelizer()
    try:
        f, i, c = _run_voxelizer(h, pts, order, 160000)
        rf, ri, rc = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
        assert np.array_equal(i, ri) and np.array_equal(c, rc)
        assert np.array_equal(f.view(np.uint16), rf.view(np.uint16))
        # ... and differs from what the fp16-rounded points give (another set of cells)
        r16 = O.voxelize(pts.astype(np.float16), synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
        assert r16[1].shape != ri.shape or not np.array_equal(r16[1], ri)
        note("an fp16 frame on the same object afterwards")
        f2, i2, c2 = _run_voxelizer(h, nuscenes_frame[:50000], order, 160000)
        rf2, ri2, rc2 = O.voxelize(nuscenes_frame[:50000], synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
        assert np.array_equal(i2, ri2) and np.array_equal(c2, rc2) and np.array_equal(f2.view(np.uint16), rf2.view(np.uint16))
    finally:
        L.scn_voxelizer_destroy(h)


def test_voxelizer_state_survives_many_forwards(nuscenes_frame):
    """The voxelizer cleans its working memory at the end of a forward instead of clearing it at the start, and never
    clears the per-voxel point slots at all (a forward writes every slot it reads): 600 forwards on one object,
    alternating three frames (a ring-ordered real one with voxels that overflow, a synthetic one, a short one), checked
    against the oracle at the first calls, at intervals and at the end; then a frame that overflows max_voxels (cells
    beyond the kept rows must be cleaned too) followed by an ordinary one."""
    L = capi.lib()
    frames = [nuscenes_frame[:120000], synth.lidar_frame(5, 90000), nuscenes_frame[200000:200700]]
    want = [O.voxelize(f, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order="zyx") for f in frames]
    devs = [to_dev(f) for f in frames]
    h = _voxelizer()
    try:
        note("600 forwards on one voxelizer, three frames in turn")
        for call in range(600):
            k = call % 3
            capi.check(L.scn_voxelizer_forward(h, ptr(devs[k]), frames[k].shape[0], capi.ORDER_ZYX, stream()))
            if call < 6 or 120 <= call <= 135 or 250 <= call <= 262 or 376 <= call <= 388 or call >= 594:
                nv = L.scn_voxelizer_num_voxels(h, stream())
                f = copy_from_ptr(L.scn_voxelizer_features(h), (nv, 5), np.float16).cpu().numpy()
                i = copy_from_ptr(L.scn_voxelizer_indices(h), (nv, 4), np.int32).cpu().numpy()
                c = copy_from_ptr(L.scn_voxelizer_points_per_voxel(h), (nv,), np.int32).cpu().numpy()
                rf, ri, rc = want[k]
                assert np.array_equal(i, ri) and np.array_equal(c, rc), call
                assert np.array_equal(f.view(np.uint16), rf.view(np.uint16)), call
    finally:
        L.scn_voxelizer_destroy(h)
    note("a frame that overflows max_voxels, then an ordinary one on the same object")
    h = _voxelizer(max_voxels=3000)
    try:
        f, i, c = _run_voxelizer(h, frames[0], "zyx", 3000)
        rf, ri, rc = O.voxelize(frames[0], synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, max_voxels=3000, order="zyx")
        assert f.shape[0] == 3000 and np.array_equal(i, ri) and np.array_equal(c, rc) and np.array_equal(f.view(np.uint16), rf.view(np.uint16))
        f, i, c = _run_voxelizer(h, frames[2], "zyx", 3000)
        rf, ri, rc = want[2]
        assert np.array_equal(i, ri) and np.array_equal(c, rc) and np.array_equal(f.view(np.uint16), rf.view(np.uint16))
    finally:
        L.scn_voxelizer_destroy(h)


@pytest.mark.parametrize("per_voxel", [1, 3, 16, 24])
def test_voxelization_points_per_voxel_limits(per_voxel, nuscenes_frame):
    """max_points_per_voxel of 1 and 3 (most voxels of a real sweep overflow: the lowest point indices must win whatever
    the arrival order), 16 (the most that the mean kernel puts in order itself) and 24 (every voxel through the
    cascade), two forwards each."""
    note(f"voxelization with at most {per_voxel} points per voxel")
    L = capi.lib()
    h = _voxelizer(per_voxel=per_voxel)
    try:
        for pts in (nuscenes_frame[:150000], nuscenes_frame[100000:220000]):
            f, i, c = _run_voxelizer(h, pts, "zyx", 160000)
            rf, ri, rc = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, max_points=per_voxel,
                                    order="zyx")
            assert np.array_equal(i, ri) and np.array_equal(c, rc)
            assert np.array_equal(f.view(np.uint16), rf.view(np.uint16))
            assert (rc > per_voxel).any()
    finally:
        L.scn_voxelizer_destroy(h)


@pytest.mark.parametrize("per_voxel", [10, 24])
def test_voxelizer_forward_replayed_from_a_graph(per_voxel, nuscenes_frame):
    """A forward captured once into a HIP graph and replayed on other frames of the same point count (the graph fixes
    the launch arguments, the point buffer's contents change): the voxelizer keeps no state on the host, so every
    replay must equal the oracle -- with 10 slots per voxel (only the overflowing voxels go through the cascade) and
    with 24 (every voxel does), direct forwards mixed in between."""
    L = capi.lib()
    n = 100000
    frames = [nuscenes_frame[:n], nuscenes_frame[150000:150000 + n], synth.lidar_frame(8, n), nuscenes_frame[60000:60000 + n]]
    want = [O.voxelize(f, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, max_points=per_voxel, order="zyx")
            for f in frames]
    note(f"voxelizer forward captured into a graph, {per_voxel} slots per voxel, replayed on four frames")
    h = _voxelizer(per_voxel=per_voxel)
    st = torch.cuda.Stream()
    sp = C.c_void_p(st.cuda_stream)
    buf = to_dev(frames[0]).clone()

    def check(k, what):
        nv = L.scn_voxelizer_num_voxels(h, sp)
        f = copy_from_ptr(L.scn_voxelizer_features(h), (nv, 5), np.float16).cpu().numpy()
        i = copy_from_ptr(L.scn_voxelizer_indices(h), (nv, 4), np.int32).cpu().numpy()
        c = copy_from_ptr(L.scn_voxelizer_points_per_voxel(h), (nv,), np.int32).cpu().numpy()
        rf, ri, rc = want[k]
        assert np.array_equal(i, ri) and np.array_equal(c, rc), (what, k)
        assert np.array_equal(f.view(np.uint16), rf.view(np.uint16)), (what, k)

    try:
        with torch.cuda.stream(st):
            capi.check(L.scn_voxelizer_forward(h, ptr(buf), n, capi.ORDER_ZYX, sp))
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            capi.check(L.scn_voxelizer_forward(h, ptr(buf), n, capi.ORDER_ZYX, sp))
        torch.cuda.synchronize()
        for rep, k in enumerate((1, 2, 0, 3, 3, 1)):
            with torch.cuda.stream(st):
                buf.copy_(to_dev(frames[k]))
                if rep == 3:     # a direct forward on another frame between two replays
                    other = to_dev(frames[2])
                    capi.check(L.scn_voxelizer_forward(h, ptr(other), n, capi.ORDER_ZYX, sp))
                g.replay()
            torch.cuda.synchronize()
            check(k, f"replay {rep}")
    finally:
        L.scn_voxelizer_destroy(h)


def test_voxelization_truncates_at_max_voxels(nuscenes_frame):
    note("voxelization with max_voxels=5000")
    L = capi.lib()
    h = _voxelizer(max_voxels=5000)
    try:
        f, i, c = _run_voxelizer(h, nuscenes_frame[:60000], "zyx", 5000)
        rf, ri, rc = O.voxelize(nuscenes_frame[:60000], synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ,
                                max_voxels=5000, order="zyx")
        assert f.shape[0] == 5000 and np.array_equal(i, ri) and np.array_equal(c, rc)
        assert np.array_equal(f.view(np.uint16), rf.view(np.uint16))
    finally:
        L.scn_voxelizer_destroy(h)
