"""Pins the CPU oracle: golden counts from the reference's fixtures, torch's dense conv3d,
closed forms and brute force.  Everything here runs without a GPU."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import scn_oracle as O
from lidar_ai_solution_amd import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
KNOWN = json.load(open(os.path.join(GOLDEN, "known_answers.json")))


# ----------------------------------------------------------------------------- half / hash
def test_half_conversion_matches_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    f = np.empty(65536, np.float32)
    O.lib().scn_ref_half2float_array(O._p(allh), O._p(f), 65536)
    ref = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1, 300, 70000)])
    # exact ties and neighbours of every representable half
    mid = (ref[:-1].astype(np.float64) + ref[1:].astype(np.float64)) / 2
    mid = mid[np.isfinite(mid)].astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                        np.array([0.0, -0.0, np.inf, -np.inf, 65504, 65519.99, 65520, 1e-10], np.float32)])
    h = np.empty(x.size, np.uint16)
    O.lib().scn_ref_float2half_array(O._p(x), O._p(h), x.size)
    with np.errstate(over="ignore"):
        assert np.array_equal(h, x.astype(np.float16).view(np.uint16))


def test_hash_is_64bit_murmur_finaliser():
    # The hash only places keys in the reference's open-addressing table; no output depends on it, so this is a guard
    # on the C restatement (64-bit evaluation, libraries/3DSparseConvolution/src/voxelization.cu:41-48), not a parity pin.
    # What the structure fixes without re-typing it: xor-shifts and odd multiplications are invertible modulo 2^64, so
    # the function is a bijection and undoing the steps with the modular inverses must give the key back.
    M = (1 << 64) - 1
    def unshift(v, s):
        r = v
        for _ in range(64 // s + 1):
            r = v ^ (r >> s)
        return r
    def inverse(h):
        h = unshift(h, 16)
        h = (h * pow(0xC2B2AE35, -1, 1 << 64)) & M
        h = unshift(h, 13)
        h = (h * pow(0x85EBCA6B, -1, 1 << 64)) & M
        return unshift(h, 16)
    rng0 = np.random.default_rng(7)
    keys = [int(v) for v in rng0.integers(0, 2 ** 32, 3000)]
    assert all(inverse(O.hash64(k)) == k for k in keys)
    assert len({O.hash64(k) for k in keys}) == len(set(keys))

    def py(k):
        M = (1 << 64) - 1
        k ^= k >> 16
        k = (k * 0x85EBCA6B) & M
        k ^= k >> 13
        k = (k * 0xC2B2AE35) & M
        k ^= k >> 16
        return k
    assert O.hash64(0) == 0
    rng = np.random.default_rng(1)
    for k in [1, 2, 0xFFFFFFFF, 85017599] + [int(v) for v in rng.integers(0, 2 ** 32, 2000)]:
        assert O.hash64(k) == py(k)
    # the 64-bit evaluation differs from a 32-bit-wrapped murmur3 fmix32 for most keys
    def fmix32(k):
        k ^= k >> 16; k = (k * 0x85EBCA6B) & 0xFFFFFFFF; k ^= k >> 13; k = (k * 0xC2B2AE35) & 0xFFFFFFFF; k ^= k >> 16
        return k
    assert any(O.hash64(k) & 0xFFFFFFFF != fmix32(k) for k in range(1000, 1100))


# ----------------------------------------------------------------------------- voxelization
def _brute_voxelize(pts16, order):
    p = pts16.astype(np.float32)
    mn = np.array(synth.MIN_RANGE, np.float32); mx = np.array(synth.MAX_RANGE, np.float32)
    vs = np.array(synth.VOXEL_SIZE, np.float32)
    ok = np.all((p[:, :3] >= mn) & (p[:, :3] < mx), axis=1)
    ijk = np.floor((p[:, :3] - mn) / vs).astype(np.int64)
    G = np.array(synth.GRID_XYZ)
    ok &= np.all((ijk >= 0) & (ijk < G), axis=1)
    if order == "zyx":
        key = (ijk[:, 2] * G[1] + ijk[:, 1]) * G[0] + ijk[:, 0]
    else:
        key = (ijk[:, 0] * G[1] + ijk[:, 1]) * G[2] + ijk[:, 2]
    ids = np.nonzero(ok)[0]
    voxels = {}
    for i in ids:
        voxels.setdefault(int(key[i]), []).append(i)
    feats, coords, counts = [], [], []
    for k in sorted(voxels):
        members = voxels[k][:10]
        s = p[members[0]].copy()
        for m in members[1:]:
            s = s + p[m]
        s = s / np.float32(len(members))
        feats.append(s.astype(np.float16))
        x, y, z = ijk[members[0]]
        coords.append([0, z, y, x] if order == "zyx" else [0, x, y, z])
        counts.append(len(voxels[k]))
    return np.array(feats), np.array(coords, np.int32), np.array(counts, np.int32), int(ok.sum())


@pytest.mark.parametrize("order", ["zyx", "xyz"])
def test_voxelize_against_brute_force(order, nuscenes_frame):
    pts = nuscenes_frame[:40000]
    f, c, n = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
    bf, bc, bn, _ = _brute_voxelize(pts, order)
    assert np.array_equal(c, bc)
    assert np.array_equal(n, bn)
    assert np.array_equal(f.view(np.uint16), bf.view(np.uint16))
    assert n.max() > 10  # the crowded-voxel rule is exercised


@pytest.mark.parametrize("order", ["zyx", "xyz"])
def test_voxelize_fp32_points_against_brute_force(order, nuscenes_frame):
    """fp32 points (CUDA-CenterPoint's preprocessing, src/preprocess_kernels.cu:70-154) that no fp16 value represents."""
    rng = np.random.default_rng(9)
    pts = nuscenes_frame[:40000].astype(np.float32)
    pts[:, :3] += rng.uniform(-0.03, 0.03, (pts.shape[0], 3)).astype(np.float32)
    assert not np.array_equal(pts, pts.astype(np.float16).astype(np.float32))
    f, c, n = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, order=order)
    bf, bc, bn, _ = _brute_voxelize(pts, order)
    assert np.array_equal(c, bc)
    assert np.array_equal(n, bn)
    assert np.array_equal(f.view(np.uint16), bf.view(np.uint16))
    assert n.max() > 10


def test_voxelize_known_answer_full_frame(nuscenes_frame):
    ka = KNOWN["nuscenes_frame"]
    assert nuscenes_frame.shape[0] == ka["points"]
    f, c, n = O.voxelize(nuscenes_frame, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ,
                         max_voxels=160000, order="zyx")
    assert f.shape[0] == ka["voxels"]
    assert int(n.sum()) == ka["in_range"]
    assert int((n > 10).sum()) == ka["voxels_over_10"]
    assert int(n.max()) == ka["max_points_in_voxel"]
    lin = (c[:, 1].astype(np.int64) * 1440 + c[:, 2]) * 1440 + c[:, 3]
    assert np.all(np.diff(lin) > 0)


def test_voxelize_truncates_in_canonical_order(nuscenes_frame):
    pts = nuscenes_frame[:20000]
    f, c, _ = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ)
    f2, c2, _ = O.voxelize(pts, synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ, max_voxels=1000)
    assert f2.shape[0] == 1000 and np.array_equal(c2, c[:1000]) and np.array_equal(f2, f[:1000])
    f0, c0, _ = O.voxelize(pts[:0], synth.MIN_RANGE, synth.MAX_RANGE, synth.VOXEL_SIZE, synth.GRID_XYZ)
    assert f0.shape == (0, 5) and c0.shape == (0, 4)


# ----------------------------------------------------------------------------- rulebooks
def test_rulebook_counts_on_reference_fixture(centerpoint_input):
    """Per-stage active-voxel and pair counts of the 79,745-voxel fixture."""
    _, idx = centerpoint_input
    ka = KNOWN["centerpoint_fixture"]
    geoms = [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
             ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((3, 1, 1), (2, 1, 1), (0, 0, 0))]
    grid = ka["grids"][0]
    for s in range(4):
        assert idx.shape[0] == ka["active"][s]
        sub = O.rulebook_subm(idx, grid, (3, 3, 3))
        assert sub.num_pairs == ka["subm_pairs"][s]
        k, st, p = geoms[s]
        rb = O.rulebook_sparse(idx, grid, k, st, p)
        assert rb.out_grid == ka["grids"][s + 1]
        assert rb.num_pairs == ka["strided_pairs"][s]
        assert rb.n_out == ka["active"][s + 1]
        idx, grid = rb.out_indices, rb.out_grid


def _random_sparse(rng, grid, n):
    vol = int(np.prod(grid))
    lin = rng.choice(vol, size=n, replace=False)
    idx = np.zeros((n, 4), np.int32)
    idx[:, 3] = lin % grid[2]
    idx[:, 2] = (lin // grid[2]) % grid[1]
    idx[:, 1] = lin // (grid[2] * grid[1])
    return idx


def test_subm_invariants():
    rng = np.random.default_rng(3)
    grid = (9, 20, 17)
    idx = _random_sparse(rng, grid, 900)
    rb = O.rulebook_subm(idx, grid, (3, 3, 3))
    offs = rb.offsets
    # centre offset: exactly one pair (r, r) per row, in row order
    c0, c1 = offs[13], offs[14]
    assert c1 - c0 == 900 and np.array_equal(rb.pair_in[c0:c1], np.arange(900)) and np.array_equal(rb.pair_out[c0:c1], np.arange(900))
    # symmetry: (i, o, k) <-> (o, i, 26-k)
    S = set()
    for k in range(27):
        for i, o in zip(rb.pair_in[offs[k]:offs[k + 1]], rb.pair_out[offs[k]:offs[k + 1]]):
            S.add((int(i), int(o), k))
    assert all((o, i, 26 - k) in S for (i, o, k) in S)
    # brute force with a dictionary
    d = {tuple(r[1:]): j for j, r in enumerate(idx)}
    B = set()
    for o, r in enumerate(idx):
        for k0 in range(3):
            for k1 in range(3):
                for k2 in range(3):
                    i = d.get((r[1] + k0 - 1, r[2] + k1 - 1, r[3] + k2 - 1))
                    if i is not None:
                        B.add((i, o, (k0 * 3 + k1) * 3 + k2))
    assert B == S
    # sorted by (k, out, in)
    for k in range(27):
        assert np.all(np.diff(rb.pair_out[offs[k]:offs[k + 1]]) > 0)


CONV_CASES = [
    # grid, n, ksize, stride, padding, dilation, subm
    ((7, 12, 10), 300, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),
    ((7, 12, 10), 300, (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1), False),
    ((5, 12, 11), 250, (3, 3, 3), (2, 2, 2), (0, 1, 1), (1, 1, 1), False),
    ((5, 9, 9), 200, (3, 1, 1), (2, 1, 1), (0, 0, 0), (1, 1, 1), False),
    ((9, 9, 5), 200, (1, 1, 3), (1, 1, 2), (0, 0, 0), (1, 1, 1), False),
    ((8, 11, 9), 260, (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1), False),
    ((8, 11, 9), 260, (3, 3, 3), (2, 1, 2), (1, 2, 0), (1, 1, 1), False),
    ((10, 12, 11), 300, (3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2), True),
    ((10, 12, 11), 300, (3, 3, 3), (2, 2, 2), (2, 2, 2), (2, 2, 2), False),
    ((6, 8, 8), 150, (1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 1, 1), True),
    ((6, 8, 8), 120, (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1), False),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_rulebook_and_int8_conv_against_dense_conv3d(case):
    """Sparse conv == torch conv3d (float64, exact for int8 data) on the zero-filled dense grid,
    sampled at the active outputs; the active output set == sites with an input in their receptive field."""
    grid, n, ks, st, pad, dil, subm = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    cin, cout = 5, 7
    idx = _random_sparse(rng, grid, n)
    x = rng.integers(-127, 128, (n, cin)).astype(np.int8)
    wq = rng.integers(-127, 128, (int(np.prod(ks)), cout, cin)).astype(np.int8)
    if subm:
        rb = O.rulebook_subm(idx, grid, ks, dil)
        tpad = [(ks[a] // 2) * dil[a] for a in range(3)]
        tst = (1, 1, 1)
    else:
        rb = O.rulebook_sparse(idx, grid, ks, st, pad, dil)
        tpad, tst = pad, st
        assert rb.out_grid == O.conv_out_size(grid, ks, st, pad, dil)
    acc = O.conv_int8_acc(x, wq, rb)
    dense = torch.zeros(1, cin, *grid, dtype=torch.float64)
    dense[0, :, idx[:, 1], idx[:, 2], idx[:, 3]] = torch.from_numpy(x.astype(np.float64)).T
    w = torch.from_numpy(wq.astype(np.float64)).reshape(*ks, cout, cin).permute(3, 4, 0, 1, 2).contiguous()
    y = torch.nn.functional.conv3d(dense, w, stride=tst, padding=tpad, dilation=dil)[0]
    occ = torch.zeros(1, 1, *grid, dtype=torch.float64)
    occ[0, 0, idx[:, 1], idx[:, 2], idx[:, 3]] = 1
    reach = torch.nn.functional.conv3d(occ, torch.ones(1, 1, *ks, dtype=torch.float64), stride=tst, padding=tpad, dilation=dil)[0, 0]
    oi = rb.out_indices
    if subm:
        assert np.array_equal(oi, idx)
    else:
        active = torch.nonzero(reach > 0).numpy()  # row-major = ascending linear index
        assert np.array_equal(oi[:, 1:], active) and np.all(oi[:, 0] == 0)
        assert rb.num_pairs == int(reach.sum().item())
    got = y[:, oi[:, 1], oi[:, 2], oi[:, 3]].T.numpy()
    assert np.array_equal(acc.astype(np.float64), got)
    # float path, same rulebook: agrees with the dense conv to rounding
    xf = rng.standard_normal((n, cin)).astype(np.float16).astype(np.float32)
    wf = (rng.standard_normal(wq.shape) * 0.1).astype(np.float16).astype(np.float32)
    accf = O.conv_f32_acc(xf, wf, rb)
    densef = torch.zeros(1, cin, *grid, dtype=torch.float64)
    densef[0, :, idx[:, 1], idx[:, 2], idx[:, 3]] = torch.from_numpy(xf.astype(np.float64)).T
    w2 = torch.from_numpy(wf.astype(np.float64)).reshape(*ks, cout, cin).permute(3, 4, 0, 1, 2).contiguous()
    yf = torch.nn.functional.conv3d(densef, w2, stride=tst, padding=tpad, dilation=dil)[0]
    gotf = yf[:, oi[:, 1], oi[:, 2], oi[:, 3]].T.numpy()
    assert np.allclose(accf, gotf, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("case", [c for c in CONV_CASES if not c[6]])
def test_inverse_rulebook_against_dense_conv_transpose3d(case):
    """SparseInverseConvolution on a strided rulebook == torch conv_transpose3d (float64, exact for int8
    data) of the zero-filled dense output grid, sampled at the forward convolution's input sites.  A kernel
    flip, a swapped operand or a wrong offset fails this."""
    grid, n, ks, st, pad, dil, _ = case
    rng = np.random.default_rng(hash(case) % (2 ** 31) + 1)
    cin, cout = 6, 4          # of the inverse convolution: cin = channels on the coarse grid
    idx = _random_sparse(rng, grid, n)
    fwd = O.rulebook_sparse(idx, grid, ks, st, pad, dil)
    inv = O.rulebook_inverse(fwd, idx, grid)
    assert inv.n_out == n and np.array_equal(inv.out_indices, idx) and inv.out_grid == list(grid)
    assert inv.num_pairs == fwd.num_pairs and np.array_equal(inv.offsets, fwd.offsets)
    for k in range(len(fwd.offsets) - 1):     # same pairs per offset, roles swapped, ordered by output
        a, b = int(fwd.offsets[k]), int(fwd.offsets[k + 1])
        assert sorted(zip(inv.pair_out[a:b], inv.pair_in[a:b])) == sorted(zip(fwd.pair_in[a:b], fwd.pair_out[a:b]))
        assert np.all(np.diff(inv.pair_out[a:b]) > 0)      # an input row has one output row per offset
    m = fwd.n_out
    x = rng.integers(-127, 128, (m, cin)).astype(np.int8)
    wq = rng.integers(-127, 128, (int(np.prod(ks)), cout, cin)).astype(np.int8)
    acc = O.conv_int8_acc(x, wq, inv)
    og = fwd.out_grid
    oi = fwd.out_indices
    dense = torch.zeros(1, cin, *og, dtype=torch.float64)
    dense[0, :, oi[:, 1], oi[:, 2], oi[:, 3]] = torch.from_numpy(x.astype(np.float64)).T
    w = torch.from_numpy(wq.astype(np.float64)).reshape(*ks, cout, cin).permute(4, 3, 0, 1, 2).contiguous()  # [Cin, Cout, k]
    opad = [grid[a] - ((og[a] - 1) * st[a] - 2 * pad[a] + dil[a] * (ks[a] - 1) + 1) for a in range(3)]
    assert all(0 <= opad[a] < max(st[a], dil[a]) or opad[a] == 0 for a in range(3))
    y = torch.nn.functional.conv_transpose3d(dense, w, stride=st, padding=pad, output_padding=opad, dilation=dil)[0]
    assert list(y.shape[1:]) == list(grid)
    got = y[:, idx[:, 1], idx[:, 2], idx[:, 3]].T.numpy()
    assert np.array_equal(acc.astype(np.float64), got)


def test_sparse_rulebook_truncation_keeps_lowest_outputs():
    rng = np.random.default_rng(5)
    grid = (7, 12, 10)
    idx = _random_sparse(rng, grid, 300)
    full = O.rulebook_sparse(idx, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    cut = O.rulebook_sparse(idx, grid, (3, 3, 3), (2, 2, 2), (1, 1, 1), max_out=50)
    assert cut.n_out == 50 and cut.n_out_total == full.n_out
    assert np.array_equal(cut.out_indices, full.out_indices[:50])
    keep = full.pair_out < 50
    assert cut.num_pairs == int(keep.sum())
    assert np.array_equal(cut.pair_in, full.pair_in[keep]) and np.array_equal(cut.pair_out, full.pair_out[keep])
    empty = O.rulebook_sparse(idx[:0], grid, (3, 3, 3), (2, 2, 2), (1, 1, 1))
    assert empty.n_out == 0 and empty.num_pairs == 0


# ----------------------------------------------------------------------------- epilogue / quantisation
def test_requant_ties_saturation_and_two_roundings():
    # out range 254 -> r = 127/254 = 0.5 exactly: ties rint(0.5)=0, rint(1.5)=2, rint(2.5)=2, rint(-0.5)=-0, rint(-1.5)=-2
    acc = np.array([[1, 3, 5, -1, -3, 254, 255, 400, -400, 0]], np.int32).T.copy()  # y = acc (scale 1, bias 0)
    out = O.epilogue(acc, np.array([1.0], np.float32), np.array([0.0], np.float32), False, True, 254.0)
    assert out[:, 0].tolist() == [0, 2, 2, 0, -2, 127, 127, 127, -127, 0]
    out = O.epilogue(acc, np.array([1.0], np.float32), np.array([0.0], np.float32), True, True, 254.0)
    assert out[:, 0].tolist() == [0, 2, 2, 0, 0, 127, 127, 127, 0, 0]
    # general case against numpy fp32 arithmetic (multiply, add, multiply by 127/amax, each rounded once)
    rng = np.random.default_rng(7)
    acc = rng.integers(-40000, 40000, (5000, 16)).astype(np.int32)
    scale = (rng.uniform(1e-5, 1e-3, 16)).astype(np.float32)
    bias = rng.standard_normal(16).astype(np.float16).astype(np.float32)
    amax = np.float32(4.7117)
    r = np.float32(127.0) / amax
    y = acc.astype(np.float32) * scale
    y = y + bias
    q = np.clip(np.rint(np.maximum(y, 0) * r), -127, 127).astype(np.int8)
    assert np.array_equal(O.epilogue(acc, scale, bias, True, True, float(amax)), q)
    assert np.array_equal(O.epilogue(acc, scale, bias, False, False).view(np.uint16), y.astype(np.float16).view(np.uint16))
    # an FMA would round differently somewhere in this sample: make sure the two-rounding rule is what runs
    y_fma = (acc.astype(np.float64) * scale.astype(np.float64) + bias.astype(np.float64)).astype(np.float32)
    assert np.any(y_fma != y)
    # multiplying by 127/amax is not the same function as dividing by amax/127 near the rounding
    # boundaries; the rule is the former (values built right at the boundaries tell the two apart)
    k = np.arange(0, 127, dtype=np.float32) + np.float32(0.5)
    yb = (k / r).astype(np.float32)
    yb = np.concatenate([yb, np.nextafter(yb, np.float32(np.inf)), np.nextafter(yb, np.float32(-np.inf))])
    want_mul = np.clip(np.rint(yb * r), -127, 127).astype(np.int8)
    want_div = np.clip(np.rint(yb / (amax / np.float32(127.0))), -127, 127).astype(np.int8)
    assert np.any(want_mul != want_div)
    got = O.quantize_f32(yb, float(amax))
    assert np.array_equal(got, want_mul)


def test_quantize_dequantize_add_closed_forms():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal(4000) * 3).astype(np.float16)
    amax = np.float32(6.35)
    r, s = np.float32(127.0) / amax, amax / np.float32(127.0)
    q = O.quantize(x, float(amax))
    assert np.array_equal(q, np.clip(np.rint(x.astype(np.float32) * r), -127, 127).astype(np.int8))
    d = O.dequantize(q, float(amax))
    assert np.array_equal(d.view(np.uint16), (q.astype(np.float32) * s).astype(np.float16).view(np.uint16))
    a = rng.integers(-127, 128, 4000).astype(np.int8)
    b = rng.integers(-127, 128, 4000).astype(np.int8)
    ra, rb, rc = np.float32(3.9), np.float32(3.4), np.float32(5.1)
    v = np.maximum(a.astype(np.float32) * (ra / np.float32(127)) + b.astype(np.float32) * (rb / np.float32(127)), 0)
    assert np.array_equal(O.add(a, float(ra), b, float(rb), True, True, float(rc)),
                          np.clip(np.rint(v * (np.float32(127) / rc)), -127, 127).astype(np.int8))
    # relu after an int8 store == int8 store of the relu'd value (what lets Add+Relu fuse)
    no_relu = O.add(a, float(ra), b, float(rb), False, True, float(rc))
    assert np.array_equal(np.maximum(no_relu, 0), O.add(a, float(ra), b, float(rb), True, True, float(rc)))
    h = O.add(x, 127.0, d, 127.0, False, False)
    assert np.array_equal(h.view(np.uint16), (x.astype(np.float32) + d.astype(np.float32)).astype(np.float16).view(np.uint16))
    # weights: per-output-channel fake quant, multiply form
    w = (rng.standard_normal((4, 3, 3, 3, 8)) * 0.02).astype(np.float16)
    ranges = np.abs(w.astype(np.float32)).reshape(4, -1).max(1)
    wq, s_w = O.quantize_weights(w, ranges)
    ref = np.clip(np.rint(w.astype(np.float32) * (np.float32(127) / ranges)[:, None, None, None, None]), -127, 127)
    assert np.array_equal(wq, ref.reshape(4, 27, 8).transpose(1, 0, 2).astype(np.int8)) and np.abs(wq).max() == 127
    assert np.array_equal(s_w, ranges / np.float32(127))


def test_scatter_dense_matches_numpy_indexing():
    rng = np.random.default_rng(9)
    dims = (2, 9, 7)
    idx = _random_sparse(rng, dims, 40)
    feat = rng.standard_normal((40, 6)).astype(np.float16)
    dense = O.scatter_dense(feat, idx, dims)
    ref = np.zeros((1, 6, *dims), np.float16)
    ref[0, :, idx[:, 1], idx[:, 2], idx[:, 3]] = feat
    assert np.array_equal(dense.view(np.uint16), ref.view(np.uint16))
    # CenterPoint view: [1, C, D, H, W] -> [1, C*D, H, W] puts channel c, depth z at c*D+z
    v = dense.reshape(1, 12, 9, 7)
    r = 5
    assert v[0, 3 * 2 + idx[r, 1], idx[r, 2], idx[r, 3]] == feat[r, 3]
