"""Exporter-side transformations (BatchNorm folding, xyz <-> zyx inversion) against closed forms and the
oracle.  CPU only."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from lidar_ai_solution_amd import export, graphs, onnx_dialect
from oracle import scn_oracle as O


def test_fuse_bn_matches_conv_followed_by_batchnorm():
    # closed form: dense conv3d then eval-mode batch norm == conv3d with the folded weights
    rng = np.random.default_rng(5)
    cin, cout = 3, 4
    w = rng.standard_normal((cout, 3, 3, 3, cin)).astype(np.float32)      # [Cout, K0, K1, K2, Cin]
    b = rng.standard_normal(cout).astype(np.float32)
    mean = rng.standard_normal(cout).astype(np.float32)
    var = rng.uniform(0.3, 2.0, cout).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, cout).astype(np.float32)
    beta = rng.standard_normal(cout).astype(np.float32)
    eps = 1e-3
    x = torch.from_numpy(rng.standard_normal((1, cin, 5, 6, 7)).astype(np.float32)).double()

    def conv(wk, bk):
        wt = torch.from_numpy(np.ascontiguousarray(wk.transpose(0, 4, 1, 2, 3))).double()
        return F.conv3d(x, wt, None if bk is None else torch.from_numpy(bk).double(), padding=1)

    for bias, g_, b_ in ((b, gamma, beta), (None, None, None), (b, None, beta)):
        want = F.batch_norm(conv(w, bias), torch.from_numpy(mean).double(), torch.from_numpy(var).double(),
                            None if g_ is None else torch.from_numpy(g_).double(),
                            None if b_ is None else torch.from_numpy(b_).double(), False, 0.0, eps)
        wf, bf = export.fuse_bn_weights(w, bias, mean, var, eps, g_, b_)
        assert wf.shape == w.shape and wf.dtype == np.float32 and bf.shape == (cout,)
        got = conv(wf, bf)
        assert float((got - want).abs().max()) < 2e-5


def _random_frame(grid, n, channels, seed):
    rng = np.random.default_rng(seed)
    cells = rng.choice(int(np.prod(grid)), n, replace=False)
    idx = np.zeros((n, 4), np.int32)
    idx[:, 1], rem = np.divmod(cells, grid[1] * grid[2])
    idx[:, 2], idx[:, 3] = np.divmod(rem, grid[2])
    feats = rng.standard_normal((n, channels)).astype(np.float16)
    return feats, idx


def _all_int8(maker, grid_kw, grid, feats, idx, seed):
    g16, _ = maker(seed=seed, channels=(16, 16, 32, 32), weight_std=0.08, **{grid_kw: grid})
    rec = {}
    O.run_graph(g16, feats, idx, list(grid), "fp16", rec)
    amax = {g16.inputs[0]: graphs.percentile_amax(np.abs(feats.astype(np.float32)))}
    for n in g16.nodes:
        if n.op_type in ("SparseConvolution", "Add", "Relu"):
            amax[n.outputs[0]] = graphs.percentile_amax(np.abs(rec[n.name]["out"].astype(np.float32)))
    g8, tags8 = maker(seed=seed, channels=(16, 16, 32, 32), weight_std=0.08, **{grid_kw: grid})
    graphs.apply_int8_plan(g8, tags8, amax, "all-int8")
    return g8


def test_inverted_bevfusion_graph_gives_the_same_dense_output(tmp_path):
    # integer arithmetic end to end ("all-int8"), so reversing the axis order must not change one bit
    grid = (48, 40, 41)
    feats, idx = _random_frame(grid, 4000, 5, seed=11)
    g = _all_int8(graphs.bevfusion_scn, "grid_xyz", grid, feats, idx, seed=2)
    want = O.run_graph(g, feats, idx, list(grid), "int8")[g.outputs[0]]
    gi = export.invert_graph(g)
    # what the reference's inverted forward hook does to the tail
    assert [n.attrs["dims"] for n in gi.nodes if n.op_type == "Transpose"] == [[0, 1, 2, 4, 3]]
    sd = [n for n in gi.nodes if n.op_type == "ScatterDense"][0]
    sd0 = [n for n in g.nodes if n.op_type == "ScatterDense"][0]
    assert sd.attrs["format"] == "zyx" and sd.attrs["output_shape"][2:] == sd0.attrs["output_shape"][2:][::-1]
    conv_out = [n for n in gi.nodes if n.op_type == "SparseConvolution"][-1]
    assert conv_out.attrs["kernel_size"] == [3, 1, 1] and conv_out.attrs["stride"] == [2, 1, 1]
    got = O.run_graph(gi, feats, export.invert_indices(idx), list(grid)[::-1], "int8")[gi.outputs[0]]
    assert got.shape == want.shape and np.abs(want.astype(np.float32)).max() > 0
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # the inverted graph survives the file format, and inverting twice is the identity
    p = str(tmp_path / "inv.onnx")
    onnx_dialect.save(gi, p)
    assert [n.attrs.get("kernel_size") for n in onnx_dialect.load(p).nodes] == [n.attrs.get("kernel_size") for n in gi.nodes]
    gb = export.invert_graph(gi)
    for k, v in g.initializers.items():
        assert np.array_equal(v, gb.initializers[k])
    assert [n.attrs for n in gb.nodes] == [n.attrs for n in g.nodes]


def test_inverting_a_graph_whose_tail_reshapes_the_dense_tensor():
    grid = (41, 40, 48)
    feats, idx = _random_frame(grid, 4000, 5, seed=12)
    g = _all_int8(graphs.centerpoint_scn, "grid_zyx", grid, feats, idx, seed=3)
    want = O.run_graph(g, feats, idx, list(grid), "int8")[g.outputs[0]]
    with pytest.raises(ValueError):
        export.invert_graph(g)
    gi = export.invert_graph(export.insert_identity_transpose(g))
    assert [n.attrs["dims"] for n in gi.nodes if n.op_type == "Transpose"] == [[0, 1, 4, 3, 2]]
    got = O.run_graph(gi, feats, export.invert_indices(idx), list(grid)[::-1], "int8")[gi.outputs[0]]
    assert np.abs(want.astype(np.float32)).max() > 0
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
