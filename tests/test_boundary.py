"""CPU-side checks of the boundary: the C-ABI library loads and exports every declared symbol, the
ONNX dialect round-trips, the .tensor format round-trips.  No GPU compute is called."""
import os
import re

import numpy as np
import pytest

from lidar_ai_solution_amd import capi, graphs, onnx_dialect, tensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "scn_c_api.h")).read()
    declared = set(re.findall(r"SCN_API[^;(]*?\b(scn_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 55
    assert declared == set(capi.declared_symbols()), declared ^ set(capi.declared_symbols())
    L = capi.lib()  # raises when the library is missing or lacks a symbol
    for name in declared:
        assert getattr(L, name) is not None
    assert L.scn_version() >= 10000
    assert L.scn_hash_u64(0) == 0
    assert L.scn_hash_capacity_for(79745) == 262144


def test_host_side_argument_checks_need_no_gpu():
    L = capi.lib()
    L.scn_set_log_level(99)
    try:
        assert L.scn_builder_push_output(None, 0) != 0
        b = L.scn_builder_create()
        assert L.scn_builder_push_input(b, b"0") == 0
        assert L.scn_builder_push_relu(b, b"r", 7, b"1") < 0  # unknown tensor handle
        assert b"invalid" in L.scn_last_error()
        L.scn_builder_destroy(b)
        assert not L.scn_engine_create_from_onnx(b"/nonexistent/file.onnx", 1, 0, 10000, None)
        assert b"Parse onnx failed" in L.scn_last_error()
    finally:
        L.scn_set_log_level(1)


@pytest.mark.parametrize("activation", ["Sigmoid", "LeakyReLU"])
def test_model_with_an_unsupported_activation_does_not_load(activation, tmp_path):
    """The exporters can write activations the engine has no epilogue for
    (CUDA-CenterPoint/qat/onnx_export/exptool.py:167-172); the loader's contract for a model it cannot run is a
    null engine (libraries/3DSparseConvolution/src/onnx-parser.cpp:216-219), never an engine that computes
    something else.  The refusal happens while the node is pushed, before anything touches a GPU."""
    L = capi.lib()
    g = graphs.single_subm_layer(seed=3)
    g.nodes[0].attrs["activation"] = activation
    path = str(tmp_path / "act.scn.onnx")
    onnx_dialect.save(g, path)
    L.scn_set_log_level(99)
    try:
        for precision in (capi.PRECISION_FP16, capi.PRECISION_INT8):
            assert not L.scn_engine_create_from_onnx(path.encode(), precision, 0, 10000, None)
            msg = L.scn_last_error()
            assert activation.encode() in msg and b"not supported" in msg
    finally:
        L.scn_set_log_level(1)


def test_log_callback_receives_messages():
    L = capi.lib()
    seen = []
    cb = capi.LOG_CALLBACK(lambda msg, level, file, line, user: seen.append((msg.decode(), level)))
    L.scn_set_log_callback(cb, None)
    old = L.scn_get_log_level()
    try:
        L.scn_set_log_level(0)
        L.scn_log(b"test.py", 1, 1, b"hello")
        L.scn_set_log_level(2)
        L.scn_log(b"test.py", 2, 1, b"filtered")
    finally:
        L.scn_set_log_callback(capi.LOG_CALLBACK(0), None)
        L.scn_set_log_level(old)
    assert seen == [("hello", 1)]


@pytest.mark.parametrize("maker", [graphs.centerpoint_scn, graphs.bevfusion_scn])
def test_onnx_dialect_round_trip(maker, tmp_path):
    g, tags = maker(seed=4)
    amax = {t: 1.0 + 0.01 * i for i, t in enumerate(["0"] + [n.outputs[0] for n in g.nodes])}
    graphs.apply_int8_plan(g, tags, amax, "centerpoint" if maker is graphs.centerpoint_scn else "bevfusion")
    p = str(tmp_path / "m.onnx")
    onnx_dialect.save(g, p)
    h = onnx_dialect.load(p)
    assert h.inputs == g.inputs and h.outputs == g.outputs and h.name == "scn"
    assert [n.op_type for n in h.nodes] == [n.op_type for n in g.nodes]
    for a, b in zip(g.nodes, h.nodes):
        assert a.name == b.name and a.inputs == b.inputs and a.outputs == b.outputs
        for k, v in a.attrs.items():
            w = b.attrs[k]
            if isinstance(v, float) or (isinstance(v, list) and v and isinstance(v[0], float)):
                assert np.allclose(np.float32(v), np.float32(w), rtol=0, atol=0)
            else:
                assert v == w, (a.name, k)
    for k, v in g.initializers.items():
        assert np.array_equal(v.view(np.uint16), h.initializers[k].view(np.uint16))
    convs = [n for n in g.nodes if n.op_type == "SparseConvolution"]
    assert len(convs) == 21 and sum(n.op_type == "Add" for n in g.nodes) == 8


def test_centerpoint_plan_matches_reference_export_plan():
    g, tags = graphs.centerpoint_scn(seed=0)
    amax = {t: 1.0 for t in ["0"] + [n.outputs[0] for n in g.nodes]}
    graphs.apply_int8_plan(g, tags, amax, "centerpoint")
    by_tag = {tags[n.name]: n for n in g.nodes if n.name in tags}
    assert by_tag["conv_input"].attrs["precision"] == "fp16" and by_tag["conv_input"].attrs["output_precision"] == "fp16"
    assert by_tag["conv1.0.quant_add"].attrs["precision"] == "fp16" and by_tag["conv1.0.quant_add"].attrs["output_precision"] == "int8"
    assert by_tag["extra_conv"].attrs["precision"] == "int8" and by_tag["extra_conv"].attrs["output_precision"] == "fp16"
    assert by_tag["conv2.0"].attrs["stride"] == [2, 2, 2] and by_tag["conv4.0"].attrs["padding"] == [0, 1, 1]
    assert by_tag["extra_conv"].attrs["kernel_size"] == [3, 1, 1]
    assert g.nodes[-2].attrs["output_shape"] == [1, 128, 2, 180, 180] and g.nodes[-1].attrs["dims"] == [1, 256, 180, 180]


def test_tensor_file_round_trip(tmp_path, centerpoint_input):
    feats, idx = centerpoint_input
    for arr in (feats[:100], idx[:100], np.arange(24, dtype=np.float32).reshape(2, 3, 4), np.arange(5, dtype=np.int8)):
        p = str(tmp_path / "t.tensor")
        tensor.save(arr, p)
        back = tensor.load(p)
        assert back.dtype == arr.dtype and np.array_equal(back, arr)
    raw = open(p, "rb").read()
    assert np.frombuffer(raw[:12], np.int32).tolist() == [0x33FF1101, 1, 7]
    with pytest.raises(RuntimeError):
        bad = str(tmp_path / "bad.tensor")
        open(bad, "wb").write(b"\x00" * 32)
        tensor.load(bad)
    ref = "/root/reference/libraries/3DSparseConvolution/workspace/centerpoint/in_features.torch.fp16.tensor"
    if os.path.exists(ref):  # the reference's own file parses to the committed fixture
        assert np.array_equal(tensor.load(ref).view(np.uint16), feats.view(np.uint16))


def test_compare_report_numbers_and_row_order_invariance(tmp_path, capsys):
    """The agreement report of the reference's tool/compare.py:71-118: its numbers on a hand-made case, and that
    a sparse tensor compares equal to a row permutation of itself once rows are put into coordinate order."""
    from lidar_ai_solution_amd import compare
    a = np.array([[0.0, 1.0, 2.0, 3.0], [4.0, 5.0, 6.0, 7.0]], np.float16)
    b = a.copy()
    b[0, 1] += 1.0      # differences: 1.0, 0.5, 0.25 and five zeros
    b[1, 0] += 0.5
    b[1, 3] += 0.25
    m = compare.metrics(a, b)
    assert m["absdiff_max"] == 1.0 and m["absdiff_sum"] == 1.75 and m["numel"] == 8
    assert (m["above_75pct_of_max"], m["above_50pct_of_max"], m["above_25pct_of_max"], m["differ"], m["equal"]) == (1, 1, 2, 3, 5)
    x, y = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    assert abs(m["cosine"] - x @ y / np.sqrt((x @ x) * (y @ y))) < 1e-12
    rng = np.random.default_rng(0)
    idx = np.stack([np.zeros(50, np.int32), rng.integers(0, 5, 50), rng.integers(0, 9, 50), np.arange(50)], 1).astype(np.int32)
    feat = rng.standard_normal((50, 8)).astype(np.float16)
    perm = rng.permutation(50)
    for name, f, i in (("p", feat, idx), ("q", feat[perm], idx[perm])):
        tensor.save(f, str(tmp_path / f"{name}.f.tensor"))
        tensor.save(i, str(tmp_path / f"{name}.i.tensor"))
    assert compare.main([str(tmp_path / "p.f.tensor:p.i.tensor"), str(tmp_path / "q.f.tensor:q.i.tensor"),
                         "--dense-grid", "5x9x50", "--detail"]) == 0
    out = capsys.readouterr().out
    assert "[absdiff]: max:0.0" in out and "[absdiff = 0]: 100.000 %, 400" in out and "[cosine]: 100.000 %" in out


def test_build_refuses_spills_in_kernels_with_counted_waits():
    """The build reads the compiler's per-kernel resource remarks and fails when a kernel whose memory waits are
    counted by hand uses scratch memory (a spill is a load those counts do not know about)."""
    from lidar_ai_solution_amd import build as B
    remark = "scn_conv_kernels.hpp:407:1: remark:     {} [-Rpass-analysis=kernel-resource-usage]"
    def report(name, scratch):
        return "\n".join([remark.format("Function Name: " + name), remark.format("VGPRs: 128"),
                          remark.format(f"ScratchSize [bytes/lane]: {scratch}"), remark.format("Occupancy [waves/SIMD]: 4")])
    lds = "_ZN3scn10k_conv_ldsILi0ELi4ELi4ELi8EEEvNS_8ConvArgsE"
    out = "\n".join([report(lds, 0), report("_ZN3scn11k_conv_tileILi1ELi1ELi1EEEvNS_8ConvArgsE", 12),
                     report(lds.replace("Li4ELi4", "Li2ELi4"), 256), "warning: something unrelated"])
    assert B.kernels_with_scratch(out) == [(lds.replace("Li4ELi4", "Li2ELi4"), 256)]
    assert B.kernels_with_scratch(report(lds, 0)) == []
