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
