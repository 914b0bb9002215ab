"""Host-side hardening of the model loader: the engine's host code (ONNX wire reader, loader, builder checks, graph
planning) is compiled with g++ -fsanitize=address,undefined together with host-only stand-ins for the kernel side
(tests/native/kernel_side_stubs.cpp) and fed every kind of broken model: prefixes of a valid one, flipped bits, replaced
bytes, endless varints, removed and repeated stretches.  Every case must end in a null engine with an error text (or in an
engine), never in a sanitizer report.  Reference for the contract: a model that cannot be loaded gives nullptr
(libraries/3DSparseConvolution/src/onnx-parser.cpp:107-110,216-219).  Runs without a GPU."""
import os
import subprocess

import pytest

from lidar_ai_solution_amd import graphs, onnx_dialect

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "lidar_ai_solution_amd", "csrc")
NATIVE = os.path.join(ROOT, "tests", "native")
FLAGS = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer",
         "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include")]


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    out = tmp_path_factory.mktemp("loader_fuzz")
    sources = [os.path.join(CSRC, "scn_engine.cpp"), os.path.join(CSRC, "scn_common.cpp"),
               os.path.join(NATIVE, "kernel_side_stubs.cpp"), os.path.join(NATIVE, "loader_fuzz.cpp")]
    procs = []
    for src in sources:
        obj = str(out / (os.path.basename(src) + ".o"))
        procs.append((obj, subprocess.Popen(["g++", *FLAGS, "-c", src, "-o", obj], stdout=subprocess.PIPE,
                                            stderr=subprocess.STDOUT, text=True)))
    for obj, p in procs:
        log, _ = p.communicate()
        assert p.returncode == 0, log
    exe = str(out / "loader_fuzz")
    r = subprocess.run(["g++", "-fsanitize=address,undefined", *[o for o, _ in procs], "-L/opt/rocm/lib", "-lamdhip64",
                        "-Wl,-rpath,/opt/rocm/lib", "-o", exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return exe


def _graph_end(model: bytes) -> int:
    """Offset of the first byte behind the ModelProto's graph field (number 7, length-delimited)."""
    def varint(p):
        v = shift = 0
        while True:
            b = model[p]
            p += 1
            v |= (b & 0x7F) << shift
            shift += 7
            if not b & 0x80:
                return v, p
    p = 0
    while p < len(model):
        key, p = varint(p)
        wt = key & 7
        if wt == 0:
            _, p = varint(p)
        elif wt == 2:
            n, p = varint(p)
            p += n
            if key >> 3 == 7:
                return p
        elif wt == 5:
            p += 4
        elif wt == 1:
            p += 8
        else:
            raise AssertionError(wt)
    raise AssertionError("no graph field")


@pytest.mark.parametrize("kind,precision", [("centerpoint", "int8"), ("unet", "fp16")])
def test_loader_survives_truncated_and_damaged_models(kind, precision, harness, tmp_path):
    if kind == "centerpoint":
        g, tags = graphs.centerpoint_scn(seed=1, channels=(8, 8, 16, 16), grid_zyx=(41, 64, 64))
        amax = {t: 1.0 + 0.1 * i for i, t in enumerate([g.inputs[0]] + [n.outputs[0] for n in g.nodes])}
        graphs.apply_int8_plan(g, tags, amax, "centerpoint")
        dense = [n for n in g.nodes if n.op_type == "ScatterDense"][0]
        dense.attrs["output_layout"] = "NCHW32"
        dense.attrs["input_dynamic_range"] = 3.0
    else:
        g, _ = graphs.unet_scn(seed=2, channels=(8, 8, 16))
    path = str(tmp_path / "model.onnx")
    onnx_dialect.save(g, path)
    with open(path, "rb") as f:
        model = f.read()
    end = _graph_end(model)
    assert 0 < end <= len(model)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([harness, path, precision, "12000", "7", str(end)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, env=env, timeout=600)
    print(r.stdout[-3000:])
    assert r.returncode == 0, r.stdout[-3000:]
    assert "runtime error" not in r.stdout and "AddressSanitizer" not in r.stdout and "LeakSanitizer" not in r.stdout
    line = [l for l in r.stdout.splitlines() if l.startswith("loader fuzz:")][-1]
    # the undamaged model passes every host-side check (it then builds, or stops at the first device allocation where
    # there is no GPU), and a good part of the damaged copies is refused by the reader or the builder's checks
    refused = int(line.split("damaged copies:")[1].split("refused")[0])
    assert 1000 < refused < 12000, line
