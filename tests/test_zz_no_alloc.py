"""The allocation-free sparse -> dense entry point (scn_scatter_dense_noalloc: row map in a static device
array) against the workspace variant (scn_scatter_dense_with_map) and the CPU oracle, bit for bit, on calls
in a row that share the array: a large input first, then smaller ones whose rows must not see what the
earlier call left in the map.  Needs a MI355X."""
import numpy as np
import pytest
import torch

from lidar_ai_solution_amd import capi
from oracle import scn_oracle as O

pytestmark = pytest.mark.gpu

from tests.gpu_helpers import DEV, i3, ptr, stream, to_dev  # noqa: E402


def _case(seed, n, c, dims, dtype):
    rng = np.random.default_rng(seed)
    vol = int(np.prod(dims))
    lin = np.sort(rng.choice(vol, size=n, replace=False))
    idx = np.zeros((n, 4), np.int32)
    idx[:, 1] = lin // (dims[1] * dims[2])
    idx[:, 2] = (lin // dims[2]) % dims[1]
    idx[:, 3] = lin % dims[2]
    if dtype == capi.DTYPE_FP16:
        feat = rng.standard_normal((n, c)).astype(np.float16)
        rows, amax = feat, 0.0
    else:
        feat = rng.integers(-127, 128, (n, c)).astype(np.int8)
        amax = 6.35
        rows = O.dequantize(feat, amax)
    return feat, rows, idx, amax


def _both(L, feat, idx, amax, dtype, c, n, n_dev, shape5, perm5, cell_map):
    """(output of the allocation-free call, output of the workspace call)."""
    oshape = [shape5[p] for p in perm5] if perm5 else list(shape5)
    d_feat, d_idx = to_dev(feat), to_dev(idx)
    shape = capi.i5(*shape5)
    pm = capi.i5(*perm5) if perm5 else None
    outs = []
    for which in ("noalloc", "with_map"):
        out = torch.full(oshape, 5, dtype=torch.float16, device=DEV)
        if which == "noalloc":
            capi.check(L.scn_scatter_dense_noalloc(ptr(d_feat), dtype, amax, c, feat.shape[1], ptr(d_idx), n, ptr(n_dev),
                                                   shape, pm, ptr(out), stream()))
        else:
            capi.check(L.scn_scatter_dense_with_map(ptr(d_feat), dtype, amax, c, feat.shape[1], ptr(d_idx), n, ptr(n_dev),
                                                    shape, pm, ptr(out), ptr(cell_map), stream()))
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    return outs


def test_noalloc_scatter_matches_workspace_variant_on_consecutive_calls():
    L = capi.lib()
    assert L.scn_scatter_dense_noalloc_max_cells() == 1 << 18
    print("[case] allocation-free sparse->dense: 128 x 2x180x180 int8 rows, then smaller inputs on the same static map",
          flush=True)
    cell_map = torch.empty(1 << 18, dtype=torch.int32, device=DEV)
    # (rows, channels, [D0, D1, D2], permutation after the scatter, element type): the first call is the largest;
    # the following ones are smaller in rows and in cells, so stale entries of the earlier maps lie both inside
    # and beyond the part of the array the later calls use
    calls = [
        (9000, 128, (2, 180, 180), None, capi.DTYPE_INT8),
        (2500, 128, (2, 180, 180), None, capi.DTYPE_INT8),
        (700, 64, (2, 96, 100), (0, 1, 2, 4, 3), capi.DTYPE_FP16),
        (0, 16, (1, 8, 8), None, capi.DTYPE_FP16),
        (40, 16, (1, 8, 8), None, capi.DTYPE_FP16),
    ]
    for k, (n, c, dims, perm, dtype) in enumerate(calls):
        print(f"[case] call {k}: n={n} c={c} dims={dims} perm={perm} dtype={dtype}", flush=True)
        feat, rows, idx, amax = _case(100 + k, n, c, dims, dtype)
        shape5 = (1, c, *dims)
        got, want = _both(L, feat, idx, amax, dtype, c, n, None, shape5, perm, cell_map)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), f"call {k}"
        ref = O.scatter_dense(rows, idx, dims) if n else np.zeros(shape5, np.float16)
        if perm:
            ref = np.ascontiguousarray(ref.transpose(perm))
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), f"call {k} against the oracle"
    print("[case] device-side row count smaller than the bound", flush=True)
    feat, rows, idx, amax = _case(7, 3000, 128, (2, 180, 180), capi.DTYPE_INT8)
    cnt = to_dev(np.array([1111], np.uint32))
    got, want = _both(L, feat, idx, amax, capi.DTYPE_INT8, 128, 3000, cnt, (1, 128, 2, 180, 180), None, cell_map)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    ref = O.scatter_dense(rows[:1111], idx[:1111], (2, 180, 180))
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_noalloc_scatter_rejects_what_it_cannot_hold():
    L = capi.lib()
    out = torch.zeros(8, dtype=torch.float16, device=DEV)
    feat = torch.zeros((1, 16), dtype=torch.float16, device=DEV)
    idx = torch.zeros((1, 4), dtype=torch.int32, device=DEV)
    print("[case] allocation-free sparse->dense: layouts beyond the static map are refused before any launch", flush=True)
    # more cells per channel plane than the static map holds
    rc = L.scn_scatter_dense_noalloc(ptr(feat), capi.DTYPE_FP16, 0.0, 16, 16, ptr(idx), 1, None,
                                     capi.i5(1, 16, 4, 360, 360), None, ptr(out), stream())
    assert rc == 3 and b"exceed" in L.scn_last_error()
    # channel-last layout: takes no row map
    rc = L.scn_scatter_dense_noalloc(ptr(feat), capi.DTYPE_FP16, 0.0, 16, 16, ptr(idx), 1, None,
                                     capi.i5(1, 16, 2, 8, 8), capi.i5(0, 2, 3, 4, 1), ptr(out), stream())
    assert rc == 4
    torch.cuda.synchronize()
