"""Agreement report between two `.tensor` files (or in-memory arrays).

The counterpart of the reference's `libraries/3DSparseConvolution/tool/compare.py:71-118`: absolute-difference
statistics, how many elements lie above 75 / 50 / 25 % of the largest difference, how many differ at all, and
the cosine between the two tensors.  A sparse tensor is named `features.tensor:indices.tensor` together with
`--dense-grid Z x Y x X`: its rows are then brought into ascending coordinate order first, because the row
order of a sparse tensor is not part of its value (`compare.py:47-69`).

    python -m lidar_ai_solution_amd.compare a.tensor b.tensor --detail
    python -m lidar_ai_solution_amd.compare a.f.tensor:a.i.tensor b.f.tensor:b.i.tensor --dense-grid 41x1440x1440
"""
from __future__ import annotations

import argparse
import os
from typing import Dict, Optional, Sequence

import numpy as np

from . import tensor


def rows_in_coordinate_order(features: np.ndarray, indices: np.ndarray, grid: Sequence[int]) -> np.ndarray:
    """Features re-ordered by ascending (batch, i0, i1, i2) of their index rows."""
    idx = np.asarray(indices, np.int64)
    g0, g1, g2 = (int(v) for v in grid)
    key = ((idx[:, 0] * g0 + idx[:, 1]) * g1 + idx[:, 2]) * g2 + idx[:, 3]
    return np.ascontiguousarray(np.asarray(features)[np.argsort(key, kind="stable")])


def _load(spec: str, grid: Optional[Sequence[int]]) -> np.ndarray:
    if grid is None:
        return tensor.load(spec)
    directory, names = os.path.split(spec)
    parts = names.split(":")
    if len(parts) != 2:
        raise RuntimeError("a sparse tensor is named features.tensor:indices.tensor")
    return rows_in_coordinate_order(tensor.load(os.path.join(directory, parts[0])),
                                    tensor.load(os.path.join(directory, parts[1])), grid)


def metrics(a: np.ndarray, b: np.ndarray) -> Dict[str, float]:
    """The numbers of the report for two arrays with the same element count."""
    if a.size != b.size:
        raise RuntimeError(f"Invalid compare with mismatched shape, {a.shape} <-----> {b.shape}")
    x = np.asarray(a, np.float32).reshape(-1)
    y = np.asarray(b, np.float32).reshape(-1)
    d = np.abs(x - y)
    top = float(d.max()) if d.size else 0.0
    out = {"absdiff_max": top, "absdiff_sum": float(d.sum(dtype=np.float64)), "absdiff_std": float(d.std()) if d.size else 0.0,
           "absdiff_mean": float(d.mean()) if d.size else 0.0, "numel": int(d.size)}
    for pct in (75, 50, 25):
        out[f"above_{pct}pct_of_max"] = int(np.count_nonzero(d > top * pct / 100.0))
    out["differ"] = int(np.count_nonzero(d > 0))
    out["equal"] = int(d.size - out["differ"])
    nx, ny = float(np.linalg.norm(x.astype(np.float64))), float(np.linalg.norm(y.astype(np.float64)))
    out["cosine"] = float(np.dot(x.astype(np.float64), y.astype(np.float64)) / (nx * ny)) if nx > 0 and ny > 0 else float(nx == ny)
    return out


def report(a: np.ndarray, b: np.ndarray, detail: bool = False, names=("A", "B")) -> str:
    m = metrics(a, b)
    lines = [f"[absdiff]: max:{m['absdiff_max']}, sum:{m['absdiff_sum']:.6f}, std:{m['absdiff_std']:.6f}, mean:{m['absdiff_mean']:.6f}"]
    if detail:
        for name, t in zip(names, (a, b)):
            v = np.asarray(t, np.float32).reshape(-1)
            lines.append(f"{name}: shape {' x '.join(map(str, t.shape))}, {t.dtype}, absmax:{np.abs(v).max():.6f}, "
                         f"min:{v.min():.6f}, std:{v.std():.6f}, mean:{v.mean():.6f}")
        n = max(m["numel"], 1)
        for pct in (75, 50, 25):
            k = m[f"above_{pct}pct_of_max"]
            lines.append(f"[absdiff > m{pct}% --- {m['absdiff_max'] * pct / 100.0:.6f}]: {k / n * 100:.3f} %, {k}")
        lines.append(f"[absdiff > 0]: {m['differ'] / n * 100:.3f} %, {m['differ']}")
        lines.append(f"[absdiff = 0]: {m['equal'] / n * 100:.3f} %, {m['equal']}")
        lines.append(f"[cosine]: {m['cosine'] * 100:.3f} %")
    return "\n".join(lines)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Compare two tensors written in the .tensor format")
    ap.add_argument("a", help="tensor file, or features.tensor:indices.tensor with --dense-grid")
    ap.add_argument("b", help="tensor file, or features.tensor:indices.tensor with --dense-grid")
    ap.add_argument("--detail", action="store_true")
    ap.add_argument("--dense-grid", type=str, help="grid of a sparse tensor, like 41x1440x1440")
    args = ap.parse_args(argv)
    grid = [int(v) for v in args.dense_grid.lower().split("x")] if args.dense_grid else None
    print(report(_load(args.a, grid), _load(args.b, grid), args.detail, (args.a, args.b)))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
