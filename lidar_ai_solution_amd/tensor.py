"""`.tensor` file format of the reference tooling.

Layout (`libraries/3DSparseConvolution/tool/tensor.py:24-69`): int32 header
`{0x33ff1101, ndim, dtype_code}`, `ndim` int32 dims, then the raw little-endian data.
dtype codes follow `spconv::DataType` (`libspconv/include/spconv/tensor.hpp:28-38`).
"""
from __future__ import annotations

import numpy as np

MAGIC = 0x33FF1101

_CODE_OF = {"int32": 1, "float16": 2, "float32": 3, "int64": 4, "uint64": 5, "uint32": 6, "int8": 7, "uint8": 8}
_DTYPE_OF = {v: np.dtype(k) for k, v in _CODE_OF.items()}


def save(tensor, file: str) -> None:
    if not isinstance(tensor, np.ndarray):
        if hasattr(tensor, "detach"):
            tensor = tensor.detach().cpu().numpy()
        else:
            tensor = np.array(tensor)
    key = str(tensor.dtype)
    if key not in _CODE_OF:
        raise RuntimeError(f"Unsupport dtype {tensor.dtype}")
    with open(file, "wb") as f:
        f.write(np.array([MAGIC, tensor.ndim, _CODE_OF[key]], dtype=np.int32).tobytes())
        f.write(np.array(tensor.shape, dtype=np.int32).tobytes())
        f.write(np.ascontiguousarray(tensor).tobytes())


def load(file: str, return_torch: bool = False):
    with open(file, "rb") as f:
        head = np.frombuffer(f.read(12), dtype=np.int32)
        if head.size != 3 or int(head[0]) != MAGIC:
            raise RuntimeError("this file is not tensor file")
        ndim, code = int(head[1]), int(head[2])
        if code not in _DTYPE_OF:
            raise RuntimeError(f"Can not find match dtype for index {code}")
        dims = np.frombuffer(f.read(ndim * 4), dtype=np.int32)
        dtype = _DTYPE_OF[code]
        count = int(np.prod(dims, dtype=np.int64)) if ndim else 1
        data = np.frombuffer(f.read(count * dtype.itemsize), dtype=dtype)
        if data.size != count:
            raise RuntimeError("truncated tensor file")
        data = data.reshape(*dims)
    if return_torch:
        import torch
        return torch.from_numpy(data.copy())
    return data
