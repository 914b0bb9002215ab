"""Small helpers for the GPU tests: torch owns the device memory, the C ABI does the work."""
import ctypes as C

import numpy as np
import torch

from lidar_ai_solution_amd import capi

DEV = "cuda:0"


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def to_dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).to(DEV).view(torch.float16)
    return torch.from_numpy(a).to(DEV)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def i3(v):
    return capi.i3(*[int(x) for x in v])


def read_u32(p):
    """Reads one uint32 from a device pointer (synchronises)."""
    out = torch.zeros(1, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    hip = capi.hip_runtime()
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(p), 4, 3) == 0
    return int(out.cpu().numpy().view(np.uint32)[0])


def copy_from_ptr(p, shape, dtype):
    """Copies device memory at raw pointer p into a new torch tensor of the given shape / numpy dtype."""
    tdt = {np.dtype(np.int32): torch.int32, np.dtype(np.int8): torch.int8, np.dtype(np.float16): torch.float16,
           np.dtype(np.float32): torch.float32, np.dtype(np.uint32): torch.int32, np.dtype(np.int64): torch.int64}[np.dtype(dtype)]
    out = torch.empty(shape, dtype=tdt, device=DEV)
    if out.numel() == 0:
        return out
    torch.cuda.synchronize()
    hip = capi.hip_runtime()
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(p), out.numel() * out.element_size(), 3) == 0
    return out


class GpuRulebook:
    def __init__(self, max_in, max_out, kvol):
        self.L = capi.lib()
        self.h = self.L.scn_rulebook_create(max_in, max_out, kvol)
        assert self.h, self.L.scn_last_error()
        self.kvol = kvol

    def __del__(self):
        if getattr(self, "h", None):
            self.L.scn_rulebook_destroy(self.h)
            self.h = None

    def build_subm(self, idx_dev, n, grid, ksize, dil=(1, 1, 1), n_dev=None):
        self._keep = idx_dev
        capi.check(self.L.scn_rulebook_build_subm(self.h, ptr(idx_dev), n, ptr(n_dev), i3(grid), i3(ksize), i3(dil), stream()))
        self.kvol = int(np.prod(ksize))

    def build_sparse(self, idx_dev, n, grid, ksize, stride, pad, dil=(1, 1, 1), n_dev=None):
        self._keep = idx_dev
        capi.check(self.L.scn_rulebook_build_sparse(self.h, ptr(idx_dev), n, ptr(n_dev), i3(grid), i3(ksize), i3(stride),
                                                   i3(pad), i3(dil), stream()))
        self.kvol = int(np.prod(ksize))

    def build_inverse(self, forward, n_in_dev=None):
        self._fwd = forward
        capi.check(self.L.scn_rulebook_build_inverse(self.h, forward.h, ptr(n_in_dev), stream()))
        self.kvol = forward.kvol

    def n_out(self):
        return read_u32(self.L.scn_rulebook_num_out_dev(self.h))

    def n_out_total(self):
        return read_u32(self.L.scn_rulebook_num_out_total_dev(self.h))

    def out_grid(self):
        g = capi.i3()
        self.L.scn_rulebook_out_grid(self.h, g)
        return [int(v) for v in g]

    def out_indices(self):
        n = self.n_out()
        return copy_from_ptr(self.L.scn_rulebook_out_indices(self.h), (n, 4), np.int32).cpu().numpy()

    def pairs(self, capacity):
        pin = torch.full((max(capacity, 1),), -7, dtype=torch.int32, device=DEV)
        pout = torch.full((max(capacity, 1),), -7, dtype=torch.int32, device=DEV)
        offs = torch.zeros(self.kvol + 1, dtype=torch.int64, device=DEV)
        capi.check(self.L.scn_rulebook_pairs(self.h, ptr(pin), ptr(pout), ptr(offs), capacity, stream()))
        torch.cuda.synchronize()
        offs = offs.cpu().numpy()
        total = int(offs[-1])
        return pin[:total].cpu().numpy(), pout[:total].cpu().numpy(), offs


class GpuConv:
    def __init__(self, w_f16, ranges, bias_f16, precision):
        self.L = capi.lib()
        w = np.ascontiguousarray(w_f16, np.float16)
        shape = capi.i5(*w.shape)
        r = None if ranges is None else np.ascontiguousarray(ranges, np.float32)
        b = None if bias_f16 is None else np.ascontiguousarray(bias_f16, np.float16)
        self.h = self.L.scn_conv_create(w.ctypes.data_as(C.c_void_p), shape, None if r is None else r.ctypes.data_as(C.c_void_p),
                                        None if b is None else b.ctypes.data_as(C.c_void_p), precision)
        assert self.h, self.L.scn_last_error()
        self.cout = w.shape[0]
        self.precision = precision

    def __del__(self):
        if getattr(self, "h", None):
            self.L.scn_conv_destroy(self.h)
            self.h = None

    def forward(self, rb, x_dev, n_out, x_range=127.0, relu=False, out_int8=False, out_range=127.0, want_acc=False,
                out_ld=None, **res):
        """out_ld: output row stride in elements (default: channels rounded up to 16, what the kernels need)."""
        io = capi.ConvIO()
        io.x_dev = x_dev.data_ptr()
        io.x_ld = x_dev.shape[1]
        io.x_dynamic_range = x_range
        io.relu = int(relu)
        io.out_dtype = capi.DTYPE_INT8 if out_int8 else capi.DTYPE_FP16
        io.out_dynamic_range = out_range
        ow = out_ld if out_ld is not None else (self.cout + 15) // 16 * 16
        out = torch.zeros((max(n_out, 1), ow), dtype=torch.int8 if out_int8 else torch.float16, device=DEV)
        io.out_dev = out.data_ptr()
        io.out_ld = ow
        acc = None
        if want_acc:
            acc = torch.zeros((max(n_out, 1), self.cout), dtype=torch.int32 if self.precision == 2 else torch.float32, device=DEV)
            io.acc_dev = acc.data_ptr()
        if res:
            r = res["res"]
            io.res_dev = r.data_ptr()
            io.res_dtype = capi.DTYPE_INT8 if r.dtype == torch.int8 else capi.DTYPE_FP16
            io.res_dynamic_range = res.get("res_range", 127.0)
            io.res_ld = r.shape[1]
            io.mid_dtype = capi.DTYPE_INT8 if res.get("mid_int8", False) else capi.DTYPE_FP16
            io.mid_dynamic_range = res.get("mid_range", 127.0)
            io.a_requant_range = res.get("a_rq", 0.0)
            io.b_requant_range = res.get("b_rq", 0.0)
            io.relu_after_add = int(res.get("relu2", False))
        capi.check(self.L.scn_conv_forward(self.h, rb.h, C.byref(io), stream()))
        torch.cuda.synchronize()
        return out[:n_out], (acc[:n_out] if acc is not None else None)
