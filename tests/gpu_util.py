"""Helpers for the GPU tests: call the C ABI of libdmm.so with raw device pointers taken
from torch tensors (torch is only the allocator and the stream here)."""
import numpy as np
import torch

from decode_matmul_amd import capi

DEV = "cuda:0"


def _p(t):
    return t.data_ptr() if t is not None and t.numel() > 0 else (t.data_ptr() if t is not None else None)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def c_decode(codes, grid, out=None):
    """dmm_decode_f16 on device tensors; returns W half [N, K]."""
    N, kc = codes.shape
    W = out if out is not None else torch.empty(N, kc * 8, dtype=torch.float16, device=codes.device)
    st = capi.lib().dmm_decode_f16(codes.data_ptr(), grid.data_ptr(), W.data_ptr(), N, kc * 8, _stream())
    capi.check("dmm_decode_f16", st)
    return W


_ENTRY = {
    "auto": "dmm_decode_matmul_f16",
    "gemv": "dmm_gemv_f16",
    "gemv8": "dmm_gemv_8bit_f16",
    "gemm": "dmm_gemm_f16",
    "generic": "dmm_generic_f16",
}


def c_matmul(x, codes, grid, scale, path="auto", out=None):
    """One operator entry point of the C ABI on device tensors; returns y half [M, N]."""
    M, K = x.shape
    N = codes.shape[0]
    assert codes.shape[1] * 8 == K
    y = out if out is not None else torch.full((M, N), float("nan"), dtype=torch.float16, device=x.device)
    fn = getattr(capi.lib(), _ENTRY[path])
    st = fn(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), float(scale), y.data_ptr(), M, N, K, _stream())
    capi.check(_ENTRY[path], st)
    return y


def bits(t):
    """uint16 bit patterns of a half tensor / array, as numpy."""
    if isinstance(t, torch.Tensor):
        return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    return np.ascontiguousarray(t).view(np.uint16)


def assert_close_to_oracle(y, ref32, what=""):
    """The operator's tolerance: |y - ref| <= 1e-2 + 1e-2 * |ref| against the fp32-accumulated
    reference (rtol 1e-2, atol 1e-2)."""
    got = y.detach().float().cpu().numpy() if isinstance(y, torch.Tensor) else np.asarray(y, dtype=np.float32)
    ref32 = np.asarray(ref32, dtype=np.float32)
    assert got.shape == ref32.shape, (got.shape, ref32.shape)
    err = np.abs(got - ref32)
    tol = 1e-2 + 1e-2 * np.abs(ref32)
    bad = ~(err <= tol)
    assert not bad.any(), "%s: %d of %d outside tolerance, worst err %.4g at %s" % (
        what, int(bad.sum()), bad.size, float(np.nanmax(err)), np.unravel_index(np.nanargmax(err), err.shape))
