"""decode_matmul_amd: decode-and-matmul for MI355X (gfx950).

Drop-in for the reference's Python module (`from decode_matmul_cuda import decode_matmul`,
/root/reference/test_decode_matmul.py:5, /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:237-239)
in the half-precision form of the same code format:

    from decode_matmul_amd import decode_matmul
    y = decode_matmul(x, codes, grid, scale)      # x half [M,K], codes int16/uint16 [N,K/8],
                                                  # grid half [256,8] -> y half [M,N]
    W = decode(codes, grid)                       # dense half [N,K], bit-exact decode

The functions are the compiled PyTorch operator (`_C`, host C++) over the C ABI of
`libdmm.so` (hand-written HIP).  GPU tensors run the HIP kernels; `decode_matmul` and `decode` also
take tensors in host memory, which go to the library's own host route (plain C++ loops, the
counterpart of the reference's CPU path, test_decode_matmul.py:29-71).  Nothing falls back: without
the built extension every operator raises ImportError (the import itself succeeds, so that
`python -m decode_matmul_amd.build` can run on a fresh tree).
"""
import os as _os

_PKG_DIR = _os.path.dirname(_os.path.abspath(__file__))
LIB_PATH = _os.path.join(_PKG_DIR, "libdmm.so")
EXT_PATH = _os.path.join(_PKG_DIR, "_C.so")

import torch as _torch  # noqa: E402  (loads the HIP runtime the extension links against)

_C = None


def _ext():
    """The compiled operator module; loaded on first use, ImportError if it is not built."""
    global _C
    if _C is None:
        if not (_os.path.exists(LIB_PATH) and _os.path.exists(EXT_PATH)):
            raise ImportError(
                "decode_matmul_amd: native libraries are not built (%s, %s); run "
                "`python -m decode_matmul_amd.build`" % (LIB_PATH, EXT_PATH)
            )
        import importlib
        _C = importlib.import_module("._C", __name__)
    return _C


if _os.path.exists(LIB_PATH) and _os.path.exists(EXT_PATH):
    _ext()

from .capi import lib  # noqa: E402,F401
from .codebook import (  # noqa: E402,F401
    build_codebook_abs,
    grid_from_codebook,
    transpose_tile,
    untranspose_tile,
)

__all__ = [
    "decode_matmul",
    "decode_matmul_path",
    "decode_matmul_int8",
    "pack_codes",
    "decode_matmul_packed",
    "decode",
    "lib",
    "build_codebook_abs",
    "grid_from_codebook",
    "transpose_tile",
    "untranspose_tile",
]


def decode_matmul(x, codes, table, scale=None):
    """The operator under the reference's name, dispatching on the dtype of x.

    Half x: `decode_matmul(x, codes, grid, scale)` -> half y[M,N] = half(scale * x @
    decode(codes, grid).T), fp32 accumulation; codes row-major [N, K/8], grid half [256,8].
    int8 x: the reference's own call `decode_matmul(x, weights_compressed, codebook_abs)`
    (decode_matmul_cuda.cu:178-181, test_decode_matmul.py:136) -> int32 [M,N], exact; codes in the
    reference's tile order (`transpose_tile`), table int64[256]; no scale.

    Runs on x's device and the current stream, asynchronously; raises RuntimeError on bad
    inputs like the reference's TORCH_CHECKs (decode_matmul_cuda.cu:182-207)."""
    if x.dtype == _torch.int8:
        if scale is not None:
            raise TypeError("decode_matmul: the integer form (int8 x) takes no scale")
        return _ext().decode_matmul_int8(x, codes, table, True)
    if scale is None:
        raise TypeError("decode_matmul: the half-precision form needs a scale")
    return _ext().decode_matmul(x, codes, table, float(scale))


def decode_matmul_path(x, codes, grid, scale, path="auto"):
    """decode_matmul through one named kernel path: "auto", "gemv", "gemm" or "generic".
    A path asked for outside its domain raises instead of falling back."""
    return _ext().decode_matmul_path(x, codes, grid, float(scale), path)


def decode_matmul_int8(x, weights_compressed, codebook_abs, tiled=True):
    """The reference's operator with its own dtypes: int8 x [M,K], int16 codes [N,K/8], int64[256]
    table -> int32 [M,N] (decode_matmul_cuda.cu:178-234).  tiled=True: codes as the reference's
    kernel reads them (`transpose_tile`, test_decode_matmul.py:101-109); False: row-major."""
    return _ext().decode_matmul_int8(x, weights_compressed, codebook_abs, bool(tiled))


def pack_codes(codes):
    """Offline repack of codes [N, K/8] (K % 256 == 0) for the batch-1 kernel: each wave's load
    becomes 1 KB of consecutive bytes.  The counterpart of the reference's `transpose_tile`
    (test_decode_matmul.py:101-109).  Returns [ceil(N/16)*16, K/8], same dtype."""
    return _ext().pack_codes(codes)


def decode_matmul_packed(x, packed, grid, scale, N):
    """`decode_matmul` on codes packed by `pack_codes`; N = rows of the original code matrix.
    Any M; bit-identical to `decode_matmul` on the row-major codes."""
    return _ext().decode_matmul_packed(x, packed, grid, float(scale), int(N))


def decode(codes, grid):
    """Dense half matrix W[N,K] from codes[N,K/8]; W[n, 8j+d] is dim d of codes[n, j]."""
    return _ext().decode(codes, grid)
