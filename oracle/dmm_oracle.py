"""CPU oracle for the decode+matmul path.  TEST INFRASTRUCTURE ONLY.

This module is the checker the HIP kernels are compared with.  Nothing in the
product package imports it; only tests, the smoke entry and the benchmark's CPU
baseline leg do.  It restates, in numpy, the algorithm the reference defines in
Python:

  * code format and scalar decode ....... /root/reference/test_decode_matmul.py:29-55
  * branch-free SWAR decode (cross-check)  /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65
  * naive matmul index convention ........ /root/reference/test_decode_matmul.py:58-71
  * E8P "abs" codebook ................... /root/reference/test_decode_matmul.py:74-86
  * MMA-fragment tiling of the codes ..... /root/reference/test_decode_matmul.py:101-109

How each function is pinned (the tests named live in tests/test_oracle.py):

  decode_i8 ........ a literal scalar loop over all 65536 codes, the SWAR form of the
                     CUDA kernel, and the C restatement must all agree with it.
  decode_f16 ....... fp16 result == int8 result / 4 for every code when the grid is
                     codebook bytes / 4 (exact in fp16); IEEE half add for other grids
                     is checked against an exact rational computation.
  matmul_* ......... brute-force loops on tiny shapes, float64 library matmul.
  build_codebook_abs the closed-form set properties (256 distinct rows, norm histogram,
                     byte alphabet, negatives only in dim 7).  PARITY UNPINNED: the row
                     ORDER, because the reference sorts with an unstable argsort over
                     heavily tied keys (test_decode_matmul.py:84); the operator treats
                     the grid as an opaque input so no result depends on that order.
  transpose_tile ... the per-lane index formula the CUDA kernel reads with
                     (decode_matmul_cuda.cu:111-112, 137-138).

The reference holds no golden vectors on disk; its one test draws inputs from the CUDA
RNG.  Parity is therefore anchored on the closed forms above.
"""
from itertools import product

import numpy as np

QUARTER = np.float16(0.25)


# --------------------------------------------------------------------------- fields
def code_fields(codes):
    """Split 16-bit codes into (row index, 8 sign bits, shift bit).

    test_decode_matmul.py:30-33 / decode_matmul_cuda.cu:49-53: bits 0-7 select the grid
    row, bits 8-14 are the sign flips of dims 0-6, the sign of dim 7 is the parity of
    those seven bits, bit 15 selects the -1/4 shift (clear selects +1/4).
    """
    c = np.asarray(codes).astype(np.uint16, copy=False).astype(np.uint32)
    idx = c & 0xFF
    s7 = (c >> 8) & 0x7F
    par = s7 ^ (s7 >> 4)
    par = par ^ (par >> 2)
    par = (par ^ (par >> 1)) & 1
    s8 = s7 | (par << 7)
    shift = (c >> 15) & 1
    return idx, s8, shift


def _sign_bits(s8):
    """[..., 8] array of 0/1: bit d of s8."""
    return (s8[..., None] >> np.arange(8, dtype=np.uint32)) & 1


# --------------------------------------------------------------------------- decode
def decode_f16(codes, grid):
    """codes [N, K/8] (any 16-bit int dtype), grid fp16 [256, 8] -> W fp16 [N, K].

    w = fp16((sign ? -g : g) + (shift ? -0.25 : +0.25)); flip first, then one IEEE half
    add (test_decode_matmul.py:41-47 in fp16 form).  W[n, 8*j + d] comes from
    codes[n, j] (test_decode_matmul.py:65-69).
    """
    codes = np.asarray(codes)
    grid = np.asarray(grid)
    assert grid.dtype == np.float16 and grid.shape == (256, 8)
    idx, s8, shift = code_fields(codes)
    g = grid[idx]                                   # [..., 8] fp16
    neg = _sign_bits(s8).astype(bool)
    v = np.where(neg, -g, g)
    delta = np.where(shift.astype(bool), -QUARTER, QUARTER)[..., None]
    w = (v + delta).astype(np.float16)              # numpy half add: exact sum, one RNE rounding
    return w.reshape(*codes.shape[:-1], codes.shape[-1] * 8)


def codebook_bytes(codebook_abs):
    """int64[256] packed table -> int8 [256, 8]; byte d is dim d (test_decode_matmul.py:38,50)."""
    cb = np.asarray(codebook_abs).astype(np.int64).view(np.uint64)
    b = (cb[:, None] >> (8 * np.arange(8, dtype=np.uint64))) & np.uint64(0xFF)
    return b.astype(np.uint8).view(np.int8)


def decode_i8(codes, codebook_abs):
    """Literal integer decode: int8 [N, K]; value = (+-byte) +- 1 (test_decode_matmul.py:38-47)."""
    codes = np.asarray(codes)
    idx, s8, shift = code_fields(codes)
    b = codebook_bytes(codebook_abs)[idx].astype(np.int32)
    neg = _sign_bits(s8).astype(bool)
    v = np.where(neg, -b, b)
    v = v + np.where(shift.astype(bool), -1, 1)[..., None]
    # the reference keeps int8 arithmetic (value *= -1; value -= 1 on an int8 tensor)
    v = v.astype(np.int8)
    return v.reshape(*codes.shape[:-1], codes.shape[-1] * 8)


def decode_swar_u64(codes, codebook_abs):
    """The CUDA kernel's branch-free decoder, restated on uint64 lanes
    (decode_matmul_cuda.cu:45-65).  Returns uint64 per code, byte d = dim d.
    Only valid for tables whose bytes are all == 2 (mod 4), as the E8P table is."""
    c = np.asarray(codes).astype(np.uint16, copy=False).astype(np.uint64)
    bits_abs = c & np.uint64(0xFF)
    bits_sign = (c >> np.uint64(8)) & np.uint64(0x7F)
    bit_shift = (c >> np.uint64(15)) & np.uint64(1)
    pop = np.zeros_like(bits_sign)
    for i in range(7):
        pop += (bits_sign >> np.uint64(i)) & np.uint64(1)
    s = bits_sign | ((pop & np.uint64(1)) << np.uint64(7))
    s = s | (s << np.uint64(28))
    s = s | (s << np.uint64(14))
    s = s | (s << np.uint64(7))
    s = s & np.uint64(0x0101010101010101)
    s = s * np.uint64(252)
    cb = np.asarray(codebook_abs).astype(np.int64).view(np.uint64)
    packed = cb[bits_abs.astype(np.int64)] ^ s
    packed = packed - bit_shift * np.uint64(0x0202020202020202)
    packed = packed | np.uint64(0x0101010101010101)
    return packed


def grid_from_codebook(codebook_abs):
    """fp16 [256, 8] grid whose entries are the table bytes / 4 (test_decode_matmul.py:85)."""
    return (codebook_bytes(codebook_abs).astype(np.float32) / 4.0).astype(np.float16)


# --------------------------------------------------------------------------- matmul
def matmul_f32(x, W, scale):
    """y_ref[m, n] = scale * sum_k fp32(x[m,k]) * fp32(W[n,k]), as float32.

    Accumulated in float64 and rounded once, so the checker is not itself a source of
    order-dependent error.  The fp16 output the operator returns is compared against this
    within rtol 1e-2 / atol 1e-2."""
    acc = np.asarray(x, dtype=np.float64) @ np.asarray(W, dtype=np.float64).T
    return (acc * np.float64(np.float32(scale))).astype(np.float32)


def decode_matmul_f16(x, codes, grid, scale):
    """The operator, end to end, on the CPU: fp16 y [M, N]."""
    W = decode_f16(codes, grid)
    return matmul_f32(x, W, scale).astype(np.float16)


def decode_matmul_i32(x, codes, codebook_abs):
    """Integer operator of the reference: int8 x [M,K], codes [N,K/8] (un-tiled),
    int64[256] table -> int32 [M,N] (test_decode_matmul.py:58-71).  The per-product
    promotion there is int8*int32 -> int32 and the sum wraps in int32."""
    W = decode_i8(codes, codebook_abs).astype(np.int64)
    acc = np.asarray(x).astype(np.int64) @ W.T
    return acc.astype(np.int32)      # wraps like int32 accumulation (never reached at tested sizes)


# --------------------------------------------------------------------------- codebook
def e8p_abs_rows():
    """The 256 rows of the E8P "abs" codebook as tuples of half-integers, in the
    enumeration order of test_decode_matmul.py:75-82 (before its sort)."""
    rows = []
    for xs in product(*([[0.5, 1.5, 2.5]] * 8)):
        if sum(xs) % 2 != 0:
            xs = (*xs[:-1], -xs[-1])
        z = sum(y * y for y in xs)
        if z <= 10 or (
            z == 12
            and all(abs(y) <= 1.5 for y in xs)
            and (sum(abs(y) == 0.5 for y in xs[0:4]) % 2 == 0)
        ):
            rows.append(xs)
    rows.append((0.5, 0.5, 0.5, 1.5, 1.5, 1.5, 1.5, -1.5))
    return rows


def build_codebook_abs():
    """int64[256]: rows sorted by squared norm, each packed as byte d = (4*v_d) & 255
    (test_decode_matmul.py:84-85).  Ties are broken by enumeration order (a stable sort);
    the reference's argsort leaves tie order unspecified."""
    rows = np.array(e8p_abs_rows(), dtype=np.float64)
    order = np.argsort((rows * rows).sum(1), kind="stable")
    rows = rows[order]
    q = (rows * 4).astype(np.int64) & 255
    packed = (q << (8 * np.arange(8, dtype=np.int64))).sum(1)
    return packed.astype(np.int64)


# --------------------------------------------------------------------------- tiling
def transpose_tile(codes):
    """[N, K'] -> same shape, permuted so that each 16-row x 4-column tile is 64
    contiguous codes ordered [row%8][col%4][row//8] (test_decode_matmul.py:101-109)."""
    codes = np.asarray(codes)
    N, Kc = codes.shape
    t = codes.reshape(N // 16, 16, Kc // 4, 4).transpose(0, 2, 1, 3)
    t = t.reshape(N // 16, Kc // 4, 2, 8, 4).transpose(0, 1, 3, 4, 2)
    return np.ascontiguousarray(t).reshape(N, Kc)


def untranspose_tile(tiled):
    """Inverse of transpose_tile."""
    tiled = np.asarray(tiled)
    N, Kc = tiled.shape
    t = tiled.reshape(N // 16, Kc // 4, 8, 4, 2).transpose(0, 1, 4, 2, 3)
    t = t.reshape(N // 16, Kc // 4, 16, 4).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(t).reshape(N, Kc)
