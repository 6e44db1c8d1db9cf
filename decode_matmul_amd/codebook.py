"""Host-side helpers of the code format: the E8P "abs" codebook and the code tiling the
reference's CUDA kernel reads.  Pure torch, CPU or GPU tensors alike.

  build_codebook_abs ... /root/reference/test_decode_matmul.py:74-86
  transpose_tile ....... /root/reference/test_decode_matmul.py:101-109
"""
from itertools import product

import torch


def _abs_rows():
    """256 rows of half-integers: all of {0.5,1.5,2.5}^8 with the last coordinate negated
    when the coordinate sum is odd, kept when the squared norm is <= 10 or it is 12 with
    every |coordinate| <= 1.5 and an even number of 0.5s among the first four; plus one
    extra row (test_decode_matmul.py:75-82)."""
    rows = []
    for xs in product((0.5, 1.5, 2.5), repeat=8):
        if sum(xs) % 2 != 0:
            xs = xs[:-1] + (-xs[-1],)
        norm2 = sum(v * v for v in xs)
        if norm2 <= 10 or (
            norm2 == 12
            and all(abs(v) <= 1.5 for v in xs)
            and sum(abs(v) == 0.5 for v in xs[:4]) % 2 == 0
        ):
            rows.append(xs)
    rows.append((0.5, 0.5, 0.5, 1.5, 1.5, 1.5, 1.5, -1.5))
    return rows


def build_codebook_abs(device="cpu"):
    """int64[256]; entry i packs byte d = (4 * row_i[d]) & 255.  Rows are ordered by squared
    norm with ties kept in enumeration order (stable).

    The SET of rows is the reference's; the ORDER is not: the reference sorts with an unstable
    argsort over keys that tie up to 126-fold (test_decode_matmul.py:84), and what that returns
    depends on the torch build (under torch 2.10 on CPU 251 of the 256 rows sit at other indices than
    here; tests/golden/reference_codebook_order.json holds that table).  Codes quantised against
    another table must be decoded with THAT table: pass it to the operator, which takes the table
    as an input and assumes no order."""
    rows = torch.tensor(_abs_rows(), dtype=torch.float64)
    order = torch.sort(rows.square().sum(1), stable=True).indices
    rows = rows[order]
    packed = (((rows * 4).to(torch.int64) & 255) << (8 * torch.arange(8))).sum(1)
    return packed.to(device)


def grid_from_codebook(codebook_abs):
    """half [256,8] grid equal to the packed table: byte d of entry i, as int8, over 4."""
    cb = codebook_abs.to(torch.int64)
    b = (cb[:, None] >> (8 * torch.arange(8, device=cb.device))) & 255
    b = torch.where(b >= 128, b - 256, b)
    return (b.to(torch.float32) / 4).to(torch.float16)


def transpose_tile(codes):
    """[N, K'] codes -> same shape, each 16-row x 4-column tile stored as 64 contiguous
    codes in [row % 8][column % 4][row // 8] order (test_decode_matmul.py:101-109)."""
    n, kc = codes.shape
    t = codes.reshape(n // 16, 16, kc // 4, 4).permute(0, 2, 1, 3)
    t = t.reshape(n // 16, kc // 4, 2, 8, 4).permute(0, 1, 3, 4, 2)
    return t.reshape(n, kc).contiguous()


def untranspose_tile(tiled):
    """Inverse of transpose_tile."""
    n, kc = tiled.shape
    t = tiled.reshape(n // 16, kc // 4, 8, 4, 2).permute(0, 1, 4, 2, 3)
    t = t.reshape(n // 16, kc // 4, 16, 4).permute(0, 2, 1, 3)
    return t.reshape(n, kc).contiguous()
