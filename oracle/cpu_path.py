"""CPU baseline of the operator: decode to a dense half matrix, then a library matmul, on
the host cores with torch.  TEST / MEASUREMENT INFRASTRUCTURE ONLY - the benchmark times
this beside the GPU path as the reported CPU figure; nothing shipped calls it.

The reference has no half-precision CPU path; its CPU oracle is the integer triple loop of
/root/reference/test_decode_matmul.py:58-71 built on the scalar decoder at :29-55.  This is
the vectorised restatement of that pair in the operator's half form (gather the grid row,
flip by the sign bits with the parity-implied eighth, add +-1/4, then x @ W.T)."""
import time

import torch


def decode_dense(codes, grid):
    """codes int16 [N, K/8], grid half [256,8] -> W half [N, K] (torch, CPU)."""
    c = codes.to(torch.int32) & 0xFFFF
    idx = c & 0xFF
    s7 = (c >> 8) & 0x7F
    par = s7 ^ (s7 >> 4)
    par = par ^ (par >> 2)
    par = (par ^ (par >> 1)) & 1
    s8 = s7 | (par << 7)
    neg = ((s8.unsqueeze(-1) >> torch.arange(8, dtype=torch.int32)) & 1).bool()
    g = grid[idx.long()]                                     # [N, K/8, 8]
    v = torch.where(neg, -g, g)
    delta = torch.where((c >> 15).bool(), -0.25, 0.25).to(torch.float16).unsqueeze(-1)
    return (v + delta).reshape(codes.shape[0], codes.shape[1] * 8)


def decode_matmul(x, codes, grid, scale):
    W = decode_dense(codes, grid)
    return ((x.float() @ W.float().T) * scale).to(torch.float16)


def time_cpu_path(x, codes, grid, scale, repeats=5):
    """Median seconds of (decode, matmul) over `repeats` runs."""
    dec, mm = [], []
    for _ in range(repeats):
        t0 = time.perf_counter()
        W = decode_dense(codes, grid)
        t1 = time.perf_counter()
        y = (x.float() @ W.float().T) * scale
        y = y.to(torch.float16)
        t2 = time.perf_counter()
        dec.append(t1 - t0)
        mm.append(t2 - t1)
    dec.sort()
    mm.sort()
    return dec[len(dec) // 2], mm[len(mm) // 2], y
