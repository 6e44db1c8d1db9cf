"""Synthetic inputs of the benchmark configurations: CPU torch.Generator, seed given, draw
order x -> codes -> grid; x ~ N(0,1) half [M,K]; codes uniform over all 65536 values
[N,K/8]; grid half [256,8] uniform from {0.25, 0.75, ..., 2.75}; scale = float32(1/sqrt(K))."""
import math

import torch

GRID_VALUES = (0.25, 0.75, 1.25, 1.75, 2.25, 2.75)

# (K, N) of the projections: in -> out
LLAMA2_7B = ((4096, 12288), (4096, 4096), (4096, 11008), (11008, 4096))
LLAMA2_70B = ((8192, 10240), (8192, 8192), (8192, 28672), (28672, 8192))
SMALL_BATCH = ((4096, 11008), (11008, 4096))
PREFILL = ((4096, 4096), (4096, 11008), (11008, 4096))


def make_inputs(M, N, K, seed=0, device="cpu"):
    """Returns (x half [M,K], codes int16 [N,K/8], grid half [256,8], scale float)."""
    assert K % 8 == 0
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    x = torch.randn(M, K, generator=gen, dtype=torch.float32).to(torch.float16)
    codes = torch.randint(0, 65536, (N, K // 8), generator=gen, dtype=torch.int32)
    codes = codes.to(torch.uint16).view(torch.int16)
    pick = torch.randint(0, len(GRID_VALUES), (256, 8), generator=gen)
    grid = torch.tensor(GRID_VALUES, dtype=torch.float32)[pick].to(torch.float16)
    scale = float(torch.tensor(1.0 / math.sqrt(K), dtype=torch.float32)) if K else 1.0
    if device != "cpu":
        x, codes, grid = x.to(device), codes.to(device), grid.to(device)
    return x, codes, grid, scale


def make_codes(N, K, seed, device="cpu"):
    """Only the code matrix (for rotating many distinct weight buffers in a benchmark)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    codes = torch.randint(0, 65536, (N, K // 8), generator=gen, dtype=torch.int32)
    codes = codes.to(torch.uint16).view(torch.int16)
    return codes.to(device) if device != "cpu" else codes


def code_bytes(N, K):
    """Bytes of codes one call reads: the numerator of the HBM roofline."""
    return N * K // 4


def flops(M, N, K):
    return 2 * M * N * K
