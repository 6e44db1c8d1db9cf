"""dmm_decode_matmul_noalloc_f16: the operator for callers that cannot allocate.  Its split-K
partial sums live in a static device array inside the library; the result must be the one
dmm_decode_matmul_ws_f16 gives with a caller's workspace, bit for bit, also when a call follows
a larger one that left the array full of other sums."""
import numpy as np
import pytest
import torch

from decode_matmul_amd import capi, workload
from tests.gpu_util import DEV, _stream, bits

pytestmark = pytest.mark.gpu


def _ws_call(x, codes, grid, scale):
    M, K = x.shape
    N = codes.shape[0]
    lib = capi.lib()
    nbytes = lib.dmm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=x.device)
    st = lib.dmm_decode_matmul_ws_f16(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), scale, y.data_ptr(),
                                      M, N, K, ws.data_ptr(), nbytes, _stream())
    capi.check("dmm_decode_matmul_ws_f16", st)
    return y, nbytes


def _noalloc_call(x, codes, grid, scale):
    M, K = x.shape
    N = codes.shape[0]
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=x.device)
    st = capi.lib().dmm_decode_matmul_noalloc_f16(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), scale,
                                                  y.data_ptr(), M, N, K, _stream())
    return y, st


def test_noalloc_matches_workspace_entry_two_calls_in_a_row():
    lib = capi.lib()
    assert lib.dmm_init(-1) == 0
    limit = lib.dmm_noalloc_scratch_bytes()
    assert limit == 16 << 20
    # a large call, then smaller ones: the second finds the first's partial sums in the buffer.
    # (48, 8192, 8192) and (40, 1024, 2048) split K; (8, 512, 1024) uses no scratch at all.
    used = []
    for seed, (M, N, K) in enumerate(((48, 8192, 8192), (40, 1024, 2048), (64, 4096, 11008), (8, 512, 1024))):
        x, codes, grid, scale = workload.make_inputs(M, N, K, seed=seed, device=DEV)
        want, nbytes = _ws_call(x, codes, grid, scale)
        assert nbytes <= limit
        used.append(nbytes)
        got, st = _noalloc_call(x, codes, grid, scale)
        capi.check("dmm_decode_matmul_noalloc_f16", st)
        torch.cuda.synchronize()
        assert not torch.isnan(got).any()
        assert np.array_equal(bits(got), bits(want)), (M, N, K)
    assert used[0] > used[1] > 0 and used[2] == limit and used[3] == 0


def test_noalloc_rejects_shapes_beyond_the_buffer():
    lib = capi.lib()
    M, N, K = 128, 4096, 11008
    assert lib.dmm_workspace_bytes(M, N, K) > lib.dmm_noalloc_scratch_bytes()
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=3, device=DEV)
    y, st = _noalloc_call(x, codes, grid, scale)
    torch.cuda.synchronize()
    assert st == -8 and "scratch" in capi.status_string(st)
    assert torch.isnan(y).all()          # nothing was launched
