"""GPU parity tests: the HIP kernels, called through the C ABI (ctypes, raw device
pointers) and through the PyTorch operator, against the CPU oracle on identical seeded
inputs.  Bar: decoded W bit-exact; y within rtol 1e-2 / atol 1e-2 of the fp32-accumulated
reference; exact where the arithmetic is exact (integer bridge)."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

import decode_matmul_amd as dmm
from decode_matmul_amd import capi, workload
from conftest import GOLDEN_DIR, quarter_grid
from gpu_util import DEV, assert_close_to_oracle, bits, c_decode, c_matmul
from oracle import dmm_oracle as orc

pytestmark = pytest.mark.gpu


def dev(a):
    if isinstance(a, np.ndarray):
        if a.dtype == np.uint16:
            a = a.view(np.int16)
        a = torch.from_numpy(np.ascontiguousarray(a))
    return a.to(DEV)


def finite_random_grid(seed):
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 65536, size=(256, 8)).astype(np.uint16)
    b[(b & 0x7C00) == 0x7C00] &= 0xBFFF          # no inf / nan
    return b.view(np.float16)


# ----------------------------------------------------------------- decode: bit-exact
@pytest.mark.parametrize("grid_kind", ["quarter0", "quarter1", "e8p", "anyhalf0", "anyhalf1", "denormal"])
def test_decode_all_65536_codes_bit_exact(grid_kind, all_codes):
    if grid_kind.startswith("quarter"):
        grid = quarter_grid(int(grid_kind[-1]))
    elif grid_kind == "e8p":
        grid = orc.grid_from_codebook(orc.build_codebook_abs())
    elif grid_kind == "denormal":
        grid = (np.arange(2048, dtype=np.uint16) * 3 % 1024).reshape(256, 8).view(np.float16)   # subnormal halves
    else:
        grid = finite_random_grid(int(grid_kind[-1]))
    codes = all_codes.reshape(256, 256)                       # N=256 rows, K=2048
    W = c_decode(dev(codes), dev(grid))
    torch.cuda.synchronize()
    want = orc.decode_f16(codes, grid)
    assert np.array_equal(bits(W), bits(want))


def test_decode_golden_sha256(all_codes):
    gold = json.load(open(os.path.join(GOLDEN_DIR, "golden.json")))["decode_all_codes"]
    grid = np.array(gold["grid_bits"], dtype=np.uint16).view(np.float16).reshape(256, 8)
    W = c_decode(dev(all_codes.reshape(65536, 1)), dev(grid))
    torch.cuda.synchronize()
    b = bits(W)
    assert hashlib.sha256(b.tobytes()).hexdigest() == gold["sha256_of_W_bits"]
    assert b[:16].tolist() == gold["first16_rows_bits"] and b[-16:].tolist() == gold["last16_rows_bits"]


@pytest.mark.parametrize("N,K,offset", [(1, 8, 0), (3, 8, 0), (7, 24, 0), (5, 40, 1), (33, 1000, 3), (4096, 4096, 0)])
def test_decode_ragged_and_unaligned(N, K, offset):
    rng = np.random.default_rng(N * 1000 + K)
    grid = quarter_grid(2)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    # an offset view makes the code pointer 2-byte aligned only -> narrow kernel
    backing = torch.zeros(N * (K // 8) + 8, dtype=torch.int16, device=DEV)
    view = backing[offset:offset + N * (K // 8)].view(N, K // 8)
    view.copy_(dev(codes))
    W = c_decode(view, dev(grid))
    torch.cuda.synchronize()
    assert np.array_equal(bits(W), bits(orc.decode_f16(codes, grid)))


# ----------------------------------------------------------------- operator vs oracle
def run_case(path, M, N, K, seed, via="c"):
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=seed)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    if via == "c":
        y = c_matmul(dev(x), dev(codes), dev(grid), scale, path)
    else:
        y = dmm.decode_matmul_path(dev(x), dev(codes), dev(grid), scale, path)
    torch.cuda.synchronize()
    assert y.dtype == torch.float16 and tuple(y.shape) == (M, N)
    assert_close_to_oracle(y, ref, "%s M=%d N=%d K=%d" % (path, M, N, K))
    return y


def test_config0_operator():
    # x [1,4096], codes [4096,512], seed 0: the reference-runnable configuration
    run_case("auto", 1, 4096, 4096, 0)
    run_case("auto", 1, 4096, 4096, 0, via="torch")


@pytest.mark.parametrize("M", [1, 2, 4, 8, 15, 16, 17, 32])
@pytest.mark.parametrize("N,K", [(4, 256), (64, 512), (100, 768), (1024, 4096), (256, 11008)])
def test_gemv_path(M, N, K):
    run_case("gemv", M, N, K, seed=M + N)


@pytest.mark.parametrize("M,N,K", [(1, 16, 64), (33, 128, 128), (128, 128, 4096), (200, 300, 448),
                                   (256, 1000, 11008), (5, 7, 64), (130, 129, 192)])
def test_gemm_path(M, N, K):
    run_case("gemm", M, N, K, seed=M)


@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (1, 5, 24), (3, 7, 1000), (9, 33, 4096), (2, 130, 11008)])
def test_generic_path(M, N, K):
    run_case("generic", M, N, K, seed=K)


@pytest.mark.parametrize("M,N,K", [(1, 8192, 8192), (4, 11008, 4096), (32, 4096, 11008), (64, 512, 4096),
                                   (1, 37, 24), (40, 64, 40)])
def test_auto_dispatch_and_torch_operator(M, N, K):
    y_c = run_case("auto", M, N, K, seed=1)
    y_t = run_case("auto", M, N, K, seed=1, via="torch")
    if capi.lib().dmm_workspace_bytes(M, N, K) == 0:
        assert torch.equal(y_c, y_t)             # same kernel either way
    else:                                        # the operator brings a workspace: compare like with like
        x, codes, grid, scale = workload.make_inputs(M, N, K, seed=1)
        y_w, _ = c_matmul_ws(dev(x), dev(codes), dev(grid), scale)
        assert torch.equal(y_w, y_t)


# ----------------------------------------------------------------- batch-1 kernel, 8-bit operands
# M <= 4 with x small enough for the LDS runs on fp8 weights / bf8 terms of x when every grid
# value fits fp8, and hands over to the 16-bit kernel inside the same launch when one does not.
def _in_8bit_domain(M, K):
    """LDS budget of the 8-bit kernels: one row of x is staged in chunks and only has to fit as halves (the
    16-bit kernel may have to take the call over); two to four rows keep all their terms in LDS."""
    if M == 1:
        return 96 * 1024 + 2 * 16 * 4 * 16 + (2 * K + 16) + 128 <= 160 * 1024
    return 96 * 1024 + 2 * 16 * 4 * M * 16 + 4 * M * (K + 16) + 2 * M * (K // 4 + 16) + 64 <= 160 * 1024


def _gemv_vs_oracle(x, codes, grid, scale, packed=False, path="gemv8"):
    W = orc.decode_f16(codes, grid)
    ref = orc.matmul_f32(x, W, scale)
    if packed:
        y = dmm.decode_matmul_packed(dev(x), dmm.pack_codes(dev(codes)), dev(grid), scale, codes.shape[0])
    else:
        y = c_matmul(dev(x), dev(codes), dev(grid), scale, path)
    torch.cuda.synchronize()
    return y, ref


@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("N,K", [(16, 256), (52, 1024), (4360, 2048), (1000, 4096), (12304, 8192)])
@pytest.mark.parametrize("grid_kind", ["e8p", "fp8_all", "half_any", "one_off"])
def test_gemv_8bit_operands_and_fallback(M, N, K, grid_kind):
    if not _in_8bit_domain(M, K):
        pytest.skip("the terms of x do not fit the LDS beside the tables: outside the kernel's domain")
    rng = np.random.default_rng(M * 7 + N + K)
    if grid_kind == "e8p":
        grid = orc.grid_from_codebook(orc.build_codebook_abs())
    elif grid_kind == "fp8_all":
        # every finite fp8 (e4m3) value, subnormals and both zeros included, as halves
        b = np.arange(256, dtype=np.uint32)
        b = b[(b & 0x7F) != 0x7F]
        e, m = (b >> 3) & 0xF, b & 7
        v = np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7)) * np.where(b & 0x80, -1.0, 1.0)
        grid = rng.choice(v, size=(256, 8)).astype(np.float16)
        grid[0, :4] = [448.0, -448.0, 2.0 ** -9, -0.0]
    elif grid_kind == "half_any":
        grid = finite_random_grid(M + N)                                     # no fp8 can hold these
        grid = (grid.astype(np.float32).clip(-8, 8)).astype(np.float16)
    else:
        grid = orc.grid_from_codebook(orc.build_codebook_abs()).copy()
        grid[rng.integers(0, 256), rng.integers(0, 8)] = np.float16(1.0 + 2.0 ** -4)   # one value with 5 significant bits
    x = rng.standard_normal((M, K)).astype(np.float16)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    # scale brings y to order 1, as the operator is used (the tolerance has an absolute part)
    scale = float(np.float32(1.0 / (np.sqrt(K) * max(1.0, float(np.sqrt(np.mean(grid.astype(np.float64) ** 2)))))))
    y, ref = _gemv_vs_oracle(x, codes, grid, scale)
    assert_close_to_oracle(y, ref, "8-bit gemv %s M=%d N=%d K=%d" % (grid_kind, M, N, K))
    ya, _ = _gemv_vs_oracle(x, codes, grid, scale, path="auto")
    yp, _ = _gemv_vs_oracle(x, codes, grid, scale, packed=True)
    assert torch.equal(ya, yp)                   # packed codes: same kernel choice, same arithmetic, same order
    if (N + 15) // 16 > 3 * 256 and grid_kind in ("e8p", "fp8_all"):
        assert torch.equal(y, ya)                # launches this long take the 8-bit kernel by themselves


@pytest.mark.parametrize("N,K", [(48, 4352), (1000, 8192), (12304, 12288), (4112, 28672), (24592, 4096),
                                 (16400, 9216), (28672, 8192)])
@pytest.mark.parametrize("grid_kind", ["e8p", "half_any"])
def test_gemv_8bit_one_row_of_x_in_chunks(N, K, grid_kind):
    """The batch-1 form of the 8-bit kernel stages x 4096 values at a time: a last chunk that is not
    full (K = 4352, 9216), x resident after one pass (K <= 8192) with one to three groups of tiles per
    workgroup (N = 24592: 1538 tiles on 256 workgroups), x staged again for every group (K = 12288 with
    two groups, K = 28672), and the hand-over to the 16-bit kernel for a grid no fp8 can hold."""
    rng = np.random.default_rng(N + K)
    grid = orc.grid_from_codebook(orc.build_codebook_abs())
    if grid_kind == "half_any":
        grid = (finite_random_grid(N).astype(np.float32).clip(-8, 8)).astype(np.float16)
    x = rng.standard_normal((1, K)).astype(np.float16)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    scale = float(np.float32(1.0 / (np.sqrt(K) * max(1.0, float(np.sqrt(np.mean(grid.astype(np.float64) ** 2)))))))
    y, ref = _gemv_vs_oracle(x, codes, grid, scale)
    assert_close_to_oracle(y, ref, "8-bit gemv in chunks %s N=%d K=%d" % (grid_kind, N, K))
    y2, _ = _gemv_vs_oracle(x, codes, grid, scale)
    assert torch.equal(y, y2)                    # same bits run after run
    ya, _ = _gemv_vs_oracle(x, codes, grid, scale, path="auto")
    yp, _ = _gemv_vs_oracle(x, codes, grid, scale, packed=True)
    assert torch.equal(ya, yp)                   # packed codes: same kernel choice, same arithmetic, same order
    if (N + 15) // 16 > 2 * 256:
        assert torch.equal(y, ya)                # launches this long take the 8-bit kernel by themselves
    if grid_kind == "half_any":                  # handed over: exactly the 16-bit streaming kernel's result
        was = capi.lib().dmm_set_gemv_8bit(0)
        was2 = capi.lib().dmm_set_choice(2, 0)   # (with the 8-bit kernels off the operator would take the other 16-bit one)
        try:
            assert capi.lib().dmm_gemv_kernel_name(1, N, K) == b"dmm::gemv_stream_kernel"
            y16 = c_matmul(dev(x), dev(codes), dev(grid), scale, "gemv")
        finally:
            capi.lib().dmm_set_gemv_8bit(was)
            capi.lib().dmm_set_choice(2, was2)
        assert torch.equal(y, y16)


def test_gemv_8bit_exact_for_extreme_x():
    """One non-zero x at a time, from all over the half range (largest, smallest normal,
    subnormals, all 11 significant bits set), against weights 0 and +-0.5: the four bf8 terms
    add up to x exactly and so does the mean of its code, so y = x w with no rounding at all."""
    K, N = 2048, 64
    grid = np.full((256, 8), 0.25, dtype=np.float16)   # w = 0.25 s + d: 0 or +-0.5
    special = np.array([65504.0, -65504.0, 2.0 ** -14, 2.0 ** -21, -24 * 2.0 ** -24, 1023.5, 0.333251953125,
                        2047.0, -6.103515625e-05 * 1.5, 40000.0, 3.0], dtype=np.float16)
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    W = orc.decode_f16(codes, grid).astype(np.float64)
    assert set(np.unique(W)) <= {-0.5, 0.0, 0.5}
    for i, v in enumerate(special):
        x = np.zeros((1, K), dtype=np.float16)
        k = int(rng.integers(0, K))
        x[0, k] = v
        y = c_matmul(dev(x), dev(codes), dev(grid), 1.0, "gemv8")
        torch.cuda.synchronize()
        want = float(v) * W[:, k]
        assert np.array_equal(y.cpu().numpy().astype(np.float64)[0], want), (i, float(v))


def _random_8bit_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        M = int(rng.integers(1, 5))
        K = 256 * int(rng.integers(1, 50))
        if not _in_8bit_domain(M, K):
            continue
        N = 4 * int(rng.integers(1, 1400)) if len(out) % 3 else 4 * int(rng.integers(1100, 2600))
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("M,N,K", _random_8bit_cases(30, 4242))
def test_gemv_8bit_random_shapes(M, N, K):
    """Seeded random shapes of the 8-bit kernel's whole domain (ragged last tiles, a single k step,
    the largest x that fits), fp8-exact grids, y inside a guarded buffer."""
    rng = np.random.default_rng(M * 1000003 + N * 101 + K)
    fp8_vals = np.array([0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.25, 2.5, 2.75, 3.5, 5.0, 7.5, 0.015625, 0.109375])
    grid = (rng.choice(fp8_vals, size=(256, 8)) * rng.choice([-1.0, 1.0], size=(256, 8))).astype(np.float16)
    x = (rng.standard_normal((M, K)) * rng.choice([0.01, 1.0, 30.0])).astype(np.float16)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    scale = float(np.float32(1.0 / (np.sqrt(K) * max(1e-3, float(np.abs(x.astype(np.float64)).mean())))))
    ref = orc.matmul_f32(x, orc.decode_f16(codes, grid), scale)
    guard = 64
    buf = torch.full((M * N + 2 * guard,), 777.0, dtype=torch.float16, device=DEV)
    y = buf[guard:guard + M * N].view(M, N)
    c_matmul(dev(x), dev(codes), dev(grid), scale, "gemv8", out=y)
    torch.cuda.synchronize()
    assert_close_to_oracle(y, ref, "8-bit random M=%d N=%d K=%d" % (M, N, K))
    assert torch.all(buf[:guard] == 777.0) and torch.all(buf[guard + M * N:] == 777.0)


def test_read_probe_reads_and_leaves_its_sink_alone():
    """The benchmark's yardstick kernel: runs on the caller's stream for short and long launches (fewer
    tiles than compute units, several per unit, N no multiple of 16), returns DMM_OK and never writes
    its sink for codes whose bytes do not cancel."""
    lib = capi.lib()
    sink = torch.full((4,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    for N, K in ((16, 256), (1000, 512), (8192, 8192), (28672, 2048)):
        _, codes, _, _ = workload.make_inputs(1, N, K, seed=N % 7)
        cd = dev(codes)
        st = lib.dmm_read_probe(cd.data_ptr(), sink.data_ptr(), N, K, torch.cuda.current_stream().cuda_stream)
        assert st == 0, capi.status_string(st)
    torch.cuda.synchronize()
    assert torch.all(sink == 0x5A5A5A5A)


def test_gemv_8bit_switch_and_kernel_name():
    """The operator's choice follows dmm_set_gemv_8bit; with the 8-bit kernel off the result is the
    16-bit kernel's, i.e. what the explicit 16-bit configuration of the same launch gives."""
    lib = capi.lib()
    M, N, K = 1, 16384, 1024                                 # 1024 tiles, four per CU: long enough for the 8-bit kernel
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=11)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    was = lib.dmm_set_gemv_8bit(1)
    try:
        assert lib.dmm_gemv_kernel_name(M, N, K) == b"dmm::gemv_q8d_kernel"
        assert lib.dmm_gemv_kernel_name(M, 8208, K) == b"dmm::gemv_q8d_kernel"        # more than two tiles per CU
        assert lib.dmm_gemv_kernel_name(M, 8192, K) == b"dmm::gemv_q8d_kernel"        # two tiles per CU
        assert lib.dmm_gemv_kernel_name(M, 4112, K) == b"dmm::gemv_q8d_kernel"        # more than one
        assert lib.dmm_gemv_kernel_name(M, 4096, K) == b"dmm::gemv_stream_kernel"     # one
        assert lib.dmm_gemv_kernel_name(M, 8192, 11008) == b"dmm::gemv_q8d_kernel"    # two, x of two and a bit chunks
        assert lib.dmm_gemv_kernel_name(M, 4096, 11008) == b"dmm::gemv_stream_kernel" # one tile per CU
        assert lib.dmm_gemv_kernel_name(M, 4096, 28672) == b"dmm::gemv_q8d_kernel"    # one, long x
        assert lib.dmm_gemv_kernel_name(M, 8208, 11008) == b"dmm::gemv_q8d_kernel"
        assert lib.dmm_gemv_kernel_name(M, 8192, 12288) == b"dmm::gemv_q8d_kernel"    # two, long x
        assert lib.dmm_gemv_kernel_name(M, N, 28672) == b"dmm::gemv_q8d_kernel"       # x goes through in chunks
        assert lib.dmm_gemv_kernel_name(M, 32768, K) == b"dmm::gemv_q8d_kernel"       # eight tiles per CU
        assert lib.dmm_gemv_kernel_name(M, 32784, K) == b"dmm::gemv_q8c_kernel"       # more: groups of three tiles
        # up to eight rows on two to eight tiles per CU: the 16-bit kernel with resident sums, whatever K
        for m in (2, 3, 4, 5, 8):
            for n, k in ((N, K), (12288, K), (8192, 256), (32768, K), (N, 28672), (28672, 8192), (4112, 4096)):
                assert lib.dmm_gemv_kernel_name(m, n, k) == b"dmm::gemv_f16d_kernel", (m, n, k)
        assert lib.dmm_gemv_kernel_name(3, 32784, K) == b"dmm::gemv_q8_kernel"        # more tiles, two to four rows: 8-bit
        assert lib.dmm_gemv_kernel_name(5, 32784, K) == b"dmm::gemv_stream_kernel"
        # nine to sixteen rows: the same kernel on eight waves, whatever the share (up to eight tiles per CU)
        for m, n, k in ((9, N, K), (9, N, 8192), (16, 4096, 4096), (12, 32768, 256), (16, 28672, 8192)):
            assert lib.dmm_gemv_kernel_name(m, n, k) == b"dmm::gemv_f16d_kernel", (m, n, k)
        assert lib.dmm_gemv_kernel_name(9, 32784, K) == b"dmm::gemv_stream_kernel"    # more tiles
        assert lib.dmm_gemv_kernel_name(9, 32784, 8192) == b"dmm::gemv_regx_kernel"   # ... and an x that does not fit the LDS
        # seventeen to 32 rows: with two MFMAs per code on two to eight tiles per CU and K >= 2048
        for m, n, k in ((17, N, 2048), (32, 28672, 8192), (24, 4112, 4096), (32, 32768, 28672)):
            assert lib.dmm_gemv_kernel_name(m, n, k) == b"dmm::gemv_f16d_kernel", (m, n, k)
        for m, n, k in ((32, N, K), (17, 4096, 8192), (32, 32784, 4096)):             # short K, one tile per CU, more than eight
            assert lib.dmm_gemv_kernel_name(m, n, k) == b"dmm::gemv_regx_kernel", (m, n, k)
        assert lib.dmm_gemv_kernel_name(33, N, 4096) == b""
        for m, n, k in ((2, 4096, K), (2, 4096, 8192), (3, 4096, 28672), (8, 16, 256)):  # two rows or more: one tile per CU too
            assert lib.dmm_gemv_kernel_name(m, n, k) == b"dmm::gemv_f16d_kernel", (m, n, k)
        was_choice = lib.dmm_set_choice(2, 0)                                           # ... and what serves with that kernel off
        assert lib.dmm_gemv_kernel_name(2, 4096, K) == b"dmm::gemv_regx_kernel"       # one tile per CU, short x
        assert lib.dmm_gemv_kernel_name(2, 4096, 8192) == b"dmm::gemv_stream_kernel"
        assert lib.dmm_gemv_kernel_name(3, 4096, 28672) == b"dmm::gemv_regx_kernel"
        assert lib.dmm_gemv_kernel_name(9, N, K) == b"dmm::gemv_stream_kernel"
        assert lib.dmm_gemv_kernel_name(32, 28672, 8192) == b"dmm::gemv_regx_kernel"
        lib.dmm_set_choice(2, was_choice)
        assert lib.dmm_gemv_kernel_name(M, N, 264) == b""
        y8 = c_matmul(dev(x), dev(codes), dev(grid), scale, "auto")
        assert torch.equal(y8, c_matmul(dev(x), dev(codes), dev(grid), scale, "gemv8"))
        assert lib.dmm_set_gemv_8bit(0) == 1
        assert lib.dmm_gemv_kernel_name(M, N, K) == b"dmm::gemv_f16d_kernel"
        assert lib.dmm_gemv_kernel_name(M, 4096, K) == b"dmm::gemv_stream_kernel"
        y16 = c_matmul(dev(x), dev(codes), dev(grid), scale, "auto")
        torch.cuda.synchronize()
        assert_close_to_oracle(y8, ref, "8-bit")
        assert_close_to_oracle(y16, ref, "16-bit")
        # the 16-bit kernel's y is the correctly rounded product
        want = (x.numpy().astype(np.float64) @ orc.decode_f16(codes.numpy(), grid.numpy()).astype(np.float64).T) * np.float64(np.float32(scale))
        assert (y16.cpu().numpy() != want.astype(np.float16)).mean() < 0.005
        assert (y8.cpu().numpy() != want.astype(np.float16)).mean() < 0.05
    finally:
        lib.dmm_set_gemv_8bit(was)


def test_gemv_8bit_non_finite_x_in_a_later_chunk():
    """One row of x, staged in chunks: an infinity in the third chunk is found after two chunks have been
    multiplied; the 16-bit kernel then does the whole call over."""
    K, N = 12288, 16400
    rng = np.random.default_rng(10)
    grid = orc.grid_from_codebook(orc.build_codebook_abs())
    x = rng.standard_normal((1, K)).astype(np.float16)
    x[0, 8200] = -np.inf
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    y, ref = _gemv_vs_oracle(x, codes, grid, 0.01)
    got = y.cpu().numpy().astype(np.float32)
    assert np.isinf(got).any() and not np.isnan(ref).any()
    assert np.array_equal(np.isinf(got), np.isinf(ref)) and np.array_equal(got[np.isinf(got)], ref[np.isinf(ref)])
    fin = np.isfinite(ref)
    assert np.all(np.abs(got[fin] - ref[fin]) <= 1e-2 + 1e-2 * np.abs(ref[fin]))


def test_gemv_8bit_non_finite_x():
    K, N = 1024, 48
    rng = np.random.default_rng(9)
    grid = orc.grid_from_codebook(orc.build_codebook_abs())
    x = rng.standard_normal((2, K)).astype(np.float16)
    x[0, 17] = np.inf
    x[1, 900] = np.nan
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    y, ref = _gemv_vs_oracle(x, codes, grid, 0.03125)
    got = y.cpu().numpy().astype(np.float32)
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.array_equal(np.isinf(got), np.isinf(ref))
    assert np.array_equal(got[np.isinf(got)], ref[np.isinf(ref)])   # the signs of the infinities


def test_empty_problems():
    grid = dev(quarter_grid(0))
    x = torch.zeros(0, 64, dtype=torch.float16, device=DEV)
    codes = torch.zeros(5, 8, dtype=torch.int16, device=DEV)
    assert tuple(dmm.decode_matmul(x, codes, grid, 1.0).shape) == (0, 5)
    x = torch.zeros(3, 64, dtype=torch.float16, device=DEV)
    codes = torch.zeros(0, 8, dtype=torch.int16, device=DEV)
    assert tuple(dmm.decode_matmul(x, codes, grid, 1.0).shape) == (3, 0)
    assert tuple(dmm.decode(codes, grid).shape) == (0, 64)
    # K = 0: the empty sum is zero
    x = torch.zeros(3, 0, dtype=torch.float16, device=DEV)
    codes = torch.zeros(4, 0, dtype=torch.int16, device=DEV)
    y = dmm.decode_matmul(x, codes, grid, 1.0)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (3, 4) and torch.all(y == 0)


# ----------------------------------------------------------------- exact integer bridge
@pytest.mark.parametrize("path,M,N,K", [("gemv", 8, 16, 4096), ("gemm", 8, 16, 4096), ("generic", 8, 16, 4096),
                                         ("gemv", 1, 64, 8192), ("gemm", 64, 64, 8192),
                                         ("gemv8", 1, 64, 8192), ("gemv8", 1, 8192, 2048), ("gemv8", 3, 4100, 4096),
                                         ("auto", 1, 16384, 4096),
                                         ("gemv", 12, 4800, 5120), ("gemv", 16, 4112, 8192), ("gemv", 32, 1028, 8192),
                                         ("auto", 64, 4096, 4096)])
def test_integer_bridge_is_exact(path, M, N, K):
    """x integer-valued, grid = E8P bytes / 4, scale a power of two: every partial sum is a
    multiple of 1/4 below 2^24 quarters, so fp32 accumulation in any order is exact and the
    half output must EQUAL half(int32_result / 4 * scale), the reference's integer operator
    (/root/reference/test_decode_matmul.py:58-71) on the same codes."""
    rng = np.random.default_rng(K + M)
    cb = orc.build_codebook_abs()
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    yi = orc.decode_matmul_i32(x, codes, cb)
    scale = 2.0 ** -8
    want = (yi.astype(np.float64) / 4 * scale).astype(np.float16)
    if path == "gemv" and M >= 12:   # nine to sixteen rows: the kernel with resident sums; 32 on one tile per CU: the small-batch kernel's passes
        assert capi.lib().dmm_gemv_kernel_name(M, N, K) == (b"dmm::gemv_f16d_kernel" if M <= 16 else b"dmm::gemv_regx_kernel")
    y = c_matmul(dev(x.astype(np.float16)), dev(codes), dev(orc.grid_from_codebook(cb)), scale, path)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), bits(want))


@pytest.mark.parametrize("N,K", [(4048, 1024), (8032, 4352), (12304, 12288), (16000, 768), (20000, 8192), (24592, 512),
                                 (28000, 4096), (32768, 512), (33000, 768), (8192, 28672)])
def test_gemv_8bit_every_share_of_tiles_is_exact(N, K):
    """One row of x on the 8-bit kernels, exactly (the integer bridge): workgroups of one to eight row tiles
    (every instantiation of the resident-accumulator kernel, with shares that differ by one between
    workgroups), one to seven chunks of x with a last chunk that is not full, fewer k steps than waves, and
    more than eight tiles per workgroup (the chunked kernel with its groups of three)."""
    lib = capi.lib()
    rng = np.random.default_rng(N + K)
    cb = orc.build_codebook_abs()
    x = rng.integers(-128, 128, size=(1, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    yi = orc.decode_matmul_i32(x, codes, cb)
    scale = 2.0 ** -8
    want = (yi.astype(np.float64) / 4 * scale).astype(np.float16)
    y = c_matmul(dev(x.astype(np.float16)), dev(codes), dev(orc.grid_from_codebook(cb)), scale, "gemv8")
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), bits(want))
    if (N + 15) // 16 > 2 * 256:
        name = lib.dmm_gemv_kernel_name(1, N, K)
        assert name == (b"dmm::gemv_q8d_kernel" if (N + 15) // 16 <= 8 * 256 else b"dmm::gemv_q8c_kernel")


@pytest.mark.parametrize("M,N,K", [(2, 6000, 16384), (4, 4112, 8448), (4, 12272, 7168), (3, 16400, 11008), (4, 20000, 8192),
                                   (2, 24592, 16384), (4, 28672, 8192), (4, 32768, 7168), (2, 8192, 28672), (3, 4100, 28672),
                                   (8, 4112, 8192), (6, 20000, 4096), (8, 28672, 4096), (5, 8192, 28672), (8, 12272, 256),
                                   (7, 32768, 512), (1, 16400, 4352), (5, 24592, 1280),
                                   # nine to sixteen rows: eight waves with pieces of sixteen rows
                                   (16, 8192, 8192), (9, 4112, 28672), (12, 12272, 2304), (16, 16400, 4096), (13, 20000, 1280),
                                   (10, 24592, 768), (16, 28672, 8192), (11, 32768, 256), (15, 10240, 8192),
                                   # seventeen to 32 rows: two groups of sixteen, one decode for both
                                   (17, 8192, 8192), (32, 4112, 28672), (24, 12272, 2304), (32, 28672, 8192), (20, 16400, 256),
                                   (31, 32768, 512), (32, 11008, 4096), (25, 20000, 1280), (18, 4096, 4096)])
def test_chunked_16bit_kernel_is_exact(M, N, K):
    """Up to 32 rows of x on the 16-bit kernel with resident sums, exactly (the integer bridge): all widths
    of the x slice (up to four, eight and sixteen rows and two groups of sixteen, full and with rows to spare), workgroups of one to eight row
    tiles (launches of two to eight per workgroup at most), one to seven chunks with a last chunk that is not
    full, fewer k steps than waves, one row of x with the 8-bit kernels switched off.  Reference: the library's own decode
    (pinned bit for bit against the oracle above) times x in fp64 on the GPU, which is exact for these
    integers, plus the oracle's integer product on the first and last rows of W."""
    lib = capi.lib()
    was = lib.dmm_set_gemv_8bit(0 if M == 1 else 1)
    was_choice = lib.dmm_set_choice(2, 1 if M > 16 else -1)   # more than sixteen rows: also where the operator would not
    try:
        assert lib.dmm_gemv_kernel_name(M, N, K) == b"dmm::gemv_f16d_kernel"
        rng = np.random.default_rng(M + N + K)
        cb = orc.build_codebook_abs()
        x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
        g = torch.Generator(device=DEV)
        g.manual_seed(M * N + K)
        codes = torch.randint(-32768, 32768, (N, K // 8), generator=g, dtype=torch.int16, device=DEV)
        scale = 2.0 ** -8
        xd, gd = dev(x.astype(np.float16)), dev(orc.grid_from_codebook(cb))
        buf = torch.full((64 + M * N + 64,), -7.0, dtype=torch.float16, device=DEV)
        y = buf[64:64 + M * N].view(M, N)
        c_matmul(xd, codes, gd, scale, "gemv", out=y)
    finally:
        lib.dmm_set_gemv_8bit(was)
        lib.dmm_set_choice(2, was_choice)
    W = c_decode(codes, gd)
    torch.cuda.synchronize()
    want = ((xd.double() @ W.double().T) * scale).to(torch.float16)
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    assert torch.all(buf[:64] == -7.0) and torch.all(buf[64 + M * N:] == -7.0)
    rows = np.concatenate([np.arange(min(24, N)), np.arange(max(N - 24, 0), N)])
    yi = orc.decode_matmul_i32(x, codes[torch.from_numpy(rows).to(DEV)].cpu().numpy(), cb)
    assert np.array_equal(bits(y[:, torch.from_numpy(rows).to(DEV)].contiguous()), bits((yi.astype(np.float64) / 4 * scale).astype(np.float16)))


def test_reference_shape_golden_case():
    """The reference's one validated shape, M=8 N=16 K=4096, from the committed fixture."""
    case = np.load(os.path.join(GOLDEN_DIR, "int8_case.npz"))
    x, codes, yi, cb = case["x"], case["codes"], case["y"], case["codebook_abs"]
    grid = dmm.grid_from_codebook(torch.from_numpy(cb))
    for path in ("auto", "gemv", "gemm", "generic"):
        y = c_matmul(dev(x.astype(np.float16)), dev(codes), grid.to(DEV), 2.0 ** -8, path)
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), bits((yi.astype(np.float64) / 4 * 2.0 ** -8).astype(np.float16))), path


# ----------------------------------------------------------------- the integer operator itself
def c_matmul_i8(x, codes, cb, tiled):
    M, K = x.shape
    N = codes.shape[0]
    out = torch.full((M, N), -12345, dtype=torch.int32, device=x.device)
    st = capi.lib().dmm_decode_matmul_i8(x.data_ptr(), codes.data_ptr(), cb.data_ptr(), out.data_ptr(), M, N, K,
                                         int(tiled), torch.cuda.current_stream().cuda_stream)
    capi.check("dmm_decode_matmul_i8", st)
    return out


@pytest.mark.parametrize("M,N,K", [(8, 16, 4096), (1, 16, 32), (3, 48, 96), (13, 160, 2048), (5, 32, 8192)])
def test_integer_operator_tiled_is_exact(M, N, K):
    """int8 x, int16 codes in the reference kernel's tile order, packed int64 table -> int32,
    equal to the reference's checker (/root/reference/test_decode_matmul.py:58-71) restated by
    the oracle, element for element."""
    rng = np.random.default_rng(N * 7 + K)
    cb = orc.build_codebook_abs()
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    want = orc.decode_matmul_i32(x, codes, cb)
    out = c_matmul_i8(dev(x), dev(orc.transpose_tile(codes)), dev(cb), True)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)
    # the torch operator with the reference's own argument list gives the same tensor
    out2 = dmm.decode_matmul_int8(dev(x), dmm.transpose_tile(dev(codes)), dev(cb))
    assert out2.dtype == torch.int32 and torch.equal(out2, out)


@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (2, 3, 32), (7, 37, 1000), (4, 5, 24)])
def test_integer_operator_row_major_any_shape(M, N, K):
    rng = np.random.default_rng(N * 11 + K)
    cb = rng.integers(-2 ** 63, 2 ** 63, size=256, dtype=np.int64)       # any table, not only E8P
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    want = orc.decode_matmul_i32(x, codes, cb)
    out = c_matmul_i8(dev(x), dev(codes), dev(cb), False)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("M,N,K,tiled,x_off", [(1, 37, 1000, False, 0), (8, 48, 1024, True, 0), (13, 48, 1024, True, 3),
                                               (9, 37, 1000, False, 1), (20, 16, 4096, True, 8)])
def test_integer_operator_table_bytes_2_mod_4(M, N, K, tiled, x_off):
    """Any table whose bytes are all 2 mod 4 takes the one-exclusive-or decode (the E8P table is
    such a table; so is this random one, with bytes from -126 to 126): batches above the 8 rows
    one pass covers, x at byte offsets that rule out 8-byte loads, both code layouts."""
    rng = np.random.default_rng(M * 131 + N)
    by = (rng.integers(0, 256, size=(256, 8)).astype(np.uint8) & 0xFC) | 2
    by[0] = [0x82, 0x7E, 0x02, 0xFE, 0x06, 0xFA, 0x7E, 0x82]
    cb = by.view(np.int64).reshape(256).copy()
    xbuf = rng.integers(-128, 128, size=M * K + 16).astype(np.int8)
    xs = xbuf[x_off:x_off + M * K].reshape(M, K)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    want = orc.decode_matmul_i32(xs, codes, cb)
    xd = dev(xbuf)[x_off:x_off + M * K].view(M, K)
    cd = dev(orc.transpose_tile(codes)) if tiled else dev(codes)
    out = c_matmul_i8(xd, cd, dev(cb), tiled)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("M,N,K,tiled,table", [
    (8, 16, 4096, True, "e8p"), (1, 4100, 256, False, "e8p"), (16, 16 * 300, 512, True, "e8p"),
    (17, 16 * (256 * 2 + 5), 256, True, "e8p"), (40, 1000, 768, False, "mod4"), (8, 16 * 1000, 1024, True, "mod4"),
    (5, 8192 + 16, 1024, True, "any"), (3, 52, 2048, False, "any"), (16, 4096, 4096, False, "e8p"),
    # workgroup shares of 3, 4, 7 and 5 tiles: row blocks of three and four tiles, partial last blocks
    (8, 16 * (256 * 3 - 10), 256, True, "e8p"), (16, 16 * (256 * 4 - 3), 256, False, "mod4"),
    (8, 28672, 256, True, "e8p"), (4, 16 * (256 * 5 - 1), 512, True, "any"),
    # more than 16 rows of x in passes of the one launch, a last pass with rows to spare
    (24, 16 * 130, 2048, True, "e8p"), (33, 1028, 8192, False, "mod4"), (64, 4096, 4096, True, "e8p"),
    (100, 2052, 1024, False, "any"), (48, 16 * (256 * 3 - 10), 512, True, "mod4")])
def test_integer_operator_matrix_unit(M, N, K, tiled, table):
    """K a multiple of 256 with 16-byte aligned buffers runs on v_mfma_i32_16x16x64_i8: one or
    several tiles per workgroup with partial last blocks, more than 16 rows of x (passes over
    the row blocks inside the one launch), both code layouts, N no multiple of 16 (row-major),
    and a table with bytes that are not 2 mod 4, which every workgroup must notice and serve
    with the scalar decode.  Exact against the oracle's restatement of
    /root/reference/test_decode_matmul.py:58-71."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    share = -(-((N + 15) // 16) // cus)
    resident = M <= 32 and 2 <= share <= 8 and K >= (4096 if M > 16 else 512 if M <= 8 and share <= 4 else 1024)   # two to eight row tiles per compute unit, K not short
    assert capi.lib().dmm_integer_kernel_name(M, N, K) == (b"dmm::int8d_kernel" if resident else b"dmm::int8x_kernel")
    rng = np.random.default_rng(M * 977 + N + K)
    if table == "e8p":
        cb = orc.build_codebook_abs()
    elif table == "mod4":
        cb = ((rng.integers(0, 256, size=(256, 8)).astype(np.uint8) & 0xFC) | 2).view(np.int64).reshape(256).copy()
    else:
        cb = rng.integers(-2 ** 63, 2 ** 63, size=256, dtype=np.int64)
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    want = orc.decode_matmul_i32(x, codes, cb)
    cd = dev(orc.transpose_tile(codes)) if tiled else dev(codes)
    out = c_matmul_i8(dev(x), cd, dev(cb), tiled)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("M,N,K,tiled,table", [
    # two to eight row tiles per compute unit (every instance of the kernel, shares that leave the last
    # tiles of an instance unused, N no multiple of 16), one k step to 33 (waves without a step, a ragged
    # last chunk), one to eight rows of x, both code layouts, every kind of table
    (1, 4100, 256, False, "e8p"), (2, 8192, 8192, True, "e8p"), (3, 16 * (256 * 2 + 5), 768, True, "mod4"),
    (4, 16 * (256 * 3 - 10), 4352, False, "e8p"), (5, 8192 + 16, 1024, True, "any"), (6, 16384, 2048, True, "e8p"),
    (7, 16 * (256 * 5 - 1), 512, False, "mod4"), (8, 16 * (256 * 6 - 100), 1280, True, "e8p"),
    (8, 28672, 256, True, "e8p"), (1, 28672, 8448, True, "e8p"), (8, 32768, 768, False, "mod4"),
    (3, 16 * (256 * 7 + 1) - 12, 512, False, "any"), (8, 10240, 8192, True, "e8p"), (1, 16 * (256 * 4), 4096, False, "e8p"),
    # nine to sixteen rows: eight waves with pieces of sixteen rows
    (16, 8192, 8192, True, "e8p"), (9, 4100, 2304, False, "mod4"), (12, 16 * (256 * 3 - 10), 256, True, "e8p"),
    (16, 28672, 1280, True, "any"), (13, 16 * (256 * 5 - 1), 768, False, "e8p"), (10, 16 * (256 * 6 - 100), 512, True, "mod4"),
    (16, 32768, 512, False, "e8p"), (15, 16384, 4352, True, "e8p"),
    # seventeen to 32 rows: two groups of sixteen, one decode for both
    (17, 8192, 8192, True, "e8p"), (32, 4100, 2304, False, "mod4"), (24, 16 * (256 * 3 - 10), 256, True, "e8p"),
    (32, 28672, 1280, True, "any"), (25, 16 * (256 * 5 - 1), 768, False, "e8p"), (31, 16 * (256 * 6 - 100), 512, True, "mod4"),
    (32, 32768, 512, False, "e8p"), (20, 16384, 4352, True, "e8p")])
def test_integer_operator_resident_sums(M, N, K, tiled, table):
    """Up to 32 rows of x with two to eight row tiles per compute unit run on the kernel that keeps the
    sums of its whole share in registers.  Exact against the oracle's decode times x in float64 (every sum
    is far below 2^53, so that product is the integer one) and, on the first and last rows of W, against
    the integer oracle itself (/root/reference/test_decode_matmul.py:58-71 restated); the row-block kernel,
    forced, gives the same tensor."""
    lib = capi.lib()
    # the operator's own rule takes this kernel from some K on; here it is tried on the shorter K as well
    share = -(-((N + 15) // 16) // torch.cuda.get_device_properties(0).multi_processor_count)
    takes = K >= (4096 if M > 16 else 512 if M <= 8 and share <= 4 else 1024)
    assert (lib.dmm_integer_kernel_name(M, N, K) == b"dmm::int8d_kernel") == takes
    rng = np.random.default_rng(M * 613 + N + K)
    if table == "e8p":
        cb = orc.build_codebook_abs()
    elif table == "mod4":
        cb = ((rng.integers(0, 256, size=(256, 8)).astype(np.uint8) & 0xFC) | 2).view(np.int64).reshape(256).copy()
    else:
        cb = rng.integers(-2 ** 63, 2 ** 63, size=256, dtype=np.int64)
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    cd = dev(orc.transpose_tile(codes)) if tiled else dev(codes)
    before, before_mm = lib.dmm_set_choice(3, 1), lib.dmm_set_choice(1, 1)   # ... and not the matrix-matrix kernel
    try:
        assert lib.dmm_integer_kernel_name(M, N, K) in (b"dmm::int8d_kernel", b"dmm::int8g_kernel")   # (the name does not see the second override)
        out = c_matmul_i8(dev(x), cd, dev(cb), tiled)
        torch.cuda.synchronize()
    finally:
        lib.dmm_set_choice(3, before)
        lib.dmm_set_choice(1, before_mm)
    got = out.cpu().numpy()
    rows = np.r_[0:40, N - 40:N]
    assert np.array_equal(got[:, rows], orc.decode_matmul_i32(x, codes[rows], cb))
    W = torch.from_numpy(orc.decode_i8(codes, cb)).to(DEV).double()
    want = (dev(x).double() @ W.T).cpu().numpy().astype(np.int64).astype(np.int32)
    del W
    assert np.array_equal(got, want)
    before, before_mm = lib.dmm_set_choice(3, 0), lib.dmm_set_choice(1, 1)
    try:
        assert lib.dmm_integer_kernel_name(M, N, K) in (b"dmm::int8x_kernel", b"dmm::int8g_kernel")
        out2 = c_matmul_i8(dev(x), cd, dev(cb), tiled)
        torch.cuda.synchronize()
    finally:
        lib.dmm_set_choice(3, before)
        lib.dmm_set_choice(1, before_mm)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("M,N,K,tiled,table", [
    (128, 32768, 256, True, "e8p"), (300, 16 * 1030, 512, False, "mod4"), (64, 40000, 256, False, "any"),
    (2048, 4096, 512, True, "e8p"), (200, 16 * 1030, 1280, True, "mod4"), (129, 16 * 1030, 256, True, "any"),
    (384, 4096, 4096, True, "e8p"), (512, 2048, 8192, False, "mod4"),
    (512, 2048, 768, False, "e8p"), (384, 4096, 2304, True, "mod4"), (640, 8192, 1536, True, "e8p")])
def test_integer_operator_matrix_matrix(M, N, K, tiled, table):
    """Many rows of x run on the int8 matrix-matrix kernel: partial tiles in M and N, both code layouts, 4 to 128 k tiles
    (2 to 64 per half of the workgroup: every count of leftover tiles after its trips of six, and none), and a
    table with bytes that are not 2 mod 4 (scalar decode per workgroup, with x rows and output
    rows offset by the workgroup's m block).  Exact against the oracle's decode times x in
    float64 (every sum is far below 2^53, so that product is the integer one)."""
    assert capi.lib().dmm_integer_kernel_name(M, N, K) == b"dmm::int8g_kernel"
    rng = np.random.default_rng(M * 31 + N + K)
    if table == "e8p":
        cb = orc.build_codebook_abs()
    elif table == "mod4":
        cb = ((rng.integers(0, 256, size=(256, 8)).astype(np.uint8) & 0xFC) | 2).view(np.int64).reshape(256).copy()
    else:
        cb = rng.integers(-2 ** 63, 2 ** 63, size=256, dtype=np.int64)
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    W = orc.decode_i8(codes, cb)
    want = (x.astype(np.float64) @ W.astype(np.float64).T).astype(np.int64).astype(np.int32)
    cd = dev(orc.transpose_tile(codes)) if tiled else dev(codes)
    out = c_matmul_i8(dev(x), cd, dev(cb), tiled)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)
    # a few rows against the integer oracle itself
    rows = np.r_[0:2, M - 2:M]
    assert np.array_equal(out.cpu().numpy()[rows], orc.decode_matmul_i32(x[rows], codes, cb))


def test_integer_operator_golden_cases_and_edges():
    case = np.load(os.path.join(GOLDEN_DIR, "int8_case.npz"))
    x, codes, yi, cb = case["x"], case["codes"], case["y"], case["codebook_abs"]
    out = c_matmul_i8(dev(x), dev(orc.transpose_tile(codes)), dev(cb), True)
    assert np.array_equal(out.cpu().numpy(), yi)
    g = json.load(open(os.path.join(GOLDEN_DIR, "golden.json")))["int8_case"]
    xs = np.array(g["x"], dtype=np.int8).reshape(g["M"], g["K"])
    cs = np.array(g["codes"], dtype=np.int16).reshape(g["N"], g["K"] // 8)
    out = c_matmul_i8(dev(xs), dev(cs), dev(cb), False)
    assert out.cpu().numpy().reshape(-1).tolist() == g["y"]
    # extremes: every product at its largest magnitude (x = -128, table byte -128 flipped stays -128)
    cbx = np.frombuffer(bytes([0x80] * 8 * 256), dtype=np.int64).copy()
    xe = np.full((2, 64), -128, dtype=np.int8)
    ce = np.array([[0x0000, 0x8000, 0x7F00, 0xFFFF, 0x0100, 0x8100, 0x00FF, 0x80FF]] * 16, dtype=np.uint16).view(np.int16)
    out = c_matmul_i8(dev(xe), dev(ce), dev(cbx), False)
    assert np.array_equal(out.cpu().numpy(), orc.decode_matmul_i32(xe, ce, cbx))
    # K == 0 gives zeros; M == 0 or N == 0 is a no-op
    z = torch.full((3, 16), 7, dtype=torch.int32, device=DEV)
    st = capi.lib().dmm_decode_matmul_i8(None, None, dev(cb).data_ptr(), z.data_ptr(), 3, 16, 0, 1, None)
    torch.cuda.synchronize()
    assert st == 0 and torch.all(z == 0)


# ----------------------------------------------------------------- full benchmark sizes
FULL = [(1, N, K) for (K, N) in workload.LLAMA2_70B + workload.LLAMA2_7B] + \
       [(M, N, K) for M in (4, 8, 16, 32) for (K, N) in workload.SMALL_BATCH] + \
       [(2048, 4096, 4096), (2048, 11008, 4096), (2048, 4096, 11008)]


@pytest.mark.parametrize("M,N,K", FULL)
def test_full_size_against_decode_then_fp32_matmul(M, N, K):
    """At the benchmark's sizes: W from the decode kernel is bit-exact against the oracle's
    numpy decode, and the fused operator matches (x.float() @ W.float().T) * scale computed
    by the library GEMM on the GPU in fp32, within the operator's tolerance."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=0)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    W = c_decode(cd, gd)
    y = c_matmul(xd, cd, gd, scale, "auto")
    torch.cuda.synchronize()
    want_W = orc.decode_f16(codes.numpy(), grid.numpy())
    assert np.array_equal(bits(W), bits(want_W))
    ref = (xd.float() @ W.float().T) * scale
    assert_close_to_oracle(y, ref.cpu().numpy(), "full M=%d N=%d K=%d" % (M, N, K))
    # linearity in x: y(2x) == 2 y(x) up to the last place (a power-of-two scaling changes
    # no rounding except in the subnormal range)
    y2 = c_matmul(xd * 2, cd, gd, scale, "auto")
    torch.cuda.synchronize()
    assert torch.allclose(y2.float(), 2 * y.float(), rtol=2e-3, atol=1e-3)


@pytest.mark.parametrize("K,N", workload.SMALL_BATCH)
@pytest.mark.parametrize("M", [32, 48, 96])
def test_full_size_m32_through_the_workspace_entry(K, N, M):
    """M = 32 at the small-batch shapes the way the benchmark calls them: through
    dmm_decode_matmul_ws_f16 with the workspace dmm_workspace_bytes asks for - none at 32 rows on
    these 11 MB code matrices (two passes of the small-batch kernel), split-K at 96 rows."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=0)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    y, want = c_matmul_ws(xd, cd, gd, scale)
    assert want == 0 if M == 32 else want > 0 if M == 96 else True   # 48 rows: either, by the cost estimate
    W = c_decode(cd, gd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(W), bits(orc.decode_f16(codes.numpy(), grid.numpy())))
    ref = (xd.float() @ W.float().T) * scale
    assert_close_to_oracle(y, ref.cpu().numpy(), "full, workspace, M=32 N=%d K=%d" % (N, K))


@pytest.mark.parametrize("M,N,K", [(40, 256, 512), (130, 260, 1024), (33, 64, 64)])
def test_matrix_matrix_with_y_only_2_byte_aligned(M, N, K):
    """x, codes and grid 16-byte aligned (so the register-operand MFMA kernel runs), y at an odd
    2-byte offset: the kernel must fall back to 2-byte stores and stay inside y."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=M)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    buf = torch.full((M * N + 64,), -7.0, dtype=torch.float16, device=DEV)
    y = buf[17:17 + M * N].view(M, N)
    assert y.data_ptr() % 8 == 2
    for path in ("gemm", "auto"):
        buf.fill_(-7.0)
        c_matmul(dev(x), dev(codes), dev(grid), scale, path, out=y)
        torch.cuda.synchronize()
        assert_close_to_oracle(y, ref, "y misaligned, %s" % path)
        assert torch.all(buf[:17] == -7.0) and torch.all(buf[17 + M * N:] == -7.0)


# ----------------------------------------------------------------- small-batch kernel, row blocks
@pytest.mark.parametrize("M,K", [(8, 4096), (16, 4096), (3, 28672), (12, 1024 * 5), (2, 28672), (5, 16384), (9, 8192),
                                 (4, 4096), (4, 3328)])
@pytest.mark.parametrize("share", [1, 2, 3, 4, 5, 7, 8, 9, 11])
def test_small_batch_row_block_sizes(M, K, share, request):
    """The register-x kernel takes one to four row tiles per block, chosen from the most tiles
    a workgroup gets (`share`): every choice, with workgroups whose last block is partial and
    an N that is no multiple of 16; and every width of the x slice it moves through the LDS (up
    to 4, 8 and 16 rows of x, full and with rows to spare).  y lies between guard bands.
    Reference: the library's own decode (pinned bit for bit against the oracle above) times x
    in fp32 on the GPU, plus the oracle itself on the first and last rows."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    N = 16 * (cus * share - 37) - 4
    # up to eight rows of x on two to eight tiles per workgroup go to the 16-bit kernel with resident sums (every
    # share of tiles it is instantiated for comes by here as well); everything else in this list to the
    # register-x kernel
    resident = M <= 8 and share <= 8
    if M > 8:   # nine to sixteen rows would take that kernel too (up to eight tiles per workgroup): kept off here
        assert capi.lib().dmm_gemv_kernel_name(M, N, K) == (b"dmm::gemv_f16d_kernel" if share <= 8 else b"dmm::gemv_regx_kernel")
        request.addfinalizer(lambda was=capi.lib().dmm_set_choice(2, 0): capi.lib().dmm_set_choice(2, was))
    assert capi.lib().dmm_gemv_kernel_name(M, N, K) == (b"dmm::gemv_f16d_kernel" if resident else b"dmm::gemv_regx_kernel")
    x, _, grid, scale = workload.make_inputs(M, 8, K, seed=share)
    g = torch.Generator(device=DEV)
    g.manual_seed(1000 * M + share)
    codes = torch.randint(-32768, 32768, (N, K // 8), generator=g, dtype=torch.int16, device=DEV)
    xd, gd = dev(x), dev(grid)
    buf = torch.full((64 + M * N + 64,), -7.0, dtype=torch.float16, device=DEV)
    y = buf[64:64 + M * N].view(M, N)
    c_matmul(xd, codes, gd, scale, "gemv", out=y)
    W = c_decode(codes, gd)
    torch.cuda.synchronize()
    assert torch.all(buf[:64] == -7.0) and torch.all(buf[64 + M * N:] == -7.0)
    ref = (xd.float() @ W.float().T) * scale
    assert_close_to_oracle(y, ref.cpu().numpy(), "regx M=%d N=%d K=%d" % (M, N, K))
    rows = torch.from_numpy(np.r_[0:24, N - 24:N]).to(DEV)
    want = orc.matmul_f32(x.numpy(), orc.decode_f16(codes[rows].cpu().numpy(), grid.numpy()), scale)
    assert_close_to_oracle(y[:, rows], want, "regx M=%d N=%d K=%d, oracle rows" % (M, N, K))


@pytest.mark.parametrize("M,N,K", [(17, 4112, 8192), (24, 2052, 28672), (32, 8200, 4096), (31, 11008, 4096),
                                   (20, 500, 2304), (48, 1028, 4096), (64, 4096, 11008), (100, 2052, 8192),
                                   (128, 4112, 4096), (33, 16 * 300 - 4, 28672)])
def test_more_than_16_rows_of_x_in_passes(M, N, K, request):
    """More than 16 rows of x go through the small-batch kernel 16 at a time inside one launch
    (every workgroup walks its row blocks once per 16 rows); beyond 32 rows the operator takes
    that route where it beats the matrix-matrix kernel, as on these shapes.  Same tolerance, y
    between guard bands, a last pass with rows to spare.  (The kernel with resident sums, which
    would serve some of these shapes up to 32 rows, is kept off.)"""
    request.addfinalizer(lambda was=capi.lib().dmm_set_choice(2, 0): capi.lib().dmm_set_choice(2, was))
    x, _, grid, scale = workload.make_inputs(M, 8, K, seed=M)
    g = torch.Generator(device=DEV)
    g.manual_seed(M * 31 + 5)
    codes = torch.randint(-32768, 32768, (N, K // 8), generator=g, dtype=torch.int16, device=DEV)
    xd, gd = dev(x), dev(grid)
    buf = torch.full((64 + M * N + 64,), -7.0, dtype=torch.float16, device=DEV)
    y = buf[64:64 + M * N].view(M, N)
    c_matmul(xd, codes, gd, scale, "gemv" if M <= 32 else "auto", out=y)
    W = c_decode(codes, gd)
    torch.cuda.synchronize()
    assert torch.all(buf[:64] == -7.0) and torch.all(buf[64 + M * N:] == -7.0)
    ref = (xd.float() @ W.float().T) * scale
    assert_close_to_oracle(y, ref.cpu().numpy(), "passes M=%d N=%d K=%d" % (M, N, K))
    rows = torch.from_numpy(np.r_[0:24, N - 24:N]).to(DEV)
    want = orc.matmul_f32(x.numpy(), orc.decode_f16(codes[rows].cpu().numpy(), grid.numpy()), scale)
    assert_close_to_oracle(y[:, rows], want, "passes M=%d N=%d K=%d, oracle rows" % (M, N, K))
    # rows 16 p .. of x as a call of their own on the same kernel give the same bits
    if M <= 32 and capi.lib().dmm_gemv_kernel_name(M - 16, N, K) == b"dmm::gemv_regx_kernel":
        y1 = c_matmul(xd[16:].contiguous(), codes, gd, scale, "gemv")
        torch.cuda.synchronize()
        assert torch.equal(y[16:], y1)
    # packed codes take the same route and give the same bits
    packed = torch.empty(capi.lib().dmm_packed_bytes(N, K), dtype=torch.uint8, device=DEV)
    capi.check("dmm_pack_codes", capi.lib().dmm_pack_codes(codes.data_ptr(), packed.data_ptr(), N, K,
                                                           torch.cuda.current_stream().cuda_stream))
    y2 = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    capi.check("dmm_decode_matmul_packed_f16",
               capi.lib().dmm_decode_matmul_packed_f16(xd.data_ptr(), packed.data_ptr(), gd.data_ptr(), float(scale),
                                                       y2.data_ptr(), M, N, K, None, 0,
                                                       torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(y2, y)


# ----------------------------------------------------------------- seeded random shapes
def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        M = int(rng.choice([1, 1, 2, 3, 5, 8, 13, 16, 17, 24, 32, 33, 47, 64, 100, 129, 200]))
        K = int(rng.choice([8, 24, 64, 72, 256, 320, 512, 1000, 1024, 2048, 2304, 4096]))
        N = int(rng.choice([1, 3, 4, 15, 16, 17, 36, 64, 100, 255, 256, 257, 500, 1024, 1500]))
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("M,N,K", _random_shapes(16, 77))
def test_random_shapes_with_2_byte_aligned_buffers(M, N, K):
    """x, codes and y at addresses that are only 2-byte aligned: the dispatcher must fall back
    to kernels without alignment demands, never fault, never write outside y."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=M + N + K)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)

    def odd(t):   # same values, storage shifted by one element (2 bytes)
        flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)
        flat[1:] = t.reshape(-1).to(DEV)
        return flat[1:].view(t.shape)
    xd, cd, gd = odd(x), odd(codes), dev(grid)
    guard = 63
    buf = torch.full((M * N + 2 * guard,), 777.0, dtype=torch.float16, device=DEV)
    y = buf[guard:guard + M * N].view(M, N)
    assert xd.data_ptr() % 4 == 2 and cd.data_ptr() % 4 == 2 and y.data_ptr() % 4 == 2
    c_matmul(xd, cd, gd, scale, "auto", out=y)
    torch.cuda.synchronize()
    assert_close_to_oracle(y, ref, "unaligned M=%d N=%d K=%d" % (M, N, K))
    assert torch.all(buf[:guard] == 777.0) and torch.all(buf[guard + M * N:] == 777.0)


@pytest.mark.parametrize("M,N,K", _random_shapes(48, 2024))
def test_random_shapes_dispatch(M, N, K):
    """Whatever the dispatcher picks for a shape (any of the kernels, with and without a
    workspace), the result is the oracle's within tolerance and nothing outside y is written."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=M * 7 + N * 3 + K)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    # y inside a guarded buffer: the halves before and after it must keep their pattern
    guard = 64
    buf = torch.full((M * N + 2 * guard,), 777.0, dtype=torch.float16, device=DEV)
    y = buf[guard:guard + M * N].view(M, N)
    c_matmul(xd, cd, gd, scale, "auto", out=y)
    torch.cuda.synchronize()
    assert_close_to_oracle(y, ref, "auto M=%d N=%d K=%d" % (M, N, K))
    assert torch.all(buf[:guard] == 777.0) and torch.all(buf[guard + M * N:] == 777.0)
    y_w, _ = c_matmul_ws(xd, cd, gd, scale)
    torch.cuda.synchronize()
    assert_close_to_oracle(y_w, ref, "workspace M=%d N=%d K=%d" % (M, N, K))


# ----------------------------------------------------------------- packed codes
def pack_codes_numpy(codes):
    """The packed layout, restated with numpy index arithmetic: 16-bit unit
    ((tile * n_steps + step) * 64 + lane) * 8 + e holds codes[16 tile + lane % 16][32 step + 8 (lane // 16) + e]."""
    N, kc = codes.shape
    n_steps = kc // 32
    tiles = (N + 15) // 16
    padded = np.zeros((tiles * 16, kc), dtype=codes.dtype)
    padded[:N] = codes
    t = padded.reshape(tiles, 16, n_steps, 4, 8)          # [tile][row c16][step][q][e]
    return np.ascontiguousarray(t.transpose(0, 2, 3, 1, 4)).reshape(tiles * 16, kc)   # [tile][step][q][c16][e]


@pytest.mark.parametrize("M,N,K", [(1, 16, 256), (1, 100, 512), (1, 4096, 4096), (3, 1000, 2048), (1, 8192, 8192),
                                   (1, 1028, 28672), (4, 11008, 4096), (8, 52, 1024), (16, 52, 1024), (8, 4096, 11008),
                                   (32, 1000, 4096), (20, 36, 256)])
def test_packed_codes_bit_identical(M, N, K):
    """dmm_pack_codes produces the documented layout, and the operator on packed codes returns
    exactly the bits of the row-major call (same arithmetic, same order) - which is itself
    checked against the oracle."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=N + K)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    lib = capi.lib()
    nbytes = lib.dmm_packed_bytes(N, K)
    assert nbytes == (N + 15) // 16 * 16 * K // 4
    packed = torch.full((nbytes // 2,), -1, dtype=torch.int16, device=DEV)
    capi.check("dmm_pack_codes", lib.dmm_pack_codes(cd.data_ptr(), packed.data_ptr(), N, K, None))
    torch.cuda.synchronize()
    assert np.array_equal(packed.cpu().numpy().reshape(-1, K // 8), pack_codes_numpy(codes.numpy()))
    y_ref = c_matmul(xd, cd, gd, scale, "gemv")
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    capi.check("dmm_gemv_packed_f16", lib.dmm_gemv_packed_f16(xd.data_ptr(), packed.data_ptr(), gd.data_ptr(), scale,
                                                              y.data_ptr(), M, N, K, None))
    torch.cuda.synchronize()
    assert torch.equal(y, y_ref)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    assert_close_to_oracle(y, ref, "packed M=%d N=%d K=%d" % (M, N, K))
    # the PyTorch wrappers
    pk = dmm.pack_codes(cd)
    assert torch.equal(pk.reshape(-1), packed)
    # (the operators bring a workspace, so for 17 <= M they split K: compare like with like)
    assert torch.equal(dmm.decode_matmul_packed(xd, pk, gd, scale, N), dmm.decode_matmul(xd, cd, gd, scale))


@pytest.mark.parametrize("M,N,K", [(40, 300, 512), (64, 1024, 1024), (200, 771, 2304), (2048, 4096, 4096),
                                   (130, 52, 256), (33, 4100, 1024)])
def test_packed_codes_matrix_matrix_bit_identical(M, N, K):
    """The operator on packed codes for many rows of x (the MFMA kernel, or passes of the
    small-batch kernel where those are cheaper), with and without a split-K workspace: the
    bits of the row-major calls that take the same route."""
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=N + K + M)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    lib = capi.lib()
    pk = dmm.pack_codes(cd)
    stream = torch.cuda.current_stream().cuda_stream
    y_ref = c_matmul(xd, cd, gd, scale, "auto")
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    capi.check("dmm_decode_matmul_packed_f16",
               lib.dmm_decode_matmul_packed_f16(xd.data_ptr(), pk.data_ptr(), gd.data_ptr(), scale, y.data_ptr(),
                                                M, N, K, None, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(y, y_ref)
    y_ws_ref, want = c_matmul_ws(xd, cd, gd, scale)
    ws = torch.empty(max(want, 16), dtype=torch.uint8, device=DEV)
    y2 = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    capi.check("dmm_decode_matmul_packed_f16",
               lib.dmm_decode_matmul_packed_f16(xd.data_ptr(), pk.data_ptr(), gd.data_ptr(), scale, y2.data_ptr(),
                                                M, N, K, ws.data_ptr(), want, stream))
    torch.cuda.synchronize()
    assert torch.equal(y2, y_ws_ref)
    assert torch.equal(dmm.decode_matmul_packed(xd, pk, gd, scale, N), y_ws_ref)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    assert_close_to_oracle(y, ref, "packed gemm M=%d N=%d K=%d" % (M, N, K))


# ----------------------------------------------------------------- split-K with a workspace
def c_matmul_ws(x, codes, grid, scale, ws_bytes=None):
    M, K = x.shape
    N = codes.shape[0]
    want = capi.lib().dmm_workspace_bytes(M, N, K)
    nbytes = want if ws_bytes is None else ws_bytes
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=x.device)
    st = capi.lib().dmm_decode_matmul_ws_f16(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), float(scale),
                                             y.data_ptr(), M, N, K, ws.data_ptr(), nbytes,
                                             torch.cuda.current_stream().cuda_stream)
    capi.check("dmm_decode_matmul_ws_f16", st)
    return y, want


@pytest.mark.parametrize("M,N,K", [(17, 512, 1088), (32, 1000, 2112), (24, 28672, 2560), (33, 514, 4096), (64, 256, 8192),
                                   (100, 771, 1088), (200, 2048, 2048), (48, 4096, 512)])
def test_split_k_workspace_path(M, N, K, request):
    """Short x with a workspace: K is split over several blocks per tile, fp32 partial sums
    are added in a fixed order.  Same tolerance as every other path, same bits run after run,
    also with a workspace too small for the preferred split, and the PyTorch operator (which
    brings its own workspace) returns the same tensor.  The split is asked for: on the third shape
    the operator's own choice is the matrix-vector kernel for up to 32 rows."""
    request.addfinalizer(lambda was=capi.lib().dmm_set_choice(0, 2): capi.lib().dmm_set_choice(0, was))
    x, codes, grid, scale = workload.make_inputs(M, N, K, seed=M + N)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
    y, want = c_matmul_ws(xd, cd, gd, scale)
    torch.cuda.synchronize()
    assert want >= 2 * M * N * 4, "this shape is meant to split"
    assert_close_to_oracle(y, ref, "split-K M=%d N=%d K=%d" % (M, N, K))
    y2, _ = c_matmul_ws(xd, cd, gd, scale)
    assert torch.equal(y, y2)
    y3, _ = c_matmul_ws(xd, cd, gd, scale, ws_bytes=2 * M * N * 4 + 64)     # room for two splits only
    assert_close_to_oracle(y3, ref, "split-K, small workspace")
    y4, _ = c_matmul_ws(xd, cd, gd, scale, ws_bytes=M * N * 4)              # too small to split: plain path
    assert_close_to_oracle(y4, ref, "split-K, workspace too small")
    assert torch.equal(dmm.decode_matmul(xd, cd, gd, scale), y)


def test_split_k_integer_bridge_is_exact():
    rng = np.random.default_rng(5)
    M, N, K = 40, 256, 8192
    cb = orc.build_codebook_abs()
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    yi = orc.decode_matmul_i32(x, codes, cb)
    scale = 2.0 ** -8
    want = (yi.astype(np.float64) / 4 * scale).astype(np.float16)
    y, wsb = c_matmul_ws(dev(x.astype(np.float16)), dev(codes), dev(orc.grid_from_codebook(cb)), scale)
    torch.cuda.synchronize()
    assert wsb > 0 and np.array_equal(bits(y), bits(want))


def test_forced_kernel_choices_give_the_same_results():
    """dmm_set_choice (the benchmark's check of the dispatch) forces a kernel, never a result: the integer
    operator is exact either way, the half-precision operator on the integer bridge too (every route's
    sums are exact there), and a forced kernel that cannot take a call leaves it to the library."""
    lib = capi.lib()
    rng = np.random.default_rng(77)
    cb = orc.build_codebook_abs()
    M, N, K = 40, 272, 1024
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    yi = orc.decode_matmul_i32(x, codes, cb)
    try:
        for value in (-1, 1, 2):
            assert lib.dmm_set_choice(1, value) >= -1
            out = c_matmul_i8(dev(x), dev(codes), dev(cb), False)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy(), yi), value
        scale = 2.0 ** -8
        want = (yi.astype(np.float64) / 4 * scale).astype(np.float16)
        xd, cd, gd = dev(x.astype(np.float16)), dev(codes), dev(orc.grid_from_codebook(cb))
        for value in (-1, 0, 1, 2):
            assert lib.dmm_set_choice(0, value) >= -1
            y, _ = c_matmul_ws(xd, cd, gd, scale)
            torch.cuda.synchronize()
            assert np.array_equal(bits(y), bits(want)), value
            y1 = c_matmul(xd[:1].contiguous(), cd, gd, scale, "auto")     # one row: the override does not apply
            torch.cuda.synchronize()
            assert np.array_equal(bits(y1), bits(want[:1])), value
    finally:
        lib.dmm_set_choice(0, -1)
        lib.dmm_set_choice(1, -1)


# ----------------------------------------------------------------- maximum sizes
def _sampled_rows_check(M, N, K, path, seed):
    """A code matrix too large to decode whole: run the operator on all of it, then check a
    sample of output columns (first, last and random rows of W, i.e. the lowest and highest
    byte offsets) against the oracle on just those rows."""
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    codes = torch.randint(-32768, 32768, (N, K // 8), generator=g, dtype=torch.int16, device=DEV)
    x, _, grid, scale = workload.make_inputs(M, 8, K, seed=seed)
    y = c_matmul(dev(x), codes, dev(grid), scale, path)
    torch.cuda.synchronize()
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([np.arange(40), np.arange(N - 72, N), rng.integers(0, N, size=64)]))
    sub = codes[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    want = orc.matmul_f32(x.numpy(), orc.decode_f16(sub, grid.numpy()), scale)
    got = y[:, torch.from_numpy(rows).to(DEV)]
    assert_close_to_oracle(got, want, "%s M=%d N=%d K=%d sampled rows" % (path, M, N, K))
    assert not torch.isnan(y).any()
    del codes, y
    torch.cuda.empty_cache()


def test_code_matrix_just_below_2_gib_streams():
    """N * K / 4 = 2^31 - 512 KiB: the largest code matrix the kernels with 31-bit buffer
    offsets address."""
    _sampled_rows_check(1, 524160, 16384, "gemv", 71)      # streaming kernel
    _sampled_rows_check(20, 524160, 16384, "gemv", 74)     # small-batch kernel
    _sampled_rows_check(40, 524160, 16384, "gemm", 75)     # register-operand matrix-matrix kernel


def test_code_matrix_above_2_gib_takes_the_64_bit_path():
    """N * K / 4 just above 2^31 bytes: the dispatcher must leave the kernels with 31-bit
    offsets (the explicit matrix-vector entry point refuses) and still be right."""
    M, N, K = 3, 524544, 16384
    p = ctypes_null_call_gemv(M, N, K)
    assert p == -5
    _sampled_rows_check(M, N, K, "auto", 72)
    _sampled_rows_check(40, N, K, "gemm", 73)


def ctypes_null_call_gemv(M, N, K):
    """Status of dmm_gemv_f16 for a shape, with dummy (never dereferenced: the call is refused
    on the host) but aligned non-null pointers."""
    buf = torch.empty(64, dtype=torch.float16, device=DEV)
    ptr = buf.data_ptr()
    return capi.lib().dmm_gemv_f16(ptr, ptr, ptr, 1.0, ptr, M, N, K, None)


def test_repeatable_and_stream_ordered():
    """Same inputs -> same bits, run after run (no atomics, no races), also on a side stream
    while the default stream is busy."""
    x, codes, grid, scale = workload.make_inputs(4, 8192, 8192, seed=5)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    first = c_matmul(xd, cd, gd, scale, "auto")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    for _ in range(5):
        with torch.cuda.stream(side):
            again = dmm.decode_matmul(xd, cd, gd, scale)
        side.synchronize()
        assert torch.equal(first, again)


def test_graph_capture_and_replay():
    """The entry points only enqueue kernels (no allocation, no synchronisation), so a decode
    step can be captured in a HIP graph.  Every replay is checked against the eager result,
    with eager work and synchronisations between the replays, after x has been changed in
    place (a replay must read the current contents of its buffers)."""
    shapes = [(1, 1024, 4096), (1, 4096, 1024), (8, 512, 2048), (160, 384, 512),
              (1, 16384, 512), (3, 16400, 768),      # the 8-bit kernel, and three rows on the 16-bit kernel with resident sums
              (12, 4800, 5120)]                      # the register-x kernel
    probs = []
    for i, (M, N, K) in enumerate(shapes):
        x, codes, grid, scale = workload.make_inputs(M, N, K, seed=40 + i)
        probs.append([dev(x), dev(codes), dev(grid), scale, torch.empty(M, N, dtype=torch.float16, device=DEV)])
    W = torch.empty(shapes[0][1], shapes[0][2], dtype=torch.float16, device=DEV)

    def step():
        for xd, cd, gd, scale, y in probs:
            c_matmul(xd, cd, gd, scale, "auto", out=y)
        c_decode(probs[0][1], probs[0][2], out=W)

    assert capi.lib().dmm_init(-1) == 0     # the once-per-device host work, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for p in probs:
            p[0].mul_(-0.5 if rep else 1.0)  # eager work between replays, changes the input
        torch.cuda.synchronize()
        for p in probs:
            p[4].fill_(float("nan"))
        W.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [p[4].clone() for p in probs] + [W.clone()]
        step()                               # eager, same buffers
        torch.cuda.synchronize()
        want = [p[4] for p in probs] + [W]
        for g, w in zip(got, want):
            assert torch.equal(g, w), rep


def test_reference_call_under_the_reference_name():
    """`decode_matmul(x int8, weights_compressed int16 tiled, codebook_abs int64) -> int32`, the
    reference's three-argument call (test_decode_matmul.py:136), works under the reference's
    function name, also through a module alias as `from decode_matmul_cuda import decode_matmul`."""
    import sys
    M, N, K = 8, 16, 4096                        # the reference's own test shape
    rng = np.random.default_rng(5)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    codes = rng.integers(-32768, 32768, size=(N, K // 8), dtype=np.int16)
    cb = orc.build_codebook_abs()
    want = orc.decode_matmul_i32(x, codes, cb)
    sys.modules.setdefault("decode_matmul_cuda", dmm)
    from decode_matmul_cuda import decode_matmul
    tiled = dmm.transpose_tile(torch.from_numpy(codes))
    out = decode_matmul(dev(torch.from_numpy(x)), dev(tiled), dev(torch.from_numpy(cb)))
    torch.cuda.synchronize()
    assert out.dtype == torch.int32 and np.array_equal(out.cpu().numpy(), want)
    with pytest.raises(TypeError):
        decode_matmul(dev(torch.from_numpy(x)), dev(tiled), dev(torch.from_numpy(cb)), 0.5)
    xh, ch, gh, scale = workload.make_inputs(1, 64, 512, seed=9)
    with pytest.raises(TypeError):
        decode_matmul(dev(xh), dev(ch), dev(gh))     # the half-precision form needs its scale


@pytest.mark.parametrize("M", [1, 4])
def test_projections_sharing_x_are_one_call_on_concatenated_rows(M):
    """Several projections of the same activations (gate and up of a Llama-2-7B MLP, 4096 -> 2 x 11008)
    need no grouped entry point: rows of W are independent, so one call on the concatenated code rows
    gives, row for row, what the separate calls give - bit for bit when both run the same kernel
    (they do here), and the oracle's product within the operator's tolerance."""
    K, N1 = 4096, 11008
    x, gate, grid, scale = workload.make_inputs(M, N1, K, seed=21)
    _, up, _, _ = workload.make_inputs(M, N1, K, seed=22)
    xd, gd = dev(x), dev(grid)
    both = torch.cat([dev(gate), dev(up)], dim=0).contiguous()
    y_cat = c_matmul(xd, both, gd, scale, "auto")
    y_gate = c_matmul(xd, dev(gate), gd, scale, "auto")
    y_up = c_matmul(xd, dev(up), gd, scale, "auto")
    torch.cuda.synchronize()
    lib = capi.lib()
    assert lib.dmm_gemv_kernel_name(M, N1, K) == lib.dmm_gemv_kernel_name(M, 2 * N1, K)
    assert torch.equal(y_cat[:, :N1], y_gate) and torch.equal(y_cat[:, N1:], y_up)
    for codes, y in ((gate, y_gate), (up, y_up)):
        ref = orc.matmul_f32(x.numpy(), orc.decode_f16(codes.numpy(), grid.numpy()), scale)
        assert_close_to_oracle(y, ref, "projection sharing x, M=%d" % M)


def test_kernel_event_hook_times_the_kernel():
    x, codes, grid, scale = workload.make_inputs(1, 8192, 8192, seed=2)
    xd, cd, gd = dev(x), dev(codes), dev(grid)
    y0 = c_matmul(xd, cd, gd, scale)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(); stop.record()                # materialise the handles
    torch.cuda.synchronize()
    lib = capi.lib()
    assert lib.dmm_set_kernel_events(start.cuda_event, stop.cuda_event) == 0
    try:
        y1 = c_matmul(xd, cd, gd, scale)
        torch.cuda.synchronize()
        ms = start.elapsed_time(stop)
    finally:
        assert lib.dmm_set_kernel_events(None, None) == 0
    assert torch.equal(y0, y1)
    assert 0.0 < ms < 5.0
