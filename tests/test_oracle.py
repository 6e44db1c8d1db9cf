"""Pins the CPU oracle (oracle/dmm_oracle.py, oracle/dmm_oracle.c) before anything is
checked against it.  No GPU.  Each check is chosen so that a plausible mistake (wrong bit
for a sign, parity on the wrong dim, shift sign inverted, add before flip, transposed
operand) fails it; none of them retypes the oracle's own formula."""
import hashlib
import json
import os
import subprocess
from fractions import Fraction

import numpy as np
import pytest

from conftest import GOLDEN_DIR, ORACLE_DIR, ptr, quarter_grid
from oracle import dmm_oracle as orc


# ----------------------------------------------------------------- literal scalar spec
def scalar_decode_i8(code, table_bytes):
    """One code -> 8 ints, written as the reference's scalar loop reads
    (/root/reference/test_decode_matmul.py:29-55): low byte picks the row; bits 8..14 are
    consumed LSB first as the signs of dims 0..6, then the parity bit for dim 7; a set top
    bit subtracts one, a clear one adds one."""
    bits_abs = code & 0xFF
    bits_sign = (code >> 8) & 0x7F
    bits_sign |= (bin(bits_sign).count("1") & 1) << 7
    bit_shift = (code >> 15) & 1
    out = []
    for i in range(8):
        value = int(table_bytes[bits_abs][i])
        if bits_sign & 1:
            value = -value
        value = value - 1 if bit_shift else value + 1
        out.append(value)
        bits_sign >>= 1
    return out


@pytest.fixture(scope="module")
def e8p():
    cb = orc.build_codebook_abs()
    return cb, orc.codebook_bytes(cb)


def test_decode_i8_exhaustive_vs_scalar_loop(all_codes, e8p):
    cb, tb = e8p
    got = orc.decode_i8(all_codes[:, None], cb)          # [65536, 8]
    tbl = tb.astype(int).tolist()
    want = np.array([scalar_decode_i8(int(c), tbl) for c in all_codes], dtype=np.int64)
    assert np.array_equal(got.astype(np.int64), want)


def test_swar_form_of_cuda_kernel_equals_spec(all_codes, e8p):
    # decode_matmul_cuda.cu:45-65 must be the same function as test_decode_matmul.py:29-55
    cb, _ = e8p
    packed = orc.decode_swar_u64(all_codes, cb)
    by = ((packed[:, None] >> (8 * np.arange(8, dtype=np.uint64))) & np.uint64(0xFF)).astype(np.uint8).view(np.int8)
    assert np.array_equal(by, orc.decode_i8(all_codes[:, None], cb))


def test_c_oracle_equals_numpy_oracle(all_codes, e8p, c_oracle):
    cb, _ = e8p
    cb = np.ascontiguousarray(cb)
    wi = np.empty((65536, 8), dtype=np.int8)
    c_oracle.dmm_oracle_decode_i8(ptr(all_codes), ptr(cb), ptr(wi), 65536)
    assert np.array_equal(wi, orc.decode_i8(all_codes[:, None], cb))
    sw = np.empty(65536, dtype=np.uint64)
    c_oracle.dmm_oracle_decode_swar(ptr(all_codes), ptr(cb), ptr(sw), 65536)
    assert np.array_equal(sw, orc.decode_swar_u64(all_codes, cb))
    for seed in (0, 1):
        grid = np.ascontiguousarray(quarter_grid(seed))
        wf = np.empty((65536, 8), dtype=np.float16)
        c_oracle.dmm_oracle_decode_f16(ptr(all_codes), ptr(grid.view(np.uint16)), ptr(wf.view(np.uint16)), 65536)
        assert np.array_equal(wf.view(np.uint16), orc.decode_f16(all_codes[:, None], grid).view(np.uint16))


def test_field_invariants(all_codes):
    idx, s8, shift = orc.code_fields(all_codes)
    # total number of flipped dims is always even (the 8th sign is the parity of the 7)
    pop = sum(((s8 >> d) & 1) for d in range(8))
    assert np.all(pop % 2 == 0)
    assert np.array_equal(idx, all_codes & 0xFF)
    assert np.array_equal(shift, all_codes >> 15)
    assert np.array_equal(s8 & 0x7F, (all_codes >> 8) & 0x7F)


def test_single_bit_semantics():
    """Known answers worked out by hand from test_decode_matmul.py:29-55 on a grid whose
    row r is [r+1, r+2, ...] quarters, so every dim and row is identifiable."""
    grid = (np.arange(256)[:, None] + np.arange(1, 9)[None, :]).astype(np.float16) / 4
    g5 = grid[5].astype(np.float32)
    def dec(c):
        return orc.decode_f16(np.array([[c]], dtype=np.uint16), grid)[0].astype(np.float32)
    assert np.array_equal(dec(0x0005), g5 + 0.25)                 # no flips, shift clear -> +1/4
    assert np.array_equal(dec(0x8005), g5 - 0.25)                 # top bit -> -1/4
    e = dec(0x0105)                                               # bit 8: dim 0 and, by parity, dim 7
    want = g5.copy(); want[0] = -want[0]; want[7] = -want[7]
    assert np.array_equal(e, want + 0.25)
    e = dec(0x4005)                                               # bit 14: dim 6 and dim 7
    want = g5.copy(); want[6] = -want[6]; want[7] = -want[7]
    assert np.array_equal(e, want + 0.25)
    e = dec(0x0305)                                               # bits 8,9: dims 0,1, even parity
    want = g5.copy(); want[0] = -want[0]; want[1] = -want[1]
    assert np.array_equal(e, want + 0.25)
    e = dec(0xFF05)                                               # all seven + parity(7)=1: all eight, shift -
    assert np.array_equal(e, -g5 - 0.25)


def test_f16_int8_bridge_exhaustive(all_codes, e8p):
    """fp16 decode == int8 decode / 4 exactly when the grid is the table's bytes / 4."""
    cb, _ = e8p
    grid = orc.grid_from_codebook(cb)
    wf = orc.decode_f16(all_codes[:, None], grid).astype(np.float32) * 4
    wi = orc.decode_i8(all_codes[:, None], cb).astype(np.float32)
    assert np.array_equal(wf, wi)


def test_signed_zero_and_flip_before_add():
    grid = np.zeros((256, 8), dtype=np.float16)
    grid[0] = 0.25
    grid[1] = [0.0, -0.0, 0.25, -0.25, 1.0, -1.0, 0.125, 3.0]
    # row 0, dim 0 flipped (and dim 7 by parity), shift +: -0.25 + 0.25 must be +0.0, not -0.0
    w = orc.decode_f16(np.array([[0x0100]], dtype=np.uint16), grid)[0]
    assert w.view(np.uint16)[0] == 0x0000 and w.view(np.uint16)[7] == 0x0000
    assert w[1] == np.float16(0.5)
    # flip first, then add: -(0.125) - 0.25 = -0.375 ; add-then-flip would give +0.125
    w = orc.decode_f16(np.array([[0xC001]], dtype=np.uint16), grid)[0]   # bit 14 -> dims 6,7 ; shift -
    assert w[6] == np.float16(-0.375) and w[7] == np.float16(-3.25)
    assert w[0] == np.float16(-0.25) and w[3] == np.float16(-0.5)


def test_half_add_rounding_against_exact_rationals():
    """Arbitrary half grids: the decode is ONE correctly rounded (nearest-even) half add.
    Checked against exact rational arithmetic over every finite half magnitude."""
    mags = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)          # all finite non-negative halves
    finite = np.concatenate([mags, -mags]).astype(np.float16)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    def rne_half(fr):
        # nearest finite half to the rational fr (ties to even mantissa), by bisection
        s = -1 if fr < 0 else 1
        a = abs(fr)
        hi = int(np.searchsorted(halves, float(a), side="left"))
        cands = [i for i in (hi - 1, hi, hi + 1) if 0 <= i < len(halves)]
        best = min(cands, key=lambda i: (abs(Fraction(float(halves[i])) - a), i & 1))
        return s * float(halves[best])
    rng = np.random.default_rng(7)
    pick = rng.choice(finite, size=256 * 8 - 64, replace=False)
    special = np.array([6.1e-5, 5.96e-8, 0.2498, 0.25, 0.2502, 1023.5, 2047.0, 2048.0, 4095.0, 0.124939,
                        1e-3, 0.37, 511.75, 1024.25, 3.0e-5, 65504.0] * 4, dtype=np.float16)
    grid = np.concatenate([pick, special]).reshape(256, 8).astype(np.float16)
    codes = np.arange(256, dtype=np.uint16)                                  # no flips, shift +
    for base, sign_all, delta in ((0x0000, 1, Fraction(1, 4)), (0x8000, 1, Fraction(-1, 4)),
                                  (0xFF00, -1, Fraction(-1, 4))):
        w = orc.decode_f16((codes | base)[:, None].astype(np.uint16), grid).astype(np.float64)
        for r in range(0, 256, 5):
            for d in range(8):
                exact = sign_all * Fraction(float(grid[r, d])) + delta
                if abs(exact) >= 65520:
                    continue
                assert w[r, d] == rne_half(exact), (r, d, grid[r, d], base)


def test_codebook_closed_form_properties(e8p):
    cb, tb = e8p
    assert cb.shape == (256,) and cb.dtype == np.int64
    rows = tb.astype(np.int32)                    # 4 * value
    assert len({tuple(r) for r in rows.tolist()}) == 256
    assert set(np.unique(tb.view(np.uint8)).tolist()) <= {2, 6, 10, 246, 250, 254}
    assert np.all(tb.view(np.uint8) % 4 == 2)     # what the XOR-0xFC negate of the CUDA kernel relies on
    assert np.all(rows[:, :7] > 0)                # negatives only in dim 7
    assert int((rows[:, 7] < 0).sum()) == 149
    norm2 = (rows.astype(np.int64) ** 2).sum(1) // 16
    hist = {int(k): int(v) for k, v in zip(*np.unique(norm2, return_counts=True))}
    assert hist == {2: 1, 4: 8, 6: 28, 8: 64, 10: 126, 12: 29}
    assert np.all(np.diff(norm2) >= 0)            # sorted by norm
    # every row has an even coordinate sum (in units of 1): the E8 condition the flip enforces
    assert np.all((rows.sum(1) // 4) % 2 == 0) and np.all(rows.sum(1) % 4 == 0)


def test_matmul_against_brute_force():
    rng = np.random.default_rng(3)
    M, N, K = 3, 5, 16
    x = rng.standard_normal((M, K)).astype(np.float16)
    grid = quarter_grid(3)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    W = orc.decode_f16(codes, grid)
    scale = 0.37
    want = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            for j in range(K // 8):
                wj = orc.decode_f16(codes[n:n + 1, j:j + 1], grid)[0]
                for d in range(8):                       # W[n, 8j+d], test_decode_matmul.py:65-69
                    want[m, n] += float(x[m, 8 * j + d]) * float(wj[d])
    got = orc.matmul_f32(x, W, scale)
    assert np.allclose(got, want * np.float32(scale), rtol=1e-6, atol=1e-6)
    # a transposed or mis-indexed W would not survive this asymmetric shape
    assert got.shape == (M, N)


def test_int_operator_and_bridge(c_oracle, e8p):
    """Integer operator vs C loop, and the exact integer<->half bridge: with x integer-valued
    and grid = bytes/4, scale a power of two, y_half == half(int32 / 4 * scale) exactly."""
    cb, _ = e8p
    cb = np.ascontiguousarray(cb)
    rng = np.random.default_rng(11)
    M, N, K = 8, 16, 256
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    codes = rng.integers(0, 65536, size=(N, K // 8)).astype(np.uint16)
    yi = orc.decode_matmul_i32(x, codes, cb)
    yc = np.empty((M, N), dtype=np.int32)
    c_oracle.dmm_oracle_decode_matmul_i32(ptr(x), ptr(codes), ptr(cb), ptr(yc), M, N, K)
    assert np.array_equal(yi, yc)
    grid = orc.grid_from_codebook(cb)
    scale = 2.0 ** -6
    yf = orc.decode_matmul_f16(x.astype(np.float16), codes, grid, scale)
    assert np.array_equal(yf, (yi.astype(np.float64) / 4 * scale).astype(np.float16))
    # C matmul agrees with numpy matmul
    W = np.ascontiguousarray(orc.decode_f16(codes, grid))
    xh = np.ascontiguousarray(x.astype(np.float16))
    yc32 = np.empty((M, N), dtype=np.float32)
    c_oracle.dmm_oracle_matmul_f16(ptr(xh.view(np.uint16)), ptr(W.view(np.uint16)), scale, ptr(yc32), M, N, K)
    assert np.array_equal(yc32, orc.matmul_f32(xh, W, scale))


def test_transpose_tile_lane_formula():
    """Lane 4g+c of the CUDA warp reads one 32-bit word = codes of rows g and g+8 at code
    column c of the tile (decode_matmul_cuda.cu:111-112, 137-138)."""
    N, Kc = 32, 16
    codes = (np.arange(N)[:, None] * 1000 + np.arange(Kc)[None, :]).astype(np.int16)
    tiled = orc.transpose_tile(codes).reshape(-1)
    tiles_k = Kc // 4
    for n_tile in range(N // 16):
        for k_tile in range(tiles_k):
            base = (n_tile * tiles_k + k_tile) * 64
            for lane in range(32):
                g, c = lane // 4, lane % 4
                assert tiled[base + 2 * lane] == codes[16 * n_tile + g, 4 * k_tile + c]
                assert tiled[base + 2 * lane + 1] == codes[16 * n_tile + g + 8, 4 * k_tile + c]
    assert np.array_equal(orc.untranspose_tile(orc.transpose_tile(codes)), codes)


def test_half_conversion_of_c_oracle(c_oracle):
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(f)
    back = np.array([c_oracle.dmm_oracle_f2h(float(v)) for v in f[finite][::7]], dtype=np.uint16)
    assert np.array_equal(back, h[finite][::7])
    rng = np.random.default_rng(5)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-8, 5, 4000),
                           np.array([65519.99, 65520.0, 2.0 ** -25, 2.0 ** -25 * 1.0001, 6.0e-8, 0.0, -0.0], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([c_oracle.dmm_oracle_f2h(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_c_oracle_sanitized():
    """The C oracle's own memory safety: address + undefined-behaviour sanitizers, host only."""
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, "oracle_asan"])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0")
    env.pop("LD_PRELOAD", None)
    out = subprocess.run([os.path.join(ORACLE_DIR, "oracle_asan")], env=env, capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "mismatches=0" in out.stdout


# ----------------------------------------------------------------- golden fixtures
def test_golden_fixtures_match_oracle(all_codes):
    with open(os.path.join(GOLDEN_DIR, "golden.json")) as f:
        gold = json.load(f)
    cb = orc.build_codebook_abs()
    assert [int(v) for v in cb] == gold["e8p_codebook_abs_int64"]
    grid = np.array(gold["decode_all_codes"]["grid_bits"], dtype=np.uint16).view(np.float16).reshape(256, 8)
    W = orc.decode_f16(all_codes[:, None], grid)
    assert hashlib.sha256(W.view(np.uint16).tobytes()).hexdigest() == gold["decode_all_codes"]["sha256_of_W_bits"]
    assert W.view(np.uint16)[:16].tolist() == gold["decode_all_codes"]["first16_rows_bits"]
    assert W.view(np.uint16)[-16:].tolist() == gold["decode_all_codes"]["last16_rows_bits"]
    case = gold["int8_case"]
    x = np.array(case["x"], dtype=np.int8).reshape(case["M"], case["K"])
    codes = np.array(case["codes"], dtype=np.int16).reshape(case["N"], case["K"] // 8)
    y = orc.decode_matmul_i32(x, codes, cb)
    assert y.reshape(-1).tolist() == case["y"]
