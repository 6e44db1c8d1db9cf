"""Writes the committed fixtures golden.json and int8_case.npz.

The reference stores no vectors of its own (its one test draws inputs from the CUDA RNG,
/root/reference/test_decode_matmul.py:95-96), so these are produced by this build's oracle
after tests/test_oracle.py has pinned it, and serve two purposes: they freeze the oracle
against accidental edits, and they give the GPU tests inputs with known outputs that do not
need the oracle to be re-run at full size.

    python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import dmm_oracle as orc  # noqa: E402


def main():
    gold = {}
    cb = orc.build_codebook_abs()
    gold["e8p_codebook_abs_int64"] = [int(v) for v in cb]

    rng = np.random.default_rng(20240)
    vals = np.array([0.25, 0.75, 1.25, 1.75, 2.25, 2.75], dtype=np.float16)
    grid = vals[rng.integers(0, 6, size=(256, 8))]
    codes = np.arange(65536, dtype=np.uint16)[:, None]
    W = orc.decode_f16(codes, grid).view(np.uint16)
    gold["decode_all_codes"] = {
        "note": "codes 0..65535 in order, one code per row; values are IEEE half bit patterns",
        "grid_bits": grid.view(np.uint16).reshape(-1).tolist(),
        "sha256_of_W_bits": hashlib.sha256(W.tobytes()).hexdigest(),
        "first16_rows_bits": W[:16].tolist(),
        "last16_rows_bits": W[-16:].tolist(),
    }

    # the reference's only validated shape (test_decode_matmul.py:126-137): M=8, N=16, K=4096
    M, N, K = 8, 16, 4096
    x = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    wc = rng.integers(-32768, 32768, size=(N, K // 8)).astype(np.int16)
    y = orc.decode_matmul_i32(x, wc, cb)
    np.savez_compressed(os.path.join(HERE, "int8_case.npz"), x=x, codes=wc, y=y, codebook_abs=cb)

    # a small copy of the same kind of case inline, readable without numpy
    Ms, Ns, Ks = 2, 3, 32
    xs = rng.integers(-128, 128, size=(Ms, Ks)).astype(np.int8)
    cs = rng.integers(-32768, 32768, size=(Ns, Ks // 8)).astype(np.int16)
    gold["int8_case"] = {
        "M": Ms, "N": Ns, "K": Ks,
        "x": xs.reshape(-1).tolist(),
        "codes": cs.reshape(-1).tolist(),
        "y": orc.decode_matmul_i32(xs, cs, cb).reshape(-1).tolist(),
    }
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(gold, f, indent=0, separators=(",", ":"))
    print("wrote golden.json, int8_case.npz")


if __name__ == "__main__":
    main()
