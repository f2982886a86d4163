"""Writes tests/golden/closed_form.npz: small GEMM cases whose answers follow from arithmetic
alone, so they pin the oracle and the HIP path without trusting either.

The reference stores no golden vectors (its test draws unseeded random inputs,
kernels/tests/gemm_test.py:23-24), so these are derived from closed forms:

  identity   A = [I | 0]            -> C[m][n] = B[n][m]            (exact)
  ones       A = B = 1, K = 256     -> C = 256                      (exact in bf16/fp16)
  onehot     A has one 1 per row    -> C[m][n] = B[n][k(m)]         (exact)
  integers   entries in [-8, 8]     -> C = rne(exact integer sum)   (sum done in int64)

Inputs and outputs are stored as raw bit patterns (uint16 for bf16/fp16, uint8 for e4m3) under
keys "<case>/<dtype>/{A,B,C,scale}".  Bit patterns come from torch's dtype casts of exactly
representable values, and the integer sums from numpy int64 — neither touches oracle/ or the
HIP library.  Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

DT = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.float8_e4m3fn}
OUT = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.bfloat16}


def bits(t):
    return t.contiguous().view(torch.uint8 if t.element_size() == 1 else torch.int16).numpy().copy()


def cases(rng):
    M, N, K = 96, 80, 128
    for name, dt in DT.items():
        out_dt = OUT[name]
        scale = 0.5 if name == "e4m3" else 1.0

        def emit(case, a_int, b_int):
            a, b = torch.from_numpy(a_int).float(), torch.from_numpy(b_int).float()
            assert torch.equal(a.to(dt).float(), a) and torch.equal(b.to(dt).float(), b)
            exact = a_int.astype(np.int64) @ b_int.astype(np.int64).T  # exact integer sums
            c = (torch.from_numpy(exact).double() * scale).float()     # exact: |sum| < 2^24
            assert torch.equal(c.double(), torch.from_numpy(exact).double() * scale)
            yield f"{case}/{name}/A", bits(a.to(dt))
            yield f"{case}/{name}/B", bits(b.to(dt))
            yield f"{case}/{name}/C", bits(c.to(out_dt))
            yield f"{case}/{name}/scale", np.float32(scale)

        b_rand = rng.integers(-8, 9, size=(N, K))
        eye = np.zeros((M, K), dtype=np.int64)
        eye[np.arange(M), np.arange(M)] = 1
        yield from emit("identity", eye, b_rand)
        yield from emit("ones", np.ones((M, 256), dtype=np.int64), np.ones((N, 256), dtype=np.int64))
        hot = np.zeros((M, K), dtype=np.int64)
        hot[np.arange(M), rng.integers(0, K, size=M)] = 1
        yield from emit("onehot", hot, b_rand)
        yield from emit("integers", rng.integers(-8, 9, size=(M, K)), b_rand)


def main():
    rng = np.random.default_rng(20240607)
    data = dict(cases(rng))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "closed_form.npz")
    np.savez_compressed(path, **data)
    print(path, os.path.getsize(path), "bytes,", len(data), "arrays")


if __name__ == "__main__":
    main()
