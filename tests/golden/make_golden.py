"""Writes tests/golden/gemm_known_answers.json: small GEMM cases with their EXACT results.

The reference ships no golden vectors (its tests draw unseeded random inputs and compare with its own CPU loop,
matmul_test.h:289-302), so these are known answers computed independently of both the CPU oracle and the GPU
kernels: the inputs are 16-bit values, every product of two of them is exact in float64 and so is a sum of a few
hundred of them (at most 22 + 9 significant bits), hence numpy's float64 matrix product IS alpha * A * Bt^T +
beta * C over the reals for these sizes (alpha, beta and C are chosen exactly representable with few bits).
A sequential fp32 sum of n terms differs from the exact sum by at most (n - 1) * 2^-24 * sum(|terms|) to first order,
which is the bound the tests apply (they work it out from the inputs); integer-valued cases must match exactly.

    python tests/golden/make_golden.py      (numpy only; deterministic)
"""
import base64
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f64(b):
    return (b.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def b64(a):
    return base64.b64encode(np.ascontiguousarray(a).tobytes()).decode()


def case(name, dtype, M, N, K, alpha, beta, kind, rng):
    if kind == "uniform":
        a32 = rng.uniform(-1.0, 1.0, (M, K)).astype(np.float32)
        b32 = rng.uniform(-1.0, 1.0, (N, K)).astype(np.float32)
    else:  # small integers: every fp32 summation order gives the same value
        a32 = rng.integers(-3, 4, (M, K)).astype(np.float32)
        b32 = rng.integers(-3, 4, (N, K)).astype(np.float32)
    if dtype == "f16":
        a16, b16 = a32.astype(np.float16), b32.astype(np.float16)
        a64, b64v = a16.astype(np.float64), b16.astype(np.float64)
        abits, bbits = a16.view(np.uint16), b16.view(np.uint16)
    else:
        abits, bbits = f32_to_bf16_bits(a32), f32_to_bf16_bits(b32)
        a64, b64v = bf16_bits_to_f64(abits), bf16_bits_to_f64(bbits)
    c = (rng.integers(-8, 9, (M, N)) / 4.0).astype(np.float32)      # multiples of 1/4: exact everywhere
    exact = alpha * (a64 @ b64v.T) + beta * c.astype(np.float64)
    return {"name": name, "dtype": dtype, "M": M, "N": N, "K": K, "alpha": alpha, "beta": beta, "kind": kind,
            "a_bits_u16": b64(abits), "bt_bits_u16": b64(bbits), "c_f32": b64(c), "exact_f64": b64(exact)}


def main():
    rng = np.random.default_rng(20251125)
    cases = [
        case("fp16 uniform, one 64 tile with edges", "f16", 48, 40, 72, 1.0, 0.0, "uniform", rng),
        case("fp16 uniform, alpha and beta", "f16", 34, 24, 136, 1.5, -0.5, "uniform", rng),
        case("bf16 uniform, K not a multiple of 8", "bf16", 40, 33, 77, 1.0, 0.0, "uniform", rng),
        case("fp16 small integers", "f16", 32, 48, 128, 2.0, -1.0, "integers", rng),
        case("bf16 small integers, two tile rows of 64", "bf16", 130, 17, 96, 1.0, 0.0, "integers", rng),
    ]
    with open(os.path.join(HERE, "gemm_known_answers.json"), "w") as f:
        json.dump({"made_by": "tests/golden/make_golden.py", "cases": cases}, f)
    print("wrote %d cases" % len(cases))


if __name__ == "__main__":
    main()
