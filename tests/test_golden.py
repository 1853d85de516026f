"""Known answers of tests/golden/gemm_known_answers.json (exact results over the reals, computed by
tests/golden/make_golden.py independently of the oracle and of the kernels) against the CPU oracle and, on a GPU,
against every GEMM kernel design through the C ABI."""
import base64
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def load_cases():
    with open(os.path.join(HERE, "golden", "gemm_known_answers.json")) as f:
        doc = json.load(f)
    out = []
    for c in doc["cases"]:
        M, N, K = c["M"], c["N"], c["K"]
        dec = lambda key, dt, shape: np.frombuffer(base64.b64decode(c[key]), dtype=dt).reshape(shape).copy()
        out.append(dict(c, a=dec("a_bits_u16", np.uint16, (M, K)), bt=dec("bt_bits_u16", np.uint16, (N, K)),
                        c=dec("c_f32", np.float32, (M, N)), exact=dec("exact_f64", np.float64, (M, N))))
    return out


def as_f64(case, bits):
    if case["dtype"] == "f16":
        return bits.view(np.float16).astype(np.float64)
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


CASES = load_cases()


def check(case, got):
    err = np.abs(got.astype(np.float64) - case["exact"])
    if case["kind"] == "integers":
        assert np.array_equal(got.astype(np.float64), case["exact"]), case["name"]
    else:
        # what any fp32 summation order of K exact products can lose, plus the epilogue's roundings
        mag = abs(case["alpha"]) * (np.abs(as_f64(case, case["a"])) @ np.abs(as_f64(case, case["bt"])).T) + abs(case["beta"]) * np.abs(case["c"])
        bound = case["K"] * 2.0 ** -24 * mag + 2.0 ** -22 * np.abs(case["exact"])
        assert np.all(err <= bound), "%s: worst excess %g" % (case["name"], float((err - bound).max()))


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_reproduces_the_known_answers(oracle, case):
    odt = oracle.DT_F16 if case["dtype"] == "f16" else oracle.DT_BF16
    for blocked in (False, True):
        got = oracle.gemm(odt, case["a"], case["bt"], case["c"], case["alpha"], case["beta"], blocked=blocked)
        check(case, got)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_kernels_reproduce_the_known_answers(ck, case):
    from tests import gpu_util as G
    dt = ck.DT_F16 if case["dtype"] == "f16" else ck.DT_BF16
    a = case["a"].view(np.float16) if case["dtype"] == "f16" else case["a"]
    bt = case["bt"].view(np.float16) if case["dtype"] == "f16" else case["bt"]
    designs = [
        G.tuning(tile_dim=64, segment_dim_k=64, num_stages=3, num_producer_warps=2, num_consumer_warps=4),            # producer/consumer
        G.tuning(tile_dim=128, segment_dim_k=64, num_stages=2, num_producer_warps=4, num_consumer_warps=8),
        G.tuning(tile_dim=128, segment_dim_k=32, num_stages=4, num_producer_warps=0, num_consumer_warps=8),           # fused
        G.tuning(tile_dim=64, segment_dim_k=128, num_stages=1, num_producer_warps=0, num_consumer_warps=4),           # synchronous
        G.tuning(tile_dim=256, segment_dim_k=32, num_stages=5, num_producer_warps=0, num_consumer_warps=8),           # straight-line
    ]
    for t in designs:
        check(case, G.run_gemm(ck, dt, a, bt, case["c"], case["alpha"], case["beta"], t=t))
