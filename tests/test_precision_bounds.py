"""The 1e-3 contract of the GEMM and attention gradients would also pass a matrix path that narrows its operands; the GPU
tests therefore assert a second, tighter bound that only full-fp32 products and sums meet (oracle_lib.fp32_gemm_bound,
FP32_ATTENTION_BOUND).  This file shows on the CPU that the bound does what it is for: an fp32 computation passes it,
the same computation with an operand cut to tf32 or bf16 mantissa width fails it while still passing 1e-3."""
import numpy as np
import pytest

from oracle_lib import FP32_ATTENTION_BOUND, fp32_gemm_bound, narrow_mantissa, rel_fro


@pytest.mark.parametrize("m,n,k", [(64, 128, 784), (256, 256, 64), (300, 260, 1028), (128, 128, 4096)])
def test_gemm_bound_separates_fp32_from_narrowed_operands(oracle, m, n, k):
    rng = np.random.default_rng(k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    bound = fp32_gemm_bound(k)
    assert rel_fro(a @ b, want) <= bound                              # fp32, blocked sums
    if m * n * k <= 2 ** 25:
        assert rel_fro(oracle.matmul(a, b), want) <= bound            # fp32, the reference's sequential sum
    for bits in (10, 7):
        err = rel_fro(narrow_mantissa(a, bits).astype(np.float64) @ b.astype(np.float64), want)
        assert bound < err <= 1e-3 * (8 if bits == 7 else 1), (bits, err)


def test_attention_bound_separates_fp32_from_narrowed_operands(oracle):
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((2, 64, 64)).astype(np.float32) for _ in range(3))
    out, _, _ = oracle.sdpa_forward(q, k, v, 0.125)
    narrowed, _, _ = oracle.sdpa_forward(narrow_mantissa(q, 10), k, v, 0.125)
    sc = np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64)) * 0.125
    pr = np.exp(sc - sc.max(-1, keepdims=True))
    want = (pr / pr.sum(-1, keepdims=True)) @ v.astype(np.float64)
    assert rel_fro(out, want) <= FP32_ATTENTION_BOUND / 2
    assert FP32_ATTENTION_BOUND < rel_fro(narrowed, want) <= 1e-3
