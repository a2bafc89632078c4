"""Pins the oracle's GEMM family: reference known-answer vectors, float64 closed form, invariants."""
import numpy as np
import pytest

from conftest import assert_close


def test_reference_known_answers(oracle, golden):
    for case in golden["gemm"]:
        out = oracle.gemm_f32(case["m"], case["n"], case["k"], case["lhs"], case["rhs"], scale=case["scale"],
                              lhs_transposed=case["lhs_transposed"])
        assert out.tolist() == case["expected"], case["source"]


def test_ones_case(oracle, golden):
    c = golden["gemm_ones"]
    lhs = np.full(c["m"] * c["k"], c["lhs_value"], np.float32)
    rhs = np.full(c["k"] * c["n"], c["rhs_value"], np.float32)
    assert (oracle.gemm_f32(c["m"], c["n"], c["k"], lhs, rhs) == c["expected_value"]).all()
    bias = np.full(c["n"], c["bias_value"], np.float32)
    fused = oracle.gemm_bias_act_f32(c["m"], c["n"], c["k"], oracle.ACT_RELU, lhs, rhs, bias)
    assert (fused == c["expected_bias_relu_value"]).all()


def test_epilogue_known_answers(oracle, golden):
    c = golden["gemm_epilogue"]
    args = (c["m"], c["n"], c["k"])
    assert oracle.gemm_bias_act_f32(*args, oracle.ACT_RELU, c["lhs"], c["rhs"], c["bias"]).tolist() == c["relu"]
    assert oracle.gemm_bias_act_f32(*args, oracle.ACT_RELU, c["lhs"], c["rhs"], c["bias"],
                                    c["residual"]).tolist() == c["residual_relu"]
    # GELU against the textbook tanh approximation evaluated in float64 (not the oracle's own formula).
    def gelu64(x):
        return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))
    for residual, pre in ((None, c["gelu_pre_activation"]), (c["residual"], c["residual_gelu_pre_activation"])):
        out = oracle.gemm_bias_act_f32(*args, oracle.ACT_GELU, c["lhs"], c["rhs"], c["bias"], residual)
        np.testing.assert_allclose(out, gelu64(np.array(pre, dtype=np.float64)), atol=2e-5, rtol=1e-6)


def test_zero_inner(oracle, golden):
    c = golden["gemm_zero_inner"]
    out = oracle.gemm_bias_act_f32(c["m"], c["n"], 0, oracle.ACT_RELU, [], [], c["bias"], c["residual"])
    assert out.tolist() == c["expected_relu"]


def test_generated_shapes_against_float64(oracle, golden):
    # Fill rule of the reference's own comparison (cpu_dense.rs:1054-1142): ((idx % 13) * 0.25) - 1.5 style.
    for m, k, n in golden["gemm_generated"]["shapes"]:
        lhs = (((np.arange(m * k) % 13) * 0.25) - 1.5).astype(np.float32)
        rhs = (((np.arange(k * n) % 7) * 0.5) - 1.0).astype(np.float32)
        want = lhs.reshape(m, k).astype(np.float64) @ rhs.reshape(k, n).astype(np.float64)
        assert_close(oracle.gemm_f32(m, n, k, lhs, rhs), want, 0, golden["gemm_generated"]["tolerance"],
                     f"gemm {m}x{k}x{n}")


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 5, 7), (33, 17, 65), (64, 64, 64), (5, 130, 9)])
def test_closed_form_and_transpose(oracle, m, n, k):
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert_close(oracle.gemm_f32(m, n, k, a, b), want, 1e-5, 1e-5, "plain")
    assert_close(oracle.gemm_f32(m, n, k, a, b, scale=-0.75), -0.75 * want, 1e-5, 1e-5, "scaled")
    # lhs stored transposed (k, m): a wrong index or a dropped transpose fails this.
    at = np.ascontiguousarray(a.T)
    assert (oracle.gemm_f32(m, n, k, at, b, lhs_transposed=True) == oracle.gemm_f32(m, n, k, a, b)).all()
    # identity and linearity invariants
    assert (oracle.gemm_f32(m, m, m, np.eye(m, dtype=np.float32), np.eye(m, dtype=np.float32)) ==
            np.eye(m, dtype=np.float32).ravel()).all()
    assert (oracle.gemm_f32(m, k, k, a, np.eye(k, dtype=np.float32)) == a.ravel()).all()


def test_sequential_order_and_separate_rounding(oracle):
    # 2^24 + 1 + 1 summed left to right in f32 stays 2^24 (each +1 is absorbed); a pairwise or
    # fused order would give 2^24 + 2.
    lhs = np.array([2.0 ** 24, 1.0, 1.0], np.float32)
    rhs = np.ones(3, np.float32)
    assert oracle.gemm_f32(1, 1, 3, lhs, rhs)[0] == np.float32(2.0 ** 24)
    # a*b - a*b with a*b inexact: separately rounded multiply gives exactly 0; an FMA would not.
    a = np.float32(1.0 + 2.0 ** -12)
    lhs = np.array([a, -a], np.float32)
    rhs = np.array([a, a], np.float32)
    assert oracle.gemm_f32(1, 1, 2, lhs, rhs)[0] == 0.0
    # scale is applied after the full sum
    assert oracle.gemm_f32(1, 1, 3, [2.0 ** 24, 1, 1], [1, 1, 1], scale=0.5)[0] == np.float32(2.0 ** 23)


def test_threads_do_not_change_values(oracle):
    rng = np.random.default_rng(7)
    a = rng.normal(size=(37, 53)).astype(np.float32)
    b = rng.normal(size=(53, 29)).astype(np.float32)
    assert (oracle.gemm_f32(37, 29, 53, a, b, threads=1) == oracle.gemm_f32(37, 29, 53, a, b, threads=4)).all()


def test_relu_semantics(oracle):
    # -0.0 and negative sums become +0.0 (value > 0 test), bias is indexed by column.
    out = oracle.gemm_bias_act_f32(2, 2, 1, oracle.ACT_RELU, [1, -1], [1, 2], [-1, 5])
    assert out.tolist() == [0.0, 7.0, 0.0, 3.0]
    assert not np.signbit(out).any()


def test_bf16_rounding_and_gemm(oracle):
    from spiraltorch_amd import inputs
    vals = np.array([1.0, 1.00390625, 1.01171875, -3.14159, 65504.0, 1e-40, np.inf], np.float32)
    bits = oracle.f32_to_bf16(vals)
    # ties to even: 1.00390625 = 1 + 2^-8 is exactly half-way between bf16(1.0) and the next -> even (1.0)
    assert bits[0] == 0x3F80 and bits[1] == 0x3F80
    # 1 + 3*2^-8 is half-way between 0x3F81 and 0x3F82 -> even (0x3F82)
    assert bits[2] == 0x3F82
    assert (bits == inputs.to_bf16(vals)).all()
    assert (oracle.bf16_to_f32(bits) == inputs.from_bf16(bits)).all()
    rng = np.random.default_rng(3)
    a = inputs.to_bf16(rng.normal(0, 0.02, (9, 40)).astype(np.float32))
    b = inputs.to_bf16(rng.normal(0, 0.02, (40, 11)).astype(np.float32))
    want = inputs.from_bf16(a).reshape(9, 40).astype(np.float64) @ inputs.from_bf16(b).reshape(40, 11).astype(np.float64)
    assert_close(oracle.gemm_bf16_f32acc(9, 11, 40, a, b), want, 1e-5, 1e-7, "bf16 gemm")


def test_packed_naive_blocks_are_the_sequential_sum(oracle):
    """matmul_naive_packed_row (pure.rs:11688-11758) adds the k products of a 4-column block strictly in order: on
    n % 4 == 0 it must agree bit for bit with the sequential GEMM, whatever the data."""
    rng = np.random.default_rng(5)
    m, n, k = 7, 12, 203
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    packed = np.ascontiguousarray(b.T)
    assert (oracle.gemm_f32_packed_naive(m, n, k, a, packed) == oracle.gemm_f32(m, n, k, a, b)).all()


def test_packed_naive_tail_columns_use_four_partial_sums(oracle):
    """dot_unrolled (pure.rs:11664-11686): with lhs = [2^24, 1, 1, 1, 1, 1, 1, 1, 1, 1] and a column of ones the
    sequential f32 sum stays at 2^24 (every +1 is lost), while four partial sums over k mod 4 give
    acc0 = 2^24 (+1 lost twice), acc1 = 3, acc2 = 2, acc3 = 2, then ((acc0 + acc1) + acc2) + acc3 = 2^24 + 7 -> the
    f32 neighbours are 2 apart: 2^24+3 -> 2^24+4 (ties to even), +2 -> 2^24+6, +2 -> 2^24+8."""
    k = 10
    lhs = np.ones(k, np.float32)
    lhs[0] = 2.0 ** 24
    for n in (1, 2, 3):  # every column is a tail column
        packed = np.ones((n, k), np.float32)
        out = oracle.gemm_f32_packed_naive(1, n, k, lhs, packed)
        assert out.tolist() == [2.0 ** 24 + 8] * n
        assert oracle.gemm_f32(1, n, k, lhs, np.ones((k, n), np.float32)).tolist() == [2.0 ** 24] * n
    # n = 5: the first four columns are a block (sequential), the fifth is a tail column
    out = oracle.gemm_f32_packed_naive(1, 5, k, lhs, np.ones((5, k), np.float32))
    assert out.tolist() == [2.0 ** 24] * 4 + [2.0 ** 24 + 8]


@pytest.mark.parametrize("m,n,k", [(3, 5, 7), (4, 7, 64), (2, 9, 131), (1, 3, 3)])
def test_packed_naive_against_float64(oracle, m, n, k):
    rng = np.random.default_rng(m + 10 * n + 100 * k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    got = oracle.gemm_f32_packed_naive(m, n, k, a, np.ascontiguousarray(b.T))
    assert_close(got, want, 1e-5, 1e-5, f"packed naive {m}x{n}x{k}")
    # and a transposed packing (k x n handed over as if it were n x k) must fail that check
    if n != k:
        wrong = oracle.gemm_f32_packed_naive(m, n, k, a, b)
        assert np.abs(wrong - want.ravel()).max() > 1e-3
