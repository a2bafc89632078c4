"""Pins the oracle's tensor utilities (row softmax, GELU backward, scale, add_row, column sums) against the
reference's own test inputs and against float64 closed forms that a dropped term or a wrong index would fail."""
import numpy as np

from conftest import assert_close


def test_row_softmax_reference_input_matches_two_pass_float64(oracle, golden):
    c = golden["row_softmax"]
    x = np.array(c["input"], np.float64).reshape(c["rows"], c["cols"])
    want = np.exp(x - x.max(axis=1, keepdims=True))
    want /= want.sum(axis=1, keepdims=True)
    got = oracle.row_softmax_f32(c["rows"], c["cols"], c["input"])
    assert_close(got, want, 0, 1e-5, c["source"])
    assert_close(got.reshape(c["rows"], c["cols"]).sum(axis=1), np.ones(c["rows"]), 0, 1e-6, "row sums")


def test_row_softmax_edge_rows(oracle):
    nan, inf = float("nan"), float("inf")
    # NaN entries are skipped and get weight 0; a row of NaNs is all zero; +inf maximum -> base 0 -> weights
    # exp(v) with an infinite sum -> one-hot of the first maximum; tiny denominators cannot occur for finite rows.
    rows = [[1.0, nan, 3.0, 2.0], [nan, nan, nan, nan], [0.0, inf, 1.0, inf], [-1000.0, -1000.0, -1000.0, -1000.0]]
    got = oracle.row_softmax_f32(4, 4, np.array(rows, np.float32).ravel()).reshape(4, 4)
    e = np.exp(np.array([1.0, 3.0, 2.0]) - 3.0)
    e /= e.sum()
    assert_close(got[0], [e[0], 0.0, e[1], e[2]], 0, 1e-6, "NaN skipped")
    assert got[1].tolist() == [0.0, 0.0, 0.0, 0.0]
    assert got[2].tolist() == [0.0, 1.0, 0.0, 0.0]
    assert_close(got[3], [0.25] * 4, 0, 1e-7, "shift invariance")


def test_gelu_backward_reference_vector_and_derivative(oracle, golden):
    c = golden["gelu_backward"]
    z, g = np.array(c["z"], np.float64), np.array(c["grad"], np.float64)
    k, a = np.sqrt(2.0 / np.pi), 0.044715
    t = np.tanh(k * (z + a * z ** 3))
    prime = 0.5 * (1 + t) + 0.5 * z * (1 - t * t) * k * (1 + 3 * a * z * z)
    assert_close(oracle.gelu_backward_f32(c["z"], c["grad"]), prime * g, 0, c["tolerance"], c["source"])
    # the derivative really is d/dz of the oracle's own GELU (central differences in float64)
    zs = np.linspace(-4, 4, 81)
    gelu = lambda x: 0.5 * x * (1 + np.tanh(k * (x + a * x ** 3)))
    numeric = (gelu(zs + 1e-6) - gelu(zs - 1e-6)) / 2e-6
    assert_close(oracle.gelu_backward_f32(zs, np.ones_like(zs)), numeric, 1e-4, 1e-5, "finite differences")


def test_scale_add_row_and_column_sums(oracle):
    rng = np.random.default_rng(3)
    rows, cols = 37, 11
    x = rng.normal(size=(rows, cols)).astype(np.float32)
    bias = rng.normal(size=cols).astype(np.float32)
    assert (oracle.scale_f32(x.ravel(), -0.5) == (x * np.float32(-0.5)).ravel()).all()
    assert (oracle.add_row_f32(rows, cols, x.ravel(), bias).reshape(rows, cols) == x + bias).all()
    sums = oracle.sum_axis0_f32(rows, cols, x.ravel())
    assert_close(sums, x.astype(np.float64).sum(axis=0), 1e-6, 1e-6, "column sums")
    # a transposed index would return row sums: make rows and columns distinguishable
    marked = np.zeros((3, 2), np.float32)
    marked[:, 1] = [1, 2, 3]
    assert oracle.sum_axis0_f32(3, 2, marked.ravel(), 2.0).tolist() == [0.0, 12.0]
    assert oracle.sum_axis0_f32(0, 4, np.zeros(0, np.float32)).tolist() == [0.0] * 4
