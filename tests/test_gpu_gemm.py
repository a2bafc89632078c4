"""Parity of the HIP f32 GEMM family against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close

pytestmark = pytest.mark.gpu


def test_reference_known_answers(hip, golden):
    for case in golden["gemm"]:
        out = np.zeros(case["m"] * case["n"], np.float32)
        lhs, rhs = np.array(case["lhs"], np.float32), np.array(case["rhs"], np.float32)
        if case["lhs_transposed"]:
            hip.gemm_lhs_transpose_scaled_f32(case["m"], case["n"], case["k"], case["scale"], lhs, rhs, out)
        else:
            hip.gemm_scaled_f32(case["m"], case["n"], case["k"], case["scale"], lhs, rhs, out)
        assert out.tolist() == case["expected"], case["source"]


def test_ones_and_epilogue_known_answers(hip, golden):
    c = golden["gemm_ones"]
    lhs = np.full(c["m"] * c["k"], c["lhs_value"], np.float32)
    rhs = np.full(c["k"] * c["n"], c["rhs_value"], np.float32)
    out = np.zeros(c["m"] * c["n"], np.float32)
    hip.gemm_f32(c["m"], c["n"], c["k"], lhs, rhs, out)
    assert (out == c["expected_value"]).all()
    hip.gemm_bias_activation_f32(c["m"], c["n"], c["k"], hip.GemmActivation.Relu, lhs, rhs,
                                 np.full(c["n"], c["bias_value"], np.float32), None, out)
    assert (out == c["expected_bias_relu_value"]).all()

    e = golden["gemm_epilogue"]
    lhs, rhs = np.array(e["lhs"], np.float32), np.array(e["rhs"], np.float32)
    bias, residual = np.array(e["bias"], np.float32), np.array(e["residual"], np.float32)
    out = np.zeros(4, np.float32)
    hip.gemm_bias_activation_f32(2, 2, 3, hip.GemmActivation.Relu, lhs, rhs, bias, None, out)
    assert out.tolist() == e["relu"]
    hip.gemm_bias_activation_f32(2, 2, 3, hip.GemmActivation.Relu, lhs, rhs, bias, residual, out)
    assert out.tolist() == e["residual_relu"]
    gelu64 = lambda x: 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))
    for res, pre in ((None, e["gelu_pre_activation"]), (residual, e["residual_gelu_pre_activation"])):
        hip.gemm_bias_activation_f32(2, 2, 3, hip.GemmActivation.Gelu, lhs, rhs, bias, res, out)
        np.testing.assert_allclose(out, gelu64(np.array(pre, np.float64)), atol=2e-5, rtol=1e-6)


def test_zero_inner_runs_the_epilogue(hip, golden):
    c = golden["gemm_zero_inner"]
    out = np.full(4, 99.0, np.float32)
    hip.gemm_bias_activation_f32(2, 2, 0, hip.GemmActivation.Relu, np.zeros(0, np.float32), np.zeros(0, np.float32),
                                 np.array(c["bias"], np.float32), np.array(c["residual"], np.float32), out)
    assert out.tolist() == c["expected_relu"]
    plain = np.full(4, 99.0, np.float32)
    hip.gemm_f32(2, 2, 0, np.zeros(0, np.float32), np.zeros(0, np.float32), plain)
    assert (plain == 0).all()


def test_validation_happens_before_mutation(hip):
    # crates/st-backend-hip/src/lib.rs:1236-1277,1310-1326
    lhs, rhs = np.array([1, 2, 3, 4], np.float32), np.array([5, 6, 7, 8], np.float32)
    out = np.full(4, 13.0, np.float32)
    with pytest.raises(hip.HipErr, match="bias buffer length 1 does not match n=2"):
        hip.gemm_bias_activation_f32(2, 2, 2, hip.GemmActivation.Relu, lhs, rhs, np.ones(1, np.float32), None, out)
    with pytest.raises(hip.HipErr, match="residual buffer length 1 does not match m\\*n=4"):
        hip.gemm_bias_activation_f32(2, 2, 2, hip.GemmActivation.Gelu, lhs, rhs, np.ones(2, np.float32),
                                     np.ones(1, np.float32), out)
    with pytest.raises(hip.HipErr, match="scale must be finite, received inf"):
        hip.gemm_scaled_f32(2, 2, 2, float("inf"), lhs, rhs, out)
    with pytest.raises(hip.HipErr, match="lhs buffer length 4 does not match m\\*k=6"):
        hip.gemm_f32(2, 2, 3, lhs, rhs, out)
    with pytest.raises(hip.HipErr, match="rhs buffer length 4 does not match k\\*n=6"):
        hip.gemm_f32(2, 3, 2, lhs, rhs, np.zeros(6, np.float32))
    with pytest.raises(hip.HipErr, match="output buffer length 4 does not match m\\*n=2"):
        hip.gemm_f32(1, 2, 2, lhs[:2], rhs, out)
    with pytest.raises(hip.HipErr, match="overflow"):
        hip.gemm_f32(2 ** 40, 2 ** 40, 2, lhs, rhs, out)
    assert (out == 13.0).all()


def test_empty_output_is_a_no_op(hip):
    hip.gemm_f32(0, 5, 3, np.zeros(0, np.float32), np.zeros(15, np.float32), np.zeros(0, np.float32))
    hip.gemm_f32(4, 0, 3, np.zeros(12, np.float32), np.zeros(0, np.float32), np.zeros(0, np.float32))


SHAPES = [(1, 1, 1), (2, 3, 4), (8, 12, 7), (10, 13, 9), (8, 16, 6), (4, 16, 5), (33, 65, 17), (64, 64, 64),
          (100, 130, 70), (129, 127, 31), (256, 64, 200), (5, 300, 19), (300, 5, 23),
          # whole 16-wide k-tiles and 16-byte aligned rows: the direct-to-LDS ring kernel, ragged in m and n
          (132, 136, 48), (260, 68, 160), (96, 260, 16), (1000, 128, 32),
          # few tiles and a long k: 32x32 tiles with k split over the wavefronts of a workgroup
          (100, 132, 256), (31, 36, 144), (64, 64, 640)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_random_shapes_match_the_oracle(hip, oracle, m, n, k):
    rng = np.random.default_rng(m * 7919 + n * 31 + k)
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    hip.gemm_f32(m, n, k, a, b, out)
    assert_close(out, oracle.gemm_f32(m, n, k, a, b), F32_REL, F32_ABS, f"gemm {m}x{n}x{k}")
    hip.gemm_scaled_f32(m, n, k, -0.37, a, b, out)
    assert_close(out, oracle.gemm_f32(m, n, k, a, b, scale=-0.37), F32_REL, F32_ABS, "scaled")
    at = np.ascontiguousarray(a.reshape(m, k).T).ravel()
    hip.gemm_lhs_transpose_scaled_f32(m, n, k, 0.5, at, b, out)
    assert_close(out, oracle.gemm_f32(m, n, k, at, b, scale=0.5, lhs_transposed=True), F32_REL, F32_ABS, "lhs^T")
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.uniform(-1, 1, m * n).astype(np.float32)
    for act, code in ((hip.GemmActivation.Relu, oracle.ACT_RELU), (hip.GemmActivation.Gelu, oracle.ACT_GELU)):
        hip.gemm_bias_activation_f32(m, n, k, act, a, b, bias, None, out)
        assert_close(out, oracle.gemm_bias_act_f32(m, n, k, code, a, b, bias), F32_REL, F32_ABS, f"bias+{act.name}")
        hip.gemm_bias_activation_f32(m, n, k, act, a, b, bias, res, out)
        assert_close(out, oracle.gemm_bias_act_f32(m, n, k, code, a, b, bias, res), F32_REL, F32_ABS,
                     f"bias+residual+{act.name}")


def test_long_reduction_against_float64(hip):
    """k = 4096 with U[-1,1) data: sums of magnitude ~20 whose value can land anywhere near zero, so the bound
    is the standard one for a reordered f32 sum, a small multiple of unit roundoff times sum |a||b| (about
    2e-4 here), checked against exact float64 — the oracle's own sequential f32 sum carries the same error."""
    rng = np.random.default_rng(77)
    m, n, k = 64, 96, 4096
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    hip.gemm_f32(m, n, k, a, b, out)
    a64, b64 = a.astype(np.float64).reshape(m, k), b.astype(np.float64).reshape(k, n)
    exact = a64 @ b64
    bound = 1e-4 * np.abs(exact) + 1e-5 + 2e-7 * (np.abs(a64) @ np.abs(b64))
    assert (np.abs(out.reshape(m, n) - exact) <= bound).all()


@pytest.mark.parametrize("m,n,k,lhs_t", [
    (64, 64, 20000, False),    # 32x32 tiles, k cut over workgroups as well as over a workgroup's wavefronts
    (256, 256, 8192, False),
    (40, 36, 2064, False),     # the last slice shorter than the others
    (4096, 1, 4096, False),    # matrix-vector: one wavefront per row of A
    (300, 3, 2048, False),     # few rows: a workgroup per row
    (5000, 2, 260, False),
    (64, 1, 64, False),
    (1000, 3, 1028, False),
    (2050, 1, 4099, False),    # k not a multiple of 4: the general tile kernel, k-sliced
    (300, 3, 2049, False),     # ragged k: the last slice ends inside a k-tile
    (1030, 2, 1100, True),     # A stored transposed
    (130, 70, 5000, True),
    (256, 192, 8192, True),    # the direct-to-LDS ring kernel, A transposed (a weight gradient Xᵀ·dY), k-sliced
    (100, 260, 4096, True),
    (1024, 1024, 1001, False), # large products with an odd k run on copies zero-padded along k
    (1024, 520, 2050, True),
    (1500, 1000, 703, False),
    (10027, 1, 9472, True),    # Aᵀ·x with A stored k×m: lanes own outputs, k cut into slices; rows of odd length
    (4096, 4, 4100, True),     # four columns; the last 32-row group of a slice is short
    (1025, 2, 64, True),       # one slice; the last lanes' quad straddles the end of the rows
    (2048, 3, 300, True),
])
def test_k_sliced_launches_against_float64(hip, m, n, k, lhs_t):
    """Few output tiles and a long k: the launch is cut along k over workgroups, the partial planes are added in slice
    order and the epilogue runs in the reduction.  Bound as in test_long_reduction_against_float64."""
    rng = np.random.default_rng(m + n + k)
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.uniform(-1, 1, m * n).astype(np.float32)
    a64 = (a.reshape(k, m).T if lhs_t else a.reshape(m, k)).astype(np.float64)
    b64 = b.astype(np.float64).reshape(k, n)
    exact = a64 @ b64
    slack = 2e-7 * (np.abs(a64) @ np.abs(b64))
    out = np.full(m * n, np.nan, np.float32)
    if lhs_t:
        hip.gemm_lhs_transpose_scaled_f32(m, n, k, 0.25, a, b, out)
        want = 0.25 * exact
        assert (np.abs(out.reshape(m, n) - want) <= 1e-4 * np.abs(want) + 1e-5 + slack).all()
        twice = np.zeros(m * n, np.float32)
        hip.gemm_lhs_transpose_scaled_f32(m, n, k, 0.25, a, b, twice)
        assert (twice == out).all(), "the slices are added in a fixed order"
        return
    hip.gemm_scaled_f32(m, n, k, -0.5, a, b, out)
    want = -0.5 * exact
    assert (np.abs(out.reshape(m, n) - want) <= 1e-4 * np.abs(want) + 1e-5 + slack).all()
    twice = np.zeros(m * n, np.float32)
    hip.gemm_scaled_f32(m, n, k, -0.5, a, b, twice)
    assert (twice == out).all(), "the slices are added in a fixed order"
    hip.gemm_bias_activation_f32(m, n, k, hip.GemmActivation.Relu, a, b, bias, res, out)
    want = np.maximum(exact + bias.astype(np.float64)[None, :] + res.astype(np.float64).reshape(m, n), 0.0)
    assert (np.abs(out.reshape(m, n) - want) <= 1e-4 * np.abs(want) + 1e-5 + slack).all()
    hip.gemm_bias_activation_f32(m, n, k, hip.GemmActivation.Gelu, a, b, bias, None, out)
    pre = exact + bias.astype(np.float64)[None, :]
    want = 0.5 * pre * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (pre + 0.044715 * pre ** 3)))
    assert (np.abs(out.reshape(m, n) - want) <= 1e-4 * np.abs(want) + 2e-5 + 2 * slack).all()


def test_lhs_of_more_than_2_gib(hip):
    """An A beyond 2^31 bytes is cut into row blocks the 32-bit-offset kernels can address; rows on both sides of the
    cut and at both ends are checked against float64."""
    m, n, k = 525000, 64, 1024
    rng = np.random.default_rng(3)
    a = rng.random(m * k, dtype=np.float32) - 0.5
    b = rng.random(k * n, dtype=np.float32) - 0.5
    bias = rng.random(n, dtype=np.float32)
    d_a, d_b, d_bias = (hip.DeviceBuffer.from_array(v) for v in (a, b, bias))
    d_out = hip.DeviceBuffer(m * n * 4)
    hip.gemm_bias_act_f32_dev(m, n, k, hip.GemmActivation.Relu, d_a, d_b, d_bias, None, d_out)
    hip.device_synchronize()
    got = d_out.to_array(np.float32, m * n).reshape(m, n)
    cut = ((1 << 31) // (k * 4) - 1) // 256 * 256
    rows = np.r_[0:3, cut - 3:cut + 3, m - 3:m, rng.integers(0, m, 40)]
    want = np.maximum(a.reshape(m, k)[rows].astype(np.float64) @ b.reshape(k, n).astype(np.float64) + bias, 0.0)
    assert_close(got[rows], want, F32_REL, 2e-5, "rows of a 2.15 GB lhs")
    assert np.isfinite(got).all() and (got >= 0).all()


def test_config1_512_cubed(hip, oracle):
    """BASELINE config 1: f32 C = A.B, M=N=K=512, U[-1,1) from the fixed seeds."""
    from spiraltorch_amd import inputs
    a = inputs.uniform(inputs.seed_for(1, 0), 512 * 512, -1.0, 1.0)
    b = inputs.uniform(inputs.seed_for(1, 1), 512 * 512, -1.0, 1.0)
    out = np.zeros(512 * 512, np.float32)
    hip.gemm_f32(512, 512, 512, a, b, out)
    assert_close(out, oracle.gemm_f32(512, 512, 512, a, b, threads=8), F32_REL, F32_ABS, "config 1")


def test_large_tile_path_and_linearity(hip, oracle):
    """Shapes that select the 128x128 tile (>= 256 tiles), checked on sampled rows and by linearity."""
    rng = np.random.default_rng(99)
    m, n, k = 2048, 2048, 160
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    hip.gemm_f32(m, n, k, a, b, out)
    rows = [0, 1, 127, 128, 1000, 2047]
    want = oracle.gemm_f32(len(rows), n, k, a.reshape(m, k)[rows].ravel(), b)
    assert_close(out.reshape(m, n)[rows], want, F32_REL, F32_ABS, "sampled rows")
    # size-independent property: (2A).B == 2(A.B) exactly (power-of-two scaling commutes with rounding)
    out2 = np.zeros(m * n, np.float32)
    hip.gemm_f32(m, n, k, 2 * a, b, out2)
    assert (out2 == 2 * out).all()


def test_ring_kernel_128_tiles_ragged_edges(hip, oracle):
    """24 x 23 tiles of 128x128 with ragged last tiles in both directions, plain and lhs-transposed, with the
    fused epilogue; every element is checked."""
    rng = np.random.default_rng(4)
    m, n, k = 3000, 2820, 64
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.uniform(-1, 1, m * n).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    want = oracle.gemm_f32(m, n, k, a, b, threads=8)
    hip.gemm_f32(m, n, k, a, b, out)
    assert_close(out, want, F32_REL, F32_ABS, "plain")
    at = np.ascontiguousarray(a.reshape(m, k).T).ravel()
    hip.gemm_lhs_transpose_scaled_f32(m, n, k, 0.5, at, b, out)
    assert_close(out, 0.5 * want.astype(np.float64), F32_REL, F32_ABS, "lhs^T scaled")
    hip.gemm_bias_activation_f32(m, n, k, hip.GemmActivation.Relu, a, b, bias, res, out)
    pre = (want.astype(np.float64).reshape(m, n) + bias).ravel() + res
    assert_close(out, np.maximum(pre, 0), F32_REL, F32_ABS, "bias+residual+relu")


@pytest.mark.parametrize("m,n,k", [(2, 2, 3), (33, 65, 17), (64, 64, 64), (132, 136, 48), (1000, 260, 32),
                                   (16384, 512, 64), (3000, 2820, 16),
                                   # a k the packed kernel does not take: B is unpacked into the stream's scratch buffer,
                                   # which the product then must not use for k-sliced partial sums
                                   (64, 64, 1026), (40, 36, 1100)])
def test_prepacked_rhs(hip, oracle, m, n, k):
    """B prepacked as its (n, k) transpose (PackedB): same results as the row-major GEMM, with and without
    bias / residual / GELU; ragged k takes the unpack-to-workspace path."""
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    packed = np.ascontiguousarray(b.reshape(k, n).T).ravel()
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.uniform(-1, 1, m * n).astype(np.float32)
    out = np.zeros(m * n, np.float32)
    plain = oracle.gemm_f32(m, n, k, a, b, threads=8)
    hip.gemm_prepacked_bias_activation_f32(m, n, k, 0, a, packed, None, None, out)
    assert_close(out, plain, F32_REL, F32_ABS, "prepacked")
    if m * n * k <= 1 << 22:  # the reference's naive packed order (four partial sums on the n % 4 tail columns)
        assert_close(out, oracle.gemm_f32_packed_naive(m, n, k, a, packed), F32_REL, F32_ABS, "prepacked vs packed-naive order")
    hip.gemm_prepacked_bias_activation_f32(m, n, k, 0, a, packed, bias, None, out)
    assert_close(out, (plain.astype(np.float64).reshape(m, n) + bias).ravel(), F32_REL, F32_ABS, "prepacked + bias")
    hip.gemm_prepacked_bias_activation_f32(m, n, k, hip.GemmActivation.Gelu, a, packed, bias, res, out)
    want = oracle.gemm_bias_act_f32(m, n, k, oracle.ACT_GELU, a, b, bias, res, threads=8)
    assert_close(out, want, F32_REL, F32_ABS, "prepacked + bias + residual + gelu")
    # packing on the device gives the same matrix
    d_b, d_p = hip.DeviceBuffer.from_array(b), hip.DeviceBuffer(b.nbytes)
    hip.pack_rhs_f32_dev(k, n, d_b, d_p)
    hip.device_synchronize()
    assert (d_p.to_array(np.float32, k * n) == packed).all()


def test_tensor_mirror_matches_the_reference_api(hip, oracle):
    from spiraltorch_amd import Tensor, TensorError
    a = Tensor(2, 3, [1, 2, 3, 4, 5, 6])
    b = Tensor(3, 2, [7, 8, 9, 10, 11, 12])
    assert a.matmul(b, backend="hip").data().tolist() == [58, 64, 139, 154]
    assert a.matmul(b).shape() == (2, 2)
    assert a.matmul_scaled(b, 0.5, backend="hip").data().tolist() == [29, 32, 69.5, 77]
    from spiraltorch_amd import PackedB
    packed = PackedB.from_tensor(b)
    assert packed.as_slice().tolist() == [7, 9, 11, 8, 10, 12] and (packed.inner(), packed.cols()) == (3, 2)
    assert a.matmul_prepacked(packed, backend="hip").data().tolist() == [58, 64, 139, 154]
    assert a.matmul_prepacked_bias(packed, [1, -1]).data().tolist() == [59, 63, 140, 153]
    with pytest.raises(TensorError) as bad:
        a.matmul_prepacked_bias(packed, [1, 2, 3])
    assert bad.value.kind == "DataLength"
    at = Tensor(3, 2, [1, 4, 2, 5, 3, 6])
    assert at.matmul_lhs_transpose_scaled(b, 1.0, backend="hip").data().tolist() == [58, 64, 139, 154]
    assert a.matmul_bias_relu(b, [-60, 1], backend="hip").data().tolist() == [0, 65, 79, 155]
    res = Tensor(2, 2, [3, -70, -140, 2])
    assert a.matmul_bias_add_relu(b, [-60, 1], res, backend="hip").data().tolist() == [1, 0, 0, 157]
    with pytest.raises(TensorError) as err:
        a.matmul(a, backend="hip")
    assert err.value.kind == "ShapeMismatch"
    big = Tensor(1, 1, [3e38])
    with pytest.raises(TensorError) as err:
        big.matmul(Tensor(1, 1, [10.0]), backend="hip")
    assert err.value.kind == "NonFiniteValue"


def test_concurrent_callers(hip, oracle):
    """Python releases the GIL in ctypes calls; the reference expects concurrent callers
    (bindings/st-py/src/tensor.rs:988-1006)."""
    import threading
    rng = np.random.default_rng(1)
    problems = []
    for i in range(8):
        m, n, k = 40 + 8 * i, 24 + 4 * i, 64 + i
        a = rng.uniform(-1, 1, m * k).astype(np.float32)
        b = rng.uniform(-1, 1, k * n).astype(np.float32)
        problems.append((m, n, k, a, b, np.zeros(m * n, np.float32)))
    def work(p):
        for _ in range(5):
            hip.gemm_f32(p[0], p[1], p[2], p[3], p[4], p[5])
    threads = [threading.Thread(target=work, args=(p,)) for p in problems]
    for t in threads: t.start()
    for t in threads: t.join()
    for m, n, k, a, b, out in problems:
        assert_close(out, oracle.gemm_f32(m, n, k, a, b), F32_REL, F32_ABS, f"thread {m}x{n}x{k}")
