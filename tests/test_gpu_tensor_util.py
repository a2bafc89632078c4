"""Parity of the tensor-utility kernels against the CPU oracle (1e-4 rel / 1e-5 abs), through the C ABI."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close

pytestmark = pytest.mark.gpu


def on_device(hip, *arrays):
    return [hip.DeviceBuffer.from_array(np.ascontiguousarray(a, dtype=np.float32)) for a in arrays]


@pytest.mark.parametrize("rows,cols", [(1, 1), (2, 4), (5, 63), (7, 64), (3, 65), (33, 1000), (1024, 256), (4, 5000), (9, 512), (6, 516), (5, 2048), (3, 2052),
                                       (16384, 512), (16387, 128), (16389, 1024),
                                       # rows longer than 2048: a workgroup per row sweeping it (1024 threads; 256 from 2048 rows on)
                                       (3, 100000), (2, 50001), (2100, 2052), (2049, 2051),
                                       # 4097 to 65536 values: the row held in the registers of a 1024-thread workgroup
                                       (5, 50257), (3, 65536), (4, 20003), (2, 8192), (300, 4098), (130, 50257), (129, 65536),
                                       # at most 128 rows of more than 65536 values: every row cut into segments over the grid
                                       (1, 65540), (8, 128256), (100, 100000), (128, 65537), (2, 1000003), (129, 100000)])
def test_row_softmax(hip, oracle, rows, cols):
    rng = np.random.default_rng(rows * 31 + cols)
    x = (rng.normal(size=rows * cols) * 3).astype(np.float32)
    (d_in,) = on_device(hip, x)
    d_out = hip.DeviceBuffer(x.nbytes)
    hip.row_softmax_f32_dev(rows, cols, d_in, d_out)
    hip.device_synchronize()
    got = d_out.to_array(np.float32, rows * cols)
    want = oracle.row_softmax_f32(rows, cols, x)
    if cols > 20000:
        # The oracle adds a row's weights one after the other in f32, as the reference does; over 100000 of them that
        # sum is itself 1.5e-4 off (measured against float64 on this input).  The kernel adds per-thread partial sums
        # in a tree and is held to the exact value; the oracle only has to agree to what its own rounding allows.
        # (that rounding grows with the length: 1e-3 up to 100000 values, 1e-2 at a million)
        assert_close(got, want, max(1e-3, 1e-8 * cols), F32_ABS, f"row_softmax {rows}x{cols} against the sequential f32 sum")
        x64 = x.astype(np.float64).reshape(rows, cols)
        weights = np.exp(x64 - x64.max(axis=1, keepdims=True))
        want = (weights / weights.sum(axis=1, keepdims=True)).ravel()
    assert_close(got, want, F32_REL, F32_ABS, f"row_softmax {rows}x{cols}")
    assert_close(got.reshape(rows, cols).sum(axis=1), np.ones(rows), F32_REL, F32_ABS, "row sums")
    # The absolute floor above is larger than every probability of a wide row, so each value is also held to its
    # float64 definition in relative terms alone (the kernels measure 3e-6 at most; denormal results are left out).
    x64 = x.astype(np.float64).reshape(rows, cols)
    weights = np.exp(x64 - x64.max(axis=1, keepdims=True))
    exact = (weights / weights.sum(axis=1, keepdims=True)).ravel()
    normal = exact > 1e-30
    assert_close(got[normal], exact[normal], 1e-5, 0.0, f"row_softmax {rows}x{cols}, relative to float64")


def test_row_softmax_reference_input_and_edge_rows(hip, oracle, golden):
    c = golden["row_softmax"]
    nan, inf = float("nan"), float("inf")
    edge = [[1.0, nan, 3.0, 2.0], [nan, nan, nan, nan], [0.0, inf, 1.0, inf], [-1000.0] * 4]
    x = np.array(list(c["input"]) + [v for row in edge for v in row], np.float32)
    (d_in,) = on_device(hip, x)
    d_out = hip.DeviceBuffer(x.nbytes)
    hip.row_softmax_f32_dev(6, 4, d_in, d_out)
    hip.device_synchronize()
    got = d_out.to_array(np.float32, 24)
    assert_close(got, oracle.row_softmax_f32(6, 4, x), F32_REL, F32_ABS, "reference input + edge rows")
    assert got[12:16].tolist() == [0.0] * 4 and got[16:20].tolist() == [0.0, 1.0, 0.0, 0.0]


@pytest.mark.parametrize("cols", [4100, 4101, 40001, 100000, 100003])
def test_row_softmax_edge_rows_of_long_rows(hip, oracle, cols):
    """(Above 65536 values these six rows are cut into segments over the grid: the second maximum of rows 2 and 4
    lies in the last segment, and the first segments of row 5 hold nothing but NaN.)"""
    rng = np.random.default_rng(cols)
    x = (rng.normal(size=6 * cols) * 3).astype(np.float32).reshape(6, cols)
    x[0, ::7] = np.nan
    x[1, :] = np.nan
    x[2, cols - 5] = x[2, 1777] = np.inf      # the first of the two becomes the one-hot
    x[3, :] = -1000.0
    x[4, :] = -np.inf
    x[4, 2500] = x[4, cols - 3] = 5.0
    x[5, :cols // 2] = np.nan
    (d_in,) = on_device(hip, x)
    d_out = hip.DeviceBuffer(x.nbytes)
    hip.row_softmax_f32_dev(6, cols, d_in, d_out)
    hip.device_synchronize()
    got = d_out.to_array(np.float32, 6 * cols).reshape(6, cols)
    assert_close(got.ravel(), oracle.row_softmax_f32(6, cols, x.ravel()), 1e-3 if cols > 20000 else F32_REL, F32_ABS, "edge rows")
    assert (got[1] == 0).all()
    assert (got[5, :cols // 2] == 0).all() and abs(float(got[5].astype(np.float64).sum()) - 1.0) < 1e-4
    assert got[4, 2500] == 0.5 and got[4, cols - 3] == 0.5
    assert got[2, 1777] == 1.0 and got[2].sum() == 1.0


@pytest.mark.parametrize("multiple_of_four", [False, True])
def test_gelu_backward(hip, oracle, golden, multiple_of_four):
    # a count that is a multiple of four takes the 128-bit kernel, any other the scalar one
    c = golden["gelu_backward"]
    rng = np.random.default_rng(8)
    extra = 100003
    while ((len(c["z"]) + extra) % 4 == 0) != multiple_of_four:
        extra += 1
    z = np.concatenate([np.array(c["z"], np.float32), (rng.normal(size=extra) * 2).astype(np.float32)])
    g = np.concatenate([np.array(c["grad"], np.float32), rng.normal(size=extra).astype(np.float32)])
    d_z, d_g = on_device(hip, z, g)
    d_out = hip.DeviceBuffer(z.nbytes)
    hip.gelu_backward_f32_dev(z.size, d_z, d_g, d_out)
    hip.device_synchronize()
    assert_close(d_out.to_array(np.float32, z.size), oracle.gelu_backward_f32(z, g), F32_REL, F32_ABS, "gelu_backward")


@pytest.mark.parametrize("rows,cols", [(301, 77), (512, 256), (33, 1028), (7, 4)])
def test_scale_and_add_row(hip, oracle, rows, cols):
    # (column counts that are multiples of four take the 128-bit kernels)
    rng = np.random.default_rng(12)
    x = rng.normal(size=rows * cols).astype(np.float32)
    bias = rng.normal(size=cols).astype(np.float32)
    d_x, d_b = on_device(hip, x, bias)
    d_out = hip.DeviceBuffer(x.nbytes)
    hip.scale_f32_dev(x.size, d_x, -0.37, d_out)
    hip.device_synchronize()
    assert (d_out.to_array(np.float32, x.size) == oracle.scale_f32(x, -0.37)).all()
    hip.add_row_f32_dev(rows, cols, d_x, d_b)
    hip.device_synchronize()
    assert (d_x.to_array(np.float32, x.size) == oracle.add_row_f32(rows, cols, x, bias)).all()
    with pytest.raises(hip.HipErr, match="scale_factor"):
        hip.scale_f32_dev(x.size, d_x, float("nan"), d_out)


def test_elementwise_kernels_on_unaligned_pointers(hip, oracle):
    """Pointers that are only 4-byte aligned must take the scalar kernels and give the same values."""
    rng = np.random.default_rng(13)
    rows, cols = 64, 256
    n = rows * cols
    x = rng.normal(size=n + 1).astype(np.float32)
    g = rng.normal(size=n + 1).astype(np.float32)
    bias = rng.normal(size=cols + 1).astype(np.float32)
    d_x, d_g, d_b = on_device(hip, x, g, bias)
    d_out = hip.DeviceBuffer((n + 1) * 4)
    hip.scale_f32_dev(n, d_x.at(4), 1.5, d_out.at(4))
    hip.device_synchronize()
    assert (d_out.to_array(np.float32, n + 1)[1:] == oracle.scale_f32(x[1:], 1.5)).all()
    hip.gelu_backward_f32_dev(n, d_x.at(4), d_g.at(4), d_out.at(4))
    hip.device_synchronize()
    assert_close(d_out.to_array(np.float32, n + 1)[1:], oracle.gelu_backward_f32(x[1:], g[1:]), F32_REL, F32_ABS, "gelu_backward")
    hip.add_row_f32_dev(rows, cols, d_x.at(4), d_b.at(4))
    hip.device_synchronize()
    assert (d_x.to_array(np.float32, n + 1)[1:] == oracle.add_row_f32(rows, cols, x[1:], bias[1:])).all()


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 2), (64, 256), (65, 257), (1000, 19), (16384, 512), (100000, 8), (37, 260), (131, 1028), (5, 4),
                                       # rows that do not start on 16-byte boundaries: 16-byte loads all the same
                                       (300, 1001), (4097, 67), (70, 50257), (129, 66)])
def test_sum_axis0(hip, oracle, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.normal(size=rows * cols).astype(np.float32)
    (d_x,) = on_device(hip, x)
    d_out = hip.DeviceBuffer(cols * 4)
    for scale in (1.0, -0.25):
        hip.sum_axis0_f32_dev(rows, cols, d_x, scale, d_out)
        hip.device_synchronize()
        got = d_out.to_array(np.float32, cols)
        # summation order differs from the oracle's row-by-row order: tolerance relative to sum of magnitudes
        want = x.astype(np.float64).reshape(rows, cols).sum(axis=0) * scale
        floor = 1e-6 * float(np.abs(x).reshape(rows, cols).sum(axis=0).max())
        assert_close(got, want, F32_REL, F32_ABS + floor, f"sum_axis0 {rows}x{cols} scale={scale}")
        assert_close(oracle.sum_axis0_f32(rows, cols, x, scale), want, F32_REL, F32_ABS + floor, "oracle agrees")
    again = hip.DeviceBuffer(cols * 4)
    hip.sum_axis0_f32_dev(rows, cols, d_x, -0.25, again)
    hip.device_synchronize()
    assert (again.to_array(np.float32, cols) == got).all(), "column sums must be reproducible"


def test_tensor_mirror_methods(hip, oracle):
    import spiraltorch_amd as st
    rng = np.random.default_rng(77)
    rows, cols = 37, 260
    x = st.Tensor(rows, cols, rng.normal(size=rows * cols).astype(np.float32))
    g = st.Tensor(rows, cols, rng.normal(size=rows * cols).astype(np.float32))
    assert_close(x.row_softmax().data(), oracle.row_softmax_f32(rows, cols, x.data()), F32_REL, F32_ABS, "row_softmax")
    assert_close(x.gelu_backward(g).data(), oracle.gelu_backward_f32(x.data(), g.data()), F32_REL, F32_ABS,
                 "gelu_backward")
    assert (x.scale(0.5).data() == oracle.scale_f32(x.data(), 0.5)).all()
    bias = rng.normal(size=cols).astype(np.float32)
    want = oracle.add_row_f32(rows, cols, x.data(), bias)
    y = st.Tensor(rows, cols, x.data().copy())
    y.add_row_inplace(bias)
    assert (y.data() == want).all()
    sums = x.sum_axis0_scaled(0.25)
    assert_close(sums, oracle.sum_axis0_f32(rows, cols, x.data(), 0.25), F32_REL, F32_ABS + 1e-5, "sum_axis0_scaled")
    assert_close(x.sum_axis0(), x.numpy().astype(np.float64).sum(axis=0), F32_REL, F32_ABS + 1e-5, "sum_axis0")
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        x.gelu_backward(st.Tensor.zeros(rows, cols + 1))
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        x.scale(float("inf"))
    with pytest.raises(st.TensorError, match="DataLength"):
        y.add_row_inplace(bias[:-1])
    bad = st.Tensor(1, 2, [1.0, float("nan")])
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        bad.row_softmax()
    assert st.Tensor.zeros(0, 5).sum_axis0().tolist() == [0.0] * 5


def test_operator_chains_stay_on_the_device(hip, oracle):
    """Linear -> GELU -> Linear through the Tensor mirror (Linear::forward = matmul_prepacked_bias,
    crates/st-nn/src/layers/linear.rs:96-104; Gelu::forward, layers/gelu.rs:78-94): every input is uploaded once,
    intermediate results never leave the device, and only the final values are downloaded."""
    import spiraltorch_amd as st
    rng = np.random.default_rng(3)
    batch, d_in, d_hidden, d_out = 96, 64, 160, 48
    x = st.Tensor(batch, d_in, rng.normal(size=batch * d_in).astype(np.float32))
    w1 = st.Tensor(d_in, d_hidden, rng.normal(0, 0.2, d_in * d_hidden).astype(np.float32))
    w2 = st.Tensor(d_hidden, d_out, rng.normal(0, 0.2, d_hidden * d_out).astype(np.float32))
    b1 = st.Tensor(1, d_hidden, rng.normal(size=d_hidden).astype(np.float32))
    b2 = st.Tensor(1, d_out, rng.normal(size=d_out).astype(np.float32))
    p1, p2 = st.PackedB.from_tensor(w1), st.PackedB.from_tensor(w2)

    hip.transfer_counters(reset=True)
    hidden = x.matmul_prepacked_bias(p1, b1)
    activated = hidden.gelu()
    y = activated.matmul_prepacked_bias(p2, b2)
    on_device = hip.transfer_counters()
    assert on_device["h2d_copies"] == 5                       # x, packed w1, b1, packed w2, b2: once each
    assert on_device["h2d_bytes"] == 4 * (x.data().size + w1.data().size + w2.data().size + d_hidden + d_out)
    assert on_device["d2h_copies"] == 0 and on_device["d2h_bytes"] == 0
    assert hidden.is_device_resident() and activated.is_device_resident()
    values = y.data()
    after = hip.transfer_counters()
    assert after["d2h_copies"] == 1 and after["d2h_bytes"] == 4 * batch * d_out
    y.data()                                                  # cached: no second download
    assert hip.transfer_counters()["d2h_copies"] == 1

    want_hidden = oracle.gemm_bias_act_f32(batch, d_hidden, d_in, oracle.ACT_GELU, x.data(), w1.data(), b1.data())
    want = oracle.gemm_f32(batch, d_out, d_hidden, want_hidden, w2.data()).reshape(batch, d_out) + b2.data()
    assert_close(values, want, F32_REL, 2 * F32_ABS, "Linear -> GELU -> Linear")

    # a second pass over the same tensors uploads nothing at all
    hip.transfer_counters(reset=True)
    again = x.matmul_prepacked_bias(p1, b1).gelu().matmul_prepacked_bias(p2, b2)
    assert hip.transfer_counters()["h2d_copies"] == 0
    assert (again.data() == values).all()

    # writing through data_mut() drops the device copy: the next operator sees the new values
    x.data_mut()[:] = 0.0
    zeroed = x.matmul_prepacked_bias(p1, b1)
    assert_close(zeroed.data(), np.tile(b1.data(), batch), 0, 1e-6, "after data_mut")
    with pytest.raises(ValueError):
        x.data()[0] = 1.0                                     # data() is read-only


def test_nonfinite_results_are_caught_on_the_device(hip):
    """The reference's output finite check (pure.rs:2169), without bringing the tensor back."""
    import spiraltorch_amd as st
    a = st.Tensor(4, 4, np.full(16, 3e38, np.float32))
    hip.transfer_counters(reset=True)
    with pytest.raises(st.TensorError) as err:
        a.matmul(st.Tensor(4, 4, np.full(16, 10.0, np.float32)))
    assert err.value.kind == "NonFiniteValue" and err.value.fields["label"] == "matmul_output"
    assert "inf" in err.value.message
    assert hip.transfer_counters()["d2h_copies"] == 0
    rng = np.random.default_rng(0)
    values = rng.normal(size=1000).astype(np.float32)
    buf = hip.DeviceBuffer.from_array(values)
    assert hip.count_nonfinite_f32_dev(1000, buf) == (0, 0, 0.0)
    values[[17, 500]] = [np.nan, -np.inf]
    buf = hip.DeviceBuffer.from_array(values)
    found, first, value = hip.count_nonfinite_f32_dev(1000, buf)
    assert (found, first) == (2, 17) and np.isnan(value)
    assert hip.count_nonfinite_f32_dev(0, None)[0] == 0


def test_gelu_forward_matches_the_oracle(hip, oracle):
    import spiraltorch_amd as st
    x = st.Tensor(3, 50, np.linspace(-6, 6, 150).astype(np.float32))
    want = np.array([oracle.gelu(float(v)) for v in x.data()])
    assert_close(x.gelu().data(), want, F32_REL, F32_ABS, "gelu")
    # a count that is a multiple of four takes the 128-bit kernel; the same values through both kernels agree bit for bit
    values = np.concatenate([np.linspace(-12, 12, 4093), [0.0, -0.0, 88.0, -88.0, 1e-30, -1e-30, 3.0e38]]).astype(np.float32)
    assert values.size % 4 == 0
    d_in, d_out, d_odd = hip.DeviceBuffer.from_array(values), hip.DeviceBuffer(values.nbytes), hip.DeviceBuffer(values.nbytes)
    hip.gelu_f32_dev(values.size, d_in, d_out)
    hip.gelu_f32_dev(values.size - 1, d_in, d_odd)
    hip.device_synchronize()
    got = d_out.to_array(np.float32, values.size)
    v64 = values.astype(np.float64)
    inner = np.sqrt(2.0 / np.pi) * (v64 + 0.044715 * v64 ** 3)
    assert_close(got, 0.5 * v64 * (1.0 + np.tanh(inner)), F32_REL, F32_ABS, "gelu, 128-bit kernel")
    assert (got[:-1] == d_odd.to_array(np.float32, values.size - 1)).all()


@pytest.mark.parametrize("tail", [1, 3])
def test_large_counts_that_are_not_multiples_of_four(hip, oracle, tail):
    """From 2^20 values on, the 128-bit kernels take all but the last one to three values and a second launch of the
    scalar kernel finishes them."""
    from spiraltorch_amd import inputs
    n = (1 << 20) + tail
    rng = np.random.default_rng(tail)
    x = (rng.normal(size=n) * 2).astype(np.float32)
    g = rng.normal(size=n).astype(np.float32)
    d_x, d_g = on_device(hip, x, g)
    d_out = hip.DeviceBuffer(n * 4)
    d_out.zero()
    hip.scale_f32_dev(n, d_x, -0.37, d_out)
    hip.device_synchronize()
    assert (d_out.to_array(np.float32, n) == oracle.scale_f32(x, -0.37)).all()
    hip.gelu_backward_f32_dev(n, d_x, d_g, d_out)
    hip.device_synchronize()
    assert_close(d_out.to_array(np.float32, n), oracle.gelu_backward_f32(x, g), F32_REL, F32_ABS, "gelu_backward")
    hip.gelu_f32_dev(n, d_x, d_out)
    hip.device_synchronize()
    x64 = x.astype(np.float64)
    want = 0.5 * x64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert_close(d_out.to_array(np.float32, n), want, F32_REL, F32_ABS, "gelu")
    d16 = hip.DeviceBuffer(n * 2)
    hip.f32_to_bf16_dev(n, d_x, d16)
    hip.device_synchronize()
    assert (d16.to_array(np.uint16, n) == inputs.to_bf16(x)).all()


def test_raw_gemm_and_probe(hip):
    """gemm_f32_raw and probe() of crates/st-backend-hip/src/lib.rs:188-207, 760-799."""
    a = np.arange(1, 7, dtype=np.float32)
    b = np.arange(7, 13, dtype=np.float32)
    out = np.zeros(4, np.float32)
    hip.gemm_f32_raw(2, 2, 3, a.ctypes.data, b.ctypes.data, out.ctypes.data)
    assert out.tolist() == [58, 64, 139, 154]                 # lib.rs:1107-1112
    with pytest.raises(hip.HipErr, match="gemm received a null pointer; provide contiguous row-major buffers"):
        hip.gemm_f32_raw(2, 2, 3, a.ctypes.data, None, out.ctypes.data)
    with pytest.raises(hip.HipErr, match="gemm dimensions overflow while constructing lhs slice"):
        hip.gemm_f32_raw(2 ** 40, 2, 2 ** 40, a.ctypes.data, b.ctypes.data, out.ctypes.data)
    assert out.tolist() == [58, 64, 139, 154]
    report = hip.probe()
    assert report["available"] and report["initialized"] and report["error"] is None
    assert len(report["devices"]) == hip.device_count() >= 1
    assert hip.runtime() is not None


def test_threads_sharing_the_null_stream_do_not_share_scratch(hip, oracle):
    """Kernels with scratch memory (here the split-k bf16 GEMM and the column sums) called from several host
    threads on the NULL stream, with sizes that make every thread's scratch grow: each result stays right."""
    import threading
    from spiraltorch_amd import inputs
    failures = []

    def work(index):
        try:
            rng = np.random.default_rng(index)
            for round_ in range(6):
                m, n, k = 8 + 8 * index, 128 * (1 + (round_ + index) % 4), 256 * (1 + round_ % 3)
                a = inputs.to_bf16(rng.normal(0, 0.5, m * k).astype(np.float32))
                b = inputs.to_bf16(rng.normal(0, 0.5, k * n).astype(np.float32))
                d_a, d_b, d_c = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(b), hip.DeviceBuffer(m * n * 4)
                hip.gemm_bf16_f32acc_dev(m, n, k, d_a, d_b, d_c)
                rows, cols = 300 + 100 * round_, 64 * (index + 1)
                x = rng.normal(size=rows * cols).astype(np.float32)
                d_x, d_s = hip.DeviceBuffer.from_array(x), hip.DeviceBuffer(cols * 4)
                hip.sum_axis0_f32_dev(rows, cols, d_x, 1.0, d_s)
                hip.device_synchronize()
                got = d_c.to_array(np.float32, m * n)
                want = oracle.gemm_bf16_f32acc(m, n, k, a, b)
                if np.abs(got - want).max() > 1e-3 * max(1.0, np.abs(want).max()):
                    failures.append(("gemm", index, round_))
                sums = d_s.to_array(np.float32, cols)
                if np.abs(sums - x.reshape(rows, cols).astype(np.float64).sum(axis=0)).max() > 1e-3:
                    failures.append(("sum", index, round_))
        except Exception as err:  # noqa: BLE001
            failures.append((index, repr(err)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures


@pytest.mark.gpu
def test_layer_norm_through_the_tensor_mirror(hip, oracle):
    """Tensor::layer_norm_affine[_add] (pure.rs:3702-3760) and the LayerNorm module's epsilon rule
    (crates/st-nn/src/layers/normalization.rs:423-426) against the oracle's layer_norm_cpu restatement."""
    import spiraltorch_amd as st
    rng = np.random.default_rng(11)
    for rows, cols in ((5, 3), (64, 512), (33, 777), (3, 5000)):
        x = st.Tensor(rows, cols, rng.normal(0.3, 1.5, rows * cols).astype(np.float32))
        res = st.Tensor(rows, cols, rng.normal(size=rows * cols).astype(np.float32))
        gamma = st.Tensor(1, cols, rng.normal(1.0, 0.2, cols).astype(np.float32))
        beta = st.Tensor(1, cols, rng.normal(0.0, 0.3, cols).astype(np.float32))
        got = x.layer_norm_affine(gamma, beta, 1e-5)
        assert got.is_device_resident()
        assert_close(got.data(), oracle.layer_norm_f32(rows, cols, x.data(), gamma.data(), beta.data(), 1e-5),
                     F32_REL, 2 * F32_ABS, f"layer_norm_affine {rows}x{cols}")
        got = x.layer_norm_affine_add(res, gamma, beta, 1e-3)
        assert_close(got.data(), oracle.layer_norm_f32(rows, cols, x.data(), gamma.data(), beta.data(), 1e-3, residual=res.data()),
                     F32_REL, 2 * F32_ABS, f"layer_norm_affine_add {rows}x{cols}")
    ln = st.LayerNorm("ln", 512, -1.0, 1e-5)
    x = st.Tensor(7, 512, rng.normal(size=7 * 512).astype(np.float32))
    want = oracle.layer_norm_f32(7, 512, x.data(), ln.gamma.data(), ln.beta.data(), ln.effective_epsilon())
    assert_close(ln.forward(x).data(), want, F32_REL, 2 * F32_ABS, "LayerNorm::forward")
    # an overflowing sum of squares surfaces as a non-finite result (the reference names the scalar, layer_norm_sumsq)
    big = st.Tensor(1, 2, [np.finfo(np.float32).max, -np.finfo(np.float32).max])
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        big.layer_norm_affine(st.Tensor(1, 2, [1.0, 1.0]), st.Tensor.zeros(1, 2), 1e-5)


@pytest.mark.gpu
def test_linear_layer_forward_and_backward_stay_on_the_device(hip, oracle):
    """Linear::forward / backward (crates/st-nn/src/layers/linear.rs:87-168) through the mirror: forward equals
    matmul + add_row (the reference's own test, linear.rs:214-223), the gradients equal the lhs-transposed product,
    the column sums and the product with the transposed weight, each scaled as the reference scales it; the weight is
    packed once on the device and nothing but the inputs ever crosses the bus."""
    import spiraltorch_amd as st
    layer = st.Linear("fc", 3, 2)
    x = st.Tensor(1, 3, [1.0, -2.0, 0.5])
    expected = x.matmul(layer.weight)
    expected.add_row_inplace(layer.bias)
    assert (layer.forward(x).data() == expected.data()).all()

    rng = np.random.default_rng(5)
    batch, d_in, d_out = 96, 200, 72
    layer = st.Linear("fc", d_in, d_out)
    layer.load_weight(st.Tensor(d_in, d_out, rng.normal(0, 0.1, d_in * d_out).astype(np.float32)),
                      st.Tensor(1, d_out, rng.normal(size=d_out).astype(np.float32)))
    x = st.Tensor(batch, d_in, rng.normal(size=batch * d_in).astype(np.float32))
    g = st.Tensor(batch, d_out, rng.normal(size=batch * d_out).astype(np.float32))
    w, b = np.array(layer.weight.data()), np.array(layer.bias.data())

    hip.transfer_counters(reset=True)
    y = layer.forward(x)
    grad_input = layer.backward(x, g)
    moved = hip.transfer_counters()
    assert moved["h2d_copies"] == 4                      # x, weight, bias, grad_output: once each; the pack is made on the device
    assert moved["h2d_bytes"] == 4 * (batch * d_in + d_in * d_out + d_out + batch * d_out)
    assert moved["d2h_copies"] == 0
    for t in (y, grad_input, layer.weight_gradient, layer.bias_gradient):
        assert t.is_device_resident()

    want_y = oracle.gemm_f32(batch, d_out, d_in, x.data(), w).reshape(batch, d_out) + b
    assert_close(y.data(), want_y, F32_REL, 2 * F32_ABS, "Linear::forward")
    assert_close(layer.weight_gradient.data(), oracle.gemm_f32(d_in, d_out, batch, x.data(), g.data(), scale=1.0 / batch, lhs_transposed=True),
                 F32_REL, 2 * F32_ABS, "linear_weight_grad")
    assert_close(layer.bias_gradient.data(), oracle.sum_axis0_f32(batch, d_out, g.data(), 1.0 / batch), F32_REL, 2 * F32_ABS,
                 "linear_bias_grad")
    w_t = np.ascontiguousarray(w.reshape(d_in, d_out).T)
    assert_close(grad_input.data(), oracle.gemm_f32(batch, d_in, d_out, g.data(), w_t), F32_REL, 2 * F32_ABS, "linear_input_grad")

    # a second forward re-uses the pack: nothing is uploaded
    hip.transfer_counters(reset=True)
    again = layer.forward(x)
    assert hip.transfer_counters()["h2d_copies"] == 0
    assert (again.data() == y.data()).all()
    # a second backward accumulates (Parameter::accumulate_euclidean)
    first = np.array(layer.weight_gradient.data())
    layer.backward(x, g)
    assert_close(layer.weight_gradient.data(), 2 * first, 1e-6, 1e-7, "accumulated weight gradient")
    # an overflowing product is reported under the layer's label (relabel_non_finite, linear.rs:30-37, test :319-333)
    tiny = st.Linear("fc", 1, 1)
    tiny.weight.data_mut()[0] = np.finfo(np.float32).max
    with pytest.raises(st.TensorError) as info:
        tiny.backward(st.Tensor(1, 1, [0.0]), st.Tensor(1, 1, [2.0]))
    assert info.value.fields["label"] == "linear_input_grad"


@pytest.mark.gpu
def test_scratch_of_exited_threads_is_reused_not_leaked(hip, oracle):
    """Scratch buffers are kept per (stream, host thread); a thread that exits leaves its buffer to the next thread
    that launches on the stream, so a pool of short-lived threads on the default stream holds a bounded number of
    buffers, and st_hip_release_scratch frees them."""
    import threading
    rows, cols = 4096, 96
    x = np.random.default_rng(21).normal(size=rows * cols).astype(np.float32)
    want = oracle.sum_axis0_f32(rows, cols, x)
    d_x = hip.DeviceBuffer.from_array(x)
    hip.release_scratch(None)
    before = hip.scratch_buffer_count()
    results, errors = [], []

    def work():
        try:
            d_out = hip.DeviceBuffer(cols * 4)
            hip.sum_axis0_f32_dev(rows, cols, d_x, 1.0, d_out)   # column sums keep their partials in scratch
            hip.device_synchronize()
            results.append(d_out.to_array(np.float32, cols))
        except Exception as err:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(err)

    for _ in range(12):                  # one after the other: each thread has exited before the next starts
        t = threading.Thread(target=work)
        t.start()
        t.join()
    assert not errors, errors
    assert hip.scratch_buffer_count() <= before + 1, "every short-lived thread left a buffer behind"
    for got in results:
        assert_close(got, want, F32_REL, 1e-3, "column sums from a short-lived thread")
    threads = [threading.Thread(target=work) for _ in range(4)]   # concurrent threads do not share a buffer
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert hip.scratch_buffer_count() <= before + 4
    for got in results[-4:]:
        assert_close(got, want, F32_REL, 1e-3, "column sums from concurrent threads")
    hip.release_scratch(None)
    assert hip.scratch_buffer_count() == before
