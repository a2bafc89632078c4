"""Parity of the conv2d backward kernels (grad_input, grad_weight, grad_bias) against the CPU oracle:
1e-4 rel / 1e-5 abs (plus a floor proportional to the summed magnitudes for the long grad_weight sums)."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close

pytestmark = pytest.mark.gpu

CASES = [
    # batch, c_in, h, w, c_out, kernel, stride, padding, dilation
    (1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1)),
    (2, 3, 8, 8, 4, (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 2, 7, 5, 5, (3, 2), (1, 2), (1, 1), (1, 1)),       # strided: adjoint gather
    (2, 2, 9, 9, 3, (3, 3), (2, 2), (1, 1), (2, 2)),       # stride 2, dilation 2
    (3, 4, 5, 6, 2, (2, 3), (2, 1), (0, 2), (1, 1)),
    (2, 16, 14, 14, 32, (3, 3), (1, 1), (1, 1), (1, 1)),   # ring forward kernel for grad_input (k = 288)
    (4, 8, 12, 12, 70, (3, 3), (1, 1), (1, 1), (1, 1)),    # ragged channel tiles
    (2, 5, 10, 11, 6, (3, 3), (1, 1), (3, 3), (1, 1)),     # padding larger than the kernel reach: adjoint gather
    (2, 4, 16, 16, 8, (5, 5), (1, 1), (2, 2), (1, 1)),
    (8, 64, 14, 14, 64, (1, 1), (1, 1), (0, 0), (1, 1)),
    (2, 64, 9, 10, 128, (3, 3), (1, 1), (1, 1), (1, 1)),   # 128 × 192 grad_weight tiles, exact fit (S = 576)
    (3, 21, 11, 7, 120, (3, 3), (1, 1), (1, 1), (1, 1)),   # 128 × 192 tiles with ragged channels and columns (S = 189)
    (2, 22, 9, 9, 250, (3, 3), (2, 1), (1, 0), (1, 1)),    # two channel tiles, strided rows (per-element gather)
]


@pytest.mark.parametrize("case", CASES)
def test_backward_matches_the_oracle(hip, oracle, case):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = case
    rng = np.random.default_rng(sum(case[:5]) * 7 + kernel[0])
    oh, ow = oracle.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wgt = (rng.normal(size=c_out * c_in * kernel[0] * kernel[1]) * 0.2).astype(np.float32)
    g = rng.normal(size=batch * c_out * oh * ow).astype(np.float32)
    gi, gw, gb = (np.zeros(n, np.float32) for n in (x.size, wgt.size, c_out))
    hip.conv2d_backward_f32(*case, x, wgt, g, gi, gw, gb)
    want_gi, want_gw, want_gb = oracle.conv2d_backward_f32(*case, x, wgt, g)
    assert_close(gi, want_gi, F32_REL, F32_ABS, f"grad_input {case}")
    # grad_weight / grad_bias add batch*oh*ow terms in a different order than the oracle
    floor = 2e-7 * float(np.abs(g).max()) * float(np.abs(x).max()) * oh * ow
    assert_close(gw, want_gw, F32_REL, F32_ABS + floor, f"grad_weight {case}")
    assert_close(gb, want_gb, F32_REL, F32_ABS + floor, f"grad_bias {case}")


def test_reference_1x1_vector(hip):
    """conv2d_backward_matches_manual_kernel11, crates/st-nn/src/layers/conv.rs:4114-4130."""
    gi, gw, gb = np.zeros(4, np.float32), np.zeros(1, np.float32), np.zeros(1, np.float32)
    f = lambda *v: np.array(v, np.float32)
    hip.conv2d_backward_f32(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), f(1, 2, 3, 4), f(1.5), f(1, 1, 1, 1), gi, gw, gb)
    assert gi.tolist() == [1.5] * 4 and gw.tolist() == [10.0] and gb.tolist() == [4.0]


def test_config2_shape_adjoint_identity(hip):
    """BASELINE config 2 geometry (batch 32, 64->128 channels, 56x56, 3x3, pad 1): size-independent properties.
    <conv(x), g> == <x, grad_input(g)>, grad_weight is linear in grad_output, grad_bias equals the plane sums."""
    from spiraltorch_amd import inputs
    shape = (32, 64, 56, 56, 128)
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    x = inputs.normal(101, 32 * 64 * 56 * 56)
    wgt = inputs.normal(102, 128 * 64 * 9, 0.0, 0.06)
    g = inputs.normal(103, 32 * 128 * 56 * 56)
    d_x, d_w, d_g = (hip.DeviceBuffer.from_array(a) for a in (x, wgt, g))
    d_y, d_gi = hip.DeviceBuffer(g.nbytes), hip.DeviceBuffer(x.nbytes)
    d_gw, d_gb = hip.DeviceBuffer(wgt.nbytes), hip.DeviceBuffer(128 * 4)
    hip.conv2d_bias_act_f32_dev(*shape, *geom, 0, d_x, d_w, None, d_y)
    hip.conv2d_grad_input_f32_dev(*shape, *geom, d_g, d_w, d_gi)
    hip.conv2d_grad_weight_f32_dev(*shape, *geom, d_x, d_g, 1.0 / 32, d_gw)
    hip.conv2d_grad_bias_f32_dev(*shape, *geom, d_g, 1.0 / 32, d_gb)
    hip.device_synchronize()
    y, gi = d_y.to_array(np.float32, g.size), d_gi.to_array(np.float32, x.size)
    lhs = float(np.dot(y.astype(np.float64), g.astype(np.float64)))
    rhs = float(np.dot(x.astype(np.float64), gi.astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-5 * abs(lhs), (lhs, rhs)
    # <W, grad_weight(g)>·batch == <conv(x), g> as well (conv is linear in W)
    gw = d_gw.to_array(np.float32, wgt.size)
    assert abs(float(np.dot(wgt.astype(np.float64), gw.astype(np.float64))) * 32 - lhs) <= 1e-5 * abs(lhs)
    gb = d_gb.to_array(np.float32, 128)
    want_gb = g.astype(np.float64).reshape(32, 128, -1).sum(axis=(0, 2)) / 32
    assert_close(gb, want_gb, 1e-4, 1e-4, "grad_bias")


def test_validation(hip):
    gi, gw, gb = np.zeros(4, np.float32), np.zeros(1, np.float32), np.zeros(1, np.float32)
    with pytest.raises(hip.HipErr, match="grad_output buffer length 3"):
        hip.conv2d_backward_f32(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), np.array([1, 2, 3, 4], np.float32),
                                np.array([1.5], np.float32), np.ones(3, np.float32), gi, gw, gb)
    # empty batch: nothing is written
    gw[:] = 7.0
    hip.conv2d_backward_f32(0, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), np.zeros(0, np.float32), np.array([1.5], np.float32),
                            np.zeros(0, np.float32), np.zeros(0, np.float32), gw, gb)
    assert gw.tolist() == [7.0]


def test_conv2d_layer_backward_accumulates(hip, oracle):
    import spiraltorch_amd as st
    rng = np.random.default_rng(5)
    conv = st.Conv2d("c", 3, 4, (3, 3), (1, 1), (1, 1), (1, 1), (6, 5))
    batch = 2
    x = st.Tensor(batch, 3 * 6 * 5, rng.normal(size=batch * 90).astype(np.float32))
    g = st.Tensor(batch, 4 * 6 * 5, rng.normal(size=batch * 120).astype(np.float32))
    gi, gw, gb = oracle.conv2d_backward_f32(batch, 3, 6, 5, 4, (3, 3), (1, 1), (1, 1), (1, 1), x.data(),
                                            conv.weight.data(), g.data())
    got = conv.backward(x, g)
    assert_close(got.data(), gi, F32_REL, F32_ABS, "grad_input")
    assert_close(conv.weight_gradient.data(), gw, F32_REL, F32_ABS, "grad_weight")
    assert_close(conv.bias_gradient.data(), gb, F32_REL, F32_ABS, "grad_bias")
    conv.backward(x, g)  # second call accumulates
    assert_close(conv.weight_gradient.data(), 2 * np.asarray(gw), F32_REL, 2 * F32_ABS, "grad_weight twice")
    assert_close(conv.bias_gradient.data(), 2 * np.asarray(gb), F32_REL, 2 * F32_ABS, "grad_bias twice")
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        conv.backward(x, st.Tensor.zeros(batch, 7))
    assert conv.backward(st.Tensor.zeros(0, 90), st.Tensor.zeros(0, 120)).shape() == (0, 90)
