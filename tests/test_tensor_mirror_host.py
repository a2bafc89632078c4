"""Host-side behaviour of the Tensor / Conv2d mirror that never reaches the device: argument validation raises the
reference's TensorError variants before anything is launched (so these run without a GPU)."""
import numpy as np
import pytest

import spiraltorch_amd as st


def test_backend_selection():
    a = st.Tensor(2, 2, [1, 2, 3, 4])
    with pytest.raises(st.TensorError, match="BackendFailure"):
        a.matmul(a, backend="wgpu")
    with pytest.raises(st.TensorError, match="BackendFailure"):
        a.row_softmax(backend="cpu")


def test_shape_and_length_errors_come_first():
    a = st.Tensor(2, 3, np.arange(6))
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        a.matmul(st.Tensor(2, 2))
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        a.gelu_backward(st.Tensor(3, 2))
    with pytest.raises(st.TensorError, match="DataLength"):
        a.add_row_inplace([1.0, 2.0])
    with pytest.raises(st.TensorError, match="DataLength"):
        st.Tensor(2, 2, [1.0, 2.0, 3.0])
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        a.scale(float("nan"))
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        st.Tensor(1, 2, [0.0, float("inf")]).row_softmax()
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        a.matmul_prepacked(st.PackedB.from_tensor(st.Tensor(2, 4)))


def test_empty_results_need_no_device():
    assert st.Tensor.zeros(0, 4).sum_axis0().tolist() == [0.0] * 4
    assert st.Tensor.zeros(3, 0).sum_axis0().size == 0
    assert st.Tensor.zeros(0, 5).scale(2.0).shape() == (0, 5)
    assert st.Tensor.zeros(0, 5).row_softmax().shape() == (0, 5)


def test_packed_rhs_layout():
    t = st.Tensor(2, 3, [1, 2, 3, 4, 5, 6])
    packed = st.PackedB.from_tensor(t)
    assert (packed.inner(), packed.cols()) == (2, 3)
    assert packed.as_slice().tolist() == [1.0, 4.0, 2.0, 5.0, 3.0, 6.0]  # pure.rs:1299-1316: column-major


def test_conv2d_configuration_errors():
    with pytest.raises(st.TensorError, match="InvalidDimensions"):
        st.Conv2d("bad", 0, 1, (3, 3), (1, 1), (1, 1), (1, 1), (8, 8))
    conv = st.Conv2d("c", 2, 3, (3, 3), (1, 1), (1, 1), (1, 1), (4, 4))
    assert conv.weight.shape() == (3, 18) and conv.bias.shape() == (1, 3)
    assert abs(float(conv.weight.data()[0]) - 0.02) < 1e-9  # first value of the deterministic ramp, conv.rs:641-649
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        conv.forward(st.Tensor(1, 5))
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        conv.backward(st.Tensor(1, 32), st.Tensor(1, 7))
    assert conv.backward(st.Tensor.zeros(0, 32), st.Tensor.zeros(0, 48)).shape() == (0, 32)


def test_fused_operands_are_checked_finite_before_the_product():
    # pure.rs:4462, 4893-4900, 5113-5120: labels {op}_bias and {op}_residual (with ReLU a NaN bias would come out as 0)
    a, b = st.Tensor(2, 2, [1, 2, 3, 4]), st.Tensor(2, 2, [1, 0, 0, 1])
    nan_bias, good_bias = [0.0, float("nan")], [0.0, 1.0]
    bad_residual = st.Tensor(2, 2, [0.0, float("inf"), 0.0, 0.0])
    for op in ("matmul_bias_relu", "matmul_bias_gelu"):
        with pytest.raises(st.TensorError) as info:
            getattr(a, op)(b, nan_bias)
        assert info.value.kind == "NonFiniteValue" and info.value.fields["label"] == f"{op}_bias"
    for op in ("matmul_bias_add_relu", "matmul_bias_add_gelu"):
        with pytest.raises(st.TensorError) as info:
            getattr(a, op)(b, nan_bias, st.Tensor(2, 2))
        assert info.value.fields["label"] == f"{op}_bias"
        with pytest.raises(st.TensorError) as info:
            getattr(a, op)(b, good_bias, bad_residual)
        assert info.value.fields["label"] == f"{op}_residual"


def test_layer_norm_argument_checks_follow_the_reference_order():
    # layer_norm_affine_add_impl, pure.rs:3750-3800; tests pure.rs:15436-15480
    x = st.Tensor(1, 2, [0.0, 1.0])
    gamma, beta = st.Tensor(1, 2, [1.0, 1.0]), st.Tensor.zeros(1, 2)
    with pytest.raises(st.TensorError) as info:
        x.layer_norm_affine(gamma, beta, -1.0)
    assert info.value.fields["label"] == "layernorm_epsilon"
    with pytest.raises(st.TensorError, match="InvalidDimensions"):
        st.Tensor.zeros(3, 0).layer_norm_affine(st.Tensor.zeros(1, 0), st.Tensor.zeros(1, 0), 1e-5)
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        x.layer_norm_affine(st.Tensor(1, 3), beta, 1e-5)
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        x.layer_norm_affine(gamma, st.Tensor(2, 1), 1e-5)
    # a non-finite gamma is reported even when there are no rows to normalise
    with pytest.raises(st.TensorError) as info:
        st.Tensor.zeros(0, 3).layer_norm_affine(st.Tensor(1, 3, [1.0, float("nan"), 1.0]), st.Tensor.zeros(1, 3), 1e-5)
    assert info.value.fields["label"] == "layer_norm_gamma"
    with pytest.raises(st.TensorError) as info:
        x.layer_norm_affine_add(st.Tensor(1, 2, [0.0, float("inf")]), gamma, beta, 1e-5)
    assert info.value.fields["label"] == "layer_norm_residual"
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        x.layer_norm_affine_add(st.Tensor(2, 2), gamma, beta, 1e-5)
    empty = st.Tensor.zeros(0, 3).layer_norm_affine_add(st.Tensor.zeros(0, 3), st.Tensor(1, 3, [1, 1, 1]), st.Tensor.zeros(1, 3), 1e-5)
    assert empty.shape() == (0, 3)


def test_layer_norm_module_configuration():
    # normalization.rs:360-390, 423-426
    with pytest.raises(st.TensorError, match="InvalidDimensions"):
        st.LayerNorm("ln", 0, -1.0, 1e-5)
    with pytest.raises(st.TensorError, match="NonHyperbolicCurvature"):
        st.LayerNorm("ln", 4, 0.5, 1e-5)
    with pytest.raises(st.TensorError, match="NonFiniteValue"):
        st.LayerNorm("ln", 4, -1.0, 0.0)
    ln = st.LayerNorm("ln", 4, -1.0, 1e-5)
    assert ln.gamma.data().tolist() == [1.0] * 4 and ln.beta.data().tolist() == [0.0] * 4
    assert abs(ln.effective_epsilon() - 1.1e-5) < 1e-11
    assert abs(st.LayerNorm("ln", 4, -4.0, 1e-5).effective_epsilon() - 1.2e-5) < 1e-11
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        ln.forward(st.Tensor(2, 3))
    assert ln.forward(st.Tensor.zeros(0, 4)).shape() == (0, 4)


def test_linear_configuration_and_argument_checks():
    # linear.rs:49-64 (parameters), :87-94 and :109-133 (shape checks), tests :228-246, :313-327
    with pytest.raises(st.TensorError, match="InvalidDimensions"):
        st.Linear("fc", 0, 2)
    layer = st.Linear("fc", 3, 2)
    assert layer.weight.shape() == (3, 2) and layer.bias.shape() == (1, 2)
    np.testing.assert_allclose(layer.weight.data(), [0.01, 0.02, 0.03, 0.04, 0.05, 0.06], rtol=1e-6)
    assert layer.bias.data().tolist() == [0.0, 0.0]
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        layer.forward(st.Tensor(1, 4))
    with pytest.raises(st.TensorError) as info:
        layer.forward(st.Tensor(1, 3, [1.0, float("nan"), 0.5]))
    assert info.value.fields["label"] == "linear_input"
    broken = st.Linear("fc", 3, 2)
    broken.weight.data_mut()[0] = float("nan")
    with pytest.raises(st.TensorError) as info:
        broken.forward(st.Tensor(1, 3, [1.0, -2.0, 0.5]))
    assert info.value.fields["label"] == "linear_weight"
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        layer.backward(st.Tensor(2, 3), st.Tensor(1, 2))
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        layer.backward(st.Tensor(1, 4), st.Tensor(1, 2))
    with pytest.raises(st.TensorError, match="ShapeMismatch"):
        layer.backward(st.Tensor(1, 3), st.Tensor(1, 5))
    with pytest.raises(st.TensorError) as info:
        layer.backward(st.Tensor(1, 3, [1.0, -2.0, 0.5]), st.Tensor(1, 2, [float("nan"), -0.4]))
    assert info.value.fields["label"] == "linear_backward_grad_output"
    assert layer.weight_gradient is None and layer.bias_gradient is None  # no update on a rejected call
    assert layer.backward(st.Tensor.zeros(0, 3), st.Tensor.zeros(0, 2)).shape() == (0, 3)


def test_packed_transpose_shares_the_tensor_buffer():
    t = st.Tensor(2, 3, [1, 2, 3, 4, 5, 6])
    packed = st.PackedB.from_tensor_transpose(t)  # the pack of the (3, 2) transpose: inner 3, cols 2
    assert (packed.inner(), packed.cols()) == (3, 2)
    direct = st.PackedB.from_tensor(st.Tensor(3, 2, [1, 4, 2, 5, 3, 6]))
    assert packed.as_slice().tolist() == direct.as_slice().tolist() == [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
