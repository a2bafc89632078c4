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
