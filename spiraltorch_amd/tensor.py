"""Mirror of the `st-tensor` operator surface that reaches the HIP backend.

`Tensor` is the reference's 2-D row-major f32 matrix (crates/st-tensor/src/pure.rs:1406-1411); the
methods below are the ones whose `MatmulBackend::GpuHip` arm exists in the reference
(pure.rs:2008-2556, 4411-4634) plus `scaled_dot_attention` (pure.rs:4061-4354) and the Conv2d layer
(crates/st-nn/src/layers/conv.rs:607-969), which this build adds to the HIP backend.  Method names and
keyword arguments follow the Python binding (bindings/st-py/src/tensor.rs:970-1299).

Only `backend="hip"` (or "auto", which selects hip) is served.  There is no CPU path in this package:
every method runs on the GPU or raises.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np

from . import hip
from . import _lib


class TensorError(Exception):
    """`TensorError` variants of the reference that this surface can raise; `kind` is the variant name."""

    def __init__(self, kind: str, message: str, **fields):
        super().__init__(f"{kind}: {message}")
        self.kind = kind
        self.message = message
        self.fields = fields


def _resolve_backend(backend: Optional[str]) -> str:
    label = "auto" if backend is None else backend
    if label in ("auto", "hip", "rocm"):
        return "hip"
    raise TensorError("BackendFailure", f"backend '{label}' is not provided by this package; only 'hip' is",
                      backend=label)


def _backend_failure(err: hip.HipErr) -> TensorError:
    # pure.rs:2158-2163 wraps HIP errors as BackendFailure{backend:"hip", message}; the finite checks the
    # Tensor layer performs itself surface as NonFiniteValue (pure.rs:5521-5533).
    if err.status == _lib.ERR_NONFINITE:
        label = err.message.split(" in ", 1)[-1].split(":", 1)[0]
        return TensorError("NonFiniteValue", err.message, label=label)
    return TensorError("BackendFailure", err.message, backend="hip")


class PackedB:
    """Right-hand operand packed once for repeated matmuls (pure.rs:1285-1400): column-major, i.e. the (cols, inner)
    row-major transpose of the (inner, cols) matrix.  Its device copy is made on first use and kept."""

    def __init__(self, inner: int, cols: int, buf: np.ndarray):
        self._inner, self._cols, self._buf = int(inner), int(cols), buf
        self._dev: Optional[hip.DeviceBuffer] = None

    @classmethod
    def from_tensor(cls, tensor: "Tensor") -> "PackedB":
        """PackedB::from_row_major, pure.rs:1299-1316: packed[c*rows + r] = data[r*cols + c]."""
        return cls(tensor.rows, tensor.cols, np.ascontiguousarray(tensor.numpy().T).reshape(-1))

    @classmethod
    def from_tensor_on_device(cls, tensor: "Tensor") -> "PackedB":
        """The same packing done by the GPU from the tensor's device copy (st_hip_pack_rhs_f32_dev): nothing crosses
        the bus for a weight that already lives on the device.  The host copy is fetched only if `as_slice` asks."""
        pack = cls(tensor.rows, tensor.cols, None)
        try:
            pack._dev = hip.DeviceBuffer(max(len(tensor), 1) * 4)
            if len(tensor):
                hip.pack_rhs_f32_dev(tensor.rows, tensor.cols, tensor._device(), pack._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return pack

    @classmethod
    def from_tensor_transpose(cls, tensor: "Tensor") -> "PackedB":
        """PackedB::from_tensor_transpose (crates/st-nn/src/module.rs:684-691): the pack of the transpose.  Packing is
        itself a transposition, so the packed transpose of a (rows, cols) tensor is the tensor's own row-major buffer,
        shared here, not copied."""
        pack = cls(tensor.cols, tensor.rows, tensor._host)
        pack._dev = tensor._dev
        pack._source = tensor
        return pack

    def inner(self) -> int:
        return self._inner

    def cols(self) -> int:
        return self._cols

    def as_slice(self) -> np.ndarray:
        if self._buf is None:
            source = getattr(self, "_source", None)
            self._buf = (np.array(source.data()) if source is not None
                         else self._dev.to_array(np.float32, self._inner * self._cols))
        return self._buf

    def _device(self) -> hip.DeviceBuffer:
        if self._dev is None:
            source = getattr(self, "_source", None)
            self._dev = source._device() if source is not None else hip.DeviceBuffer.from_array(self._buf)
        return self._dev


class Tensor:
    """2-D row-major float32 matrix (pure.rs:1406-1411) with a device-resident twin.

    A tensor built from host values is uploaded the first time an operator needs it and the device copy is kept;
    an operator's result is born on the device and is downloaded only when its values are read (`data()`,
    `numpy()`).  A chain of operators therefore costs one upload per input and one download at the end, instead of
    the reference HIP backend's three allocations and three copies per call
    (crates/st-backend-hip/src/real.rs:718-756).  `data()` returns a read-only view; `data_mut()` returns a writable
    one and drops the device copy."""

    def __init__(self, rows: int, cols: int, data=None):
        if data is None:
            buf = np.zeros(rows * cols, dtype=np.float32)
        else:
            buf = np.array(data, dtype=np.float32).reshape(-1)
            if buf.size != rows * cols:
                raise TensorError("DataLength", f"expected {rows * cols} values, got {buf.size}",
                                  expected=rows * cols, got=buf.size)
        self.rows, self.cols = int(rows), int(cols)
        self._host: Optional[np.ndarray] = buf
        self._dev: Optional[hip.DeviceBuffer] = None
        self._finite: Optional[bool] = None  # None: not examined yet

    @classmethod
    def zeros(cls, rows: int, cols: int) -> "Tensor":
        return cls(rows, cols)

    @classmethod
    def from_numpy(cls, array) -> "Tensor":
        a = np.asarray(array, dtype=np.float32)
        if a.ndim != 2:
            raise TensorError("InvalidDimensions", "expected a 2-D array", rows=a.ndim, cols=2)
        return cls(a.shape[0], a.shape[1], a)

    @classmethod
    def _on_device_result(cls, rows: int, cols: int) -> "Tensor":
        """A result tensor that exists only on the device so far."""
        out = cls.__new__(cls)
        out.rows, out.cols = int(rows), int(cols)
        out._host = None
        try:
            out._dev = hip.DeviceBuffer(max(out.rows * out.cols, 1) * 4)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        out._finite = None
        return out

    def shape(self) -> Tuple[int, int]:
        return (self.rows, self.cols)

    def __len__(self) -> int:
        return self.rows * self.cols

    def is_device_resident(self) -> bool:
        return self._dev is not None

    def _host_values(self) -> np.ndarray:
        if self._host is None:
            try:
                self._host = self._dev.to_array(np.float32, self.rows * self.cols)
            except hip.HipErr as err:
                raise _backend_failure(err) from err
        return self._host

    def data(self) -> np.ndarray:
        """The values, row-major, as a read-only array (downloaded once if they live on the device)."""
        view = self._host_values().view()
        view.flags.writeable = False
        return view

    def data_mut(self) -> np.ndarray:
        """Writable values (Tensor::data_mut): the device copy is dropped and re-made on the next use."""
        values = self._host_values()
        self._dev = None
        self._finite = None
        return values

    def numpy(self) -> np.ndarray:
        return self.data().reshape(self.rows, self.cols)

    def _device(self) -> hip.DeviceBuffer:
        if self._dev is None:
            try:
                self._dev = hip.DeviceBuffer.from_array(self._host)
            except hip.HipErr as err:
                raise _backend_failure(err) from err
        return self._dev

    def _require_finite(self, label: str) -> None:
        """validate_finite_tensor_util_slice (pure.rs:5521-5533) on an operand, wherever it lives; the answer is
        remembered, so an operator's validated result is not examined again when it feeds the next operator."""
        if self._finite is None:
            if self._host is not None:
                bad = self._host[~np.isfinite(self._host)]
                self._finite = bad.size == 0
                if not self._finite:
                    raise TensorError("NonFiniteValue", f"non-finite value encountered in {label}: {bad[0]}", label=label)
            else:
                self._validate_result(label)
        elif not self._finite:
            raise TensorError("NonFiniteValue", f"non-finite value encountered in {label}", label=label)

    def _validate_result(self, label: str) -> "Tensor":
        """The post-operator finite check (pure.rs:2169, 4537) on the device: sixteen bytes come back, not the tensor."""
        try:
            found, _, value = hip.count_nonfinite_f32_dev(self.rows * self.cols, self._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        self._finite = found == 0
        if found:
            raise TensorError("NonFiniteValue", f"non-finite value encountered in {label}: {value}", label=label)
        return self

    @staticmethod
    def _row_vector(values, expected: int) -> "Tensor":
        """A bias given as a Tensor is used (and kept on the device) as it is; anything else becomes a 1×n Tensor."""
        if isinstance(values, Tensor):
            if values.rows * values.cols != expected:
                raise TensorError("DataLength", f"expected {expected} values, got {values.rows * values.cols}",
                                  expected=expected, got=values.rows * values.cols)
            return values
        flat = np.ascontiguousarray(np.asarray(values, dtype=np.float32)).reshape(-1)
        if flat.size != expected:
            raise TensorError("DataLength", f"expected {expected} values, got {flat.size}", expected=expected,
                              got=flat.size)
        return Tensor(1, expected, flat)

    # ---- dense matmul family ---------------------------------------------------------------------
    def _check_inner(self, other: "Tensor") -> None:
        if self.cols != other.rows:
            raise TensorError("ShapeMismatch", f"left {self.shape()} right {other.shape()}",
                              left=self.shape(), right=other.shape())

    def matmul(self, other: "Tensor", *, backend: Optional[str] = None) -> "Tensor":
        """C = A·B — Tensor::matmul_with_backend, pure.rs:2013-2197."""
        return self.matmul_scaled(other, 1.0, backend=backend, _op="matmul")

    def matmul_scaled(self, other: "Tensor", scale: float, *, backend: Optional[str] = None,
                      _op: str = "matmul_scaled") -> "Tensor":
        """C = (A·B)·scale — pure.rs:2200-2369."""
        _resolve_backend(backend)
        self._check_inner(other)
        out = Tensor._on_device_result(self.rows, other.cols)
        try:
            hip.gemm_f32_dev(self.rows, other.cols, self.cols, scale, False, self._device(), other._device(), out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out._validate_result(f"{_op}_output")  # pure.rs:2169

    def matmul_lhs_transpose_scaled(self, other: "Tensor", scale: float, *,
                                    backend: Optional[str] = None) -> "Tensor":
        """C = (Aᵀ·B)·scale with A stored (k, m) — pure.rs:2372-2556."""
        _resolve_backend(backend)
        if self.rows != other.rows:
            raise TensorError("ShapeMismatch", f"left {self.shape()} right {other.shape()}",
                              left=self.shape(), right=other.shape())
        out = Tensor._on_device_result(self.cols, other.cols)
        try:
            hip.gemm_f32_dev(self.cols, other.cols, self.rows, scale, True, self._device(), other._device(), out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out._validate_result("matmul_lhs_transpose_scaled_output")

    def _fused(self, other: "Tensor", bias, residual: Optional["Tensor"], activation, label: str) -> "Tensor":
        self._check_inner(other)
        bias = Tensor._row_vector(bias, other.cols)
        if residual is not None and residual.shape() != (self.rows, other.cols):
            raise TensorError("ShapeMismatch", f"left {residual.shape()} right {(self.rows, other.cols)}",
                              left=residual.shape(), right=(self.rows, other.cols))
        # Operand checks made before the product (pure.rs:4462, 4893-4900, 5113-5120): with ReLU a NaN bias would
        # otherwise come out as a finite 0.
        op = label[:-len("_output")]
        bias._require_finite(f"{op}_bias")
        if residual is not None:
            residual._require_finite(f"{op}_residual")
        out = Tensor._on_device_result(self.rows, other.cols)
        try:
            hip.gemm_bias_act_f32_dev(self.rows, other.cols, self.cols, activation, self._device(), other._device(),
                                      bias._device(), None if residual is None else residual._device(), out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out._validate_result(label)  # pure.rs:4537

    def matmul_bias_relu(self, other: "Tensor", bias, *, backend: Optional[str] = None) -> "Tensor":
        """relu(A·B + bias) — pure.rs:4411-4550."""
        _resolve_backend(backend)
        return self._fused(other, bias, None, hip.GemmActivation.Relu, "matmul_bias_relu_output")

    def matmul_bias_gelu(self, other: "Tensor", bias, *, backend: Optional[str] = None) -> "Tensor":
        _resolve_backend(backend)
        return self._fused(other, bias, None, hip.GemmActivation.Gelu, "matmul_bias_gelu_output")

    def matmul_bias_add_relu(self, other: "Tensor", bias, residual: "Tensor", *,
                             backend: Optional[str] = None) -> "Tensor":
        _resolve_backend(backend)
        return self._fused(other, bias, residual, hip.GemmActivation.Relu, "matmul_bias_add_relu_output")

    def matmul_bias_add_gelu(self, other: "Tensor", bias, residual: "Tensor", *,
                             backend: Optional[str] = None) -> "Tensor":
        _resolve_backend(backend)
        return self._fused(other, bias, residual, hip.GemmActivation.Gelu, "matmul_bias_add_gelu_output")

    def matmul_prepacked(self, packed: "PackedB", *, backend: Optional[str] = None) -> "Tensor":
        """C = A·B with B prepacked — pure.rs:2559-2575."""
        return self._prepacked(packed, None, "matmul_prepacked_output", backend)

    def matmul_prepacked_bias(self, packed: "PackedB", bias, *, backend: Optional[str] = None) -> "Tensor":
        """C = A·B + bias with B prepacked — pure.rs:2577-2757 (what Linear::forward calls, linear.rs:96-104)."""
        if self.cols == packed.inner():
            bias = Tensor._row_vector(bias, packed.cols())
            bias._require_finite("matmul_prepacked_bias_bias")
        return self._prepacked(packed, bias, "matmul_prepacked_bias_output", backend)

    def _prepacked(self, packed: "PackedB", bias, label: str, backend: Optional[str]) -> "Tensor":
        _resolve_backend(backend)
        if self.cols != packed.inner():
            raise TensorError("ShapeMismatch", f"left {self.shape()} right {(packed.inner(), packed.cols())}",
                              left=self.shape(), right=(packed.inner(), packed.cols()))
        out = Tensor._on_device_result(self.rows, packed.cols())
        try:
            hip.gemm_prepacked_bias_act_f32_dev(self.rows, packed.cols(), self.cols, 0, self._device(),
                                                packed._device(), None if bias is None else bias._device(), None,
                                                out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out._validate_result(label)

    # ---- tensor utilities ------------------------------------------------------------------------
    def _elementwise(self, run, rows: int, cols: int) -> "Tensor":
        out = Tensor._on_device_result(rows, cols)
        try:
            run(out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out

    def row_softmax(self, *, backend: Optional[str] = None) -> "Tensor":
        """Row-wise softmax — Tensor::row_softmax_with_backend, pure.rs:3282-3330 (inputs must be finite)."""
        _resolve_backend(backend)
        self._require_finite("row_softmax_input")
        if len(self) == 0:
            return Tensor.zeros(self.rows, self.cols)
        out = self._elementwise(lambda y: hip.row_softmax_f32_dev(self.rows, self.cols, self._device(), y), self.rows,
                                self.cols)
        return out._validate_result("row_softmax_output")

    def gelu(self, *, backend: Optional[str] = None) -> "Tensor":
        """gelu(self) — Gelu::forward, crates/st-nn/src/layers/gelu.rs:78-94."""
        _resolve_backend(backend)
        if len(self) == 0:
            return Tensor.zeros(self.rows, self.cols)
        out = self._elementwise(lambda y: hip.gelu_f32_dev(len(self), self._device(), y), self.rows, self.cols)
        return out._validate_result("gelu_output")

    def gelu_backward(self, grad_output: "Tensor", *, backend: Optional[str] = None) -> "Tensor":
        """gelu'(self) ⊙ grad_output — Tensor::gelu_backward_with_backend, pure.rs:6459-6560."""
        _resolve_backend(backend)
        if self.shape() != grad_output.shape():
            raise TensorError("ShapeMismatch", f"left {self.shape()} right {grad_output.shape()}",
                              left=self.shape(), right=grad_output.shape())
        if len(self) == 0:
            return Tensor.zeros(self.rows, self.cols)
        return self._elementwise(lambda y: hip.gelu_backward_f32_dev(len(self), self._device(), grad_output._device(), y),
                                 self.rows, self.cols)

    def scale(self, value: float, *, backend: Optional[str] = None) -> "Tensor":
        """self · value — Tensor::scale_with_backend, pure.rs:5517-5620 (value must be finite)."""
        _resolve_backend(backend)
        if not np.isfinite(value):
            raise TensorError("NonFiniteValue", f"non-finite value encountered in scale_factor: {value}",
                              label="scale_factor")
        if len(self) == 0:
            return Tensor.zeros(self.rows, self.cols)
        return self._elementwise(lambda y: hip.scale_f32_dev(len(self), self._device(), float(value), y), self.rows,
                                 self.cols)

    def add_row_inplace(self, bias, *, backend: Optional[str] = None) -> None:
        """self[r, :] += bias — Tensor::add_row_inplace_with_backend, pure.rs:6201-6290."""
        _resolve_backend(backend)
        bias = Tensor._row_vector(bias, self.cols)
        if len(self) == 0:
            return
        try:
            hip.add_row_f32_dev(self.rows, self.cols, self._device(), bias._device())
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        self._host = None   # the device copy is now the tensor
        self._finite = None

    def sum_axis0(self, *, backend: Optional[str] = None) -> np.ndarray:
        """Column sums — Tensor::sum_axis0_with_backend, pure.rs:7009-7116."""
        return self.sum_axis0_scaled(1.0, backend=backend)

    def sum_axis0_scaled(self, scale: float, *, backend: Optional[str] = None) -> np.ndarray:
        """scale · column sums — Tensor::sum_axis0_scaled_with_backend, pure.rs:7118-7230 (a Vec<f32> there, a host
        array here)."""
        _resolve_backend(backend)
        if self.cols == 0:
            return np.zeros(0, dtype=np.float32)
        if self.rows == 0:
            return np.zeros(self.cols, dtype=np.float32)
        out = self._elementwise(lambda y: hip.sum_axis0_f32_dev(self.rows, self.cols, self._device(), float(scale), y),
                                1, self.cols)
        return np.array(out.data())

    def layer_norm_affine(self, gamma: "Tensor", beta: "Tensor", epsilon: float, *,
                          backend: Optional[str] = None) -> "Tensor":
        """Layer normalisation over the columns with affine parameters — Tensor::layer_norm_affine_with_backend,
        pure.rs:3702-3720; arithmetic of layer_norm_cpu, pure.rs:4008-4058."""
        return self._layer_norm(None, gamma, beta, epsilon, backend)

    def layer_norm_affine_add(self, residual: "Tensor", gamma: "Tensor", beta: "Tensor", epsilon: float, *,
                              backend: Optional[str] = None) -> "Tensor":
        """Layer normalisation of `self + residual` — Tensor::layer_norm_affine_add_with_backend, pure.rs:3722-3748."""
        return self._layer_norm(residual, gamma, beta, epsilon, backend)

    def _layer_norm(self, residual: Optional["Tensor"], gamma: "Tensor", beta: "Tensor", epsilon: float,
                    backend: Optional[str]) -> "Tensor":
        # Checks in the order of layer_norm_affine_add_impl, pure.rs:3750-3800.
        _resolve_backend(backend)
        if not np.isfinite(epsilon) or epsilon < 0.0:
            raise TensorError("NonFiniteValue", f"non-finite value encountered in layernorm_epsilon: {epsilon}",
                              label="layernorm_epsilon")
        if self.cols == 0:
            raise TensorError("InvalidDimensions", f"rows {self.rows} cols {self.cols}", rows=self.rows, cols=self.cols)
        for t in (gamma, beta):
            if t.shape() != (1, self.cols):
                raise TensorError("ShapeMismatch", f"left {t.shape()} right {(1, self.cols)}", left=t.shape(),
                                  right=(1, self.cols))
        self._require_finite("layer_norm_input")
        gamma._require_finite("layer_norm_gamma")
        beta._require_finite("layer_norm_beta")
        if residual is not None:
            if residual.shape() != self.shape():
                raise TensorError("ShapeMismatch", f"left {residual.shape()} right {self.shape()}",
                                  left=residual.shape(), right=self.shape())
            residual._require_finite("layer_norm_residual")
        if self.rows == 0:
            return Tensor.zeros(self.rows, self.cols)
        out = self._elementwise(
            lambda y: hip.layer_norm_f32_dev(self.rows, self.cols, self._device(),
                                             None if residual is None else residual._device(), gamma._device(),
                                             beta._device(), float(epsilon), y, None), self.rows, self.cols)
        return out._validate_result("layer_norm_output")

    def _sum_axis0_tensor(self, scale: float) -> "Tensor":
        """scale · column sums as a (1, cols) tensor that stays on the device."""
        return self._elementwise(lambda y: hip.sum_axis0_f32_dev(self.rows, self.cols, self._device(), float(scale), y),
                                 1, self.cols)

    # ---- attention -------------------------------------------------------------------------------
    def scaled_dot_attention(self, keys: "Tensor", values: "Tensor", *, contexts: int, sequence: int,
                             scale: float, z_bias: Optional["Tensor"] = None,
                             attn_bias: Optional["Tensor"] = None, causal: bool = False,
                             backend: Optional[str] = None) -> "Tensor":
        """softmax(QKᵀ·scale + biases)·V per context — pure.rs:4083-4354.  `causal` is this build's
        addition (keys 0..=query, crates/st-core/src/backend/cuda_attention.cu:160-164)."""
        _resolve_backend(backend)
        expected_rows = contexts * sequence
        for t in (self, keys, values):
            if t.rows != expected_rows or t.cols != self.cols:
                raise TensorError("ShapeMismatch", f"left {t.shape()} right {(expected_rows, self.cols)}",
                                  left=t.shape(), right=(expected_rows, self.cols))
        if z_bias is not None and z_bias.shape() != (contexts, sequence):
            raise TensorError("ShapeMismatch", f"left {z_bias.shape()} right {(contexts, sequence)}",
                              left=z_bias.shape(), right=(contexts, sequence))
        if attn_bias is not None and attn_bias.shape() != (expected_rows, sequence):
            raise TensorError("ShapeMismatch", f"left {attn_bias.shape()} right {(expected_rows, sequence)}",
                              left=attn_bias.shape(), right=(expected_rows, sequence))
        # Finite checks in the order of pure.rs:4148-4157.
        if not np.isfinite(scale):
            raise TensorError("NonFiniteValue", f"non-finite value encountered in scaled_dot_attention_scale: {scale}",
                              label="scaled_dot_attention_scale")
        for t, name in ((self, "query"), (keys, "key"), (values, "value"), (z_bias, "z_bias"), (attn_bias, "attn_bias")):
            if t is not None:
                t._require_finite(f"scaled_dot_attention_{name}")
        if expected_rows == 0 or self.cols == 0:
            return Tensor.zeros(expected_rows, self.cols)  # pure.rs:4171-4193
        out = Tensor._on_device_result(expected_rows, self.cols)
        try:
            hip.attention_f32_dev(contexts, sequence, self.cols, scale, causal, self._device(), keys._device(),
                                  values._device(), None if z_bias is None else z_bias._device(),
                                  None if attn_bias is None else attn_bias._device(), out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out._validate_result("scaled_dot_attention_output")  # pure.rs:4206-4210


class Conv2d:
    """Conv2d layer of crates/st-nn/src/layers/conv.rs:607-1013 (forward and backward), with the optional fused
    activation the reference composes as a separate Relu layer.  `backward` accumulates into `weight_gradient` and
    `bias_gradient` the way Parameter::accumulate_euclidean does (crates/st-nn/src/module.rs:329-350)."""

    def __init__(self, name: str, in_channels: int, out_channels: int, kernel, stride, padding, dilation,
                 input_hw, activation: int = hip.ACT_NONE):
        self.name = name
        self.in_channels, self.out_channels = int(in_channels), int(out_channels)
        self.kernel, self.stride = tuple(kernel), tuple(stride)
        self.padding, self.dilation = tuple(padding), tuple(dilation)
        self.input_hw = tuple(input_hw)
        self.activation = activation
        for value, label in ((in_channels, "in_channels"), (out_channels, "out_channels"),
                             (self.kernel[0], "kernel_h"), (self.kernel[1], "kernel_w"),
                             (self.stride[0], "stride_h"), (self.stride[1], "stride_w"),
                             (self.dilation[0], "dilation_h"), (self.dilation[1], "dilation_w"),
                             (self.input_hw[0], "input_height"), (self.input_hw[1], "input_width")):
            if value <= 0:
                raise TensorError("InvalidDimensions", f"{label} must be positive", rows=value, cols=0)
        span = self.in_channels * self.kernel[0] * self.kernel[1]
        # Deterministic default weight ramp and zero bias of Conv2d::new (conv.rs:641-649).
        seed = np.float32(0.02)
        ramp = np.empty(self.out_channels * span, dtype=np.float32)
        for i in range(ramp.size):
            ramp[i] = seed
            seed = np.float32(max(np.fmod(np.float32(seed * np.float32(1.57)), np.float32(0.15)), np.float32(5e-3)))
        self.weight = Tensor(self.out_channels, span, ramp)
        self.bias = Tensor.zeros(1, self.out_channels)
        self.weight_gradient: Optional[Tensor] = None
        self.bias_gradient: Optional[Tensor] = None
        self.output_hw()  # validates the configuration once (conv.rs:662)

    def output_hw(self) -> Tuple[int, int]:
        try:
            return hip.conv2d_output_hw(self.input_hw[0], self.input_hw[1], self.kernel, self.stride, self.padding,
                                        self.dilation)
        except hip.HipErr as err:
            raise TensorError("InvalidDimensions", err.message) from err

    def forward(self, input: Tensor) -> Tensor:
        h, w = self.input_hw
        if input.cols != self.in_channels * h * w:
            raise TensorError("ShapeMismatch", f"left {input.shape()} right {(input.rows, self.in_channels * h * w)}",
                              left=input.shape(), right=(input.rows, self.in_channels * h * w))
        oh, ow = self.output_hw()
        if input.rows == 0:
            return Tensor.zeros(0, self.out_channels * oh * ow)  # conv.rs:4132-4137
        out = Tensor._on_device_result(input.rows, self.out_channels * oh * ow)
        try:
            hip.conv2d_bias_act_f32_dev(input.rows, self.in_channels, h, w, self.out_channels, self.kernel, self.stride,
                                        self.padding, self.dilation, self.activation, input._device(),
                                        self.weight._device(), self.bias._device(), out._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        return out

    def backward(self, input: Tensor, grad_output: Tensor) -> Tensor:
        """Conv2d::backward (conv.rs:971-992, 780-811): returns the input gradient and accumulates the weight and
        bias gradients, both scaled by 1/batch.  Defined for activation None, as in the reference."""
        if self.activation != hip.ACT_NONE:
            raise TensorError("BackendFailure", "backward is defined for a Conv2d without fused activation",
                              backend="hip")
        h, w = self.input_hw
        if input.cols != self.in_channels * h * w:
            raise TensorError("ShapeMismatch", f"left {(1, input.cols)} right {(1, self.in_channels * h * w)}",
                              left=(1, input.cols), right=(1, self.in_channels * h * w))
        oh, ow = self.output_hw()
        if grad_output.shape() != (input.rows, self.out_channels * oh * ow):
            raise TensorError("ShapeMismatch",
                              f"left {grad_output.shape()} right {(input.rows, self.out_channels * oh * ow)}",
                              left=grad_output.shape(), right=(input.rows, self.out_channels * oh * ow))
        if input.rows == 0:
            return Tensor.zeros(0, input.cols)
        grad_input = Tensor._on_device_result(input.rows, input.cols)
        grad_weight = Tensor._on_device_result(*self.weight.shape())
        grad_bias = Tensor._on_device_result(1, self.out_channels)
        shape = (input.rows, self.in_channels, h, w, self.out_channels, self.kernel, self.stride, self.padding,
                 self.dilation)
        scale = 1.0 / input.rows  # conv.rs:793,799
        try:
            hip.conv2d_grad_weight_f32_dev(*shape, input._device(), grad_output._device(), scale, grad_weight._dev)
            hip.conv2d_grad_bias_f32_dev(*shape, grad_output._device(), scale, grad_bias._dev)
            hip.conv2d_grad_input_f32_dev(*shape, grad_output._device(), self.weight._device(), grad_input._dev)
        except hip.HipErr as err:
            raise _backend_failure(err) from err
        for name, update in (("weight_gradient", grad_weight), ("bias_gradient", grad_bias)):
            existing = getattr(self, name)
            if existing is None:
                setattr(self, name, update)
            else:
                existing.data_mut()[:] += update.data()
        return grad_input

    def zero_accumulators(self) -> None:
        self.weight_gradient = None
        self.bias_gradient = None


def _accumulate(existing: Optional["Tensor"], update: "Tensor") -> "Tensor":
    """Parameter::accumulate_euclidean (crates/st-nn/src/module.rs:329-350): the first gradient is adopted as it is
    (on the device), later ones are added to it."""
    if existing is None:
        return update
    existing.data_mut()[:] += update.data()
    return existing


class Linear:
    """Fully-connected layer of crates/st-nn/src/layers/linear.rs:41-168: weight (input_dim, output_dim), bias
    (1, output_dim), y = x·W + b.  `forward` multiplies by the weight prepacked once per parameter value
    (Parameter::ensure_matmul_pack, crates/st-nn/src/module.rs:674) — packed on the device from the weight's device
    copy —, `backward` returns the input gradient and accumulates the weight and bias gradients scaled by 1/batch.
    Inputs, results and gradients stay on the device."""

    def __init__(self, name: str, input_dim: int, output_dim: int):
        if input_dim <= 0 or output_dim <= 0:
            raise TensorError("InvalidDimensions", "input_dim and output_dim must be positive", rows=input_dim,
                              cols=output_dim)
        self.name = name
        # Deterministic small parameters of Linear::new (linear.rs:56-63): 0.01, 0.02, ... accumulated in f32.
        ramp = np.cumsum(np.full(input_dim * output_dim, 0.01, dtype=np.float32), dtype=np.float32)
        self.weight = Tensor(input_dim, output_dim, ramp)
        self.bias = Tensor.zeros(1, output_dim)
        self.weight_gradient: Optional[Tensor] = None
        self.bias_gradient: Optional[Tensor] = None
        self._pack: Optional[PackedB] = None
        self._pack_transpose: Optional[PackedB] = None
        self._packed_from: Optional[Tensor] = None

    def load_weight(self, weight: Tensor, bias: Optional[Tensor] = None) -> None:
        """Parameter::load_value (module.rs:698-703): replaces the values and drops the cached packs."""
        if weight.shape() != self.weight.shape():
            raise TensorError("ShapeMismatch", f"left {weight.shape()} right {self.weight.shape()}",
                              left=weight.shape(), right=self.weight.shape())
        self.weight = weight
        if bias is not None:
            if bias.shape() != self.bias.shape():
                raise TensorError("ShapeMismatch", f"left {bias.shape()} right {self.bias.shape()}",
                                  left=bias.shape(), right=self.bias.shape())
            self.bias = bias
        self._pack = self._pack_transpose = self._packed_from = None

    def _packs(self) -> Tuple[PackedB, PackedB]:
        if self._packed_from is not self.weight or self._pack is None:
            self._pack = PackedB.from_tensor_on_device(self.weight)
            self._pack_transpose = PackedB.from_tensor_transpose(self.weight)
            self._packed_from = self.weight
        return self._pack, self._pack_transpose

    def _validate_parameters(self) -> None:
        self.weight._require_finite("linear_weight")
        self.bias._require_finite("linear_bias")

    @staticmethod
    def _relabel(err: TensorError, label: str) -> TensorError:
        if err.kind == "NonFiniteValue":  # relabel_non_finite, linear.rs:30-37
            return TensorError("NonFiniteValue", f"non-finite value encountered in {label}", label=label)
        return err

    def forward(self, input: Tensor) -> Tensor:
        """Linear::forward, linear.rs:87-107."""
        if input.cols != self.weight.rows:
            raise TensorError("ShapeMismatch", f"left {input.shape()} right {self.weight.shape()}",
                              left=input.shape(), right=self.weight.shape())
        input._require_finite("linear_input")
        self._validate_parameters()
        pack, _ = self._packs()
        try:
            return input.matmul_prepacked_bias(pack, self.bias)
        except TensorError as err:
            raise Linear._relabel(err, "linear_output") from err

    def backward(self, input: Tensor, grad_output: Tensor) -> Tensor:
        """Linear::backward, linear.rs:109-168: grad_W = inputᵀ·grad_output / batch (lhsᵀ GEMM), grad_b = column sums
        of grad_output / batch, grad_input = grad_output·Wᵀ through the pack of the transpose."""
        if input.rows != grad_output.rows:
            raise TensorError("ShapeMismatch", f"left {input.shape()} right {grad_output.shape()}",
                              left=input.shape(), right=grad_output.shape())
        if input.cols != self.weight.rows:
            raise TensorError("ShapeMismatch", f"left {input.shape()} right {self.weight.shape()}",
                              left=input.shape(), right=self.weight.shape())
        if grad_output.cols != self.weight.cols:
            raise TensorError("ShapeMismatch", f"left {grad_output.shape()} right {(input.rows, self.weight.cols)}",
                              left=grad_output.shape(), right=(input.rows, self.weight.cols))
        input._require_finite("linear_backward_input")
        grad_output._require_finite("linear_backward_grad_output")
        self._validate_parameters()
        if input.rows == 0:
            return Tensor.zeros(0, input.cols)
        scale = 1.0 / input.rows
        steps = (("linear_weight_grad", lambda: input.matmul_lhs_transpose_scaled(grad_output, scale)),
                 ("linear_bias_grad", lambda: grad_output._sum_axis0_tensor(scale)._validate_result("linear_bias_grad")),
                 ("linear_input_grad", lambda: grad_output.matmul_prepacked(self._packs()[1])))
        results = []
        for label, run in steps:
            try:
                results.append(run())
            except TensorError as err:
                raise Linear._relabel(err, label) from err
        grad_w, grad_b, grad_input = results
        self.weight_gradient = _accumulate(self.weight_gradient, grad_w)
        self.bias_gradient = _accumulate(self.bias_gradient, grad_b)
        return grad_input

    def zero_accumulators(self) -> None:
        self.weight_gradient = None
        self.bias_gradient = None


class LayerNorm:
    """LayerNorm of crates/st-nn/src/layers/normalization.rs:349-427, 1956-1969 (forward): gamma = 1 and beta = 0
    initially, and the epsilon handed to the tensor operator is epsilon·(1 + 0.1·sqrt(−curvature))."""

    def __init__(self, name: str, features: int, curvature: float, epsilon: float):
        if features <= 0:
            raise TensorError("InvalidDimensions", "features must be positive", rows=1, cols=features)
        if not np.isfinite(curvature) or curvature >= 0.0:
            raise TensorError("NonHyperbolicCurvature", f"curvature {curvature} is not negative", curvature=curvature)
        if not np.isfinite(epsilon) or epsilon <= 0.0:
            raise TensorError("NonFiniteValue", f"non-finite value encountered in layernorm_epsilon: {epsilon}",
                              label="layernorm_epsilon")
        self.name, self.features = name, int(features)
        self.curvature, self.epsilon = float(curvature), float(epsilon)
        self.gamma = Tensor(1, features, np.ones(features, dtype=np.float32))
        self.beta = Tensor.zeros(1, features)

    def effective_epsilon(self) -> float:
        scale = np.sqrt(np.float32(-self.curvature))
        return float(np.float32(self.epsilon) * (np.float32(1.0) + scale * np.float32(0.1)))

    def forward(self, input: Tensor) -> Tensor:
        if input.cols != self.features:
            raise TensorError("ShapeMismatch", f"left {input.shape()} right {(input.rows, self.features)}",
                              left=input.shape(), right=(input.rows, self.features))
        if input.rows == 0:
            return Tensor.zeros(0, input.cols)
        return input.layer_norm_affine(self.gamma, self.beta, self.effective_epsilon())
