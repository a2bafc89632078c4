"""Python mirror of the `st_backend_hip` crate's public functions, on top of libsthip.so.

Names, argument order and error behaviour follow crates/st-backend-hip/src/lib.rs:607-799 of the
reference (gemm_f32, gemm_scaled_f32, gemm_lhs_transpose_scaled_f32, gemm_bias_activation_f32) so that
tests written against the Rust crate read the same here.  Buffers are flat float32 numpy arrays standing
in for Rust slices; `out` is written in place.  Everything executes on the GPU: a missing library or
device raises HipErr, nothing falls back to the CPU.
"""
from __future__ import annotations

import ctypes
import enum
from typing import Optional

import numpy as np

from . import _lib


class HipErr(Exception):
    """`HipErr::{NotEnabled, Other}` of crates/st-backend-hip/src/lib.rs:14-20, plus the status code."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status
        self.kind = "NotEnabled" if status == _lib.ERR_NOT_ENABLED else "Other"
        self.message = message


class GemmActivation(enum.IntEnum):
    """Wire codes of crates/st-backend-hip/src/lib.rs:29-34."""

    Relu = 1
    Gelu = 2


ACT_NONE = 0


def _check(status: int) -> None:
    if status != _lib.OK:
        raise HipErr(status, _lib.last_error())


def _f32(array, name: str) -> np.ndarray:
    a = np.asarray(array)
    if a.dtype != np.float32 or not a.flags["C_CONTIGUOUS"]:
        raise TypeError(f"{name} must be a C-contiguous float32 array")
    return a


def _u16(array, name: str) -> np.ndarray:
    a = np.asarray(array)
    if a.dtype != np.uint16 or not a.flags["C_CONTIGUOUS"]:
        raise TypeError(f"{name} must be a C-contiguous uint16 (bf16 bit pattern) array")
    return a


def _out(array, name: str) -> np.ndarray:
    if not isinstance(array, np.ndarray) or array.dtype != np.float32 or not array.flags["C_CONTIGUOUS"] \
            or not array.flags["WRITEABLE"]:
        raise TypeError(f"{name} must be a writable C-contiguous float32 ndarray")
    return array


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


# ---- runtime -------------------------------------------------------------------------------------

def real_backend_compiled() -> bool:
    return bool(_lib.load().st_hip_real_backend_compiled())


def init() -> None:
    _check(_lib.load().st_hip_init())


def hip_available() -> bool:
    try:
        return _lib.load().st_hip_init() == _lib.OK
    except OSError:
        return False


def probe() -> dict:
    """`probe()` of crates/st-backend-hip/src/lib.rs:188-207: tries init() and reports (HipProbe's fields)."""
    result = _lib.ProbeResult()
    _check(_lib.load().st_hip_probe(ctypes.byref(result)))
    error = result.error.decode("utf-8", "replace")
    return {"available": bool(result.available), "initialized": bool(result.initialized),
            "devices": device_info() if result.initialized else [], "error": error or None}


def runtime():
    """`runtime()` of lib.rs:164-166: the initialised runtime (here: its device list), or None before init()."""
    return device_info() if hip_available() else None


def device_count() -> int:
    return int(_lib.load().st_hip_device_count())


def device_properties(index: int = 0) -> dict:
    props = _lib.DeviceProps()
    _check(_lib.load().st_hip_device_properties(index, ctypes.byref(props)))
    out = {name: getattr(props, name) for name, _ in props._fields_}
    out["arch"] = props.arch.decode()
    return out


def device_info() -> list:
    lib = _lib.load()
    infos = []
    for index in range(lib.st_hip_device_count()):
        buf = ctypes.create_string_buffer(256)
        _check(lib.st_hip_device_name(index, buf, 256))
        infos.append({"id": index, "name": buf.value.decode(), "multi_node": False})
    return infos


# ---- host-slice operators ------------------------------------------------------------------------

def gemm_scaled_f32(m: int, n: int, k: int, scale: float, lhs, rhs, out) -> None:
    """out = (lhs @ rhs) * scale — lib.rs:619-632."""
    lhs, rhs, out = _f32(lhs, "lhs"), _f32(rhs, "rhs"), _out(out, "out")
    _check(_lib.load().st_hip_gemm_f32(m, n, k, scale, 0, _ptr(lhs), lhs.size, _ptr(rhs), rhs.size, _ptr(out),
                                       out.size))


def gemm_f32(m: int, n: int, k: int, lhs, rhs, out) -> None:
    """lib.rs:607-616."""
    gemm_scaled_f32(m, n, k, 1.0, lhs, rhs, out)


def gemm_f32_raw(m: int, n: int, k: int, lhs_address, rhs_address, out_address) -> None:
    """`gemm_f32_raw` of lib.rs:760-799: raw host addresses (ints or None), lengths implied by m, n, k."""
    as_ptr = lambda a: None if not a else ctypes.c_void_p(int(a))
    _check(_lib.load().st_hip_gemm_f32_raw(m, n, k, as_ptr(lhs_address), as_ptr(rhs_address), as_ptr(out_address)))


def gemm_lhs_transpose_scaled_f32(m: int, n: int, k: int, scale: float, lhs, rhs, out) -> None:
    """out = (lhs.T @ rhs) * scale with lhs stored (k, m) — lib.rs:666-680."""
    lhs, rhs, out = _f32(lhs, "lhs"), _f32(rhs, "rhs"), _out(out, "out")
    _check(_lib.load().st_hip_gemm_f32(m, n, k, scale, 1, _ptr(lhs), lhs.size, _ptr(rhs), rhs.size, _ptr(out),
                                       out.size))


def gemm_bias_activation_f32(m: int, n: int, k: int, activation: GemmActivation, lhs, rhs, bias,
                             residual, out) -> None:
    """out = act((lhs @ rhs + bias) + residual) — lib.rs:682-720; `residual` may be None."""
    lhs, rhs, bias, out = _f32(lhs, "lhs"), _f32(rhs, "rhs"), _f32(bias, "bias"), _out(out, "out")
    res = None if residual is None else _f32(residual, "residual")
    _check(_lib.load().st_hip_gemm_bias_act_f32(
        m, n, k, int(activation), _ptr(lhs), lhs.size, _ptr(rhs), rhs.size, _ptr(bias), bias.size,
        _ptr(res), 0 if res is None else res.size, _ptr(out), out.size))


def gemm_prepacked_bias_activation_f32(m: int, n: int, k: int, activation, lhs, packed_rhs, bias, residual,
                                       out) -> None:
    """out = act((lhs @ B + bias) + residual) with B given prepacked as its (n, k) transpose — the PackedB path
    of pure.rs:2559-2757; `bias` and `residual` may be None, `activation` may be 0."""
    lhs, packed, out = _f32(lhs, "lhs"), _f32(packed_rhs, "packed_rhs"), _out(out, "out")
    b = None if bias is None else _f32(bias, "bias")
    res = None if residual is None else _f32(residual, "residual")
    _check(_lib.load().st_hip_gemm_prepacked_bias_act_f32(
        m, n, k, int(activation), _ptr(lhs), lhs.size, _ptr(packed), packed.size, _ptr(b),
        0 if b is None else b.size, _ptr(res), 0 if res is None else res.size, _ptr(out), out.size))


def gemm_bf16_f32acc(m: int, n: int, k: int, lhs_bf16, rhs_bf16, out) -> None:
    lhs, rhs, out = _u16(lhs_bf16, "lhs"), _u16(rhs_bf16, "rhs"), _out(out, "out")
    _check(_lib.load().st_hip_gemm_bf16_f32acc(m, n, k, _ptr(lhs), lhs.size, _ptr(rhs), rhs.size, _ptr(out),
                                               out.size))


def conv2d_output_hw(h, w, kernel, stride, padding, dilation):
    oh, ow = ctypes.c_size_t(), ctypes.c_size_t()
    _check(_lib.load().st_hip_conv2d_output_hw(h, w, kernel[0], kernel[1], stride[0], stride[1], padding[0],
                                               padding[1], dilation[0], dilation[1], ctypes.byref(oh),
                                               ctypes.byref(ow)))
    return oh.value, ow.value


CONV_FAMILIES = {"auto": 0, "tile": 1, "ring": 2, "strip": 3}
CONV_KERNELS = {0: None, 1: "tile", 2: "ring", 3: "strip12", 4: "strip12_wide", 5: "strip9", 6: "adjoint", 7: "col2im", 8: "tile_ksliced", 9: "direct"}


def conv2d_force_family(family: str) -> None:
    """Process-wide diagnostic switch: "auto" (the dispatcher decides), "tile", "ring" or "strip".  With a family
    forced, a shape it cannot serve raises HipErr instead of running another kernel."""
    _check(_lib.load().st_hip_conv2d_force_family(CONV_FAMILIES[family]))


def conv2d_planned_kernel(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, direction="forward"):
    """Name of the kernel the dispatcher runs for this shape ("forward" or "grad_input"); None when the forced
    family cannot serve it."""
    which = ctypes.c_int()
    _check(_lib.load().st_hip_conv2d_planned_kernel(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], {"forward": 0, "grad_input": 1}[direction], ctypes.byref(which)))
    return CONV_KERNELS[which.value]


def conv2d_bias_activation_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, activation,
                               input, weight, bias, out) -> None:
    x, wgt, out = _f32(input, "input"), _f32(weight, "weight"), _out(out, "out")
    b = None if bias is None else _f32(bias, "bias")
    _check(_lib.load().st_hip_conv2d_bias_act_f32(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1],
        dilation[0], dilation[1], int(activation), _ptr(x), x.size, _ptr(wgt), wgt.size, _ptr(b),
        0 if b is None else b.size, _ptr(out), out.size))


def conv2d_backward_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, input, weight, grad_output,
                        grad_input, grad_weight, grad_bias) -> None:
    """Conv2d::backward (conv.rs:780-813): fills grad_input, grad_weight (scaled 1/batch) and grad_bias (1/batch)."""
    x, wgt, g = _f32(input, "input"), _f32(weight, "weight"), _f32(grad_output, "grad_output")
    gi, gw, gb = _out(grad_input, "grad_input"), _out(grad_weight, "grad_weight"), _out(grad_bias, "grad_bias")
    _check(_lib.load().st_hip_conv2d_backward_f32(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], _ptr(x), x.size, _ptr(wgt), wgt.size, _ptr(g), g.size, _ptr(gi), gi.size, _ptr(gw), gw.size,
        _ptr(gb), gb.size))


ATTENTION_KERNELS = {1: "general", 2: "fast", 3: "fast_biased", 4: "tiny"}


def attention_f32_launch_plan(contexts, sequence, head_dim, causal=False, biased=False) -> dict:
    """The launch arithmetic of the f32 attention for a shape, with the whole grid decoded on the host the way the
    kernel decodes it (no device is touched)."""
    plan = _lib.AttentionPlan()
    _check(_lib.load().st_hip_attention_f32_launch_plan(contexts, sequence, head_dim, int(bool(causal)), int(bool(biased)),
                                                         ctypes.byref(plan)))
    out = {name: int(getattr(plan, name)) for name, _ in _lib.AttentionPlan._fields_}
    out["kernel"] = ATTENTION_KERNELS.get(out["kernel"], "none")
    return out


def gemm_bf16_tile_plan(m: int, n: int, k: int) -> dict:
    """Tiling and k-split of the 256-row bf16 GEMM kernels for a shape, with the whole grid decoded on the host."""
    plan = _lib.GemmTilePlan()
    _check(_lib.load().st_hip_gemm_bf16_tile_plan(m, n, k, ctypes.byref(plan)))
    return {name: int(getattr(plan, name)) for name, _ in _lib.GemmTilePlan._fields_}


def gemm_row_block(k: int, element_bytes: int) -> int:
    """Rows of A per launch when an A of 2 GiB or more is cut into row blocks (0: not even 256 rows fit)."""
    return int(_lib.load().st_hip_gemm_row_block(k, element_bytes))


def attention_f32(contexts, sequence, head_dim, scale, causal, q, k, v, z_bias, attn_bias, out) -> None:
    q, k, v, out = _f32(q, "q"), _f32(k, "k"), _f32(v, "v"), _out(out, "out")
    zb = None if z_bias is None else _f32(z_bias, "z_bias")
    ab = None if attn_bias is None else _f32(attn_bias, "attn_bias")
    _check(_lib.load().st_hip_attention_f32(
        contexts, sequence, head_dim, scale, int(bool(causal)), _ptr(q), q.size, _ptr(k), k.size, _ptr(v), v.size,
        _ptr(zb), 0 if zb is None else zb.size, _ptr(ab), 0 if ab is None else ab.size, _ptr(out), out.size))


# ---- device-resident helpers (benchmarks, decoder, tests) ----------------------------------------

class DeviceBuffer:
    """Owning device allocation (DeviceBuffer of crates/st-backend-hip/src/real.rs:649-667)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        ptr = ctypes.c_void_p()
        _check(_lib.load().st_hip_malloc(ctypes.byref(ptr), self.nbytes))
        self.ptr = ptr

    @classmethod
    def from_array(cls, array: np.ndarray, stream=None) -> "DeviceBuffer":
        a = np.ascontiguousarray(array)
        buf = cls(a.nbytes)
        _check(_lib.load().st_hip_memcpy_h2d(buf.ptr, ctypes.c_void_p(a.ctypes.data), a.nbytes, _stream_ptr(stream)))
        return buf

    def upload(self, array: np.ndarray, byte_offset: int = 0, stream=None) -> None:
        """Copies a host array into the allocation starting `byte_offset` bytes in."""
        a = np.ascontiguousarray(array)
        if byte_offset < 0 or byte_offset + a.nbytes > self.nbytes:
            raise ValueError("array does not fit the device buffer at that offset")
        _check(_lib.load().st_hip_memcpy_h2d(ctypes.c_void_p(self.at(byte_offset)), ctypes.c_void_p(a.ctypes.data),
                                             a.nbytes, _stream_ptr(stream)))

    def to_array(self, dtype, shape, stream=None) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        if out.nbytes > self.nbytes:
            raise ValueError("device buffer is smaller than the requested array")
        _check(_lib.load().st_hip_memcpy_d2h(ctypes.c_void_p(out.ctypes.data), self.ptr, out.nbytes,
                                             _stream_ptr(stream)))
        return out

    def at(self, byte_offset: int) -> int:
        """Device address `byte_offset` bytes into the allocation (for entry points that take sub-ranges)."""
        if not 0 <= byte_offset <= self.nbytes:
            raise ValueError("offset outside the device buffer")
        return int(self.ptr.value) + int(byte_offset)

    def zero(self, stream=None) -> None:
        _check(_lib.load().st_hip_memset_zero(self.ptr, self.nbytes, _stream_ptr(stream)))

    def free(self) -> None:
        if self.ptr is not None and self.ptr.value:
            _lib.load().st_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    """Owning stream handle (HipStream of real.rs:190-214); default priority."""

    def __init__(self):
        ptr = ctypes.c_void_p()
        _check(_lib.load().st_hip_stream_create(ctypes.byref(ptr)))
        self.ptr = ptr

    def synchronize(self) -> None:
        _check(_lib.load().st_hip_stream_synchronize(self.ptr))

    def destroy(self) -> None:
        if self.ptr is not None and self.ptr.value:
            _lib.load().st_hip_stream_destroy(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Event:
    def __init__(self):
        ptr = ctypes.c_void_p()
        _check(_lib.load().st_hip_event_create(ctypes.byref(ptr)))
        self.ptr = ptr

    def record(self, stream=None) -> None:
        _check(_lib.load().st_hip_event_record(self.ptr, _stream_ptr(stream)))

    def synchronize(self) -> None:
        _check(_lib.load().st_hip_event_synchronize(self.ptr))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = ctypes.c_float()
        _check(_lib.load().st_hip_event_elapsed_ms(self.ptr, stop.ptr, ctypes.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if self.ptr is not None and self.ptr.value:
                _lib.load().st_hip_event_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass


def _stream_ptr(stream):
    if stream is None:
        return None
    return stream.ptr if isinstance(stream, Stream) else stream


def _dev(buf):
    if buf is None:
        return None
    return buf.ptr if isinstance(buf, DeviceBuffer) else buf


def release_scratch(stream=None) -> None:
    """Waits for the stream (None: the default stream) and frees the scratch buffers the library keeps for it."""
    _check(_lib.load().st_hip_release_scratch(_stream_ptr(stream)))


def scratch_buffer_count() -> int:
    return int(_lib.load().st_hip_scratch_buffer_count())


def device_synchronize() -> None:
    _check(_lib.load().st_hip_device_synchronize())


def gemm_f32_dev(m, n, k, scale, lhs_transposed, lhs, rhs, out, stream=None) -> None:
    _check(_lib.load().st_hip_gemm_f32_dev(m, n, k, scale, int(bool(lhs_transposed)), _dev(lhs), _dev(rhs),
                                           _dev(out), _stream_ptr(stream)))


def gemm_bias_act_f32_dev(m, n, k, activation, lhs, rhs, bias, residual, out, stream=None) -> None:
    _check(_lib.load().st_hip_gemm_bias_act_f32_dev(m, n, k, int(activation), _dev(lhs), _dev(rhs), _dev(bias),
                                                    _dev(residual), _dev(out), _stream_ptr(stream)))


def gemm_prepacked_bias_act_f32_dev(m, n, k, activation, lhs, packed_rhs, bias, residual, out, stream=None) -> None:
    _check(_lib.load().st_hip_gemm_prepacked_bias_act_f32_dev(m, n, k, int(activation), _dev(lhs), _dev(packed_rhs),
                                                              _dev(bias), _dev(residual), _dev(out),
                                                              _stream_ptr(stream)))


def pack_rhs_f32_dev(k, n, rhs, packed, stream=None) -> None:
    """packed (n, k) = rhs (k, n) transposed, on the device."""
    _check(_lib.load().st_hip_pack_rhs_f32_dev(k, n, _dev(rhs), _dev(packed), _stream_ptr(stream)))


def gemm_bf16_f32acc_dev(m, n, k, lhs, rhs, out, stream=None) -> None:
    _check(_lib.load().st_hip_gemm_bf16_f32acc_dev(m, n, k, _dev(lhs), _dev(rhs), _dev(out), _stream_ptr(stream)))


def gemm_bf16_bias_act_dev(m, n, k, activation, lhs, rhs, bias, residual, out_f32, out_bf16, stream=None) -> None:
    _check(_lib.load().st_hip_gemm_bf16_bias_act_dev(m, n, k, int(activation), _dev(lhs), _dev(rhs), _dev(bias),
                                                     _dev(residual), _dev(out_f32), _dev(out_bf16),
                                                     _stream_ptr(stream)))


def gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, lhs, packed_rhs, bias, residual, out_f32, out_bf16,
                                     stream=None) -> None:
    """gemm_bf16_bias_act_dev with B given as its (n, k) transpose (the PackedB layout)."""
    _check(_lib.load().st_hip_gemm_bf16_prepacked_bias_act_dev(m, n, k, int(activation), _dev(lhs), _dev(packed_rhs),
                                                               _dev(bias), _dev(residual), _dev(out_f32),
                                                               _dev(out_bf16), _stream_ptr(stream)))


def gemm_bf16_prepacked_residual_layer_norm_dev(m, n, k, lhs, packed_rhs, bias, residual, gamma, beta, epsilon, out_f32,
                                                out_ln_bf16, stream=None) -> None:
    """out_f32 = (lhs @ rhs + bias) + residual and out_ln_bf16 = layer_norm(out_f32) rounded to bf16: Linear + residual +
    LayerNorm of a pre-norm transformer block (crates/st-vision/src/models/vit.rs:256-265) in one call."""
    _check(_lib.load().st_hip_gemm_bf16_prepacked_residual_layer_norm_dev(
        m, n, k, _dev(lhs), _dev(packed_rhs), _dev(bias), _dev(residual), _dev(gamma), _dev(beta), float(epsilon),
        _dev(out_f32), _dev(out_ln_bf16), _stream_ptr(stream)))


def pack_rhs_bf16_dev(k, n, rhs, packed, stream=None) -> None:
    """packed (n, k) = rhs (k, n) transposed, bf16 bit patterns, on the device."""
    _check(_lib.load().st_hip_pack_rhs_bf16_dev(k, n, _dev(rhs), _dev(packed), _stream_ptr(stream)))


def conv2d_bias_act_f32_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, activation, input, weight,
                            bias, out, stream=None) -> None:
    _check(_lib.load().st_hip_conv2d_bias_act_f32_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], int(activation), _dev(input), _dev(weight), _dev(bias), _dev(out), _stream_ptr(stream)))


def conv2d_bias_act_bf16_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, activation, input, weight,
                             bias, out_f32, out_bf16, stream=None) -> None:
    """Fused conv2d on bf16 NCHW images and OIHW weights (bit patterns), f32 accumulation; f32 and/or bf16 output."""
    _check(_lib.load().st_hip_conv2d_bias_act_bf16_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], int(activation), _dev(input), _dev(weight), _dev(bias), _dev(out_f32), _dev(out_bf16),
        _stream_ptr(stream)))


def conv2d_grad_input_f32_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, grad_output, weight,
                              grad_input, stream=None) -> None:
    _check(_lib.load().st_hip_conv2d_grad_input_f32_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], _dev(grad_output), _dev(weight), _dev(grad_input), _stream_ptr(stream)))


NOALLOC_SCRATCH_BYTES = 16 << 20


def conv2d_grad_input_f32_noalloc_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, grad_output, weight,
                                      grad_input, stream=None) -> None:
    """conv2d_grad_input_f32_dev that allocates nothing: the re-laid weights go to a static device array of
    NOALLOC_SCRATCH_BYTES (larger weights raise HipErr).  Calls that overlap on one GPU race on that array."""
    _check(_lib.load().st_hip_conv2d_grad_input_f32_noalloc_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], _dev(grad_output), _dev(weight), _dev(grad_input), _stream_ptr(stream)))


def conv2d_grad_weight_f32_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, input, grad_output, scale,
                               grad_weight, stream=None) -> None:
    _check(_lib.load().st_hip_conv2d_grad_weight_f32_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], _dev(input), _dev(grad_output), scale, _dev(grad_weight), _stream_ptr(stream)))


def conv2d_grad_bias_f32_dev(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, grad_output, scale,
                             grad_bias, stream=None) -> None:
    _check(_lib.load().st_hip_conv2d_grad_bias_f32_dev(
        batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1], dilation[0],
        dilation[1], _dev(grad_output), scale, _dev(grad_bias), _stream_ptr(stream)))


def attention_f32_dev(contexts, sequence, head_dim, scale, causal, q, k, v, z_bias, attn_bias, out,
                      stream=None) -> None:
    _check(_lib.load().st_hip_attention_f32_dev(contexts, sequence, head_dim, scale, int(bool(causal)), _dev(q),
                                                _dev(k), _dev(v), _dev(z_bias), _dev(attn_bias), _dev(out),
                                                _stream_ptr(stream)))


def attention_bf16_dev(batch, heads, sequence, head_dim, scale, causal, q, k, v, ld_in, out, ld_out,
                       stream=None) -> None:
    """bf16 attention over heads stored as column slices of (batch*sequence, ld) matrices; q/k/v/out are
    DeviceBuffers or raw device addresses (DeviceBuffer.at) of bf16 bit patterns."""
    _check(_lib.load().st_hip_attention_bf16_dev(batch, heads, sequence, head_dim, scale, int(bool(causal)), _dev(q),
                                                 _dev(k), _dev(v), ld_in, _dev(out), ld_out, _stream_ptr(stream)))


def probe_mfma_bf16_dev(workgroups, iterations, operands, sink, stream=None) -> None:
    """A loop of bf16 matrix instructions on register operands (measurement aid; see st_hip_probe_mfma_bf16_dev)."""
    _check(_lib.load().st_hip_probe_mfma_bf16_dev(workgroups, iterations, _dev(operands), _dev(sink), _stream_ptr(stream)))


def probe_mfma_f32_dev(workgroups, iterations, operands, sink, stream=None) -> None:
    """A loop of f32 matrix instructions on register operands (measurement aid; see st_hip_probe_mfma_f32_dev)."""
    _check(_lib.load().st_hip_probe_mfma_f32_dev(workgroups, iterations, _dev(operands), _dev(sink), _stream_ptr(stream)))


def probe_stream_lds_dev(workgroups, iterations, region, region_bytes, stream=None) -> None:
    """A loop of direct-to-LDS loads over a device region (measurement aid; see st_hip_probe_stream_lds_dev)."""
    _check(_lib.load().st_hip_probe_stream_lds_dev(workgroups, iterations, _dev(region), region_bytes, _stream_ptr(stream)))


def row_softmax_f32_dev(rows, cols, src, dst, stream=None) -> None:
    _check(_lib.load().st_hip_row_softmax_f32_dev(rows, cols, _dev(src), _dev(dst), _stream_ptr(stream)))


def gelu_f32_dev(count, src, dst, stream=None) -> None:
    _check(_lib.load().st_hip_gelu_f32_dev(count, _dev(src), _dev(dst), _stream_ptr(stream)))


def count_nonfinite_f32_dev(count, data, stream=None):
    """(number of non-finite values, index of the first, its value) of a device buffer; synchronous."""
    found, first = ctypes.c_uint64(), ctypes.c_uint64()
    value = ctypes.c_float()
    _check(_lib.load().st_hip_count_nonfinite_f32_dev(count, _dev(data), ctypes.byref(found), ctypes.byref(first),
                                                      ctypes.byref(value), _stream_ptr(stream)))
    return int(found.value), int(first.value), float(value.value)


def transfer_counters(reset: bool = False) -> dict:
    """Host<->device copies made through the library: copies and bytes in each direction."""
    raw = (ctypes.c_uint64 * 4)()
    _check(_lib.load().st_hip_transfer_counters(raw, int(reset)))
    return {"h2d_copies": int(raw[0]), "h2d_bytes": int(raw[1]), "d2h_copies": int(raw[2]), "d2h_bytes": int(raw[3])}


def gelu_backward_f32_dev(count, z, grad, out, stream=None) -> None:
    _check(_lib.load().st_hip_gelu_backward_f32_dev(count, _dev(z), _dev(grad), _dev(out), _stream_ptr(stream)))


def scale_f32_dev(count, src, scale, dst, stream=None) -> None:
    _check(_lib.load().st_hip_scale_f32_dev(count, _dev(src), scale, _dev(dst), _stream_ptr(stream)))


def add_row_f32_dev(rows, cols, data, bias, stream=None) -> None:
    _check(_lib.load().st_hip_add_row_f32_dev(rows, cols, _dev(data), _dev(bias), _stream_ptr(stream)))


def sum_axis0_f32_dev(rows, cols, src, scale, dst, stream=None) -> None:
    _check(_lib.load().st_hip_sum_axis0_f32_dev(rows, cols, _dev(src), scale, _dev(dst), _stream_ptr(stream)))


def layer_norm_f32_dev(rows, cols, x, residual, gamma, beta, epsilon, out_f32, out_bf16, stream=None) -> None:
    _check(_lib.load().st_hip_layer_norm_f32_dev(rows, cols, _dev(x), _dev(residual), _dev(gamma), _dev(beta),
                                                 epsilon, _dev(out_f32), _dev(out_bf16), _stream_ptr(stream)))


def embedding_f32_dev(tokens, vocab, dim, token_ids, table, out, stream=None) -> None:
    _check(_lib.load().st_hip_embedding_f32_dev(tokens, vocab, dim, _dev(token_ids), _dev(table), _dev(out),
                                                _stream_ptr(stream)))


def f32_to_bf16_dev(count, src, dst, stream=None) -> None:
    _check(_lib.load().st_hip_f32_to_bf16_dev(count, _dev(src), _dev(dst), _stream_ptr(stream)))


def split_heads_f32_dev(batch, seq, heads, head_dim, qkv, q, k, v, stream=None) -> None:
    _check(_lib.load().st_hip_split_heads_f32_dev(batch, seq, heads, head_dim, _dev(qkv), _dev(q), _dev(k), _dev(v),
                                                  _stream_ptr(stream)))


def merge_heads_f32_dev(batch, seq, heads, head_dim, contexts_in, out_f32, out_bf16, stream=None) -> None:
    _check(_lib.load().st_hip_merge_heads_f32_dev(batch, seq, heads, head_dim, _dev(contexts_in), _dev(out_f32),
                                                  _dev(out_bf16), _stream_ptr(stream)))


class Decoder:
    """Device-resident byte-level decoder stack (st_hip_decoder_* of include/st_hip.h)."""

    def __init__(self, vocab, d_model, heads, layers, d_ff, batch, seq, ln_eps, weights: np.ndarray):
        self.config = _lib.DecoderConfig(vocab, d_model, heads, layers, d_ff, batch, seq, ln_eps)
        w = _f32(weights, "weights")
        handle = ctypes.c_void_p()
        _check(_lib.load().st_hip_decoder_create(ctypes.byref(self.config), _ptr(w), w.size, ctypes.byref(handle)))
        self.handle = handle

    @staticmethod
    def weight_count(vocab, d_model, heads, layers, d_ff, batch=1, seq=1) -> int:
        cfg = _lib.DecoderConfig(vocab, d_model, heads, layers, d_ff, batch, seq, 1e-5)
        return int(_lib.load().st_hip_decoder_weight_count(ctypes.byref(cfg)))

    def forward_dev(self, tokens, logits, stream=None) -> None:
        _check(_lib.load().st_hip_decoder_forward_dev(self.handle, _dev(tokens), _dev(logits), _stream_ptr(stream)))

    def destroy(self) -> None:
        if self.handle is not None and self.handle.value:
            _lib.load().st_hip_decoder_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
