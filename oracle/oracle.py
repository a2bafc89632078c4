"""ctypes wrapper of oracle/libst_oracle.so — the CPU restatement of the reference's dense CPU path.

TEST INFRASTRUCTURE ONLY.  Nothing under spiraltorch_amd/ may import this module; it exists so that
tests, the smoke check and the benchmark's CPU-baseline leg can check / time the reference algorithm.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import POINTER, c_double, c_float, c_int, c_size_t, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libst_oracle.so")

ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
NONFINITE_LABELS = {
    1: "scaled_dot_attention_dot",
    2: "scaled_dot_attention_logit",
    3: "scaled_dot_attention_denom",
    4: "scaled_dot_attention_weight",
    5: "scaled_dot_attention_accumulator",
    6: "layer_norm",
}


class OracleError(Exception):
    def __init__(self, code: int):
        self.code = code
        self.label = NONFINITE_LABELS.get(code)
        super().__init__(f"oracle status {code}" + (f" (NonFiniteValue: {self.label})" if self.label else ""))


class DecoderConfig(ctypes.Structure):
    _fields_ = [("vocab", c_size_t), ("d_model", c_size_t), ("heads", c_size_t), ("layers", c_size_t),
                ("d_ff", c_size_t), ("batch", c_size_t), ("seq", c_size_t), ("ln_eps", c_float)]


_lib = None


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "libst_oracle.so"], check=True, capture_output=True)


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        build()
    lib = ctypes.CDLL(LIBRARY_PATH)
    S, P, F, I = c_size_t, c_void_p, c_float, c_int
    lib.st_oracle_gemm_f32.argtypes = [S, S, S, F, I, P, P, P, I]
    lib.st_oracle_gemm_f32_packed_naive.argtypes = [S, S, S, P, P, P]
    lib.st_oracle_gemm_bias_act_f32.argtypes = [S, S, S, I, P, P, P, P, P, I]
    lib.st_oracle_gemm_bf16_f32acc.argtypes = [S, S, S, P, P, P, I]
    lib.st_oracle_conv2d_output_hw.argtypes = [S] * 10 + [POINTER(S), POINTER(S)]
    lib.st_oracle_conv2d_bias_act_f32.argtypes = [S] * 13 + [I, P, P, P, P, I]
    lib.st_oracle_conv2d_backward_f32.argtypes = [S] * 13 + [P, P, P, F, P, P, P]
    lib.st_oracle_attention_f32.argtypes = [S, S, S, F, I, P, P, P, P, P, P, I]
    lib.st_oracle_attention_f64.argtypes = [S, S, S, c_double, I, P, P, P, P, P, P]
    lib.st_oracle_layer_norm_f32.argtypes = [S, S, P, P, P, P, F, P]
    lib.st_oracle_embedding_f32.argtypes = [S, S, S, P, P, P]
    lib.st_oracle_row_softmax_f32.argtypes = [S, S, P, P]
    lib.st_oracle_gelu_backward_f32.argtypes = [S, P, P, P]
    lib.st_oracle_scale_f32.argtypes = [S, P, F, P]
    lib.st_oracle_add_row_f32.argtypes = [S, S, P, P]
    lib.st_oracle_sum_axis0_f32.argtypes = [S, S, P, F, P]
    lib.st_oracle_gelu.argtypes = [F]
    lib.st_oracle_gelu.restype = F
    lib.st_oracle_f32_to_bf16.argtypes = [S, P, P]
    lib.st_oracle_f32_to_bf16.restype = None
    lib.st_oracle_bf16_to_f32.argtypes = [S, P, P]
    lib.st_oracle_bf16_to_f32.restype = None
    lib.st_oracle_decoder_weight_count.argtypes = [POINTER(DecoderConfig)]
    lib.st_oracle_decoder_weight_count.restype = S
    lib.st_oracle_decoder_forward.argtypes = [POINTER(DecoderConfig), P, P, S, P, I]
    _lib = lib
    return lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _p(a):
    return None if a is None else c_void_p(a.ctypes.data)


def _check(rc: int) -> None:
    if rc != 0:
        raise OracleError(rc)


def gemm_f32(m, n, k, lhs, rhs, scale=1.0, lhs_transposed=False, threads=1) -> np.ndarray:
    lhs, rhs = _f32(lhs), _f32(rhs)
    assert lhs.size == m * k and rhs.size == k * n
    out = np.zeros(m * n, dtype=np.float32)
    _check(load().st_oracle_gemm_f32(m, n, k, scale, int(lhs_transposed), _p(lhs), _p(rhs), _p(out), threads))
    return out


def gemm_f32_packed_naive(m, n, k, lhs, packed_rhs) -> np.ndarray:
    """`packed_rhs` is the (n, k) transpose of B (PackedB's layout)."""
    lhs, packed_rhs = _f32(lhs), _f32(packed_rhs)
    assert lhs.size == m * k and packed_rhs.size == k * n
    out = np.zeros(m * n, dtype=np.float32)
    _check(load().st_oracle_gemm_f32_packed_naive(m, n, k, _p(lhs), _p(packed_rhs), _p(out)))
    return out


def gemm_bias_act_f32(m, n, k, activation, lhs, rhs, bias, residual=None, threads=1) -> np.ndarray:
    lhs, rhs = _f32(lhs), _f32(rhs)
    bias = None if bias is None else _f32(bias)
    residual = None if residual is None else _f32(residual)
    assert lhs.size == m * k and rhs.size == k * n
    out = np.zeros(m * n, dtype=np.float32)
    _check(load().st_oracle_gemm_bias_act_f32(m, n, k, activation, _p(lhs), _p(rhs), _p(bias), _p(residual), _p(out),
                                              threads))
    return out


def gemm_bf16_f32acc(m, n, k, lhs_bits, rhs_bits, threads=1) -> np.ndarray:
    lhs = np.ascontiguousarray(lhs_bits, dtype=np.uint16)
    rhs = np.ascontiguousarray(rhs_bits, dtype=np.uint16)
    assert lhs.size == m * k and rhs.size == k * n
    out = np.zeros(m * n, dtype=np.float32)
    _check(load().st_oracle_gemm_bf16_f32acc(m, n, k, _p(lhs), _p(rhs), _p(out), threads))
    return out


def conv2d_output_hw(h, w, kernel, stride, padding, dilation):
    oh, ow = c_size_t(), c_size_t()
    _check(load().st_oracle_conv2d_output_hw(h, w, kernel[0], kernel[1], stride[0], stride[1], padding[0], padding[1],
                                             dilation[0], dilation[1], ctypes.byref(oh), ctypes.byref(ow)))
    return oh.value, ow.value


def conv2d_bias_act_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, activation, x, weight, bias,
                        threads=1) -> np.ndarray:
    x, weight = _f32(x), _f32(weight)
    bias = None if bias is None else _f32(bias)
    oh, ow = conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    assert x.size == batch * c_in * h * w and weight.size == c_out * c_in * kernel[0] * kernel[1]
    out = np.zeros(batch * c_out * oh * ow, dtype=np.float32)
    _check(load().st_oracle_conv2d_bias_act_f32(batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1],
                                                padding[0], padding[1], dilation[0], dilation[1], activation, _p(x),
                                                _p(weight), _p(bias), _p(out), threads))
    return out


def conv2d_backward_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, input, weight, grad_output,
                        weight_scale=None):
    """Returns (grad_input, grad_weight, grad_bias); weight_scale defaults to the reference's 1/batch."""
    x, wgt, g = _f32(input), _f32(weight), _f32(grad_output)
    scale = (1.0 / batch if batch else 1.0) if weight_scale is None else weight_scale
    grad_input = np.zeros(batch * c_in * h * w, dtype=np.float32)
    grad_weight = np.zeros(c_out * c_in * kernel[0] * kernel[1], dtype=np.float32)
    grad_bias = np.zeros(c_out, dtype=np.float32)
    _check(load().st_oracle_conv2d_backward_f32(batch, c_in, h, w, c_out, kernel[0], kernel[1], stride[0], stride[1],
                                                padding[0], padding[1], dilation[0], dilation[1], _p(x), _p(wgt),
                                                _p(g), scale, _p(grad_input), _p(grad_weight), _p(grad_bias)))
    return grad_input, grad_weight, grad_bias


def attention_f32(contexts, sequence, head_dim, scale, q, k, v, z_bias=None, attn_bias=None, causal=False,
                  threads=1) -> np.ndarray:
    q, k, v = _f32(q), _f32(k), _f32(v)
    z_bias = None if z_bias is None else _f32(z_bias)
    attn_bias = None if attn_bias is None else _f32(attn_bias)
    assert q.size == k.size == v.size == contexts * sequence * head_dim
    out = np.zeros(contexts * sequence * head_dim, dtype=np.float32)
    _check(load().st_oracle_attention_f32(contexts, sequence, head_dim, scale, int(causal), _p(q), _p(k), _p(v),
                                          _p(z_bias), _p(attn_bias), _p(out), threads))
    return out


def attention_f64(contexts, sequence, head_dim, scale, q, k, v, z_bias=None, attn_bias=None,
                  causal=False) -> np.ndarray:
    q, k, v = _f32(q), _f32(k), _f32(v)
    z_bias = None if z_bias is None else _f32(z_bias)
    attn_bias = None if attn_bias is None else _f32(attn_bias)
    out = np.zeros(contexts * sequence * head_dim, dtype=np.float64)
    _check(load().st_oracle_attention_f64(contexts, sequence, head_dim, float(scale), int(causal), _p(q), _p(k),
                                          _p(v), _p(z_bias), _p(attn_bias), _p(out)))
    return out


def layer_norm_f32(rows, cols, x, gamma, beta, epsilon, residual=None) -> np.ndarray:
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    residual = None if residual is None else _f32(residual)
    out = np.zeros(rows * cols, dtype=np.float32)
    _check(load().st_oracle_layer_norm_f32(rows, cols, _p(x), _p(residual), _p(gamma), _p(beta), epsilon, _p(out)))
    return out


def row_softmax_f32(rows, cols, x) -> np.ndarray:
    x = _f32(x)
    out = np.zeros(rows * cols, dtype=np.float32)
    _check(load().st_oracle_row_softmax_f32(rows, cols, _p(x), _p(out)))
    return out


def gelu_backward_f32(z, grad) -> np.ndarray:
    z, grad = _f32(z), _f32(grad)
    out = np.zeros(z.size, dtype=np.float32)
    _check(load().st_oracle_gelu_backward_f32(z.size, _p(z), _p(grad), _p(out)))
    return out


def scale_f32(x, scale) -> np.ndarray:
    x = _f32(x)
    out = np.zeros(x.size, dtype=np.float32)
    _check(load().st_oracle_scale_f32(x.size, _p(x), scale, _p(out)))
    return out


def add_row_f32(rows, cols, data, bias) -> np.ndarray:
    out, bias = _f32(data).copy(), _f32(bias)
    _check(load().st_oracle_add_row_f32(rows, cols, _p(out), _p(bias)))
    return out


def sum_axis0_f32(rows, cols, x, scale=1.0) -> np.ndarray:
    x = _f32(x)
    out = np.zeros(cols, dtype=np.float32)
    _check(load().st_oracle_sum_axis0_f32(rows, cols, _p(x), scale, _p(out)))
    return out


def embedding_f32(tokens, vocab, dim, token_ids, table) -> np.ndarray:
    token_ids, table = _f32(token_ids), _f32(table)
    out = np.zeros(tokens * dim, dtype=np.float32)
    _check(load().st_oracle_embedding_f32(tokens, vocab, dim, _p(token_ids), _p(table), _p(out)))
    return out


def gelu(x: float) -> float:
    return float(load().st_oracle_gelu(x))


def f32_to_bf16(values) -> np.ndarray:
    values = _f32(values)
    out = np.zeros(values.size, dtype=np.uint16)
    load().st_oracle_f32_to_bf16(values.size, _p(values), _p(out))
    return out


def bf16_to_f32(bits) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.zeros(bits.size, dtype=np.float32)
    load().st_oracle_bf16_to_f32(bits.size, _p(bits), _p(out))
    return out


def decoder_weight_count(vocab, d_model, heads, layers, d_ff) -> int:
    cfg = DecoderConfig(vocab, d_model, heads, layers, d_ff, 1, 1, 1e-5)
    return int(load().st_oracle_decoder_weight_count(ctypes.byref(cfg)))


def decoder_forward(vocab, d_model, heads, layers, d_ff, batch, seq, ln_eps, weights, tokens, layers_to_run=None,
                    threads=1) -> np.ndarray:
    cfg = DecoderConfig(vocab, d_model, heads, layers, d_ff, batch, seq, ln_eps)
    weights, tokens = _f32(weights), _f32(tokens)
    assert weights.size == decoder_weight_count(vocab, d_model, heads, layers, d_ff)
    assert tokens.size == batch * seq
    logits = np.zeros(batch * seq * vocab, dtype=np.float32)
    run = layers if layers_to_run is None else layers_to_run
    _check(load().st_oracle_decoder_forward(ctypes.byref(cfg), _p(weights), _p(tokens), run, _p(logits), threads))
    return logits
