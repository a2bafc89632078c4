"""Pins the oracle's conv2d: reference layout vector, output-size vector, float64 direct convolution."""
import numpy as np
import pytest

from conftest import assert_close


def direct_conv64(x, w, b, stride, padding, dilation):
    """Textbook direct convolution in float64 (independent of the oracle's im2col formulation)."""
    n, c, h, wd = x.shape
    o, _, kh, kw = w.shape
    (sh, sw), (ph, pw), (dh, dw) = stride, padding, dilation
    oh = (h + 2 * ph - ((kh - 1) * dh + 1)) // sh + 1
    ow = (wd + 2 * pw - ((kw - 1) * dw + 1)) // sw + 1
    xp = np.zeros((n, c, h + 2 * ph, wd + 2 * pw), np.float64)
    xp[:, :, ph:ph + h, pw:pw + wd] = x
    out = np.zeros((n, o, oh, ow), np.float64)
    for i in range(kh):
        for j in range(kw):
            patch = xp[:, :, i * dh:i * dh + (oh - 1) * sh + 1:sh, j * dw:j * dw + (ow - 1) * sw + 1:sw]
            out += np.einsum("nchw,oc->nohw", patch, w[:, :, i, j].astype(np.float64))
    return out + b.reshape(1, o, 1, 1)


def generated_case(case):
    """Inputs of the reference's generator-defined conv tests (tests/golden/reference_vectors.json)."""
    c_in, c_out = case["c_in"], case["c_out"]
    kh, kw = case["kernel"]
    h, w = case["input_hw"]
    idx = np.arange(c_out * c_in * kh * kw, dtype=np.float32)
    if case["weight_rule"] == "sin(idx)":
        weight = np.sin(idx).astype(np.float32)
        bias = (np.arange(c_out, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
        row, col = np.meshgrid(np.arange(case["batch"]), np.arange(c_in * h * w), indexing="ij")
        x = (((row * 97 + col * 31) % 23).astype(np.float32) * np.float32(0.05)).astype(np.float32)
    else:
        weight = (np.sin(idx * np.float32(0.137)) * np.float32(0.4) -
                  (np.arange(idx.size) % 3).astype(np.float32) * np.float32(0.02)).astype(np.float32)
        bias = (np.arange(c_out, dtype=np.float32) * np.float32(0.037) - np.float32(0.05)).astype(np.float32)
        row, col = np.meshgrid(np.arange(case["batch"]), np.arange(c_in * h * w), indexing="ij")
        x = (((row * 41 + col * 17) % 29).astype(np.float32) * np.float32(0.031) - np.float32(0.2)).astype(np.float32)
    return x, weight, bias


def test_layout_known_answer(oracle, golden):
    c = golden["conv_layout"]
    out = oracle.conv2d_bias_act_f32(c["batch"], c["c_in"], *c["input_hw"], c["c_out"], c["kernel"], c["stride"],
                                     c["padding"], c["dilation"], oracle.ACT_NONE, c["input"], c["weight"], c["bias"])
    assert out.tolist() == c["expected"]


def test_output_hw_known_answer(oracle, golden):
    for c in golden["conv_output_hw"]:
        assert list(oracle.conv2d_output_hw(*c["input_hw"], c["kernel"], c["stride"], c["padding"],
                                            c["dilation"])) == c["expected"]
    with pytest.raises(oracle.OracleError):
        oracle.conv2d_output_hw(2, 2, (5, 5), (1, 1), (0, 0), (1, 1))


def test_generated_cases_against_direct_convolution(oracle, golden):
    for case in golden["conv_generated"]:
        x, weight, bias = generated_case(case)
        h, w = case["input_hw"]
        out = oracle.conv2d_bias_act_f32(case["batch"], case["c_in"], h, w, case["c_out"], case["kernel"],
                                         case["stride"], case["padding"], case["dilation"], oracle.ACT_NONE, x,
                                         weight, bias)
        want = direct_conv64(x.reshape(case["batch"], case["c_in"], h, w).astype(np.float64),
                             weight.reshape(case["c_out"], case["c_in"], *case["kernel"]), bias.astype(np.float64),
                             case["stride"], case["padding"], case["dilation"])
        assert_close(out, want, 0, case["tolerance"], case["source"])


@pytest.mark.parametrize("shape", [
    # batch, c_in, h, w, c_out, kernel, stride, padding, dilation
    (2, 3, 9, 7, 4, (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 2, 9, 9, 3, (3, 3), (1, 1), (0, 0), (2, 2)),
    (3, 5, 6, 11, 7, (2, 4), (2, 3), (1, 2), (1, 1)),
    (2, 4, 5, 5, 6, (1, 1), (1, 1), (0, 0), (1, 1)),
    (1, 1, 4, 4, 1, (4, 4), (1, 1), (0, 0), (1, 1)),
])
def test_random_shapes_against_direct_convolution(oracle, shape):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    rng = np.random.default_rng(hash(shape) % 2 ** 32)
    x = rng.normal(size=(batch, c_in, h, w)).astype(np.float32)
    wt = rng.normal(size=(c_out, c_in, *kernel)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    want = direct_conv64(x.astype(np.float64), wt, b.astype(np.float64), stride, padding, dilation)
    out = oracle.conv2d_bias_act_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, oracle.ACT_NONE,
                                     x, wt, b)
    assert_close(out, want, 1e-5, 1e-5, f"conv {shape}")
    relu = oracle.conv2d_bias_act_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, oracle.ACT_RELU,
                                      x, wt, b)
    assert (relu == np.maximum(out, 0)).all()
    nobias = oracle.conv2d_bias_act_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, oracle.ACT_NONE,
                                        x, wt, None)
    assert_close(nobias, want - b.astype(np.float64).reshape(1, c_out, 1, 1), 1e-5, 1e-5, "no bias")


def test_1x1_conv_is_a_gemm(oracle):
    # 1x1 stride-1 convolution == W(c_out x c_in) . X(c_in x H*W) per image, bit for bit.
    rng = np.random.default_rng(11)
    x = rng.normal(size=(2, 6, 5, 4)).astype(np.float32)
    wt = rng.normal(size=(3, 6)).astype(np.float32)
    out = oracle.conv2d_bias_act_f32(2, 6, 5, 4, 3, (1, 1), (1, 1), (0, 0), (1, 1), oracle.ACT_NONE, x, wt, None)
    for b in range(2):
        want = oracle.gemm_f32(3, 20, 6, wt, x[b].reshape(6, 20))
        assert (out.reshape(2, 3, 20)[b].ravel() == want).all()


def test_empty_batch(oracle):
    out = oracle.conv2d_bias_act_f32(0, 2, 4, 4, 3, (3, 3), (1, 1), (1, 1), (1, 1), oracle.ACT_NONE,
                                     np.zeros(0, np.float32), np.ones(54, np.float32), None)
    assert out.size == 0


# ---- backward -------------------------------------------------------------------------------------------

def test_backward_reference_1x1_vector(oracle):
    """conv2d_backward_matches_manual_kernel11, crates/st-nn/src/layers/conv.rs:4114-4130: weight 1.5, input
    [1,2,3,4] on 2x2, grad_output ones -> grad_input 1.5 everywhere, grad_weight 10, grad_bias 4."""
    gi, gw, gb = oracle.conv2d_backward_f32(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), [1, 2, 3, 4], [1.5],
                                            [1, 1, 1, 1])
    assert gi.tolist() == [1.5] * 4 and gw.tolist() == [10.0] and gb.tolist() == [4.0]


def _direct_backward_f64(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, x, wgt, g):
    """Closed form of the three gradients written from the definition (not via patches)."""
    kh, kw = kernel
    oh = (h + 2 * padding[0] - ((kh - 1) * dilation[0] + 1)) // stride[0] + 1
    ow = (w + 2 * padding[1] - ((kw - 1) * dilation[1] + 1)) // stride[1] + 1
    x = np.asarray(x, np.float64).reshape(batch, c_in, h, w)
    wgt = np.asarray(wgt, np.float64).reshape(c_out, c_in, kh, kw)
    g = np.asarray(g, np.float64).reshape(batch, c_out, oh, ow)
    gi, gw = np.zeros_like(x), np.zeros_like(wgt)
    for oy in range(oh):
        for ox in range(ow):
            for ky in range(kh):
                for kx in range(kw):
                    iy = oy * stride[0] + ky * dilation[0] - padding[0]
                    ix = ox * stride[1] + kx * dilation[1] - padding[1]
                    if 0 <= iy < h and 0 <= ix < w:
                        gi[:, :, iy, ix] += g[:, :, oy, ox] @ wgt[:, :, ky, kx]
                        gw[:, :, ky, kx] += g[:, :, oy, ox].T @ x[:, :, iy, ix]
    return gi.ravel(), gw.ravel() / batch, g.sum(axis=(0, 2, 3)) / batch


BACKWARD_CASES = [
    (2, 3, 8, 8, 4, (3, 3), (1, 1), (1, 1), (1, 1)), (1, 2, 7, 5, 5, (3, 2), (1, 2), (1, 1), (1, 1)),
    (2, 2, 9, 9, 3, (3, 3), (2, 2), (1, 1), (2, 2)), (1, 1, 6, 6, 2, (1, 1), (1, 1), (0, 0), (1, 1)),
    (3, 4, 5, 6, 2, (2, 3), (2, 1), (0, 2), (1, 1)),
]


@pytest.mark.parametrize("case", BACKWARD_CASES)
def test_backward_matches_the_definition_and_the_adjoint_identity(oracle, case):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = case
    rng = np.random.default_rng(sum(case[:5]))
    oh, ow = oracle.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wgt = rng.normal(size=c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
    g = rng.normal(size=batch * c_out * oh * ow).astype(np.float32)
    gi, gw, gb = oracle.conv2d_backward_f32(*case, x, wgt, g)
    want_gi, want_gw, want_gb = _direct_backward_f64(*case, x, wgt, g)
    assert_close(gi, want_gi, 1e-5, 1e-5, "grad_input")
    assert_close(gw, want_gw, 1e-5, 1e-5, "grad_weight")
    assert_close(gb, want_gb, 1e-5, 1e-5, "grad_bias")
    # <conv(x), g> == <x, grad_input(g)>: ties the backward to the (separately pinned) forward
    y = oracle.conv2d_bias_act_f32(*case[:5], kernel, stride, padding, dilation, oracle.ACT_NONE, x, wgt, None)
    lhs = float(np.dot(y.astype(np.float64), g.astype(np.float64)))
    rhs = float(np.dot(x.astype(np.float64), gi.astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))
