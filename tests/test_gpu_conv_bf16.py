"""Parity of the bf16 implicit-GEMM conv2d (+bias, +activation; f32 accumulation) against the CPU oracle: the oracle's
conv restatement (crates/st-nn/src/layers/conv.rs:685-748, 2559-2599) run on the bf16-rounded operands.  Products of
two bf16 values are exact in f32, so the only difference is the order of the f32 sums; the bar is the 2e-2 relative of
the bf16 paths, with the tighter bound the arithmetic supports checked beside it."""
import math

import numpy as np
import pytest

from conftest import BF16_REL, assert_close

pytestmark = pytest.mark.gpu


def run(hip, shape, act, x16, w16, bias, want_f32=True, want_bf16=False):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    oh, ow = hip.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    count = batch * c_out * oh * ow
    d_x, d_w = hip.DeviceBuffer.from_array(x16), hip.DeviceBuffer.from_array(w16)
    d_b = None if bias is None else hip.DeviceBuffer.from_array(bias)
    d32 = hip.DeviceBuffer(max(count, 1) * 4) if want_f32 else None
    d16 = hip.DeviceBuffer(max(count, 1) * 2) if want_bf16 else None
    hip.conv2d_bias_act_bf16_dev(*shape, act, d_x, d_w, d_b, d32, d16)
    hip.device_synchronize()
    return (d32.to_array(np.float32, count) if want_f32 else None, d16.to_array(np.uint16, count) if want_bf16 else None)


def operands(rng, shape, weight_std=None):
    from spiraltorch_amd import inputs
    batch, c_in, h, w, c_out, kernel, _, _, _ = shape
    std = weight_std or math.sqrt(2.0 / (c_in * kernel[0] * kernel[1]))
    x16 = inputs.to_bf16(rng.normal(size=batch * c_in * h * w).astype(np.float32))
    w16 = inputs.to_bf16(rng.normal(0, std, c_out * c_in * kernel[0] * kernel[1]).astype(np.float32))
    bias = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    return x16, w16, bias


def check(got, want, what):
    floor = BF16_REL * float(np.sqrt(np.mean(np.square(want)))) * 1e-2
    assert_close(got, want, BF16_REL, floor, what)
    scale = float(np.abs(want).max()) or 1.0
    assert float(np.abs(got - want).max()) <= 1e-4 * scale, what  # f32 summation order only


SHAPES = [
    (2, 3, 9, 7, 4, (3, 3), (1, 1), (1, 1), (1, 1)),        # three channels padded to 64; a plane of 63 pixels (not a multiple of 4)
    (1, 2, 9, 9, 3, (3, 3), (1, 1), (0, 0), (2, 2)),        # dilation, no padding
    (3, 5, 6, 11, 7, (2, 4), (2, 3), (1, 2), (1, 1)),       # ragged kernel, strides and padding
    (2, 4, 5, 5, 6, (1, 1), (1, 1), (0, 0), (1, 1)),        # 1×1
    (1, 1, 4, 4, 1, (4, 4), (1, 1), (0, 0), (1, 1)),        # a single output value
    (2, 64, 20, 20, 70, (3, 3), (1, 1), (1, 1), (1, 1)),    # one channel block, 800 pixels: several pixel tiles
    (1, 70, 33, 17, 130, (5, 3), (2, 1), (2, 1), (1, 2)),   # two channel blocks (70 -> 128), 130 output channels (256-row tiles)
    (5, 128, 12, 12, 64, (3, 3), (2, 2), (0, 0), (1, 1)),   # planes of 25 pixels: a tile spans several images
    (3, 192, 14, 14, 300, (3, 3), (1, 1), (1, 1), (1, 1)),  # three channel blocks, two row tiles of 256 channels
    (40, 64, 28, 28, 256, (3, 3), (1, 1), (1, 1), (1, 1)),  # 31360 pixels × 256 channels: the 256×256 tiles
    (2, 16, 7, 7, 8, (7, 7), (1, 1), (3, 3), (1, 1)),       # 49 taps
    (17, 8, 55, 53, 70, (3, 3), (1, 1), (1, 1), (1, 1)),    # 49555 pixels (odd planes) × 70 channels: pixels on the 256-row side
    (16, 128, 64, 64, 128, (1, 1), (1, 1), (0, 0), (1, 1)), # the same tiling, two channel blocks, one tap
    (2, 3, 3, 1000, 4, (1, 3), (1, 1), (0, 1), (1, 1)),     # rows wider than the re-layout tile: copied in pieces
    (1, 5, 40, 225, 6, (3, 3), (1, 2), (2, 2), (1, 1)),     # one row per re-layout group, several rows of padding
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("act", [0, 1, 2])
def test_family_of_shapes_against_the_oracle(hip, oracle, shape, act):
    from spiraltorch_amd import inputs
    if act == 2 and shape[0] * shape[4] > 2000:
        pytest.skip("GELU is checked on the small shapes")
    rng = np.random.default_rng(abs(hash((shape, act))) % 2 ** 32)
    x16, w16, bias = operands(rng, shape)
    got, _ = run(hip, shape, act, x16, w16, bias)
    want = oracle.conv2d_bias_act_f32(*shape, act, inputs.from_bf16(x16), inputs.from_bf16(w16), bias, threads=8)
    check(got, want, f"bf16 conv {shape} act {act}")


def test_outputs_bias_and_exact_small_integers(hip, oracle):
    from spiraltorch_amd import inputs
    # the reference's 1×1 layout vector (conv.rs:3839-3856): in [1,2,3,4], W [1,10] -> [1,2,3,4,10,20,30,40]; exact in bf16
    x16 = inputs.to_bf16(np.array([1, 2, 3, 4], np.float32))
    w16 = inputs.to_bf16(np.array([1, 10], np.float32))
    shape = (1, 1, 2, 2, 2, (1, 1), (1, 1), (0, 0), (1, 1))
    got, got16 = run(hip, shape, 0, x16, w16, None, want_f32=True, want_bf16=True)
    assert got.tolist() == [1, 2, 3, 4, 10, 20, 30, 40]
    assert inputs.from_bf16(got16).tolist() == [1, 2, 3, 4, 10, 20, 30, 40]
    # bf16 output = nearest-even rounding of the f32 output, whichever outputs are asked for; no bias = bias of zeros
    shape = (3, 64, 10, 12, 130, (3, 3), (1, 1), (1, 1), (1, 1))
    rng = np.random.default_rng(9)
    x16, w16, bias = operands(rng, shape)
    both32, both16 = run(hip, shape, 1, x16, w16, bias, True, True)
    only32, _ = run(hip, shape, 1, x16, w16, bias, True, False)
    _, only16 = run(hip, shape, 1, x16, w16, bias, False, True)
    assert (both32.view(np.uint32) == only32.view(np.uint32)).all()
    assert (both16 == only16).all() and (both16 == inputs.to_bf16(both32)).all()
    none32, _ = run(hip, shape, 0, x16, w16, None)
    zero32, _ = run(hip, shape, 0, x16, w16, np.zeros(130, np.float32))
    assert (none32.view(np.uint32) == zero32.view(np.uint32)).all()
    # the same convolution in f32 on the same (bf16-representable) values
    oh, ow = hip.conv2d_output_hw(10, 12, (3, 3), (1, 1), (1, 1), (1, 1))
    f32 = np.zeros(3 * 130 * oh * ow, np.float32)
    hip.conv2d_bias_activation_f32(*shape, 1, inputs.from_bf16(x16), inputs.from_bf16(w16), bias, f32)
    check(both32, f32, "bf16 conv against the f32 kernels on the same values")


def test_config2_geometry(hip, oracle):
    """BASELINE config 2's layer (N32 C64->128 56×56 3×3 s1 p1, + bias + ReLU) on bf16-rounded operands: two images
    elementwise against the oracle, every image against the first through a permutation of the batch, and exact
    doubling (a power-of-two scale of the image scales the pre-activation sums exactly when the bias is zero)."""
    from spiraltorch_amd import inputs
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    shape = (batch, c_in, h, w, c_out, *geom)
    x16 = inputs.to_bf16(inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w))
    w16 = inputs.to_bf16(inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, math.sqrt(2.0 / (c_in * 9))))
    bias = inputs.uniform(inputs.seed_for(2, 2), c_out, -0.1, 0.1)
    got, _ = run(hip, shape, 1, x16, w16, bias)
    plane_in, plane_out = c_in * h * w, c_out * h * w
    for image in (0, 17):
        want = oracle.conv2d_bias_act_f32(1, c_in, h, w, c_out, *geom, oracle.ACT_RELU,
                                          inputs.from_bf16(x16[image * plane_in:(image + 1) * plane_in]), inputs.from_bf16(w16), bias,
                                          threads=8)
        check(got[image * plane_out:(image + 1) * plane_out], want, f"config 2, image {image}")
    order = np.random.default_rng(4).permutation(batch)
    permuted = x16.reshape(batch, plane_in)[order].ravel()
    again, _ = run(hip, shape, 1, permuted, w16, bias)
    assert (again.reshape(batch, plane_out).view(np.uint32) == got.reshape(batch, plane_out)[order].view(np.uint32)).all()
    plain, _ = run(hip, shape, 0, x16, w16, None)
    doubled, _ = run(hip, shape, 0, inputs.to_bf16(2.0 * inputs.from_bf16(x16)), w16, None)
    assert (doubled.view(np.uint32) == (2.0 * plain).view(np.uint32)).all()


def test_unsupported_and_invalid_arguments(hip):
    d = hip.DeviceBuffer(1 << 12)
    with pytest.raises(hip.HipErr):   # no output at all
        hip.conv2d_bias_act_bf16_dev(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), 0, d, d, None, None, None)
    with pytest.raises(hip.HipErr):   # kernel larger than the padded image
        hip.conv2d_bias_act_bf16_dev(1, 1, 2, 2, 1, (5, 5), (1, 1), (0, 0), (1, 1), 0, d, d, None, d, None)
    with pytest.raises(hip.HipErr):   # unknown activation
        hip.conv2d_bias_act_bf16_dev(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), 7, d, d, None, d, None)
    with pytest.raises(hip.HipErr) as info:  # misaligned f32 output
        hip.conv2d_bias_act_bf16_dev(1, 1, 2, 2, 1, (1, 1), (1, 1), (0, 0), (1, 1), 0, d, d, None, d.at(4), None)
    assert info.value.kind == "Unsupported" or "aligned" in info.value.message
    # an empty batch is a no-op
    hip.conv2d_bias_act_bf16_dev(0, 3, 8, 8, 4, (3, 3), (1, 1), (1, 1), (1, 1), 0, d, d, None, d, None)
