"""The allocation-free grad_input entry point (weights re-laid into a static device array) against the entry point
it is a variant of: bit-identical results wherever both run the same kernels (within the f32 parity bar where the
allocating entry point cuts a long reduction into slices kept in scratch memory, which this one must not touch), on
calls in a row, each second one with a smaller input; oversized weights are refused before anything is launched."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close

pytestmark = pytest.mark.gpu

G33 = ((3, 3), (1, 1), (1, 1), (1, 1))
CALLS = [
    # batch, c_in, h, w, c_out, kernel, stride, padding, dilation — run in this order on one stream
    (4, 64, 28, 28, 128, *G33),                            # strip kernel on 128 'input' channels
    (2, 16, 14, 14, 32, *G33),                             # smaller: reuses the front of the array
    (2, 64, 9, 9, 250, (3, 3), (2, 1), (1, 0), (1, 1)),    # strided: adjoint gather in both entry points
    (1, 3, 8, 8, 4, (5, 5), (1, 1), (2, 2), (1, 1)),       # smaller again, general kernel
]


def test_matches_the_allocating_entry_point_call_after_call(hip):
    stream = hip.Stream()
    for repeat in range(2):
        for case in CALLS:
            batch, c_in, h, w, c_out, kernel, stride, padding, dilation = case
            oh, ow = hip.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
            rng = np.random.default_rng(c_in * 1000 + c_out + repeat)
            wgt = rng.normal(0, 0.1, c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
            g = rng.normal(size=batch * c_out * oh * ow).astype(np.float32)
            d_g, d_w = hip.DeviceBuffer.from_array(g), hip.DeviceBuffer.from_array(wgt)
            n = batch * c_in * h * w
            d_want, d_got = hip.DeviceBuffer(n * 4), hip.DeviceBuffer(n * 4)
            d_got.zero(stream)
            hip.conv2d_grad_input_f32_dev(*case, d_g, d_w, d_want, stream)
            hip.conv2d_grad_input_f32_noalloc_dev(*case, d_g, d_w, d_got, stream)
            stream.synchronize()
            want, got = d_want.to_array(np.float32, n), d_got.to_array(np.float32, n)
            assert np.isfinite(want).all() and np.abs(want).max() > 0
            if hip.conv2d_planned_kernel(*case, direction="grad_input") == "tile_ksliced":
                assert_close(got, want, F32_REL, F32_ABS, f"{case} (pass {repeat})")
            else:
                assert (got == want).all(), f"{case} (pass {repeat})"
    stream.destroy()


def test_weights_beyond_the_static_array_are_refused(hip):
    # 900 -> 900 channels, 3x3: 29 MB of weights against 16 MiB of scratch; rejected before any pointer is used
    case = (1, 900, 4, 4, 900, *G33)
    assert 900 * 900 * 9 * 4 > hip.NOALLOC_SCRATCH_BYTES
    with pytest.raises(hip.HipErr, match="exceed the static scratch"):
        hip.conv2d_grad_input_f32_noalloc_dev(*case, 16, 16, 16)
    # the largest that fits: exactly 16 MiB of weights (2048 x 2048, 1x1)
    case = (1, 2048, 2, 2, 2048, (1, 1), (1, 1), (0, 0), (1, 1))
    rng = np.random.default_rng(5)
    wgt = rng.normal(0, 0.02, 2048 * 2048).astype(np.float32)
    g = rng.normal(size=2048 * 4).astype(np.float32)
    d_g, d_w = hip.DeviceBuffer.from_array(g), hip.DeviceBuffer.from_array(wgt)
    d_want, d_got = hip.DeviceBuffer(2048 * 4 * 4), hip.DeviceBuffer(2048 * 4 * 4)
    hip.conv2d_grad_input_f32_dev(*case, d_g, d_w, d_want)
    hip.conv2d_grad_input_f32_noalloc_dev(*case, d_g, d_w, d_got)
    hip.device_synchronize()
    # (the allocating entry point cuts this 2048-term reduction over 16 tiles into slices; this one may not)
    assert hip.conv2d_planned_kernel(*case, direction="grad_input") == "tile_ksliced"
    assert_close(d_got.to_array(np.float32, 2048 * 4), d_want.to_array(np.float32, 2048 * 4), F32_REL, F32_ABS, "16 MiB of weights")
