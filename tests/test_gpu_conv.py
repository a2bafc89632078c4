"""Parity of the fused implicit-GEMM conv2d (+bias, +activation) against the CPU oracle."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close
from test_oracle_conv import generated_case

pytestmark = pytest.mark.gpu


def run(hip, batch, c_in, h, w, c_out, kernel, stride, padding, dilation, act, x, wt, b):
    oh, ow = hip.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    out = np.zeros(batch * c_out * oh * ow, np.float32)
    hip.conv2d_bias_activation_f32(batch, c_in, h, w, c_out, kernel, stride, padding, dilation, act,
                                   np.ascontiguousarray(x, np.float32).ravel(),
                                   np.ascontiguousarray(wt, np.float32).ravel(), b, out)
    return out


def test_layout_known_answer(hip, golden):
    c = golden["conv_layout"]
    out = run(hip, c["batch"], c["c_in"], *c["input_hw"], c["c_out"], c["kernel"], c["stride"], c["padding"],
              c["dilation"], 0, np.array(c["input"], np.float32), np.array(c["weight"], np.float32),
              np.array(c["bias"], np.float32))
    assert out.tolist() == c["expected"]


def test_output_hw(hip, golden):
    for c in golden["conv_output_hw"]:
        assert list(hip.conv2d_output_hw(*c["input_hw"], c["kernel"], c["stride"], c["padding"],
                                         c["dilation"])) == c["expected"]
    with pytest.raises(hip.HipErr):
        hip.conv2d_output_hw(2, 2, (5, 5), (1, 1), (0, 0), (1, 1))


def test_reference_generated_cases(hip, oracle, golden):
    for case in golden["conv_generated"]:
        x, weight, bias = generated_case(case)
        h, w = case["input_hw"]
        args = (case["batch"], case["c_in"], h, w, case["c_out"], case["kernel"], case["stride"], case["padding"],
                case["dilation"])
        got = run(hip, *args, 0, x, weight, bias)
        want = oracle.conv2d_bias_act_f32(*args, oracle.ACT_NONE, x, weight, bias)
        assert_close(got, want, 0, case["tolerance"], case["source"])


@pytest.mark.parametrize("shape", [
    (2, 3, 9, 7, 4, (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 2, 9, 9, 3, (3, 3), (1, 1), (0, 0), (2, 2)),
    (3, 5, 6, 11, 7, (2, 4), (2, 3), (1, 2), (1, 1)),
    (2, 4, 5, 5, 6, (1, 1), (1, 1), (0, 0), (1, 1)),
    (1, 1, 4, 4, 1, (4, 4), (1, 1), (0, 0), (1, 1)),
    (2, 16, 20, 20, 70, (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 8, 33, 17, 130, (5, 3), (2, 1), (2, 1), (1, 2)),
    (5, 7, 12, 12, 64, (3, 3), (2, 2), (0, 0), (1, 1)),
])
def test_random_shapes(hip, oracle, shape):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    rng = np.random.default_rng(abs(hash(shape)) % 2 ** 32)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, np.sqrt(2.0 / (c_in * kernel[0] * kernel[1])), c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    for act, code in ((0, oracle.ACT_NONE), (1, oracle.ACT_RELU), (2, oracle.ACT_GELU)):
        got = run(hip, *shape, act, x, wt, b)
        want = oracle.conv2d_bias_act_f32(*shape, code, x, wt, b)
        assert_close(got, want, F32_REL, F32_ABS, f"conv {shape} act={act}")
    got = run(hip, *shape, 1, x, wt, None)
    assert_close(got, oracle.conv2d_bias_act_f32(*shape, oracle.ACT_RELU, x, wt, None), F32_REL, F32_ABS, "no bias")


@pytest.fixture
def force_family(hip):
    """Forces a conv kernel family for one test and gives the choice back to the dispatcher afterwards."""
    yield hip.conv2d_force_family
    hip.conv2d_force_family("auto")


@pytest.mark.parametrize("family", ["tile", "auto"])
@pytest.mark.parametrize("shape", [
    (1, 192, 12, 12, 40, (7, 7), (1, 1), (3, 3), (1, 1)),    # 9408 terms: two table segments (ConvNeXt-style 7×7)
    (2, 170, 9, 9, 70, (7, 7), (2, 2), (3, 3), (1, 1)),      # 8330 terms, k % 16 != 0, strided
    (1, 384, 8, 8, 33, (7, 7), (1, 1), (3, 3), (1, 1)),      # 18816 terms: three segments
    (1, 1030, 6, 6, 20, (3, 3), (1, 1), (1, 1), (1, 1)),     # 9270 terms, k % 4 != 0: scalar weight staging
])
def test_reductions_longer_than_the_offset_table(hip, oracle, force_family, shape, family):
    """c_in·kh·kw beyond the 8192 entries of the general kernel's LDS offset table: the table is rebuilt segment by
    segment while the accumulators run on (the general kernel forced), or — the dispatcher's own choice for these few
    tiles — the reduction is cut into slices over workgroups.  He-scaled weights; compared against the oracle with the
    bound a reordered f32 sum of that length supports (a small multiple of unit roundoff times sum |x||w|)."""
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    force_family(family)
    assert hip.conv2d_planned_kernel(*shape) == ("tile" if family == "tile" else "tile_ksliced")
    rng = np.random.default_rng(c_in * 31 + c_out)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, np.sqrt(2.0 / (c_in * kernel[0] * kernel[1])), c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    got = run(hip, *shape, 1, x, wt, b)
    want = oracle.conv2d_bias_act_f32(*shape, oracle.ACT_RELU, x, wt, b)
    magnitude = oracle.conv2d_bias_act_f32(*shape, oracle.ACT_NONE, np.abs(x), np.abs(wt), None)
    assert_close(got, want, F32_REL, F32_ABS + 2 * 2.0 ** -24 * float(magnitude.max()), f"conv {shape}")
    assert float(np.abs(got).max()) > 0.1  # the comparison is not about zeros


@pytest.mark.parametrize("shape", [
    (1, 512, 7, 7, 512, (3, 3), (1, 1), (1, 1), (1, 1)),      # deep layer on a tiny plane at batch 1: 4608 terms, 4 tiles
    (2, 351, 7, 10, 47, (4, 4), (1, 1), (3, 1), (1, 1)),
    (1, 130, 9, 9, 40, (3, 3), (1, 1), (1, 1), (1, 1)),       # 1170 terms: the last slice ends inside a k-tile
    (3, 157, 19, 15, 1, (7, 7), (1, 1), (0, 0), (1, 1)),      # one output channel
    (1, 2048, 7, 7, 512, (1, 1), (1, 1), (0, 0), (1, 1)),
    (2, 366, 5, 44, 24, (4, 4), (2, 2), (3, 0), (2, 2)),      # strided and dilated
])
def test_few_tiles_with_a_long_reduction_are_cut_into_slices(hip, oracle, shape):
    """Every kernel walks c_in·kh·kw serially inside a workgroup; when the tiles alone would leave most of the chip idle
    the reduction is cut over workgroups, the partial planes are added in slice order and bias and activation follow."""
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    assert hip.conv2d_planned_kernel(*shape) == "tile_ksliced"
    rng = np.random.default_rng(c_in * 7 + c_out)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, np.sqrt(2.0 / (c_in * kernel[0] * kernel[1])), c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
    b = rng.uniform(-0.5, 0.5, c_out).astype(np.float32)
    magnitude = oracle.conv2d_bias_act_f32(*shape, oracle.ACT_NONE, np.abs(x), np.abs(wt), None)
    slack = F32_ABS + 2 * 2.0 ** -24 * float(magnitude.max())
    for act, code in ((0, oracle.ACT_NONE), (1, oracle.ACT_RELU), (2, oracle.ACT_GELU)):
        got = run(hip, *shape, act, x, wt, b)
        assert_close(got, oracle.conv2d_bias_act_f32(*shape, code, x, wt, b), F32_REL, slack, f"conv {shape} act={act}")
        assert (run(hip, *shape, act, x, wt, b) == got).all(), "slices are added in a fixed order"
    got = run(hip, *shape, 0, x, wt, None)
    assert_close(got, oracle.conv2d_bias_act_f32(*shape, oracle.ACT_NONE, x, wt, None), F32_REL, slack, "no bias")


@pytest.mark.parametrize("shape", [
    (8, 16, 96, 96, 3, (3, 3), (1, 1), (1, 1), (1, 1)),       # an RGB head
    (4, 5, 130, 131, 1, (5, 5), (1, 1), (2, 2), (1, 1)),      # one channel; rows that are not a multiple of 4 pixels
    (2, 4, 190, 190, 2, (7, 7), (1, 1), (3, 3), (1, 1)),      # seven taps a row: the loop over kernel rows is not unrolled
    (4, 3, 130, 130, 2, (3, 5), (1, 1), (1, 2), (1, 1)),      # kernel height and width differ
    (8, 8, 200, 200, 4, (3, 3), (2, 2), (1, 1), (1, 1)),      # strided along x: a thread per pixel
    (7, 6, 100, 101, 2, (3, 3), (1, 1), (2, 2), (2, 2)),      # dilated
    (8, 2, 140, 120, 3, (2, 4), (1, 2), (3, 0), (1, 1)),      # padding wider than the kernel's reach on one side
])
def test_few_output_channels_over_many_pixels(hip, oracle, shape):
    """At most four output channels over at least 65536 output pixels: a thread per output pixel (or per four adjacent
    ones) instead of matrix tiles that would be mostly padding."""
    assert hip.conv2d_planned_kernel(*shape) == "direct"
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    rng = np.random.default_rng(c_in * 7 + c_out + h)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, np.sqrt(2.0 / (c_in * kernel[0] * kernel[1])), c_out * c_in * kernel[0] * kernel[1]).astype(np.float32)
    b = rng.uniform(-0.5, 0.5, c_out).astype(np.float32)
    for act, code in ((0, oracle.ACT_NONE), (1, oracle.ACT_RELU), (2, oracle.ACT_GELU)):
        got = run(hip, *shape, act, x, wt, b)
        assert_close(got, oracle.conv2d_bias_act_f32(*shape, code, x, wt, b), F32_REL, F32_ABS, f"conv {shape} act={act}")
    got = run(hip, *shape, 0, x, wt, None)
    assert_close(got, oracle.conv2d_bias_act_f32(*shape, oracle.ACT_NONE, x, wt, None), F32_REL, F32_ABS, "no bias")
    assert float(np.abs(got).max()) > 0.1


G33 = ((3, 3), (1, 1), (1, 1), (1, 1))
FAMILY_SHAPES = {
    # name: (batch, c_in, h, w, c_out, kernel, stride, padding, dilation)
    "ragged_strip": (2, 16, 20, 20, 70, *G33),           # ragged channel strip, 13 pixel blocks, ragged last block
    "c130": (1, 130, 12, 12, 40, *G33),                  # packed weight rows, K % 4 != 0: scalar weight staging
    "chunks_c4": (1, 4, 60, 60, 33, *G33),               # several pixel chunks per image
    "stride2_c8": (5, 8, 13, 12, 64, (3, 3), (2, 2), (0, 0), (1, 1)),
    "dilated_c6": (2, 6, 15, 14, 32, (3, 3), (1, 2), (2, 3), (2, 1)),   # dilation, wide padding, three channel pairs
    "row_of_nine": (2, 32, 9, 9, 16, (1, 9), (1, 1), (0, 4), (1, 1)),    # nine taps in one row
    "blocks56": (64, 2, 42, 42, 128, *G33),              # 56 blocks per workgroup: seven per wavefront
    "blocks44": (64, 2, 44, 32, 128, *G33),              # 44 blocks: six and five per wavefront
    "c112": (2, 112, 14, 14, 40, *G33),                  # packed rows (more than 104 channels), ragged second strip
    "c128_odd_plane": (3, 128, 11, 13, 70, *G33),        # packed rows, plane of 143 pixels (not a multiple of 4)
    "c96": (2, 96, 12, 12, 64, *G33),                    # padded rows but no LDS left for the 128-bit store path
    "stride2_c32": (2, 32, 21, 21, 48, (3, 3), (2, 2), (1, 1), (1, 1)),  # stride 2, plane of 121 pixels
    "dilated_c48": (2, 48, 19, 17, 33, (3, 3), (1, 1), (2, 2), (2, 2)),  # dilation 2, plane of 323 pixels
    "chunks_c16": (1, 16, 64, 64, 32, *G33),             # 128 blocks of one image split over several workgroups
    "fuzz_c64_p0": (3, 64, 33, 33, 160, (3, 3), (1, 1), (0, 0), (1, 1)),  # no padding, two channel tiles
    "ring64": (2, 16, 20, 20, 40, *G33),                 # 64-row ring tiles
    "ring_5x5": (2, 16, 15, 15, 130, (5, 5), (1, 1), (2, 2), (1, 1)),    # 25 taps, ragged channel tile
    "ring_7x7": (2, 32, 17, 15, 70, (7, 7), (1, 1), (3, 3), (1, 1)),     # 49 taps: the upper word of the tap mask
    "ring_7x7_s2": (2, 16, 23, 23, 40, (7, 7), (2, 2), (3, 3), (1, 1)),  # 49 taps, stride 2, 64-row tiles
}
# (shape, forced family, the kernel that has to run)
FAMILY_CASES = [
    ("ragged_strip", "strip", "strip12_wide"), ("c130", "strip", "strip9"), ("chunks_c4", "strip", "strip12_wide"),
    ("stride2_c8", "strip", "strip12"), ("dilated_c6", "strip", "strip12"), ("row_of_nine", "strip", "strip12"),
    ("blocks56", "strip", "strip12_wide"), ("blocks44", "strip", "strip12_wide"), ("c112", "strip", "strip9"),
    ("c128_odd_plane", "strip", "strip9"), ("c96", "strip", "strip12"), ("stride2_c32", "strip", "strip12"),
    ("dilated_c48", "strip", "strip12"), ("chunks_c16", "strip", "strip12_wide"), ("fuzz_c64_p0", "strip", "strip12"),
    ("ragged_strip", "ring", "ring"), ("row_of_nine", "ring", "ring"), ("c112", "ring", "ring"),
    ("c128_odd_plane", "ring", "ring"), ("stride2_c32", "ring", "ring"), ("dilated_c48", "ring", "ring"),
    ("chunks_c16", "ring", "ring"), ("fuzz_c64_p0", "ring", "ring"), ("ring64", "ring", "ring"),
    ("ring_5x5", "ring", "ring"), ("ring_7x7", "ring", "ring"), ("ring_7x7_s2", "ring", "ring"), ("ring_7x7", "tile", "tile"),
    ("ragged_strip", "tile", "tile"), ("c130", "tile", "tile"), ("chunks_c4", "tile", "tile"),
    ("stride2_c8", "tile", "tile"), ("dilated_c6", "tile", "tile"), ("row_of_nine", "tile", "tile"),
    ("blocks56", "tile", "tile"), ("c112", "tile", "tile"), ("stride2_c32", "tile", "tile"),
    ("dilated_c48", "tile", "tile"), ("ring_5x5", "tile", "tile"),
]


@pytest.mark.parametrize("name,family,kernel", FAMILY_CASES)
def test_kernel_families(hip, oracle, force_family, name, family, kernel):
    """Each kernel family (chosen by shape in normal use) forced on shapes that exercise its edges; the dispatcher
    is asked which kernel it runs, so a case cannot pass on another family's kernel."""
    shape = FAMILY_SHAPES[name]
    force_family(family)
    assert hip.conv2d_planned_kernel(*shape) == kernel
    batch, c_in, h, w, c_out, kernel_hw, stride, padding, dilation = shape
    rng = np.random.default_rng(batch * 1000 + c_in * 10 + c_out)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, np.sqrt(2.0 / (c_in * 9)), c_out * c_in * kernel_hw[0] * kernel_hw[1]).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    got = run(hip, *shape, 1, x, wt, b)
    want = oracle.conv2d_bias_act_f32(*shape, oracle.ACT_RELU, x, wt, b, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"conv {name} {shape} family={family}")


def test_forced_family_that_cannot_serve_is_an_error(hip, force_family):
    """A forced family never silently falls back: the ring kernel needs c_in*kh*kw % 16 == 0, the strip kernel nine
    taps and an even channel count."""
    shape = (1, 4, 8, 8, 8, *G33)
    x, wt = np.zeros(4 * 64, np.float32), np.zeros(8 * 36, np.float32)
    out = np.full(8 * 64, 13.0, np.float32)
    force_family("ring")
    assert hip.conv2d_planned_kernel(*shape) is None
    with pytest.raises(hip.HipErr, match="forced conv2d kernel family cannot serve"):
        hip.conv2d_bias_activation_f32(*shape, 0, x, wt, None, out)
    force_family("strip")
    odd = (1, 3, 8, 8, 8, *G33)
    assert hip.conv2d_planned_kernel(*odd) is None
    with pytest.raises(hip.HipErr, match="forced conv2d kernel family cannot serve"):
        hip.conv2d_bias_activation_f32(*odd, 0, np.zeros(3 * 64, np.float32), np.zeros(8 * 27, np.float32), None, out)
    assert (out == 13.0).all()
    with pytest.raises(hip.HipErr, match="unknown conv2d kernel family"):
        hip._check(hip._lib.load().st_hip_conv2d_force_family(9))


def test_dispatcher_choices(hip):
    """What runs without forcing: config 2 and its grad_input on the strip kernels, many-tile layers on the ring
    kernel, reductions that are not a multiple of 16 on the general kernel."""
    assert hip.conv2d_planned_kernel(32, 64, 56, 56, 128, *G33) == "strip12_wide"
    assert hip.conv2d_planned_kernel(32, 64, 56, 56, 128, *G33, direction="grad_input") == "strip9"
    assert hip.conv2d_planned_kernel(64, 64, 56, 56, 256, *G33) == "ring"
    assert hip.conv2d_planned_kernel(8, 3, 32, 32, 16, *G33) == "tile"
    assert hip.conv2d_planned_kernel(1, 512, 7, 7, 512, *G33) == "tile_ksliced"
    assert hip.conv2d_planned_kernel(64, 512, 7, 7, 512, *G33) == "ring"
    assert hip.conv2d_planned_kernel(2, 8, 9, 9, 4, (3, 3), (2, 2), (1, 1), (1, 1), direction="grad_input") == "col2im"
    assert hip.conv2d_planned_kernel(2, 64, 9, 9, 4, (3, 3), (2, 1), (1, 1), (1, 1), direction="grad_input") == "adjoint"
    assert hip.conv2d_planned_kernel(32, 3, 224, 224, 768, (16, 16), (16, 16), (0, 0), (1, 1), direction="grad_input") == "col2im"


def test_strip_kernel_store_paths_agree(hip, oracle, force_family):
    """The strip kernel stores 128 bits per lane through an LDS tile when the output is 16-byte aligned and the
    plane size is a multiple of four, 32 bits per lane otherwise: same values either way."""
    force_family("strip")
    shape = (3, 16, 20, 20, 70, (3, 3), (1, 1), (1, 1), (1, 1))
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = shape
    rng = np.random.default_rng(77)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wt = rng.normal(0, 0.1, c_out * c_in * 9).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, c_out).astype(np.float32)
    n_out = batch * c_out * 20 * 20
    d_x, d_w, d_b = (hip.DeviceBuffer.from_array(a) for a in (x, wt, b))
    d_out = hip.DeviceBuffer((n_out + 1) * 4)
    hip.conv2d_bias_act_f32_dev(*shape, 1, d_x, d_w, d_b, d_out)
    hip.device_synchronize()
    aligned = d_out.to_array(np.float32, n_out + 1)[:n_out].copy()
    d_out.zero()
    hip.conv2d_bias_act_f32_dev(*shape, 1, d_x, d_w, d_b, d_out.at(4))
    hip.device_synchronize()
    shifted = d_out.to_array(np.float32, n_out + 1)[1:]
    assert (aligned == shifted).all()
    assert_close(aligned, oracle.conv2d_bias_act_f32(*shape, oracle.ACT_RELU, x, wt, b, threads=8), F32_REL, F32_ABS, "strip stores")


def test_conv2d_layer_mirror(hip, oracle):
    from spiraltorch_amd import Conv2d, Tensor, TensorError
    conv = Conv2d("conv_gpu", 3, 8, (3, 3), (1, 1), (1, 1), (1, 1), (8, 8))
    assert conv.output_hw() == (8, 8)
    assert conv.bias.data().tolist() == [0.0] * 8
    x = Tensor(4, 3 * 8 * 8, np.random.default_rng(0).normal(size=4 * 192))
    got = conv.forward(x)
    want = oracle.conv2d_bias_act_f32(4, 3, 8, 8, 8, (3, 3), (1, 1), (1, 1), (1, 1), oracle.ACT_NONE, x.data(),
                                      conv.weight.data(), conv.bias.data())
    assert got.shape() == (4, 8 * 8 * 8)
    assert_close(got.data(), want, F32_REL, F32_ABS, "Conv2d.forward")
    with pytest.raises(TensorError):
        conv.forward(Tensor(4, 10))
    with pytest.raises(TensorError):
        Conv2d("bad", 1, 1, (5, 5), (1, 1), (0, 0), (1, 1), (2, 2))
    empty = conv.forward(Tensor(0, 192))
    assert empty.shape() == (0, 512)  # conv.rs:4132-4137


def test_validation_before_mutation(hip):
    out = np.full(2 * 4 * 4 * 4, 13.0, np.float32)
    x = np.zeros(2 * 3 * 4 * 4, np.float32)
    w = np.zeros(4 * 3 * 3 * 3, np.float32)
    args = (2, 3, 4, 4, 4, (3, 3), (1, 1), (1, 1), (1, 1), 1)
    with pytest.raises(hip.HipErr, match="input buffer length"):
        hip.conv2d_bias_activation_f32(*args, x[:-1], w, None, out)
    with pytest.raises(hip.HipErr, match="weight buffer length"):
        hip.conv2d_bias_activation_f32(*args, x, w[:-1], None, out)
    with pytest.raises(hip.HipErr, match="bias buffer length 3 does not match c_out=4"):
        hip.conv2d_bias_activation_f32(*args, x, w, np.zeros(3, np.float32), out)
    with pytest.raises(hip.HipErr, match="output buffer length"):
        hip.conv2d_bias_activation_f32(*args, x, w, None, out[:-1])
    with pytest.raises(hip.HipErr, match="unknown activation"):
        hip.conv2d_bias_activation_f32(*args[:-1], 7, x, w, None, out)
    assert (out == 13.0).all()


def test_config2_full_size(hip, oracle):
    """BASELINE config 2: N32 C64->128 56x56 3x3 s1 p1, bias + ReLU.  The oracle checks two whole images
    (first and last); all 32 are covered by batch-permutation equivariance and by exact 2x linearity."""
    from spiraltorch_amd import inputs
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    x = inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w)
    wt = inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, float(np.sqrt(2.0 / (c_in * 9))))
    b = inputs.uniform(inputs.seed_for(2, 2), c_out, -0.1, 0.1)
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    got = run(hip, batch, c_in, h, w, c_out, *geom, 1, x, wt, b).reshape(batch, -1)
    xi = x.reshape(batch, -1)
    for image in (0, 31):
        want = oracle.conv2d_bias_act_f32(1, c_in, h, w, c_out, *geom, oracle.ACT_RELU, xi[image], wt, b, threads=8)
        assert_close(got[image], want, F32_REL, F32_ABS, f"config 2 image {image}")
    perm = np.random.default_rng(2).permutation(batch)
    got_perm = run(hip, batch, c_in, h, w, c_out, *geom, 1, xi[perm], wt, b).reshape(batch, -1)
    assert (got_perm == got[perm]).all()
    doubled = run(hip, batch, c_in, h, w, c_out, *geom, 1, 2 * x, wt, 2 * b).reshape(batch, -1)
    assert (doubled == 2 * got).all()
