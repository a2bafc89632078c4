"""Parity of the conv2d backward kernels (grad_input, grad_weight, grad_bias) against the CPU oracle:
1e-4 rel / 1e-5 abs (plus a floor proportional to the summed magnitudes for the long grad_weight sums, and for
grad_input reductions of ~1000 products the rounding term stated in assert_grad_input)."""
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
    (1, 24, 10, 10, 192, (7, 7), (1, 1), (3, 3), (1, 1)),  # c_out*kh*kw = 9408: more than one offset-table segment
    (1, 20, 11, 11, 180, (7, 7), (2, 2), (3, 3), (1, 1)),  # stride 2, 8820 terms: GEMM + col2im
    (1, 128, 11, 11, 180, (7, 7), (1, 2), (3, 3), (1, 1)), # the same through the adjoint gather (whole channel tile, stride 1×2)
    # grad_weight with three runs of steps per workgroup (128 × 192 tiles, at least three runs per tile):
    (1, 64, 25, 25, 128, (3, 3), (1, 1), (1, 1), (1, 1)),  # 40 runs of one step: the last workgroup has one busy set of three
    (7, 64, 33, 31, 128, (3, 3), (1, 1), (1, 1), (1, 1)),  # 224 runs of two steps: the last workgroup has two busy sets
    (2, 128, 12, 12, 256, (3, 3), (1, 1), (1, 1), (1, 1)), # twelve tiles (two channel tiles × six column tiles), 18 runs
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
    if c_out * kernel[0] * kernel[1] > 2000:
        assert_grad_input(gi, case, g, wgt, want_gi, f"grad_input {case}")  # long reduction: bound from float64
    else:
        assert_close(gi, want_gi, F32_REL, F32_ABS, f"grad_input {case}")
    # grad_weight / grad_bias add batch*oh*ow terms in a different order than the oracle
    floor = 2e-7 * float(np.abs(g).max()) * float(np.abs(x).max()) * oh * ow
    assert_close(gw, want_gw, F32_REL, F32_ABS + floor, f"grad_weight {case}")
    assert_close(gb, want_gb, F32_REL, F32_ABS + floor, f"grad_bias {case}")


def grad_input_f64(case, g, wgt, magnitudes=False):
    """grad_input from its definition in float64 (no patch matrix): every (ky, kx) tap scatters
    grad_output · W[:, :, ky, kx] to the input positions it read.  With `magnitudes` the same sum over |g|·|w|,
    the quantity a rounding-error bound of the reduction is proportional to."""
    batch, c_in, h, w, c_out, (kh, kw), (sh, sw), (ph, pw), (dh, dw) = case
    oh = (h + 2 * ph - ((kh - 1) * dh + 1)) // sh + 1
    ow = (w + 2 * pw - ((kw - 1) * dw + 1)) // sw + 1
    G = np.asarray(g, np.float64).reshape(batch, c_out, oh, ow)
    W = np.asarray(wgt, np.float64).reshape(c_out, c_in, kh, kw)
    if magnitudes:
        G, W = np.abs(G), np.abs(W)
    gi = np.zeros((batch, c_in, h, w))
    oy, ox = np.arange(oh), np.arange(ow)
    for ky in range(kh):
        iy = oy * sh + ky * dh - ph
        vy = (iy >= 0) & (iy < h)
        for kx in range(kw):
            ix = ox * sw + kx * dw - pw
            vx = (ix >= 0) & (ix < w)
            contrib = np.einsum("nohw,oc->nchw", G[:, :, vy][:, :, :, vx], W[:, :, ky, kx])
            gi[np.ix_(np.arange(batch), np.arange(c_in), iy[vy], ix[vx])] += contrib
    return gi.ravel()


EPS32 = 2.0 ** -24


def assert_grad_input(got, case, g, wgt, oracle_value, what):
    """grad_input against exact float64 with the bound the arithmetic supports.  The kernels add the c_out*kh*kw
    products of one input position in a single chain of f32 fused multiply-adds (what the f32 matrix instruction
    is: bit-identical to fmaf applied in k order); the reference — and the oracle — first add c_out products per tap
    (G·W) and then the taps (col2im), a blocked sum whose error is about sqrt(kh*kw) smaller.  Where the result
    lands near zero (He-scaled weights, c_out*kh*kw ~ 1000) neither 1e-4 relative nor 1e-5 absolute describes the
    chain's error, so the bound carries the standard term for a reordered f32 sum, a small multiple of unit
    roundoff times sum |g||w| (measured need on the shapes below: at most 0.2 of that unit; the oracle itself sits
    within the same bound)."""
    exact = grad_input_f64(case, g, wgt)
    bound = F32_REL * np.abs(exact) + F32_ABS + 2 * EPS32 * grad_input_f64(case, g, wgt, magnitudes=True)
    for name, value in (("gpu", got), ("oracle", oracle_value)):
        err = np.abs(np.asarray(value, np.float64) - exact)
        worst = int(np.argmax(err - bound))
        assert (err <= bound).all(), f"{what}: {name} grad_input off at {worst}: |diff| {err[worst]:.3e} bound {bound[worst]:.3e}"


HE_CASES = [
    # the shapes a randomised search found outside 1e-4 / 1e-5 against the oracle: He-scaled weights, c_out >= 100
    ("ring", "ring", (3, 64, 33, 33, 160, (3, 3), (1, 1), (0, 0), (1, 1))),
    ("tile", "tile", (4, 16, 19, 26, 100, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("tile", "tile", (3, 2, 38, 35, 160, (3, 3), (1, 1), (2, 0), (1, 2))),
    ("auto", "col2im", (3, 2, 38, 24, 128, (3, 3), (2, 1), (0, 1), (2, 1))),
    ("auto", "adjoint", (3, 64, 20, 18, 128, (3, 3), (2, 1), (0, 1), (2, 1))),
    ("ring", "ring", (4, 16, 28, 32, 160, (3, 3), (1, 1), (0, 0), (1, 1))),
    ("strip", "strip9", (2, 16, 30, 30, 128, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("strip", "strip12", (2, 32, 17, 19, 100, (3, 3), (1, 1), (1, 1), (1, 1))),
]


@pytest.mark.parametrize("family,kernel,case", HE_CASES)
def test_grad_input_long_reductions_with_he_scaled_weights(hip, oracle, force_family, family, kernel, case):
    batch, c_in, h, w, c_out, kernel_hw, stride, padding, dilation = case
    force_family(family)
    assert hip.conv2d_planned_kernel(*case, direction="grad_input") == kernel
    rng = np.random.default_rng(c_in * 1000 + c_out)
    oh, ow = oracle.conv2d_output_hw(h, w, kernel_hw, stride, padding, dilation)
    x = rng.normal(size=batch * c_in * h * w).astype(np.float32)
    wgt = rng.normal(0, np.sqrt(2.0 / (c_in * 9)), c_out * c_in * 9).astype(np.float32)
    g = rng.normal(size=batch * c_out * oh * ow).astype(np.float32)
    gi, gw, gb = (np.zeros(n, np.float32) for n in (x.size, wgt.size, c_out))
    hip.conv2d_backward_f32(*case, x, wgt, g, gi, gw, gb)
    want_gi, want_gw, want_gb = oracle.conv2d_backward_f32(*case, x, wgt, g)
    assert_grad_input(gi, case, g, wgt, want_gi, f"{case}")
    floor = 2e-7 * float(np.abs(g).max()) * float(np.abs(x).max()) * oh * ow
    assert_close(gw, want_gw, F32_REL, F32_ABS + floor, f"grad_weight {case}")
    assert_close(gb, want_gb, F32_REL, F32_ABS + floor, f"grad_bias {case}")


@pytest.fixture
def force_family(hip):
    yield hip.conv2d_force_family
    hip.conv2d_force_family("auto")


GRAD_INPUT_FAMILY_CASES = [
    # forced family, kernel that has to run, (batch, c_in, h, w, c_out, kernel, stride, padding, dilation);
    # the forward kernels see c_out as their input channels
    ("strip", "strip9", (2, 24, 14, 14, 112, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("strip", "strip9", (3, 70, 11, 13, 128, (3, 3), (1, 1), (1, 1), (1, 1))),     # ragged strips, plane of 143
    ("strip", "strip9", (2, 33, 12, 12, 130, (3, 3), (1, 1), (0, 0), (1, 1))),     # adjoint padding 2, K % 4 != 0
    ("strip", "strip12", (2, 40, 13, 11, 96, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("strip", "strip12_wide", (2, 40, 12, 12, 64, (3, 3), (1, 1), (1, 1), (2, 2))),  # dilation 2 -> adjoint padding 3
    ("strip", "strip12_wide", (1, 8, 64, 64, 16, (3, 3), (1, 1), (1, 1), (1, 1))),   # several chunks per image
    ("ring", "ring", (2, 70, 20, 20, 16, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("ring", "ring", (2, 130, 15, 15, 16, (5, 5), (1, 1), (2, 2), (1, 1))),
    ("ring", "ring", (2, 24, 14, 14, 112, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("ring", "ring", (2, 20, 13, 12, 32, (7, 7), (1, 1), (3, 3), (1, 1))),          # 49 taps
    ("tile", "tile", (2, 24, 14, 14, 112, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("tile", "tile", (2, 5, 10, 11, 6, (3, 3), (1, 1), (2, 2), (1, 1))),
    # the first layer of an image model: its grad_input has three 'output' channels over many pixels
    ("auto", "direct", (8, 3, 96, 96, 16, (3, 3), (1, 1), (1, 1), (1, 1))),
    ("auto", "adjoint", (2, 64, 9, 9, 250, (3, 3), (2, 1), (1, 0), (1, 1))),        # whole channel tile, stride 2×1
    ("auto", "adjoint", (2, 128, 10, 11, 6, (3, 3), (1, 1), (3, 3), (1, 1))),       # padding beyond the kernel's reach
    ("auto", "col2im", (2, 22, 9, 9, 250, (3, 3), (2, 1), (1, 0), (1, 1))),         # ragged channel tile: GEMM + col2im
    ("auto", "col2im", (2, 5, 10, 11, 6, (3, 3), (1, 1), (3, 3), (1, 1))),          # padding beyond the kernel's reach
    ("auto", "col2im", (3, 3, 32, 32, 40, (16, 16), (16, 16), (0, 0), (1, 1))),     # patch embedding: one tap per position
    ("auto", "col2im", (2, 3, 30, 29, 16, (7, 7), (2, 2), (3, 3), (1, 1))),         # stem: 7×7 at stride 2
    ("auto", "col2im", (2, 8, 17, 19, 12, (3, 3), (2, 3), (1, 2), (2, 1))),         # dilation along one axis, stride 2×3
    ("auto", "col2im", (5, 16, 12, 12, 24, (2, 2), (2, 2), (0, 0), (1, 1))),        # 2×2 at stride 2 (down-sampling)
    # many output channels: the per-image products have few tiles and a long k, and their results live in the scratch
    # buffer a k-sliced product would write its partial sums to
    ("auto", "col2im", (2, 3, 32, 32, 2048, (16, 16), (16, 16), (0, 0), (1, 1))),
]


@pytest.mark.parametrize("family,kernel,case", GRAD_INPUT_FAMILY_CASES)
def test_grad_input_kernel_families(hip, oracle, force_family, family, kernel, case):
    """grad_input through every kernel that can produce it, the dispatcher asked which one runs."""
    batch, c_in, h, w, c_out, kernel_hw, stride, padding, dilation = case
    force_family(family)
    assert hip.conv2d_planned_kernel(*case, direction="grad_input") == kernel
    rng = np.random.default_rng(c_in * 100 + c_out)
    oh, ow = oracle.conv2d_output_hw(h, w, kernel_hw, stride, padding, dilation)
    wgt = rng.normal(0, np.sqrt(2.0 / (c_in * kernel_hw[0] * kernel_hw[1])), c_out * c_in * kernel_hw[0] * kernel_hw[1]).astype(np.float32)
    g = rng.normal(size=batch * c_out * oh * ow).astype(np.float32)
    d_g, d_w = hip.DeviceBuffer.from_array(g), hip.DeviceBuffer.from_array(wgt)
    d_gi = hip.DeviceBuffer(batch * c_in * h * w * 4)
    hip.conv2d_grad_input_f32_dev(*case, d_g, d_w, d_gi)
    hip.device_synchronize()
    gi = d_gi.to_array(np.float32, batch * c_in * h * w)
    want_gi, _, _ = oracle.conv2d_backward_f32(*case, np.zeros(batch * c_in * h * w, np.float32), wgt, g)
    assert_grad_input(gi, case, g, wgt, want_gi, f"{family} {case}")


def test_config2_grad_input_elementwise(hip, oracle, force_family):
    """BASELINE config 2's geometry (64 -> 128 channels, 56x56, 3x3, pad 1): grad_input runs the packed-row strip
    kernel on 128 'input' channels.  Two images with that kernel forced, then the full batch of 32 as dispatched,
    images 0 and 31 against the oracle element by element."""
    from spiraltorch_amd import inputs
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    wgt = inputs.normal(102, 128 * 64 * 9, 0.0, float(np.sqrt(2.0 / (64 * 9))))
    per_image = 128 * 56 * 56
    g = inputs.normal(103, 32 * per_image)
    d_w = hip.DeviceBuffer.from_array(wgt)
    zeros = np.zeros(64 * 56 * 56, np.float32)
    want = {i: oracle.conv2d_backward_f32(1, 64, 56, 56, 128, *geom, zeros, wgt, g[i * per_image:(i + 1) * per_image])[0]
            for i in (0, 1, 31)}

    two = (2, 64, 56, 56, 128, *geom)
    force_family("strip")
    assert hip.conv2d_planned_kernel(*two, direction="grad_input") == "strip9"
    d_g2, d_gi2 = hip.DeviceBuffer.from_array(g[:2 * per_image]), hip.DeviceBuffer(2 * zeros.nbytes)
    hip.conv2d_grad_input_f32_dev(*two, d_g2, d_w, d_gi2)
    hip.device_synchronize()
    gi2 = d_gi2.to_array(np.float32, 2 * zeros.size).reshape(2, -1)
    for i in (0, 1):
        case = (1, 64, 56, 56, 128, *geom)
        assert_grad_input(gi2[i], case, g[i * per_image:(i + 1) * per_image], wgt, want[i], f"two images, image {i}")

    force_family("auto")
    full = (32, 64, 56, 56, 128, *geom)
    assert hip.conv2d_planned_kernel(*full, direction="grad_input") == "strip9"
    d_g, d_gi = hip.DeviceBuffer.from_array(g), hip.DeviceBuffer(32 * zeros.nbytes)
    hip.conv2d_grad_input_f32_dev(*full, d_g, d_w, d_gi)
    hip.device_synchronize()
    gi = d_gi.to_array(np.float32, 32 * zeros.size).reshape(32, -1)
    for i in (0, 31):
        case = (1, 64, 56, 56, 128, *geom)
        assert_grad_input(gi[i], case, g[i * per_image:(i + 1) * per_image], wgt, want[i], f"batch of 32, image {i}")
    assert (gi[:2] == gi2).all()   # the same images give the same bits whatever the batch around them


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


def test_config2_grad_weight_sampled_entries_against_float64(hip):
    """BASELINE config 2 at full size through the kernel its shape takes (three runs of steps per workgroup, 251 runs: the
    last workgroup has two busy sets): 96 entries of grad_weight — every tap, the first and last channels of both kinds,
    and random ones — against their definition in float64,
    grad_weight[o, c, ky, kx] = scale · Σ_{n, y, x} grad_output[n, o, y, x] · input[n, c, y + ky − 1, x + kx − 1]."""
    from spiraltorch_amd import inputs
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    x = inputs.normal(201, batch * c_in * h * w)
    g = inputs.normal(202, batch * c_out * h * w)
    d_gw = hip.DeviceBuffer(c_out * c_in * 9 * 4)
    hip.conv2d_grad_weight_f32_dev(batch, c_in, h, w, c_out, *geom, hip.DeviceBuffer.from_array(x), hip.DeviceBuffer.from_array(g),
                                   1.0 / batch, d_gw)
    hip.device_synchronize()
    gw = d_gw.to_array(np.float32, c_out * c_in * 9).reshape(c_out, c_in, 3, 3)
    X = np.zeros((batch, c_in, h + 2, w + 2), np.float64)
    X[:, :, 1:-1, 1:-1] = x.reshape(batch, c_in, h, w)
    G = g.reshape(batch, c_out, h, w).astype(np.float64)
    rng = np.random.default_rng(5)
    entries = [(o, c, ky, kx) for (o, c) in ((0, 0), (127, 63)) for ky in range(3) for kx in range(3)]
    entries += [(int(rng.integers(c_out)), int(rng.integers(c_in)), int(rng.integers(3)), int(rng.integers(3))) for _ in range(78)]
    got = np.array([gw[e] for e in entries], np.float64)
    want = np.array([float((G[:, o] * X[:, c, ky:ky + h, kx:kx + w]).sum()) / batch for (o, c, ky, kx) in entries])
    assert_close(got, want, 1e-4, 1e-4, "config 2 grad_weight, sampled entries")
    assert np.isfinite(gw).all()


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
