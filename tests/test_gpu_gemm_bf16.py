"""Parity of the bf16 GEMM (f32 accumulate) against the CPU oracle: 2e-2 relative."""
import numpy as np
import pytest

from conftest import BF16_REL, assert_close

pytestmark = pytest.mark.gpu


def bf16_pair(rng, m, n, k, std=0.02):
    from spiraltorch_amd import inputs
    a = inputs.to_bf16(rng.normal(0, std, m * k).astype(np.float32))
    b = inputs.to_bf16(rng.normal(0, std, k * n).astype(np.float32))
    return a, b


def check(out, want, what):
    # 2e-2 relative per element, with an absolute floor of 2e-2 x the typical magnitude for sums that
    # cancel to (almost) zero.  In practice the only difference is f32 summation order (~1e-6 relative).
    floor = BF16_REL * float(np.sqrt(np.mean(np.square(want)))) * 1e-2
    assert_close(out, want, BF16_REL, floor, what)
    # and the tighter bound the arithmetic actually supports
    scale = float(np.abs(want).max()) or 1.0
    assert float(np.abs(out - want).max()) <= 1e-4 * scale, what


@pytest.mark.parametrize("m,n,k", [(1, 8, 8), (16, 64, 32), (33, 40, 72), (128, 128, 128), (130, 136, 264),
                                   (16, 256, 512), (7, 24, 1000), (200, 8, 16)])
def test_random_shapes(hip, oracle, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k)
    a, b = bf16_pair(rng, m, n, k, std=1.0)
    out = np.zeros(m * n, np.float32)
    hip.gemm_bf16_f32acc(m, n, k, a, b, out)
    check(out, oracle.gemm_bf16_f32acc(m, n, k, a, b), f"bf16 gemm {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k", [(5, 7, 9), (17, 33, 20), (64, 100, 36)])
def test_unaligned_shapes(hip, oracle, m, n, k):
    rng = np.random.default_rng(m + n + k)
    a, b = bf16_pair(rng, m, n, k, std=1.0)
    out = np.zeros(m * n, np.float32)
    hip.gemm_bf16_f32acc(m, n, k, a, b, out)
    check(out, oracle.gemm_bf16_f32acc(m, n, k, a, b), f"unaligned {m}x{n}x{k}")


def test_exact_small_integers(hip):
    from spiraltorch_amd import inputs
    a = inputs.to_bf16(np.arange(1, 7, dtype=np.float32))
    b = inputs.to_bf16(np.arange(7, 13, dtype=np.float32))
    out = np.zeros(4, np.float32)
    hip.gemm_bf16_f32acc(2, 2, 3, a, b, out)
    assert out.tolist() == [58, 64, 139, 154]


def test_config4_skinny(hip, oracle):
    """BASELINE config 4 (decode-like): M=16, N=K=4096, N(0, 0.02^2) rounded to bf16."""
    from spiraltorch_amd import inputs
    m, n, k = 16, 4096, 4096
    a = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 2), m * k, 0.0, 0.02))
    b = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), k * n, 0.0, 0.02))
    out = np.zeros(m * n, np.float32)
    hip.gemm_bf16_f32acc(m, n, k, a, b, out)
    check(out, oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8), "config 4 skinny")


def test_config4_4096_cubed_sampled_rows_and_properties(hip, oracle):
    """BASELINE config 4: M=N=K=4096.  The oracle checks 24 sampled rows; the rest of the matrix is
    covered by size-independent properties (row permutation equivariance, exact power-of-two linearity)."""
    from spiraltorch_amd import inputs
    n = 4096
    a = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 0), n * n, 0.0, 0.02))
    b = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), n * n, 0.0, 0.02))
    d_a, d_b = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(b)
    d_out = hip.DeviceBuffer(n * n * 4)
    hip.gemm_bf16_f32acc_dev(n, n, n, d_a, d_b, d_out)
    hip.device_synchronize()
    out = d_out.to_array(np.float32, (n, n))
    rows = [0, 1, 31, 32, 255, 256, 257, 1023, 2048, 3000, 4094, 4095] + list(range(1500, 1512))
    want = oracle.gemm_bf16_f32acc(len(rows), n, n, a.reshape(n, n)[rows].ravel(), b, threads=8)
    check(out[rows].ravel(), want, "4096^3 sampled rows")
    # permuting the rows of A permutes the rows of C (every row goes through a different tile position)
    perm = np.random.default_rng(0).permutation(n)
    d_ap = hip.DeviceBuffer.from_array(a.reshape(n, n)[perm])
    hip.gemm_bf16_f32acc_dev(n, n, n, d_ap, d_b, d_out)
    hip.device_synchronize()
    assert (d_out.to_array(np.float32, (n, n)) == out[perm]).all()
    # doubling A (exact in bf16) doubles C exactly
    a2 = inputs.to_bf16(2 * inputs.from_bf16(a))
    d_a2 = hip.DeviceBuffer.from_array(a2)
    hip.gemm_bf16_f32acc_dev(n, n, n, d_a2, d_b, d_out)
    hip.device_synchronize()
    assert (d_out.to_array(np.float32, (n, n)) == 2 * out).all()


@pytest.mark.parametrize("m,n,k", [(1, 128, 256), (16, 384, 320), (33, 256, 512), (64, 128, 1024), (7, 1024, 2048)])
def test_skinny_split_k_path(hip, oracle, m, n, k):
    """Decode-like shapes (M <= 64) take the split-k kernel; partial sums are reduced in a fixed order."""
    rng = np.random.default_rng(m * 7 + n + k)
    a, b = bf16_pair(rng, m, n, k, std=1.0)
    out = np.zeros(m * n, np.float32)
    hip.gemm_bf16_f32acc(m, n, k, a, b, out)
    check(out, oracle.gemm_bf16_f32acc(m, n, k, a, b), f"skinny {m}x{n}x{k}")
    again = np.zeros(m * n, np.float32)
    hip.gemm_bf16_f32acc(m, n, k, a, b, again)
    assert (again == out).all(), "split-k reduction must be reproducible"


@pytest.mark.parametrize("m,n,k", [(96, 160, 64), (24, 256, 512), (256, 512, 128)])
def test_fused_epilogue_and_bf16_output(hip, oracle, m, n, k):
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(21)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d32, d16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b).astype(np.float64)
    for act in (0, 1, 2):
        hip.gemm_bf16_bias_act_dev(m, n, k, act, d["a"], d["b"], d["bias"], d["res"], d32, d16)
        hip.device_synchronize()
        pre = (base.reshape(m, n) + bias).ravel() + res
        if act == 1:
            want = np.maximum(pre, 0)
        elif act == 2:
            want = np.array([oracle.gelu(float(np.float32(x))) for x in pre])
        else:
            want = pre
        got32 = d32.to_array(np.float32, m * n)
        assert_close(got32, want, 1e-4, 1e-5, f"epilogue act={act}")
        got16 = d16.to_array(np.uint16, m * n)
        assert (got16 == inputs.to_bf16(got32)).all(), "bf16 output must be the RNE rounding of the f32 output"


@pytest.mark.parametrize("m,n,k,ragged", [(8192, 1024, 128, 0), (8192, 2048, 64, 0), (16384, 512, 192, 0),
                                          (8192 - 37, 2048, 128, 1), (16384 - 5, 768, 64, 1),
                                          # few tiles: the same kernels serve every shape they can address
                                          (65, 128, 64, 1), (300, 384, 192, 1), (257, 256, 64, 1), (512, 512, 512, 0),
                                          (100, 1152, 320, 1),
                                          # n not a multiple of 128: the row-major B is packed on the way in
                                          (2048, 1003, 128, 0), (777, 1500, 256, 1), (300, 2052, 64, 1)])
def test_large_tile_kernels_with_epilogue(hip, oracle, m, n, k, ragged):
    """Shapes that take the 256x256 and 256x128 tile kernels, with bias + residual + GELU and
    both output types; m may be ragged."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m + n + k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d32, d16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8).astype(np.float64)
    pre = (base.reshape(m, n) + bias).ravel() + res
    for act in (0, 2):
        hip.gemm_bf16_bias_act_dev(m, n, k, act, d["a"], d["b"], d["bias"], d["res"], d32, d16)
        hip.device_synchronize()
        want = pre if act == 0 else 0.5 * pre * (1.0 + np.tanh(0.7978846 * (pre + 0.044715 * pre ** 3)))
        got32 = d32.to_array(np.float32, m * n)
        assert_close(got32, want, 1e-4, 1e-5, f"{m}x{n}x{k} act={act}")
        got16 = d16.to_array(np.uint16, m * n)
        assert (got16 == inputs.to_bf16(got32)).all(), "bf16 output must be the RNE rounding of the f32 output"


PACKED_SHAPES = [
    # m, n, k — the packed 256-row kernels (k % 64 == 0, n % 128 == 0), full and ragged in m, one to many k-tiles
    (256, 256, 64), (512, 512, 512), (300, 384, 192), (8192 - 37, 2048, 128), (16384, 512, 192), (257, 256, 1024),
    (100, 1152, 320), (4096, 128, 4096),
    # n not a multiple of 128 (rows of the packed B past n read as zero, stores at any alignment): 128- and 256-wide
    # tiles, an odd n, k split over workgroups, one long row of tiles
    (300, 1000, 192), (1024, 257, 64), (513, 2051, 128), (4096, 129, 4096), (200, 50257, 64), (130, 3000, 1024),
    # shapes they do not take are unpacked on the device first (general kernel); up to 64 rows the row-major entry point
    # runs the skinny split-k kernel, the prepacked one the 256-row kernels
    (33, 40, 72), (130, 136, 264), (5, 7, 9), (16, 384, 320), (64, 128, 1024), (1, 8, 8),
]


@pytest.mark.parametrize("m,n,k", PACKED_SHAPES)
def test_prepacked_rhs(hip, oracle, m, n, k):
    """B given as its (n, k) transpose (PackedB's layout): packed on the device, checked against the oracle on the
    unpacked operands and, with the epilogue, bit for bit against the k×n entry point."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m * 31 + n * 7 + k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d_packed = hip.DeviceBuffer(k * n * 2)
    hip.pack_rhs_bf16_dev(k, n, d["b"], d_packed)
    hip.device_synchronize()
    assert (d_packed.to_array(np.uint16, k * n).reshape(n, k) == b.reshape(k, n).T).all()
    plain = hip.DeviceBuffer(m * n * 4)
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, None, None, plain, None)
    hip.device_synchronize()
    check(plain.to_array(np.float32, m * n), oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8), f"prepacked {m}x{n}x{k}")
    want32, want16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    got32, got16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    hip.gemm_bf16_bias_act_dev(m, n, k, 2, d["a"], d["b"], d["bias"], d["res"], want32, want16)
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 2, d["a"], d_packed, d["bias"], d["res"], got32, got16)
    hip.device_synchronize()
    if m <= 64 and n % 128 == 0 and k % 64 == 0 and k >= 256:
        # up to 64 rows a row-major B goes to the skinny kernel while a prepacked B stays on the 256-row kernels
        # (unpacking it would cost a pass over B per call): same sums in another order
        assert_close(got32.to_array(np.float32, m * n), want32.to_array(np.float32, m * n), 1e-4, 1e-5, "layouts agree")
    else:
        assert (got32.to_array(np.float32, m * n) == want32.to_array(np.float32, m * n)).all()
        assert (got16.to_array(np.uint16, m * n) == want16.to_array(np.uint16, m * n)).all()


@pytest.mark.parametrize("m,n,k", [(1, 1024, 128), (16, 4096, 4096), (17, 1024, 384), (32, 2048, 1152), (5, 1040, 2176),
                                   (9, 1024, 896), (31, 4096, 1024),
                                   # not taken by that kernel (m > 32, k not a multiple of 128): unpacked first
                                   (64, 1024, 4096), (48, 4096, 512), (5, 1040, 2080)])
def test_skinny_prepacked_single_launch(hip, oracle, m, n, k):
    """Decode-like shapes on a prepacked B (m <= 32, at least 64 strips of 16 columns, k a multiple of 128) take the
    single-launch kernel whose eight wavefronts each stream a k-range and add their tiles in a fixed order."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m * 13 + n * 3 + k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("bias", bias), ("res", res))}
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    out = hip.DeviceBuffer(m * n * 4)
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, None, None, out, None)
    hip.device_synchronize()
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8)
    first = out.to_array(np.float32, m * n)
    check(first, base, f"skinny prepacked {m}x{n}x{k}")
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, None, None, out, None)
    hip.device_synchronize()
    assert (out.to_array(np.float32, m * n) == first).all(), "the k-range sums must be added in a fixed order"
    d16 = hip.DeviceBuffer(m * n * 2)
    pre = (base.astype(np.float64).reshape(m, n) + bias).ravel() + res
    for act in (0, 1, 2):
        hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, act, d["a"], d_packed, d["bias"], d["res"], out, d16)
        hip.device_synchronize()
        want = pre if act == 0 else np.maximum(pre, 0) if act == 1 else \
            0.5 * pre * (1.0 + np.tanh(0.7978846 * (pre + 0.044715 * pre ** 3)))
        got32 = out.to_array(np.float32, m * n)
        assert_close(got32, want, 1e-4, 2e-5 * max(1.0, float(np.abs(base).max())), f"skinny prepacked epilogue act={act}")
        assert (d16.to_array(np.uint16, m * n) == inputs.to_bf16(got32)).all()


@pytest.mark.parametrize("m,n,k", [(65, 512, 64), (1000, 512, 512), (16384, 512, 192), (130, 512, 2048), (1, 512, 128), (65, 512, 1024), (300, 512, 1024),
                                   (64, 512, 512), (256, 512, 1024),
                                   # other widths: the GEMM and the layer-norm kernel one after the other
                                   (300, 384, 128), (33, 512, 96), (70, 1024, 256)])
def test_gemm_residual_layer_norm(hip, oracle, m, n, k):
    """Linear + residual + LayerNorm in one call: the rows before normalisation against the oracle's GEMM (+ bias +
    residual), the normalised bf16 rows against the oracle's layer-norm of those rows (within one bf16 step: the
    row statistics are summed in another order), and against the separate GEMM and layer-norm kernels (the same
    arithmetic in the same order: equal bits)."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m + 3 * n + 5 * k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    gamma = rng.normal(1.0, 0.2, size=n).astype(np.float32)
    beta = rng.normal(0.0, 0.2, size=n).astype(np.float32)
    eps = 1e-5
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("bias", bias), ("res", res), ("g", gamma), ("b", beta))}
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    x32, ln16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    hip.gemm_bf16_prepacked_residual_layer_norm_dev(m, n, k, d["a"], d_packed, d["bias"], d["res"], d["g"], d["b"], eps, x32, ln16)
    hip.device_synchronize()
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8)
    want_x = ((base.reshape(m, n) + bias).astype(np.float32).ravel() + res).astype(np.float32)
    got_x = x32.to_array(np.float32, m * n)
    assert_close(got_x, want_x, 1e-4, 1e-4, f"rows before normalisation {m}x{n}x{k}")
    # the normalisation is checked on the rows the GPU produced, so that only the layer-norm itself is compared
    want_ln = oracle.layer_norm_f32(m, n, got_x, gamma, beta, eps)
    got_ln = inputs.from_bf16(ln16.to_array(np.uint16, m * n))
    step = np.maximum(np.abs(want_ln), 2.0 ** -120) * 2.0 ** -7  # one bf16 step is at most 2^-7 relative
    assert (np.abs(got_ln - want_ln) <= step + 1e-6).all(), "normalised rows differ from the oracle by more than one bf16 step"
    # separate kernels on the same operands
    y32, y16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, d["bias"], d["res"], y32, None)
    hip.layer_norm_f32_dev(m, n, y32, None, d["g"], d["b"], eps, None, y16)
    hip.device_synchronize()
    assert (y32.to_array(np.float32, m * n) == got_x).all(), "both kernels add the k products in the same order"
    sep = y16.to_array(np.uint16, m * n)
    assert (sep == ln16.to_array(np.uint16, m * n)).all(), "fused and separate normalisation add a row in the same order"
    # without bias and residual
    hip.gemm_bf16_prepacked_residual_layer_norm_dev(m, n, k, d["a"], d_packed, None, None, d["g"], d["b"], eps, x32, ln16)
    hip.device_synchronize()
    plain = x32.to_array(np.float32, m * n)
    assert_close(plain, base, 1e-4, 1e-4, "no bias, no residual")
    want_ln = oracle.layer_norm_f32(m, n, plain, gamma, beta, eps)
    got_ln = inputs.from_bf16(ln16.to_array(np.uint16, m * n))
    step = np.maximum(np.abs(want_ln), 2.0 ** -120) * 2.0 ** -7
    assert (np.abs(got_ln - want_ln) <= step + 1e-6).all()


@pytest.mark.parametrize("m,n,k", [(100, 4096, 4096), (256, 1024, 4096), (130, 2048, 2048), (65, 128, 8192), (4096, 128, 4096),
                                   (300, 384, 1984),
                                   # shapes of the general 128x128 kernel (n not a multiple of 128), k-sliced the same way
                                   (64, 64, 20000), (4096, 16, 4096), (4096, 1, 4100), (300, 72, 3000), (130, 136, 1064),
                                   # at most 8 columns: a stream over A, one wavefront or workgroup per row
                                   (4096, 8, 4096), (4096, 1, 4096), (300, 5, 4096), (1000, 7, 520), (64, 3, 64), (5000, 2, 264)])
def test_few_tiles_with_a_long_k_split_k(hip, oracle, m, n, k):
    """Launches of few tiles with many k-tiles split k over workgroups (raw partial sums, added in split order by
    a second kernel that applies the epilogue): both layouts of B, the fused epilogue with both output types, and the
    same bits from call to call and from either layout."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m + 7 * n + 3 * k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    out = hip.DeviceBuffer(m * n * 4)
    hip.gemm_bf16_f32acc_dev(m, n, k, d["a"], d["b"], out)
    hip.device_synchronize()
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8)
    plain = out.to_array(np.float32, m * n)
    check(plain, base, f"row-major {m}x{n}x{k}")
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, None, None, out, None)
    hip.device_synchronize()
    assert (out.to_array(np.float32, m * n) == plain).all(), "both layouts split k the same way"
    hip.gemm_bf16_f32acc_dev(m, n, k, d["a"], d["b"], out)
    hip.device_synchronize()
    assert (out.to_array(np.float32, m * n) == plain).all(), "the splits are added in a fixed order"
    d16 = hip.DeviceBuffer(m * n * 2)
    pre = (base.astype(np.float64).reshape(m, n) + bias).ravel() + res
    want = 0.5 * pre * (1.0 + np.tanh(0.7978846 * (pre + 0.044715 * pre ** 3)))
    for packed in (False, True):
        if packed:
            hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 2, d["a"], d_packed, d["bias"], d["res"], out, d16)
        else:
            hip.gemm_bf16_bias_act_dev(m, n, k, 2, d["a"], d["b"], d["bias"], d["res"], out, d16)
        hip.device_synchronize()
        got32 = out.to_array(np.float32, m * n)
        assert_close(got32, want, 1e-4, 2e-5 * max(1.0, float(np.abs(base).max())), f"split-k epilogue packed={packed}")
        assert (d16.to_array(np.uint16, m * n) == inputs.to_bf16(got32)).all()


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1000), (2048, 512, 1001), (4096, 1000, 300), (1000, 1024, 1100), (4096, 512, 784)])
def test_k_that_is_not_a_multiple_of_64(hip, oracle, m, n, k):
    """Large products whose k the direct-to-LDS kernels do not take run on zero-padded copies of both operands (kept in
    a scratch buffer of their own while the product's kernels use the other): both layouts of B, odd row lengths, a
    ragged n, the fused epilogue with both output types, and twice in a row with another product in between (which
    re-uses and may grow the scratch buffers)."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m + 7 * n + 3 * k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    out, other = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 4)
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8)
    hip.gemm_bf16_f32acc_dev(m, n, k, d["a"], d["b"], out)
    hip.device_synchronize()
    plain = out.to_array(np.float32, m * n)
    check(plain, base, f"row-major {m}x{n}x{k}")
    hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d["a"], d_packed, None, None, other, None)
    hip.gemm_bf16_f32acc_dev(m, n, k, d["a"], d["b"], out)
    hip.device_synchronize()
    check(other.to_array(np.float32, m * n), base, f"prepacked {m}x{n}x{k}")
    assert (out.to_array(np.float32, m * n) == plain).all(), "same bits from call to call"
    d16 = hip.DeviceBuffer(m * n * 2)
    pre = (base.astype(np.float64).reshape(m, n) + bias).ravel() + res
    want = np.maximum(pre, 0.0)
    for packed in (False, True):
        if packed:
            hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 1, d["a"], d_packed, d["bias"], d["res"], out, d16)
        else:
            hip.gemm_bf16_bias_act_dev(m, n, k, 1, d["a"], d["b"], d["bias"], d["res"], out, d16)
        hip.device_synchronize()
        got32 = out.to_array(np.float32, m * n)
        assert_close(got32, want, 1e-4, 2e-5 * max(1.0, float(np.abs(base).max())), f"epilogue packed={packed}")
        assert (d16.to_array(np.uint16, m * n) == inputs.to_bf16(got32)).all()


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (300, 1024, 512), (130, 2048, 256), (1000, 1280, 192), (2048, 2048, 64),
                                   (513, 384, 448)])
def test_mid_size_128_row_tiles(hip, oracle, m, n, k):
    """A launch whose 256-row tiling leaves most compute units idle runs 128×128 tiles, two workgroups per compute
    unit, for either layout of B: plain product against the oracle (ragged last row tiles included), every activation
    with bias and residual into both output types, bf16-only output, and the same bits from both layouts."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(5 * m + 3 * n + k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    res = rng.normal(size=m * n).astype(np.float32)
    d = {name: hip.DeviceBuffer.from_array(v) for name, v in (("a", a), ("b", b), ("bias", bias), ("res", res))}
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    out = hip.DeviceBuffer(m * n * 4)
    d16 = hip.DeviceBuffer(m * n * 2)
    base = oracle.gemm_bf16_f32acc(m, n, k, a, b, threads=8)
    pre = (base.astype(np.float64).reshape(m, n) + bias).ravel() + res
    bits = {}
    for packed in (True, False):
        def run(activation, bias_, res_, out32, out16):
            if packed:
                hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, d["a"], d_packed, bias_, res_, out32, out16)
            else:
                hip.gemm_bf16_bias_act_dev(m, n, k, activation, d["a"], d["b"], bias_, res_, out32, out16)
            hip.device_synchronize()
        run(0, None, None, out, None)
        bits[packed] = out.to_array(np.float32, m * n)
        check(bits[packed], base, f"128-row tiles {m}x{n}x{k} packed={packed}")
        for activation, want in ((0, pre), (1, np.maximum(pre, 0.0)),
                                 (2, 0.5 * pre * (1.0 + np.tanh(0.7978846 * (pre + 0.044715 * pre ** 3))))):
            run(activation, d["bias"], d["res"], out, d16)
            got32 = out.to_array(np.float32, m * n)
            assert_close(got32, want, 1e-4, 2e-5 * max(1.0, float(np.abs(base).max())), f"activation {activation}")
            assert (d16.to_array(np.uint16, m * n) == inputs.to_bf16(got32)).all()
        run(1, d["bias"], None, None, d16)
        want16 = np.maximum((base.astype(np.float64).reshape(m, n) + bias).ravel(), 0.0)
        got16 = inputs.from_bf16(d16.to_array(np.uint16, m * n))
        assert_close(got16, want16, 2 ** -7, 2e-5 * max(1.0, float(np.abs(base).max())), "bf16-only output")
    assert (bits[True] == bits[False]).all(), "both layouts accumulate in the same order"


@pytest.mark.parametrize("m,n,k,activation", [(16384, 1536, 512, 0), (16384, 2048, 512, 2), (8192, 4352, 64, 1), (2304, 3968, 128, 2),
                                              (4096, 2176, 320, 0), (512, 66048, 192, 1)])
def test_prepacked_bf16_output_over_several_rounds_of_tiles(hip, oracle, m, n, k, activation):
    """More 256×128 tiles than compute units, bf16 the only output, M a multiple of 256: the persistent kernel (a ninth
    wavefront loads, eight compute and store).  Bit for bit the bf16 rounding of what the same call returns when it
    also asks for the f32 output (which takes the one-tile-per-workgroup kernel), and sampled rows against the oracle."""
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    d_a, d_bias = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(bias)
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    d32, d16, d16_ref = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2), hip.DeviceBuffer(m * n * 2)
    for use_bias in (True, False):
        hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, d_a, d_packed, d_bias if use_bias else None, None, d32, d16_ref)
        hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, d_a, d_packed, d_bias if use_bias else None, None, None, d16)
        hip.device_synchronize()
        got = d16.to_array(np.uint16, m * n)
        assert (got == d16_ref.to_array(np.uint16, m * n)).all(), f"bias={use_bias}"
    rows = sorted(set([0, 1, 255, 256, m // 2 + 3, m - 257, m - 1]))
    base = oracle.gemm_bf16_f32acc(len(rows), n, k, a.reshape(m, k)[rows].ravel(), b, threads=8).astype(np.float64).reshape(len(rows), n)
    want = base  # the last call ran without a bias
    if activation == 1:
        want = np.maximum(want, 0.0)
    elif activation == 2:
        want = 0.5 * want * (1.0 + np.tanh(0.7978846 * (want + 0.044715 * want ** 3)))
    got_rows = inputs.from_bf16(got.reshape(m, n)[rows].ravel())
    assert_close(got_rows, want.ravel(), 2 ** -7, 2e-5 * max(1.0, float(np.abs(base).max())), "sampled rows")


def test_config4_4096_cubed_prepacked(hip, oracle):
    """BASELINE config 4 with B prepacked: 24 sampled rows against the oracle, the rest of the matrix bit for bit
    against the k×n kernel (checked itself above), and exact power-of-two linearity."""
    from spiraltorch_amd import inputs
    n = 4096
    a = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 0), n * n, 0.0, 0.02))
    b = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), n * n, 0.0, 0.02))
    d_a, d_b = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(b)
    d_packed, d_out, d_ref = hip.DeviceBuffer(n * n * 2), hip.DeviceBuffer(n * n * 4), hip.DeviceBuffer(n * n * 4)
    hip.pack_rhs_bf16_dev(n, n, d_b, d_packed)
    hip.gemm_bf16_prepacked_bias_act_dev(n, n, n, 0, d_a, d_packed, None, None, d_out, None)
    hip.gemm_bf16_f32acc_dev(n, n, n, d_a, d_b, d_ref)
    hip.device_synchronize()
    out = d_out.to_array(np.float32, (n, n))
    rows = [0, 1, 31, 32, 255, 256, 257, 1023, 2048, 3000, 4094, 4095] + list(range(1500, 1512))
    want = oracle.gemm_bf16_f32acc(len(rows), n, n, a.reshape(n, n)[rows].ravel(), b, threads=8)
    check(out[rows].ravel(), want, "4096^3 prepacked, sampled rows")
    assert (out == d_ref.to_array(np.float32, (n, n))).all()
    d_a2 = hip.DeviceBuffer.from_array(inputs.to_bf16(2 * inputs.from_bf16(a)))
    hip.gemm_bf16_prepacked_bias_act_dev(n, n, n, 0, d_a2, d_packed, None, None, d_ref, None)
    hip.device_synchronize()
    assert (d_ref.to_array(np.float32, (n, n)) == 2 * out).all()


def test_lhs_of_more_than_2_gib(hip):
    """An A beyond 2^31 bytes is cut into row blocks the 32-bit-offset kernels can address; rows on both sides of the
    cut and at both ends are checked against float64, for both outputs."""
    from spiraltorch_amd import inputs
    m, n, k = 1050000, 128, 1024
    rng = np.random.default_rng(4)
    a = inputs.to_bf16(rng.random(m * k, dtype=np.float32) - 0.5)
    b = inputs.to_bf16(rng.random(k * n, dtype=np.float32) - 0.5)
    bias = rng.random(n, dtype=np.float32)
    d_a, d_b, d_bias = (hip.DeviceBuffer.from_array(v) for v in (a, b, bias))
    d32, d16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    hip.gemm_bf16_bias_act_dev(m, n, k, 0, d_a, d_b, d_bias, None, d32, d16)
    hip.device_synchronize()
    got = d32.to_array(np.float32, m * n).reshape(m, n)
    cut = ((1 << 31) // (k * 2) - 1) // 256 * 256
    rows = np.r_[0:3, cut - 3:cut + 3, m - 3:m, rng.integers(0, m, 40)]
    want = inputs.from_bf16(a.reshape(m, k)[rows]).astype(np.float64) @ inputs.from_bf16(b).reshape(k, n).astype(np.float64) + bias
    assert_close(got[rows], want, 1e-4, 2e-5, "rows of a 2.15 GB lhs")
    got16 = d16.to_array(np.uint16, m * n).reshape(m, n)
    assert (got16[rows] == inputs.to_bf16(got[rows].ravel()).reshape(len(rows), n)).all()
    assert np.isfinite(got).all()


def test_validation(hip):
    out = np.full(4, 13.0, np.float32)
    with pytest.raises(hip.HipErr, match="lhs buffer length 4 does not match m\\*k=6"):
        hip.gemm_bf16_f32acc(2, 2, 3, np.zeros(4, np.uint16), np.zeros(6, np.uint16), out)
    assert (out == 13.0).all()


@pytest.mark.parametrize("m,n,k,activation", [(16384, 4096, 512, 0), (2048, 16384, 128, 2), (4096, 8192, 320, 1)])
def test_prepacked_f32_output_over_many_rounds_of_tiles_with_a_short_k(hip, oracle, m, n, k, activation):
    """At least 1024 tiles of 256×128, k up to 512, f32 the only output: the persistent kernel with its f32 epilogue.
    Bit for bit what the same call returns when it also asks for the bf16 output (which takes the one-tile-per-workgroup
    kernel: same products added in the same order), with and without a bias; sampled rows against the oracle."""
    rng = np.random.default_rng(2 * m + 3 * n + 5 * k)
    a, b = bf16_pair(rng, m, n, k, std=0.5)
    bias = rng.normal(size=n).astype(np.float32)
    d_a, d_bias = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(bias)
    d_packed = hip.DeviceBuffer.from_array(np.ascontiguousarray(b.reshape(k, n).T))
    d32, d32_ref, d16 = hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 4), hip.DeviceBuffer(m * n * 2)
    for use_bias in (True, False):
        d32.zero()
        hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, d_a, d_packed, d_bias if use_bias else None, None, d32_ref, d16)
        hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, activation, d_a, d_packed, d_bias if use_bias else None, None, d32, None)
        hip.device_synchronize()
        got = d32.to_array(np.float32, m * n)
        assert (got.view(np.uint32) == d32_ref.to_array(np.float32, m * n).view(np.uint32)).all(), f"bias={use_bias}"
    rows = sorted(set([0, 1, 255, 256, m // 2 + 3, m - 257, m - 1]))
    base = oracle.gemm_bf16_f32acc(len(rows), n, k, a.reshape(m, k)[rows].ravel(), b, threads=8).astype(np.float64).reshape(len(rows), n)
    want = base  # the last call ran without a bias
    if activation == 1:
        want = np.maximum(want, 0.0)
    elif activation == 2:
        want = 0.5 * want * (1.0 + np.tanh(0.7978846 * (want + 0.044715 * want ** 3)))
    assert_close(got.reshape(m, n)[rows].ravel(), want.ravel(), BF16_REL, 2e-5 * max(1.0, float(np.abs(base).max())), "sampled rows")


def test_layer_norm_routes_round_alike_next_to_a_bf16_boundary(hip):
    """A row a randomised sweep found (tests/golden/layer_norm_row_near_bf16_boundary.npz: 512 values, gamma, beta): with
    E[x²] − mean² and normalised·γ + β in separately rounded steps — the reference's arithmetic — element 481 lands exactly on
    a bf16 rounding boundary (0xbd6e8000 → 0xbd6e); a fused multiply-add in either place moves it by 2 or 7 ulps, and when
    the stand-alone kernel fused both and the GEMM kernel that normalises its own rows only the second, the two routes
    came out one bf16 step apart.  Both routes against an f32 emulation of the arithmetic, operation by operation."""
    import os
    from spiraltorch_amd import inputs
    row = np.load(os.path.join(os.path.dirname(__file__), "golden", "layer_norm_row_near_bf16_boundary.npz"))
    x, gamma, beta = row["x"], row["gamma"], row["beta"]
    n, eps = 512, np.float32(1e-5)
    f32 = np.float32

    def fma(a, b, c):  # the product of two f32 is exact in f64
        return f32(np.float64(a) * np.float64(b) + np.float64(c))

    lane_sum, lane_sq = [], []
    for lane in range(64):  # lane L of the row's wavefront holds columns 4L.. and 256 + 4L..
        s, q = f32(0), f32(0)
        for i in range(2):
            v = x[(lane + 64 * i) * 4:(lane + 64 * i) * 4 + 4]
            s = f32(s + f32(f32(v[0] + v[1]) + f32(v[2] + v[3])))
            q = f32(q + f32(fma(v[0], v[0], f32(v[1] * v[1])) + fma(v[2], v[2], f32(v[3] * v[3]))))
        lane_sum.append(s)
        lane_sq.append(q)
    for offset in (32, 16, 8, 4, 2, 1):  # the exchanges over 32, 16, ... 1 lanes
        lane_sum = [f32(lane_sum[i] + lane_sum[i ^ offset]) for i in range(64)]
        lane_sq = [f32(lane_sq[i] + lane_sq[i ^ offset]) for i in range(64)]
    mean = f32(lane_sum[0] / f32(n))
    var = max(f32(f32(lane_sq[0] / f32(n)) - f32(mean * mean)), f32(0))
    denom = f32(np.sqrt(np.float64(f32(var + eps))))
    inv = f32(f32(1) / denom)
    want = np.zeros(n, np.float32)
    for c in range(n):
        a = f32(x[c] - mean)
        t = f32(a * inv)
        quotient = fma(fma(-t, denom, a), inv, t)  # the correctly rounded a / denom
        want[c] = f32(f32(quotient * gamma[c]) + beta[c])
    assert want[481:482].view(np.uint32)[0] == 0xbd6e8000

    rows = 130  # more than 64: the fused call takes the kernel that normalises its own rows
    d_x = hip.DeviceBuffer.from_array(np.tile(x, rows))
    d_g, d_b = hip.DeviceBuffer.from_array(gamma), hip.DeviceBuffer.from_array(beta)
    d_f32, d_16 = hip.DeviceBuffer(rows * n * 4), hip.DeviceBuffer(rows * n * 2)
    hip.layer_norm_f32_dev(rows, n, d_x, None, d_g, d_b, float(eps), d_f32, d_16)
    hip.device_synchronize()
    got = d_f32.to_array(np.float32, rows * n).reshape(rows, n)
    assert (got == want[None, :]).all(), "stand-alone layer norm, f32"
    assert (d_16.to_array(np.uint16, rows * n).reshape(rows, n) == inputs.to_bf16(want)[None, :]).all(), "stand-alone layer norm, bf16"
    # the GEMM route: a zero product, so that the rows before normalisation are the residual rows exactly
    k = 64
    d_a = hip.DeviceBuffer.from_array(np.zeros(rows * k, np.uint16))
    d_w = hip.DeviceBuffer.from_array(inputs.to_bf16(np.random.default_rng(0).normal(size=n * k).astype(np.float32)))
    x32, ln16 = hip.DeviceBuffer(rows * n * 4), hip.DeviceBuffer(rows * n * 2)
    hip.gemm_bf16_prepacked_residual_layer_norm_dev(rows, n, k, d_a, d_w, None, d_x, d_g, d_b, float(eps), x32, ln16)
    hip.device_synchronize()
    assert (x32.to_array(np.float32, rows * n).reshape(rows, n) == x[None, :]).all()
    assert (ln16.to_array(np.uint16, rows * n).reshape(rows, n) == inputs.to_bf16(want)[None, :]).all(), "GEMM + residual + layer norm"
