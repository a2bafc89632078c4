"""Device operands that start 4 bytes (f32) or 2 bytes (bf16) past a 16-byte boundary — a view into a larger
allocation.  Every `_dev` entry point must either give the values it gives on aligned operands (the 128-bit kernels
fall back to narrower ones, whose sums may associate differently: the parity tolerance applies, not bit equality) or
refuse with an error; it must never write outside its output.  The aligned results are the ones the other test files
hold to the oracle."""
import numpy as np
import pytest

from spiraltorch_amd import inputs

pytestmark = pytest.mark.gpu

GUARD = 32


class Operand:
    """An array placed `shift` elements into a zeroed device allocation with GUARD spare bytes."""

    def __init__(self, hip, array=None, nbytes=None, itemsize=4, shift=0):
        self.nbytes = array.nbytes if array is not None else nbytes
        self.offset = shift * (array.itemsize if array is not None else itemsize)
        self.buf = hip.DeviceBuffer(self.nbytes + GUARD)
        self.buf.zero()
        if array is not None:
            self.buf.upload(np.ascontiguousarray(array), self.offset)
        self.address = self.buf.at(self.offset)

    def read(self, dtype):
        raw = self.buf.to_array(np.uint8, self.nbytes + GUARD)
        outside = np.concatenate([raw[:self.offset], raw[self.offset + self.nbytes:]])
        assert (outside == 0).all(), "bytes outside the output were written"
        return raw[self.offset:self.offset + self.nbytes].view(dtype).copy()


def run_shifted(hip, call, arrays, outputs, shifts_in, shifts_out):
    """outputs: (element count, dtype) or None per output.  Returns the outputs as float64 arrays (bf16 decoded)."""
    d_in = [None if a is None else Operand(hip, array=a, shift=s) for a, s in zip(arrays, shifts_in)]
    d_out = [None if o is None else Operand(hip, nbytes=o[0] * np.dtype(o[1]).itemsize, itemsize=np.dtype(o[1]).itemsize, shift=s)
             for o, s in zip(outputs, shifts_out)]
    call(*[None if d is None else d.address for d in d_in], *[None if d is None else d.address for d in d_out])
    hip.device_synchronize()
    results = []
    for d, o in zip(d_out, outputs):
        if d is None:
            results.append(None)
            continue
        got = d.read(o[1])
        results.append((inputs.from_bf16(got) if o[1] == np.uint16 else got).astype(np.float64))
    return results


def check(hip, call, arrays, outputs, rel, floor, what, patterns=None):
    base = run_shifted(hip, call, arrays, outputs, [0] * len(arrays), [0] * len(outputs))
    n_in, n_out = len(arrays), len(outputs)
    patterns = patterns or [([1] * n_in, [0] * n_out), ([0] * n_in, [1] * n_out), ([1] * n_in, [1] * n_out),
                            ([i % 2 for i in range(n_in)], [(i + 1) % 2 for i in range(n_out)])]
    for shifts_in, shifts_out in patterns:
        got = run_shifted(hip, call, arrays, outputs, shifts_in, shifts_out)
        for g, b, o in zip(got, base, outputs):
            if g is None:
                continue
            tolerance = floor + (max(rel, 2.0 ** -7) if o[1] == np.uint16 and rel > 0 else rel) * np.abs(b)
            assert np.isfinite(g).all(), f"{what}: non-finite values with shifts {shifts_in} {shifts_out}"
            assert (np.abs(g - b) <= tolerance).all(), f"{what}: shifts {shifts_in} {shifts_out}: largest difference {np.abs(g - b).max():.3e}"


def f32(rng, count, sd=1.0):
    return rng.normal(0, sd, count).astype(np.float32)


def b16(rng, count, sd=1.0):
    return inputs.to_bf16(rng.normal(0, sd, count).astype(np.float32))


@pytest.mark.parametrize("m,n,k,lhs_transposed", [(256, 256, 256, False), (500, 200, 100, True), (16, 512, 2048, False), (1024, 4, 64, True)])
def test_gemm_f32(hip, m, n, k, lhs_transposed):
    rng = np.random.default_rng(m + n + k)
    floor = 1e-5 * np.sqrt(k)
    check(hip, lambda a, b, o: hip.gemm_f32_dev(m, n, k, 0.5, lhs_transposed, a, b, o), [f32(rng, m * k), f32(rng, k * n)],
          [(m * n, np.float32)], 1e-4, floor, "gemm_f32")
    check(hip, lambda a, b, bias, res, o: hip.gemm_bias_act_f32_dev(m, n, k, 2, a, b, bias, res, o),
          [f32(rng, m * k), f32(rng, k * n), f32(rng, n), f32(rng, m * n)], [(m * n, np.float32)], 1e-4, floor, "gemm_bias_act_f32")
    check(hip, lambda a, b, bias, res, o: hip.gemm_prepacked_bias_act_f32_dev(m, n, k, 1, a, b, bias, res, o),
          [f32(rng, m * k), f32(rng, n * k), f32(rng, n), f32(rng, m * n)], [(m * n, np.float32)], 1e-4, floor, "gemm_prepacked_f32")


@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (16, 1024, 1024), (500, 1040, 64), (63, 128, 128)])
def test_gemm_bf16(hip, m, n, k):
    rng = np.random.default_rng(m + n + k)
    for name, fn in (("row-major", hip.gemm_bf16_bias_act_dev), ("prepacked", hip.gemm_bf16_prepacked_bias_act_dev)):
        check(hip, lambda a, b, bias, res, o32, o16: fn(m, n, k, 2, a, b, bias, res, o32, o16),
              [b16(rng, m * k, 0.5), b16(rng, k * n, 0.5), f32(rng, n), f32(rng, m * n)], [(m * n, np.float32), (m * n, np.uint16)],
              1e-4, 1e-5 * np.sqrt(k), f"bf16 gemm, {name}")
    if n in (256, 1024):
        check(hip, lambda a, b, bias, res, g, be, o32, o16: hip.gemm_bf16_prepacked_residual_layer_norm_dev(m, n, k, a, b, bias, res, g, be, 1e-5, o32, o16),
              [b16(rng, m * k, 0.5), b16(rng, n * k, 0.5), f32(rng, n), f32(rng, m * n), f32(rng, n), f32(rng, n)],
              [(m * n, np.float32), (m * n, np.uint16)], 1e-4, 1e-4, "bf16 gemm + residual + layer norm")


@pytest.mark.parametrize("geometry", [(2, 16, 20, 20, 64, (3, 3), (1, 1), (1, 1), (1, 1)), (1, 3, 14, 28, 8, (5, 5), (2, 2), (2, 2), (1, 1)),
                                      (3, 64, 8, 8, 128, (1, 1), (1, 1), (0, 0), (1, 1))])
def test_conv2d_forward_and_gradients(hip, geometry):
    batch, c_in, h, w, c_out, kernel, stride, padding, dilation = geometry
    oh, ow = hip.conv2d_output_hw(h, w, kernel, stride, padding, dilation)
    n_in, n_w, n_out = batch * c_in * h * w, c_out * c_in * kernel[0] * kernel[1], batch * c_out * oh * ow
    rng = np.random.default_rng(n_in + n_out)
    check(hip, lambda x, wt, b, o: hip.conv2d_bias_act_f32_dev(*geometry, 1, x, wt, b, o), [f32(rng, n_in), f32(rng, n_w, 0.1), f32(rng, c_out)],
          [(n_out, np.float32)], 1e-4, 1e-5 * np.sqrt(c_in * kernel[0] * kernel[1]), "conv2d f32")
    check(hip, lambda g, wt, o: hip.conv2d_grad_input_f32_dev(*geometry, g, wt, o), [f32(rng, n_out), f32(rng, n_w, 0.1)],
          [(n_in, np.float32)], 1e-4, 1e-5 * np.sqrt(c_out * kernel[0] * kernel[1]), "conv2d grad_input")
    check(hip, lambda x, g, o: hip.conv2d_grad_weight_f32_dev(*geometry, x, g, 0.5, o), [f32(rng, n_in), f32(rng, n_out)],
          [(n_w, np.float32)], 1e-4, 1e-5 * np.sqrt(batch * oh * ow), "conv2d grad_weight")
    check(hip, lambda g, o: hip.conv2d_grad_bias_f32_dev(*geometry, g, 0.5, o), [f32(rng, n_out)],
          [(c_out, np.float32)], 1e-4, 1e-5 * np.sqrt(batch * oh * ow), "conv2d grad_bias")
    # bf16 operands may start at any 2-byte boundary; the outputs must be aligned (refused otherwise, see test_gpu_conv_bf16)
    check(hip, lambda x, wt, b, o32, o16: hip.conv2d_bias_act_bf16_dev(*geometry, 1, x, wt, b, o32, o16),
          [b16(rng, n_in), b16(rng, n_w, 0.1), f32(rng, c_out)], [(n_out, np.float32), (n_out, np.uint16)], 1e-4,
          1e-5 * np.sqrt(c_in * kernel[0] * kernel[1]), "conv2d bf16", patterns=[([1, 1, 1], [0, 0]), ([1, 0, 1], [0, 0]), ([0, 1, 0], [0, 0])])


@pytest.mark.parametrize("contexts,sequence,head_dim,causal", [(2, 256, 64, True), (3, 100, 20, False), (1, 512, 128, False), (4, 7, 8, True)])
def test_attention_f32(hip, contexts, sequence, head_dim, causal):
    rng = np.random.default_rng(contexts + sequence + head_dim)
    count = contexts * sequence * head_dim
    for z_bias, attn_bias in ((False, False), (True, True)):
        check(hip, lambda q, k, v, z, a, o: hip.attention_f32_dev(contexts, sequence, head_dim, head_dim ** -0.5, causal, q, k, v, z, a, o),
              [f32(rng, count), f32(rng, count), f32(rng, count), f32(rng, contexts * sequence) if z_bias else None,
               f32(rng, contexts * sequence * sequence) if attn_bias else None], [(count, np.float32)], 1e-4, 1e-5, "attention f32")


def test_attention_bf16_refuses_misaligned_operands(hip):
    rng = np.random.default_rng(5)
    count = 2 * 128 * 64
    q, k, v = (Operand(hip, array=b16(rng, count), shift=1) for _ in range(3))
    out = Operand(hip, nbytes=count * 2, itemsize=2)
    with pytest.raises(hip.HipErr, match="aligned"):
        hip.attention_bf16_dev(2, 1, 128, 64, 0.125, True, q.address, k.address, v.address, 64, out.address, 64)
    assert (out.read(np.uint16) == 0).all()


@pytest.mark.parametrize("rows,cols", [(3, 512), (4000, 2048), (100, 2052), (3, 50257), (64, 100), (9000, 256)])
def test_row_operators(hip, rows, cols):
    rng = np.random.default_rng(rows + cols)
    count = rows * cols
    check(hip, lambda x, r, g, b, o32, o16: hip.layer_norm_f32_dev(rows, cols, x, r, g, b, 1e-5, o32, o16),
          [f32(rng, count), f32(rng, count), f32(rng, cols), f32(rng, cols)], [(count, np.float32), (count, np.uint16)], 1e-4, 2e-5, "layer norm")
    check(hip, lambda x, o: hip.row_softmax_f32_dev(rows, cols, x, o), [f32(rng, count, 3.0)], [(count, np.float32)], 1e-4, 1e-7, "row softmax")
    check(hip, lambda x, o: hip.sum_axis0_f32_dev(rows, cols, x, 0.25, o), [f32(rng, count)], [(cols, np.float32)], 1e-4, 1e-5 * np.sqrt(rows), "column sums")
    check(hip, lambda x, o: hip.gelu_f32_dev(count, x, o), [f32(rng, count)], [(count, np.float32)], 1e-4, 1e-6, "gelu")
    check(hip, lambda x, o: hip.f32_to_bf16_dev(count, x, o), [f32(rng, count)], [(count, np.uint16)], 0.0, 0.0, "f32 -> bf16")


def test_gathers_and_head_layouts(hip):
    rng = np.random.default_rng(11)
    for tokens, vocab, dim in ((509, 256, 512), (33, 7, 2052), (5, 3, 3)):
        ids = rng.uniform(-1, vocab + 1, tokens).astype(np.float32)
        check(hip, lambda i, t, o: hip.embedding_f32_dev(tokens, vocab, dim, i, t, o), [ids, f32(rng, vocab * dim)],
              [(tokens * dim, np.float32)], 0.0, 0.0, "embedding")
    for batch, seq, heads, dim in ((2, 64, 4, 24), (1, 5, 2, 64)):
        count = batch * seq * heads * dim
        check(hip, lambda x, q, k, v: hip.split_heads_f32_dev(batch, seq, heads, dim, x, q, k, v), [f32(rng, 3 * count)],
              [(count, np.float32)] * 3, 0.0, 0.0, "split heads")
        check(hip, lambda x, o32, o16: hip.merge_heads_f32_dev(batch, seq, heads, dim, x, o32, o16), [f32(rng, count)],
              [(count, np.float32), (count, np.uint16)], 0.0, 0.0, "merge heads")
