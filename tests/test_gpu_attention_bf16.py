"""Parity of the bf16 attention kernel (heads read in place from (batch*seq, ld) matrices) against the CPU
oracle run on the same bf16-rounded inputs.  Tolerance: 2e-2 relative plus 1e-2 absolute — the output is
rounded to bf16 (2^-9 relative) and the softmax weights enter the value product as bf16."""
import numpy as np
import pytest

from conftest import BF16_REL, assert_close
from spiraltorch_amd import inputs

pytestmark = pytest.mark.gpu

ABS = 1e-2


def run_fused(hip, batch, heads, seq, dim, scale, qkv_bits, causal):
    """qkv_bits: (batch*seq, 3*heads*dim) uint16 with column blocks [Q | K | V]."""
    width = heads * dim
    d_qkv = hip.DeviceBuffer.from_array(qkv_bits)
    d_out = hip.DeviceBuffer(batch * seq * width * 2)
    d_out.zero()
    hip.attention_bf16_dev(batch, heads, seq, dim, scale, causal, d_qkv, d_qkv.at(width * 2), d_qkv.at(2 * width * 2),
                           3 * width, d_out, width)
    hip.device_synchronize()
    return inputs.from_bf16(d_out.to_array(np.uint16, batch * seq * width)).reshape(batch * seq, width)


def oracle_fused(oracle, batch, heads, seq, dim, scale, qkv_bits, causal):
    width = heads * dim
    qkv = inputs.from_bf16(qkv_bits.ravel()).reshape(batch, seq, 3, heads, dim)
    # (batch, seq, heads, dim) -> (batch*heads, seq, dim)
    split = [np.ascontiguousarray(qkv[:, :, i].transpose(0, 2, 1, 3)).ravel() for i in range(3)]
    out = oracle.attention_f32(batch * heads, seq, dim, scale, *split, causal=causal, threads=8)
    return out.reshape(batch, heads, seq, dim).transpose(0, 2, 1, 3).reshape(batch * seq, width)


CASES = [
    # batch, heads, seq, dim, causal
    (1, 1, 1, 64, False), (1, 1, 1, 64, True), (2, 3, 33, 64, True), (1, 2, 64, 64, False), (2, 2, 129, 64, True),
    (1, 4, 200, 64, False), (2, 1, 257, 128, True), (1, 2, 130, 128, False), (4, 2, 384, 64, True),
    (1, 8, 640, 64, True),
]


@pytest.mark.parametrize("batch,heads,seq,dim,causal", CASES)
def test_fused_qkv_layout(hip, oracle, batch, heads, seq, dim, causal):
    rng = np.random.default_rng(batch * 1000 + heads * 100 + seq + dim)
    qkv_bits = inputs.to_bf16(rng.normal(size=batch * seq * 3 * heads * dim).astype(np.float32))
    scale = float(1.0 / np.sqrt(dim))
    got = run_fused(hip, batch, heads, seq, dim, scale, qkv_bits, causal)
    want = oracle_fused(oracle, batch, heads, seq, dim, scale, qkv_bits, causal)
    assert_close(got, want, BF16_REL, ABS, f"bf16 attention b{batch} h{heads} s{seq} d{dim} causal={causal}")


@pytest.mark.parametrize("scale", [-0.2, 0.0, 3.0])
@pytest.mark.parametrize("causal", [False, True])
def test_unusual_scales(hip, oracle, scale, causal):
    """Negative, zero and large scales (the kernel folds |scale| into the exponent and moves the sign into Q)."""
    batch, heads, seq, dim = 1, 2, 97, 64
    rng = np.random.default_rng(int(scale * 10) + 100 + causal)
    qkv_bits = inputs.to_bf16((rng.normal(size=batch * seq * 3 * heads * dim) * 0.5).astype(np.float32))
    got = run_fused(hip, batch, heads, seq, dim, scale, qkv_bits, causal)
    want = oracle_fused(oracle, batch, heads, seq, dim, scale, qkv_bits, causal)
    assert_close(got, want, BF16_REL, ABS, f"bf16 attention scale={scale} causal={causal}")


def test_contiguous_contexts_and_row_sums(hip, oracle):
    """heads = 1, ld = head_dim is the (contexts*seq, head_dim) layout of the f32 entry point; V = 1 must give
    rows that sum to one (every output element equals 1 up to the bf16 rounding of the result)."""
    contexts, seq, dim = 5, 150, 64
    rng = np.random.default_rng(9)
    q, k, v = (inputs.to_bf16(rng.normal(size=contexts * seq * dim).astype(np.float32)) for _ in range(3))
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(a) for a in (q, k, v))
    d_out = hip.DeviceBuffer(contexts * seq * dim * 2)
    for causal in (False, True):
        hip.attention_bf16_dev(contexts, 1, seq, dim, 0.125, causal, d_q, d_k, d_v, dim, d_out, dim)
        hip.device_synchronize()
        got = inputs.from_bf16(d_out.to_array(np.uint16, contexts * seq * dim))
        want = oracle.attention_f32(contexts, seq, dim, 0.125, inputs.from_bf16(q), inputs.from_bf16(k),
                                    inputs.from_bf16(v), causal=causal, threads=8)
        assert_close(got, want, BF16_REL, ABS, f"contiguous layout causal={causal}")
        d_ones = hip.DeviceBuffer.from_array(inputs.to_bf16(np.ones(contexts * seq * dim, np.float32)))
        hip.attention_bf16_dev(contexts, 1, seq, dim, 0.125, causal, d_q, d_k, d_ones, dim, d_out, dim)
        hip.device_synchronize()
        ones = inputs.from_bf16(d_out.to_array(np.uint16, contexts * seq * dim))
        assert_close(ones, np.ones_like(ones), 2.0 ** -8, 0.0, "row sums")


def test_decoder_shape_properties(hip):
    """Full decoder shape (batch 16, 8 heads, seq 1024, head_dim 64, causal): size-independent properties only.
    Row 0 of every context attends to key 0 alone, so it must return V[0] bit for bit; Q = 0 gives prefix means."""
    batch, heads, seq, dim = 16, 8, 1024, 64
    width = heads * dim
    bits = inputs.to_bf16(inputs.normal(77, batch * seq * 3 * width)).reshape(batch * seq, 3 * width)
    got = run_fused(hip, batch, heads, seq, dim, 0.125, bits, True).reshape(batch, seq, width)
    v = inputs.from_bf16(bits[:, 2 * width:].ravel()).reshape(batch, seq, width)
    assert np.array_equal(got[:, 0], v[:, 0]), "first causal row must equal V[0]"
    assert np.isfinite(got).all()
    zero_q = bits.copy()
    zero_q[:, :width] = 0
    got = run_fused(hip, batch, heads, seq, dim, 0.125, zero_q, True).reshape(batch, seq, width)
    prefix = np.cumsum(v.astype(np.float64), axis=1) / np.arange(1, seq + 1).reshape(1, seq, 1)
    assert_close(got, prefix, BF16_REL, ABS, "prefix means at the decoder shape")


def test_unsupported_shapes_are_rejected(hip):
    buf = hip.DeviceBuffer(1 << 16)
    with pytest.raises(hip.HipErr):
        hip.attention_bf16_dev(1, 1, 8, 32, 0.1, False, buf, buf, buf, 32, buf, 32)      # head_dim
    with pytest.raises(hip.HipErr):
        hip.attention_bf16_dev(1, 2, 8, 64, 0.1, False, buf, buf, buf, 64, buf, 128)     # ld_in < heads*head_dim
    with pytest.raises(hip.HipErr):
        hip.attention_bf16_dev(1, 1, 8, 64, float("inf"), False, buf, buf, buf, 64, buf, 64)
