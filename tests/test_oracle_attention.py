"""Pins the oracle's attention recurrence: reference vectors vs two-pass softmax, closed form, invariants."""
import numpy as np
import pytest

from conftest import assert_close


def two_pass64(q, k, v, contexts, seq, dim, scale, z_bias=None, attn_bias=None, causal=False):
    """softmax(QK^T*scale + biases) V in float64 with numpy (independent of the oracle library)."""
    q = np.asarray(q, np.float64).reshape(contexts, seq, dim)
    k = np.asarray(k, np.float64).reshape(contexts, seq, dim)
    v = np.asarray(v, np.float64).reshape(contexts, seq, dim)
    logits = np.einsum("cid,cjd->cij", q, k) * scale
    if z_bias is not None:
        logits = logits + np.asarray(z_bias, np.float64).reshape(contexts, 1, seq)
    if attn_bias is not None:
        logits = logits + np.asarray(attn_bias, np.float64).reshape(contexts, seq, seq)
    if causal:
        mask = np.triu(np.ones((seq, seq), bool), 1)
        logits = np.where(mask[None], -np.inf, logits)
    logits -= logits.max(axis=-1, keepdims=True)
    p = np.exp(logits)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("cij,cjd->cid", p, v).reshape(-1)


def test_reference_vectors(oracle, golden):
    for c in golden["attention"]:
        out = oracle.attention_f32(c["contexts"], c["sequence"], c["head_dim"], c["scale"], c["q"], c["k"], c["v"],
                                   c["z_bias"], c["attn_bias"])
        want = two_pass64(c["q"], c["k"], c["v"], c["contexts"], c["sequence"], c["head_dim"], c["scale"],
                          c["z_bias"], c["attn_bias"])
        assert_close(out, want, 0, c["tolerance"], c["source"])


def test_nonfinite_dot_is_reported(oracle, golden):
    c = golden["attention_nonfinite"]
    with pytest.raises(oracle.OracleError) as info:
        oracle.attention_f32(1, 1, 1, c["scale"], [np.finfo(np.float32).max], c["k"], c["v"])
    assert info.value.label == c["label"]


@pytest.mark.parametrize("contexts,seq,dim,causal,biased", [
    (1, 1, 1, False, False), (2, 7, 3, False, False), (3, 33, 8, True, False), (2, 19, 5, False, True),
    (1, 40, 16, True, True), (4, 64, 64, False, False),
])
def test_closed_form(oracle, contexts, seq, dim, causal, biased):
    rng = np.random.default_rng(contexts * 100 + seq + dim)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    zb = rng.normal(size=contexts * seq).astype(np.float32) if biased else None
    ab = rng.normal(size=contexts * seq * seq).astype(np.float32) if biased else None
    scale = 1.0 / np.sqrt(dim)
    out = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, zb, ab, causal)
    want = two_pass64(q, k, v, contexts, seq, dim, scale, zb, ab, causal)
    assert_close(out, want, 1e-5, 1e-5, "online vs two-pass")
    assert_close(oracle.attention_f64(contexts, seq, dim, scale, q, k, v, zb, ab, causal), want, 1e-12, 1e-12,
                 "f64 closed form in C")


def test_invariants(oracle):
    rng = np.random.default_rng(5)
    contexts, seq, dim = 2, 23, 4
    q, k = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(2))
    v = rng.normal(size=contexts * seq * dim).astype(np.float32)
    # V = 1 -> every output is 1 (softmax rows sum to one)
    ones = oracle.attention_f32(contexts, seq, dim, 0.5, q, k, np.ones_like(v))
    assert_close(ones, np.ones_like(ones), 1e-6, 1e-6, "row sums")
    # Q = 0 -> uniform weights -> column means of V (prefix means when causal)
    vv = v.reshape(contexts, seq, dim).astype(np.float64)
    mean = oracle.attention_f32(contexts, seq, dim, 0.5, np.zeros_like(q), k, v)
    assert_close(mean, np.repeat(vv.mean(axis=1, keepdims=True), seq, axis=1), 1e-5, 1e-6, "column means")
    prefix = oracle.attention_f32(contexts, seq, dim, 0.5, np.zeros_like(q), k, v, causal=True)
    want = np.cumsum(vv, axis=1) / np.arange(1, seq + 1).reshape(1, seq, 1)
    assert_close(prefix, want, 1e-5, 1e-6, "prefix means")
    # causal row 0 returns V[0] exactly
    causal = oracle.attention_f32(contexts, seq, dim, 0.5, q, k, v, causal=True).reshape(contexts, seq, dim)
    assert (causal[:, 0, :] == v.reshape(contexts, seq, dim)[:, 0, :]).all()
    # causal == additive bias of -1e30 above the diagonal (how the reference expresses masks)
    bias = np.where(np.triu(np.ones((seq, seq), bool), 1), np.float32(-1e30), np.float32(0))
    bias = np.tile(bias.reshape(1, seq, seq), (contexts, 1, 1)).astype(np.float32)
    masked = oracle.attention_f32(contexts, seq, dim, 0.5, q, k, v, attn_bias=bias)
    assert (masked == causal.ravel()).all()
    # shift invariance: adding a per-context constant through z_bias changes nothing beyond rounding
    base = oracle.attention_f32(contexts, seq, dim, 0.5, q, k, v)
    shifted = oracle.attention_f32(contexts, seq, dim, 0.5, q, k, v, z_bias=np.full(contexts * seq, 3.0, np.float32))
    assert_close(shifted, base, 1e-5, 1e-6, "shift invariance")


def test_empty(oracle):
    assert oracle.attention_f32(0, 5, 4, 1.0, [], [], []).size == 0
    assert oracle.attention_f32(3, 5, 0, 1.0, [], [], []).size == 0
