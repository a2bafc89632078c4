"""Parity of the flash-style attention kernel against the CPU oracle (1e-4 rel / 1e-5 abs, row sums)."""
import numpy as np
import pytest

from conftest import F32_ABS, F32_REL, assert_close

pytestmark = pytest.mark.gpu


def run(hip, contexts, seq, dim, scale, q, k, v, zb=None, ab=None, causal=False):
    out = np.zeros(contexts * seq * dim, np.float32)
    hip.attention_f32(contexts, seq, dim, scale, causal, q, k, v, zb, ab, out)
    return out


def test_reference_vectors(hip, oracle, golden):
    for c in golden["attention"]:
        f = lambda name: None if c[name] is None else np.array(c[name], np.float32)
        got = run(hip, c["contexts"], c["sequence"], c["head_dim"], c["scale"], f("q"), f("k"), f("v"), f("z_bias"),
                  f("attn_bias"))
        want = oracle.attention_f64(c["contexts"], c["sequence"], c["head_dim"], c["scale"], c["q"], c["k"], c["v"],
                                    c["z_bias"], c["attn_bias"])
        assert_close(got, want, 0, c["tolerance"], c["source"])


CASES = [
    # contexts, seq, dim, causal, biased
    (1, 1, 1, False, False), (2, 7, 3, False, False), (3, 33, 8, True, False), (2, 19, 5, False, True),
    (1, 40, 16, True, True), (4, 64, 64, False, False), (2, 129, 64, True, False), (3, 200, 32, False, False),
    (2, 257, 64, False, True), (1, 300, 128, True, False), (1, 130, 80, False, False), (2, 96, 256, True, False),
    (1, 70, 200, False, True), (5, 128, 64, True, True), (8, 384, 64, True, False),
    # causal query tiles are taken in pairs (j, last - j): five tiles (the middle one alone), four tiles, one XCD slice each
    (8, 600, 64, True, False), (16, 512, 32, True, False), (3, 1100, 64, True, False),
    # 256 paired causal workgroups: too many to split the keys, one chunk per tile would be nothing to merge
    (256, 256, 64, True, False), (255, 256, 32, True, False),
]


@pytest.mark.parametrize("contexts,seq,dim,causal,biased", CASES)
def test_random_cases(hip, oracle, contexts, seq, dim, causal, biased):
    rng = np.random.default_rng(contexts * 1000 + seq * 7 + dim)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    zb = rng.normal(size=contexts * seq).astype(np.float32) if biased else None
    ab = rng.normal(size=contexts * seq * seq).astype(np.float32) if biased else None
    scale = float(1.0 / np.sqrt(dim))
    got = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, causal)
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, zb, ab, causal, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"attention {contexts}x{seq}x{dim} causal={causal} bias={biased}")
    # softmax row sums: V = 1 must give exactly-normalised rows
    ones = run(hip, contexts, seq, dim, scale, q, k, np.ones_like(v), zb, ab, causal)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")


@pytest.mark.parametrize("contexts,seq,dim,causal,scale", [
    (256, 16, 64, False, 0.125), (257, 16, 64, True, 0.125), (300, 49, 32, False, 0.1768), (301, 49, 32, True, 0.1768),
    (1000, 1, 64, False, 0.125), (513, 31, 128, True, 0.0884), (258, 32, 128, False, 0.0884), (259, 33, 128, True, 0.0884),
    (400, 64, 64, False, 0.125), (402, 64, 64, True, 0.125), (262, 64, 128, False, -0.2), (300, 7, 8, True, 0.35),
    (260, 50, 40, False, 0.158), (261, 20, 100, True, 0.1), (333, 64, 32, True, 3.0), (270, 48, 64, False, 0.0),
    (2048, 16, 32, False, 0.1768)])
def test_many_short_contexts(hip, oracle, contexts, seq, dim, causal, scale):
    """Windowed attention: at least 256 contexts of at most 64 positions each are handled a wavefront per context.
    Context counts that do not fill the last workgroup, lengths either side of the 32-key tile, head sizes that are
    padded to the next kernel (8, 40, 100), a peaked softmax (scale 3), a flat one (scale 0) and a negative scale;
    output positions past each context's end stay untouched (the buffer's tail keeps its fill)."""
    rng = np.random.default_rng(contexts * 131 + seq * 7 + dim)
    n = contexts * seq * dim
    q, k, v = (rng.normal(size=n).astype(np.float32) for _ in range(3))
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(a) for a in (q, k, v))
    tail = 4096
    d_out = hip.DeviceBuffer.from_array(np.full(n + tail, 7.5, np.float32))
    hip.attention_f32_dev(contexts, seq, dim, scale, causal, d_q, d_k, d_v, None, None, d_out)
    hip.device_synchronize()
    both = d_out.to_array(np.float32, n + tail)
    got = both[:n]
    assert (both[n:] == 7.5).all(), "wrote past the last context"
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, None, None, causal, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"short contexts {contexts}x{seq}x{dim} causal={causal}")
    d_ones = hip.DeviceBuffer.from_array(np.ones(n, np.float32))
    hip.attention_f32_dev(contexts, seq, dim, scale, causal, d_q, d_k, d_ones, None, None, d_out)
    hip.device_synchronize()
    ones = d_out.to_array(np.float32, n)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")
    if causal:  # position 0 attends to itself only
        assert_close(got.reshape(contexts, seq, dim)[:, 0], v.reshape(contexts, seq, dim)[:, 0], F32_REL, F32_ABS, "first row")


@pytest.mark.parametrize("contexts,seq,dim,biased,scale", [
    (1, 2048, 64, True, 0.125), (1, 2048, 64, False, 0.125), (3, 1000, 32, True, 0.2), (2, 300, 128, False, -0.4),
    (1, 512, 64, False, 3.0), (5, 260, 64, True, 0.0), (1, 4096, 16, False, 0.25), (7, 384, 64, False, 0.125)])
def test_keys_split_over_workgroups(hip, oracle, contexts, seq, dim, biased, scale):
    """Non-causal calls with few query tiles (the reference's own caller attends within one context) split the keys
    over workgroups and merge the partial rows: same values as the oracle, rows still sum to one, and a softmax so
    peaked (scale 3) that one split holds nearly all of a row's weight."""
    rng = np.random.default_rng(contexts * 31 + seq + dim)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    zb = rng.normal(size=contexts * seq).astype(np.float32) if biased else None
    ab = rng.normal(0, 2.0, size=contexts * seq * seq).astype(np.float32) if biased else None
    got = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, False)
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, zb, ab, False, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"split keys {contexts}x{seq}x{dim} bias={biased} scale={scale}")
    ones = run(hip, contexts, seq, dim, scale, q, k, np.ones_like(v), zb, ab, False)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")
    again = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, False)
    assert (again == got).all(), "the splits are merged in a fixed order"


@pytest.mark.parametrize("contexts,seq,dim,biased,scale", [
    (8, 2048, 128, False, 0.0884), (4, 4096, 64, False, 0.125), (12, 1000, 64, False, 0.125), (1, 2048, 64, True, 0.125),
    (3, 300, 32, True, -0.2), (2, 260, 64, False, 2.0), (5, 640, 16, False, 0.25)])
def test_causal_keys_split_per_query_tile(hip, oracle, contexts, seq, dim, biased, scale):
    """Causal calls with few contexts give every query tile one workgroup per chunk of its keys (tile j sees (j+1)*128
    keys) instead of pairing tiles: rows early in a tile see none of a late chunk's keys (a partial row of weight zero),
    the last chunk of a tile is cut by the diagonal, and the merge adds a different number of chunks per tile."""
    rng = np.random.default_rng(contexts * 17 + seq + dim)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    zb = rng.normal(size=contexts * seq).astype(np.float32) if biased else None
    ab = rng.normal(0, 2.0, size=contexts * seq * seq).astype(np.float32) if biased else None
    got = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, True)
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, zb, ab, True, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"causal split {contexts}x{seq}x{dim} bias={biased} scale={scale}")
    ones = run(hip, contexts, seq, dim, scale, q, k, np.ones_like(v), zb, ab, True)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")
    first = got.reshape(contexts, seq, dim)[:, 0, :]
    assert_close(first, v.reshape(contexts, seq, dim)[:, 0, :], 1e-6, 1e-6, "causal row 0 is V[0]")
    again = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, True)
    assert (again == got).all()


@pytest.mark.parametrize("contexts,seq,dim,biased", [(6, 300, 128, False), (2, 384, 128, True)])
def test_large_logits_against_float64(hip, oracle, contexts, seq, dim, biased):
    """scale = 1 with head_dim 128 makes logits of magnitude 30-45, where an f32 dot product of 128 terms is itself
    uncertain by a few 1e-5: the f32 oracle then misses the 1e-4 / 1e-5 bar against exact float64 by up to 1.8x, and
    two f32 evaluations that add in different orders (the oracle's loop, the matrix instruction's k order) can differ
    by more than the bar although neither is wrong.  A randomised sweep found such cases (1.09x and 1.12x against the
    oracle); at the configurations' own scale (1/sqrt(d)) the same shapes sit at 0.05 of the bar.  So here the kernel
    and the oracle are both measured against float64: the kernel may not be less accurate than the oracle is."""
    for seed in range(3):
        rng = np.random.default_rng(seed)
        q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
        zb = rng.normal(size=contexts * seq).astype(np.float32) if biased else None
        got = run(hip, contexts, seq, dim, 1.0, q, k, v, zb, None, False)
        f32 = oracle.attention_f32(contexts, seq, dim, 1.0, q, k, v, zb, None, False, threads=8)
        exact = oracle.attention_f64(contexts, seq, dim, 1.0, q, k, v, zb, None)
        bar = F32_ABS + F32_REL * np.abs(exact)
        gpu_err, oracle_err = np.abs(got - exact) / bar, np.abs(f32 - exact) / bar
        assert np.sqrt(np.mean(gpu_err ** 2)) <= 1.25 * np.sqrt(np.mean(oracle_err ** 2)), "rms error against float64"
        assert gpu_err.max() <= max(2.0 * oracle_err.max(), 1.0), "largest error against float64"
        assert gpu_err.max() <= 3.0  # and in absolute terms it stays within three times the bar


@pytest.mark.parametrize("scale", [-0.3, 0.0, 2.5])
@pytest.mark.parametrize("causal", [False, True])
def test_unusual_scales(hip, oracle, scale, causal):
    """Negative, zero and large scales on the fast path (|scale| is folded into the exponent, the sign into Q; a large
    scale makes running maxima jump by more than the lag the kernel tolerates before rescaling)."""
    contexts, seq, dim = 2, 150, 64
    rng = np.random.default_rng(int(scale * 10) + 50 + causal)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    got = run(hip, contexts, seq, dim, scale, q, k, v, None, None, causal)
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, None, None, causal, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"attention scale={scale} causal={causal}")
    ones = run(hip, contexts, seq, dim, scale, q, k, np.ones_like(v), None, None, causal)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")


@pytest.mark.parametrize("contexts,seq,dim,causal,which,scale", [
    (4, 256, 64, False, "both", 0.125), (2, 300, 32, True, "both", 0.2), (8, 132, 64, False, "attn", 0.125),
    (3, 64, 48, True, "z", 0.15), (1, 1024, 64, False, "attn", 0.125), (2, 200, 64, True, "both", -0.3),
    (2, 96, 20, False, "both", 0.0),
])
def test_biases_in_the_matrix_core_kernel(hip, oracle, contexts, seq, dim, causal, which, scale):
    """Sequences that are a multiple of four with head_dim <= 64 keep the flash-style kernel when z_bias / attn_bias
    are given (the shape of the reference's own caller, crates/st-nn/src/z_rba/attention.rs:586-595: one context,
    an attn_bias kernel matrix): logit = (dot*scale + z_bias[key]) + attn_bias[query][key], pure.rs:11870-11880."""
    rng = np.random.default_rng(contexts * 100 + seq + dim)
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    zb = rng.normal(size=contexts * seq).astype(np.float32) if which in ("z", "both") else None
    ab = rng.normal(0, 2.0, size=contexts * seq * seq).astype(np.float32) if which in ("attn", "both") else None
    got = run(hip, contexts, seq, dim, scale, q, k, v, zb, ab, causal)
    want = oracle.attention_f32(contexts, seq, dim, scale, q, k, v, zb, ab, causal, threads=8)
    assert_close(got, want, F32_REL, F32_ABS, f"biased attention {contexts}x{seq}x{dim} {which} causal={causal}")
    ones = run(hip, contexts, seq, dim, scale, q, k, np.ones_like(v), zb, ab, causal)
    assert_close(ones, np.ones_like(ones), F32_REL, F32_ABS, "row sums")
    if which == "attn" and not causal:
        # a -1e30 bias above the diagonal is the reference's way of masking: same values as the causal flag
        mask = np.where(np.triu(np.ones((seq, seq), bool), 1), np.float32(-1e30), np.float32(0))
        masked = run(hip, contexts, seq, dim, scale, q, k, v, None,
                     np.ascontiguousarray(np.tile(mask.reshape(1, seq, seq), (contexts, 1, 1)), np.float32).ravel())
        assert_close(masked, run(hip, contexts, seq, dim, scale, q, k, v, causal=True), F32_REL, F32_ABS, "mask == causal")


def test_invariants(hip, oracle):
    rng = np.random.default_rng(5)
    contexts, seq, dim = 3, 150, 64
    q, k, v = (rng.normal(size=contexts * seq * dim).astype(np.float32) for _ in range(3))
    vv = v.reshape(contexts, seq, dim).astype(np.float64)
    mean = run(hip, contexts, seq, dim, 0.125, np.zeros_like(q), k, v)
    assert_close(mean, np.repeat(vv.mean(axis=1, keepdims=True), seq, axis=1), F32_REL, F32_ABS, "column means")
    prefix = run(hip, contexts, seq, dim, 0.125, np.zeros_like(q), k, v, causal=True)
    assert_close(prefix, np.cumsum(vv, axis=1) / np.arange(1, seq + 1).reshape(1, seq, 1), F32_REL, F32_ABS,
                 "prefix means")
    causal = run(hip, contexts, seq, dim, 0.125, q, k, v, causal=True).reshape(contexts, seq, dim)
    assert_close(causal[:, 0, :], v.reshape(contexts, seq, dim)[:, 0, :], 1e-6, 1e-6, "causal row 0 is V[0]")
    # the causal flag equals the reference's way of masking: a large negative additive bias
    bias = np.where(np.triu(np.ones((seq, seq), bool), 1), np.float32(-1e30), np.float32(0))
    bias = np.ascontiguousarray(np.tile(bias.reshape(1, seq, seq), (contexts, 1, 1)), np.float32).ravel()
    masked = run(hip, contexts, seq, dim, 0.125, q, k, v, ab=bias)
    assert_close(masked, causal, F32_REL, F32_ABS, "causal == -1e30 bias")


def test_empty_and_validation(hip):
    out = np.zeros(0, np.float32)
    e = np.zeros(0, np.float32)
    hip.attention_f32(0, 5, 4, 1.0, False, e, e, e, None, None, out)
    hip.attention_f32(3, 5, 0, 1.0, False, e, e, e, None, None, out)
    q = np.ones(8, np.float32)
    keep = np.full(8, 13.0, np.float32)
    with pytest.raises(hip.HipErr, match="key buffer length"):
        hip.attention_f32(1, 4, 2, 1.0, False, q, q[:-1], q, None, None, keep)
    with pytest.raises(hip.HipErr, match="z_bias buffer length"):
        hip.attention_f32(1, 4, 2, 1.0, False, q, q, q, np.zeros(3, np.float32), None, keep)
    with pytest.raises(hip.HipErr, match="attn_bias buffer length"):
        hip.attention_f32(1, 4, 2, 1.0, False, q, q, q, None, np.zeros(15, np.float32), keep)
    with pytest.raises(hip.HipErr, match="scaled_dot_attention_scale"):
        hip.attention_f32(1, 4, 2, float("nan"), False, q, q, q, None, None, keep)
    bad = q.copy()
    bad[3] = np.inf
    with pytest.raises(hip.HipErr, match="scaled_dot_attention_key"):
        hip.attention_f32(1, 4, 2, 1.0, False, q, bad, q, None, None, keep)
    with pytest.raises(hip.HipErr, match="head_dim 300 exceeds"):
        hip.attention_f32(1, 1, 300, 1.0, False, np.ones(300, np.float32), np.ones(300, np.float32),
                          np.ones(300, np.float32), None, None, np.zeros(300, np.float32))
    assert (keep == 13.0).all()


def test_overflow_is_reported_as_nonfinite(hip, golden):
    """crates/st-tensor/src/pure.rs:15365-15389: q = f32::MAX, k = 2 overflows.  The CPU path names the
    first overflowing intermediate (…_dot); the GPU path reports the non-finite output (…_output)."""
    from spiraltorch_amd import Tensor, TensorError
    q = Tensor(1, 1, [np.finfo(np.float32).max])
    with pytest.raises(TensorError) as err:
        q.scaled_dot_attention(Tensor(1, 1, [2.0]), Tensor(1, 1, [1.0]), contexts=1, sequence=1, scale=1.0)
    assert err.value.kind == "NonFiniteValue"
    assert err.value.fields["label"] == "scaled_dot_attention_output"


def test_tensor_mirror(hip, oracle, golden):
    from spiraltorch_amd import Tensor, TensorError
    c = golden["attention"][1]
    q, k, v = (Tensor(2, 2, c[name]) for name in ("q", "k", "v"))
    out = q.scaled_dot_attention(k, v, contexts=1, sequence=2, scale=1.0, z_bias=Tensor(1, 2, c["z_bias"]),
                                 attn_bias=Tensor(2, 2, c["attn_bias"]), backend="hip")
    want = oracle.attention_f64(1, 2, 2, 1.0, c["q"], c["k"], c["v"], c["z_bias"], c["attn_bias"])
    assert out.shape() == (2, 2)
    assert_close(out.data(), want, 0, 1e-5, "Tensor.scaled_dot_attention")
    with pytest.raises(TensorError) as err:
        q.scaled_dot_attention(k, Tensor(3, 2), contexts=1, sequence=2, scale=1.0)
    assert err.value.kind == "ShapeMismatch"


def test_config3_full_size(hip, oracle):
    """BASELINE config 3: B8 H16 S2048 D64 (128 contexts), scale 1/8, non-causal and causal.
    The oracle checks three whole contexts per mode; every context is covered by the row-sum check
    (V = 1) and by context-permutation equivariance."""
    from spiraltorch_amd import inputs
    contexts, seq, dim = 128, 2048, 64
    count = contexts * seq * dim
    q = inputs.normal(inputs.seed_for(3, 0), count)
    k = inputs.normal(inputs.seed_for(3, 1), count)
    v = inputs.normal(inputs.seed_for(3, 2), count)
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(a) for a in (q, k, v))
    d_ones = hip.DeviceBuffer.from_array(np.ones(count, np.float32))
    d_out = hip.DeviceBuffer(count * 4)
    per = seq * dim
    for causal in (False, True):
        hip.attention_f32_dev(contexts, seq, dim, 0.125, causal, d_q, d_k, d_v, None, None, d_out)
        hip.device_synchronize()
        got = d_out.to_array(np.float32, (contexts, per))
        for ctx in (0, 77, 127):
            sl = slice(ctx * per, (ctx + 1) * per)
            want = oracle.attention_f32(1, seq, dim, 0.125, q[sl], k[sl], v[sl], causal=causal)
            assert_close(got[ctx], want, F32_REL, F32_ABS, f"config 3 causal={causal} context {ctx}")
        hip.attention_f32_dev(contexts, seq, dim, 0.125, causal, d_q, d_k, d_ones, None, None, d_out)
        hip.device_synchronize()
        sums = d_out.to_array(np.float32, count)
        assert_close(sums, np.ones(count), F32_REL, F32_ABS, f"config 3 causal={causal} row sums")
        # contexts are independent: reversing their order reverses the output blocks bit for bit
        rev = lambda a: np.ascontiguousarray(a.reshape(contexts, per)[::-1])
        d_qr, d_kr, d_vr = (hip.DeviceBuffer.from_array(rev(a)) for a in (q, k, v))
        hip.attention_f32_dev(contexts, seq, dim, 0.125, causal, d_qr, d_kr, d_vr, None, None, d_out)
        hip.device_synchronize()
        assert (d_out.to_array(np.float32, (contexts, per)) == got[::-1]).all()
