"""The measurement aids behind `bench.py --probes` do what their declarations say: the matrix-instruction loops are checked
through the sums they leave behind (exact on small integers), the load loop through its argument checks."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _expected_mfma_sum(values, k_per_lane, halves, iterations):
    """values: (16, 256, k_per_lane) fragment values as thread t of the workgroup holds them for fragment f = s*8 + i (A)
    or s*8 + 4 + j (B).  Lane l of a wavefront holds row l % 32 and the k-values k_per_lane*(l // 32) + e.  The sum over
    all outputs of A·Bᵀ is the dot product of the operands' column sums, so per wavefront and iteration the loop adds
    sum_s sum_k (sum_i colsum(A_si)[k]) * (sum_j colsum(B_sj)[k])."""
    total = np.zeros(4, np.float64)
    for wave in range(4):
        lanes = values[:, wave * 64:(wave + 1) * 64, :].astype(np.float64)           # (16, 64, k_per_lane)
        colsum = lanes.reshape(16, halves, 32, k_per_lane).sum(axis=2).reshape(16, halves * k_per_lane)  # (16, K)
        for s in range(2):
            a = colsum[s * 8:s * 8 + 4].sum(axis=0)
            b = colsum[s * 8 + 4:s * 8 + 8].sum(axis=0)
            total[wave] += float((a * b).sum())
    return total * iterations


def test_bf16_matrix_instruction_loop_sums(hip):
    from spiraltorch_amd import inputs
    rng = np.random.default_rng(11)
    values = rng.integers(-2, 3, size=(16, 256, 8)).astype(np.float32)
    d_ops = hip.DeviceBuffer.from_array(inputs.to_bf16(values.ravel()))
    workgroups, iterations = 3, 5
    sink = hip.DeviceBuffer(workgroups * 256 * 4)
    hip.probe_mfma_bf16_dev(workgroups, iterations, d_ops, sink)
    hip.device_synchronize()
    got = sink.to_array(np.float32, workgroups * 256).reshape(workgroups, 4, 64).astype(np.float64).sum(axis=2)
    want = _expected_mfma_sum(values, 8, 2, iterations)
    assert (got == want[None, :]).all(), (got, want)


def test_f32_matrix_instruction_loop_sums(hip):
    rng = np.random.default_rng(12)
    values = rng.integers(-3, 4, size=(16, 256, 1)).astype(np.float32)
    d_ops = hip.DeviceBuffer.from_array(values.ravel())
    workgroups, iterations = 2, 7
    sink = hip.DeviceBuffer(workgroups * 256 * 4)
    hip.probe_mfma_f32_dev(workgroups, iterations, d_ops, sink)
    hip.device_synchronize()
    got = sink.to_array(np.float32, workgroups * 256).reshape(workgroups, 4, 64).astype(np.float64).sum(axis=2)
    want = _expected_mfma_sum(values, 1, 2, iterations)
    assert (got == want[None, :]).all(), (got, want)


def test_load_loop_runs_and_checks_its_arguments(hip):
    region_bytes = 1 << 20
    region = hip.DeviceBuffer(region_bytes)
    region.zero()
    hip.probe_stream_lds_dev(4, 3, region, region_bytes)
    hip.probe_stream_lds_dev(0, 3, region, region_bytes)  # nothing to do
    hip.device_synchronize()
    with pytest.raises(hip.HipErr):
        hip.probe_stream_lds_dev(4, 3, region, 4096)       # below 64 KiB
    with pytest.raises(hip.HipErr):
        hip.probe_stream_lds_dev(4, 3, region, 1 << 31)    # not below 2 GiB
    with pytest.raises(hip.HipErr):
        hip.probe_stream_lds_dev(4, 3, None, region_bytes)
