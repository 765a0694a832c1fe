"""The benchmark's input generator (mcc_fill_normal_f32, mcc_fill_counter_state_u8) against a numpy
restatement of its definition: lowbias32 of (index ^ lowbias32(stream id)), 24 bits to a uniform in
(0, 1), Box-Muller's cosine branch; codes as the high part of hash x n_codes."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def lowbias32(x):
    x = np.asarray(x, dtype=np.uint64) & 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def uniform(h):
    return ((h >> 8).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)


@pytest.mark.parametrize("n,stream_id,sigma", [(1, 0, 1.0), (1000003, 7, 1.0), (4096, 0xDEADBEEF, 0.01)])
def test_fill_normal_follows_its_definition(n, stream_id, sigma):
    import torch
    from motifcl_amd import ops
    got = ops.fill_normal(torch.empty(n, device="cuda"), stream_id, sigma).cpu().numpy()
    i = np.arange(n, dtype=np.uint64)
    salt = lowbias32(stream_id)
    u1, u2 = uniform(lowbias32((2 * i) ^ salt)), uniform(lowbias32((2 * i + 1) ^ salt))
    want = sigma * np.sqrt(-2.0 * np.log(u1.astype(np.float64))) * np.cos(2.0 * np.pi * u2.astype(np.float64))
    # float32 log and cosine on the device against float64 here
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6 * sigma)
    if n > 100000:
        assert abs(got.mean()) < 4 * sigma / np.sqrt(n)
        assert abs(got.std() / sigma - 1.0) < 5e-3
        assert abs((got ** 4).mean() / sigma ** 4 - 3.0) < 0.05  # a normal's fourth moment


@pytest.mark.parametrize("groups,stream_id,n_codes", [(1, 0, 63), (250001, 3, 63), (999, 5, 64), (999, 5, 1)])
def test_fill_counter_state_follows_its_definition(groups, stream_id, n_codes):
    import torch
    from motifcl_amd import ops
    got = ops.fill_counter_state(torch.empty(groups * 3, dtype=torch.uint8, device="cuda"), stream_id, n_codes).cpu().numpy()
    e = np.arange(4 * groups, dtype=np.uint64)
    codes = (lowbias32(e ^ lowbias32(stream_id ^ 0x5BD1E995)) * n_codes) >> 32
    assert codes.max() < n_codes
    c = codes.reshape(groups, 4)
    word = c[:, 0] | (c[:, 1] << 6) | (c[:, 2] << 12) | (c[:, 3] << 18)
    want = np.stack([word & 255, (word >> 8) & 255, (word >> 16) & 255], axis=1).astype(np.uint8).reshape(-1)
    assert np.array_equal(got, want)
    if groups > 100000 and n_codes == 63:
        counts = np.bincount(codes.astype(np.int64), minlength=63)
        assert counts.min() > 0.95 * codes.size / 63 and counts.max() < 1.05 * codes.size / 63


def test_fill_rejects_bad_arguments():
    import torch
    from motifcl_amd import ops
    with pytest.raises(Exception):
        ops.fill_counter_state(torch.empty(30, dtype=torch.uint8, device="cuda"), 0, 65)
    with pytest.raises(ValueError):
        ops.fill_counter_state(torch.empty(31, dtype=torch.uint8, device="cuda"), 0, 63)
