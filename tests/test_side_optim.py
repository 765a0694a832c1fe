"""FP32 side optimizers (src/ops/optim.cpp:17-86, kernels/optim.cl:1-7,31-53 of MotifCL): the
oracle against the reference's own expectation and closed forms, then the HIP kernels against
the oracle, bit for bit."""
import numpy as np
import pytest

F = np.float32


def np_adam(p, g, m, v, lr, b1, b2, eps, step, wd):
    """Independent float32 restatement with numpy scalars (one rounding per operation)."""
    p, g, m, v = (np.asarray(a, dtype=F) for a in (p, g, m, v))
    lr, b1, b2, eps, wd = F(lr), F(b1), F(b2), F(eps), F(wd)
    # beta^step: the binary32 power rounded from a double-precision one (the C library's powf is
    # correctly rounded on these inputs; numpy's float32 power is not always)
    ib1 = F(1) / (F(1) - F(np.float64(b1) ** step))
    ib2 = F(1) / (F(1) - F(np.float64(b2) ** step))
    mt = b1 * m + (F(1) - b1) * g
    vt = b2 * v + ((F(1) - b2) * g) * g
    upd = (mt * ib1) / (np.sqrt(vt * ib2, dtype=F) + eps)
    return (p - lr * upd) - (lr * wd) * p, mt, vt


def test_oracle_reproduces_the_reference_test_expectation(oracle):
    # tests/test_adam.cpp:22-42: p = 1..5, g = 1, lr = 1e-2, weight decay 0.1, first step
    p0 = np.arange(1, 6, dtype=F)
    p, m, v = oracle.adam_update(p0, np.ones(5, F), np.zeros(5, F), np.zeros(5, F), 1e-2, 0.9, 0.999, 1e-8, 1, 0.1)
    assert np.abs(p - (p0 - 1e-2 - 1e-2 * 0.1 * p0)).max() <= 1e-4
    assert np.allclose(m, 0.1) and np.allclose(v, 0.001)


def test_oracle_closed_forms(oracle):
    rng = np.random.default_rng(0)
    g = rng.standard_normal(1000).astype(F)
    p0 = rng.standard_normal(1000).astype(F)
    # first step from zero moments moves every parameter by lr * sign(g) (up to eps)
    p, m, v = oracle.adam_update(p0, g, np.zeros_like(g), np.zeros_like(g), 1e-3, 0.9, 0.999, 1e-12, 1, 0.0)
    assert np.abs((p0 - p) / 1e-3 - np.sign(g)).max() < 1e-3
    # zero gradient: moments decay, the parameter only sees weight decay
    m0, v0 = np.abs(g), g * g
    p, m, v = oracle.adam_update(p0, np.zeros_like(g), m0 * 0, v0, 1e-3, 0.9, 0.999, 1e-8, 7, 0.25)
    assert np.array_equal(m, np.zeros_like(g)) and np.array_equal(v, F(0.999) * v0)
    assert np.array_equal(p, (p0 - F(1e-3) * F(0)) - (F(1e-3) * F(0.25)) * p0)
    assert np.array_equal(oracle.sgd_update(p0, g, 0.5), p0 - F(0.5) * g)


@pytest.mark.parametrize("step", [1, 2, 10, 1000])
def test_oracle_matches_the_numpy_model_bit_for_bit(oracle, step):
    rng = np.random.default_rng(step)
    p0, g, m0 = (rng.standard_normal(4097).astype(F) for _ in range(3))
    v0 = (rng.random(4097) * 0.01).astype(F)
    got = oracle.adam_update(p0, g, m0, v0, 3e-4, 0.9, 0.95, 1e-8, step, 0.01)
    exp = np_adam(p0, g, m0, v0, 3e-4, 0.9, 0.95, 1e-8, step, 0.01)
    for a, b in zip(got, exp):
        assert np.array_equal(a, b)


@pytest.fixture(scope="module")
def ops():
    import torch
    import motifcl_amd
    motifcl_amd.load()
    from motifcl_amd import ops as _ops
    assert torch.cuda.is_available()
    return _ops


@pytest.mark.gpu
@pytest.mark.parametrize("n, offset", [(1, 0), (5, 0), (4096, 0), (100003, 0), (1 << 22, 0), (1001, 1), (4099, 3)])
def test_gpu_adam_and_sgd_match_the_oracle(ops, oracle, n, offset):
    import torch
    rng = np.random.default_rng(n)
    host = [rng.standard_normal(n + offset).astype(F) for _ in range(3)] + [(rng.random(n + offset) * 0.01).astype(F)]
    p0, g, m0, v0 = (a[offset:] for a in host)          # offset > 0: buffers not 16-byte aligned
    dev = [torch.from_numpy(a).cuda()[offset:] for a in host]
    exp = (p0, m0, v0)
    for step in (1, 2, 3):
        ops.adam_update(dev[0], dev[1], dev[2], dev[3], 3e-4, 0.9, 0.95, 1e-8, step, 0.01)
        exp = oracle.adam_update(exp[0], g, exp[1], exp[2], 3e-4, 0.9, 0.95, 1e-8, step, 0.01)
    torch.cuda.synchronize()
    for got, want in zip((dev[0], dev[2], dev[3]), exp):
        assert np.array_equal(got.cpu().numpy(), want)
    ops.sgd_update(dev[0], dev[1], 0.125)
    assert np.array_equal(dev[0].cpu().numpy(), oracle.sgd_update(exp[0], g, 0.125))


@pytest.mark.gpu
def test_gpu_side_optim_validation(ops):
    import torch
    from motifcl_amd.lib import MccError
    a = torch.zeros(8, device="cuda")
    with pytest.raises(MccError, match="step must be positive"):
        ops.adam_update(a, a.clone(), a.clone(), a.clone(), 1e-3, 0.9, 0.999, 1e-8, 0)
    with pytest.raises(MccError, match="shape mismatch"):
        ops.adam_update(a, a.clone()[:4], a.clone(), a.clone(), 1e-3, 0.9, 0.999, 1e-8, 1)
