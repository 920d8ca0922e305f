"""Fused optimizer updates on the GPU against the float64 oracle (itself pinned to
torch.optim in tests/test_oracle.py).  Elementwise fp32 arithmetic of about ten operations:
held to rtol 1e-5 / atol 1e-7 per step, over several steps with moments carried on the
device."""
import numpy as np
import pytest

from helpers import assert_close, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import F32, AnyBuffer, MogradError  # noqa: E402

RTOL, ATOL = 1e-5, 1e-7


@pytest.mark.parametrize("decoupled,wd", [(0, 0.0), (0, 0.1), (1, 0.1), (1, 0.0)])
@pytest.mark.parametrize("n", [1, 5, 1024, 100003])
def test_adam_steps(device, decoupled, wd, n):
    lib, st = device.lib, device.stream
    # the library receives fp32 hyper-parameters; the oracle gets the same rounded values
    # (1 - beta2 evaluated from 0.999 and from float32(0.999) differ by 5e-5 relative)
    lr, b1, b2, eps, wd = (float(np.float32(h)) for h in (3e-3, 0.9, 0.999, 1e-8, wd))
    w = normal(80, 0, (n,))
    bw = AnyBuffer.from_numpy(device, w)
    bm = AnyBuffer.create(F32, device, n, fill=0.0)
    bv = AnyBuffer.create(F32, device, n, fill=0.0)
    ow, om, ov = w.astype(np.float64), np.zeros(n), np.zeros(n)
    for t, scale in enumerate((1.0, 0.1, 3.0, 1e-3), start=1):
        g = normal(80, t, (n,), std=scale)
        bg = AnyBuffer.from_numpy(device, g)
        lib.mg_adam_step(bw.data_ptr(), bg.data_ptr(), bm.data_ptr(), bv.data_ptr(), n, lr, b1, b2, eps, wd, t, decoupled, st)
        ow, om, ov = O.adam_step(ow, g, om, ov, lr, b1, b2, eps, wd, t, bool(decoupled))
        assert_close(bw.to_numpy(), ow, RTOL, ATOL, f"w step {t}")
        assert_close(bm.to_numpy(), om, RTOL, ATOL, f"m step {t}")
        assert_close(bv.to_numpy(), ov, RTOL, 1e-9, f"v step {t}")


def test_adam_first_step_moves_by_lr(device):
    # closed form: with m = v = 0 and t = 1, m_hat = g and v_hat = g^2, so the first update is
    # lr * g / (|g| + eps) = lr * sign(g) for any gradient scale
    n, lr = 4096, 1e-2
    w = normal(81, 0, (n,))
    g = normal(81, 1, (n,)) * 10.0 ** normal(81, 2, (n,))
    bw, bg = AnyBuffer.from_numpy(device, w), AnyBuffer.from_numpy(device, g)
    bm, bv = AnyBuffer.create(F32, device, n, fill=0.0), AnyBuffer.create(F32, device, n, fill=0.0)
    device.lib.mg_adam_step(bw.data_ptr(), bg.data_ptr(), bm.data_ptr(), bv.data_ptr(), n, lr, 0.9, 0.999, 1e-12, 0.0, 1,
                            0, device.stream)
    np.testing.assert_allclose(bw.to_numpy() - w, -lr * np.sign(g), rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("t", [100_000, 1_000_000])
def test_adam_late_steps(device, t):
    # Far into training: the bias corrections 1 - beta**t must still be the fp32 rounding of
    # the exact power (0.999**100000 = 3.5e-44 is still a nonzero fp32 denormal), and a call
    # must not cost host time in proportion to t.
    import time

    lib, st = device.lib, device.stream
    n = 4096
    lr, b1, b2, eps = (float(np.float32(h)) for h in (3e-3, 0.9, 0.999, 1e-8))
    w, g, m, v = normal(83, 0, (n,)), normal(83, 1, (n,)), normal(83, 2, (n,), std=0.1), np.abs(normal(83, 3, (n,), std=0.1))
    bw, bg, bm, bv = (AnyBuffer.from_numpy(device, a) for a in (w, g, m, v))
    lib.mg_adam_step(bw.data_ptr(), bg.data_ptr(), bm.data_ptr(), bv.data_ptr(), n, lr, b1, b2, eps, 0.0, t, 0, st)
    ow, om, ov = O.adam_step(w, g, m, v, lr, b1, b2, eps, 0.0, t, False)
    assert_close(bw.to_numpy(), ow, RTOL, ATOL, "w")
    assert_close(bm.to_numpy(), om, RTOL, ATOL, "m")

    def host_seconds(step):
        device.synchronize()
        t0 = time.perf_counter()
        for _ in range(200):
            lib.mg_adam_step(bw.data_ptr(), bg.data_ptr(), bm.data_ptr(), bv.data_ptr(), n, lr, b1, b2, eps, 0.0, step, 0, st)
        dt = time.perf_counter() - t0
        device.synchronize()
        return dt

    host_seconds(1)
    early, late = host_seconds(1), host_seconds(t)
    assert late < 3 * early + 2e-3, f"200 calls: {early * 1e3:.2f} ms at t=1, {late * 1e3:.2f} ms at t={t}"


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_sgd_step(device, n):
    w, g = normal(82, 0, (n,)), normal(82, 1, (n,))
    bw, bg = AnyBuffer.from_numpy(device, w), AnyBuffer.from_numpy(device, g)
    device.lib.mg_sgd_step(bw.data_ptr(), bg.data_ptr(), n, 0.05, device.stream)
    # one multiply and one subtract in fp32: the same two roundings as numpy's
    np.testing.assert_array_equal(bw.to_numpy(), w - g * np.float32(0.05))


def test_optim_errors(device):
    b = AnyBuffer.create(F32, device, 8)
    p = b.data_ptr()
    with pytest.raises(MogradError, match="t=0"):
        device.lib.mg_adam_step(p, p, p, p, 8, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, 0, device.stream)
    with pytest.raises(MogradError, match="null pointer"):
        device.lib.mg_sgd_step(p, None, 8, 0.1, device.stream)
