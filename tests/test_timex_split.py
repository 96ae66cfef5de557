"""CPU: the arithmetic of the depthwise_conv1d matrix-core kernels (csrc/timex.hip), restated in numpy.

Every fp32 operand x is carried as two fp16 terms after a power of two per unit, x 2^s = h + l, and a product as
h h' + h l' + l h' in fp32.  What the kernels' comments claim about this scheme is checked here on the CPU: the scale puts
the unit's largest magnitude in [2^14, 2^15) and is an exact power of two; the two terms reproduce an operand to 2^-22 of
its size or 2^-25 absolute (fp16's subnormal spacing), whichever is larger; a sum of such products against fp64 has the
error of an fp32 loop, also when the rows of a unit differ in size by 1e4."""
import numpy as np
import pytest


def scale_for(m):
    """2^s with m 2^s in [2^14, 2^15) (s = 0 for zero, subnormal or infinite m; |s| <= 100), as scale_for in timex.hip."""
    bits = np.float32(m).view(np.uint32)
    e = int((bits >> 23) & 255)
    s = max(-100, min(100, 14 + 127 - e))
    if e == 0 or e == 255:
        s = 0
    return np.float32(2.0) ** np.float32(s), np.float32(2.0) ** np.float32(-s)


def split2(x, up):
    """h, l of x * up: nearest fp16, then the nearest fp16 of the exact remainder (split2x4 in timex.hip)."""
    xs = (x.astype(np.float32) * up).astype(np.float32)
    h = xs.astype(np.float16)
    l = (xs - h.astype(np.float32)).astype(np.float16)
    return xs, h, l


@pytest.mark.parametrize("m", [1.0, 3.7, 65504.0, 1e-3, 2.5e6, 7e-30, 3e30])
def test_scale_is_a_power_of_two_and_lands_in_range(m):
    up, down = scale_for(m)
    assert up * down == 1.0
    assert float(np.log2(up)) == round(float(np.log2(up)))
    if 2.0 ** -86 < m < 2.0 ** 114:             # (beyond, the shift is clamped to 100 places)
        assert 2.0 ** 14 <= m * float(up) < 2.0 ** 15


def test_scale_of_zero_subnormal_and_infinite_is_one():
    for m in (0.0, 1e-45, float("inf")):
        assert scale_for(m) == (1.0, 1.0)


def test_two_terms_reproduce_an_operand():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * 10.0 ** rng.uniform(-6, 0, 20000)).astype(np.float32)
    up, _ = scale_for(np.abs(x).max())
    xs, h, l = split2(x, up)
    assert np.all(np.isfinite(h.astype(np.float32)))
    err = np.abs(xs.astype(np.float64) - h.astype(np.float64) - l.astype(np.float64))
    assert np.all(err <= np.maximum(2.0 ** -22 * np.abs(xs), 2.0 ** -25))


@pytest.mark.parametrize("spread", [0.0, 4.0])
def test_convolution_error_is_that_of_an_fp32_loop(spread):
    """One channel, 32 batch rows of a unit (sizes 10^-spread .. 1 apart), T = 256: x[b,t] = sum_u w[T-1-(t-u)] k[b,u]."""
    rng = np.random.default_rng(1)
    B, T = 32, 256
    k = (rng.standard_normal((B, T)) * 10.0 ** (-spread * rng.random((B, 1)))).astype(np.float32)
    w = (rng.standard_normal(T) * 3e5).astype(np.float32)
    W = np.zeros((T, T))
    for t in range(T):
        W[t, :t + 1] = [w[T - 1 - (t - u)] for u in range(t + 1)]
    ref = k.astype(np.float64) @ W.T
    upk, dnk = scale_for(np.abs(k).max())
    upw, dnw = scale_for(np.abs(w).max())
    _, kh, kl = split2(k, upk)
    _, wh, wl = split2(w, upw)
    Wh, Wl = np.zeros((T, T), np.float32), np.zeros((T, T), np.float32)
    for t in range(T):
        for u in range(t + 1):
            Wh[t, u] = wh[T - 1 - (t - u)]
            Wl[t, u] = wl[T - 1 - (t - u)]
    f32 = np.float32
    got = (kh.astype(f32) @ Wh.T + (kh.astype(f32) @ Wl.T + kl.astype(f32) @ Wh.T)) * f32(dnk * dnw)
    for b in range(B):                          # every batch row on the bar of the fp32 operators by itself
        e = np.sqrt(np.mean((got[b].astype(np.float64) - ref[b]) ** 2) / np.mean(ref[b] ** 2))
        assert e <= 1e-5, (b, e)
    e_all = np.sqrt(np.mean((got.astype(np.float64) - ref) ** 2) / np.mean(ref ** 2))
    assert e_all <= 5e-7
