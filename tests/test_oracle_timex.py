"""Pins the depthwise_conv1d oracle (CPU only)."""
import torch

from oracle import timex as O
from oracle import err_ratio

D = torch.float64


def test_definition_vs_conv1d_and_impulse():
    B, C, T = 3, 5, 16
    g = torch.Generator().manual_seed(0)
    w = torch.randn(C, T, generator=g, dtype=D)
    k = torch.randn(B, C, T, generator=g, dtype=D)
    a = O.toeplitz_form(w, k, B, C, T, 0.25)
    b = O.conv_form(w, k, B, C, T, 0.25)
    assert err_ratio(a, b) < 1e-14
    u = 5
    imp = torch.zeros(1, C, T, dtype=D)
    imp[:, :, u] = 1.0
    out = O.conv_form(w, imp, 1, C, T, 0.0)
    for t in range(T):
        expect = w[:, T - 1 - (t - u)] if t >= u else torch.zeros(C, dtype=D)
        assert (out[0, :, t] - expect).abs().max() < 1e-14


def test_closed_form_grads_vs_autograd():
    B, C, T = 3, 4, 12
    g = torch.Generator().manual_seed(1)
    w = torch.randn(C, T, generator=g, dtype=D)
    k = torch.randn(B, C, T, generator=g, dtype=D)
    gy = torch.randn(B, C, T, generator=g, dtype=D)
    _, gw, gk = O.grads(w, k, gy, B, C, T)
    gw2, gk2 = O.grads_closed_form(w, k, gy, B, C, T)
    assert err_ratio(gw, gw2.sum(0)) < 1e-13
    assert err_ratio(gk, gk2) < 1e-13
