"""Pins the wkv4 oracle (CPU only)."""
import torch

from oracle import wkv4 as O
from oracle import err_ratio, max_rel_to_peak

D = torch.float64


def _inputs(B, T, C, seed=0):
    g = torch.Generator().manual_seed(seed)
    w_raw = torch.randn(C, generator=g, dtype=D) * 0.5
    u = torch.randn(C, generator=g, dtype=D) * 0.5
    k = torch.randn(B, T, C, generator=g, dtype=D).clamp(-8, 8)
    v = torch.randn(B, T, C, generator=g, dtype=D)
    gy = torch.randn(B, T, C, generator=g, dtype=D)
    return w_raw, u, k, v, gy


def test_three_forms_agree():
    B, T, C = 2, 17, 6
    w_raw, u, k, v, gy = _inputs(B, T, C, 1)
    y1 = O.sumform(B, T, C, w_raw, u, k, v)
    y2 = O.conv_form(B, T, C, w_raw, u, k, v)
    y3 = O.streaming(B, T, C, -torch.exp(w_raw), u, k, v)
    assert max_rel_to_peak(y1, y2) < 1e-12
    assert max_rel_to_peak(y1, y3) < 1e-12
    # dropping the bonus or mis-timing the decay must show
    y4 = O.streaming(B, T, C, -torch.exp(w_raw), torch.zeros_like(u), k, v)
    assert max_rel_to_peak(y1, y4) > 1e-3


def test_invariants():
    B, T, C = 2, 33, 5
    w_raw, u, k, v, gy = _inputs(B, T, C, 2)
    w = -torch.exp(w_raw)
    y = O.streaming(B, T, C, w, u, k, v)
    assert (y[:, 0] - v[:, 0]).abs().max() < 1e-14                      # y_0 = v_0
    cmax = torch.cummax(v, 1).values
    cmin = torch.cummin(v, 1).values
    assert (y <= cmax + 1e-12).all() and (y >= cmin - 1e-12).all()      # convex combination of v_{<=t}
    y2 = O.streaming(B, T, C, w, u, k + 3.7, v)
    assert (y - y2).abs().max() < 1e-12                                 # shift invariance in k
    g = torch.Generator().manual_seed(5)
    kbig = (torch.rand(B, T, C, generator=g, dtype=D) * 2000 - 1000).float()
    ybig = O.streaming(B, T, C, w.float(), u.float(), kbig, v.float())  # wkv/run.py:159-169
    assert torch.isfinite(ybig).all()


def test_kernel_order_backward_vs_autograd():
    B, T, C = 3, 40, 7
    w_raw, u, k, v, gy = _inputs(B, T, C, 3)
    y, gw, gu, gk, gv = O.grads(B, T, C, w_raw, u, k, v, gy)
    # autograd through the overflow-free definition is the anchor
    leaves = [x.clone().requires_grad_(True) for x in (w_raw, u, k, v)]
    O.sumform(B, T, C, *leaves).backward(gy)
    for a, b in zip(leaves, (gw, gu, gk, gv)):
        assert err_ratio(a.grad, b) < 1e-11
    hw, hu, hk, hv = O.backward_kernel_order(B, T, C, -torch.exp(w_raw), u, k, v, gy)
    # the kernel's gw is d/dw_raw up to the chain-rule factor it includes: gw_raw = w * dL/dw
    assert err_ratio(gw, hw.sum(0)) < 1e-11
    assert err_ratio(gu, hu.sum(0)) < 1e-11
    assert err_ratio(gk, hk) < 1e-11
    assert err_ratio(gv, hv) < 1e-11
    yp, gwp, gup, _, _ = O.grads(B, T, C, w_raw, u, k, v, gy, per_batch=True)
    assert err_ratio(hw, gwp) < 1e-11 and err_ratio(hu, gup) < 1e-11
