"""Pins the wkv5a oracle (CPU only): each check fails for a plausible mistake (the two sides swapped,
bonus applied to the state, decay applied before the read-out, a dropped factor in the decay gradient)."""
import torch

from oracle import wkv5a as A
from oracle import wkv56 as O
from oracle import err_ratio

D = torch.float64


def _inputs(B, T, H, N, seed):
    g = torch.Generator().manual_seed(seed)
    C = H * N
    u = lambda *s, lo=-1.0, hi=1.0: torch.rand(*s, generator=g, dtype=D) * (hi - lo) + lo
    r, k, v, gy = u(B, T, C), u(B, T, C), u(B, T, C), u(B, T, C)
    w1, w2 = u(H, N, lo=-3.0), u(H, N, lo=-3.0)                # raw; the reference draws uniform(-8, 1)
    return C, r, k, v, w1, u(H, N), w2, u(H, N), gy


def test_sum_form_vs_recurrent_form():
    B, T, H, N = 2, 6, 2, 4
    C, r, k, v, w1, u1, w2, u2, _ = _inputs(B, T, H, N, 1)
    y1 = A.sumform(B, T, C, H, r, k, v, A.decays(w1), u1, A.decays(w2), u2)
    y2 = A.recurrent(B, T, C, H, r, k, v, A.decays(w1), u1, A.decays(w2), u2)
    assert err_ratio(y1, y2) < 1e-13


def test_reduces_to_wkv5_when_the_second_side_is_neutral():
    B, T, H, N = 2, 9, 2, 4
    C, r, k, v, w1, u1, _, _, gy = _inputs(B, T, H, N, 2)
    one, zero = torch.ones(H, N, dtype=D), torch.zeros(H, N, dtype=D)
    y = A.recurrent(B, T, C, H, r, k, v, A.decays(w1), u1, one, zero)
    y5, _ = O.wkv_recurrent(B, T, C, H, r, k, v, A.decays(w1), u1)
    assert err_ratio(y5, y) < 1e-13
    # raw w2 = -40 is a decay of exactly 1 in fp64: the gradients of the first side are wkv5's
    g = A.grads(B, T, C, H, r, k, v, w1, u1, torch.full((H, N), -40.0, dtype=D), zero, gy)
    g5 = O.wkv5_grads(B, T, C, H, r, k, v, w1, u1, gy)
    for a, b in zip(g5, g[:6]):
        assert err_ratio(a, b) < 1e-12


def test_the_two_sides_are_not_interchangeable():
    B, T, H, N = 1, 5, 1, 4
    C, r, k, v, w1, u1, w2, u2, _ = _inputs(B, T, H, N, 3)
    y = A.recurrent(B, T, C, H, r, k, v, A.decays(w1), u1, A.decays(w2), u2)
    y_swapped = A.recurrent(B, T, C, H, r, k, v, A.decays(w2), u2, A.decays(w1), u1)
    assert err_ratio(y, y_swapped) > 1e-2
    # side 2 indexes the output channel: scaling u2[i0] moves only y[..., i0]; side 1 moves every channel
    u2b = u2.clone(); u2b[0, 1] += 1.0
    dy = (A.recurrent(B, T, C, H, r, k, v, A.decays(w1), u1, A.decays(w2), u2b) - y).reshape(B, T, H, N)
    assert float(dy[..., 1].abs().max()) > 1e-3 and float(dy[..., [0, 2, 3]].abs().max()) == 0.0
    u1b = u1.clone(); u1b[0, 1] += 1.0
    dy = (A.recurrent(B, T, C, H, r, k, v, A.decays(w1), u1b, A.decays(w2), u2) - y).reshape(B, T, H, N)
    assert float(dy.abs().amax(dim=(0, 1, 2)).min()) > 1e-4


def test_decay_gradients_match_the_closed_form():
    B, T, H, N = 2, 7, 2, 3
    C, r, k, v, w1, u1, w2, u2, gy = _inputs(B, T, H, N, 4)
    g = A.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy)
    gw1, gw2 = A.decay_grads_closed_form(B, T, C, H, r, k, v, w1, w2, gy)
    assert err_ratio(gw1, g[4]) < 1e-12
    assert err_ratio(gw2, g[6]) < 1e-12


def test_bonus_gradients_closed_form_and_batch_partials():
    B, T, H, N = 3, 5, 2, 4
    C, r, k, v, w1, u1, w2, u2, gy = _inputs(B, T, H, N, 5)
    g = A.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy)
    r4, k4, v4, g4 = (x.reshape(B, T, H, N) for x in (r, k, v, gy))
    vg = (v4 * g4).sum(-1, keepdim=True)                     # sum_i v gy
    rk = (r4 * k4).sum(-1, keepdim=True)                     # sum_j r k
    assert err_ratio((r4 * k4 * vg).sum((0, 1)), g[5]) < 1e-12          # gu1, wkv5a/run.py:241
    assert err_ratio((v4 * g4 * rk).sum((0, 1)), g[7]) < 1e-12          # gu2, wkv5a/run.py:243
    gp = A.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy, per_batch=True)
    for a, b in zip(g[4:], gp[4:]):
        assert b.shape == (B, H, N) and err_ratio(a, b.sum(0)) < 1e-12
