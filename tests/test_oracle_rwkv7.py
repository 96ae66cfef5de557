"""Pins the rwkv7 state-passing oracle (CPU only)."""
import torch

from oracle import rwkv7 as O
from oracle import err_ratio

D = torch.float64


def _inputs(B, T, H, N, seed=0):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=D)
    r, k, v = rn(B, T, H, N), rn(B, T, H, N), rn(B, T, H, N)
    w = rn(B, T, H, N) + 0.5
    kk = torch.nn.functional.normalize(rn(B, T, H, N), dim=-1)
    a = -kk
    b = kk * torch.sigmoid(rn(B, T, H, N))
    s0 = rn(B, H, N, N)
    dy = rn(B, T, H, N)
    dsT = rn(B, H, N, N)
    return s0, r, w, k, v, a, b, dy, dsT


def test_decay_forms_agree_and_range():
    x = torch.linspace(-20, 20, 401, dtype=D)
    assert (O.decay_sigmoid(x) - O.decay_softplus(x)).abs().max() < 1e-14
    assert O.decay_sigmoid(x).min() > 0.545 and O.decay_sigmoid(x).max() <= 1.0


def test_step_form_vs_matrix_products():
    s0, r, w, k, v, a, b, _, _ = _inputs(2, 5, 2, 4, 1)
    y1, s1 = O.recurrent(s0, r, w, k, v, a, b)
    y2, s2 = O.matrix_product_form(s0, r, w, k, v, a, b)
    assert err_ratio(y2, y1) < 1e-13 and err_ratio(s2, s1) < 1e-13
    # a and b are not interchangeable, and sa uses the state BEFORE the update
    y3, _ = O.recurrent(s0, r, w, k, v, b, a)
    assert err_ratio(y1, y3) > 1e-2


def test_unit_decay_no_delta_is_linear_attention():
    s0, r, w, k, v, a, b, _, _ = _inputs(2, 9, 2, 4, 2)
    z = torch.zeros_like(a)
    y, _ = O.recurrent(torch.zeros_like(s0), r, torch.full_like(w, -1e4), k, v, z, z)
    kv = torch.cumsum(v[..., :, None] * k[..., None, :], dim=1)
    y2 = (kv * r[..., None, :]).sum(-1)
    assert err_ratio(y2, y) < 1e-13


def test_chained_calls_equal_one_call():
    args = _inputs(2, 16, 2, 4, 3)
    one = O.grads(*args)
    four = O.grads(*args, splits=4)
    for x, y in zip(one, four):
        assert err_ratio(x, y) < 1e-12


def test_hand_backward_vs_autograd():
    args = _inputs(2, 32, 2, 4, 4)
    ref = O.grads(*args)
    for invert in (False, True):
        out = O.backward_hand(*args, invert=invert, chunk_len=16)
        for x, y in zip(ref, out):
            assert err_ratio(x, y) < (1e-9 if invert else 1e-12)


def test_emulator_close_to_fp64():
    args = _inputs(2, 32, 2, 8, 5)
    q = [x.to(torch.bfloat16) if i not in (0, 8) else x.float() for i, x in enumerate(args)]
    ref = O.grads(*q)
    emu = O.emulate_bf16(*q)
    for x, y in zip(ref, emu):
        assert err_ratio(x, y.double()) < 6e-3
