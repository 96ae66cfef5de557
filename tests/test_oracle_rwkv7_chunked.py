"""The chunked (matrix-product) form of the RWKV-7 recurrence, oracle/rwkv7_chunked.py, against the step form
(oracle/rwkv7.py, which follows rwkv7_cuda_benchmark_state_passing.py:46-68) and fp64 autograd.  CPU only."""
import pytest
import torch

from oracle import rwkv7 as O
from oracle import rwkv7_chunked as C

DT = torch.float64


def _inputs(B, T, H, N, seed, w_shift=0.5):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=DT)
    r, k, v = (0.5 * rn(B, T, H, N) for _ in range(3))
    w = rn(B, T, H, N) + w_shift
    kk = torch.nn.functional.normalize(rn(B, T, H, N), dim=-1)
    a, b = -kk, kk * torch.sigmoid(rn(B, T, H, N))
    s0 = 0.1 * rn(B, H, N, N)
    return s0, r, w, k, v, a, b, rn(B, T, H, N), rn(B, H, N, N)


@pytest.mark.parametrize("L", [4, 16, 32])
def test_forward_equals_step_form_and_saves_what_the_reference_saves(L):
    s0, r, w, k, v, a, b, _, _ = _inputs(2, 64, 2, 8, seed=1)
    y, sT, sa, chk = C.forward(s0, r, w, k, v, a, b, chunk_len=L)
    y_ref, sT_ref = O.recurrent(s0, r, w, k, v, a, b)
    assert torch.allclose(y, y_ref, rtol=0, atol=1e-12)
    assert torch.allclose(sT, sT_ref, rtol=0, atol=1e-12)
    # sa_t = S_t a_t and the state at the end of every chunk, step by step
    S = s0
    wd = O.decay_sigmoid(w)
    for t in range(r.shape[1]):
        sat = torch.einsum('bhij,bhj->bhi', S, a[:, t])
        assert torch.allclose(sa[:, t], sat, rtol=0, atol=1e-12)
        S = S * wd[:, t, :, None, :] + sat[..., :, None] * b[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :]
        if (t + 1) % L == 0:
            assert torch.allclose(chk[:, :, t // L], S, rtol=0, atol=1e-12)


@pytest.mark.parametrize("L,w_shift", [(16, 0.5), (8, -3.0), (16, 6.0)])
def test_backward_equals_autograd(L, w_shift):
    args = _inputs(2, 48, 2, 8, seed=2, w_shift=w_shift)
    ref = O.grads(*args)
    out = C.backward(*args, chunk_len=L)
    for name, x, z in zip(("y", "sT", "ds0", "dr", "dw", "dk", "dv", "da", "db"), out, ref):
        assert torch.allclose(x, z, rtol=0, atol=1e-11 * max(1.0, float(z.abs().max()))), name


def test_backward_without_incoming_state_gradient_and_from_zero_state():
    s0, r, w, k, v, a, b, dy, dsT = _inputs(1, 32, 3, 16, seed=3)
    z = torch.zeros_like
    ref = O.grads(z(s0), r, w, k, v, a, b, dy, z(dsT))
    out = C.backward(z(s0), r, w, k, v, a, b, dy, z(dsT), chunk_len=16)
    for x, y in zip(out, ref):
        assert torch.allclose(x, y, rtol=0, atol=1e-11)


def test_factors_stay_bounded_at_the_clamp():
    """The clamp keeps every in-chunk factor within e^{+-0.607 L/2}: the form is safe in bf16 / fp16 ranges for L = 16."""
    lam = torch.full((1, 1, 16, 4), O.W_SCALE, dtype=DT)          # the fastest decay the clamp allows, every step
    ea, er, eb, d1, d2, dec = C._factors(lam)
    bound = torch.exp(torch.tensor(-O.W_SCALE * 8, dtype=DT))
    for f in (ea, er, eb, d1, d2):
        assert float(f.max()) <= float(bound) * (1 + 1e-12) and float(f.min()) >= 1 / float(bound) * (1 - 1e-12)
