"""CPU oracle: depthwise_conv1d / "TimeX" (TEST INFRASTRUCTURE, not product code).

    out[b,c,t] = eps + sum_{u<=t} w[c, T-1-(t-u)] * k[b,c,u]

Pinning (tests/test_oracle_timex.py): the definition as an explicit lower-triangular Toeplitz
matrix product vs the zero-padded grouped F.conv1d (a library routine); impulse response
(k = delta_u gives out[t] = w[T-1-(t-u)]); closed-form gradients vs autograd.
"""

import torch
import torch.nn.functional as F


def toeplitz_form(w, k, B, C, T, eps):
    """The definition (README.md:12-18; RUN_FORMULA_VERY_SLOW, depthwise_conv1d/run.py:45-55):
    M_c[t,u] = w[c, T-1-(t-u)] for u <= t, out = eps + M k."""
    t = torch.arange(T)
    idx = (T - 1) - (t[:, None] - t[None, :])
    M = torch.where((t[:, None] >= t[None, :])[None], w[:, idx.clamp(0, T - 1)], torch.zeros((), dtype=w.dtype))
    return eps + torch.einsum('ctu,bcu->bct', M, k)


def conv_form(w, k, B, C, T, eps):
    """Zero-padded grouped conv.  Follows RUN_PYTORCH, depthwise_conv1d/run.py:58-60."""
    return F.conv1d(F.pad(k, (T - 1, 0)), w.unsqueeze(1), groups=C) + eps


def grads_closed_form(w, k, g, B, C, T):
    """gk[b,c,u] = sum_{t>=u} w[c,T-1-(t-u)] g[b,c,t];  gw[b,c,T-1-d] = sum_u g[b,c,u+d] k[b,c,u]
    (per batch, as the kernels write it).  Follows kernel_backward, timex_cuda_v0.cu:28-44."""
    t = torch.arange(T)
    idx = (T - 1) - (t[:, None] - t[None, :])
    M = torch.where((t[:, None] >= t[None, :])[None], w[:, idx.clamp(0, T - 1)], torch.zeros((), dtype=w.dtype))
    gk = torch.einsum('ctu,bct->bcu', M, g)
    gw = torch.zeros(B, C, T, dtype=w.dtype)
    for d in range(T):
        gw[:, :, T - 1 - d] = (g[:, :, d:] * k[:, :, :T - d]).sum(-1)
    return gw, gk


def grads(w, k, g, B, C, T, dtype=torch.float64):
    """out, gw (summed over B), gk by autograd through the conv form."""
    w_ = w.detach().to(dtype).clone().requires_grad_(True)
    k_ = k.detach().to(dtype).clone().requires_grad_(True)
    out = conv_form(w_, k_, B, C, T, 0.0)
    out.backward(g.to(dtype))
    return out.detach(), w_.grad, k_.grad
