"""CPU oracle: RWKV-4 wkv, fp32 op (TEST INFRASTRUCTURE, not product code).

For one (b, c), with w = -exp(w_raw) < 0 the per-step log-decay and u the bonus:
    y_t = (sum_{s<t} e^{(t-1-s) w + k_s} v_s + e^{u + k_t} v_t) / (sum_{s<t} e^{(t-1-s) w + k_s} + e^{u + k_t})

Pinning (tests/test_oracle_wkv4.py): the definition in log-sum-exp form vs the grouped
F.conv1d formulation (a library routine) vs the streaming form with a running maximum;
y_0 = v_0; y is a convex combination of v_{<=t}; adding a constant to every k changes nothing;
k ~ U(-1000,1000) stays finite in the streaming form; the kernel-order backward vs fp64 autograd.
"""

import torch
import torch.nn.functional as F


def sumform(B, T, C, w_raw, u, k, v):
    """The definition (RUN_FORMULA_VERY_SLOW, wkv/run.py:46-63), vectorised over (b,c) with the
    exponentials taken through a softmax over s so that it cannot overflow.  O(T^2) memory: small shapes."""
    w = -torch.exp(w_raw)                                        # [C]
    t = torch.arange(T)
    d = (t[:, None] - 1 - t[None, :]).to(k.dtype)                # (t-1-s)
    logit = d[None, :, :, None] * w[None, None, None, :] + k[:, None, :, :]          # [B,t,s,C]
    diag = (u[None, None, :] + k)                                                    # s == t term
    logit = torch.where((t[:, None] > t[None, :])[None, :, :, None], logit, torch.full_like(logit, -float('inf')))
    eye = (t[:, None] == t[None, :])[None, :, :, None]
    logit = torch.where(eye, diag[:, :, None, :].expand(B, T, T, C), logit)
    p = torch.softmax(logit, dim=2)
    return (p * v[:, None, :, :]).sum(2)


def conv_form(B, T, C, w_raw, u, k, v):
    """wkv = conv(e^k v) / conv(e^k) with the causal kernel [.., e^{2w}, e^{w}, 1, e^{u}] per channel,
    by grouped F.conv1d.  Follows RUN_PYTORCH, wkv/run.py:66-78 (its time_curve is -(T-2)..0).
    Not overflow-safe: moderate k only."""
    ek = torch.exp(k.transpose(1, 2))
    ekv = ek * v.transpose(1, 2)
    curve = torch.arange(-(T - 2), 1, dtype=k.dtype)[None, :]                        # [1,T-1]
    time_w = torch.cat([torch.exp(w_raw)[:, None] * curve, u[:, None]], dim=-1)      # [C,T]
    kern = torch.exp(time_w)[:, None, :]
    wkv = F.conv1d(F.pad(ekv, (T - 1, 0)), kern, groups=C)
    wk = F.conv1d(F.pad(ek, (T - 1, 0)), kern, groups=C)
    return (wkv / wk).transpose(1, 2)


def streaming(B, T, C, w, u, k, v):
    """Streaming form with running maximum o; `w` is already -exp(w_raw).
    Follows kernel_forward, wkv/cuda/wkv_cuda_v2.cu:20-37.  Differentiable."""
    p = torch.zeros(B, C, dtype=k.dtype)
    q = torch.zeros(B, C, dtype=k.dtype)
    o = torch.full((B, C), -65500.0, dtype=k.dtype)
    ys = []
    for t in range(T):
        kt, vt = k[:, t], v[:, t]
        no = torch.maximum(o, u + kt)
        A = torch.exp(o - no)
        Bq = torch.exp(u + kt - no)
        ys.append((A * p + Bq * vt) / (A * q + Bq))
        no = torch.maximum(w + o, kt)
        A = torch.exp(w + o - no)
        Bq = torch.exp(kt - no)
        p = A * p + Bq * vt
        q = A * q + Bq
        o = no
    return torch.stack(ys, 1)


def grads(B, T, C, w_raw, u, k, v, gy, dtype=torch.float64, per_batch=False):
    """y and (gw_raw, gu, gk, gv) by autograd through the streaming form.  per_batch=True returns
    gw, gu as the [B,C] partials the kernel accumulates (wkv/run.py:110-116)."""
    k_, v_ = (x.detach().to(dtype).clone().requires_grad_(True) for x in (k, v))
    if per_batch:
        w_ = w_raw.detach().to(dtype)[None].expand(B, C).clone().requires_grad_(True)
        u_ = u.detach().to(dtype)[None].expand(B, C).clone().requires_grad_(True)
    else:
        w_, u_ = (x.detach().to(dtype).clone().requires_grad_(True) for x in (w_raw, u))
    y = streaming(B, T, C, -torch.exp(w_), u_, k_, v_)
    y.backward(gy.to(dtype))
    zero = lambda x: torch.zeros_like(x) if x.grad is None else x.grad      # T == 1: w never reaches y
    return y.detach(), zero(w_), zero(u_), zero(k_), zero(v_)


def backward_kernel_order(B, T, C, w, u, k, v, gy):
    """Two-sweep hand backward.  Follows kernel_backward, wkv/cuda/wkv_cuda_v2.cu:40-114: the
    ascending sweep keeps y_t, z_t = 1/den_t, zexp_t and accumulates gw, gu; the descending sweep
    carries (gp, gq, o).  `w` is -exp(w_raw); returned gw carries the factor w (:112).
    Returns per-batch gw[B,C], gu[B,C], gk, gv."""
    dt = k.dtype
    p = torch.zeros(B, C, dtype=dt); q = torch.zeros(B, C, dtype=dt)
    dpdw = torch.zeros(B, C, dtype=dt); dqdw = torch.zeros(B, C, dtype=dt)
    o = torch.full((B, C), -65500.0, dtype=dt)
    gw = torch.zeros(B, C, dtype=dt); gu = torch.zeros(B, C, dtype=dt)
    ys, zs, zexps = [], [], []
    for t in range(T):
        kt, vt, gt = k[:, t], v[:, t], gy[:, t]
        no = torch.maximum(o, kt + u)
        A = torch.exp(o - no)
        Bq = torch.exp(kt + u - no)
        num = A * p + Bq * vt
        iden = 1 / (A * q + Bq)
        y = num * iden
        ys.append(y); zs.append(iden); zexps.append(kt + u - no)
        gw = gw + gt * (dpdw - dqdw * y) * iden * A
        gu = gu + gt * (vt - y) * Bq * iden
        no = torch.maximum(w + o, kt)
        A = torch.exp(w + o - no)
        Bq = torch.exp(kt - no)
        dpdw = A * (p + dpdw)
        dqdw = A * (q + dqdw)
        p = A * p + Bq * vt
        q = A * q + Bq
        o = no
    gp = torch.zeros(B, C, dtype=dt); gq = torch.zeros(B, C, dtype=dt)
    o = torch.full((B, C), -65500.0, dtype=dt)
    gk = torch.empty_like(k); gv = torch.empty_like(k)
    for t in range(T - 1, -1, -1):
        kt, vt, gt = k[:, t], v[:, t], gy[:, t]
        A = gt * zs[t] * torch.exp(zexps[t])
        Bq = torch.exp(kt + o)
        gk[:, t] = A * (vt - ys[t]) + Bq * (gp * vt + gq)
        gv[:, t] = A + Bq * gp
        no = torch.maximum(w + o, zexps[t] - kt - u)
        A = torch.exp(w + o - no)
        Bq = gt * zs[t] * torch.exp(zexps[t] - kt - u - no)
        gp = A * gp + Bq
        gq = A * gq - Bq * ys[t]
        o = no
    return gw * w, gu, gk, gv
