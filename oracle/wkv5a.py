"""CPU oracle for wkv5a, the RWKV-5 wkv with two-sided decay and bonus (fp32 op).  TEST INFRASTRUCTURE ONLY.

State element [i][j] (i = value/output channel, j = key channel) of head h decays by w1[h,j] * w2[h,i]
per step and the current token enters the output with the bonus u1[h,j] + u2[h,i]
(wkv5a/run.py:164-190, wkv5a_cuda_v1a2.cu:37-61).

Pinned by tests/test_oracle_wkv5a.py: sum form (PYTHON_1) against recurrent form (PYTHON_2); reduction
to the wkv5 oracle when w2 = 1 and u2 = 0; the decay gradients of fp64 autograd against the closed
form of PYTHON_1_BWD; a transposition check that swaps the two sides.
"""

import torch


def decays(w_raw):
    """decay = exp(-exp(w_raw)), wkv5a/run.py:165-167 (and the wrapper's eew, :123-126)."""
    return torch.exp(-torch.exp(w_raw))


def sumform(B, T, C, H, r, k, v, w1, u1, w2, u2):
    """out[b,t,h,i] = sum_j sum_{tt<=t} r[t,j] ww k[tt,j] v[tt,i], ww = u1[j]+u2[i] if tt == t else
    (w1[j] w2[i])**(t-tt-1).  Follows PYTHON_1, wkv5a/run.py:164-190.  w1, w2 are decays [H,N]."""
    N = C // H
    r, k, v = (x.reshape(B, T, H, N) for x in (r, k, v))
    out = torch.zeros(B, T, H, N, dtype=r.dtype)
    W = w2[:, :, None] * w1[:, None, :]                                    # [H,i,j]
    U = u2[:, :, None] + u1[:, None, :]
    for t in range(T):
        for tt in range(t + 1):
            ww = U if tt == t else W ** (t - tt - 1)
            # out[b,h,i] += sum_j r[t,j] ww[i,j] k[tt,j] * v[tt,i]
            out[:, t] += torch.einsum('bhj,hij,bhj->bhi', r[:, t], ww, k[:, tt]) * v[:, tt]
    return out.reshape(B, T, C)


def recurrent(B, T, C, H, r, k, v, w1, u1, w2, u2):
    """Recurrent form: the state enters the output before it is updated.  Follows PYTHON_2,
    wkv5a/run.py:260-289.  w1, w2 are decays; parameters are [H,N] or, for per-batch gradient
    partials, [B,H,N].  Differentiable; dtype follows the inputs."""
    N = C // H
    r, k, v = (x.reshape(B, T, H, N) for x in (r, k, v))
    w1, u1, w2, u2 = (x.reshape(-1, H, N) for x in (w1, u1, w2, u2))
    W = w2[:, :, :, None] * w1[:, :, None, :]                              # [.,H,i,j]
    U = u2[:, :, :, None] + u1[:, :, None, :]
    S = torch.zeros(B, H, N, N, dtype=r.dtype)
    ys = []
    for t in range(T):
        kv = v[:, t, :, :, None] * k[:, t, :, None, :]                     # [B,H,i,j]
        ys.append(((S + U * kv) * r[:, t, :, None, :]).sum(-1))
        S = S * W + kv
    return torch.stack(ys, 1).reshape(B, T, C)


def decay_grads_closed_form(B, T, C, H, r, k, v, w1_raw, w2_raw, gy):
    """gw1_raw[h,j], gw2_raw[h,i] from the definition: the term of (t, tt) carries (w1[j] w2[i])**n with
    n = t-tt-1, whose derivative w.r.t. either raw parameter is n * (-exp(raw)) * (w1 w2)**n.
    Follows PYTHON_1_BWD, wkv5a/run.py:245-254 (whose i/j name the other way round)."""
    N = C // H
    r, k, v, gy = (x.reshape(B, T, H, N) for x in (r, k, v, gy))
    e1, e2 = -torch.exp(w1_raw), -torch.exp(w2_raw)
    W = torch.exp(e2)[:, :, None] * torch.exp(e1)[:, None, :]              # [H,i,j]
    g = torch.zeros(H, N, N, dtype=r.dtype)                                # d loss / d log W[i,j]
    for t in range(T):
        for tt in range(t - 1):
            n = t - tt - 1
            g += n * W ** n * torch.einsum('bhj,bhj,bhi,bhi->hij', r[:, t], k[:, tt], v[:, tt], gy[:, t])
    return e1 * g.sum(1), e2 * g.sum(2)


def grads(B, T, C, H, r, k, v, w1_raw, u1, w2_raw, u2, gy, dtype=torch.float64, per_batch=False):
    """y and (gr, gk, gv, gw1_raw, gu1, gw2_raw, gu2) by autograd through the recurrent form.
    per_batch=True returns the parameter gradients as [B,H,N] partials (what the kernels write
    before the wrapper's sums, wkv5a/run.py:150-153)."""
    N = C // H
    leaf = lambda x: x.detach().to(dtype).clone().requires_grad_(True)
    r_, k_, v_ = (leaf(x) for x in (r, k, v))
    shape = (lambda x: x.reshape(1, H, N).expand(B, H, N)) if per_batch else (lambda x: x.reshape(H, N))
    p = [leaf(shape(x)) for x in (w1_raw, u1, w2_raw, u2)]
    y = recurrent(B, T, C, H, r_, k_, v_, decays(p[0]), p[1], decays(p[2]), p[3])
    y.backward(gy.to(dtype))
    return (y.detach(), r_.grad, k_.grad, v_.grad, p[0].grad, p[1].grad, p[2].grad, p[3].grad)
