"""CPU oracle: RWKV-7 "clamp-w" generalised delta rule with state passing
(TEST INFRASTRUCTURE, not product code).

    w_t     = exp(-e^{-0.5} * sigmoid(w_raw_t))                       decay in (0.545, 1)
    sa_t    = S_t a_t                                                  S[b,h,i,j], i = value, j = key
    S_{t+1} = S_t diag(w_t) + sa_t b_t^T + v_t k_t^T
    y_t     = S_{t+1} r_t                                              (post-update state, no bonus)
    sT      = S_T

Pinning (tests/test_oracle_rwkv7.py): the step form vs an explicit product of the matrices
M_t = diag(w_t) + a_t b_t^T (torch.matmul on tiny shapes); the sigmoid form of the decay vs
the reference's softplus form; w = 1, a = b = 0 vs cumsum linear attention; four chained
T/4 calls vs one T call (outputs and every gradient); the hand-derived backward vs fp64 autograd.
"""

import math

import torch

W_SCALE = -math.exp(-0.5)   # rwkv7_statepassing_clampw.cu:16


def decay_sigmoid(w_raw):
    """Kernel form: exp(W_SCALE * sigmoid(w_raw)).  Follows rwkv7_statepassing_clampw.cu:45."""
    return torch.exp(W_SCALE * torch.sigmoid(w_raw))


def decay_softplus(w_raw):
    """Python-reference form: w = -softplus(-w_raw) - 0.5; exp(-exp(w)).
    Follows rwkv7_cuda_benchmark_state_passing.py:53-54."""
    return torch.exp(-torch.exp(-torch.nn.functional.softplus(-w_raw) - 0.5))


def recurrent(s0, r, w_raw, k, v, a, b):
    """Step form.  Follows RWKV7_STATE_PASSING_CLAMPW_REF,
    rwkv7_cuda_benchmark_state_passing.py:46-68.  Tensors [B,T,H,N]; s0 [B,H,N,N].
    Returns (y[B,T,H,N], sT)."""
    B, T, H, N = r.shape
    w = decay_sigmoid(w_raw)
    S = s0
    ys = []
    for t in range(T):
        sa = torch.einsum('bhij,bhj->bhi', S, a[:, t])
        S = S * w[:, t, :, None, :] + sa[..., :, None] * b[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :]
        ys.append(torch.einsum('bhij,bhj->bhi', S, r[:, t]))
    return torch.stack(ys, 1), S


def matrix_product_form(s0, r, w_raw, k, v, a, b):
    """S_{t+1} = S_t M_t + v_t k_t^T with M_t = diag(w_t) + a_t b_t^T, unrolled:
    S_{t+1} = s0 M_0..M_t + sum_s v_s k_s^T M_{s+1}..M_t, every product by torch.matmul.  Tiny shapes only."""
    B, T, H, N = r.shape
    w = decay_sigmoid(w_raw)
    eye = torch.eye(N, dtype=r.dtype)
    M = [eye * w[:, t, :, None, :] + a[:, t, :, :, None] * b[:, t, :, None, :] for t in range(T)]
    ys = []
    S = None
    for t in range(T):
        S = s0
        for z in range(t + 1):
            S = S @ M[z]
        for s in range(t + 1):
            term = v[:, s, :, :, None] * k[:, s, :, None, :]
            for z in range(s + 1, t + 1):
                term = term @ M[z]
            S = S + term
        ys.append((S @ r[:, t, :, :, None]).squeeze(-1))
    return torch.stack(ys, 1), S


def grads(s0, r, w_raw, k, v, a, b, dy, dsT, dtype=torch.float64, splits=1):
    """(y, sT, ds0, dr, dw, dk, dv, da, db) by autograd; `splits` > 1 chains that many
    consecutive calls, each final state feeding the next (the state-passing use)."""
    leaves = [x.detach().to(dtype).clone().requires_grad_(True) for x in (s0, r, w_raw, k, v, a, b)]
    T = r.shape[1]
    step = T // splits
    S = leaves[0]
    ys = []
    for c in range(splits):
        sl = slice(c * step, (c + 1) * step)
        y, S = recurrent(S, *(x[:, sl] for x in leaves[1:]))
        ys.append(y)
    y = torch.cat(ys, 1)
    torch.autograd.backward([y, S], [dy.to(dtype), dsT.to(dtype)])
    return [y.detach(), S.detach()] + [x.grad for x in leaves]


def backward_hand(s0, r, w_raw, k, v, a, b, dy, dsT, dtype=torch.float64, chunk_len=16, invert=False,
                  round_bf16=False):
    """Forward + hand-derived backward in the order the reference kernels use.

    Forward (rwkv7_statepassing_clampw.cu:20-81) keeps sa_t and a state checkpoint at the end of
    every chunk_len steps.  Backward (:89-187) walks t down; with invert=True the state S_t is
    recovered from S_{t+1} by inverting the step, S_t = (S_{t+1} - v k^T - sa b^T) / w (:143-146),
    restarting from the checkpoint at chunk ends (:122-134), which is what sets the fp32 error
    of the original kernel; with invert=False every S_t comes from the stored forward states.
    round_bf16 rounds y and the six tensor gradients to bf16 where the kernels store them.

        dr_t = S_{t+1}^T dy_t;  dS += dy_t r_t^T;  dw_t[j] = sum_i dS[i,j] S_t[i,j];
        dk_t = dS^T v_t;  dv_t = dS k_t;  db_t = dS^T sa_t;  dsa = dS b_t;  da_t = S_t^T dsa;
        dS <- dS diag(w_t) + dsa a_t^T;   dw_raw = W_SCALE * dw * w * sig * (1 - sig);   ds0 = dS.
    """
    s0, r, w_raw, k, v, a, b, dy, dsT = (x.to(dtype) for x in (s0, r, w_raw, k, v, a, b, dy, dsT))
    B, T, H, N = r.shape
    sig = torch.sigmoid(w_raw)
    w = torch.exp(W_SCALE * sig)
    S = s0.clone()
    states = []
    sa_all = torch.empty_like(r)
    y = torch.empty_like(r)
    for t in range(T):
        if not invert:
            states.append(S)
        sa = torch.einsum('bhij,bhj->bhi', S, a[:, t])
        sa_all[:, t] = sa
        S = S * w[:, t, :, None, :] + sa[..., :, None] * b[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :]
        y[:, t] = torch.einsum('bhij,bhj->bhi', S, r[:, t])
        if invert and (t + 1) % chunk_len == 0:
            states.append(S)                       # checkpoint c = S_{(c+1)*chunk_len}
    sT = S
    dS = dsT.clone()
    dr, dw, dk, dv, da, db = (torch.empty_like(r) for _ in range(6))
    Snext = sT
    for t in range(T - 1, -1, -1):
        if invert and (t + 1) % chunk_len == 0:
            Snext = states[t // chunk_len]
        dr[:, t] = torch.einsum('bhij,bhi->bhj', Snext, dy[:, t])
        if invert:
            St = (Snext - v[:, t, :, :, None] * k[:, t, :, None, :]
                  - sa_all[:, t, :, :, None] * b[:, t, :, None, :]) / w[:, t, :, None, :]
        else:
            St = states[t]
        dS = dS + dy[:, t, :, :, None] * r[:, t, :, None, :]
        dwt = (dS * St).sum(-2)
        dk[:, t] = torch.einsum('bhij,bhi->bhj', dS, v[:, t])
        dv[:, t] = torch.einsum('bhij,bhj->bhi', dS, k[:, t])
        db[:, t] = torch.einsum('bhij,bhi->bhj', dS, sa_all[:, t])
        dsa = torch.einsum('bhij,bhj->bhi', dS, b[:, t])
        da[:, t] = torch.einsum('bhij,bhi->bhj', St, dsa)
        dw[:, t] = W_SCALE * dwt * w[:, t] * sig[:, t] * (1 - sig[:, t])
        dS = dS * w[:, t, :, None, :] + dsa[..., :, None] * a[:, t, :, None, :]
        Snext = St
    out = [y, sT, dS, dr, dw, dk, dv, da, db]
    if round_bf16:
        out = [out[0].to(torch.bfloat16), out[1], out[2]] + [x.to(torch.bfloat16) for x in out[3:]]
    return out


def emulate_bf16(s0, r, w_raw, k, v, a, b, dy, dsT, chunk_len=16):
    """Error bar for the bf16 path: fp32 math on the bf16 inputs, in-chunk inversion, checkpoints
    every chunk_len steps, sa kept in fp32, outputs rounded to bf16 -- the rounding points of
    rwkv7_statepassing_clampw.cu (:56,66 forward; :141,160-164,175 backward); states stay fp32."""
    return backward_hand(s0, r, w_raw, k, v, a, b, dy, dsT, dtype=torch.float32, chunk_len=chunk_len,
                         invert=True, round_bf16=True)
