"""CPU oracle: the RWKV-7 clamp-w recurrence in CHUNKED (matrix-product) form, forward and backward
(TEST INFRASTRUCTURE, not product code; no kernel uses this form yet -- it is the specification a
matrix-core kernel would be written against, pinned here against the step form).

Step form (oracle/rwkv7.py, rwkv7_cuda_benchmark_state_passing.py:58-66), one head, S[i][j] (i value, j key):
    sa_t = S_t a_t;   S_{t+1} = S_t diag(w_t) + sa_t b_t^T + v_t k_t^T;   y_t = S_{t+1} r_t

A chunk of L steps, local t = 0..L-1, S0 the state entering it.  With lam_t = log w_t, c_t = sum_{z<t} lam_z
(c_0 = 0) and the chunk's middle m = L/2 as the reference point (the clamp keeps |c_t - c_m| <= 0.607 L/2,
so no factor can run away):
    A'_t = a_t e^{c_t - c_m}      R'_t = r_t e^{c_{t+1} - c_m}      B'_s = b_s e^{c_m - c_{s+1}}      K'_s = k_s e^{c_m - c_{s+1}}
    d1 = e^{c_m}    d2 = e^{c_L - c_m}    dec = e^{c_L}
    AB = tril_-(A' B'^T)   AK = tril_-(A' K'^T)   RB = tril(R' B'^T)   RK = tril(R' K'^T)          [L x L]
    U  = (I - AB)^{-1} ((A' d1) S0^T + AK V)           rows of U are sa_t  (what the reference stores as `sa`)
    Y  = (R' d1) S0^T + RB U + RK V
    S_L = S0 diag(dec) + U^T (B' d2) + V^T (K' d2)     (what the reference stores as checkpoint `s`)

Backward of one chunk from dY and dS_L (gradient of the loss w.r.t. S_L through everything after the chunk):
    dU  = RB^T dY + (B' d2) dS_L^T            dW = (I - AB)^{-T} dU
    dAB = tril_-(dW U^T)   dAK = tril_-(dW V^T)   dRB = tril(dY U^T)   dRK = tril(dY V^T)
    dV  = AK^T dW + RK^T dY + (K' d2) dS_L^T
    dS0 = dS_L diag(dec) + dY^T (R' d1) + dW^T (A' d1)
    dA' = dAB B' + dAK K' + d1 (dW S0)        dR' = dRB B' + dRK K' + d1 (dY S0)
    dB' = dAB^T A' + dRB^T R' + d2 (U dS_L)    dK' = dAK^T A' + dRK^T R' + d2 (V dS_L)
    da_t = dA'_t e^{c_t - c_m}  and likewise dr, db, dk (the decay factors held fixed: a, b, k, r are independent inputs)
The decay gradient needs no further product.  With P_t[j] = sum_i dS_t[i][j] S_t[i][j] (dS_t: gradient w.r.t. S_t through
steps >= t) and G_t = dL/d lam_t:
    G_t = P_{t+1} + r_t dr_t - b_t db_t - k_t dk_t,      P_t = G_t + a_t da_t,
all elementwise per key channel, P at the chunk's end taken exactly as sum_i dS_L o S_L from the carried dS_L and the
stored checkpoint (so nothing accumulates across chunks);  dw_raw = G W_SCALE sig (1 - sig).
"""

import torch

from .rwkv7 import W_SCALE


def _bh(x):
    """[B,T,H,N] -> [B,H,T,N]"""
    return x.transpose(1, 2)


def _factors(lam):
    """lam [B,H,L,N] = log decay of a chunk.  Returns the exponents' values (e^{c_t - c_m}, e^{c_{t+1} - c_m},
    e^{c_m - c_{t+1}}) per step and (d1, d2, dec) per channel."""
    L = lam.shape[-2]
    cin = torch.cumsum(lam, -2)                    # c_{t+1}
    c = cin - lam                                  # c_t
    cm = c[..., L // 2, :].unsqueeze(-2)
    cL = cin[..., -1, :].unsqueeze(-2)
    return torch.exp(c - cm), torch.exp(cin - cm), torch.exp(cm - cin), torch.exp(cm), torch.exp(cL - cm), torch.exp(cL)


def _chunk_forward(S0, r, lam, k, v, a, b):
    """One chunk, tensors [B,H,L,N], S0 [B,H,N,N].  Returns (Y, S_L, U, saved)."""
    L = r.shape[-2]
    ea, er, eb, d1, d2, dec = _factors(lam)
    A, R, Bp, K = a * ea, r * er, b * eb, k * eb
    lo = torch.tril(torch.ones(L, L, dtype=r.dtype), -1)
    lod = torch.tril(torch.ones(L, L, dtype=r.dtype))
    AB, AK = (A @ Bp.mT) * lo, (A @ K.mT) * lo
    RB, RK = (R @ Bp.mT) * lod, (R @ K.mT) * lod
    eye = torch.eye(L, dtype=r.dtype)
    W = (A * d1) @ S0.mT + AK @ v
    U = torch.linalg.solve_triangular(eye - AB, W, upper=False, unitriangular=True)
    Y = (R * d1) @ S0.mT + RB @ U + RK @ v
    SL = S0 * dec + U.mT @ (Bp * d2) + v.mT @ (K * d2)
    return Y, SL, U, (A, R, Bp, K, AB, AK, RB, RK, d1, d2, dec, ea, er, eb, lo, lod)


def forward(s0, r, w_raw, k, v, a, b, chunk_len=16):
    """Chunked forward.  [B,T,H,N] tensors, s0 [B,H,N,N]; T % chunk_len == 0.
    Returns (y [B,T,H,N], sT, sa [B,T,H,N], checkpoints [B,H,T/chunk_len,N,N])."""
    B, T, H, N = r.shape
    lam = W_SCALE * torch.sigmoid(_bh(w_raw))
    rr, kk, vv, aa, bb = (_bh(x) for x in (r, k, v, a, b))
    S = s0
    ys, sas, chk = [], [], []
    for c0 in range(0, T, chunk_len):
        sl = slice(c0, c0 + chunk_len)
        Y, S, U, _ = _chunk_forward(S, rr[:, :, sl], lam[:, :, sl], kk[:, :, sl], vv[:, :, sl], aa[:, :, sl], bb[:, :, sl])
        ys.append(Y); sas.append(U); chk.append(S)
    return torch.cat(ys, 2).transpose(1, 2), S, torch.cat(sas, 2).transpose(1, 2), torch.stack(chk, 2)


def backward(s0, r, w_raw, k, v, a, b, dy, dsT, chunk_len=16):
    """Chunked forward + backward.  Returns [y, sT, ds0, dr, dw, dk, dv, da, db] like oracle.rwkv7.grads."""
    B, T, H, N = r.shape
    sig = torch.sigmoid(_bh(w_raw))
    lam = W_SCALE * sig
    rr, kk, vv, aa, bb, dyy = (_bh(x) for x in (r, k, v, a, b, dy))
    S = s0
    starts, ys = [], []
    for c0 in range(0, T, chunk_len):
        sl = slice(c0, c0 + chunk_len)
        starts.append(S)
        Y, S, _, _ = _chunk_forward(S, rr[:, :, sl], lam[:, :, sl], kk[:, :, sl], vv[:, :, sl], aa[:, :, sl], bb[:, :, sl])
        ys.append(Y)
    sT = S
    dS = dsT
    Send = sT
    dr, dlam, dk, dv, da, db = (torch.empty_like(rr) for _ in range(6))
    for ci in range(T // chunk_len - 1, -1, -1):
        sl = slice(ci * chunk_len, (ci + 1) * chunk_len)
        S0 = starts[ci]
        rc, kc, vc, ac, bc, dY = rr[:, :, sl], kk[:, :, sl], vv[:, :, sl], aa[:, :, sl], bb[:, :, sl], dyy[:, :, sl]
        _, _, U, (A, R, Bp, K, AB, AK, RB, RK, d1, d2, dec, ea, er, eb, lo, lod) = _chunk_forward(S0, rc, lam[:, :, sl], kc, vc, ac, bc)
        L = chunk_len
        eye = torch.eye(L, dtype=rr.dtype)
        dU = RB.mT @ dY + (Bp * d2) @ dS.mT
        dW = torch.linalg.solve_triangular((eye - AB).mT, dU, upper=True, unitriangular=True)
        dAB, dAK = (dW @ U.mT) * lo, (dW @ vc.mT) * lo
        dRB, dRK = (dY @ U.mT) * lod, (dY @ vc.mT) * lod
        dv[:, :, sl] = AK.mT @ dW + RK.mT @ dY + (K * d2) @ dS.mT
        dA = dAB @ Bp + dAK @ K + d1 * (dW @ S0)
        dR = dRB @ Bp + dRK @ K + d1 * (dY @ S0)
        dB = dAB.mT @ A + dRB.mT @ R + d2 * (U @ dS)
        dK = dAK.mT @ A + dRK.mT @ R + d2 * (vc @ dS)
        dac, drc, dbc, dkc = dA * ea, dR * er, dB * eb, dK * eb
        da[:, :, sl], dr[:, :, sl], db[:, :, sl], dk[:, :, sl] = dac, drc, dbc, dkc
        # decay gradient: elementwise scan from P at the chunk's end
        P = (dS * Send).sum(-2)                                     # [B,H,N]
        for t in range(L - 1, -1, -1):
            G = P + rc[:, :, t] * drc[:, :, t] - bc[:, :, t] * dbc[:, :, t] - kc[:, :, t] * dkc[:, :, t]
            dlam[:, :, sl.start + t] = G
            P = G + ac[:, :, t] * dac[:, :, t]
        dS = dS * dec + dY.mT @ (R * d1) + dW.mT @ (A * d1)
        Send = S0
    dw = dlam * W_SCALE * sig * (1 - sig)
    y = torch.cat(ys, 2).transpose(1, 2)
    return [y, sT, dS] + [x.transpose(1, 2) for x in (dr, dw, dk, dv, da, db)]
