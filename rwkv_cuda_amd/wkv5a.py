"""RWKV-5 WKV with two-sided decay and bonus, fp32: drop-in for wkv5a/run.py:100-157 (class WKV_5A, CUDA_1)."""

import torch

from ._call import call, check_tensors, require

MAX_HEAD_SIZE = 128      # 64 runs on the kernels written for it, other sizes on the row kernels


class WKV_5A(torch.autograd.Function):
    """Same signature as WKV_5A, wkv5a/run.py:100-154: r,k,v[B,T,C]; w1,u1,w2,u2[H,N]; all fp32, w raw.
    The reference reads B,T,C,H from module globals (:111-115); here they come from the tensors.
    State element [i][j] (i = value channel) decays by exp(-exp(w1[j])) * exp(-exp(w2[i])), and the
    current token's bonus is u1[j] + u2[i]."""

    @staticmethod
    def forward(ctx, r, k, v, w1, u1, w2, u2):
        with torch.no_grad():
            dev = check_tensors((r, k, v, w1, u1, w2, u2), torch.float32, ("r", "k", "v", "w1", "u1", "w2", "u2"))
            require(r.dim() == 3 and w1.dim() == 2, "r,k,v are [B,T,C]; w1,u1,w2,u2 are [H,N]")
            B, T, C = r.shape
            H = w1.shape[0]
            require(C % H == 0 and w1.shape[1] == C // H and C // H <= MAX_HEAD_SIZE, "w1 is [H, C/H] with a head size of at most 128")
            require(k.shape == r.shape and v.shape == r.shape, "shape mismatch")
            require(u1.shape == w1.shape and w2.shape == w1.shape and u2.shape == w1.shape, "shape mismatch")
            ctx.dims = (B, T, C, H)
            ew1 = (-torch.exp(w1)).contiguous()
            eew1 = torch.exp(ew1).contiguous()
            ew2 = (-torch.exp(w2)).contiguous()
            eew2 = torch.exp(ew2).contiguous()
            ctx.save_for_backward(r, k, v, eew1, ew1, u1, eew2, ew2, u2)
            y = torch.empty((B, T, C), device=dev, dtype=torch.float32)
            call("rwkv_wkv5a_forward", dev, B, T, C, H, r, k, v, eew1, u1, eew2, u2, y)
            return y

    @staticmethod
    def backward(ctx, gy):
        with torch.no_grad():
            B, T, C, H = ctx.dims
            r, k, v, eew1, ew1, u1, eew2, ew2, u2 = ctx.saved_tensors
            gy = gy.contiguous()
            dev = check_tensors((gy,), torch.float32, ("gy",))
            new = lambda *shape: torch.empty(shape, device=dev, dtype=torch.float32)
            gr, gk, gv = new(B, T, C), new(B, T, C), new(B, T, C)
            gw1, gu1, gw2, gu2 = new(B, C), new(B, C), new(B, C), new(B, C)
            call("rwkv_wkv5a_backward", dev, B, T, C, H, r, k, v, eew1, ew1, u1, eew2, ew2, u2, gy,
                 gr, gk, gv, gw1, gu1, gw2, gu2)
            fold = lambda g: torch.sum(g, 0).view(H, C // H)
            return (gr, gk, gv, fold(gw1), fold(gu1), fold(gw2), fold(gu2))


def CUDA_1(r, k, v, w1, u1, w2, u2):
    return WKV_5A.apply(r, k, v, w1, u1, w2, u2)
