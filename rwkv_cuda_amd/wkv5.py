"""RWKV-5 WKV, fp32: drop-in for wkv5/run.py:469-507 (class WKV_5, RUN_CUDA)."""

import torch

from ._call import call, check_tensors, require

HEAD_SIZE = 64          # the size the matrix-core kernels are written for; any size up to MAX_HEAD_SIZE runs
MAX_HEAD_SIZE = 128


class WKV_5(torch.autograd.Function):
    """Same signature as WKV_5, wkv5/run.py:469-504: r,k,v[B,T,C], w,u with C elements ([C] in the
    reference's checks, :519-520), all fp32, w raw.  ew = -exp(w) and eew = exp(ew) are made by the
    wrapper (:482-483); gw and gu come back in the shape of w and u."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u):
        with torch.no_grad():
            dev = check_tensors((r, k, v, w, u), torch.float32, "rkvwu")
            require(C % H == 0 and C // H <= MAX_HEAD_SIZE, "C must be a multiple of H with a head size of at most 128")
            require(r.numel() == B * T * C and w.numel() == C and u.numel() == C, "shape mismatch")
            ctx.B, ctx.T, ctx.C, ctx.H = B, T, C, H
            ctx.wshape, ctx.ushape = w.shape, u.shape
            ew = (-torch.exp(w)).contiguous()
            eew = (torch.exp(ew)).contiguous()
            ctx.save_for_backward(r, k, v, eew, ew, u)
            y = torch.empty((B, T, C), device=dev, dtype=torch.float32)
            call("rwkv_wkv5f32_forward", dev, B, T, C, H, r, k, v, eew, u, y)
            return y

    @staticmethod
    def backward(ctx, gy):
        with torch.no_grad():
            B, T, C, H = ctx.B, ctx.T, ctx.C, ctx.H
            r, k, v, eew, ew, u = ctx.saved_tensors
            gy = gy.contiguous()
            dev = check_tensors((gy,), torch.float32, ("gy",))
            new = lambda *shape: torch.empty(shape, device=dev, dtype=torch.float32)
            gr, gk, gv = new(B, T, C), new(B, T, C), new(B, T, C)
            gw, gu = new(B, C), new(B, C)
            call("rwkv_wkv5f32_backward", dev, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu)
            gw = torch.sum(gw, 0).view(ctx.wshape)
            gu = torch.sum(gu, 0).view(ctx.ushape)
            return (None, None, None, None, gr, gk, gv, gw, gu)


def RUN_CUDA(B, T, C, H, r, k, v, w, u):
    return WKV_5.apply(B, T, C, H, r, k, v, w, u)
