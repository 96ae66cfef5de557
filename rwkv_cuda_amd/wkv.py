"""RWKV-4 WKV, fp32: drop-in for wkv/run.py:89-120 (class WKV, RUN_CUDA)."""

import torch

from . import _lib
from ._call import call, check_tensors, require


class WKV(torch.autograd.Function):
    """Same signature as WKV, wkv/run.py:89-117: w,u[C] (w raw), k,v[B,T,C], fp32."""

    @staticmethod
    def forward(ctx, B, T, C, w, u, k, v):
        ctx.B, ctx.T, ctx.C = B, T, C
        w = -torch.exp(w.contiguous())
        u, k, v = u.contiguous(), k.contiguous(), v.contiguous()
        dev = check_tensors((w, u, k, v), torch.float32, "wukv")
        require(k.numel() == B * T * C and w.numel() == C, "shape mismatch")
        ctx.save_for_backward(w, u, k, v)
        y = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        call("rwkv_wkv4_forward", dev, B, T, C, w, u, k, v, y)
        return y

    @staticmethod
    def backward(ctx, gy):
        B, T, C = ctx.B, ctx.T, ctx.C
        w, u, k, v = ctx.saved_tensors
        gy = gy.contiguous()
        dev = check_tensors((gy,), torch.float32, ("gy",))
        gw = torch.zeros((B, C), device=dev, dtype=torch.float32)
        gu = torch.zeros((B, C), device=dev, dtype=torch.float32)
        gk = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        gv = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        nbytes = _lib.load().rwkv_wkv4_backward_workspace_bytes(B, T, C)
        ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
        call("rwkv_wkv4_backward", dev, B, T, C, w, u, k, v, gy, gw, gu, gk, gv, ws, nbytes)
        gw = torch.sum(gw, dim=0)
        gu = torch.sum(gu, dim=0)
        return (None, None, None, gw, gu, gk, gv)


def RUN_CUDA(B, T, C, w, u, k, v):
    return WKV.apply(B, T, C, w.cuda(), u.cuda(), k.cuda(), v.cuda())
