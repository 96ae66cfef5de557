"""RWKV-4 WKV, fp32: drop-in for wkv/run.py:89-120 (class WKV, RUN_CUDA)."""

import torch

from . import _lib
from ._call import call, check_tensors, require


class WKV(torch.autograd.Function):
    """Same signature as WKV, wkv/run.py:89-117: w,u[C] (w raw), k,v[B,T,C], fp32."""

    @staticmethod
    def forward(ctx, B, T, C, w, u, k, v):
        ctx.B, ctx.T, ctx.C = B, T, C
        # w = -exp(w) of the reference wrapper (:95) happens inside the kernels (rwkv_wkv4raw_*)
        w, u, k, v = w.contiguous(), u.contiguous(), k.contiguous(), v.contiguous()
        dev = check_tensors((w, u, k, v), torch.float32, "wukv")
        require(k.numel() == B * T * C and w.numel() == C, "shape mismatch")
        ctx.save_for_backward(w, u, k, v)
        y = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        call("rwkv_wkv4raw_forward", dev, B, T, C, w, u, k, v, y)
        return y

    @staticmethod
    def backward(ctx, gy):
        B, T, C = ctx.B, ctx.T, ctx.C
        w, u, k, v = ctx.saved_tensors
        gy = gy.contiguous()
        dev = check_tensors((gy,), torch.float32, ("gy",))
        gw = torch.empty((C,), device=dev, dtype=torch.float32)      # summed over the batch by the library (:115-116)
        gu = torch.empty((C,), device=dev, dtype=torch.float32)
        gk = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        gv = torch.empty((B, T, C), device=dev, dtype=torch.float32)
        nbytes = _lib.load().rwkv_wkv4raw_backward_workspace_bytes(B, T, C)
        ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
        call("rwkv_wkv4raw_backward", dev, B, T, C, w, u, k, v, gy, gw, gu, gk, gv, ws, nbytes)
        return (None, None, None, gw, gu, gk, gv)


def RUN_CUDA(B, T, C, w, u, k, v):
    return WKV.apply(B, T, C, w.cuda(), u.cuda(), k.cuda(), v.cuda())
