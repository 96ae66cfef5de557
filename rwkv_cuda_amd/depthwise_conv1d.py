"""depthwise_conv1d ("TimeX"), fp32: drop-in for depthwise_conv1d/run.py:76-106 (class TimeX, RUN_CUDA)."""

import torch

from ._call import call, check_tensors, require

T_MAX = 4096
T_SUM_MAX = 1024      # rwkv_timex_backward_sum: T % 32 == 0 and T <= 1024


class TimeX(torch.autograd.Function):
    """Same signature as TimeX, depthwise_conv1d/run.py:76-102: w[C,T], k[B,C,T] fp32.
    T % 4 == 0 is required as in the reference; the reference's B % 8 and T <= 768 limits are not."""

    @staticmethod
    def forward(ctx, w, k, B, C, T, eps):
        ctx.B, ctx.C, ctx.T = B, C, T
        require(T % 4 == 0 and T <= T_MAX, "require T % 4 == 0 and T <= T_MAX")
        w, k = w.contiguous(), k.contiguous()
        dev = check_tensors((w, k), torch.float32, "wk")
        require(w.numel() == C * T and k.numel() == B * C * T, "shape mismatch")
        ctx.save_for_backward(w, k)
        wk = torch.empty((B, C, T), device=dev, dtype=torch.float32)
        call("rwkv_timex_forward", dev, w, k, wk, float(eps), B, C, T)
        return wk

    @staticmethod
    def backward(ctx, gwk):
        w, k = ctx.saved_tensors
        gwk = gwk.contiguous()
        dev = check_tensors((gwk,), torch.float32, ("gwk",))
        gk = torch.empty((ctx.B, ctx.C, ctx.T), device=dev, dtype=torch.float32)
        if ctx.T % 32 == 0 and ctx.T <= T_SUM_MAX:       # the sum over the batch of run.py:102 happens in the kernel
            gw = torch.empty((ctx.C, ctx.T), device=dev, dtype=torch.float32)
            call("rwkv_timex_backward_sum", dev, w, k, gwk, gw, gk, ctx.B, ctx.C, ctx.T)
            return (gw, gk, None, None, None, None)
        gw = torch.empty((ctx.B, ctx.C, ctx.T), device=dev, dtype=torch.float32)
        call("rwkv_timex_backward", dev, w, k, gwk, gw, gk, ctx.B, ctx.C, ctx.T)
        return (gw.sum(dim=0), gk, None, None, None, None)


def RUN_CUDA(w, k, B, C, T, eps):
    return TimeX.apply(w.cuda(), k.cuda(), B, C, T, eps)
