"""RWKV-6 WKV with initial state: drop-in for wkv6_state/run.py:80-127 (class WKV_6STATE, RUN_CUDA)."""

import torch

from . import _lib, options
from ._call import call, check_tensors, require

HEAD_SIZE = 64          # the size the matrix-core kernels are written for; any size up to MAX_HEAD_SIZE runs
MAX_HEAD_SIZE = 128


class WKV_6STATE(torch.autograd.Function):
    """Same signature, dtypes and returned gradients as WKV_6STATE, wkv6_state/run.py:80-124:
    r,k,v,w[B,T,C], u[H,N], s[B,H,N,N], all bf16; w is the raw decay parameter."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u, s):
        with torch.no_grad():
            dev = check_tensors((r, k, v, w, u, s), torch.bfloat16, "rkvwus")
            require(C % H == 0 and C // H <= MAX_HEAD_SIZE, "C must be a multiple of H with a head size of at most 128")
            require(r.numel() == B * T * C and s.numel() == B * H * (C // H) * (C // H), "shape mismatch")
            ctx.B, ctx.T, ctx.C, ctx.H = B, T, C, H
            ctx.flags = options.current_flags()
            y = torch.empty((B, T, C), device=dev, dtype=torch.bfloat16)
            # the forward keeps the state entering every 64th token for the backward's single reverse sweep (no bytes for
            # head sizes and options that take the two-sweep kernels)
            nsaved = _lib.load().rwkv_wkv6f_saved_bytes(B, T, C, H)
            saved = torch.empty(nsaved, device=dev, dtype=torch.uint8)
            call("rwkv_wkv6f_forward", dev, B, T, C, H, r, k, v, w, u, s, y, saved if nsaved else None, nsaved, ctx.flags)
            ctx.save_for_backward(r, k, v, w, u, s, saved)
            return y

    @staticmethod
    def backward(ctx, gy):
        with torch.no_grad():
            B, T, C, H = ctx.B, ctx.T, ctx.C, ctx.H
            r, k, v, w, u, s, saved = ctx.saved_tensors
            gy = gy.contiguous()
            dev = check_tensors((gy,), torch.bfloat16, ("gy",))
            new = lambda *shape: torch.empty(shape, device=dev, dtype=torch.bfloat16)
            gr, gk, gv, gw = new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C)
            gu = new(H, C // H)                               # summed over the batch by the library (:123)
            gs = new(B, H, C // H, C // H)
            nbytes = _lib.load().rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
            ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
            call("rwkv_wkv6f_backward_saved", dev, B, T, C, H, r, k, v, w, u, s, gy,
                 gr, gk, gv, gw, gu, gs, saved if saved.numel() else None, saved.numel(), ws, nbytes, ctx.flags)
            return (None, None, None, None, gr, gk, gv, gw, gu, gs)


def RUN_CUDA(B, T, C, H, r, k, v, w, u, s):
    return WKV_6STATE.apply(B, T, C, H, r, k, v, w, u, s)
