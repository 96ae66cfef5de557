"""RWKV-5 WKV, bf16: drop-in for wkv5_bf16/run.py:44-91 (class WKV_5, RUN_CUDA)."""

import torch

from . import _lib, options
from ._call import call, check_tensors, require

HEAD_SIZE = 64          # the size the matrix-core kernels are written for; any size up to MAX_HEAD_SIZE runs
MAX_HEAD_SIZE = 128


class WKV_5(torch.autograd.Function):
    """Same signature as WKV_5, wkv5_bf16/run.py:44-88: r,k,v[B,T,C], w,u[H,N], all bf16, w raw.
    ew = -exp(w) and eew = exp(ew) are made in fp32 by the wrapper (:63-64)."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u):
        with torch.no_grad():
            dev = check_tensors((r, k, v, w, u), torch.bfloat16, "rkvwu")
            require(C % H == 0 and C // H <= MAX_HEAD_SIZE, "C must be a multiple of H with a head size of at most 128")
            require(r.numel() == B * T * C and w.numel() == C, "shape mismatch")
            ctx.B, ctx.T, ctx.C, ctx.H = B, T, C, H
            ctx.flags = options.current_flags()
            # ew = -exp(w.float()), eew = exp(ew) (:63-64) are made by the library into `decay` = [eew | ew]
            decay = torch.empty(2 * C, device=dev, dtype=torch.float32)
            y = torch.empty((B, T, C), device=dev, dtype=torch.bfloat16)
            lib = _lib.load()
            nsaved = lib.rwkv_wkv5s_saved_bytes(B, T, C, H) if C == H * HEAD_SIZE else 0
            if nsaved > 0:
                # head size 64: one forward and one reverse sweep; the forward keeps the state entering every 64th token
                saved = torch.empty(nsaved, device=dev, dtype=torch.uint8)
                call("rwkv_wkv5s_forward", dev, B, T, C, H, r, k, v, w, u, y, decay, saved, nsaved, ctx.flags)
                ctx.nsaved = nsaved
                ctx.save_for_backward(r, k, v, decay, u, w, saved)
                return y
            # heads of 128 channels run as four heads of 64 whose fp32 terms need scratch; every other size needs none
            nbytes = lib.rwkv_wkv5_forward_workspace_bytes(B, T, C, H)
            ws = torch.empty(max(nbytes, 16), device=dev, dtype=torch.uint8)
            call("rwkv_wkv5raw_forward_ws", dev, B, T, C, H, r, k, v, w, u, y, decay, ws, nbytes, ctx.flags)
            ctx.nsaved = 0
            ctx.save_for_backward(r, k, v, decay, u)
            return y

    @staticmethod
    def backward(ctx, gy):
        with torch.no_grad():
            B, T, C, H = ctx.B, ctx.T, ctx.C, ctx.H
            r, k, v, decay, u = ctx.saved_tensors[:5]
            gy = gy.contiguous()
            dev = check_tensors((gy,), torch.bfloat16, ("gy",))
            new = lambda *shape: torch.empty(shape, device=dev, dtype=torch.bfloat16)
            gr, gk, gv = new(B, T, C), new(B, T, C), new(B, T, C)
            gw, gu = new(H, C // H), new(H, C // H)           # summed over the batch by the library (:86-87)
            if ctx.nsaved > 0:
                w, saved = ctx.saved_tensors[5:]
                nbytes = _lib.load().rwkv_wkv5s_backward_workspace_bytes(B, T, C, H)
                ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
                call("rwkv_wkv5s_backward", dev, B, T, C, H, r, k, v, w, decay, u, gy, gr, gk, gv, gw, gu, saved, ctx.nsaved, ws, nbytes, ctx.flags)
                return (None, None, None, None, gr, gk, gv, gw, gu)
            nbytes = _lib.load().rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H)
            ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
            call("rwkv_wkv5raw_backward", dev, B, T, C, H, r, k, v, decay, u, gy, gr, gk, gv, gw, gu, ws, nbytes, ctx.flags)
            return (None, None, None, None, gr, gk, gv, gw, gu)


def RUN_CUDA(B, T, C, H, r, k, v, w, u):
    return WKV_5.apply(B, T, C, H, r, k, v, w, u)
