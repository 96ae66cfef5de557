"""RWKV-7 clamp-w, bf16 or fp32 (the dtype of r selects the mode the reference fixes at build time with DTYPE /
-D_FP32_, rwkv7_cuda_benchmark.py:14,76,102): drop-ins for
rwkv7_fast_fused/rwkv7_cuda_benchmark_state_passing.py:75-103 (RWKV7_STATE_PASSING_CLAMPW_CUDA_OP, ..._CUDA),
rwkv7_fast_fused/rwkv7_cuda_benchmark_state.py:75-102 (RWKV7_STATE_CLAMPW_CUDA_OP, ..._CUDA: initial state only) and
rwkv7_fast_fused/rwkv7_cuda_benchmark.py:76-100 (RWKV7_CLAMPW_CUDA_OP, ..._CUDA: no state)."""

import torch

from . import options
from ._call import call, check_tensors, require

HEAD_SIZE = 64
CHUNK_LEN = 16


def _mode(r):
    """(element dtype, entry-point suffix) for the bf16 and the fp32 build of the reference."""
    require(r.dtype in (torch.bfloat16, torch.float32), f"r.dtype must be bfloat16 or float32, got {r.dtype}")
    return (torch.float32, "_f32") if r.dtype == torch.float32 else (torch.bfloat16, "")


class RWKV7_STATE_PASSING_CLAMPW_CUDA_OP(torch.autograd.Function):
    """forward(s0, r, w, k, v, a, b) -> (y[B,T,H*N], sT); r..b are [B,T,H,N] bf16 (or all fp32), s0/sT fp32 [B,H,N,N].
    Allocations and saved tensors follow :77-90 (the checkpoint tensor `s` and `sa` are scratch
    whose inner layout belongs to the library)."""

    @staticmethod
    def forward(ctx, s0, r, w, k, v, a, b):
        B, T, H, N = r.shape
        require(N == HEAD_SIZE, "head size must be 64")
        require(T % CHUNK_LEN == 0, "T must be a multiple of CHUNK_LEN")
        dt, sfx = _mode(r)
        dev = check_tensors((r, w, k, v, a, b), dt, "rwkvab")
        check_tensors((s0,), torch.float32, ("s0",))
        require(s0.device == dev and tuple(s0.shape) == (B, H, N, N), "s0 must be [B,H,N,N] on the same device")
        y = torch.empty_like(v)
        sT = torch.empty_like(s0)
        s = torch.empty(B, H, T // CHUNK_LEN, N, N, dtype=torch.float32, device=dev)
        sa = torch.empty(B, T, H, N, dtype=torch.float32, device=dev)
        # bf16 mode: chunked matrix-core kernels unless options.algorithm("sweeps") is active; the backward must follow the
        # forward's choice (the two kernel families lay `s` out differently), so the flags ride on the context
        ctx.flags = options.current_flags()
        if sfx:
            call("rwkv7_statepassing_forward_f32", dev, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa)
        else:
            call("rwkv7_statepassing_forward_ex", dev, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa, ctx.flags)
        ctx.save_for_backward(r, w, k, v, a, b, s, sa)
        return y.view(B, T, H * N), sT

    @staticmethod
    def backward(ctx, dy, dsT):
        r, w, k, v, a, b, s, sa = ctx.saved_tensors
        B, T, H, N = r.shape
        dy = dy.contiguous()
        dsT = dsT.contiguous()
        dt, sfx = _mode(r)
        dev = check_tensors((dy,), dt, ("dy",))
        check_tensors((dsT,), torch.float32, ("dsT",))
        ds0, dr, dw, dk, dv, da, db = [torch.empty_like(x) for x in [dsT, r, w, k, v, a, b]]
        if sfx:
            call("rwkv7_statepassing_backward_f32", dev, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db)
        else:
            call("rwkv7_statepassing_backward_ex", dev, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, dr, dw, dk, dv, da, db, ctx.flags)
        return ds0, dr, dw, dk, dv, da, db


def RWKV7_STATE_PASSING_CLAMPW_CUDA(s0, r, w, k, v, a, b):
    B, T, HC = r.shape
    r, w, k, v, a, b = [i.view(B, T, HC // HEAD_SIZE, HEAD_SIZE) for i in [r, w, k, v, a, b]]
    return RWKV7_STATE_PASSING_CLAMPW_CUDA_OP.apply(s0, r, w, k, v, a, b)


def _scratch(r):
    B, T, H, N = r.shape
    s = torch.empty(B, H, T // CHUNK_LEN, N, N, dtype=torch.float32, device=r.device)
    sa = torch.empty(B, T, H, N, dtype=torch.float32, device=r.device)
    return s, sa


class RWKV7_STATE_CLAMPW_CUDA_OP(torch.autograd.Function):
    """forward(s0, r, w, k, v, a, b) -> y[B,T,H,N]; backward returns (ds0, dr, dw, dk, dv, da, db)
    (rwkv7_cuda_benchmark_state.py:77-98)."""

    @staticmethod
    def forward(ctx, s0, r, w, k, v, a, b):
        B, T, H, N = r.shape
        require(N == HEAD_SIZE, "head size must be 64")
        require(T % CHUNK_LEN == 0, "T must be a multiple of CHUNK_LEN")
        dt, sfx = _mode(r)
        dev = check_tensors((r, w, k, v, a, b), dt, "rwkvab")
        check_tensors((s0,), torch.float32, ("s0",))
        require(s0.device == dev and tuple(s0.shape) == (B, H, N, N), "s0 must be [B,H,N,N] on the same device")
        y = torch.empty_like(v)
        s, sa = _scratch(r)
        call("rwkv7_state_forward" + sfx, dev, B, T, H, s0, r, w, k, v, a, b, y, s, sa)
        ctx.save_for_backward(r, w, k, v, a, b, s, sa)
        return y

    @staticmethod
    def backward(ctx, dy):
        r, w, k, v, a, b, s, sa = ctx.saved_tensors
        B, T, H, N = r.shape
        dy = dy.contiguous()
        dt, sfx = _mode(r)
        dev = check_tensors((dy,), dt, ("dy",))
        ds0 = torch.empty(B, H, N, N, dtype=torch.float32, device=dev)
        dr, dw, dk, dv, da, db = [torch.empty_like(x) for x in [r, w, k, v, a, b]]
        call("rwkv7_state_backward" + sfx, dev, B, T, H, r, w, k, v, a, b, dy, s, sa, ds0, dr, dw, dk, dv, da, db)
        return ds0, dr, dw, dk, dv, da, db


def RWKV7_STATE_CLAMPW_CUDA(s0, r, w, k, v, a, b):
    B, T, HC = r.shape
    r, w, k, v, a, b = [i.view(B, T, HC // HEAD_SIZE, HEAD_SIZE) for i in [r, w, k, v, a, b]]
    return RWKV7_STATE_CLAMPW_CUDA_OP.apply(s0, r, w, k, v, a, b).view(B, T, HC)


class RWKV7_CLAMPW_CUDA_OP(torch.autograd.Function):
    """forward(r, w, k, v, a, b) -> y[B,T,H,N] from a zero state; backward returns (dr, dw, dk, dv, da, db)
    (rwkv7_cuda_benchmark.py:78-96)."""

    @staticmethod
    def forward(ctx, r, w, k, v, a, b):
        B, T, H, N = r.shape
        require(N == HEAD_SIZE, "head size must be 64")
        require(T % CHUNK_LEN == 0, "T must be a multiple of CHUNK_LEN")
        dt, sfx = _mode(r)
        dev = check_tensors((r, w, k, v, a, b), dt, "rwkvab")
        y = torch.empty_like(v)
        s, sa = _scratch(r)
        call("rwkv7_forward" + sfx, dev, B, T, H, r, w, k, v, a, b, y, s, sa)
        ctx.save_for_backward(r, w, k, v, a, b, s, sa)
        return y

    @staticmethod
    def backward(ctx, dy):
        r, w, k, v, a, b, s, sa = ctx.saved_tensors
        B, T, H, N = r.shape
        dy = dy.contiguous()
        dt, sfx = _mode(r)
        dev = check_tensors((dy,), dt, ("dy",))
        dr, dw, dk, dv, da, db = [torch.empty_like(x) for x in [r, w, k, v, a, b]]
        call("rwkv7_backward" + sfx, dev, B, T, H, r, w, k, v, a, b, dy, s, sa, dr, dw, dk, dv, da, db)
        return dr, dw, dk, dv, da, db


def RWKV7_CLAMPW_CUDA(r, w, k, v, a, b):
    B, T, HC = r.shape
    r, w, k, v, a, b = [i.view(B, T, HC // HEAD_SIZE, HEAD_SIZE) for i in [r, w, k, v, a, b]]
    return RWKV7_CLAMPW_CUDA_OP.apply(r, w, k, v, a, b).view(B, T, HC)
