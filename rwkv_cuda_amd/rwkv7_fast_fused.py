"""RWKV-7 clamp-w with state passing: drop-in for
rwkv7_fast_fused/rwkv7_cuda_benchmark_state_passing.py:75-103
(RWKV7_STATE_PASSING_CLAMPW_CUDA_OP, RWKV7_STATE_PASSING_CLAMPW_CUDA)."""

import torch

from ._call import call, check_tensors, require

HEAD_SIZE = 64
CHUNK_LEN = 16


class RWKV7_STATE_PASSING_CLAMPW_CUDA_OP(torch.autograd.Function):
    """forward(s0, r, w, k, v, a, b) -> (y[B,T,H*N], sT); r..b are [B,T,H,N] bf16, s0/sT fp32 [B,H,N,N].
    Allocations and saved tensors follow :77-90 (the checkpoint tensor `s` and `sa` are scratch
    whose inner layout belongs to the library)."""

    @staticmethod
    def forward(ctx, s0, r, w, k, v, a, b):
        B, T, H, N = r.shape
        require(N == HEAD_SIZE, "head size must be 64")
        require(T % CHUNK_LEN == 0, "T must be a multiple of CHUNK_LEN")
        dev = check_tensors((r, w, k, v, a, b), torch.bfloat16, "rwkvab")
        check_tensors((s0,), torch.float32, ("s0",))
        require(s0.device == dev and tuple(s0.shape) == (B, H, N, N), "s0 must be [B,H,N,N] on the same device")
        y = torch.empty_like(v)
        sT = torch.empty_like(s0)
        s = torch.empty(B, H, T // CHUNK_LEN, N, N, dtype=torch.float32, device=dev)
        sa = torch.empty(B, T, H, N, dtype=torch.float32, device=dev)
        call("rwkv7_statepassing_forward", dev, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa)
        ctx.save_for_backward(r, w, k, v, a, b, s, sa)
        return y.view(B, T, H * N), sT

    @staticmethod
    def backward(ctx, dy, dsT):
        r, w, k, v, a, b, s, sa = ctx.saved_tensors
        B, T, H, N = r.shape
        dy = dy.contiguous()
        dsT = dsT.contiguous()
        dev = check_tensors((dy,), torch.bfloat16, ("dy",))
        check_tensors((dsT,), torch.float32, ("dsT",))
        ds0, dr, dw, dk, dv, da, db = [torch.empty_like(x) for x in [dsT, r, w, k, v, a, b]]
        call("rwkv7_statepassing_backward", dev, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa,
             ds0, dr, dw, dk, dv, da, db)
        return ds0, dr, dw, dk, dv, da, db


def RWKV7_STATE_PASSING_CLAMPW_CUDA(s0, r, w, k, v, a, b):
    B, T, HC = r.shape
    r, w, k, v, a, b = [i.view(B, T, HC // HEAD_SIZE, HEAD_SIZE) for i in [r, w, k, v, a, b]]
    return RWKV7_STATE_PASSING_CLAMPW_CUDA_OP.apply(s0, r, w, k, v, a, b)
