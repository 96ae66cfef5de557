"""Seeded synthetic inputs for the five benchmark configurations (drawn on the CPU in fp32 so
that a CPU checker and the GPU see identical bits), used by bench.py and the tests."""

import math

import torch


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def wkv4_inputs(B, T, C, seed=42):
    """w_raw[C] = 0.5 N(0,1) (the op applies w = -exp(w_raw)), u ~ N(0,0.5), k = clamp(N(0,1),-8,8), v, gy ~ N(0,1)."""
    g = _gen(seed)
    w_raw = torch.randn(C, generator=g) * 0.5
    u = torch.randn(C, generator=g) * 0.5
    k = torch.randn(B, T, C, generator=g).clamp_(-8, 8)
    v = torch.randn(B, T, C, generator=g)
    gy = torch.randn(B, T, C, generator=g)
    return w_raw, u, k, v, gy


def timex_inputs(B, C, T, seed=42):
    """w[C,T] = N(0,1)/sqrt(T), k[B,C,T] ~ N(0,1), upstream grad ~ N(0,1)."""
    g = _gen(seed)
    w = torch.randn(C, T, generator=g) / math.sqrt(T)
    k = torch.randn(B, C, T, generator=g)
    gwk = torch.randn(B, C, T, generator=g)
    return w, k, gwk


def wkv5_inputs(B, T, C, H, seed=42):
    """r,k,v = bf16(0.5 N(0,1)); w_raw[H,N] ~ N(-0.5,0.5) (decay exp(-exp(w_raw))); u ~ N(0,0.3); gy = bf16(N(0,1))."""
    g = _gen(seed)
    N = C // H
    bf = torch.bfloat16
    r, k, v = ((torch.randn(B, T, C, generator=g) * 0.5).to(bf) for _ in range(3))
    w_raw = (torch.randn(H, N, generator=g) * 0.5 - 0.5).to(bf)
    u = (torch.randn(H, N, generator=g) * 0.3).to(bf)
    gy = torch.randn(B, T, C, generator=g).to(bf)
    return r, k, v, w_raw, u, gy


def wkv6_inputs(B, T, C, H, seed=42, state=False):
    """As wkv5 but w_raw[B,T,C] = bf16(N(-0.6,0.7)); with state: s0[B,H,N,N] ~ N(0,0.1) in bf16."""
    g = _gen(seed)
    N = C // H
    bf = torch.bfloat16
    r, k, v = ((torch.randn(B, T, C, generator=g) * 0.5).to(bf) for _ in range(3))
    w_raw = (torch.randn(B, T, C, generator=g) * 0.7 - 0.6).to(bf)
    u = (torch.randn(H, N, generator=g) * 0.3).to(bf)
    gy = torch.randn(B, T, C, generator=g).to(bf)
    s0 = (torch.randn(B, H, N, N, generator=g) * 0.1).to(bf) if state else None
    return r, k, v, w_raw, u, gy, s0


def rwkv7_inputs(B, T, H, N, seed=42):
    """r,k,v = bf16(0.5 N(0,1)); w_raw = N(0,1)+0.5; kk = per-head L2-normalised N(0,1), a = -kk,
    b = kk*sigmoid(N(0,1)); s0[B,H,N,N] ~ N(0,0.1) fp32; upstream dy ~ N(0,1) bf16, dsT ~ N(0,0.1) fp32."""
    g = _gen(seed)
    bf = torch.bfloat16
    r, k, v = ((torch.randn(B, T, H, N, generator=g) * 0.5).to(bf) for _ in range(3))
    w = (torch.randn(B, T, H, N, generator=g) + 0.5).to(bf)
    kk = torch.nn.functional.normalize(torch.randn(B, T, H, N, generator=g), dim=-1, p=2.0)
    a = (-kk).to(bf)
    b = (kk * torch.sigmoid(torch.randn(B, T, H, N, generator=g))).to(bf)
    s0 = torch.randn(B, H, N, N, generator=g) * 0.1
    dy = torch.randn(B, T, H, N, generator=g).to(bf)
    dsT = torch.randn(B, H, N, N, generator=g) * 0.1
    return s0, r, w, k, v, a, b, dy, dsT
