"""GPU: the chunked matrix-core kernels against the sequential fp32 sweeps on random shapes and decay strengths.

Both algorithms round the same quantities to bf16, so they may differ by one bf16 unit of the value (2^-8 relative to the value, under 2^-7 of the tensor's peak);
a slip in the chunk logic (a partial last chunk, the exact-path switch, state passing) shows up as an error of order one.
Every result is also checked against the fp64 oracle with the usual bar."""
import random

import pytest
import torch

from oracle import wkv56 as O
from rwkv_cuda_amd import options, synth
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, assert_no_worse, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _run(lib, algo, B, T, C, H, d):
    flags = options.FLAG_SWEEPS if algo else 0
    y = garbage((B, T, C), BF)
    call("rwkv_wkv6state_forward_ex", d[0].device, B, T, C, H, *d[:6], y, flags)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu = garbage((B, C), BF)
    gs = garbage((B, H, 64, 64), BF)
    n = lib.rwkv_wkv6state_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(max(n, 16), device=DEV, dtype=torch.uint8)
    call("rwkv_wkv6state_backward_ex", d[0].device, B, T, C, H, *d[:6], d[6], gr, gk, gv, gw, gu, gs, ws, n, flags)
    torch.cuda.synchronize()
    return [y, gr, gk, gv, gw, gu.sum(0).view(H, 64), gs]


@pytest.mark.parametrize("seed", range(8))
def test_wkv6_state_chunked_equals_sweeps(lib, seed):
    rng = random.Random(seed)
    B, H, T = rng.randint(1, 3), rng.randint(1, 3), rng.choice([rng.randint(1, 31), rng.randint(32, 200), 32 * rng.randint(1, 5)])
    C = H * 64
    print(f"\nseed {seed}: B={B} T={T} H={H}", flush=True)
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=100 + seed, state=True)
    if seed % 2:
        # Single tokens whose decay is strong.  w_raw = 4.5 (the state loses e^-90 in one step) is beyond what the mid-point
        # factors of a half-chunk may span, so that chunk takes the exact path: about one hit per two chunks and head, exact
        # and chunked chunks alternate.  w_raw = 2.5 (e^-12) stays on the chunked path with factors of e^+-12.
        g = torch.Generator().manual_seed(seed)
        pick = torch.rand(B, T, C, generator=g)
        w = torch.where(pick < 0.0002, torch.full_like(w, 4.5), w)
        w = torch.where((pick >= 0.0002) & (pick < 0.0006), torch.full_like(w, 2.5), w)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    d = [x.to(DEV) for x in (r, k, v, w, u, s0, gy)]
    chunked = _run(lib, 0, B, T, C, H, d)
    sweeps = _run(lib, 1, B, T, C, H, d)
    for name, a, e, c, s in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, chunked, sweeps):
        assert_no_worse(name + " (chunked)", a, e, c)
        peak = float(a.abs().max())
        if peak > 0.0:
            diff = float((c.float() - s.float()).abs().max()) / peak
            print(f"  {name}: chunked vs sweeps, max difference / peak {diff:.3e}", flush=True)
            assert diff <= 2.0 ** -7, (name, diff)


REGIMES = ["wide", "alternating", "tiny", "zero_k", "big_u", "large_inputs"]


@pytest.mark.parametrize("regime", REGIMES)
@pytest.mark.parametrize("algo", [0, 1])
def test_wkv6_state_input_regimes(lib, algo, regime):
    """Input regimes away from the benchmark's: decays spread over exp(-exp(-18..12)) (every chunk on the exact path,
    many decays exactly 0 or 1), decays alternating between almost 0 and almost 1 token by token, no decay at all,
    k = 0 (the state never changes), a bonus of order 10, inputs of order 8."""
    rng = random.Random(REGIMES.index(regime))
    B, H, T = rng.randint(1, 2), rng.randint(1, 2), rng.choice([5, 33, 64, 100])
    C = H * 64
    print(f"\nregime {regime} algo={algo} B={B} T={T} H={H}", flush=True)
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=300 + REGIMES.index(regime), state=True)
    g = torch.Generator().manual_seed(7)
    if regime == "wide":
        w = (torch.rand(B, T, C, generator=g) * 30 - 18).to(BF)
    elif regime == "alternating":
        w = torch.full((B, T, C), -6.0)
        w[:, ::2] = 3.5
        w[:, :, ::3] = -1.0
        w = w.to(BF)
    elif regime == "tiny":
        w = torch.full((B, T, C), -25.0).to(BF)
    elif regime == "zero_k":
        k = torch.zeros_like(k)
    elif regime == "big_u":
        u = (u.float() * 30).to(BF)
    elif regime == "large_inputs":
        r, k, v, gy, s0 = ((x.float() * 16).to(BF) for x in (r, k, v, gy, s0))
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    d = [x.to(DEV) for x in (r, k, v, w, u, s0, gy)]
    got = _run(lib, algo, B, T, C, H, d)
    for name, a, e, q in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, got):
        assert torch.isfinite(q.float()).all(), name
        assert_no_worse(name, a, e, q)
