"""GPU parity: wkv5a (two-sided decay and bonus, fp32) through the C ABI and its autograd wrapper
against the fp64 oracle.  Bar for this fp32 path: rms error ratio <= 1e-5 on every output."""
import pytest
import torch

from oracle import wkv5a as A
from oracle import err_ratio
from rwkv_cuda_amd import wkv5a
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, garbage

pytestmark = pytest.mark.gpu
TOL = 1e-5
NAMES = ["y", "gr", "gk", "gv", "gw1", "gu1", "gw2", "gu2"]


def reference_style_inputs(B, T, H, seed, w_lo=-8.0):
    """r,k,v,u ~ uniform(-1,1), raw w ~ uniform(-8,1) as the reference's check draws them
    (wkv5a/run.py:389-398); gy likewise uniform(-1,1)."""
    g = torch.Generator().manual_seed(seed)
    C = H * 64
    rnd = lambda *s, lo=-1.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo
    return (rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(H, 64, lo=w_lo), rnd(H, 64), rnd(H, 64, lo=w_lo), rnd(H, 64),
            rnd(B, T, C))


def check(ref, got, skip=()):
    for name, a, g in zip(NAMES, ref, got):
        if name in skip:
            continue
        e = err_ratio(a, g.detach().double().cpu().reshape(a.shape))
        print(f"  {name}: {e:.3e}", flush=True)
        assert e <= TOL, f"{name}: {e:.3e}"


@pytest.mark.parametrize("B,T,H", [(2, 50, 2), (1, 97, 3), (2, 64, 1), (3, 1, 1), (1, 7, 2)])
def test_wkv5a_c_abi_write_coverage(lib, B, T, H):
    print(f"\nwkv5a C-ABI B={B} T={T} H={H}", flush=True)
    C = H * 64
    r, k, v, w1, u1, w2, u2, gy = reference_style_inputs(B, T, H, seed=41)
    ref = A.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy, per_batch=True)
    ew1, ew2 = -torch.exp(w1), -torch.exp(w2)
    d = [x.to(DEV).contiguous() for x in (r, k, v, torch.exp(ew1), ew1, u1, torch.exp(ew2), ew2, u2, gy)]
    f32 = torch.float32
    y = garbage((B, T, C), f32)
    call("rwkv_wkv5a_forward", d[0].device, B, T, C, H, d[0], d[1], d[2], d[3], d[5], d[6], d[8], y)
    gr, gk, gv = (garbage((B, T, C), f32) for _ in range(3))
    gw1, gu1, gw2, gu2 = (garbage((B, C), f32) for _ in range(4))
    call("rwkv_wkv5a_backward", d[0].device, B, T, C, H, *d, gr, gk, gv, gw1, gu1, gw2, gu2)
    torch.cuda.synchronize()
    if T == 1:                                   # one step: the decays feed nothing
        assert float(gw1.abs().max()) == 0.0 and float(gw2.abs().max()) == 0.0
    check(ref, [y, gr, gk, gv, gw1, gu1, gw2, gu2], skip=("gw1", "gw2") if T == 1 else ())


def test_wkv5a_autograd_long(lib):
    B, T, H = 1, 1024, 2
    C = H * 64
    r, k, v, w1, u1, w2, u2, gy = reference_style_inputs(B, T, H, seed=42, w_lo=-5.0)
    ref = A.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w1, u1, w2, u2)]
    y = wkv5a.CUDA_1(*t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    check(ref, [y] + [x.grad for x in t])


def test_wkv5a_with_neutral_second_side_is_wkv5(lib):
    """decay 1 and bonus 0 on the second side: the fp32 wkv5 op on the same inputs, bit for bit in y
    (the same kernels, the same operation order)."""
    from rwkv_cuda_amd import wkv5
    B, T, H = 2, 70, 2
    C = H * 64
    r, k, v, w1, u1, _, _, _ = reference_style_inputs(B, T, H, seed=43)
    d = lambda x: x.to(DEV)
    w2 = torch.full((H, 64), -200.0)             # exp(-exp(-200)) == 1 in fp32
    ya = wkv5a.CUDA_1(d(r), d(k), d(v), d(w1), d(u1), d(w2), d(torch.zeros(H, 64)))
    y5 = wkv5.RUN_CUDA(B, T, C, H, d(r), d(k), d(v), d(w1), d(u1))
    torch.cuda.synchronize()
    assert err_ratio(y5, ya) < 1e-6
