"""GPU parity: the fp32 wkv5 op (wkv5/run.py) through the C ABI and its autograd wrapper against
the fp64 oracle.  Bar for this fp32 path: rms error ratio <= 1e-5 on every output."""
import pytest
import torch

from oracle import wkv56 as O
from oracle import err_ratio
from rwkv_cuda_amd import wkv5
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, garbage

pytestmark = pytest.mark.gpu
TOL = 1e-5


def reference_style_inputs(B, T, C, seed):
    """uniform(-1,1) for r,k,v,w,u as CHECK_CORRECT draws them (wkv5/run.py:516-520); gy likewise."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.rand(*s, generator=g) * 2 - 1
    return rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(C), rnd(C), rnd(B, T, C)


def check(names, ref, got):
    for name, a, g in zip(names, ref, got):
        e = err_ratio(a, g.detach().double().cpu().reshape(a.shape))
        print(f"  {name}: {e:.3e}", flush=True)
        assert e <= TOL, f"{name}: {e:.3e}"


@pytest.mark.parametrize("B,T,H", [(2, 50, 2), (1, 97, 3), (2, 64, 1), (3, 1, 1), (1, 7, 2)])
def test_wkv5_fp32_c_abi_write_coverage(lib, B, T, H):
    print(f"\nwkv5 fp32 C-ABI B={B} T={T} H={H}", flush=True)
    C = H * 64
    r, k, v, w, u, gy = reference_style_inputs(B, T, C, seed=31)
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy, per_batch=True)
    ew = -torch.exp(w)
    d = [x.to(DEV) for x in (r, k, v, torch.exp(ew), ew, u, gy)]
    f32 = torch.float32
    y = garbage((B, T, C), f32)
    call("rwkv_wkv5f32_forward", d[0].device, B, T, C, H, d[0], d[1], d[2], d[3], d[5], y)
    gr, gk, gv = (garbage((B, T, C), f32) for _ in range(3))
    gw, gu = garbage((B, C), f32), garbage((B, C), f32)
    call("rwkv_wkv5f32_backward", d[0].device, B, T, C, H, *d, gr, gk, gv, gw, gu)
    torch.cuda.synchronize()
    names = ["y", "gr", "gk", "gv", "gw", "gu"]
    if T == 1:                                   # one step: the decay feeds nothing
        assert float(gw.abs().max()) == 0.0
        names, ref, got = names[:4] + names[5:], ref[:4] + ref[5:], [y, gr, gk, gv, gu]
    else:
        got = [y, gr, gk, gv, gw, gu]
    check(names, ref, got)


def test_wkv5_fp32_autograd_long(lib):
    """The reference's benchmark head size at a length where the decay-gradient recurrence has run
    for thousands of steps; w,u flat [C] as the reference passes them (wkv5/run.py:519-520)."""
    B, T, H = 1, 2048, 2
    C = H * 64
    r, k, v, w, u, gy = reference_style_inputs(B, T, C, seed=32)
    w = w * 2 - 1.5                               # decays from 0.92 down to 0.2 per step
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    y = wkv5.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    assert t[3].grad.shape == (C,) and t[4].grad.shape == (C,)
    check(["y", "gr", "gk", "gv", "gw", "gu"], ref, [y] + [x.grad for x in t])
