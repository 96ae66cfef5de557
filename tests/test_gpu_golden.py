"""GPU: the HIP kernels on the stored golden inputs against the stored fp64 results (tests/golden/*.npz).
Nothing here computes a reference at run time.  Bars: bf16 ops rms error ratio <= 5e-3 (their outputs carry
2^-9 relative rounding: 1.7e-3 rms on tensors, up to 3e-3 on summed parameter gradients); fp32 ops <= 1e-5."""
import os

import numpy as np
import pytest
import torch

from oracle import err_ratio
from rwkv_cuda_amd import depthwise_conv1d, rwkv7_fast_fused, wkv, wkv5_bf16, wkv5a, wkv6, wkv6_state
from _gpu_util import DEV

pytestmark = pytest.mark.gpu
HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
BF_TOL, F32_TOL = 5e-3, 1e-5


def load(name):
    f = np.load(os.path.join(HERE, name + ".npz"))
    ins, outs = {}, {}
    for key in f.files:
        if key.startswith("in_"):
            k = key[3:]
            a = f[key]
            if bool(f["bf16_" + k]):
                ins[k] = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(DEV)
            else:
                ins[k] = torch.from_numpy(a.copy()).to(DEV)
        elif key.startswith("out_"):
            outs[key[4:]] = torch.from_numpy(f[key])
    return ins, outs


def compare(name, outs, got, tol):
    for k, want in outs.items():
        e = err_ratio(want, got[k].detach().double().cpu().reshape(want.shape))
        print(f"  {name} {k}: {e:.3e}", flush=True)
        assert e <= tol, (name, k, e)


def test_wkv6_state_and_wkv6(lib):
    for name, with_state in (("wkv6_state_B2_T32_H1", True), ("wkv6_B2_T32_H1", False)):
        i, o = load(name)
        B, T, C = i["r"].shape
        H = C // 64
        t = [i[k].requires_grad_(True) for k in (["r", "k", "v", "w", "u"] + (["s0"] if with_state else []))]
        y = (wkv6_state if with_state else wkv6).RUN_CUDA(B, T, C, H, *t)
        y.backward(i["gy"])
        torch.cuda.synchronize()
        got = dict(zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], [y] + [x.grad for x in t]))
        compare(name, o, got, BF_TOL)


def test_wkv5_and_wkv5a(lib):
    i, o = load("wkv5_B2_T32_H1")
    B, T, C = i["r"].shape
    t = [i[k].requires_grad_(True) for k in ("r", "k", "v", "w", "u")]
    y = wkv5_bf16.RUN_CUDA(B, T, C, C // 64, *t)
    y.backward(i["gy"])
    torch.cuda.synchronize()
    compare("wkv5", o, dict(zip(["y", "gr", "gk", "gv", "gw", "gu"], [y] + [x.grad for x in t])), BF_TOL)
    i, o = load("wkv5a_B1_T24_H1")
    t = [i[k].requires_grad_(True) for k in ("r", "k", "v", "w1", "u1", "w2", "u2")]
    y = wkv5a.CUDA_1(*t)
    y.backward(i["gy"])
    torch.cuda.synchronize()
    compare("wkv5a", o, dict(zip(["y", "gr", "gk", "gv", "gw1", "gu1", "gw2", "gu2"], [y] + [x.grad for x in t])), F32_TOL)


def test_wkv4_and_timex(lib):
    i, o = load("wkv4_B2_T32_C16")
    B, T, C = i["k"].shape
    t = [i[k].requires_grad_(True) for k in ("w", "u", "k", "v")]
    y = wkv.WKV.apply(B, T, C, *t)
    y.backward(i["gy"])
    torch.cuda.synchronize()
    compare("wkv4", o, dict(zip(["y", "gw", "gu", "gk", "gv"], [y] + [x.grad for x in t])), F32_TOL)
    i, o = load("timex_B2_C4_T32")
    B, C, T = i["k"].shape
    w, k = i["w"].requires_grad_(True), i["k"].requires_grad_(True)
    y = depthwise_conv1d.TimeX.apply(w, k, B, C, T, 0.25)
    y.backward(i["gwk"])
    torch.cuda.synchronize()
    o["gw"] = o["gw"].sum(0)                       # the fixture holds per-batch rows; the op returns their sum
    compare("timex", o, dict(y=y, gw=w.grad, gk=k.grad), F32_TOL)


def test_rwkv7(lib):
    i, o = load("rwkv7_B1_T32_H1")
    B, T, H, N = i["r"].shape
    t = [i[k].requires_grad_(True) for k in ("s0", "r", "w", "k", "v", "a", "b")]
    y, sT = rwkv7_fast_fused.RWKV7_STATE_PASSING_CLAMPW_CUDA(t[0], *(x.view(B, T, H * N) for x in t[1:]))
    torch.autograd.backward([y, sT], [i["dy"].view(B, T, H * N), i["dsT"]])
    torch.cuda.synchronize()
    got = dict(zip(["y", "sT", "ds0", "dr", "dw", "dk", "dv", "da", "db"], [y.view(B, T, H, N), sT] + [x.grad for x in t]))
    for k in ("sT", "ds0"):                        # fp32 state tensors
        compare("rwkv7", {k: o.pop(k)}, got, 1e-4)
    compare("rwkv7", o, got, BF_TOL)
