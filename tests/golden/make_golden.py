"""Writes the golden fixtures of this directory from the CPU oracle (fp64), with fixed seeds.

    python tests/golden/make_golden.py

The reference repository holds no stored vectors for these kernels (its drivers compare live GPU
results), so the fixtures are the oracle's own output, frozen: tests/test_golden.py checks that the
oracle still reproduces them (a change in the oracle is then a visible diff of this directory, not
a silent shift of the bar), and tests/test_gpu_golden.py runs the HIP kernels on the stored inputs.
Inputs are stored in the dtype the op takes (bf16 as uint16 bit patterns); expected outputs as fp64.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import rwkv7 as O7, timex as OT, wkv4 as O4, wkv5a as O5A, wkv56 as O  # noqa: E402
from rwkv_cuda_amd import synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def store(x):
    """bf16 tensors as their uint16 bit patterns (numpy has no bfloat16); everything else as is."""
    if x.dtype == torch.bfloat16:
        return x.view(torch.int16).numpy().view(np.uint16)
    return x.numpy()


def cases():
    B, T, H = 2, 32, 1
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=901, state=True)
    names = ["y", "gr", "gk", "gv", "gw", "gu", "gs"]
    yield "wkv6_state_B2_T32_H1", dict(r=r, k=k, v=v, w=w, u=u, s0=s0, gy=gy), \
        dict(zip(names, O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)))
    yield "wkv6_B2_T32_H1", dict(r=r, k=k, v=v, w=w, u=u, gy=gy), \
        dict(zip(names[:6], O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy)))
    r, k, v, w5, u, gy = synth.wkv5_inputs(B, T, C, H, seed=902)
    yield "wkv5_B2_T32_H1", dict(r=r, k=k, v=v, w=w5, u=u, gy=gy), \
        dict(zip(names[:6], O.wkv5_grads(B, T, C, H, r, k, v, w5, u, gy)))
    g = torch.Generator().manual_seed(903)
    rnd = lambda *s, lo=-1.0: torch.rand(*s, generator=g) * (1.0 - lo) + lo
    a = dict(r=rnd(1, 24, 64), k=rnd(1, 24, 64), v=rnd(1, 24, 64), w1=rnd(1, 64, lo=-8.0), u1=rnd(1, 64),
             w2=rnd(1, 64, lo=-8.0), u2=rnd(1, 64), gy=rnd(1, 24, 64))
    out = O5A.grads(1, 24, 64, 1, a["r"], a["k"], a["v"], a["w1"], a["u1"], a["w2"], a["u2"], a["gy"])
    yield "wkv5a_B1_T24_H1", a, dict(zip(["y", "gr", "gk", "gv", "gw1", "gu1", "gw2", "gu2"], out))
    w_raw, u4, k4, v4, gy4 = synth.wkv4_inputs(2, 32, 16, seed=904)
    yield "wkv4_B2_T32_C16", dict(w=w_raw, u=u4, k=k4, v=v4, gy=gy4), \
        dict(zip(["y", "gw", "gu", "gk", "gv"], O4.grads(2, 32, 16, w_raw, u4, k4, v4, gy4)))
    g = torch.Generator().manual_seed(905)
    wt, kt, gt = torch.randn(4, 32, generator=g), torch.randn(2, 4, 32, generator=g), torch.randn(2, 4, 32, generator=g)
    gw_t, gk_t = OT.grads_closed_form(wt.double(), kt.double(), gt.double(), 2, 4, 32)     # gw per batch row
    yield "timex_B2_C4_T32", dict(w=wt, k=kt, gwk=gt), \
        dict(y=OT.toeplitz_form(wt.double(), kt.double(), 2, 4, 32, 0.25), gw=gw_t, gk=gk_t)
    args = synth.rwkv7_inputs(1, 32, 1, 64, seed=906)
    yield "rwkv7_B1_T32_H1", dict(zip(["s0", "r", "w", "k", "v", "a", "b", "dy", "dsT"], args)), \
        dict(zip(["y", "sT", "ds0", "dr", "dw", "dk", "dv", "da", "db"], O7.grads(*args)))


def main():
    for name, inputs, expected in cases():
        data = {"in_" + k: store(v) for k, v in inputs.items()}
        data.update({"bf16_" + k: np.array(v.dtype == torch.bfloat16) for k, v in inputs.items()})
        data.update({"out_" + k: v.detach().double().numpy() for k, v in expected.items()})
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
        print(name, {k: tuple(v.shape) for k, v in expected.items()})


if __name__ == "__main__":
    main()
