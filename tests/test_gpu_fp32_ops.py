"""GPU parity of the fp32 ops: RWKV-4 wkv and depthwise_conv1d, against the fp64 oracle.
Tolerance (both ops): max|x-y| / max|y| <= 1e-5 and RMS error ratio <= 1e-5."""
import pytest
import torch

from oracle import wkv4 as O4
from oracle import timex as OT
from oracle import err_ratio, max_rel_to_peak
from rwkv_cuda_amd import synth, wkv, depthwise_conv1d
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, garbage

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _check(name, ref, got):
    if float(ref.abs().max()) == 0.0:
        assert float(got.abs().max()) == 0.0, name
        return
    a, b = err_ratio(ref, got.detach().cpu()), max_rel_to_peak(ref, got.detach().cpu())
    print(f"  {name}: err_ratio {a:.3e}  max/peak {b:.3e}", flush=True)
    assert a <= TOL and b <= TOL, (name, a, b)


# T <= 512: inputs in registers, 16 channels a workgroup; 513..1024: 8 channels a workgroup; up to 32768: blocks of 512
# steps with the state handed on; beyond: the form that parks the ascending sweep's results in memory.  Each boundary
# from both sides, ragged last segments and last blocks, channel counts that leave a workgroup partly empty.
@pytest.mark.parametrize("B,T,C", [(2, 37, 70), (1, 1, 3), (3, 333, 50), (1, 4100, 20), (4, 512, 768),
                                   (2, 511, 17), (2, 513, 17), (1, 1000, 9), (2, 1024, 40), (2, 1025, 40), (1, 64, 8), (1, 65, 33),
                                   (2, 1536, 33), (1, 2048, 16), (1, 2049, 7), (1, 33000, 3)])
def test_wkv4(lib, B, T, C):
    print(f"\nwkv4 B={B} T={T} C={C}", flush=True)
    w_raw, u, k, v, gy = synth.wkv4_inputs(B, T, C, seed=21)
    ref = O4.grads(B, T, C, w_raw, u, k, v, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (w_raw, u, k, v)]
    y = wkv.WKV.apply(B, T, C, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, g in zip(["y", "gw", "gu", "gk", "gv"], ref, [y] + [x.grad for x in t]):
        _check(name, a, g)


@pytest.mark.parametrize("seed", range(10))
def test_wkv4_random_shapes(lib, seed):
    """Shapes drawn at random across the four kernel forms, through the reference-signature entry points (w = -exp(w_raw)
    in, per-batch gw, gu added into zeroed buffers) instead of the fused ones that the autograd wrapper uses."""
    g = torch.Generator().manual_seed(1000 + seed)
    B = int(torch.randint(1, 5, (1,), generator=g))
    T = int(torch.randint(1, [40, 600, 1100, 2600][seed % 4], (1,), generator=g))
    C = int(torch.randint(1, 90, (1,), generator=g))
    print(f"\nwkv4 random B={B} T={T} C={C}", flush=True)
    w_raw, u, k, v, gy = synth.wkv4_inputs(B, T, C, seed=seed)
    ref = O4.grads(B, T, C, w_raw, u, k, v, gy)
    d = [x.to(DEV) for x in (-torch.exp(w_raw), u, k, v, gy)]
    y, gk, gv = (garbage((B, T, C), torch.float32) for _ in range(3))
    gw, gu = torch.zeros(B, C, device=DEV), torch.zeros(B, C, device=DEV)
    n = lib.rwkv_wkv4_backward_workspace_bytes(B, T, C)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv4_forward", d[0].device, B, T, C, d[0], d[1], d[2], d[3], y)
    call("rwkv_wkv4_backward", d[0].device, B, T, C, *d, gw, gu, gk, gv, ws, n)
    torch.cuda.synchronize()
    for name, a, got in zip(["y", "gw", "gu", "gk", "gv"], ref, [y, gw.sum(0), gu.sum(0), gk, gv]):
        _check(name, a, got)


def test_wkv4_more_batch_rows_than_a_grid_dimension(lib):
    """B > 65535 takes the one-lane-per-scan kernels (the time-parallel ones put B on the grid's y axis)."""
    B, T, C = 65536, 3, 1
    w_raw, u, k, v, gy = synth.wkv4_inputs(B, T, C, seed=25)
    ref = O4.grads(B, T, C, w_raw, u, k, v, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (w_raw, u, k, v)]
    y = wkv.WKV.apply(B, T, C, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, g in zip(["y", "gw", "gu", "gk", "gv"], ref, [y] + [x.grad for x in t]):
        _check(name, a, g)


def test_wkv4_extreme_k_stays_finite(lib):
    """k ~ U(-1000,1000): the stabilised kernel must not overflow (wkv/run.py:159-169)."""
    B, T, C = 2, 64, 128
    w_raw, u, k, v, gy = synth.wkv4_inputs(B, T, C, seed=22)
    k = torch.rand(B, T, C, generator=torch.Generator().manual_seed(1)) * 2000 - 1000
    y = wkv.WKV.apply(B, T, C, w_raw.to(DEV), u.to(DEV), k.to(DEV), v.to(DEV))
    ref = O4.streaming(B, T, C, -torch.exp(w_raw.double()), u.double(), k.double(), v.double())
    assert torch.isfinite(y).all()
    # exponents of magnitude 1000 carry an absolute fp32 rounding error of ~6e-5 before exp(), in
    # any fp32 implementation, so the 1e-5 bar of the ordinary range does not apply here
    e = err_ratio(ref, y.cpu())
    print(f"  y: err_ratio {e:.3e}", flush=True)
    assert e < 1e-3


# the last two: T above the matrix-core kernels' limit (VALU kernels, 1024 threads, near the LDS limit), T % 32 != 0 and T = T_MAX
# T % 32 == 0 up to 1024 with 8 or more batch rows runs on the matrix cores with two-term fp16 products (one tile, a
# ragged last group of 32 rows, a last pass of one row for the batch-summed gradient, the longest T)
@pytest.mark.parametrize("B,C,T", [(3, 5, 64), (9, 2, 4), (40, 3, 96), (17, 2, 1024), (32, 768, 768), (3, 2, 1100), (2, 3, 4096),
                                   (8, 3, 32), (9, 2, 64), (33, 2, 736), (17, 5, 768), (48, 2, 128), (16, 1, 800),
                                   (9, 3, 992), (40, 2, 1024), (8, 2, 96), (70, 1, 160)])
def test_timex(lib, B, C, T):
    print(f"\ntimex B={B} C={C} T={T}", flush=True)
    w, k, g = synth.timex_inputs(B, C, T, seed=23)
    eps = 0.25
    d = [x.to(DEV) for x in (w, k, g)]
    x = garbage((B, C, T), torch.float32)
    call("rwkv_timex_forward", d[0].device, d[0], d[1], x, eps, B, C, T)
    gw = garbage((B, C, T), torch.float32)
    gk = garbage((B, C, T), torch.float32)
    call("rwkv_timex_backward", d[0].device, d[0], d[1], d[2], gw, gk, B, C, T)
    torch.cuda.synchronize()
    cs = slice(0, min(C, 48))                 # channels are independent: an exact check on a subset
    ref = OT.grads(w[cs], k[:, cs], g[:, cs], B, cs.stop, T)
    _check("x", ref[0] + eps, x[:, cs])
    _check("gw", ref[1], gw.sum(0)[cs])
    _check("gk", ref[2], gk[:, cs])
    if T % 32 == 0 and T <= 1024:             # the entry point that sums gw over the batch itself
        gws = garbage((C, T), torch.float32)
        gk2 = garbage((B, C, T), torch.float32)
        call("rwkv_timex_backward_sum", d[0].device, d[0], d[1], d[2], gws, gk2, B, C, T)
        again = garbage((C, T), torch.float32)
        call("rwkv_timex_backward_sum", d[0].device, d[0], d[1], d[2], again, gk2, B, C, T)
        torch.cuda.synchronize()
        _check("gw summed in the kernel", ref[1], gws[cs])
        assert torch.equal(gk2, gk) and torch.equal(gws, again)
    if T <= 64:                               # per-batch gw against the closed form
        gwb, _ = OT.grads_closed_form(w.double(), k.double(), g.double(), B, C, T)
        _check("gw per batch", gwb, gw)


def test_timex_rows_of_very_different_size(lib):
    """The matrix-core kernels bring a unit's rows into the range of fp16 with one power of two per unit (32 batch rows of a
    channel; 16 rows of both tensors per pass of the batch-summed gradient).  Rows up to 1e4 smaller than their neighbours,
    a kernel row near 1e6 and gradients near 1e-7: every batch row on the 1e-5 bar by itself."""
    B, C, T = 40, 3, 96
    w, k, g = synth.timex_inputs(B, C, T, seed=26)
    gen = torch.Generator().manual_seed(27)
    w = w * 3.0e5
    k = k * 10.0 ** (-4.0 * torch.rand(B, 1, 1, generator=gen))
    g = g * 1.0e-7 * 10.0 ** (-4.0 * torch.rand(B, 1, 1, generator=gen))
    d = [x.to(DEV) for x in (w, k, g)]
    x = garbage((B, C, T), torch.float32)
    call("rwkv_timex_forward", d[0].device, d[0], d[1], x, 0.0, B, C, T)
    gws = garbage((C, T), torch.float32)
    gk = garbage((B, C, T), torch.float32)
    call("rwkv_timex_backward_sum", d[0].device, d[0], d[1], d[2], gws, gk, B, C, T)
    torch.cuda.synchronize()
    ref = OT.grads(w, k, g, B, C, T)
    for b in range(B):
        _check(f"x, batch row {b}", ref[0][b], x[b])
        _check(f"gk, batch row {b}", ref[2][b], gk[b])
    _check("gw summed in the kernel", ref[1], gws)


def test_timex_autograd_and_impulse(lib):
    B, C, T = 8, 6, 32
    w, k, g = synth.timex_inputs(B, C, T, seed=24)
    wd = w.to(DEV).requires_grad_(True)
    kd = k.to(DEV).requires_grad_(True)
    out = depthwise_conv1d.TimeX.apply(wd, kd, B, C, T, 0.0)
    out.backward(g.to(DEV))
    ref = OT.grads(w, k, g, B, C, T)
    for name, a, got in zip(["x", "gw", "gk"], ref, [out, wd.grad, kd.grad]):
        _check(name, a, got)
    u = 5
    imp = torch.zeros(B, C, T)
    imp[:, :, u] = 1.0
    out = depthwise_conv1d.TimeX.apply(w.to(DEV), imp.to(DEV), B, C, T, 0.0).cpu()
    for t in range(T):
        expect = w[:, T - 1 - (t - u)] if t >= u else torch.zeros(C)
        # (the matrix-core kernels carry 22 bits of every operand: two fp16 terms.  An impulse therefore returns the taps to
        #  2^-22 of the largest one; the bar for the fp32 operators is 1e-5)
        assert (out[0, :, t] - expect).abs().max() <= 2.0 ** -22 * float(w.abs().max())
