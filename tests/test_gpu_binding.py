"""GPU: the reference-style extension (csrc/binding.cpp, built with torch.utils.cpp_extension) against the ctypes path.

A driver of BlinkDL/RWKV-CUDA calls `ext.forward(B,T,C,H,r,k,v,w,u,s,y)` on the pybind module that `load()` returns
(wkv6_state/run.py:77,103,122) or `torch.ops.<lib>.forward(...)` (rwkv7_cuda_benchmark_state_passing.py:87,98).  Both
routes must give bit for bit what the same C-ABI entry point gives through ctypes: the shim adds no arithmetic."""
import pytest
import torch

from rwkv_cuda_amd import binding, synth
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.fixture(scope="module")
def ext(lib):
    return binding.load()


def test_wkv6state_pybind_and_torch_ops_match_ctypes(lib, ext):
    B, T, H = 2, 70, 2
    C = H * 64
    r, k, v, w, u, gy, s0 = (x.to(DEV) for x in synth.wkv6_inputs(B, T, C, H, seed=61, state=True))
    n = lib.rwkv_wkv6state_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)

    def outputs():
        return [garbage((B, T, C), BF) for _ in range(5)] + [garbage((B, C), BF), garbage((B, H, 64, 64), BF)]

    y0, gr0, gk0, gv0, gw0, gu0, gs0 = outputs()
    call("rwkv_wkv6state_forward", r.device, B, T, C, H, r, k, v, w, u, s0, y0)
    call("rwkv_wkv6state_backward", r.device, B, T, C, H, r, k, v, w, u, s0, gy, gr0, gk0, gv0, gw0, gu0, gs0, ws, n)
    for route in ("pybind", "torch.ops"):
        print(f"\nwkv6state via {route}", flush=True)
        y, gr, gk, gv, gw, gu, gs = outputs()
        if route == "pybind":
            ext.wkv6state.forward(B, T, C, H, r, k, v, w, u, s0, y)
            ext.wkv6state.backward(B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu, gs)
        else:
            torch.ops.wkv6b.forward(B, T, C, H, r, k, v, w, u, s0, y)
            torch.ops.wkv6b.backward(B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu, gs)
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "gr", "gk", "gv", "gw", "gu", "gs"), (y0, gr0, gk0, gv0, gw0, gu0, gs0), (y, gr, gk, gv, gw, gu, gs)):
            assert torch.equal(a, b), (route, name)


@pytest.mark.parametrize("dtype", [BF, torch.float32])
def test_rwkv7_statepassing_torch_ops_match_ctypes(lib, ext, dtype):
    B, T, H, N = 2, 48, 2, 64
    s0, r, w, k, v, a, b, dy, dsT = (x.to(DEV) for x in synth.rwkv7_inputs(B, T, H, N, seed=62))
    if dtype == torch.float32:
        r, w, k, v, a, b, dy = (x.float() for x in (r, w, k, v, a, b, dy))
    sfx = "_f32" if dtype == torch.float32 else ""
    f32 = dict(device=DEV, dtype=torch.float32)

    def run(via_ops):
        y = garbage((B, T, H, N), dtype)
        sT = garbage((B, H, N, N), torch.float32)
        s = torch.empty(B, H, T // 16, N, N, **f32)
        sa = torch.empty(B, T, H, N, **f32)
        grads = [garbage((B, T, H, N), dtype) for _ in range(6)]
        ds0 = garbage((B, H, N, N), torch.float32)
        if via_ops:
            torch.ops.rwkv7_statepassing_clampw.forward(s0, r, w, k, v, a, b, y, sT, s, sa)
            torch.ops.rwkv7_statepassing_clampw.backward(r, w, k, v, a, b, dy, dsT, s, sa, ds0, *grads)
        else:
            call("rwkv7_statepassing_forward" + sfx, r.device, B, T, H, s0, r, w, k, v, a, b, y, sT, s, sa)
            call("rwkv7_statepassing_backward" + sfx, r.device, B, T, H, r, w, k, v, a, b, dy, dsT, s, sa, ds0, *grads)
        torch.cuda.synchronize()
        return [y, sT, ds0] + grads

    for name, x, z in zip(("y", "sT", "ds0", "dr", "dw", "dk", "dv", "da", "db"), run(False), run(True)):
        assert torch.equal(x, z), name


def test_remaining_extensions_match_ctypes(lib, ext):
    # wkv (RWKV-4)
    B, T, C = 2, 40, 48
    w_raw, u, k, v, gy = (x.to(DEV) for x in synth.wkv4_inputs(B, T, C, seed=63))
    w = -torch.exp(w_raw)
    n = lib.rwkv_wkv4_backward_workspace_bytes(B, T, C)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    res = []
    for via in (False, True):
        y = garbage((B, T, C), torch.float32)
        gw, gu = torch.zeros(B, C, device=DEV), torch.zeros(B, C, device=DEV)
        gk, gv = garbage((B, T, C), torch.float32), garbage((B, T, C), torch.float32)
        if via:
            ext.wkv.forward(B, T, C, w, u, k, v, y)
            torch.ops.wkv.backward(B, T, C, w, u, k, v, gy, gw, gu, gk, gv)
        else:
            call("rwkv_wkv4_forward", w.device, B, T, C, w, u, k, v, y)
            call("rwkv_wkv4_backward", w.device, B, T, C, w, u, k, v, gy, gw, gu, gk, gv, ws, n)
        torch.cuda.synchronize()
        res.append((y, gw, gu, gk, gv))
    for a, b in zip(*res):
        assert torch.equal(a, b)

    # timex
    B, C, T = 9, 3, 64
    w, k, g = (x.to(DEV) for x in synth.timex_inputs(B, C, T, seed=64))
    res = []
    for via in (False, True):
        x, gw, gk = (garbage((B, C, T), torch.float32) for _ in range(3))
        if via:
            torch.ops.timex.forward(w, k, x, 0.5, B, C, T)
            ext.timex.backward(w, k, g, gw, gk, B, C, T)
        else:
            call("rwkv_timex_forward", w.device, w, k, x, 0.5, B, C, T)
            call("rwkv_timex_backward", w.device, w, k, g, gw, gk, B, C, T)
        torch.cuda.synchronize()
        res.append((x, gw, gk))
    for a, b in zip(*res):
        assert torch.equal(a, b)

    # wkv5 in both element types, wkv6 with the fp32 ew of the reference boundary
    B, T, H = 2, 50, 2
    C = H * 64
    r, k, v, w5, u, gy = (x.to(DEV) for x in synth.wkv5_inputs(B, T, C, H, seed=65))
    for dt, fw, bw in ((BF, "rwkv_wkv5_forward", "rwkv_wkv5_backward"), (torch.float32, "rwkv_wkv5f32_forward", "rwkv_wkv5f32_backward")):
        rr, kk, vv, uu, gg = (x.to(dt) for x in (r, k, v, u, gy))
        ew = (-torch.exp(w5.float())).contiguous().view(-1)
        eew = torch.exp(ew).contiguous()
        res = []
        for via in (False, True):
            y, gr, gk, gv = (garbage((B, T, C), dt) for _ in range(4))
            gw, gu = garbage((B, C), dt), garbage((B, C), dt)
            if via:
                ext.wkv5.forward(B, T, C, H, rr, kk, vv, eew, uu.view(-1), y)
                torch.ops.wkv5.backward(B, T, C, H, rr, kk, vv, eew, ew, uu.view(-1), gg, gr, gk, gv, gw, gu)
            elif dt == BF:
                n = lib.rwkv_wkv5_backward_workspace_bytes(B, T, C, H)
                ws = torch.empty(n, device=DEV, dtype=torch.uint8)
                call(fw, rr.device, B, T, C, H, rr, kk, vv, eew, uu, y)
                call(bw, rr.device, B, T, C, H, rr, kk, vv, eew, ew, uu, gg, gr, gk, gv, gw, gu, ws, n)
            else:
                call(fw, rr.device, B, T, C, H, rr, kk, vv, eew, uu, y)
                call(bw, rr.device, B, T, C, H, rr, kk, vv, eew, ew, uu, gg, gr, gk, gv, gw, gu)
            torch.cuda.synchronize()
            res.append((y, gr, gk, gv, gw, gu))
        for name, a, b in zip("y gr gk gv gw gu".split(), *res):
            assert torch.equal(a, b), (dt, name)

    r, k, v, w6, u, gy, _ = (x.to(DEV) if x is not None else None for x in synth.wkv6_inputs(B, T, C, H, seed=66))
    ew = (-torch.exp(w6.float())).contiguous()
    n = lib.rwkv_wkv6_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    res = []
    for via in (False, True):
        y, gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(5))
        gu = garbage((B, C), BF)
        if via:
            torch.ops.wkv6.forward(B, T, C, H, r, k, v, ew, u, y)
            ext.wkv6.backward(B, T, C, H, r, k, v, ew, u, gy, gr, gk, gv, gw, gu)
        else:
            call("rwkv_wkv6_forward", r.device, B, T, C, H, r, k, v, ew, u, y)
            call("rwkv_wkv6_backward", r.device, B, T, C, H, r, k, v, ew, u, gy, gr, gk, gv, gw, gu, ws, n)
        torch.cuda.synchronize()
        res.append((y, gr, gk, gv, gw, gu))
    for name, a, b in zip("y gr gk gv gw gu".split(), *res):
        assert torch.equal(a, b), name


def test_wkv5_head_size_128_through_the_shim(lib, ext):
    """wkv5_bf16/run.py:21 ships head size 128: the shim allocates the forward's scratch itself (the reference's forward
    takes none) and must give what the C ABI gives with a caller's workspace."""
    B, T, H = 2, 70, 2
    C = H * 128
    r, k, v, w5, u, gy = (x.to(DEV) for x in synth.wkv5_inputs(B, T, C, H, seed=67))
    ew = (-torch.exp(w5.float())).contiguous().view(-1)
    eew = torch.exp(ew).contiguous()
    res = []
    for via in (False, True):
        y, gr, gk, gv = (garbage((B, T, C), BF) for _ in range(4))
        gw, gu = garbage((B, C), BF), garbage((B, C), BF)
        if via:
            ext.wkv5.forward(B, T, C, H, r, k, v, eew, u.view(-1), y)
            torch.ops.wkv5.backward(B, T, C, H, r, k, v, eew, ew, u.view(-1), gy, gr, gk, gv, gw, gu)
        else:
            nf = lib.rwkv_wkv5_forward_workspace_bytes(B, T, C, H)
            n = lib.rwkv_wkv5_backward_workspace_bytes(B, T, C, H)
            assert nf > 0 and n > nf
            fws, ws = torch.empty(nf, device=DEV, dtype=torch.uint8), torch.empty(n, device=DEV, dtype=torch.uint8)
            call("rwkv_wkv5_forward_ws", r.device, B, T, C, H, r, k, v, eew, u, y, fws, nf, 0)
            call("rwkv_wkv5_backward", r.device, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu, ws, n)
        torch.cuda.synchronize()
        res.append((y, gr, gk, gv, gw, gu))
    for name, a, b in zip("y gr gk gv gw gu".split(), *res):
        assert torch.equal(a, b), name


def test_shim_rejects_wrong_dtype_and_cpu_tensors(ext):
    x = torch.zeros(2, 16, 64, device=DEV, dtype=torch.float32)          # bf16 expected
    u = torch.zeros(64, device=DEV, dtype=BF)
    s = torch.zeros(2, 1, 64, 64, device=DEV, dtype=BF)
    with pytest.raises(RuntimeError, match="must be"):
        ext.wkv6state.forward(2, 16, 64, 1, x, x, x, x, u, s, x)
    c = torch.zeros(4)
    with pytest.raises(RuntimeError, match="HIP device"):
        torch.ops.wkv.forward(1, 1, 4, c, c, c, c, c)


def test_shim_is_built_against_the_loaded_abi_and_refuses_sizes_beyond_int(lib, ext):
    assert ext.abi_version == lib.rwkv_abi_version()
    x = torch.zeros(16, device=DEV, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="outside 1 .. 2147483647"):
        ext.wkv.forward(2 ** 31, 1, 1, x, x, x, x, x)               # would be narrowed to a negative int
    with pytest.raises(RuntimeError, match="outside 1 .. 2147483647"):
        ext.wkv6.forward(1, 0, 64, 1, x, x, x, x, x, x)
