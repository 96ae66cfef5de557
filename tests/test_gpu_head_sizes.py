"""GPU: head sizes other than 64.

The reference compiles its kernels with -D_N_=HEAD_SIZE: wkv5_bf16/run.py:21 ships 128, the self-checks of
wkv5/run.py:366, wkv6/run.py:35 and wkv6_state/run.py:39 use 2 and 4, wkv5a/run.py:60 lists 17.  Here head size 64 takes
the matrix-core kernels, bf16 wkv5 with head size 128 the same kernels with every head as four heads of 64, and every other
case up to 128 the row-per-thread kernels of csrc/wkv56.hip (`wkv_rows`); the bar is the one of the 64-wide kernels: fp64
oracle, bf16 ops no worse than the reference kernel's arithmetic, fp32 ops 1e-5."""
import pytest
import torch

from oracle import wkv56 as O
from oracle import err_ratio
from oracle import wkv5a as A5
from rwkv_cuda_amd import synth, wkv5_bf16, wkv5a, wkv6, wkv6_state
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, assert_no_worse, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
SIZES = [2, 4, 8, 17, 32, 48, 128]
SWEEPS = 0x100                      # RWKV_FLAG_SWEEPS


@pytest.mark.parametrize("N", SIZES)
def test_wkv5_bf16_any_head_size(lib, N):
    B, T, H = 2, 37, 3
    C = H * N
    print(f"\nwkv5 bf16 N={N} B={B} T={T} H={H}", flush=True)
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=200 + N)
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse(f"wkv5 N={N} {name}", a, e.reshape(a.shape), g.reshape(a.shape))


@pytest.mark.parametrize("state", [False, True])
@pytest.mark.parametrize("N", SIZES)
def test_wkv6_any_head_size(lib, N, state):
    B, T, H = 2, 41, 2
    C = H * N
    print(f"\nwkv6 N={N} state={state} B={B} T={T} H={H}", flush=True)
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=300 + N, state=state)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    ins = (r, k, v, w, u, s0) if state else (r, k, v, w, u)
    t = [x.to(DEV).requires_grad_(True) for x in ins]
    y = (wkv6_state if state else wkv6).RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    names = ["y", "gr", "gk", "gv", "gw", "gu"] + (["gs"] if state else [])
    for name, a, e, g in zip(names, ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse(f"wkv6 N={N} {name}", a, e.reshape(a.shape), g.reshape(a.shape))
    if not state:
        assert float(t[3].grad[:, 0].abs().max()) == 0.0          # no state before the first token: an exact zero


@pytest.mark.parametrize("T", [1, 16, 33])
def test_wkv6_state_short_sequences_head_size_8(lib, T):
    """One step, exactly one staged chunk of 16 steps, and two chunks and a step."""
    B, H, N = 3, 2, 8
    C = H * N
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=700 + T, state=True)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u, s0)]
    y = wkv6_state.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse(f"wkv6_state N=8 T={T} {name}", a, e.reshape(a.shape), g.reshape(a.shape))


@pytest.mark.parametrize("N", [2, 17, 128])
def test_wkv6_fp32_ew_interface_any_head_size(lib, N):
    """The reference's own signature (fp32 ew = -exp(w), per-batch gu; wkv6/cuda/wkv6_op.cpp:5-6) with garbage-filled outputs."""
    B, T, H = 2, 19, 2
    C = H * N
    r, k, v, w, u, gy, _ = synth.wkv6_inputs(B, T, C, H, seed=400 + N)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, per_batch=True)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy)
    d = [x.to(DEV) for x in (r, k, v, w, u, gy)]
    ew = (-torch.exp(d[3].float())).contiguous()
    y, gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(5))
    gu = garbage((B, C), BF)
    n = lib.rwkv_wkv6_backward_workspace_bytes(B, T, C, H)
    assert n >= B * T * C * 4
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv6_forward", d[0].device, B, T, C, H, d[0], d[1], d[2], ew, d[4], y)
    call("rwkv_wkv6_backward", d[0].device, B, T, C, H, d[0], d[1], d[2], ew, d[4], d[5], gr, gk, gv, gw, gu, ws, n)
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw"], ref, emu, [y, gr, gk, gv, gw]):
        assert_no_worse(f"wkv6 ew N={N} {name}", a, e, g)
    gu_ref = ref[5]
    e = err_ratio(gu_ref.sum(0).reshape(-1), gu.double().cpu().sum(0).reshape(-1))
    print(f"  gu (summed over the batch): {e:.3e}", flush=True)
    assert e < 6e-3


@pytest.mark.parametrize("N", [2, 4, 17, 48, 128])
def test_wkv5_fp32_any_head_size(lib, N):
    B, T, H = 2, 53, 2
    C = H * N
    g = torch.Generator().manual_seed(500 + N)
    rnd = lambda *s: torch.rand(*s, generator=g) * 2 - 1
    r, k, v, w, u, gy = rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(C), rnd(C), rnd(B, T, C)
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
    for name, a, got in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, [y, gr, gk, gv, gw, gu]):
        e = err_ratio(a, got.double().cpu().reshape(a.shape))
        print(f"  wkv5 fp32 N={N} {name}: {e:.3e}", flush=True)
        assert e <= 1e-5, (name, e)


@pytest.mark.parametrize("N", [1, 4, 17, 48, 128])
def test_wkv5a_any_head_size(lib, N):
    """wkv5a/run.py:38-72 lists head sizes 4, 17, 64 and 128 for its jobs."""
    B, T, H = 2, 45, 2
    C = H * N
    g = torch.Generator().manual_seed(600 + N)
    rnd = lambda *s, lo=-1.0, hi=1.0: torch.rand(*s, generator=g) * (hi - lo) + lo
    r, k, v, gy = rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(B, T, C)
    w1, u1, w2, u2 = rnd(H, N, lo=-8.0), rnd(H, N), rnd(H, N, lo=-8.0), rnd(H, N)
    ref = A5.grads(B, T, C, H, r, k, v, w1, u1, w2, u2, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w1, u1, w2, u2)]
    y = wkv5a.CUDA_1(*t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, got in zip(["y", "gr", "gk", "gv", "gw1", "gu1", "gw2", "gu2"], ref, [y] + [x.grad for x in t]):
        e = err_ratio(a, got.detach().double().cpu().reshape(a.shape))
        print(f"  wkv5a N={N} {name}: {e:.3e}", flush=True)
        assert e <= 1e-5, (name, e)


def test_wkv5_bf16_reference_default_shape_sampled_heads(lib):
    """wkv5_bf16/run.py:17-22 as shipped: B8 T4096 C4096, head size 128.  Two heads against the fp64 oracle."""
    B, T, N = 8, 4096, 128
    C, H = 4096, 32
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=44)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    print("\nwkv5 bf16 head size 128, full size launch", flush=True)
    y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    got_all = [y.detach()] + [x.grad for x in t]
    # one head as a small problem: the fp64 oracle and the emulation of the reference kernel (fp32 math, its rounding
    # points), both by the hand-derived backward
    hs = [29]
    n = N * len(hs)
    ch = torch.cat([torch.arange(h * N, (h + 1) * N) for h in hs])
    rr, kk, vv, gg = (x[:, :, ch].contiguous() for x in (r, k, v, gy))
    uu, wr = u[hs].contiguous(), w[hs].contiguous()
    ref = list(O.wkv_grads_by_hand(B, T, n, len(hs), rr, kk, vv, wr.reshape(1, 1, n).expand(B, T, n), uu, gg, None, torch.float64))[:6]
    ref[4] = ref[4].sum((0, 1)).reshape(len(hs), N)
    ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv5_bf16(B, T, n, len(hs), rr, kk, vv, wr, uu, gg, hand=True)
    chd = ch.to(DEV)
    got = [got_all[0][:, :, chd], got_all[1][:, :, chd], got_all[2][:, :, chd], got_all[3][:, :, chd], got_all[4][hs], got_all[5][hs]]
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, got):
        assert_no_worse("wkv5 N=128 full size " + name, a, e, g)


def _wkv5_c_abi(lib, B, T, C, H, r, k, v, w, u, gy, flags, with_forward_workspace):
    """rwkv_wkv5_forward_ws / rwkv_wkv5_backward_ex: the reference's argument lists (eew, ew in fp32, per-batch gw, gu)."""
    ew = -torch.exp(w.float().reshape(-1))
    d = [x.to(DEV) for x in (r, k, v, torch.exp(ew), ew, u, gy)]
    y, gr, gk, gv = (garbage((B, T, C), BF) for _ in range(4))
    gw, gu = garbage((B, C), BF), garbage((B, C), BF)
    if with_forward_workspace:
        n = lib.rwkv_wkv5_forward_workspace_bytes(B, T, C, H)
        ws = torch.empty(max(n, 16), device=DEV, dtype=torch.uint8)
        call("rwkv_wkv5_forward_ws", DEV, B, T, C, H, d[0], d[1], d[2], d[3], d[5], y, ws, n, flags)
    else:
        call("rwkv_wkv5_forward_ex", DEV, B, T, C, H, d[0], d[1], d[2], d[3], d[5], y, flags)
    n = lib.rwkv_wkv5_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv5_backward_ex", DEV, B, T, C, H, *d, gr, gk, gv, gw, gu, ws, n, flags)
    torch.cuda.synchronize()
    return [y, gr, gk, gv, gw, gu]


@pytest.mark.parametrize("B,T,H", [(2, 37, 3), (1, 1, 1), (3, 160, 2), (1, 515, 1)])
def test_wkv5_bf16_head_size_128_both_kernel_families(lib, B, T, H):
    """Heads of 128 as four heads of 64 on the matrix cores (forward with its workspace), and on the row kernels (the
    forward without a workspace; RWKV_FLAG_SWEEPS for the backward): each against the oracle, per-batch gw and gu."""
    N = 128
    C = H * N
    assert lib.rwkv_wkv5_forward_workspace_bytes(B, T, C, H) == B * T * C * 4
    assert lib.rwkv_wkv5_forward_workspace_bytes(B, T, H * 64, H) == 0
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=500 + T)
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy)
    for flags, fws, what in ((0, True, "four heads of 64"), (SWEEPS, False, "row kernels")):
        print(f"\nwkv5 bf16 N=128 B={B} T={T} H={H}: {what}", flush=True)
        got = _wkv5_c_abi(lib, B, T, C, H, r, k, v, w, u, gy, flags, fws)
        got[4], got[5] = torch.sum(got[4], 0), torch.sum(got[5], 0)       # as the wrapper does (wkv5_bf16/run.py:86-87)
        names = ["y", "gr", "gk", "gv", "gw", "gu"]
        if T == 1:                                                        # one step: the decay feeds nothing
            assert float(got[4].float().abs().max()) == 0.0
        for name, a, e, g in zip(names, ref, emu, got):
            assert_no_worse(f"wkv5 N=128 {what} {name}", a, e.reshape(a.shape), g.reshape(a.shape))


def test_wkv5_bf16_head_size_128_fast_decay_takes_the_step_by_step_path(lib):
    """A channel that decays by e^-20 per step sends the blocks holding it down the kernels' exact path; the other blocks of
    the same head stay on the matrix cores."""
    B, T, H, N = 2, 100, 2, 128
    C = H * N
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=77)
    w = w.clone()
    w[0, 70] = 3.0                                     # second key block of head 0
    w[1, 3] = 2.5                                      # first key block of head 1
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy)
    got = _wkv5_c_abi(lib, B, T, C, H, r, k, v, w, u, gy, 0, True)
    got[4], got[5] = torch.sum(got[4], 0), torch.sum(got[5], 0)
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, got):
        assert_no_worse(f"wkv5 N=128 fast decay {name}", a, e.reshape(a.shape), g.reshape(a.shape))


def test_wkv5_bf16_head_size_128_workspace_is_checked(lib):
    B, T, H, C = 1, 40, 1, 128
    x = torch.zeros(B * T * C, device=DEV, dtype=BF)
    f = torch.zeros(C, device=DEV)
    small = torch.empty(64, device=DEV, dtype=torch.uint8)
    p = x.data_ptr()
    assert lib.rwkv_wkv5_forward_ws(None, B, T, C, H, p, p, p, f.data_ptr(), p, p, small.data_ptr(), 64, 0) == -4
    assert lib.rwkv_wkv5_forward_ws(None, B, T, C, H, p, p, p, f.data_ptr(), p, p, None, 0, 0) == -4
    # the row kernels need none
    assert lib.rwkv_wkv5_forward_ws(None, B, T, C, H, p, p, p, f.data_ptr(), p, p, None, 0, SWEEPS) == 0
    torch.cuda.synchronize()


def test_head_size_limits(lib):
    x = torch.zeros(2 * 8 * 258, device=DEV, dtype=BF)
    f = torch.zeros(2 * 258, device=DEV)
    # 129 > 128, and C not a multiple of H
    assert lib.rwkv_wkv6raw_forward(None, 2, 8, 129, 1, *(x.data_ptr(),) * 6) == -1
    assert lib.rwkv_wkv6raw_forward(None, 2, 8, 130, 4, *(x.data_ptr(),) * 6) == -1
    assert lib.rwkv_wkv5f32_forward(None, 2, 8, 129, 1, *(f.data_ptr(),) * 6) == -1
    assert lib.rwkv_wkv5a_forward(None, 2, 8, 129, 1, f.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(),
                                  f.data_ptr(), f.data_ptr(), f.data_ptr()) == -1
