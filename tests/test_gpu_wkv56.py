"""GPU parity: wkv5 / wkv6 / wkv6_state through the C ABI against the CPU oracle."""
import pytest
import torch

from oracle import wkv56 as O
from oracle import err_ratio
from rwkv_cuda_amd import _lib, options, synth, wkv5_bf16, wkv6, wkv6_state
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, assert_no_worse, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16

# (B, T, H): T below one staging chunk, not a multiple of it, a multiple, and T = 1
ALGOS = ["chunked", "sweeps"]
SHAPES = [(2, 50, 2), (1, 97, 3), (2, 64, 1), (3, 1, 1), (1, 7, 2)]


@pytest.mark.parametrize("B,T,H", SHAPES)
def test_wkv6_state_c_abi_write_coverage(lib, B, T, H):
    print(f"\nwkv6_state C-ABI B={B} T={T} H={H}", flush=True)
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=11, state=True)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    d = [x.to(DEV) for x in (r, k, v, w, u, s0, gy)]
    y = garbage((B, T, C), BF)
    call("rwkv_wkv6state_forward", d[0].device, B, T, C, H, *d[:6], y)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu = garbage((B, C), BF)
    gs = garbage((B, H, 64, 64), BF)
    n = lib.rwkv_wkv6state_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv6state_backward", d[0].device, B, T, C, H, *d[:6], d[6], gr, gk, gv, gw, gu, gs, ws, n)
    torch.cuda.synchronize()
    got = [y, gr, gk, gv, gw, gu.sum(0).view(H, 64), gs]
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, got):
        assert_no_worse(name, a, e, g)
    assert float(gw[:, T - 1].float().abs().max()) == 0.0          # w_{T-1} feeds nothing


@pytest.mark.parametrize("B,T,H", SHAPES[:3])
def test_wkv6_autograd(lib, B, T, H):
    print(f"\nwkv6 autograd B={B} T={T} H={H}", flush=True)
    C = H * 64
    r, k, v, w, u, gy, _ = synth.wkv6_inputs(B, T, C, H, seed=12)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    y = wkv6.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse(name, a, e, g)
    gw = t[3].grad.float()
    assert float(gw[:, 0].abs().max()) == 0.0 and float(gw[:, T - 1].abs().max()) == 0.0


@pytest.mark.parametrize("B,T,H", SHAPES[:3])
def test_wkv5_autograd(lib, B, T, H):
    print(f"\nwkv5 autograd B={B} T={T} H={H}", flush=True)
    C = H * 64
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=13)
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse(name, a, e, g)


def test_wkv6_equals_wkv5_when_decay_is_time_constant(lib):
    B, T, H = 2, 40, 2
    C = H * 64
    r, k, v, w5, u, gy = synth.wkv5_inputs(B, T, C, H, seed=14)
    w6 = w5.reshape(1, 1, C).expand(B, T, C).contiguous()
    d = lambda x: x.to(DEV)
    y5 = wkv5_bf16.RUN_CUDA(B, T, C, H, d(r), d(k), d(v), d(w5), d(u))
    y6 = wkv6.RUN_CUDA(B, T, C, H, d(r), d(k), d(v), d(w6), d(u))
    ys = wkv6_state.RUN_CUDA(B, T, C, H, d(r), d(k), d(v), d(w6), d(u), torch.zeros(B, H, 64, 64, device=DEV, dtype=BF))
    torch.cuda.synchronize()
    assert err_ratio(y5.float().cpu(), y6.float().cpu()) < 2e-3
    assert err_ratio(y6.float().cpu(), ys.float().cpu()) < 2e-3


def test_wkv6_full_size_sampled_heads(lib):
    """The headline shape B8 T4096 C2048: heads are independent, so the fp64 oracle on a few heads
    (all batches, full T) is an exact check of those heads, including gu and gs."""
    B, T, H = 8, 4096, 32
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=42, state=True)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u, s0)]
    print("\nwkv6_state full size launch", flush=True)
    y = wkv6_state.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    got_all = [y.detach()] + [x.grad for x in t]
    # the sampled heads as one small problem of two heads: the fp64 oracle and the emulation of the reference kernel
    # (fp32 math, its rounding points), both by the hand-derived backward, which costs a third of autograd at this length
    hs = [0, 31]
    ch = torch.cat([torch.arange(h * 64, (h + 1) * 64) for h in hs])
    rr, kk, vv, ww, gg = (x[:, :, ch].contiguous() for x in (r, k, v, w, gy))
    uu, ss = u[hs].contiguous(), s0[:, hs].contiguous()
    ref = list(O.wkv_grads_by_hand(B, T, 64 * len(hs), len(hs), rr, kk, vv, ww, uu, gg, ss, torch.float64))
    ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv6_bf16(B, T, 64 * len(hs), len(hs), rr, kk, vv, ww, uu, gg, s0=ss, hand=True)
    chd = ch.to(DEV)
    got = [got_all[0][:, :, chd], got_all[1][:, :, chd], got_all[2][:, :, chd], got_all[3][:, :, chd],
           got_all[4][:, :, chd], got_all[5][hs], got_all[6][:, hs]]
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, got):
        assert_no_worse("wkv6_state full size " + name, a, e, g)


@pytest.mark.parametrize("entry", ["raw", "ew"])
def test_wkv6_stateless_full_size_sampled_heads(lib, entry):
    """The stateless ops at the headline shape B8 T4096 C2048, through the C ABI: rwkv_wkv6raw_* (raw bf16 decay, what
    WKV_6 and the benchmark call) and rwkv_wkv6_* (fp32 ew = -exp(w), the boundary of wkv6/cuda/wkv6_op.cpp:5-6).
    Two heads, all batches, full T, against the fp64 oracle; without a state the decay of token 0 feeds nothing."""
    B, T, H = 8, 4096, 32
    C = H * 64
    r, k, v, w, u, gy, _ = synth.wkv6_inputs(B, T, C, H, seed=44)
    d = [x.to(DEV) for x in (r, k, v, w, u, gy)]
    wd = d[3] if entry == "raw" else (-torch.exp(d[3].float())).contiguous()
    name_f, name_b = ("rwkv_wkv6raw_forward", "rwkv_wkv6raw_backward") if entry == "raw" else ("rwkv_wkv6_forward", "rwkv_wkv6_backward")
    print(f"\nwkv6 stateless full size, entry {entry}", flush=True)
    y = garbage((B, T, C), BF)
    call(name_f, d[0].device, B, T, C, H, d[0], d[1], d[2], wd, d[4], y)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu = garbage((B, C), BF)
    n = lib.rwkv_wkv6_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call(name_b, d[0].device, B, T, C, H, d[0], d[1], d[2], wd, d[4], d[5], gr, gk, gv, gw, gu, ws, n)
    torch.cuda.synchronize()
    assert float(gw[:, 0].float().abs().max()) == 0.0 and float(gw[:, T - 1].float().abs().max()) == 0.0
    gu_sum = gu.sum(0).view(H, 64)                              # what the wrapper does: a bf16 sum of the per-batch rows
    hs = [3, 28]
    ch = torch.cat([torch.arange(h * 64, (h + 1) * 64) for h in hs])
    rr, kk, vv, ww, gg = (x[:, :, ch].contiguous() for x in (r, k, v, w, gy))
    uu = u[hs].contiguous()
    ref = list(O.wkv_grads_by_hand(B, T, 64 * len(hs), len(hs), rr, kk, vv, ww, uu, gg, None, torch.float64))[:6]
    ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv6_bf16(B, T, 64 * len(hs), len(hs), rr, kk, vv, ww, uu, gg, hand=True)
    chd = ch.to(DEV)
    got = [y[:, :, chd], gr[:, :, chd], gk[:, :, chd], gv[:, :, chd], gw[:, :, chd], gu_sum[hs]]
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, got):
        assert_no_worse(f"wkv6 {entry} full size " + name, a, e, g)


def test_wkv5_full_size_sampled_heads(lib):
    """wkv5 at B8 T4096 C2048 (per-head constant decay, 128 chunks per sequence): two heads against the fp64 oracle."""
    B, T, H = 8, 4096, 32
    C = H * 64
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=43)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
    print("\nwkv5 full size launch", flush=True)
    y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    got_all = [y.detach()] + [x.grad for x in t]
    hs = [5, 30]
    ch = torch.cat([torch.arange(h * 64, (h + 1) * 64) for h in hs])
    rr, kk, vv, gg = (x[:, :, ch].contiguous() for x in (r, k, v, gy))
    uu, wr = u[hs].contiguous(), w[hs].contiguous()
    n = 64 * len(hs)
    ref = list(O.wkv_grads_by_hand(B, T, n, len(hs), rr, kk, vv, wr.reshape(1, 1, n).expand(B, T, n), uu, gg, None, torch.float64))[:6]
    ref[4] = ref[4].sum((0, 1)).reshape(len(hs), 64)
    ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv5_bf16(B, T, n, len(hs), rr, kk, vv, wr, uu, gg, hand=True)
    chd = ch.to(DEV)
    got = [got_all[0][:, :, chd], got_all[1][:, :, chd], got_all[2][:, :, chd], got_all[3][:, :, chd], got_all[4][hs], got_all[5][hs]]
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, got):
        assert_no_worse("wkv5 full size " + name, a, e, g)


def test_long_sequence_is_no_worse_than_the_reference_kernel(lib):
    """T = 4096 on one head: errors that grow with the sequence length (the running P of the decay gradient did, until
    it was re-derived from the states every few chunks) are invisible at the small shapes above."""
    B, T, H = 1, 4096, 1
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=46, state=True)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u, s0)]
    y = wkv6_state.RUN_CUDA(B, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse("wkv6_state T4096 " + name, a, e, g)

    r, k, v, w5, u, gy = synth.wkv5_inputs(2, T, C, H, seed=47)
    ref = O.wkv5_grads(2, T, C, H, r, k, v, w5, u, gy)
    emu = O.emulate_wkv5_bf16(2, T, C, H, r, k, v, w5, u, gy)
    t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w5, u)]
    y = wkv5_bf16.RUN_CUDA(2, T, C, H, *t)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
        assert_no_worse("wkv5 T4096 " + name, a, e, g)


def test_wkv6_fp32_ew_c_abi(lib):
    """The reference's own wkv6 boundary: the decay arrives as fp32 ew = -exp(w) (wkv6/run.py:147)."""
    B, T, H = 2, 70, 2
    C = H * 64
    r, k, v, w, u, gy, _ = synth.wkv6_inputs(B, T, C, H, seed=15)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy)
    d = [x.to(DEV) for x in (r, k, v, w, u, gy)]
    ew = (-torch.exp(d[3].float())).contiguous()
    for algo in (0, 1):
        print(f"\nwkv6 fp32-ew C-ABI algo={algo}", flush=True)
        flags = options.FLAG_SWEEPS if algo else 0
        y = garbage((B, T, C), BF)
        call("rwkv_wkv6_forward_ex", d[0].device, B, T, C, H, d[0], d[1], d[2], ew, d[4], y, flags)
        gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
        gu = garbage((B, C), BF)
        n = lib.rwkv_wkv6_backward_workspace_bytes(B, T, C, H)
        ws = torch.empty(n, device=DEV, dtype=torch.uint8)
        call("rwkv_wkv6_backward_ex", d[0].device, B, T, C, H, d[0], d[1], d[2], ew, d[4], d[5], gr, gk, gv, gw, gu, ws, n, flags)
        torch.cuda.synchronize()
        for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y, gr, gk, gv, gw, gu.sum(0).view(H, 64)]):
            assert_no_worse(name, a, e, g)


@pytest.mark.parametrize("algo", [0, 1])
def test_wkv6_state_both_algorithms_and_extreme_decays(lib, algo):
    """Chunked (matrix-core) and sequential kernels against the oracle, on ordinary inputs and on decays so strong
    (w_raw up to 3: one step multiplies the state by e^-20) that the chunked kernels must take their exact path."""
    B, T, H = 2, 100, 2
    C = H * 64
    for extreme in (False, True):
        r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=16, state=True)
        if extreme:
            w = w.float()
            w[:, 40:60, :64] = 2.5
            w[1, 70:, 100] = 3.0
            w[0, 5:9, 70:90] = 2.0
            w = w.to(BF)
        ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
        emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
        print(f"\nwkv6_state algo={algo} extreme={extreme}", flush=True)
        t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u, s0)]
        with options.algorithm(ALGOS[algo]):
            y = wkv6_state.RUN_CUDA(B, T, C, H, *t)
        y.backward(gy.to(DEV))               # outside the block: the backward follows the forward's choice
        torch.cuda.synchronize()
        for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, [y] + [x.grad for x in t]):
            assert torch.isfinite(g).all(), name
            assert_no_worse(name, a, e, g)


@pytest.mark.parametrize("algo", [0, 1])
def test_wkv5_both_algorithms_and_strong_decays(lib, algo):
    """wkv5 (one decay per head channel) on the chunked and on the sequential kernels; with w_raw up to 2.5 some
    channels lose e^-12 per step, which sends every chunk of that head down the chunked kernels' exact path."""
    B, T, H = 2, 83, 2
    C = H * 64
    for strong in (False, True):
        r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=21)
        if strong:
            w = w.float()
            w[1, 10:20] = 2.5
            w[1, 40] = 1.5
            w = w.to(BF)
        ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy)
        emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy)
        print(f"\nwkv5 algo={algo} strong={strong}", flush=True)
        t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
        with options.algorithm(ALGOS[algo]):
            y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
            y.backward(gy.to(DEV))
        torch.cuda.synchronize()
        for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
            assert torch.isfinite(g).all(), name
            assert_no_worse(name, a, e, g)


def _low_rank_decay(B, T, C, seed):
    """w = w0 + (x @ ww1) @ ww2 as the reference's wkv6 checks build it (wkv6_state/run.py:183-186,214): at C = 128
    it spans about -18 .. +15, so a seventh of the decays exp(-exp(w)) are exactly zero in fp32 and others are 1."""
    g = torch.Generator().manual_seed(seed)
    U = lambda lo, hi, *s: (torch.rand(*s, generator=g) * (hi - lo) + lo).to(BF).float()
    return (U(-3, 1, 1, 1, C) + (U(-1, 1, B, T, C) @ U(-1, 1, C, 3)) @ U(-1, 1, 3, C)).to(BF)


@pytest.mark.parametrize("algo", [0, 1])
def test_decay_gradient_where_the_decay_has_vanished(lib, algo):
    """gw = -exp(w_raw) G, and G comes from a recurrence whose rounding noise does not shrink with the decay: at
    w_raw = 15 the factor is 3e6 and would turn 1e-6 of noise into O(1) gradients where the true value (and the
    reference kernel's) is an exact zero."""
    B, T, H = 2, 64, 2
    C = H * 64
    r, k, v, _, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=51, state=True)
    w = _low_rank_decay(B, T, C, seed=52)
    assert float(w.max()) > 8 and float(w.min()) < -8
    gone = w.float() > 4.5                                   # exp(-exp(4.5)) < 1e-39
    with options.algorithm(ALGOS[algo]):
        for state in (None, s0):
            print(f"\nlow-rank decays algo={algo} state={state is not None}", flush=True)
            ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=state)
            emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=state)
            t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w, u)]
            if state is None:
                y = wkv6.RUN_CUDA(B, T, C, H, *t)
            else:
                t.append(state.to(DEV).requires_grad_(True))
                y = wkv6_state.RUN_CUDA(B, T, C, H, *t)
            y.backward(gy.to(DEV))
            torch.cuda.synchronize()
            for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, [y] + [x.grad for x in t]):
                assert_no_worse(name, a, e, g)
            assert float(t[3].grad.float().cpu()[gone].abs().max()) == 0.0
        # wkv5: per-channel decays up to w_raw = 6 (the state of those channels is wiped every step)
        r, k, v, w5, u, gy = synth.wkv5_inputs(B, T, C, H, seed=53)
        w5 = w5.float()
        w5[0, 5:12] = 6.0
        w5[1, 30] = 4.0
        w5 = w5.to(BF)
        ref = O.wkv5_grads(B, T, C, H, r, k, v, w5, u, gy)
        emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w5, u, gy)
        t = [x.to(DEV).requires_grad_(True) for x in (r, k, v, w5, u)]
        y = wkv5_bf16.RUN_CUDA(B, T, C, H, *t)
        y.backward(gy.to(DEV))
        torch.cuda.synchronize()
        for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y] + [x.grad for x in t]):
            assert_no_worse("wkv5 " + name, a, e, g)
        assert float(t[3].grad.float().cpu()[0, 5:12].abs().max()) == 0.0


def test_two_threads_run_different_algorithms_concurrently(lib):
    """The kernel choice is a per-call argument: one thread runs the chunked kernels and another the sequential sweeps
    at the same time, on two streams, and each gets exactly what it gets when it runs alone."""
    import threading
    B, T, H = 2, 200, 2
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=71, state=True)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    d = [x.to(DEV) for x in (r, k, v, w, u, s0, gy)]
    n = lib.rwkv_wkv6state_backward_workspace_bytes(B, T, C, H)

    def run(flags, stream, reps, out):
        with torch.cuda.stream(stream):
            for _ in range(reps):
                ws = torch.empty(n, device=DEV, dtype=torch.uint8)
                y, gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(5))
                gu, gs = garbage((B, C), BF), garbage((B, H, 64, 64), BF)
                call("rwkv_wkv6state_forward_ex", d[0].device, B, T, C, H, *d[:6], y, flags)
                call("rwkv_wkv6state_backward_ex", d[0].device, B, T, C, H, *d[:6], d[6], gr, gk, gv, gw, gu, gs, ws, n, flags)
                out.append([y, gr, gk, gv, gw, gu, gs])
            stream.synchronize()

    torch.cuda.synchronize()
    alone = {}
    for flags in (0, options.FLAG_SWEEPS):
        res = []
        run(flags, torch.cuda.Stream(), 1, res)
        alone[flags] = res[0]
    results = {0: [], options.FLAG_SWEEPS: []}
    threads = [threading.Thread(target=run, args=(f, torch.cuda.Stream(), 6, results[f])) for f in results]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for flags, runs in results.items():
        assert len(runs) == 6
        for got in runs:
            for name, a, b in zip(("y", "gr", "gk", "gv", "gw", "gu", "gs"), alone[flags], got):
                assert torch.equal(a, b), (flags, name)
        got = runs[-1]
        got[5] = got[5].sum(0).view(H, 64)
        for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu", "gs"], ref, emu, got):
            assert_no_worse(f"flags {flags:#x} {name}", a, e, g)
