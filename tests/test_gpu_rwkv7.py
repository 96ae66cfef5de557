"""GPU parity: rwkv7 clamp-w with state passing through the C ABI against the CPU oracle."""
import pytest
import torch

from oracle import rwkv7 as O
from oracle import err_ratio
from rwkv_cuda_amd import options, synth, rwkv7_fast_fused as R
from _gpu_util import DEV, assert_no_worse

pytestmark = pytest.mark.gpu
NAMES = ["y", "sT", "ds0", "dr", "dw", "dk", "dv", "da", "db"]


def _run(args, splits=1):
    s0, r, w, k, v, a, b, dy, dsT = args
    B, T, H, N = r.shape
    t = [x.to(DEV).requires_grad_(True) for x in (s0, r, w, k, v, a, b)]
    S = t[0]
    ys = []
    step = T // splits
    for c in range(splits):
        sl = slice(c * step, (c + 1) * step)
        y, S = R.RWKV7_STATE_PASSING_CLAMPW_CUDA(S, *(x[:, sl].contiguous().view(B, step, H * N) for x in t[1:]))
        ys.append(y)
    y = torch.cat(ys, 1)
    torch.autograd.backward([y, S], [dy.to(DEV).view(B, T, H * N), dsT.to(DEV)])
    torch.cuda.synchronize()
    return [y.detach().view(B, T, H, N), S.detach()] + [x.grad for x in t]


@pytest.mark.parametrize("algo", ["chunked", "sweeps"])
@pytest.mark.parametrize("B,T,H", [(2, 32, 2), (1, 64, 3), (3, 16, 1)])
def test_rwkv7_small(lib, B, T, H, algo):
    """Both kernel families: the chunked matrix-core kernels (default) and the step-by-step recurrence."""
    print(f"\nrwkv7 B={B} T={T} H={H} {algo}", flush=True)
    args = synth.rwkv7_inputs(B, T, H, 64, seed=31)
    ref = O.grads(*args)
    emu = O.emulate_bf16(*args)
    with options.algorithm(algo):
        got = _run(args)
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse(name, a, e, g)


def test_rwkv7_chained_calls_small(lib):
    """Four chained T/4 calls (state handed over) against the fp64 oracle of one T call."""
    B, T, H = 2, 128, 2
    args = synth.rwkv7_inputs(B, T, H, 64, seed=32)
    ref = O.grads(*args)
    emu = O.emulate_bf16(*args)
    got = _run(args, splits=4)
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse(name, a, e, g)


def test_rwkv7_full_size_chain_equals_one_call(lib):
    """B8 T4096 C4096 (H64): 4 x T1024 chained must reproduce one T4096 call.  Forward values are
    bit-identical (same arithmetic, states handed over in fp32); gradients agree to rounding."""
    B, T, H = 8, 4096, 64
    args = synth.rwkv7_inputs(B, T, H, 64, seed=42)
    print("\nrwkv7 full size: one call", flush=True)
    one = _run(args)
    print("rwkv7 full size: four chained calls", flush=True)
    four = _run(args, splits=4)
    assert torch.equal(one[0], four[0]) and torch.equal(one[1], four[1])
    for name, x, y in zip(NAMES[2:], one[2:], four[2:]):
        e = err_ratio(x.float().cpu(), y.float().cpu())
        print(f"  {name}: {e:.3e}", flush=True)
        assert e < 1e-3, (name, e)
    # one head against the fp64 oracle (all batches, full T)
    h = 5
    sub = [args[0][:, h:h + 1]] + [x[:, :, h:h + 1] for x in args[1:8]] + [args[8][:, h:h + 1]]
    ref = O.backward_hand(*sub)
    emu = O.emulate_bf16(*sub)
    got = [one[0][:, :, h:h + 1], one[1][:, h:h + 1], one[2][:, h:h + 1]] + [x[:, :, h:h + 1] for x in one[3:]]
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse(f"rwkv7 full size head {h} " + name, a, e, g)


@pytest.mark.parametrize("B,T,H", [(2, 32, 2), (1, 48, 1)])
def test_rwkv7_state_only_and_stateless_ops(lib, B, T, H):
    """The siblings of the state-passing op (rwkv7_state_clampw: s0 and ds0, no final state; rwkv7_clampw: no state
    at all) are the state-passing formula with dsT = 0, respectively s0 = 0 and dsT = 0."""
    print(f"\nrwkv7 siblings B={B} T={T} H={H}", flush=True)
    s0, r, w, k, v, a, b, dy, dsT = synth.rwkv7_inputs(B, T, H, 64, seed=33)
    N = 64
    flat = lambda x: x.contiguous().view(B, T, H * N)

    # initial state only
    args = (s0, r, w, k, v, a, b, dy, torch.zeros_like(dsT))
    ref, emu = O.grads(*args), O.emulate_bf16(*args)
    t = [x.to(DEV).requires_grad_(True) for x in (s0, r, w, k, v, a, b)]
    y = R.RWKV7_STATE_CLAMPW_CUDA(t[0], *(flat(x) for x in t[1:]))
    y.backward(flat(dy.to(DEV)))
    torch.cuda.synchronize()
    got = [y.detach().view(B, T, H, N), None] + [x.grad for x in t]
    for name, a_, e, g in zip(NAMES, ref, emu, got):
        if g is not None:
            assert_no_worse("state op " + name, a_, e, g)

    # no state
    args = (torch.zeros_like(s0), r, w, k, v, a, b, dy, torch.zeros_like(dsT))
    ref, emu = O.grads(*args), O.emulate_bf16(*args)
    t = [x.to(DEV).requires_grad_(True) for x in (r, w, k, v, a, b)]
    y = R.RWKV7_CLAMPW_CUDA(*(flat(x) for x in t))
    y.backward(flat(dy.to(DEV)))
    torch.cuda.synchronize()
    got = [y.detach().view(B, T, H, N), None, None] + [x.grad for x in t]
    for name, a_, e, g in zip(NAMES, ref, emu, got):
        if g is not None:
            assert_no_worse("stateless op " + name, a_, e, g)


def test_rwkv7_long_sequence_is_no_worse_than_the_reference_kernel(lib):
    """T = 4096 on one head (the length of one call at the benchmark shape): the in-chunk inversion of the backward and the
    fp32 state must not lose accuracy with length."""
    B, T, H = 1, 4096, 1
    args = synth.rwkv7_inputs(B, T, H, 64, seed=34)
    ref = O.grads(*args)
    emu = O.emulate_bf16(*args)
    got = _run(args)
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse("rwkv7 T4096 " + name, a, e, g)


def _fp32_inputs(B, T, H, seed):
    """The bf16 test inputs plus an fp32 perturbation below bf16 resolution, so that the fp32 mode is
    seen to read all 32 bits of every element."""
    g = torch.Generator().manual_seed(seed + 1000)
    args = synth.rwkv7_inputs(B, T, H, 64, seed=seed)
    jig = lambda x: x.float() * (1 + 1e-3 * torch.rand(x.shape, generator=g))
    s0, r, w, k, v, a, b, dy, dsT = args
    return (s0, jig(r), jig(w), jig(k), jig(v), jig(a), jig(b), jig(dy), dsT)


def assert_fp32_mode(name, ref64, emu, got):
    """fp32 mode: the error against fp64 may not exceed twice that of the reference kernel's arithmetic
    (fp32, in-chunk inversion, checkpoints every 16 steps) emulated on the CPU.  The two differ only
    in summation order, so their errors are independent samples of the same size; 2x covers that."""
    e_hip = err_ratio(ref64, got.detach().double().cpu())
    e_emu = err_ratio(ref64, emu.double())
    print(f"  {name}: hip {e_hip:.3e}  reference-kernel arithmetic {e_emu:.3e}", flush=True)
    assert e_hip <= 2.0 * e_emu + 1e-6, f"{name}: {e_hip:.3e} vs {e_emu:.3e}"
    assert e_hip < 1e-3, name                       # and far below what a bf16 rounding anywhere would leave


@pytest.mark.parametrize("B,T,H", [(2, 32, 2), (1, 256, 1)])
def test_rwkv7_fp32_mode(lib, B, T, H):
    """The reference's -D_FP32_ build (rwkv7_cuda_benchmark_state_passing.py:105-131): every tensor fp32."""
    print(f"\nrwkv7 fp32 mode B={B} T={T} H={H}", flush=True)
    args = _fp32_inputs(B, T, H, seed=35)
    ref = O.grads(*args)
    emu = O.backward_hand(*args, dtype=torch.float32, invert=True)
    got = _run(args)
    assert got[0].dtype == torch.float32 and got[3].dtype == torch.float32
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_fp32_mode(name, a, e, g)


def test_rwkv7_fp32_mode_siblings(lib):
    B, T, H, N = 2, 32, 2, 64
    s0, r, w, k, v, a, b, dy, dsT = _fp32_inputs(B, T, H, seed=36)
    flat = lambda x: x.contiguous().view(B, T, H * N)
    args = (s0, r, w, k, v, a, b, dy, torch.zeros_like(dsT))
    ref, emu = O.grads(*args), O.backward_hand(*args, dtype=torch.float32, invert=True)
    t = [x.to(DEV).requires_grad_(True) for x in (s0, r, w, k, v, a, b)]
    y = R.RWKV7_STATE_CLAMPW_CUDA(t[0], *(flat(x) for x in t[1:]))
    y.backward(flat(dy.to(DEV)))
    torch.cuda.synchronize()
    got = [y.detach().view(B, T, H, N), None] + [x.grad for x in t]
    for name, a_, e, g in zip(NAMES, ref, emu, got):
        if g is not None:
            assert_fp32_mode("fp32 state op " + name, a_, e, g)
    args = (torch.zeros_like(s0), r, w, k, v, a, b, dy, torch.zeros_like(dsT))
    ref, emu = O.grads(*args), O.backward_hand(*args, dtype=torch.float32, invert=True)
    t = [x.to(DEV).requires_grad_(True) for x in (r, w, k, v, a, b)]
    y = R.RWKV7_CLAMPW_CUDA(*(flat(x) for x in t))
    y.backward(flat(dy.to(DEV)))
    torch.cuda.synchronize()
    got = [y.detach().view(B, T, H, N), None, None] + [x.grad for x in t]
    for name, a_, e, g in zip(NAMES, ref, emu, got):
        if g is not None:
            assert_fp32_mode("fp32 stateless op " + name, a_, e, g)


def test_rwkv7_backward_uses_the_kernel_family_of_its_forward(lib):
    """The two kernel families lay the checkpoint tensor `s` out differently and nothing in it says which one wrote it: a
    backward must run with the flags of its forward.  The wrapper keeps them on the autograd context, so a forward issued
    inside `algorithm("sweeps")` gets the step kernels' backward even when autograd runs it after the block has ended."""
    B, T, H = 2, 48, 2
    args = synth.rwkv7_inputs(B, T, H, 64, seed=35)
    ref, emu = O.grads(*args), O.emulate_bf16(*args)
    s0, r, w, k, v, a, b, dy, dsT = args
    t = [x.to(DEV).requires_grad_(True) for x in (s0, r, w, k, v, a, b)]
    with options.algorithm("sweeps"):
        y, S = R.RWKV7_STATE_PASSING_CLAMPW_CUDA(t[0], *(x.contiguous().view(B, T, H * 64) for x in t[1:]))
    assert options.current_flags() == 0                            # the block has ended: the default family is current again
    torch.autograd.backward([y, S], [dy.to(DEV).view(B, T, H * 64), dsT.to(DEV)])
    torch.cuda.synchronize()
    got = [y.detach().view(B, T, H, 64), S.detach()] + [x.grad for x in t]
    for name, a_, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse("sweeps forward, backward after the block: " + name, a_, e, g)
