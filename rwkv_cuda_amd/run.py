"""Self-check driver in the style of the reference's run.py scripts:

    python -m rwkv_cuda_amd.run OP [check|benchmark] [--B n --T n --H n]

    OP: wkv  depthwise_conv1d  wkv5  wkv5_bf16  wkv5a  wkv6  wkv6_state  rwkv7  rwkv7_fp32

`check` runs the HIP op forward and backward (through the "strange loss" of the reference's checks,
wkv6_state/run.py:171-172) beside a plain torch formula of the same op evaluated in fp32 on the same
device, and prints one line per tensor, `correct = allclose, err ratio = ...`, as
wkv6_state/run.py:272,287-301 and wkv5/run.py:530-579 do.  For wkv6 and wkv6_state the decay comes from
the caller one step up, the low-rank form w = w0 + (x @ ww1) @ ww2 (wkv6_state/run.py:183-186,214), and
the gradients of x, ww1, ww2 are compared too.  `benchmark` times forward and backward at the
reference's benchmark shape under the torch profiler and prints its table (wkv6_state/run.py:267-281).

The torch formulas below exist for this driver only: no operator of the package calls them, and there
is no fallback from the HIP kernels to them.  A HIP device is required.
"""

import argparse
import sys

import torch
import torch.nn.functional as F

N = 64  # head size of every multi-head op here


def get_err_ratio(x, y):
    """wkv/run.py:26-29."""
    err = (x - y).flatten().square().mean().sqrt().item()
    base = x.flatten().square().mean().sqrt().item()
    return err / base


def LOSS(y):
    """wkv6_state/run.py:171-172."""
    return ((y * y) - torch.tanh(y)).sum()


# ---------------------------------------------------------------------------------------------
# plain torch formulas (fp32, any device); i = value channel, j = key channel, state S[b,h,i,j]
# ---------------------------------------------------------------------------------------------

def formula_wkv4(B, T, C, w, u, k, v):
    """y_t = (sum_{s<t} e^{(t-1-s) w + k_s} v_s + e^{u + k_t} v_t) / (same with v -> 1), w = -exp(w_raw)
    (wkv/run.py:38-62), in the numerically plain form: fine for the small T of a check."""
    w = -torch.exp(w)
    ys = []
    num = torch.zeros(B, C, device=k.device)
    den = torch.zeros(B, C, device=k.device)
    for t in range(T):
        e = torch.exp(u + k[:, t])
        ys.append((num + e * v[:, t]) / (den + e))
        ek = torch.exp(k[:, t])
        num = torch.exp(w) * num + ek * v[:, t]
        den = torch.exp(w) * den + ek
    return torch.stack(ys, 1)


def formula_timex(w, k, B, C, T, eps):
    """Causal depthwise convolution with the tap-reversed kernel (depthwise_conv1d/run.py:58-60)."""
    return F.conv1d(F.pad(k, (T - 1, 0)), w.unsqueeze(1), groups=C) + eps


def formula_wkv(B, T, C, H, r, k, v, decay, u, s0=None, decay2=None, u2=None):
    """wkv5 / wkv6 / wkv6_state / wkv5a in the recurrent form (wkv5/run.py:67-87, wkv6/run.py:207-216,
    wkv5a/run.py:260-289): y_t[i] = sum_j r[j] ((u[j] (+ u2[i])) k[j] v[i] + S[i,j]);
    S <- S * decay[j] (* decay2[i]) + k[j] v[i].  decay is [H,N] or [B,T,H,N]."""
    r, k, v = (x.reshape(B, T, H, N) for x in (r, k, v))
    S = torch.zeros(B, H, N, N, device=r.device) if s0 is None else s0.reshape(B, H, N, N)
    U = u.reshape(H, 1, N) if u2 is None else u.reshape(H, 1, N) + u2.reshape(H, N, 1)
    ys = []
    for t in range(T):
        kv = v[:, t, :, :, None] * k[:, t, :, None, :]
        ys.append(((S + U * kv) * r[:, t, :, None, :]).sum(-1))
        d = decay.reshape(H, 1, N) if decay.dim() == 2 else decay[:, t, :, None, :]
        if decay2 is not None:
            d = d * decay2.reshape(H, N, 1)
        S = S * d + kv
    return torch.stack(ys, 1).reshape(B, T, C)


def formula_rwkv7(s0, r, w, k, v, a, b):
    """rwkv7 clamp-w with state passing (rwkv7_cuda_benchmark_state_passing.py:46-68):
    w = exp(-exp(-softplus(-w_raw) - 0.5)); S <- S diag(w) + (S a) b^T + v k^T; y = S r."""
    B, T, H, _ = r.shape
    w = torch.exp(-torch.exp(-F.softplus(-w) - 0.5))
    S = s0
    ys = []
    for t in range(T):
        sa = torch.einsum('bhij,bhj->bhi', S, a[:, t])
        S = S * w[:, t, :, None, :] + sa[..., None] * b[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :]
        ys.append(torch.einsum('bhij,bhj->bhi', S, r[:, t]))
    return torch.stack(ys, 1), S


# ---------------------------------------------------------------------------------------------
# one case per op: inputs as the reference's checks draw them, the formula, the HIP op
# ---------------------------------------------------------------------------------------------

def _uniform(dev, lo, hi, *shape):
    return torch.empty(*shape, device=dev).uniform_(lo, hi)


def case(op, dev, B, T, H, bench=False):
    """Returns (names, fp32 leaf tensors, formula(leaves) -> outputs, hip(leaves cast to the op's dtype) -> outputs,
    the op's dtype).  Outputs are tuples; every output enters the loss.  With bench=True the wkv6 decays are the
    per-channel uniform(-8, 1) of the reference's speed runs (wkv6_state/run.py:188,284) instead of the low-rank form,
    whose spread grows with C until every decay is 0 or 1."""
    from . import depthwise_conv1d, rwkv7_fast_fused, wkv, wkv5, wkv5_bf16, wkv5a, wkv6, wkv6_state
    C = H * N
    bf = torch.bfloat16
    U = lambda lo, hi, *s: _uniform(dev, lo, hi, *s)
    rb = lambda x: x.to(bf).float()                  # bf16 ops: both sides start from bf16-representable values
    if op == "wkv":                                  # wkv/run.py:129-136
        names, t = ["w", "u", "k", "v"], [U(-1, 1, C), U(-1, 1, C), U(-1, 1, B, T, C), U(-1, 1, B, T, C)]
        return names, t, lambda w, u, k, v: (formula_wkv4(B, T, C, w, u, k, v),), \
            lambda w, u, k, v: (wkv.RUN_CUDA(B, T, C, w, u, k, v),), torch.float32
    if op == "depthwise_conv1d":                     # depthwise_conv1d/run.py:112-118: channels C, length T
        names, t = ["w", "k"], [U(-1, 1, C, T), U(-1, 1, B, C, T)]
        return names, t, lambda w, k: (formula_timex(w, k, B, C, T, 0.1),), \
            lambda w, k: (depthwise_conv1d.RUN_CUDA(w, k, B, C, T, 0.1),), torch.float32
    if op in ("wkv5", "wkv5_bf16"):                  # wkv5/run.py:516-520
        f32 = op == "wkv5"
        q = (lambda x: x) if f32 else rb
        names = ["r", "k", "v", "w", "u"]
        t = [q(U(-1, 1, B, T, C)), q(U(-1, 1, B, T, C)), q(U(-1, 1, B, T, C)), q(U(-1, 1, H, N)), q(U(-1, 1, H, N))]
        mod = wkv5 if f32 else wkv5_bf16
        return names, t, lambda r, k, v, w, u: (formula_wkv(B, T, C, H, r, k, v, torch.exp(-torch.exp(w)), u),), \
            lambda r, k, v, w, u: (mod.RUN_CUDA(B, T, C, H, r, k, v, w, u),), torch.float32 if f32 else bf
    if op == "wkv5a":                                # wkv5a/run.py:389-398
        names = ["r", "k", "v", "w1", "u1", "w2", "u2"]
        t = [U(-1, 1, B, T, C), U(-1, 1, B, T, C), U(-1, 1, B, T, C), U(-8, 1, H, N), U(-1, 1, H, N), U(-8, 1, H, N), U(-1, 1, H, N)]
        dec = lambda w: torch.exp(-torch.exp(w))
        return names, t, lambda r, k, v, w1, u1, w2, u2: (formula_wkv(B, T, C, H, r, k, v, dec(w1), u1, None, dec(w2), u2),), \
            lambda *a: (wkv5a.CUDA_1(*a),), torch.float32
    if op in ("wkv6", "wkv6_state"):                 # wkv6_state/run.py:174-186: low-rank data-dependent decay
        state = op == "wkv6_state"
        names = ["r", "k", "v", "w0", "x", "ww1", "ww2", "u"] + (["s"] if state else [])
        t = [rb(U(-1, 1, B, T, C)), rb(U(-1, 1, B, T, C)), rb(U(-1, 1, B, T, C)), rb(U(-3, 1, 1, 1, C)),
             rb(U(-1, 1, B, T, C)), rb(U(-1, 1, C, 3)), rb(U(-1, 1, 3, C)), rb(U(-1, 1, H, N))]
        if state:
            t.append(rb(U(-1, 1, B, H, N, N)))
        if bench:
            t[3], t[5] = rb(U(-8, 1, 1, 1, C)), torch.zeros(C, 3, device=dev)

        def formula(r, k, v, w0, x, ww1, ww2, u, s=None):
            ww = w0 + (x @ ww1) @ ww2                                          # wkv6_state/run.py:214
            return (formula_wkv(B, T, C, H, r, k, v, torch.exp(-torch.exp(ww.reshape(B, T, H, N))), u, s),)

        def hip(r, k, v, w0, x, ww1, ww2, u, s=None):
            ww = (w0 + (x @ ww1) @ ww2).contiguous()                           # bf16 matmuls, as wkv6_state/run.py:282
            if state:
                return (wkv6_state.RUN_CUDA(B, T, C, H, r, k, v, ww, u, s),)
            return (wkv6.RUN_CUDA(B, T, C, H, r, k, v, ww, u),)
        return names, t, formula, hip, bf
    if op in ("rwkv7", "rwkv7_fp32"):                # rwkv7_cuda_benchmark_state_passing.py:137-147
        f32 = op == "rwkv7_fp32"
        q = (lambda x: x) if f32 else rb
        kk = F.normalize(U(-1, 1, B, T, H, N), dim=-1, p=2.0)
        names = ["s0", "r", "w", "k", "v", "a", "b"]
        t = [U(-1, 1, B, H, N, N) * 0.1, q(U(-1, 1, B, T, H, N)), q(U(-6, 0, B, T, H, N)), q(U(-1, 1, B, T, H, N)),
             q(U(-1, 1, B, T, H, N)), q(-kk), q(kk * U(0, 1, B, T, H, N))]

        def hip(s0, r, w, k, v, a, b):
            flat = lambda x: x.reshape(B, T, C)
            y, sT = rwkv7_fast_fused.RWKV7_STATE_PASSING_CLAMPW_CUDA(s0.float(), *(flat(x) for x in (r, w, k, v, a, b)))
            return y.view(B, T, H, N), sT
        return names, t, formula_rwkv7, hip, torch.float32 if f32 else bf
    raise SystemExit(f"unknown op {op!r}")


OPS = ["wkv", "depthwise_conv1d", "wkv5", "wkv5_bf16", "wkv5a", "wkv6", "wkv6_state", "rwkv7", "rwkv7_fp32"]
# err-ratio bars of `check`: bf16 outputs carry 2^-9 relative rounding; fp32 paths sum in a different order only
BAR = {torch.bfloat16: 2e-2, torch.float32: 2e-4}


def check(op, dev, B, T, H, out=print):
    """Returns the worst err ratio; prints the reference-style lines."""
    torch.manual_seed(42)
    names, leaves, formula, hip, dtype = case(op, dev, B, T, H)
    out(f"{op}: B={B} T={T} C={H * N} HEAD_SIZE={N}   [torch fp32 formula] vs [HIP kernels, {str(dtype).replace('torch.', '')}]")
    ref_in = [x.clone().requires_grad_(True) for x in leaves]
    ys = formula(*ref_in)
    sum(LOSS(y) for y in ys).backward()
    # the HIP side: leaves in the op's dtype (state tensors of rwkv7 stay fp32 inside the wrapper)
    hip_in = [x.clone().to(dtype).requires_grad_(True) for x in leaves]
    ys1 = hip(*hip_in)
    sum(LOSS(y.float()) for y in ys1).backward()
    torch.cuda.synchronize(dev)
    worst = 0.0
    for i, (y, y1) in enumerate(zip(ys, ys1)):
        e = get_err_ratio(y.detach().float(), y1.detach().float().reshape(y.shape))
        worst = max(worst, e)
        out(f"!!! HIP y{i if len(ys) > 1 else ''} correct = {torch.allclose(y.detach().float(), y1.detach().float().reshape(y.shape))}, err ratio = {e}")
    for n, a, b in zip(names, ref_in, hip_in):
        e = get_err_ratio(a.grad.float(), b.grad.float().reshape(a.grad.shape))
        worst = max(worst, e)
        out(f"!!! HIP g_{n} correct = {torch.allclose(a.grad.float(), b.grad.float().reshape(a.grad.shape))}, err ratio = {e}")
    return worst, BAR[dtype]


# the reference's benchmark shapes: (B, T, H)
BENCH_SHAPE = {"wkv": (4, 512, 12), "depthwise_conv1d": (32, 768, 12), "wkv5": (8, 4096, 64), "wkv5_bf16": (8, 4096, 32),
               "wkv5a": (8, 4096, 64), "wkv6": (8, 4096, 32), "wkv6_state": (8, 4096, 32), "rwkv7": (8, 1024, 64),
               "rwkv7_fp32": (8, 1024, 64)}


def benchmark(op, dev, B, T, H, out=print):
    torch.manual_seed(42)
    names, leaves, _, hip, dtype = case(op, dev, B, T, H, bench=True)
    hip_in = [x.clone().to(dtype).requires_grad_(True) for x in leaves]
    out(f"{op}: B={B} T={T} C={H * N} HEAD_SIZE={N}")
    for silent in (True, False):                      # warm-up pass first, wkv5/run.py:769-770
        with torch.autograd.profiler.profile(use_device="cuda") as prof:
            ys = hip(*hip_in)
        if not silent:
            out("HIP forward\n" + prof.key_averages().table(sort_by="self_device_time_total", row_limit=4))
        with torch.autograd.profiler.profile(use_device="cuda") as prof:
            sum(LOSS(y.float()) for y in ys).backward()
        if not silent:
            out("HIP backward\n" + prof.key_averages().table(sort_by="self_device_time_total", row_limit=6))


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m rwkv_cuda_amd.run", description=__doc__.split("\n\n")[0])
    ap.add_argument("op", choices=OPS)
    ap.add_argument("job", nargs="?", default="check", choices=["check", "benchmark"])
    ap.add_argument("--B", type=int)
    ap.add_argument("--T", type=int)
    ap.add_argument("--H", type=int, help="heads (channels = head size x H; for wkv and depthwise_conv1d: channels / 64)")
    ap.add_argument("--N", type=int, help="head size for wkv5, wkv5_bf16, wkv5a, wkv6, wkv6_state (default 64; 1..128, as the "
                                          "reference's -D_N_: its checks use 2 and 4, wkv5_bf16/run.py ships 128)")
    args = ap.parse_args(argv)
    if args.N is not None:
        if not 1 <= args.N <= 128 or (args.N != 64 and args.op not in ("wkv5", "wkv5_bf16", "wkv5a", "wkv6", "wkv6_state")):
            ap.error("--N: 1..128 for wkv5, wkv5_bf16, wkv5a, wkv6, wkv6_state; the other ops have head size 64")
        global N
        N = args.N
    if not torch.cuda.is_available():
        raise SystemExit("rwkv_cuda_amd.run needs a HIP device: the kernels have no CPU path")
    dev = torch.device("cuda:0")
    if args.job == "check":
        B, T, H = args.B or 2, args.T or 64, args.H or 2
        worst, bar = check(args.op, dev, B, T, H)
        print(f"worst err ratio {worst:.3e} (bar {bar:.0e})")
        return 0 if worst <= bar else 1
    B, T, H = BENCH_SHAPE[args.op]
    benchmark(args.op, dev, args.B or B, args.T or T, args.H or H)
    return 0


if __name__ == "__main__":
    sys.exit(main())
