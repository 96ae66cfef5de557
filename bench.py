#!/usr/bin/env python3
"""Headline benchmark: WKV6 bf16 forward+backward at B=8, T=4096, C=2048 (H=32, N=64) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload wkv6|wkv6_state|wkv6_b1|wkv5|wkv5_n128|rwkv7|wkv4|wkv4_b32|timex|...]

A "step" is one forward + one backward of the operator over one batch of synthetic inputs that are
already resident in HBM, through the same C-ABI calls and the same wrapper-side torch work
(decay pre-transform, per-batch gradient sums) as the autograd.Function does.  Prints ONE JSON line.

  value            whole-job throughput in Mtokens/s (tokens = B*T per step)
  roofline         the slowest kernel of the step, timed alone with HIP events on the stream it is
                   launched on: achieved = its algorithmic bytes / its mean duration, against 8 TB/s
  cpu_baseline     the CPU oracle (a port of the reference's PyTorch recurrence, fp32, autograd) timed on
                   this host's cores on a bounded sample (T_cpu steps of the same B, H, N)
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X published dense fp32 matrix rate
F16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 (and bf16) matrix rate
# depthwise_conv1d up to T = 1024 forms every fp32 product from three fp16 matrix products (two fp16 terms per operand):
# its ceiling in algorithmic (fp32) flops is a third of the fp16 rate
H2_PRODUCTS = 3
PREWARM_S = 0.3                # seconds of untimed load before the warmup steps (clock ramp)
ALGO = "chunked"
FLAGS = 0                      # RWKV_FLAG_SWEEPS when --algo sweeps: passed per call to the *_ex entry points

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see profiles/), keyed
# by kernel label at the headline shape; None = not measured for the current kernels.
TRAFFIC_MEASURED = {
    # profiles/wkv6_fused_kernels_B8_T4096_C2048.md  (FETCH_SIZE x 2 KiB + WRITE_SIZE x 1 KiB)
    "wkv6_fwd_fused (keeps states)": 537.2e6 + 335.6e6,
    "wkv6_bwd_fused (+ gu batch sum)": 872.9e6 + 536.9e6,
    # profiles/wkv5_fused_kernels_B8_T4096_C2048.md
    "wkv6_fwd_fused<head decay> (keeps states)": 402.9e6 + 335.6e6,
    "wkv6_bwd_fused<head decay> (+ batch sums)": 738.7e6 + 402.7e6,
    # profiles/wkv5_ws_kernels_B8_T4096_C2048.md
    "wkv6_fwd_ws<head decay>": 403e6 + 134e6,
    "wkv6_bwd_a_ws<head decay>": 548e6 + 533e6,
    "wkv6_bwd_b_ws<head decay>": 957e6 + 269e6,
    # profiles/wkv5_fp32_sweep_kernels_B8_T4096_C4096.md, profiles/wkv5a_sweep_kernels_B8_T4096_C4096.md
    "wkv_sweep<gr+gu+gw, fp32 I/O>": 2148e6 + 537e6,
    "wkv_sweep<gr+gu+gw, two-sided>": 2148e6 + 537e6,
    # profiles/rwkv7_chunk_kernels_B8_T4096_C4096.md (four calls of T = 1024)
    "rwkv7c_fwd x4 (T=1024 each)": 4 * (411.2e6 + 746.6e6),
    "rwkv7c_bwd x4": 4 * (1149.7e6 + 411.0e6),
    # profiles/wkv5_split_kernels_B8_T4096_C4096_N128.md (both launches of a kernel and the sums that follow them)
    "wkv6_fwd_ws<head decay, split> x2": (805.7e6 + 536.9e6) + (1342.5e6 + 268.5e6),
    "wkv6_bwd_a_ws<head decay, split> x2": (1095.4e6 + 1334.3e6) + (1638.6e6 + 1065.4e6),
    "wkv6_bwd_b_ws<head decay, split> x2 + split_sum x2": 2 * (1911.1e6 + 1076.0e6) + 2 * (1073.7e6 + 268.4e6),
    # profiles/wkv4_reg_kernels_B4_T512_C768.md
    "wkv4_fwd_reg": 12.7e6 + 6.3e6,
    "wkv4_bwd_reg + wkv4_batch_sum": 19.1e6 + 12.6e6,
    # profiles/wkv4_reg_kernels_B32_T768_C768.md
    "wkv4_fwd_reg B32 T768": 152.5e6 + 78.4e6,
    "wkv4_bwd_reg + wkv4_batch_sum B32 T768": 227.2e6 + 151.7e6,
    # profiles/timex_h2_kernels_B32_C768_T768.md
    "timex_conv_h2 (forward)": 78.0e6 + 75.5e6,
    "timex backward (timex_conv_h2 + timex_gw_sum_h2)": (78.0e6 + 75.5e6) + (151.2e6 + 2.4e6),
}


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_gpu(fn, iters, warmup):
    """Mean milliseconds per call of fn, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = _events(2)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


# --------------------------------------------------------------------------------------------
# workloads: each returns (step_fn, tokens_per_step, kernels, config, cpu_baseline_fn)
# kernels: list of (label, fn, algorithmic_bytes) -- every kernel the step launches from the library
# --------------------------------------------------------------------------------------------

def make_wkv6(dev, state, B=8):
    from rwkv_cuda_amd import _lib, synth
    from rwkv_cuda_amd._call import call
    lib = _lib.load()
    T, H, N = 4096, 32, 64
    C = H * N
    bf = torch.bfloat16
    r, k, v, w, u, gy, s0 = (x.to(dev) if x is not None else None for x in synth.wkv6_inputs(B, T, C, H, seed=42, state=state))
    new = lambda *s: torch.empty(s, device=dev, dtype=bf)
    y, gr, gk, gv, gw, gu = new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C), new(B, C)
    gu_sum = new(H, N)
    nbytes = lib.rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
    ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    nsaved = lib.rwkv_wkv6f_saved_bytes(B, T, C, H)
    saved = torch.empty(nsaved, device=dev, dtype=torch.uint8)   # the states the forward hands to the backward
    tok = B * T
    gs = new(B, H, N, N) if state else None
    name = "wkv6_state" if state else "wkv6"
    # what WKV_6 / WKV_6STATE.forward and backward do: raw bf16 decay straight into the kernels, the forward keeps the state
    # entering every 64th token, the backward is one reverse sweep, and the wrapper's torch.sum(gu, 0) (wkv6/run.py:169,
    # wkv6_state/run.py:123) runs inside the library
    fwd = lambda: call("rwkv_wkv6f_forward", dev, B, T, C, H, r, k, v, w, u, s0, y, saved, nsaved, FLAGS)
    bwd_all = lambda: call("rwkv_wkv6f_backward_saved", dev, B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu_sum, gs,
                           saved, nsaved, ws, nbytes, FLAGS)

    def step():
        fwd()
        bwd_all()

    def bwd(mask):
        def run():
            if state:
                call("rwkv_wkv6state_backward_ex", dev, B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu, gs, ws, nbytes, mask | FLAGS)
            else:
                call("rwkv_wkv6raw_backward_ex", dev, B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu, ws, nbytes, mask | FLAGS)
        return run

    # algorithmic bytes per kernel: tensors it must read once + outputs it must write once, 2 B per element
    if ALGO == "chunked":
        kernels = [("wkv6_fwd_fused (keeps states)", fwd, 10 * C * tok),                      # r k v w -> y
                   ("wkv6_bwd_fused (+ gu batch sum)", bwd_all, 18 * C * tok)]              # r k v w gy -> gr gk gv gw
    else:
        kernels = [("wkv_sweep<FWD>", fwd, 10 * C * tok),
                   ("wkv_sweep<GR>", bwd(1), 12 * C * tok),               # r k v w gy -> gr
                   ("wkv_sweep<GV>", bwd(2), 10 * C * tok),               # r k w gy -> gv
                   ("wkv_sweep<GK>", bwd(4), 14 * C * tok)]               # r k v w gy -> gk gw

    def cpu_baseline(t_cpu=256):
        from oracle import wkv56 as O
        rr, kk, vv, ww, uu, gg, ss = synth.wkv6_inputs(B, t_cpu, C, H, seed=42, state=state)
        f = torch.float32
        t0 = time.perf_counter()
        O.wkv6_grads(B, t_cpu, C, H, rr.float(), kk.float(), vv.float(), ww.float(), uu.float(), gg.float(),
                     s0=None if ss is None else ss.float(), dtype=f)
        dt = time.perf_counter() - t0
        return B * t_cpu / dt / 1e6, f"{name} fwd+bwd, fp32 autograd of the recurrent form, B{B} H{H} N{N}, T_cpu={t_cpu} ({dt:.1f} s)"

    cfg = {"workload": f"{name} bf16 fwd+bwd B{B} T{T} C{C} H{H} N{N}", "B": B, "T": T, "C": C, "H": H, "N": N,
           "algorithmic_bytes_per_token": 28 * C}
    if B * H < 256 and ALGO == "chunked":
        # fewer sequences than CUs: the library cuts them into blocks joined by a scan; the same step with one workgroup
        # per sequence (RWKV_FLAG_WHOLE, 0x200) for comparison
        def whole():
            call("rwkv_wkv6f_forward", dev, B, T, C, H, r, k, v, w, u, s0, y, saved, nsaved, FLAGS | 0x200)
            call("rwkv_wkv6f_backward_saved", dev, B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu_sum, gs, saved, nsaved, ws, nbytes, FLAGS | 0x200)
        for _ in range(5):
            whole()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            whole()
        e1.record()
        torch.cuda.synchronize()
        cfg["ms_per_step_one_workgroup_per_sequence"] = round(e0.elapsed_time(e1) / 50, 4)
    return step, tok, kernels, cfg, cpu_baseline, 28 * C * tok


def make_wkv5(dev, H=32, N=64):
    """N = 64: the matrix-core kernels at B8 T4096 C2048; N = 128: wkv5_bf16/run.py:17-22 as shipped (B8 T4096 C4096),
    which runs on the same kernels with every head taken as four heads of 64 (two launches per kernel, fp32 terms added)."""
    from rwkv_cuda_amd import _lib, synth
    from rwkv_cuda_amd._call import call
    lib = _lib.load()
    B, T = 8, 4096
    C = H * N
    bf = torch.bfloat16
    r, k, v, w, u, gy = (x.to(dev) for x in synth.wkv5_inputs(B, T, C, H, seed=42))
    new = lambda *s: torch.empty(s, device=dev, dtype=bf)
    y, gr, gk, gv, gw, gu = new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C), new(B, C), new(B, C)
    gw_sum, gu_sum = new(H, N), new(H, N)
    decay = torch.empty(2 * C, device=dev, dtype=torch.float32)
    nbytes = lib.rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    fbytes = lib.rwkv_wkv5_forward_workspace_bytes(B, T, C, H)            # 0 unless N = 128
    fws = torch.empty(max(fbytes, 16), device=dev, dtype=torch.uint8)
    tok = B * T
    ew = (-torch.exp(w.float())).contiguous()
    eew = torch.exp(ew).contiguous()

    one_sweep = N == 64 and ALGO == "chunked"
    if one_sweep:
        nsaved = lib.rwkv_wkv5s_saved_bytes(B, T, C, H)
        saved = torch.empty(nsaved, device=dev, dtype=torch.uint8)
        sbytes = lib.rwkv_wkv5s_backward_workspace_bytes(B, T, C, H)
        sws = torch.empty(sbytes, device=dev, dtype=torch.uint8)
    fwd1 = lambda: call("rwkv_wkv5s_forward", dev, B, T, C, H, r, k, v, w, u, y, decay, saved, nsaved, FLAGS)
    bwd1 = lambda: call("rwkv_wkv5s_backward", dev, B, T, C, H, r, k, v, w, decay, u, gy, gr, gk, gv, gw_sum, gu_sum, saved, nsaved, sws, sbytes, FLAGS)

    def step():
        # what WKV_5.forward / backward do; the decay transforms (wkv5_bf16/run.py:63-64) and the sums over the batch
        # (:86-87) run inside the library.  Head size 64: one forward and one reverse sweep (the kernels of wkv6).
        if one_sweep:
            fwd1()
            bwd1()
            return
        call("rwkv_wkv5raw_forward_ws", dev, B, T, C, H, r, k, v, w, u, y, decay, fws, fbytes, FLAGS)
        call("rwkv_wkv5raw_backward", dev, B, T, C, H, r, k, v, decay, u, gy, gr, gk, gv, gw_sum, gu_sum, ws, nbytes, FLAGS)

    def bwd(mask):
        def run():
            call("rwkv_wkv5_backward_ex", dev, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu, ws, nbytes, mask | FLAGS)
        return run

    if one_sweep:
        kernels = [("wkv6_fwd_fused<head decay> (keeps states)", fwd1, 8 * C * tok),       # r k v -> y
                   ("wkv6_bwd_fused<head decay> (+ batch sums)", bwd1, 14 * C * tok)]      # r k v gy -> gr gk gv
    elif N == 64:
        kernels = [("wkv6_fwd_ws<head decay>", lambda: call("rwkv_wkv5_forward_ex", dev, B, T, C, H, r, k, v, eew, u, y, FLAGS), 8 * C * tok),
                   ("wkv6_bwd_a_ws<head decay>", bwd(1), 10 * C * tok),           # r k v gy -> gr (+ fp32 workspace)
                   ("wkv6_bwd_b_ws<head decay>", bwd(4), 12 * C * tok)]           # r k v gy -> gk gv
    else:
        kernels = [("wkv6_fwd_ws<head decay, split> x2", lambda: call("rwkv_wkv5_forward_ws", dev, B, T, C, H, r, k, v, eew, u, y, fws, fbytes, FLAGS), 8 * C * tok),
                   ("wkv6_bwd_a_ws<head decay, split> x2", bwd(1), 10 * C * tok),
                   ("wkv6_bwd_b_ws<head decay, split> x2 + split_sum x2", bwd(4), 12 * C * tok)]

    def cpu_baseline(t_cpu=256):
        from oracle import wkv56 as O
        rr, kk, vv, ww, uu, gg = synth.wkv5_inputs(B, t_cpu, C, H, seed=42)
        t0 = time.perf_counter()
        O.wkv5_grads(B, t_cpu, C, H, rr.float(), kk.float(), vv.float(), ww.float(), uu.float(), gg.float(), dtype=torch.float32)
        dt = time.perf_counter() - t0
        return B * t_cpu / dt / 1e6, f"wkv5 fwd+bwd, fp32 autograd of the recurrent form, B{B} H{H} N{N}, T_cpu={t_cpu} ({dt:.1f} s)"

    cfg = {"workload": f"wkv5 bf16 fwd+bwd B{B} T{T} C{C} H{H} N{N}", "B": B, "T": T, "C": C, "H": H, "N": N,
           "algorithmic_bytes_per_token": 22 * C}
    return step, tok, kernels, cfg, cpu_baseline, 22 * C * tok


def make_wkv5_fp32(dev):
    """The fp32 wkv5 op at the reference's own benchmark shape (wkv5/run.py:395-399)."""
    from rwkv_cuda_amd import _lib
    from rwkv_cuda_amd._call import call
    lib = _lib.load()
    B, T, H, N = 8, 4096, 64, 64
    C = H * N
    g = torch.Generator().manual_seed(42)
    rnd = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(dev)      # uniform(-1,1) as in wkv5/run.py:516-520
    r, k, v, gy = rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(B, T, C)
    w, u = rnd(C), rnd(C)
    new = lambda *s: torch.empty(s, device=dev, dtype=torch.float32)
    y, gr, gk, gv, gw, gu = new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C), new(B, C), new(B, C)
    tok = B * T
    ew = (-torch.exp(w)).contiguous()
    eew = torch.exp(ew).contiguous()

    def step():
        ew_ = (-torch.exp(w)).contiguous()
        eew_ = torch.exp(ew_).contiguous()
        call("rwkv_wkv5f32_forward", dev, B, T, C, H, r, k, v, eew_, u, y)
        call("rwkv_wkv5f32_backward", dev, B, T, C, H, r, k, v, eew_, ew_, u, gy, gr, gk, gv, gw, gu)
        return torch.sum(gw, 0), torch.sum(gu, 0)

    def bwd(mask):
        def run():
            call("rwkv_wkv5f32_backward_ex", dev, B, T, C, H, r, k, v, eew, ew, u, gy, gr, gk, gv, gw, gu, mask | FLAGS)
        return run

    kernels = [("wkv_sweep<fwd, fp32 I/O>", lambda: call("rwkv_wkv5f32_forward", dev, B, T, C, H, r, k, v, eew, u, y), 16 * C * tok),
               ("wkv_sweep<gr+gu+gw, fp32 I/O>", bwd(1), 20 * C * tok),       # r k v gy -> gr
               ("wkv_sweep<gv, fp32 I/O>", bwd(2), 16 * C * tok),             # r k gy -> gv
               ("wkv_sweep<gk, fp32 I/O>", bwd(4), 20 * C * tok)]             # r k v gy -> gk

    def cpu_baseline(t_cpu=128):
        from oracle import wkv56 as O
        gg = torch.Generator().manual_seed(42)
        rn = lambda *s: torch.rand(*s, generator=gg) * 2 - 1
        a = [rn(B, t_cpu, C), rn(B, t_cpu, C), rn(B, t_cpu, C), rn(C), rn(C), rn(B, t_cpu, C)]
        t0 = time.perf_counter()
        O.wkv5_grads(B, t_cpu, C, H, *a, dtype=torch.float32)
        dt = time.perf_counter() - t0
        return B * t_cpu / dt / 1e6, f"wkv5 fwd+bwd, fp32 autograd of the recurrent form, B{B} H{H} N{N}, T_cpu={t_cpu} ({dt:.1f} s)"

    cfg = {"workload": f"wkv5 fp32 fwd+bwd B{B} T{T} C{C} H{H} N{N}", "B": B, "T": T, "C": C, "H": H, "N": N,
           "algorithmic_bytes_per_token": 44 * C}
    return step, tok, kernels, cfg, cpu_baseline, 44 * C * tok


def make_wkv5a(dev):
    """wkv5a (two-sided decay and bonus, fp32) at the reference's timing shape (wkv5a/run.py:62-66)."""
    from rwkv_cuda_amd import _lib
    from rwkv_cuda_amd._call import call
    lib = _lib.load()
    B, T, H, N = 8, 4096, 64, 64
    C = H * N
    g = torch.Generator().manual_seed(42)
    rnd = lambda *s, lo=-1.0: (torch.rand(*s, generator=g) * (1.0 - lo) + lo).to(dev)   # wkv5a/run.py:389-398
    r, k, v, gy = rnd(B, T, C), rnd(B, T, C), rnd(B, T, C), rnd(B, T, C)
    w1, u1, w2, u2 = rnd(H, N, lo=-8.0), rnd(H, N), rnd(H, N, lo=-8.0), rnd(H, N)
    new = lambda *s: torch.empty(s, device=dev, dtype=torch.float32)
    y, gr, gk, gv = new(B, T, C), new(B, T, C), new(B, T, C), new(B, T, C)
    gw1, gu1, gw2, gu2 = new(B, C), new(B, C), new(B, C), new(B, C)
    tok = B * T
    dec = lambda w: ((-torch.exp(w)).contiguous(), torch.exp(-torch.exp(w)).contiguous())
    (ew1, eew1), (ew2, eew2) = dec(w1), dec(w2)

    def step():
        (a1, b1), (a2, b2) = dec(w1), dec(w2)
        call("rwkv_wkv5a_forward", dev, B, T, C, H, r, k, v, b1, u1, b2, u2, y)
        call("rwkv_wkv5a_backward", dev, B, T, C, H, r, k, v, b1, a1, u1, b2, a2, u2, gy, gr, gk, gv, gw1, gu1, gw2, gu2)
        return torch.sum(gw1, 0), torch.sum(gu1, 0), torch.sum(gw2, 0), torch.sum(gu2, 0)

    def bwd(mask):
        def run():
            call("rwkv_wkv5a_backward_ex", dev, B, T, C, H, r, k, v, eew1, ew1, u1, eew2, ew2, u2, gy, gr, gk, gv, gw1, gu1, gw2, gu2, mask | FLAGS)
        return run

    kernels = [("wkv_sweep<fwd, two-sided>", lambda: call("rwkv_wkv5a_forward", dev, B, T, C, H, r, k, v, eew1, u1, eew2, u2, y), 16 * C * tok),
               ("wkv_sweep<gr+gu+gw, two-sided>", bwd(1), 20 * C * tok),
               ("wkv_sweep<gv, two-sided>", bwd(2), 16 * C * tok),
               ("wkv_sweep<gk, two-sided>", bwd(4), 20 * C * tok)]

    def cpu_baseline(t_cpu=128):
        from oracle import wkv5a as A
        gg = torch.Generator().manual_seed(42)
        rn = lambda *s, lo=-1.0: torch.rand(*s, generator=gg) * (1.0 - lo) + lo
        a = [rn(B, t_cpu, C), rn(B, t_cpu, C), rn(B, t_cpu, C), rn(H, N, lo=-8.0), rn(H, N), rn(H, N, lo=-8.0), rn(H, N), rn(B, t_cpu, C)]
        t0 = time.perf_counter()
        A.grads(B, t_cpu, C, H, *a, dtype=torch.float32)
        dt = time.perf_counter() - t0
        return B * t_cpu / dt / 1e6, f"wkv5a fwd+bwd, fp32 autograd of the recurrent form, B{B} H{H} N{N}, T_cpu={t_cpu} ({dt:.1f} s)"

    cfg = {"workload": f"wkv5a fp32 fwd+bwd B{B} T{T} C{C} H{H} N{N}", "B": B, "T": T, "C": C, "H": H, "N": N,
           "algorithmic_bytes_per_token": 44 * C}
    return step, tok, kernels, cfg, cpu_baseline, 44 * C * tok


def make_rwkv7(dev, fp32=False):
    """fp32=True: the reference's -D_FP32_ mode (every bf16 tensor fp32), same kernels with fp32 loads and stores."""
    from rwkv_cuda_amd import synth
    from rwkv_cuda_amd._call import call
    B, T, H, N = 8, 4096, 64, 64
    C = H * N
    TS = T // 4                                                   # four chained T=1024 calls
    sfx, eb = ("_f32", 4) if fp32 else ("", 2)                    # entry-point suffix, bytes per element
    s0, r, w, k, v, a, b, dy, dsT = (x.to(dev) for x in synth.rwkv7_inputs(B, T, H, N, seed=42))
    if fp32:
        r, w, k, v, a, b, dy = (x.float() for x in (r, w, k, v, a, b, dy))
    seg = [[x[:, i * TS:(i + 1) * TS].contiguous() for x in (r, w, k, v, a, b, dy)] for i in range(4)]
    f32 = dict(device=dev, dtype=torch.float32)
    ys = [torch.empty_like(s[0]) for s in seg]
    sTs = [torch.empty_like(s0) for _ in range(4)]
    ss = [torch.empty(B, H, TS // 16, N, N, **f32) for _ in range(4)]
    sas = [torch.empty(B, TS, H, N, **f32) for _ in range(4)]
    grads = [[torch.empty_like(s[0]) for _ in range(6)] for s in seg]
    ds = [torch.empty_like(s0) for _ in range(4)]
    tok = B * T

    def fwd():
        st = s0
        for i in range(4):
            rr, ww, kk, vv, aa, bb, _ = seg[i]
            if fp32:
                call("rwkv7_statepassing_forward_f32", dev, B, TS, H, st, rr, ww, kk, vv, aa, bb, ys[i], sTs[i], ss[i], sas[i])
            else:
                call("rwkv7_statepassing_forward_ex", dev, B, TS, H, st, rr, ww, kk, vv, aa, bb, ys[i], sTs[i], ss[i], sas[i], FLAGS)
            st = sTs[i]

    def bwd():
        g = dsT
        for i in (3, 2, 1, 0):
            rr, ww, kk, vv, aa, bb, dd = seg[i]
            if fp32:
                call("rwkv7_statepassing_backward_f32", dev, B, TS, H, rr, ww, kk, vv, aa, bb, dd, g, ss[i], sas[i], ds[i], *grads[i])
            else:
                call("rwkv7_statepassing_backward_ex", dev, B, TS, H, rr, ww, kk, vv, aa, bb, dd, g, ss[i], sas[i], ds[i], *grads[i], FLAGS)
            g = ds[i]

    def step():
        fwd()
        bwd()

    chunked = not fp32 and ALGO == "chunked"
    kernels = [("rwkv7c_fwd x4 (T=1024 each)" if chunked else "rwkv7_fwd x4 (T=1024 each)", fwd, 7 * eb * C * tok),
               ("rwkv7c_bwd x4" if chunked else "rwkv7_bwd x4", bwd, 13 * eb * C * tok)]

    def cpu_baseline(t_cpu=64):
        from oracle import rwkv7 as O
        args = synth.rwkv7_inputs(B, t_cpu, H, N, seed=42)
        t0 = time.perf_counter()
        O.grads(*[x.float() for x in args], dtype=torch.float32)
        dt = time.perf_counter() - t0
        return B * t_cpu / dt / 1e6, f"rwkv7 fwd+bwd, fp32 autograd of the einsum step, B{B} H{H} N{N}, T_cpu={t_cpu} ({dt:.1f} s)"

    cfg = {"workload": f"rwkv7 state-passing {'fp32' if fp32 else 'bf16'} fwd+bwd B{B} T{T} (4 x {TS}) C{C} H{H} N{N}", "B": B, "T": T,
           "C": C, "H": H, "N": N, "algorithmic_bytes_per_token": 20 * eb * C}
    return step, tok, kernels, cfg, cpu_baseline, 20 * eb * C * tok


def make_wkv4(dev, B=4, T=512):
    """B4 T512: the configuration of the contract; B32 T768: the shape of the reference's own check (wkv/run.py:152-154)."""
    from rwkv_cuda_amd import _lib, synth
    from rwkv_cuda_amd._call import call
    lib = _lib.load()
    C = 768
    w_raw, u, k, v, gy = (x.to(dev) for x in synth.wkv4_inputs(B, T, C, seed=42))
    y, gk, gv = (torch.empty(B, T, C, device=dev) for _ in range(3))
    nbytes = lib.rwkv_wkv4raw_backward_workspace_bytes(B, T, C)
    ws = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    tok = B * T
    gw, gu = torch.empty(C, device=dev), torch.empty(C, device=dev)

    def step():
        # what WKV.forward / backward do; w = -exp(w_raw), the zero-fills and the sums over the batch (wkv/run.py:95,110-116)
        # run inside the library
        call("rwkv_wkv4raw_forward", dev, B, T, C, w_raw, u, k, v, y)
        call("rwkv_wkv4raw_backward", dev, B, T, C, w_raw, u, k, v, gy, gw, gu, gk, gv, ws, nbytes)

    tag = "" if (B, T) == (4, 512) else f" B{B} T{T}"
    kernels = [("wkv4_fwd_reg" + tag, lambda: call("rwkv_wkv4raw_forward", dev, B, T, C, w_raw, u, k, v, y), 12 * C * tok),
               ("wkv4_bwd_reg + wkv4_batch_sum" + tag, lambda: call("rwkv_wkv4raw_backward", dev, B, T, C, w_raw, u, k, v, gy, gw, gu, gk, gv, ws, nbytes), 20 * C * tok)]

    def cpu_baseline():
        from oracle import wkv4 as O
        ww, uu, kk, vv, gg = synth.wkv4_inputs(B, T, C, seed=42)
        t0 = time.perf_counter()
        kk_, vv_, ww_, uu_ = (x.clone().requires_grad_(True) for x in (kk, vv, ww, uu))
        O.conv_form(B, T, C, ww_, uu_, kk_, vv_).backward(gg)
        dt = time.perf_counter() - t0
        return B * T / dt / 1e6, f"wkv4 fwd+bwd, grouped F.conv1d formulation, fp32, full B{B} T{T} C{C} ({dt:.1f} s)"

    cfg = {"workload": f"wkv4 fp32 fwd+bwd B{B} T{T} C{C}", "B": B, "T": T, "C": C, "algorithmic_bytes_per_token": 32 * C}
    # The step is three launches of 4 to 17 us: at this size the gaps between launches are a third of it.  A caller who
    # replays the step from a HIP graph does not pay them; the same step captured once and replayed, for comparison
    # (no entry point allocates, synchronises or records a memset, so the calls capture as they are).
    try:
        step()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            step()                                         # warm the stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(10):
                    step()
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(30):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        cfg["ms_per_step_replayed_from_a_hip_graph"] = round(e0.elapsed_time(e1) / 300, 5)
    except Exception as exc:                               # graphs are an extra: never let them fail the benchmark
        cfg["ms_per_step_replayed_from_a_hip_graph"] = f"not measured: {type(exc).__name__}"
    return step, tok, kernels, cfg, cpu_baseline, 32 * C * tok


def make_timex(dev):
    from rwkv_cuda_amd import synth
    from rwkv_cuda_amd._call import call
    B, C, T = 32, 768, 768
    w, k, g = (x.to(dev) for x in synth.timex_inputs(B, C, T, seed=42))
    x, gk = (torch.empty(B, C, T, device=dev) for _ in range(2))
    gw = torch.empty(C, T, device=dev)
    tok = B * T

    # what TimeX.apply(...).backward() launches at this shape: gw comes out summed over the batch
    def step():
        call("rwkv_timex_forward", dev, w, k, x, 0.0, B, C, T)
        call("rwkv_timex_backward_sum", dev, w, k, g, gw, gk, B, C, T)

    fwd_bytes = (C * T + 2 * B * C * T) * 4
    bwd_bytes = (2 * C * T + 3 * B * C * T) * 4
    # The direct convolution does T (T + 1) / 2 multiply-adds per row and output array, in fp32: 95 flop per byte in the
    # forward and 125 in the backward at T = 768, against a ridge of 104 (a third of the fp16 matrix rate over the HBM
    # peak): the kernels sit at the ridge, and the matrix rate is the bound that is reported.
    conv_flops = B * C * T * (T + 1)
    kernels = [("timex_conv_h2 (forward)", lambda: call("rwkv_timex_forward", dev, w, k, x, 0.0, B, C, T), fwd_bytes, conv_flops),
               ("timex backward (timex_conv_h2 + timex_gw_sum_h2)",
                lambda: call("rwkv_timex_backward_sum", dev, w, k, g, gw, gk, B, C, T), bwd_bytes, 2 * conv_flops)]

    def cpu_baseline(bs=4):
        from oracle import timex as O
        ww, kk, gg = synth.timex_inputs(bs, C, T, seed=42)
        t0 = time.perf_counter()
        O.grads(ww, kk, gg, bs, C, T, dtype=torch.float32)
        dt = time.perf_counter() - t0
        return bs * T / dt / 1e6, f"depthwise_conv1d fwd+bwd, zero-padded grouped F.conv1d, fp32, B={bs} of 32, C{C} T{T} ({dt:.1f} s)"

    cfg = {"workload": f"depthwise_conv1d fp32 fwd+bwd B{B} C{C} T{T}", "B": B, "C": C, "T": T,
           "algorithmic_bytes_per_step": fwd_bytes + bwd_bytes, "algorithmic_flops_per_step": 3 * conv_flops}
    return step, tok, kernels, cfg, cpu_baseline, fwd_bytes + bwd_bytes


WORKLOADS = {
    "wkv6": lambda dev: make_wkv6(dev, False),
    "wkv6_state": lambda dev: make_wkv6(dev, True),
    "wkv6_b1": lambda dev: make_wkv6(dev, False, B=1),
    "wkv5": make_wkv5,
    "wkv5_n128": lambda dev: make_wkv5(dev, H=32, N=128),
    "wkv5_fp32": make_wkv5_fp32,
    "wkv5a": make_wkv5a,
    "rwkv7": make_rwkv7,
    "rwkv7_fp32": lambda dev: make_rwkv7(dev, fp32=True),
    "wkv4": make_wkv4,
    "wkv4_b32": lambda dev: make_wkv4(dev, B=32, T=768),
    "timex": make_timex,
}
DTYPES = {"wkv6": "bf16", "wkv6_state": "bf16", "wkv6_b1": "bf16", "wkv5": "bf16", "wkv5_n128": "bf16", "wkv5_fp32": "f32", "wkv5a": "f32", "rwkv7": "bf16", "rwkv7_fp32": "f32", "wkv4": "f32", "wkv4_b32": "f32", "timex": "f16x2 (every fp32 operand as two fp16 terms, fp32 accumulation)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="wkv6", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--algo", default="chunked", choices=["chunked", "sweeps"],
                    help="wkv5 / wkv6 / rwkv7 kernels: chunked matrix-core formulation (default) or the sequential fp32 recurrence")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, so that a rocprofv3 --pmc run holds a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; every (batch, head) is an independent unit and no "
                 "multi-GPU path exists, so --gpus must be 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible; the kernels have no CPU path")

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    from rwkv_cuda_amd import _lib
    global ALGO, FLAGS
    ALGO = args.algo
    FLAGS = 0x100 if args.algo == "sweeps" else 0
    step, tok, kernels, cfg, cpu_baseline, step_bytes = WORKLOADS[args.workload](dev)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)                       # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # The GPU raises its clocks over the first tens of milliseconds of load (a 20-step run of the headline workload reads
    # 12 % slower than a 300-step one), so the device is first kept busy with the same step for PREWARM_S seconds; this
    # is reported as "prewarm_s" and is separate from the W warmup steps and the K timed steps.
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREWARM_S:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # EXACTLY K timed steps between two synchronisations (the contract's figure), with a HIP event after every step so
    # that the spread over the steps can be reported too (an event record costs no kernel and ~1 us of host time)
    marks = _events(args.steps + 1)
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = 1e3 * dt / args.steps
    mtok = tok / (dt / args.steps) / 1e6
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    ms_min, ms_median = per_step[0], per_step[len(per_step) // 2]

    # what a plain copy reaches on this device (read 1 GiB + write 1 GiB per launch): the achievable HBM rate beside the 8 TB/s peak
    src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
    dst = torch.empty_like(src)
    copy_ms = time_gpu(lambda: dst.copy_(src), 10, 3)
    copy_gbps = 2 * src.numel() * 4 / (copy_ms * 1e-3) / 1e9
    # the same 1 GiB as a read-only stream and as a write-only stream (rwkv_hbm_probe: 16 bytes per lane, grid-stride):
    # a kernel that mostly reads is priced against the first, one that mostly writes against the second
    from rwkv_cuda_amd._call import call as _call
    nb = src.numel() * 4
    read_ms = time_gpu(lambda: _call("rwkv_hbm_probe", dev, 0, src, dst, nb), 10, 3)
    write_ms = time_gpu(lambda: _call("rwkv_hbm_probe", dev, 1, None, dst, nb), 10, 3)
    read_gbps = src.numel() * 4 / (read_ms * 1e-3) / 1e9
    write_gbps = src.numel() * 4 / (write_ms * 1e-3) / 1e9
    del src, dst

    # per-kernel timing, HIP events on the launch stream
    per_kernel = []
    for label, fn, nbytes, *flops in kernels:
        ms = time_gpu(fn, max(5, args.steps), 2)
        per_kernel.append({"kernel": label, "ms": round(ms, 4), "algorithmic_bytes": nbytes,
                           "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)})
        if flops:                                # a kernel bound by the matrix cores, not by HBM
            per_kernel[-1].update(algorithmic_flops=flops[0], TFLOPs=round(flops[0] / (ms * 1e-3) / 1e12, 2))
    dom = max(per_kernel, key=lambda d: d["ms"])
    traffic = TRAFFIC_MEASURED.get(dom["kernel"]) if ALGO == "chunked" and args.workload != "wkv6_b1" else None   # counted at B = 8
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(dom["GBps"] / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_over_algorithmic": round(traffic / dom["algorithmic_bytes"], 3) if traffic else None,
                "launch_ms": dom["ms"], "algorithmic_bytes": dom["algorithmic_bytes"],
                "whole_step_frac": round(step_gbps / HBM_PEAK_GBS, 4),
                "hbm_copy_GBps": round(copy_gbps, 1), "frac_of_copy": round(dom["GBps"] / copy_gbps, 4),
                "whole_step_frac_of_copy": round(step_gbps / copy_gbps, 4),
                "hbm_read_GBps": round(read_gbps, 1), "hbm_write_GBps": round(write_gbps, 1)}
    if "TFLOPs" in dom:
        peak = F16_MFMA_PEAK_TFLOPS / H2_PRODUCTS
        roofline = {"bound": "mfma", "kernel": dom["kernel"], "achieved": dom["TFLOPs"], "peak": round(peak, 1),
                    "peak_is": "fp16 dense 2500 TFLOP/s / 3 fp16 products per fp32 product",
                    "unit": "TFLOP/s", "frac": round(dom["TFLOPs"] / peak, 4),
                    "frac_of_fp32_matrix_peak": round(dom["TFLOPs"] / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": traffic,
                    "traffic_over_algorithmic": round(traffic / dom["algorithmic_bytes"], 3) if traffic else None,
                    "launch_ms": dom["ms"], "algorithmic_flops": dom["algorithmic_flops"],
                    "hbm_frac": round(dom["GBps"] / HBM_PEAK_GBS, 4), "hbm_copy_GBps": round(copy_gbps, 1)}

    out = {
        "metric": "WKV6 bf16 fwd+bwd Mtokens/s @B8 T4096 C2048; % HBM peak achieved" if args.workload == "wkv6"
                  else f"{args.workload} fwd+bwd Mtokens/s; % HBM peak achieved",
        "value": round(mtok, 3), "unit": "Mtokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "ms_per_step_min": round(ms_min, 4), "ms_per_step_median": round(ms_median, 4),
        "prewarm_s": PREWARM_S, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": DTYPES[args.workload], "data": "synthetic", "config": cfg,
        "pct_hbm_peak": round(100 * step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "roofline": roofline, "kernels": per_kernel,
    }
    if not args.no_cpu_baseline:
        vals, t0 = [], time.perf_counter()
        while True:                              # bounded sample, repeated for about 10 s of CPU work
            val, sample = cpu_baseline()
            vals.append(val)
            if time.perf_counter() - t0 > 10.0 or len(vals) >= 20:
                break
        val = sum(vals) / len(vals)
        sample += f"; mean of {len(vals)} repeats"
        out["cpu_baseline"] = {"value": round(val, 5), "unit": "Mtokens/s", "cores": torch.get_num_threads(),
                               "kind": "port", "sample": sample, "host_cpus": os.cpu_count()}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
