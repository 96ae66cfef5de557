"""GPU parity of the wkv6 / wkv6_state pair that hands chunk states from the forward to a one-sweep backward
(rwkv_wkv6f_forward + rwkv_wkv6f_backward_saved), through the C ABI, against the CPU oracle and against the two-sweep
kernels.  The bar is the reference kernel's own error (fp32 emulation with its rounding points), as everywhere."""
import pytest
import torch

from oracle import wkv56 as O
from rwkv_cuda_amd import options, synth
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, assert_no_worse, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
NAMES = ["y", "gr", "gk", "gv", "gw", "gu", "gs"]


def run_pair(lib, B, T, H, r, k, v, w, u, s0, gy, flags=0, saved_fill=None):
    """forward + backward through the C ABI; every output and the handed-over states start as garbage"""
    C = H * 64
    d = [x.to(DEV) if x is not None else None for x in (r, k, v, w, u, s0, gy)]
    y = garbage((B, T, C), BF)
    nsv = lib.rwkv_wkv6f_saved_bytes(B, T, C, H)
    saved = torch.empty(nsv, device=DEV, dtype=torch.uint8)
    if saved_fill is not None:
        saved.fill_(saved_fill)
    call("rwkv_wkv6f_forward", DEV, B, T, C, H, *d[:6], y, saved, nsv, flags)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu = garbage((H, 64), BF)
    gs = garbage((B, H, 64, 64), BF) if s0 is not None else None
    n = lib.rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8).fill_(0x7f)
    call("rwkv_wkv6f_backward_saved", DEV, B, T, C, H, *d[:6], d[6], gr, gk, gv, gw, gu, gs, saved, nsv, ws, n, flags)
    torch.cuda.synchronize()
    off = (lib.rwkv_wkv6f_backward_workspace_bytes(B, T, C, H) + 15) // 16 * 16     # the flag words follow the two-sweep workspace
    handed_back = int(ws[off:off + B * H * 32].view(torch.int32).ne(0).view(B * H, 8).any(1).sum())
    return [y, gr, gk, gv, gw, gu] + ([gs] if s0 is not None else []), handed_back


# (B, T, H, state): one chunk, a cut chunk, an odd and an even number of chunks, T = 1, many chunks
# (from 256 tokens on these small batches run as several blocks per sequence: local states, a scan, the outputs)
SHAPES = [(1, 32, 1, False), (2, 50, 2, True), (1, 97, 3, True), (2, 64, 1, False), (3, 1, 1, True), (1, 7, 2, False),
          (2, 96, 2, True), (1, 200, 1, False), (1, 1000, 2, True), (1, 300, 2, True), (1, 257, 3, False), (2, 640, 1, True)]


@pytest.mark.parametrize("B,T,H,state", SHAPES)
def test_one_sweep_against_the_oracle(lib, B, T, H, state):
    print(f"\nwkv6 one sweep B={B} T={T} H={H} state={state}", flush=True)
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=300 + T, state=state)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    got, handed_back = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy, saved_fill=0x7f)
    assert handed_back == 0                                     # these decays stay inside the range of the mid-point factors
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert torch.isfinite(g.float()).all(), name
        assert_no_worse(name, a, e, g)
    gw = got[4].float()
    assert float(gw[:, T - 1].abs().max()) == 0.0              # w_{T-1} feeds nothing
    if not state:
        assert float(gw[:, 0].abs().max()) == 0.0              # nothing to decay at t = 0 without an initial state


@pytest.mark.parametrize("B,H,state", [(1, 8, True), (2, 32, False)])
def test_few_sequences_run_as_blocks_with_a_scan(lib, B, H, state):
    """B H below the number of CUs at T = 4096: the sequences are cut into blocks (32 of 128 tokens at B1 H8, 4 of 1024 at
    B2 H32), every block builds its state and gradient state from nothing, a scan hands each block what enters it, and the
    outputs follow.  Two heads against the oracle on the bar of the reference kernel; the saved states say how it was cut."""
    T, C = 4096, H * 64
    print(f"\nwkv6 blocks B={B} H={H} state={state}", flush=True)
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=330 + H, state=state)
    got, handed_back = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy, saved_fill=0x7f)
    assert handed_back == 0
    assert lib.rwkv_wkv6f_saved_bytes(B, T, C, H) > B * H * 64 * (64 * 64 * 3) + B * H * 32      # room for the scan
    hs = [1, H - 1]
    ch = torch.cat([torch.arange(h * 64, (h + 1) * 64) for h in hs])
    rr, kk, vv, ww, gg = (x[:, :, ch].contiguous() for x in (r, k, v, w, gy))
    uu = u[hs].contiguous()
    ss = s0[:, hs].contiguous() if state else None
    ref = list(O.wkv_grads_by_hand(B, T, 128, 2, rr, kk, vv, ww, uu, gg, ss, torch.float64))
    ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv6_bf16(B, T, 128, 2, rr, kk, vv, ww, uu, gg, s0=ss, hand=True)
    chd = ch.to(DEV)
    sub = [got[0][:, :, chd], got[1][:, :, chd], got[2][:, :, chd], got[3][:, :, chd], got[4][:, :, chd], got[5][hs]]
    if state:
        sub.append(got[6][:, hs])
    for name, a, e, g in zip(NAMES, ref, emu, sub):
        assert torch.isfinite(g.float()).all(), name
        assert_no_worse(f"blocks B{B} H{H} " + name, a, e, g)
    gw = got[4].float()
    assert float(gw[:, T - 1].abs().max()) == 0.0
    if not state:
        assert float(gw[:, 0].abs().max()) == 0.0


def test_one_sweep_hands_strong_decays_to_the_two_sweep_kernels(lib):
    """Decays so strong that a channel loses more than e^-60 over 16 tokens: those (batch, head) pairs are flagged by the
    one-sweep kernel and redone by the two-sweep kernels, whose chunks have a step-by-step path; the others are not."""
    B, T, H = 2, 100, 3
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=316, state=True)
    w = w.float()
    w[:, 40:60, :64] = 2.5                                      # head 0 of both batch rows
    w[1, 70:, 100] = 3.0                                        # one channel of (1, head 1), up to the last token
    w = w.to(BF)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    got, handed_back = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy)
    assert handed_back == 3, handed_back                        # (0,0), (1,0), (1,1); head 2 and (0,1) stay
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert torch.isfinite(g.float()).all(), name
        assert_no_worse(name, a, e, g)


def test_blocks_hand_strong_decays_back_too(lib):
    """The same with sequences long enough to be cut into blocks: a flag raised by any block of a head hands the head back."""
    B, T, H = 1, 700, 3
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=319, state=True)
    w = w.float()
    w[0, 400:430, 64:128] = 2.5                                 # head 1, inside one of the blocks
    w = w.to(BF)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    got, handed_back = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy)
    assert handed_back == 1, handed_back
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert torch.isfinite(g.float()).all(), name
        assert_no_worse(name, a, e, g)


def test_one_sweep_agrees_with_the_two_sweep_kernels(lib):
    """Same inputs through both pairs of kernels of the library: the results differ by at most one bf16 unit of the
    tensor's peak (they round the same fp32 quantities, formed in a different order)."""
    B, T, H = 2, 333, 2
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=317, state=True)
    one, _ = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy)
    d = [x.to(DEV) for x in (r, k, v, w, u, s0, gy)]
    y = garbage((B, T, C), BF)
    call("rwkv_wkv6state_forward", DEV, B, T, C, H, *d[:6], y)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu, gs = garbage((H, 64), BF), garbage((B, H, 64, 64), BF)
    n = lib.rwkv_wkv6f_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv6f_backward", DEV, B, T, C, H, *d[:6], d[6], gr, gk, gv, gw, gu, gs, ws, n, 0)
    torch.cuda.synchronize()
    for name, a, b in zip(NAMES, one, [y, gr, gk, gv, gw, gu, gs]):
        diff = float((a.float() - b.float()).abs().max()) / float(b.float().abs().max())
        print(f"  {name}: max difference {diff:.2e} of the peak", flush=True)
        assert diff <= 2.0 ** -7, name


def test_other_head_sizes_and_options_take_the_two_sweep_kernels(lib):
    """With a head size other than 64 there is nothing to hand over (0 bytes) and the pair runs the row kernels; with the
    sequential-sweeps option the handed-over buffer is ignored.  Results as good as ever."""
    B, T, H, N = 2, 40, 2, 32
    C = H * N
    g = torch.Generator().manual_seed(5)
    r, k, v = ((torch.randn(B, T, C, generator=g) * 0.5).to(BF) for _ in range(3))
    w = (torch.randn(B, T, C, generator=g) * 0.7 - 0.6).to(BF)
    u = (torch.randn(H, N, generator=g) * 0.3).to(BF)
    gy = torch.randn(B, T, C, generator=g).to(BF)
    assert lib.rwkv_wkv6f_saved_bytes(B, T, C, H) == 0
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy)
    d = [x.to(DEV) for x in (r, k, v, w, u, gy)]
    y = garbage((B, T, C), BF)
    call("rwkv_wkv6f_forward", DEV, B, T, C, H, *d[:5], None, y, None, 0, 0)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu = garbage((H, N), BF)
    n = lib.rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv6f_backward_saved", DEV, B, T, C, H, *d[:5], None, d[5], gr, gk, gv, gw, gu, None, None, 0, ws, n, 0)
    torch.cuda.synchronize()
    for name, a, e, got in zip(NAMES, ref, emu, [y, gr, gk, gv, gw, gu]):
        assert_no_worse(name, a, e, got)
    # head size 64 with the sequential sweeps: the states are not written and not read
    B, T, H = 1, 70, 2
    C = H * 64
    r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=318, state=True)
    ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
    got, _ = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy, flags=options.FLAG_SWEEPS, saved_fill=0x7f)
    for name, a, e, g in zip(NAMES, ref, emu, got):
        assert_no_worse("sweeps " + name, a, e, g)


def test_one_sweep_rejects_bad_arguments(lib):
    B, T, H = 1, 64, 1
    C = 64
    r, k, v, w, u, gy, _ = (x.to(DEV) if x is not None else None for x in synth.wkv6_inputs(B, T, C, H, seed=1))
    y = torch.empty((B, T, C), device=DEV, dtype=BF)
    nsv = lib.rwkv_wkv6f_saved_bytes(B, T, C, H)
    assert nsv == 64 * 64 * 3 + 32                              # one segment of 64 tokens (24 bits a value), eight flag words
    saved = torch.empty(nsv, device=DEV, dtype=torch.uint8)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    assert lib.rwkv_wkv6f_forward(st, B, T, C, H, p(r), p(k), p(v), p(w), p(u), None, p(y), p(saved), nsv - 1, 0) == -4   # too small
    assert lib.rwkv_wkv6f_forward(st, B, 0, C, H, p(r), p(k), p(v), p(w), p(u), None, p(y), p(saved), nsv, 0) == -1       # bad shape
    g4 = [torch.empty((B, T, C), device=DEV, dtype=BF) for _ in range(4)]
    gu = torch.empty((H, 64), device=DEV, dtype=BF)
    n = lib.rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)
    args = [st, B, T, C, H, p(r), p(k), p(v), p(w), p(u), None, p(gy)] + [p(x) for x in g4] + [p(gu), None, p(saved), nsv, p(ws)]
    assert lib.rwkv_wkv6f_backward_saved(*args, n - 1, 0) == -4                                                          # workspace too small
    args[10] = p(torch.empty((B, H, 64, 64), device=DEV, dtype=BF))                                                      # a state without its gradient
    assert lib.rwkv_wkv6f_backward_saved(*args, n, 0) == -2
    torch.cuda.synchronize()


@pytest.mark.parametrize("B,T,H,fast", [(2, 50, 2, False), (1, 700, 3, False), (3, 64, 1, False), (1, 4096, 2, False), (2, 100, 3, True), (1, 300, 2, True)])
def test_wkv5_on_the_one_sweep_pair(lib, B, T, H, fast):
    """wkv5 at head size 64 through rwkv_wkv5s_forward / rwkv_wkv5s_backward: the raw decay of a channel stands in for every
    token's, gw is summed over the tokens inside the kernel and over the batch after it ((1, 700, 3), (1, 4096, 2) and
    (1, 300, 2) run as blocks with a scan).  fast: one channel of head 1 decays by more than e^-60 over 16 tokens, so the
    kernels hand that head (its per-batch gw, gu rows included) to the two-sweep kernels."""
    print(f"\nwkv5 one sweep B={B} T={T} H={H} fast={fast}", flush=True)
    C = H * 64
    r, k, v, w, u, gy = synth.wkv5_inputs(B, T, C, H, seed=340 + T)
    if fast:
        w = w.float()
        w.view(-1)[64 + 17] = 1.5                                # exp(1.5) = 4.48 per token: e^-72 over 16 tokens
        w = w.to(BF)
    ref = O.wkv5_grads(B, T, C, H, r, k, v, w, u, gy) if T < 2000 else None
    if ref is None:
        ref = list(O.wkv_grads_by_hand(B, T, C, H, r, k, v, w.reshape(1, 1, C).expand(B, T, C), u, gy, None, torch.float64))[:6]
        ref[4] = ref[4].sum((0, 1)).reshape(H, 64)
        ref[5] = ref[5].sum(0)
    emu = O.emulate_wkv5_bf16(B, T, C, H, r, k, v, w, u, gy, hand=T >= 2000)
    d = [x.to(DEV) for x in (r, k, v, w, u, gy)]
    y = garbage((B, T, C), BF)
    decay = torch.full((2 * C,), float("nan"), device=DEV, dtype=torch.float32)
    nsv = lib.rwkv_wkv5s_saved_bytes(B, T, C, H)
    saved = torch.empty(nsv, device=DEV, dtype=torch.uint8).fill_(0x7f)
    call("rwkv_wkv5s_forward", DEV, B, T, C, H, *d[:5], y, decay, saved, nsv, 0)
    # the forward leaves the wrapper-side transform of the decay (wkv5_bf16/run.py:63-64) for the backward
    ew = -torch.exp(w.double().reshape(-1))
    assert torch.allclose(decay[C:].cpu().double(), ew, rtol=2e-6, atol=0) and torch.allclose(decay[:C].cpu().double(), torch.exp(ew), rtol=2e-6, atol=0)
    gr, gk, gv = (garbage((B, T, C), BF) for _ in range(3))
    gw, gu = garbage((H, 64), BF), garbage((H, 64), BF)
    n = lib.rwkv_wkv5s_backward_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8).fill_(0x7f)
    call("rwkv_wkv5s_backward", DEV, B, T, C, H, d[0], d[1], d[2], d[3], decay, d[4], d[5], gr, gk, gv, gw, gu, saved, nsv, ws, n, 0)
    torch.cuda.synchronize()
    # the words in which the kernels flag the (batch, head) pairs they hand back, after the two-sweep kernels' own workspace
    off = (lib.rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H) + 15) // 16 * 16
    flags = ws[off:off + B * H * 8 * 4].view(torch.int32).view(B * H, 8)
    assert int((flags != 0).any(1).sum()) == (B if fast else 0)
    for name, a, e, g in zip(["y", "gr", "gk", "gv", "gw", "gu"], ref, emu, [y, gr, gk, gv, gw, gu]):
        assert torch.isfinite(g.float()).all(), name
        assert_no_worse("wkv5 " + name, a, e, g)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    assert lib.rwkv_wkv5s_forward(st, B, T, C, H, p(d[0]), p(d[1]), p(d[2]), p(d[3]), p(d[4]), p(y), p(decay), p(saved), nsv - 1, 0) == -4
    torch.cuda.synchronize()


def test_random_shapes_states_and_decays(lib):
    """Twenty seeded random cases of the wkv6 pair: batch 1..3, heads 1..3, T up to 900 (cut chunks, odd chunk counts, one to
    seven blocks, a cut last block), with or without a state, a third of them with a stretch of strong decays somewhere
    (inside a block, across a block boundary, in the cut chunk)."""
    g = torch.Generator().manual_seed(2024)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    for case in range(20):
        B, H, T = ri(1, 3), ri(1, 3), ri(1, 900)
        state = bool(ri(0, 1))
        C = H * 64
        r, k, v, w, u, gy, s0 = synth.wkv6_inputs(B, T, C, H, seed=400 + case, state=state)
        strong = case % 3 == 0 and T > 40
        if strong:
            t0 = ri(0, T - 20)
            h = ri(0, H - 1)
            w = w.float()
            w[ri(0, B - 1), t0:t0 + 20, 64 * h:64 * h + ri(1, 64)] = 2.5
            w = w.to(BF)
        print(f"\ncase {case}: B={B} T={T} H={H} state={state} strong={strong}", flush=True)
        ref = O.wkv6_grads(B, T, C, H, r, k, v, w, u, gy, s0=s0)
        emu = O.emulate_wkv6_bf16(B, T, C, H, r, k, v, w, u, gy, s0=s0)
        got, handed_back = run_pair(lib, B, T, H, r, k, v, w, u, s0, gy, saved_fill=0x7f)
        assert handed_back == (1 if strong else 0), (case, handed_back)
        for name, a, e, x in zip(NAMES, ref, emu, got):
            assert torch.isfinite(x.float()).all(), (case, name)
            assert_no_worse(f"case {case} {name}", a, e, x)


def test_the_pair_replays_from_a_hip_graph(lib):
    """Forward and backward of a step captured once and replayed: no entry point allocates, synchronises or records a
    memset (the flag words of the block form are cleared by a fill kernel), so replays give the eager results every time,
    also with the program's own work and synchronisations between them.  A shape that runs as blocks with a scan."""
    B, T, H = 1, 512, 4
    C = H * 64
    r, k, v, w, u, gy, s0 = (x.to(DEV) if x is not None else None for x in synth.wkv6_inputs(B, T, C, H, seed=350, state=True))
    y = garbage((B, T, C), BF)
    gr, gk, gv, gw = (garbage((B, T, C), BF) for _ in range(4))
    gu, gs = garbage((H, 64), BF), garbage((B, H, 64, 64), BF)
    nsv = lib.rwkv_wkv6f_saved_bytes(B, T, C, H)
    saved = torch.empty(nsv, device=DEV, dtype=torch.uint8)
    n = lib.rwkv_wkv6f_backward_saved_workspace_bytes(B, T, C, H)
    ws = torch.empty(n, device=DEV, dtype=torch.uint8)

    def step():
        call("rwkv_wkv6f_forward", DEV, B, T, C, H, r, k, v, w, u, s0, y, saved, nsv, 0)
        call("rwkv_wkv6f_backward_saved", DEV, B, T, C, H, r, k, v, w, u, s0, gy, gr, gk, gv, gw, gu, gs, saved, nsv, ws, n, 0)

    step()
    torch.cuda.synchronize()
    eager = [x.clone() for x in (y, gr, gk, gv, gw, gu, gs)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        for x in (y, gr, gk, gv, gw, gu, gs):
            x.fill_(float("nan"))
        saved.fill_(0x7f)
        ws.fill_(0x7f)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(NAMES, eager, (y, gr, gk, gv, gw, gu, gs)):
            assert torch.equal(a, b), (rep, name)
