"""GPU: the entry points that fold the wrapper-side torch steps into the library (raw decay parameter in, parameter gradients
summed over the batch out) against the reference-signature entry points followed by the same steps in torch.

  rwkv_wkv4raw_*      wkv/run.py:95,110-116        w = -exp(w_raw); zero-filled gw, gu; gw.sum(0), gu.sum(0)
  rwkv_wkv5raw_*      wkv5_bf16/run.py:63-64,86-87 ew = -exp(w.float()), eew = exp(ew); gw.sum(0), gu.sum(0)
  rwkv_wkv6f_backward wkv6/run.py:169, wkv6_state/run.py:123   gu.sum(0)
The big tensors must agree bit for bit (same kernels); the summed parameter gradients to the rounding of one fp32 sum."""
import pytest
import torch

from rwkv_cuda_amd import synth
from rwkv_cuda_amd._call import call
from _gpu_util import DEV, garbage

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.mark.parametrize("B,T,C", [(4, 512, 768), (3, 37, 80)])
def test_wkv4raw_equals_reference_entry_points_plus_torch(lib, B, T, C):
    w_raw, u, k, v, gy = (x.to(DEV) for x in synth.wkv4_inputs(B, T, C, seed=81))
    w = -torch.exp(w_raw)
    y0, gk0, gv0 = (garbage((B, T, C), torch.float32) for _ in range(3))
    gw0, gu0 = torch.zeros(B, C, device=DEV), torch.zeros(B, C, device=DEV)
    n0 = lib.rwkv_wkv4_backward_workspace_bytes(B, T, C)
    ws0 = torch.empty(n0, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv4_forward", w.device, B, T, C, w, u, k, v, y0)
    call("rwkv_wkv4_backward", w.device, B, T, C, w, u, k, v, gy, gw0, gu0, gk0, gv0, ws0, n0)
    y1, gk1, gv1 = (garbage((B, T, C), torch.float32) for _ in range(3))
    gw1, gu1 = garbage((C,), torch.float32), garbage((C,), torch.float32)
    n1 = lib.rwkv_wkv4raw_backward_workspace_bytes(B, T, C)
    assert n1 == n0 + 2 * B * C * 4
    ws1 = torch.empty(n1, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv4raw_forward", w.device, B, T, C, w_raw, u, k, v, y1)
    call("rwkv_wkv4raw_backward", w.device, B, T, C, w_raw, u, k, v, gy, gw1, gu1, gk1, gv1, ws1, n1)
    torch.cuda.synchronize()
    # -exp(w_raw) inside the kernel (expf) and torch's exp may differ in the last bit of w; everything downstream follows
    for name, a, b in (("y", y0, y1), ("gk", gk0, gk1), ("gv", gv0, gv1), ("gw", gw0.sum(0), gw1), ("gu", gu0.sum(0), gu1)):
        err = float((a - b).abs().max()) / float(a.abs().max())
        print(f"  wkv4raw {name}: max difference / peak {err:.2e}", flush=True)
        assert err < 2e-6, (name, err)


def test_wkv5raw_and_wkv6f_equal_reference_entry_points_plus_torch(lib):
    B, T, H = 3, 70, 2
    C = H * 64
    # ---- wkv5
    r, k, v, w, u, gy = (x.to(DEV) for x in synth.wkv5_inputs(B, T, C, H, seed=82))
    ew = (-torch.exp(w.float())).contiguous().view(-1)
    eew = torch.exp(ew).contiguous()
    y0, gr0, gk0, gv0 = (garbage((B, T, C), BF) for _ in range(4))
    gw0, gu0 = garbage((B, C), BF), garbage((B, C), BF)
    n0 = lib.rwkv_wkv5_backward_workspace_bytes(B, T, C, H)
    ws0 = torch.empty(n0, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv5_forward", r.device, B, T, C, H, r, k, v, eew, u, y0)
    call("rwkv_wkv5_backward", r.device, B, T, C, H, r, k, v, eew, ew, u, gy, gr0, gk0, gv0, gw0, gu0, ws0, n0)
    y1, gr1, gk1, gv1 = (garbage((B, T, C), BF) for _ in range(4))
    gw1, gu1 = garbage((H, 64), BF), garbage((H, 64), BF)
    decay = garbage((2 * C,), torch.float32)
    n1 = lib.rwkv_wkv5raw_backward_workspace_bytes(B, T, C, H)
    ws1 = torch.empty(n1, device=DEV, dtype=torch.uint8)
    call("rwkv_wkv5raw_forward", r.device, B, T, C, H, r, k, v, w, u, y1, decay, 0)
    call("rwkv_wkv5raw_backward", r.device, B, T, C, H, r, k, v, decay, u, gy, gr1, gk1, gv1, gw1, gu1, ws1, n1, 0)
    torch.cuda.synchronize()
    assert float((decay[:C] - eew).abs().max()) <= 1.2e-7 * float(eew.abs().max())
    assert float((decay[C:] - ew).abs().max()) <= 2.4e-7 * float(ew.abs().max())
    same_decay = torch.equal(decay[:C], eew) and torch.equal(decay[C:], ew)
    for name, a, b in (("y", y0, y1), ("gr", gr0, gr1), ("gk", gk0, gk1), ("gv", gv0, gv1),
                       ("gw", torch.sum(gw0, 0).view(H, 64), gw1), ("gu", torch.sum(gu0, 0).view(H, 64), gu1)):
        if same_decay:
            assert torch.equal(a, b), name
        else:                                                   # a last-bit difference in the decay: one bf16 unit at most
            assert float((a.float() - b.float()).abs().max()) <= 2.0 ** -7 * float(a.float().abs().max()), name
    # ---- wkv6 without and with state
    r, k, v, w, u, gy, s0 = (x.to(DEV) for x in synth.wkv6_inputs(B, T, C, H, seed=83, state=True))
    n0 = lib.rwkv_wkv6_backward_workspace_bytes(B, T, C, H)
    n1 = lib.rwkv_wkv6f_backward_workspace_bytes(B, T, C, H)
    for state in (None, s0):
        gr0, gk0, gv0, gw0 = (garbage((B, T, C), BF) for _ in range(4))
        gu0, gs0 = garbage((B, C), BF), garbage((B, H, 64, 64), BF)
        ws0 = torch.empty(n0, device=DEV, dtype=torch.uint8)
        if state is None:
            call("rwkv_wkv6raw_backward", r.device, B, T, C, H, r, k, v, w, u, gy, gr0, gk0, gv0, gw0, gu0, ws0, n0)
        else:
            call("rwkv_wkv6state_backward", r.device, B, T, C, H, r, k, v, w, u, state, gy, gr0, gk0, gv0, gw0, gu0, gs0, ws0, n0)
        gr1, gk1, gv1, gw1 = (garbage((B, T, C), BF) for _ in range(4))
        gu1, gs1 = garbage((H, 64), BF), garbage((B, H, 64, 64), BF)
        ws1 = torch.empty(n1, device=DEV, dtype=torch.uint8)
        call("rwkv_wkv6f_backward", r.device, B, T, C, H, r, k, v, w, u, state, gy, gr1, gk1, gv1, gw1, gu1,
             None if state is None else gs1, ws1, n1, 0)
        torch.cuda.synchronize()
        for name, a, b in (("gr", gr0, gr1), ("gk", gk0, gk1), ("gv", gv0, gv1), ("gw", gw0, gw1), ("gu", torch.sum(gu0, 0).view(H, 64), gu1)):
            assert torch.equal(a, b), (name, state is not None)
        if state is not None:
            assert torch.equal(gs0, gs1)
    # a state without its gradient (or the reverse) is refused
    p = r.data_ptr()
    assert lib.rwkv_wkv6f_backward(None, B, T, C, H, p, p, p, p, p, p, p, p, p, p, p, p, None, ws1.data_ptr(), n1, 0) == -2
