"""GPU: the entry point that allocates nothing (rwkv_wkv4_backward_noalloc) against rwkv_wkv4_backward, through the
C ABI, on two calls in a row, the second with a smaller input (the shared scratch keeps the first call's contents)."""
import pytest
import torch

from rwkv_cuda_amd import synth
from rwkv_cuda_amd._call import call
from _gpu_util import DEV

pytestmark = pytest.mark.gpu


def _both(lib, B, T, C, seed):
    w_raw, u, k, v, gy = (x.to(DEV) for x in synth.wkv4_inputs(B, T, C, seed=seed))
    w = -torch.exp(w_raw)
    out = []
    for noalloc in (False, True):
        gw = torch.zeros(B, C, device=DEV, dtype=torch.float32)
        gu = torch.zeros(B, C, device=DEV, dtype=torch.float32)
        gk = torch.full((B, T, C), 7.0, device=DEV, dtype=torch.float32)
        gv = torch.full((B, T, C), -7.0, device=DEV, dtype=torch.float32)
        if noalloc:
            call("rwkv_wkv4_backward_noalloc", gy.device, B, T, C, w, u, k, v, gy, gw, gu, gk, gv)
        else:
            n = lib.rwkv_wkv4_backward_workspace_bytes(B, T, C)
            ws = torch.empty(n, device=DEV, dtype=torch.uint8)
            call("rwkv_wkv4_backward", gy.device, B, T, C, w, u, k, v, gy, gw, gu, gk, gv, ws, n)
        torch.cuda.synchronize()
        out.append((gw, gu, gk, gv))
    return out


def test_noalloc_equals_workspace_entry_point_twice(lib):
    assert lib.rwkv_wkv4_backward_noalloc_max_elems() == 1 << 21
    # only beyond T = 32768 does the backward park its ascending sweep's results in the scratch (shorter sequences keep them
    # in registers); every call is smaller than the one before, the last two do not touch the scratch
    for B, T, C, seed in ((1, 40000, 52, 5), (1, 33000, 16, 6), (4, 512, 768, 7), (2, 37, 80, 8)):
        print(f"\nwkv4 noalloc B={B} T={T} C={C}", flush=True)
        ref, got = _both(lib, B, T, C, seed)
        for name, a, g in zip(("gw", "gu", "gk", "gv"), ref, got):
            assert torch.equal(a, g), name                         # same kernels, same order of operations: bit-identical


def test_noalloc_limit_applies_only_where_the_scratch_is_used(lib):
    """Sequences up to 32768 tokens run on kernels that keep their intermediates on the chip: no scratch, no limit (the
    reference's own shapes B32 T768 C768 and B4 T1024 C768 are above 2^21 elements).  Beyond that length the kernel parks
    B T C floats in the scratch, and a shape that does not fit is refused."""
    for B, T, C, seed in ((32, 768, 768, 9), (4, 1024, 768, 10)):
        assert B * T * C > lib.rwkv_wkv4_backward_noalloc_max_elems()
        print(f"\nwkv4 noalloc, no scratch needed: B={B} T={T} C={C}", flush=True)
        ref, got = _both(lib, B, T, C, seed)
        for name, a, g in zip(("gw", "gu", "gk", "gv"), ref, got):
            assert torch.equal(a, g), name
    B, T, C = 2, 40000, 64                                         # 5 120 000 elements > 2 097 152, and T > 32768
    z = torch.zeros(16, device=DEV, dtype=torch.float32)
    status = lib.rwkv_wkv4_backward_noalloc(None, B, T, C, *([z.data_ptr()] * 9))
    assert status == -4
