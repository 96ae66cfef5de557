"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
and rejects bad arguments with status codes before anything reaches the GPU."""
import ctypes
import os
import re

import pytest
import torch

from rwkv_cuda_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "rwkv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rwkv7?_[a-z0-9_]+)\s*\(", text)))


def test_header_and_bindings_agree(lib):
    names = _declared_symbols()
    assert len(names) == len(_lib.SIGNATURES) and len(names) >= 48
    assert sorted(_lib.SIGNATURES) == names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in rwkv_hip.h but not exported"


def test_status_text(lib):
    assert lib.rwkv_abi_version() == 4
    assert lib.rwkv_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -99):
        assert len(lib.rwkv_strerror(code)) > 0


def test_bad_arguments_are_rejected_without_a_launch(lib):
    p = 0x1000  # never dereferenced: every call below fails validation first
    # shapes
    assert lib.rwkv_wkv6_forward(None, 0, 8, 64, 1, p, p, p, p, p, p) == -1
    assert lib.rwkv_wkv6_forward(None, 1, 8, 97, 2, p, p, p, p, p, p) == -1          # C not a multiple of H
    assert lib.rwkv_wkv5_forward(None, 1, 8, 129, 1, p, p, p, p, p, p) == -1         # head size above 128
    assert lib.rwkv_wkv5f32_forward(None, 1, 8, 258, 2, p, p, p, p, p, p) == -1
    assert lib.rwkv7_statepassing_forward(None, 1, 24, 1, *([p] * 11)) == -1         # T % 16
    assert lib.rwkv7_state_forward(None, 1, 24, 1, *([p] * 10)) == -1
    assert lib.rwkv7_forward(None, 1, 16, 1, *([p] * 8), None) == -2
    assert lib.rwkv7_backward(None, 0, 16, 1, *([p] * 15)) == -1
    assert lib.rwkv7_statepassing_forward_f32(None, 1, 24, 1, *([p] * 11)) == -1
    assert lib.rwkv7_state_backward_f32(None, 1, 16, 1, *([p] * 15), p + 8) == -3
    assert lib.rwkv7_backward_f32(None, 1, 16, 1, *([p] * 14), None) == -2
    assert lib.rwkv_timex_forward(None, p, p, p, 0.0, 1, 1, 6) == -1                 # T % 4
    assert lib.rwkv_timex_backward_sum(None, p, p, p, p, p, 2, 1, 48) == -1           # T % 32
    assert lib.rwkv_timex_backward_sum(None, p, p, p, p, p, 2, 1, 2048) == -1         # T > 1024
    assert lib.rwkv_timex_backward_sum(None, p, p, p, None, p, 2, 1, 64) == -2
    assert lib.rwkv_wkv4_forward(None, 1, 0, 4, p, p, p, p, p) == -1
    # null / misaligned pointers
    assert lib.rwkv_wkv6_forward(None, 1, 8, 64, 1, p, p, None, p, p, p) == -2
    assert lib.rwkv_wkv6state_forward(None, 1, 8, 64, 1, p, p, p, p, p, p + 2, p) == -3
    assert lib.rwkv_wkv4_forward(None, 1, 4, 4, p, p, p, p, None) == -2
    # workspace
    need = lib.rwkv_wkv6state_backward_workspace_bytes(2, 8, 128, 2)
    assert need == 2 * 8 * 128 * 4 + 2 * 2 * 1 * 64 * 64 * 4      # r*dr' and one stored state per (b,h) for the single chunk
    assert lib.rwkv_wkv6state_backward(None, 2, 8, 128, 2, *([p] * 13), None, 0) == -4
    assert lib.rwkv_wkv6state_backward(None, 2, 8, 128, 2, *([p] * 13), p, need - 1) == -4
    assert lib.rwkv_wkv6_backward_workspace_bytes(1, 1, 129, 1) == 0
    assert lib.rwkv_wkv5f32_backward(None, 2, 8, 128, 2, *([p] * 11), None) == -2
    assert lib.rwkv_wkv5a_forward(None, 1, 8, 130, 1, *([p] * 8)) == -1
    assert lib.rwkv_wkv5a_backward(None, 2, 8, 128, 2, *([p] * 16), p + 4) == -3
    assert lib.rwkv_wkv4_backward(None, 1, 4, 4, *([p] * 9), None, 0) == -4
    # the entry point that allocates nothing rejects sizes beyond its built-in scratch before it touches the device
    assert lib.rwkv_wkv4_backward_noalloc(None, 2, 40000, 64, *([p] * 9)) == -4      # T > 32768: the kernel that uses the scratch
    # per-call flags: same validation as the plain entry points
    assert lib.rwkv_wkv6state_backward_ex(None, 2, 8, 128, 2, *([p] * 13), None, 0, 0x100) == -4
    assert lib.rwkv_wkv6raw_forward_ex(None, 1, 8, 130, 1, p, p, p, p, p, p, 0) == -1
    with pytest.raises(_lib.RwkvHipError):
        _lib.check(-1)


def test_ops_refuse_cpu_tensors():
    from rwkv_cuda_amd import wkv6_state, wkv, rwkv7_fast_fused
    bf = torch.bfloat16
    B, T, H = 1, 16, 1
    C = 64
    x = torch.zeros(B, T, C, dtype=bf)
    with pytest.raises(AssertionError):
        wkv6_state.RUN_CUDA(B, T, C, H, x, x, x, x, torch.zeros(H, 64, dtype=bf), torch.zeros(B, H, 64, 64, dtype=bf))
    with pytest.raises(AssertionError):
        wkv.WKV.apply(B, T, C, torch.zeros(C), torch.zeros(C), x.float(), x.float())
    x4 = x.view(B, T, H, 64)
    with pytest.raises(AssertionError):
        rwkv7_fast_fused.RWKV7_STATE_PASSING_CLAMPW_CUDA_OP.apply(torch.zeros(B, H, 64, 64), x4, x4, x4, x4, x4, x4)


def test_reference_style_extension_loads_and_registers_its_ops(lib):
    """csrc/binding.cpp: one pybind submodule per reference extension and the TORCH_LIBRARY names of the *_op.cpp files."""
    from rwkv_cuda_amd import binding
    ext = binding.load()
    for name in ("wkv", "timex", "wkv5", "wkv5a", "wkv6", "wkv6state", "rwkv7_clampw", "rwkv7_state_clampw", "rwkv7_statepassing_clampw"):
        sub = getattr(ext, name)
        assert callable(sub.forward) and callable(sub.backward)
    for ns in ("wkv", "timex", "wkv5", "wkv5a", "wkv6", "wkv6b", "rwkv7_clampw", "rwkv7_state_clampw", "rwkv7_statepassing_clampw"):
        assert getattr(torch.ops, ns).forward is not None and getattr(torch.ops, ns).backward is not None
    c = torch.zeros(4)
    with pytest.raises(RuntimeError, match="HIP device"):
        ext.wkv.forward(1, 1, 4, c, c, c, c, c)
