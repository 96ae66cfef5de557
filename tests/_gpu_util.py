"""Helpers for the GPU parity tests."""
import torch

from oracle import err_ratio

DEV = "cuda"

# bf16 paths: the acceptance bar is the error of the reference kernel itself (fp32 math on bf16
# inputs, outputs rounded to bf16) against an fp64 evaluation of the formula; ours may not be
# worse.  Both errors are dominated by the same final rounding, so on large outputs they agree to a
# fraction of a percent; SLACK covers that.  Each error is an rms over the n output elements, i.e. a
# sample estimate with relative deviation ~1/sqrt(2n): for small outputs (the [B,C] parameter
# gradients of wkv5: n = 128 at H = 1) two correct kernels differ by several percent, so three
# standard deviations of the difference, 3/sqrt(n), are allowed on top.  FLOOR covers fp32-exact outputs.
SLACK = 1.05
FLOOR = 3e-7


def assert_no_worse(name, ref64, emu, got):
    if float(ref64.abs().max()) == 0.0:          # e.g. the decay gradient when T == 1
        assert float(got.float().abs().max()) == 0.0, name
        return
    e_hip = err_ratio(ref64, got.detach().double().cpu())
    e_emu = err_ratio(ref64, emu.double())
    print(f"  {name}: hip {e_hip:.3e}  reference-kernel emulation {e_emu:.3e}", flush=True)
    slack = SLACK + 3.0 / ref64.numel() ** 0.5
    assert e_hip <= slack * e_emu + FLOOR, f"{name}: {e_hip:.3e} worse than the reference kernel's {e_emu:.3e}"


def garbage(shape, dtype):
    """Outputs pre-filled with large values: an element the kernel fails to write shows up as a
    huge error (the write-coverage trick of wkv6_state/run.py:102,116-121)."""
    return torch.empty(shape, device=DEV, dtype=torch.float32).uniform_(-100, 100).to(dtype)
