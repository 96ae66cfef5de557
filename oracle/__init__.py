"""CPU oracle for the WKV recurrence family and depthwise_conv1d.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only the tests, the smoke check and the cpu_baseline leg of the
benchmark do, and there only as the checker / the timed CPU baseline.

Every function restates, on the CPU with torch tensors, a formula that the
reference repository (BlinkDL/RWKV-CUDA) holds as Python or CUDA text; each
docstring cites the reference file:line it follows.  Nothing is imported from
the reference.  How each restatement is pinned (sum form against recurrent form,
special cases that reduce to library routines, closed forms, brute force on tiny
shapes, fp64 autograd against hand-derived gradients) is stated per module and
exercised by tests/test_oracle_*.py.

Modules
  wkv4     RWKV-4 wkv (fp32)                       wkv/run.py, wkv/cuda/wkv_cuda_v2.cu
  timex    depthwise_conv1d                        depthwise_conv1d/run.py, cuda/timex_cuda_v0.cu
  wkv56    wkv5 / wkv6 / wkv6_state (bf16 I/O)     wkv5/run.py, wkv6/run.py, wkv6_state/run.py (+ kernels)
  wkv5a    wkv5 with two-sided decay/bonus (fp32)   wkv5a/run.py (+ wkv5a_cuda_v1a2.cu)
  rwkv7    rwkv7 clamp-w with state passing        rwkv7_fast_fused/rwkv7_cuda_benchmark_state_passing.py (+ kernel)
  rwkv7_chunked  the same recurrence in chunked (matrix-product) form, forward and backward; pinned against rwkv7
"""

import torch


def err_ratio(x, y):
    """RMS error ratio ||x-y||_rms / ||x||_rms (x is the trusted side).

    Follows get_err_ratio, wkv/run.py:26-29 (identical in every reference driver).
    """
    x = x.double().flatten()
    y = y.double().flatten()
    return ((x - y).square().mean().sqrt() / x.square().mean().sqrt()).item()


def max_rel_to_peak(x, y):
    """max|x-y| / max|x| : the element-wise bound used for the fp32 paths."""
    x = x.double().flatten()
    y = y.double().flatten()
    return ((x - y).abs().max() / x.abs().max()).item()


def bf16_round(x):
    """Round to bfloat16 (round-to-nearest-even) and return in x's dtype."""
    return x.to(torch.bfloat16).to(x.dtype)
