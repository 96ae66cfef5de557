"""Plumbing shared by the operator wrappers: tensor checks, stream and device handling."""

import torch

from . import _lib


def require(cond, msg):
    # the reference uses bare asserts (e.g. wkv6_state/run.py:84-100); an AssertionError keeps that contract
    if not cond:
        raise AssertionError(msg)


def check_tensors(tensors, dtype, names):
    dev = tensors[0].device
    require(dev.type == "cuda", "tensors must live on a HIP device: there is no CPU path")
    for t, n in zip(tensors, names):
        require(t.dtype == dtype, f"{n}.dtype must be {dtype}, got {t.dtype}")
        require(t.is_contiguous(), f"{n} must be contiguous")
        require(t.device == dev, f"{n} is on {t.device}, expected {dev}")
    return dev


def call(name, dev, *args):
    """Call one C-ABI entry point on torch's current stream of `dev`.  Tensors become raw pointers."""
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        conv = [a.data_ptr() if isinstance(a, torch.Tensor) else a for a in args]
        _lib.check(getattr(lib, name)(stream, *conv))
