"""Per-call kernel options for the wkv5 / wkv6 / wkv6_state wrappers.

The C ABI takes them as the `flags` word of its *_ex entry points; nothing is process-wide there.  On the Python side a
`with algorithm("sweeps"):` block selects the sequential kernels for every forward issued inside it by this thread; the
choice is stored on the autograd context, so the matching backward (which the autograd engine may run on another
thread, after the block has ended) uses the same kernels.
"""
import contextlib
import threading

PASS_GR, PASS_GV, PASS_GK, PASS_ALL = 1, 2, 4, 7
FLAG_SWEEPS = 0x100
FLAG_WHOLE = 0x200      # wkv6 one-sweep pair: one workgroup per sequence also for few sequences (no blocks, no scan)

_tls = threading.local()


def current_flags():
    return getattr(_tls, "flags", 0)


@contextlib.contextmanager
def algorithm(name):
    """name: "chunked" (default kernels) or "sweeps" (sequential fp32 recurrence)."""
    if name not in ("chunked", "sweeps"):
        raise ValueError(name)
    old = current_flags()
    _tls.flags = FLAG_SWEEPS if name == "sweeps" else 0
    try:
        yield
    finally:
        _tls.flags = old
