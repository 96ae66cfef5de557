"""Build and load librwkv_hip.so (the C ABI declared in include/rwkv_hip.h) through ctypes.

`build()` always compiles (hipcc cross-compiles gfx950 without a GPU); `load()` uses the
library that is already built and only builds when there is none.  There is no CPU or
PyTorch fallback: if the library cannot be loaded the import of an op fails loudly.
"""

import ctypes
import hashlib
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
_CSRC = os.path.join(_HERE, "csrc")
_INCLUDE = os.path.join(_ROOT, "include")
LIB_PATH = os.path.join(_HERE, "librwkv_hip.so")
HASH_PATH = LIB_PATH + ".srchash"        # digest of the sources the library was built from (content, not mtime)

SOURCES = ["abi.hip", "wkv56.hip", "wkv6_fwd.hip", "wkv6_bwd_a.hip", "wkv6_bwd_b.hip", "wkv6_fwd_f.hip", "wkv6_bwd_f.hip", "wkv4.hip", "timex.hip", "rwkv7.hip", "rwkv7_chunk.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU ops stay off on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # per-kernel register / scratch report on stderr, parsed by build()
    "-Rpass-analysis=kernel-resource-usage",
]

# The prep waves of these kernels load through inline asm and wait with a hand-counted vmcnt, so the compiler does not
# know when such a register is valid: a spill of one of them (they have the longest live ranges) would save garbage.
# The backward sweep B keeps one index of its state waves' epilogue in scratch, outside the loops (three values in the
# wkv5 instantiation, ILi0E, one of them reloaded once per chunk by a state wave); anything beyond these counts fails the
# build.
# The row-per-thread kernels for other head sizes (wkv_rows) keep a whole state row in registers; an instantiation that
# no longer fits gave wrong results on the GPU (fp32 decay-gradient sweep at 128), so none may spill.
# The wkv4 kernels that hold a segment's inputs in registers exist to avoid memory round trips: a spill defeats them.
# The depthwise_conv1d matrix-core kernels hold the next unit's rows in registers across their product loops, which run at
# the register limit: a spill there is scratch traffic in the innermost loop.
# The one-sweep kernels let the compiler count their waits: a spill inside their loops would put scratch traffic between a
# prefetch and its use (and a forward variant that spilled eleven registers gave wrong results): none may spill.
SPILL_LIMIT = {"wkv6_bwd_fused": 0, "wkv6_fwd_fused": 0, "wkv6_fwd_ws": 0, "wkv6_bwd_a_ws": 0, "wkv6_bwd_b_wsILi0E": 3, "wkv6_bwd_b_wsILi1E": 1, "wkv6_bwd_b_wsILi2E": 1,
               "wkv_rows": 0, "wkv4_fwd_reg": 0, "wkv4_bwd_reg": 0, "timex_conv_h2": 0, "timex_gw_sum_h2": 0}

_lib = None


def source_hash():
    h = hashlib.sha256()
    # the kernel sources and their headers; csrc/binding.cpp is the torch-side shim, built separately (binding.py)
    files = sorted(f for f in os.listdir(_CSRC) if f.endswith((".hip", ".h")))
    for path in [os.path.join(_CSRC, f) for f in files] + [os.path.join(_INCLUDE, "rwkv_hip.h")]:
        with open(path, "rb") as f:
            h.update(os.path.basename(path).encode() + b"\0" + f.read())
    return h.hexdigest()


def _compile_one(args):
    hipcc, src, obj = args
    cmd = [hipcc] + HIPCC_FLAGS + ["-c", "-I", _INCLUDE, "-I", _CSRC, "-o", obj, src]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return " ".join(cmd), res.returncode, res.stdout


def build(verbose=False):
    """Compile every HIP source (one hipcc process per file, side by side) and link them into one shared library, in-tree."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(_HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = [(hipcc, os.path.join(_CSRC, s), os.path.join(objdir, s + ".o")) for s in SOURCES]
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        results = list(pool.map(_compile_one, jobs))
    lines = []
    for cmd, rc, text in results:
        if verbose:
            print(cmd, flush=True)
        if rc != 0:
            raise RuntimeError("hipcc failed:\n" + "\n".join(l for l in text.splitlines() if "is not a recognized feature" not in l and "kernel-resource-usage" not in l))
        lines += text.splitlines()
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + [j[2] for j in jobs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    out = "\n".join(l for l in lines if "is not a recognized feature" not in l and "kernel-resource-usage" not in l)
    kernel = None
    report = []
    for l in lines:
        m = re.search(r"remark: Function Name: (\S+)", l)
        if m:
            kernel = m.group(1)
        m = re.search(r"remark:\s+VGPRs Spill: (\d+)", l)
        if m and kernel:
            for name, limit in SPILL_LIMIT.items():
                if name in kernel and int(m.group(1)) > limit:
                    os.remove(LIB_PATH)
                    raise RuntimeError(f"{kernel}: {m.group(1)} spilled VGPRs (limit {limit}); see SPILL_LIMIT")
    if verbose and out.strip():
        print(out, flush=True)
    with open(HASH_PATH, "w") as f:
        f.write(source_hash() + "\n")
    return LIB_PATH


_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_Z = ctypes.c_size_t
_U = ctypes.c_uint

# name -> (restype, argtypes): one row per symbol in include/rwkv_hip.h
SIGNATURES = {
    "rwkv_strerror": (ctypes.c_char_p, [_I]),
    "rwkv_last_hip_error": (_I, []),
    "rwkv_abi_version": (_I, []),
    "rwkv_hbm_probe": (_I, [_P, _I, _P, _P, _Z]),
    "rwkv_wkv4_forward": (_I, [_P, _I, _I, _I] + [_P] * 5),
    "rwkv_wkv4_backward_workspace_bytes": (_Z, [_I, _I, _I]),
    "rwkv_wkv4_backward": (_I, [_P, _I, _I, _I] + [_P] * 9 + [_P, _Z]),
    "rwkv_wkv4raw_forward": (_I, [_P, _I, _I, _I] + [_P] * 5),
    "rwkv_wkv4raw_backward_workspace_bytes": (_Z, [_I, _I, _I]),
    "rwkv_wkv4raw_backward": (_I, [_P, _I, _I, _I] + [_P] * 9 + [_P, _Z]),
    "rwkv_wkv4_backward_noalloc_max_elems": (_Z, []),
    "rwkv_wkv4_backward_noalloc": (_I, [_P, _I, _I, _I] + [_P] * 9),
    "rwkv_timex_forward": (_I, [_P, _P, _P, _P, _F, _I, _I, _I]),
    "rwkv_timex_backward": (_I, [_P] * 6 + [_I, _I, _I]),
    "rwkv_timex_backward_sum": (_I, [_P] * 6 + [_I, _I, _I]),
    "rwkv_wkv5_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 6),
    "rwkv_wkv5_forward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 6 + [_U]),
    "rwkv_wkv5_forward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv5_forward_ws": (_I, [_P, _I, _I, _I, _I] + [_P] * 6 + [_P, _Z, _U]),
    "rwkv_wkv5raw_forward_ws": (_I, [_P, _I, _I, _I, _I] + [_P] * 7 + [_P, _Z, _U]),
    "rwkv_wkv5_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv5_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 12 + [_P, _Z]),
    "rwkv_wkv5_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 12 + [_P, _Z] + [_U]),
    "rwkv_wkv5raw_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 7 + [_U]),
    "rwkv_wkv5raw_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv5raw_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 11 + [_P, _Z, _U]),
    "rwkv_wkv6f_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv6f_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 13 + [_P, _Z, _U]),
    "rwkv_wkv6f_saved_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv6f_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 7 + [_P, _Z, _U]),
    "rwkv_wkv6f_backward_saved_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv6f_backward_saved": (_I, [_P, _I, _I, _I, _I] + [_P] * 13 + [_P, _Z, _P, _Z, _U]),
    "rwkv_wkv5s_saved_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv5s_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 7 + [_P, _Z, _U]),
    "rwkv_wkv5s_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv5s_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 12 + [_P, _Z, _P, _Z, _U]),
    "rwkv_wkv5f32_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 6),
    "rwkv_wkv5f32_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 12),
    "rwkv_wkv5f32_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 12 + [_U]),
    "rwkv_wkv5a_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 8),
    "rwkv_wkv5a_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 17),
    "rwkv_wkv5a_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 17 + [_U]),
    "rwkv_wkv6_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 6),
    "rwkv_wkv6_forward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 6 + [_U]),
    "rwkv_wkv6_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv6_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 11 + [_P, _Z]),
    "rwkv_wkv6_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 11 + [_P, _Z] + [_U]),
    "rwkv_wkv6raw_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 6),
    "rwkv_wkv6raw_forward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 6 + [_U]),
    "rwkv_wkv6raw_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 11 + [_P, _Z]),
    "rwkv_wkv6raw_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 11 + [_P, _Z] + [_U]),
    "rwkv_wkv6state_forward": (_I, [_P, _I, _I, _I, _I] + [_P] * 7),
    "rwkv_wkv6state_forward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 7 + [_U]),
    "rwkv_wkv6state_backward_workspace_bytes": (_Z, [_I, _I, _I, _I]),
    "rwkv_wkv6state_backward": (_I, [_P, _I, _I, _I, _I] + [_P] * 13 + [_P, _Z]),
    "rwkv_wkv6state_backward_ex": (_I, [_P, _I, _I, _I, _I] + [_P] * 13 + [_P, _Z] + [_U]),
    "rwkv7_statepassing_forward": (_I, [_P, _I, _I, _I] + [_P] * 11),
    "rwkv7_statepassing_backward": (_I, [_P, _I, _I, _I] + [_P] * 17),
    "rwkv7_statepassing_forward_ex": (_I, [_P, _I, _I, _I] + [_P] * 11 + [_U]),
    "rwkv7_statepassing_backward_ex": (_I, [_P, _I, _I, _I] + [_P] * 17 + [_U]),
    "rwkv7_state_forward": (_I, [_P, _I, _I, _I] + [_P] * 10),
    "rwkv7_state_backward": (_I, [_P, _I, _I, _I] + [_P] * 16),
    "rwkv7_forward": (_I, [_P, _I, _I, _I] + [_P] * 9),
    "rwkv7_backward": (_I, [_P, _I, _I, _I] + [_P] * 15),
    "rwkv7_statepassing_forward_f32": (_I, [_P, _I, _I, _I] + [_P] * 11),
    "rwkv7_statepassing_backward_f32": (_I, [_P, _I, _I, _I] + [_P] * 17),
    "rwkv7_state_forward_f32": (_I, [_P, _I, _I, _I] + [_P] * 10),
    "rwkv7_state_backward_f32": (_I, [_P, _I, _I, _I] + [_P] * 16),
    "rwkv7_forward_f32": (_I, [_P, _I, _I, _I] + [_P] * 9),
    "rwkv7_backward_f32": (_I, [_P, _I, _I, _I] + [_P] * 15),
}


def load():
    """Return the ctypes handle of the built library (building it once if it is absent)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    elif os.path.exists(HASH_PATH):
        # a library built from other sources than the ones beside it would silently run yesterday's kernels
        with open(HASH_PATH) as f:
            if f.read().strip() != source_hash():
                raise RuntimeError(f"{LIB_PATH} was built from different sources: rebuild it (python __graft_entry__.py)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)        # AttributeError here = header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class RwkvHipError(RuntimeError):
    pass


def check(status):
    """Raise on a non-zero status from the C ABI."""
    if status != 0:
        lib = load()
        msg = lib.rwkv_strerror(status).decode()
        if status == -5:
            msg += f" (hipError {lib.rwkv_last_hip_error()})"
        raise RwkvHipError(f"librwkv_hip: status {status}: {msg}")
