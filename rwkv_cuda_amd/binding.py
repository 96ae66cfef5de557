"""The reference's own extension interface on top of librwkv_hip.so.

BlinkDL/RWKV-CUDA binds every kernel pair through a small C++ shim (`*_op.cpp`) that
`torch.utils.cpp_extension.load` compiles into a pybind module with `forward` / `backward` and, for rwkv7, into
`torch.ops.<lib>.forward/backward` only (wkv6_state/run.py:77, rwkv7_cuda_benchmark_state_passing.py:74,87,98).
csrc/binding.cpp is that shim for all nine extensions at once, calling the C ABI on torch's current HIP stream.

    ext = binding.load()                       # builds nothing if rwkv_hip_binding.so is there
    ext.wkv6state.forward(B, T, C, H, r, k, v, w, u, s, y)            # = wkv6state_cuda.forward(...)
    torch.ops.rwkv7_statepassing_clampw.forward(s0, r, w, k, v, a, b, y, sT, s, sa)

build() compiles with torch.utils.cpp_extension (the same route as the reference) and keeps the result in-tree.
"""
import importlib.machinery
import importlib.util
import os
import shutil
import subprocess
import sys

from . import _lib

NAME = "rwkv_hip_binding"
_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, NAME + ".so")
_BUILD_DIR = os.path.join(_HERE, "build", NAME)

_ext = None


def _compile(verbose):
    import torch
    from torch.utils import cpp_extension
    os.makedirs(_BUILD_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_HOME", "/opt/rocm")
    cpp_extension.load(
        name=NAME,
        sources=[os.path.join(_HERE, "csrc", "binding.cpp")],
        extra_include_paths=[os.path.join(os.path.dirname(_HERE), "include"), os.path.join(rocm, "include")],
        extra_cflags=["-O2", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1"],
        # the dollar signs survive ninja and the shell as a literal $ORIGIN: the extension finds librwkv_hip.so beside itself
        extra_ldflags=[f"-L{_HERE}", "-lrwkv_hip", "-Wl,-rpath,\\$$ORIGIN:\\$$ORIGIN/../..", f"-L{torch_lib}", "-lc10_hip", "-ltorch_hip",
                       f"-L{os.path.join(rocm, 'lib')}", "-lamdhip64"],
        build_directory=_BUILD_DIR,
        is_python_module=False,
        verbose=verbose,
    )


def build(verbose=False):
    """Compile csrc/binding.cpp against the built librwkv_hip.so with torch.utils.cpp_extension and keep the result
    in-tree.  The compile runs in a child process: cpp_extension.load also loads what it built, and a TORCH_LIBRARY
    namespace can be registered only once per process, so the caller's process must load the in-tree copy alone."""
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    code = f"import sys; sys.path.insert(0, {os.path.dirname(_HERE)!r}); from rwkv_cuda_amd import binding; binding._compile({bool(verbose)})"
    res = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout, flush=True)
    if res.returncode != 0:
        raise RuntimeError("building csrc/binding.cpp failed")
    shutil.copyfile(os.path.join(_BUILD_DIR, NAME + ".so"), SO_PATH)
    return SO_PATH


def load():
    """Import the in-tree extension (registers the torch.ops libraries as a side effect)."""
    global _ext
    if _ext is not None:
        return _ext
    if NAME in sys.modules:
        _ext = sys.modules[NAME]
        return _ext
    if not os.path.exists(SO_PATH):
        build()
    _lib.load()                      # fail early, with a clear message, if the kernel library is missing or stale
    import torch                     # noqa: F401  (libtorch must be loaded before the extension)
    loader = importlib.machinery.ExtensionFileLoader(NAME, SO_PATH)
    spec = importlib.util.spec_from_loader(NAME, loader)
    mod = importlib.util.module_from_spec(spec)
    loader.exec_module(mod)
    # a shim built against another version of the C ABI would resolve its symbols lazily and fail, or misbehave, at call time
    have, want = getattr(mod, "abi_version", None), _lib.load().rwkv_abi_version()
    if have != want:
        raise RuntimeError(f"{SO_PATH} was built against ABI version {have}, librwkv_hip.so is version {want}: "
                           "rebuild it (rwkv_cuda_amd.binding.build())")
    sys.modules[NAME] = mod
    _ext = mod
    return mod
