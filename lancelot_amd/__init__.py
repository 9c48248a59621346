"""MI355X-native CKKS engine behind CAHEL's pyCAHEL interface.

    import lancelot_amd            # loads the native module and registers it as `pyCAHEL`
    import pyCAHEL as cahel        # what lancelot-main-GPU/utils/byzantine_fl.py does

The package holds three native pieces, all built in-tree by `python -m lancelot_amd.build`:
  libcahel_hip.so   hand-written HIP kernels for gfx950 behind the C-ABI of include/cahel_hip.h
  pyCAHEL*.so       C++ host layer (context, encoder, keys, evaluator) + pybind11 binding
  capi              ctypes view of the C-ABI for callers that bring their own device buffers
There is no CPU fallback: without the built libraries, or without a GPU, the calls raise.
"""
import importlib
import os
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))


def _load():
    try:
        mod = importlib.import_module(__name__ + ".pyCAHEL")
    except ImportError as exc:  # not built yet
        raise ImportError(
            "lancelot_amd native module is missing; build it with `python -m lancelot_amd.build` "
            "(needs hipcc and g++): %s" % exc) from exc
    sys.modules.setdefault("pyCAHEL", mod)
    return mod


def _building() -> bool:
    """True while the package is imported only to reach its build module (`python -m lancelot_amd.build`, or a
    caller that set LANCELOT_AMD_BUILD=1 around the import): the native module cannot exist yet."""
    argv = list(getattr(sys, "orig_argv", []))
    return os.environ.get("LANCELOT_AMD_BUILD") == "1" or any(
        a == "-m" and b == __name__ + ".build" for a, b in zip(argv, argv[1:]))


if not _building():
    pyCAHEL = _load()
    from . import capi  # noqa: E402,F401
