"""Loader of the fused softmax / rotary kernels.

Keeps the two entry points of GPT-NeoX's ``megatron/fused_kernels/__init__.py``
(``load`` at :35-143, ``load_fused_kernels`` at :167-181). Instead of JIT-building
three pybind11 extensions, ``load`` makes sure ``libneox_hotpath.so`` (hand-written
gfx950 kernels behind a C ABI) is built and importable; the three extension
module names of the reference (``scaled_upper_triang_masked_softmax_cuda``,
``scaled_masked_softmax_cuda``, ``fused_rotary_positional_embedding``) are thin
modules over that library and are registered in ``sys.modules`` here.
"""
import importlib
import os
import sys

from . import _hotpath

_EXTENSION_MODULES = (
    "scaled_upper_triang_masked_softmax_cuda",
    "scaled_masked_softmax_cuda",
    "fused_rotary_positional_embedding",
)

# The extension modules live next to the ``megatron`` package.
_PKG_ROOT = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))


def _register_extension_modules():
    if _PKG_ROOT not in sys.path:
        sys.path.append(_PKG_ROOT)
    for name in _EXTENSION_MODULES:
        importlib.import_module(name)


def load(neox_args=None):
    """Build (if needed) and load the kernels.

    ``neox_args`` is only consulted for ``rank`` to decide verbosity, as in the
    reference. Raises if the build or the load fails.
    """
    verbose = True if neox_args is None else (getattr(neox_args, "rank", 0) == 0)
    if not os.path.exists(_hotpath.LIB_PATH):
        if verbose:
            print(f"building {_hotpath.LIB_PATH} for gfx950 ...", flush=True)
        _hotpath.build(verbose=verbose)
    _hotpath.lib()
    _register_extension_modules()


def load_fused_kernels():
    """Check that the three extension modules import; print a banner and exit
    otherwise (same behaviour as the reference)."""
    try:
        _register_extension_modules()
        _hotpath.lib()
    except (ImportError, ModuleNotFoundError) as e:
        print("\n")
        print(e)
        print("=" * 100)
        print(
            "ERROR: Fused kernels configured but not properly installed. Please run "
            "`from megatron.fused_kernels import load` then `load()` to load them correctly"
        )
        print("=" * 100)
        exit()
    return
