"""flh_amd -- MI355X (gfx950) implementation of FLH's W4A4 linear-layer hot path.

The package keeps the reference's layout and names (``flh.nn``, ``flh.functional``,
``flh.cuda``, ``flh._CUDA``, ``flh.PackedQuantizedTensor``; reference: flh/__init__.py)
so that existing code can switch by importing ``flh_amd`` under the name ``flh``
(see :func:`install_as_flh`).  All ops run on hand-written HIP kernels reached through
the C ABI of ``libflh_hip.so``; there is no CPU or torch fallback for them -- using an op
without the built library raises :class:`flh_amd._lib.FLHLibraryError`.
"""
import os
import pathlib
import sys
import types

import torch

from . import _lib


class _LazyOps(types.ModuleType):
    """Stands where the reference has the compiled ``flh._CUDA`` module.  The HIP library
    is loaded on first attribute access, so importing the package works on a machine
    without it (e.g. to use the torch-side helpers); calling an op there fails loudly.
    With the PyTorch-ROCm extension built (flh_amd/_flh_torch.so) the ops are its C++ functions
    (``_ext_ops``); without it, or with FLH_OPS=ctypes in the environment, the ctypes route
    (``_ops``).  Both call the same C ABI of libflh_hip.so -- neither is a fallback off the GPU."""

    _impl = None

    def __getattr__(self, name):
        impl = _LazyOps._impl
        if impl is None:
            _lib.load()  # raises FLHLibraryError with build instructions when missing
            ext = pathlib.Path(__file__).with_name("_flh_torch.so")
            if ext.exists() and os.environ.get("FLH_OPS", "") != "ctypes":
                from . import _ext_ops as impl
            else:
                from . import _ops as impl
            _LazyOps._impl = impl
        return getattr(impl, name)


_CUDA = _LazyOps("flh_amd._CUDA")


class PackedQuantizedTensor:
    """Packed int4 codes together with their scales (reference: flh/__init__.py:37-53)."""

    def __init__(self, quantized_x: torch.Tensor, scales_x: torch.Tensor):
        self.quantized_x = quantized_x
        self.scales_x = scales_x

    def size(self):
        return self.quantized_x.size()

    @property
    def device(self):
        return self.quantized_x.device

    @property
    def dtype(self):
        return self.quantized_x.dtype


from . import functional, nn, cuda, hql  # noqa: E402,F401


def install_as_flh():
    """Register this package under the name ``flh`` (and its submodules under
    ``flh.nn`` ...), so that ``import flh`` in existing code resolves to it."""
    me = sys.modules[__name__]
    sys.modules.setdefault("flh", me)
    for name, mod in list(sys.modules.items()):
        if name.startswith(__name__ + "."):
            sys.modules.setdefault("flh" + name[len(__name__):], mod)
    return me
