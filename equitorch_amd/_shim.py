"""Loader of the PyTorch C++ extension over the C ABI (``equitorch_amd/lib/_cgtp_torch.so``, built from
``csrc/torch_shim/cgtp_torch.cpp``): the autograd node and per-call marshalling of the fused edge product in C++.
The extension is an accelerator of the host side only — every launch still goes through ``libcgtp.so``; without it
(not built, or ``CGTP_TORCH_SHIM=0``) the same launches are issued through ``ctypes``."""
import importlib.util
import os

from . import _lib

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "_cgtp_torch.so")
_module = None
_tried = False


def module():
    """The extension module, or None."""
    global _module, _tried
    if not _tried:
        _tried = True
        if os.environ.get("CGTP_TORCH_SHIM", "1") != "0" and os.path.exists(_PATH):
            spec = importlib.util.spec_from_file_location("_cgtp_torch", _PATH)
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            if mod.abi_version() != _lib.lib.cgtp_version():
                raise _lib.CgtpError("_cgtp_torch.so was built against another libcgtp.so: rebuild "
                                     "(python -m equitorch_amd.csrc.build)")
            _module = mod
    return _module
