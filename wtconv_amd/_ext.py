"""Loader of the C++ autograd node (wtconv_amd/csrc/torch_binding.cpp, built in-tree as _wtconv_torch.so).

The node is an optimisation of the host path only: it launches the same library calls as
wtconv_amd/functional.py without the interpreter.  Where the module has not been built, `get()` returns None
and the Python autograd function is used; WTCONV_NO_CPP_NODE=1 in the environment forces that as well."""
import ctypes
import importlib.util
import os

from . import _build, _lib

# order of the addresses bind() takes (torch_binding.cpp)
_ENTRY_POINTS = ("wtconv2d_forward", "wtconv2d_backward", "wtconv2d_backward_input", "wtconv2d_backward_params",
                 "wtconv2d_workspace_bytes",
                 "wtconv1d_forward", "wtconv1d_backward", "wtconv1d_backward_input", "wtconv1d_backward_params",
                 "wtconv1d_workspace_bytes", "wtconv_last_error")

_mod = None
_tried = False


def get():
    """The bound extension module, or None."""
    global _mod, _tried
    if _tried:
        return _mod
    _tried = True
    if os.environ.get("WTCONV_NO_CPP_NODE") == "1" or not os.path.exists(_build.BINDING_PATH):
        return None
    import torch  # noqa: F401  (the module links against PyTorch's libraries, which must be loaded first)
    spec = importlib.util.spec_from_file_location(_build.BINDING_NAME, _build.BINDING_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    lib = _lib.load()
    mod.bind([ctypes.cast(getattr(lib, name), ctypes.c_void_p).value for name in _ENTRY_POINTS])
    _mod = mod
    return _mod
