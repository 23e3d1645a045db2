"""Loader of the compiled operator layer (csrc/op_layer.cpp -> _simnets_native.so next to this file).

Importing the module also registers torch.ops.simnets.* (TORCH_LIBRARY).  It links against libsimnets_hip.so in the
same directory; both are built by build.py.  There is nothing to fall back to when it is missing."""
import importlib.util
import os

HERE = os.path.dirname(os.path.abspath(__file__))
PATH = os.path.join(HERE, "_simnets_native.so")

_module = None


def module():
    global _module
    if _module is None:
        if not os.path.exists(PATH):
            raise RuntimeError("_simnets_native.so is missing (%s): build it with `python simnets-tf_amd/build.py`; "
                               "this package has no CPU fallback" % PATH)
        import torch  # noqa: F401  (libtorch must be loaded first)
        spec = importlib.util.spec_from_file_location("_simnets_native", PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _module = mod
    return _module
