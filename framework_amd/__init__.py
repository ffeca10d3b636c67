"""MI355X (gfx950) backend for the fp32 matmul path of mni-ml/framework.

`framework_amd.rocm()` gives the kernel-level C ABI, `framework_amd.api()` the
Tensor / Linear / Adam wrappers bound to the HIP engine.  Both load
framework_amd/lib/libmni_rocm.so and raise if it is missing.
"""
from . import synth  # noqa: F401

_api = None
_rocm = None


def rocm():
    global _rocm
    if _rocm is None:
        from .native import Rocm
        _rocm = Rocm()
    return _rocm


def api():
    global _api
    if _api is None:
        from .api import bind
        from .native import Native
        _api = bind(Native())
    return _api
