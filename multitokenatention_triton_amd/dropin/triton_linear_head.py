"""Import shim: put this directory on sys.path and `import triton_linear_head` resolves to the HIP build."""
from multitokenatention_triton_amd.triton_linear_head import *  # noqa: F401,F403
from multitokenatention_triton_amd import triton_linear_head as _impl

__all__ = getattr(_impl, "__all__", [n for n in dir(_impl) if not n.startswith("_")])
