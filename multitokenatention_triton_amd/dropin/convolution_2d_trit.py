"""Import shim: put this directory on sys.path and `import convolution_2d_trit` resolves to the HIP build."""
from multitokenatention_triton_amd.convolution_2d_trit import *  # noqa: F401,F403
from multitokenatention_triton_amd import convolution_2d_trit as _impl

__all__ = getattr(_impl, "__all__", [n for n in dir(_impl) if not n.startswith("_")])
