"""Import shim: put this directory on sys.path and `import conv_attention_triton` resolves to the HIP build."""
from multitokenatention_triton_amd.conv_attention_triton import *  # noqa: F401,F403
from multitokenatention_triton_amd import conv_attention_triton as _impl

__all__ = getattr(_impl, "__all__", [n for n in dir(_impl) if not n.startswith("_")])
