"""MI355X-native Multi-Token-Attention forward path.

Hand-written HIP kernels (libmta_hip.so, C ABI in include/mta_hip.h) behind the Python
call surface of Gusanidas/multitokenatention_triton:

    MTAAttentionTriton      full MTA forward           (mta_attention_triton.py)
    TritonConvAttention     fused QK^T+conv+softmax+PV (conv_attention_triton.py)
    Conv2dTriton            depthwise causal 2-D conv  (convolution_2d_trit.py)
    TritonLinearHead        head mixing                (triton_linear_head.py)
"""
from .convolution_2d_trit import Conv2dTriton, Conv2dTritonFunction, PytorchConv, add_causal_mask, pytorch_conv
from .triton_linear_head import TritonLinearHead, TritonLinearHeadFunction
from .conv_attention_triton import TritonAttention, TritonConvAttention
from .mta_attention_triton import MTAAttentionTriton, MTAConfig, WeightStructure
from . import ops

__all__ = ["Conv2dTriton", "Conv2dTritonFunction", "PytorchConv", "pytorch_conv", "add_causal_mask", "TritonLinearHead", "TritonLinearHeadFunction",
           "TritonAttention", "TritonConvAttention", "MTAAttentionTriton", "MTAConfig", "WeightStructure",
           "ops"]
