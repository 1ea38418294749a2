// Version and error-string entry points of the C ABI.
#include "common.hpp"

extern "C" int mta_abi_version(void) { return MTA_ABI_VERSION; }

extern "C" const char *mta_strerror(int code)
{
    switch (code) {
    case MTA_OK: return "ok";
    case MTA_ERR_NULL: return "null pointer argument";
    case MTA_ERR_DTYPE: return "unsupported dtype code";
    case MTA_ERR_SHAPE: return "size is not positive or exceeds the kernel's index range";
    case MTA_ERR_KERNEL_SIZE:
        return "conv kernel size outside the supported range (conv operator and its gradients: 1x1 to 80x95 rows x keys; "
               "fused conv-attention, scores and conv + head-mixing kernels: up to 32x63)";
    case MTA_ERR_GROUP: return "group size does not divide the number of heads";
    case MTA_ERR_ALIGN: return "pointer not aligned to its element size";
    case MTA_ERR_HEAD_DIM: return "head dimension not supported by the fused kernel";
    case MTA_ERR_DEVICE: return "no usable gfx950 device";
    case MTA_ERR_UNSUPPORTED: return "no kernel for this dtype / size combination (use the unfused route)";
    case MTA_ERR_WORKSPACE: return "workspace smaller than the matching *_workspace() call reports";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}
