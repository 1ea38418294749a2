#include "common.hpp"
extern "C" int mta_conv_attn_fwd(const void *, const void *, const void *, const void *, void *, int64_t, int64_t,
                                 int64_t, int64_t, int, int, int, float, int, int, void *)
{
    return MTA_ERR_HEAD_DIM;
}
