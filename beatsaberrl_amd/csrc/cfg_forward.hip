// Whole-forward persistent kernel (placeholder until the kernel lands).
#include "bsrl_common.h"
extern "C" int64_t bsrl_cfg_pack_size(const bsrl_cfg_desc*) { return 0; }
extern "C" int bsrl_cfg_pack(const bsrl_cfg_desc*, const bsrl_cfg_params*, void*, bsrl_stream) { return BSRL_UNSUPPORTED; }
extern "C" int bsrl_cfg_forward(const bsrl_cfg_desc*, const void*, const void*, int64_t, int, const int32_t*, float*,
                                float*, int64_t, bsrl_stream) { return BSRL_UNSUPPORTED; }
