// Fused FFN (placeholder until the kernel lands: reports "unsupported").
#include "bsrl_common.h"
extern "C" int bsrl_ffn_fused_supported(int64_t, int64_t, int) { return 0; }
extern "C" int bsrl_ffn_fused(const void*, const void*, const void*, const float*, const void*, const float*,
                              const float*, const float*, float, void*, void*, int64_t, int64_t, int64_t, int, int,
                              bsrl_stream) { return BSRL_UNSUPPORTED; }
