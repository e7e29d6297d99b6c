// placeholder until the sliding-window kernels land
#include "common.hpp"
extern "C" BASED_API int based_swa_prefill(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t,
    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
    int, float, int, void*) { based::set_error("swa_prefill: not built yet"); return BASED_ERR_SHAPE; }
extern "C" BASED_API int based_swa_step(const void*, const void*, const void*, void*, void*, void*, const int32_t*, int64_t,
    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
    int64_t, int64_t, int64_t, int, float, int, void*) { based::set_error("swa_step: not built yet"); return BASED_ERR_SHAPE; }
