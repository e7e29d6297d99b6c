// placeholder until the prefill kernel lands
#include "common.hpp"
extern "C" BASED_API int based_linear_attn_prefill(const void*, const void*, const void*, void*, float*, float*,
    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, float, int, void*) {
  based::set_error("linear_attn_prefill: not built yet"); return BASED_ERR_SHAPE; }
