#include "common.h"
extern "C" int tlf_varlen_prefill_attn(const void *, int64_t, const void *, int64_t, const void *, int64_t, int32_t, const float *, const float *, const int32_t *, const int32_t *, const int32_t *, int64_t, void *, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int64_t, float, void *) { return TLF_E_UNSUPPORTED; }
