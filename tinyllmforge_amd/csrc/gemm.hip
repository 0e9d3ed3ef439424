#include "common.h"
extern "C" size_t tlf_w8a16_gemm_workspace_bytes(int32_t, int32_t, int32_t) { return 0; }
extern "C" int tlf_w8a16_gemm(const void *, int64_t, const void *, const float *, void *, int32_t, int32_t, int32_t, void *, size_t, void *) { return TLF_E_UNSUPPORTED; }
extern "C" int tlf_bf16_gemm(const void *, int64_t, const void *, void *, int32_t, int32_t, int32_t, void *, size_t, void *) { return TLF_E_UNSUPPORTED; }
