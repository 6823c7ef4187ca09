#include "common.h"
extern "C" int trn_prenorm_qkv_f16(const void*, const void*, const void*, const void*, const void*, void*, void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, float, int32_t, void*) { return TRN_E_UNSUPPORTED; }
