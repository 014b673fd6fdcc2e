// placeholder until the attention kernels land
#include "ckv_common.h"
extern "C" int64_t ckv_attn_workspace_bytes(int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int32_t) { return 0; }
extern "C" int ckv_attn(const ckv_attn_args*, void*) { return CKV_ERR_UNSUPPORTED; }
extern "C" int64_t ckv_dense_workspace_bytes(int64_t, int64_t, int64_t, int64_t, int64_t, int32_t) { return 0; }
extern "C" int ckv_attn_dense(const ckv_dense_args*, void*) { return CKV_ERR_UNSUPPORTED; }
