// Entry points of libckv that are not tied to one kernel family.
#include "ckv_common.h"

extern "C" const char* ckv_strerror(int status) {
    switch (status) {
        case CKV_OK: return "ok";
        case CKV_ERR_NULL: return "a required pointer is NULL";
        case CKV_ERR_SHAPE: return "inconsistent sizes";
        case CKV_ERR_STRIDE: return "unsupported memory layout";
        case CKV_ERR_DTYPE: return "unknown dtype";
        case CKV_ERR_WORKSPACE: return "workspace missing or too small";
        case CKV_ERR_UNSUPPORTED: return "request outside what the kernels implement";
        case CKV_ERR_LAUNCH: return "the HIP runtime rejected a launch";
        default: return "unknown ckv status";
    }
}

extern "C" int ckv_abi_version(void) { return CKV_ABI_VERSION; }

// struct sizes, so a foreign-language binding can check its mirror of the header
extern "C" int64_t ckv_sizeof_update_args(void) { return (int64_t)sizeof(ckv_update_args); }
extern "C" int64_t ckv_sizeof_attn_args(void) { return (int64_t)sizeof(ckv_attn_args); }
extern "C" int64_t ckv_sizeof_dense_args(void) { return (int64_t)sizeof(ckv_dense_args); }
