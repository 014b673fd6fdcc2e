// Entry points of libckv that are not tied to one kernel family.
#include "ckv_common.h"

#include <vector>

namespace ckv {
namespace {
struct Span {
    int stage;
    hipEvent_t t0, t1;
};
bool g_prof_on = false;
std::vector<Span> g_spans;
hipEvent_t g_open[CKV_STAGE_COUNT];
}  // namespace

void prof_begin(int stage, hipStream_t stream) {
    if (!g_prof_on) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    g_open[stage] = e;
}

void prof_end(int stage, hipStream_t stream) {
    if (!g_prof_on || !g_open[stage]) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    g_spans.push_back(Span{stage, g_open[stage], e});
    g_open[stage] = nullptr;
}
}  // namespace ckv

extern "C" int ckv_profile_enable(int on) {
    const int prev = ckv::g_prof_on ? 1 : 0;
    ckv::g_prof_on = on != 0;
    return prev;
}

extern "C" int ckv_profile_read(double* ms, int64_t* launches) {
    if (!ms || !launches) return CKV_ERR_NULL;
    for (auto& s : ckv::g_spans) {
        float t = 0.f;
        if (hipEventSynchronize(s.t1) == hipSuccess && hipEventElapsedTime(&t, s.t0, s.t1) == hipSuccess) {
            ms[s.stage] += t;
            launches[s.stage] += 1;
        }
        (void)hipEventDestroy(s.t0);
        (void)hipEventDestroy(s.t1);
    }
    ckv::g_spans.clear();
    return CKV_OK;
}

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
