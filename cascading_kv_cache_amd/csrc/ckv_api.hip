// Entry points of libckv that are not tied to one kernel family.
#include "ckv_common.h"

#include <cstdint>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace ckv {
namespace {
struct Span {
    int stage;
    hipEvent_t t0, t1;
};
int g_prof_level = 0;  // 0 off, 1 every stage, 2 attention main kernels only, 3 update kernels only, 4 = 2 sampled
int64_t g_sample_count[CKV_STAGE_COUNT] = {};
std::vector<Span> g_spans;
hipEvent_t g_open[CKV_STAGE_COUNT];
std::mutex g_prof_mutex;  // guards g_spans and g_open: calls on several host threads may time stages at once

constexpr int kMaxDevices = 64;
std::mutex g_dev_mutex;
DeviceInfo g_dev[kMaxDevices];
bool g_dev_known[kMaxDevices];
std::unordered_map<const void*, int> g_lds_set[kMaxDevices];  // dynamic LDS limit already set per kernel
}  // namespace

int current_device_info(DeviceInfo* info) {
    int dev = 0;
    CKV_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return CKV_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    if (!g_dev_known[dev]) {
        DeviceInfo d;
        d.device = dev;
        d.cus = 256;
        d.lds_max = 65536;
        CKV_HIP_TRY(hipDeviceGetAttribute(&d.cus, hipDeviceAttributeMultiprocessorCount, dev));
        CKV_HIP_TRY(hipDeviceGetAttribute(&d.lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
        g_dev[dev] = d;
        g_dev_known[dev] = true;
    }
    *info = g_dev[dev];
    return CKV_OK;
}

int ensure_dynamic_lds(const void* func, int bytes) {
    if (bytes <= 48 * 1024) return CKV_OK;  // within the limit every kernel starts with
    int dev = 0;
    CKV_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return CKV_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    int& have = g_lds_set[dev][func];
    if (have >= bytes) return CKV_OK;
    CKV_HIP_TRY(hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    have = bytes;
    return CKV_OK;
}

// level 2: the attention main kernels; level 3: the kernels of the cache update; level 4: the attention main
// kernels, every fourth launch of each.  All time single kernels by events attached to their dispatch.
constexpr int kSamplePeriod = 4;
static bool dispatch_timed(int stage) {
    return ((g_prof_level == 2 || g_prof_level == 4) && (stage == CKV_STAGE_FWD || stage == CKV_STAGE_DECODE)) ||
           (g_prof_level == 3 && (stage == CKV_STAGE_PLAN || stage == CKV_STAGE_APPLY));
}

static bool prof_wanted(int stage) { return g_prof_level == 1 || dispatch_timed(stage); }

bool prof_kernel_events_wanted(int stage) { return dispatch_timed(stage); }

void prof_kernel_events(int stage, hipEvent_t* start, hipEvent_t* stop) {
    *start = *stop = nullptr;
    if (!prof_kernel_events_wanted(stage)) return;
    if (g_prof_level == 4) {  // the first launch of a stage after the level was set, then every kSamplePeriod-th
        std::lock_guard<std::mutex> lock(g_prof_mutex);
        if (g_sample_count[stage]++ % kSamplePeriod != 0) return;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return;
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return;
    }
    {
        std::lock_guard<std::mutex> lock(g_prof_mutex);
        g_spans.push_back(Span{stage, e0, e1});
    }
    *start = e0;
    *stop = e1;
}

void prof_begin(int stage, hipStream_t stream) {
    if (!prof_wanted(stage)) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    g_open[stage] = e;
}

void prof_end(int stage, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (!g_open[stage]) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, stream);
    g_spans.push_back(Span{stage, g_open[stage], e});
    g_open[stage] = nullptr;
}
}  // namespace ckv

extern "C" int ckv_profile_enable(int on) {
    const int prev = ckv::g_prof_level;
    ckv::g_prof_level = on < 0 || on > 4 ? 1 : on;
    {
        std::lock_guard<std::mutex> lock(ckv::g_prof_mutex);
        for (int i = 0; i < CKV_STAGE_COUNT; i++) ckv::g_sample_count[i] = 0;
    }
    return prev;
}

extern "C" int ckv_profile_read(double* ms, int64_t* launches) {
    if (!ms || !launches) return CKV_ERR_NULL;
    std::lock_guard<std::mutex> lock(ckv::g_prof_mutex);
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

namespace ckv {
namespace {
__global__ void __launch_bounds__(1024) chunk_positions_kernel(const int64_t* key_pos, int64_t n_key, int64_t key_shift,
                                                               const int64_t* sink_pos, int64_t n_sink, int64_t q_len,
                                                               int64_t* q_pos) {
    __shared__ int64_t red[16];
    const int tid = threadIdx.x;
    int64_t base = 0;
    if (key_pos || sink_pos) {
        int64_t m = INT64_MIN;
        // one workgroup reads the whole row: eight independent 16-byte loads per thread and trip keep
        // enough requests in flight for that
        int64_t i0 = 0;
        if ((reinterpret_cast<uintptr_t>(key_pos) & 15u) == 0) {
            const longlong2* kp2 = reinterpret_cast<const longlong2*>(key_pos);
            const int64_t n2 = n_key / 2;
            int64_t i = tid;
            for (; i + 7 * 1024 < n2; i += 8 * 1024) {
                longlong2 v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = kp2[i + u * 1024];
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    const int64_t a = v[u].x > v[u].y ? v[u].x : v[u].y;
                    m = a > m ? a : m;
                }
            }
            for (; i < n2; i += 1024) {
                const longlong2 v = kp2[i];
                const int64_t a = v.x > v.y ? v.x : v.y;
                m = a > m ? a : m;
            }
            i0 = 2 * n2;
        }
        for (int64_t i = i0 + tid; i < n_key; i += 1024) {
            const int64_t v = key_pos[i];
            m = v > m ? v : m;
        }
        if (m != INT64_MIN) m += key_shift;
        for (int64_t i = tid; i < n_sink; i += 1024) {
            const int64_t v = sink_pos[i];
            m = v > m ? v : m;
        }
        for (int off = 32; off > 0; off >>= 1) {
            const int64_t o = __shfl_xor(m, off);
            m = o > m ? o : m;
        }
        if ((tid & 63) == 0) red[tid >> 6] = m;
        __syncthreads();
        m = red[0];
        for (int w = 1; w < 16; w++) m = red[w] > m ? red[w] : m;
        base = m + 1;
    }
    for (int64_t i = tid; i < q_len; i += 1024) q_pos[i] = base + i;
}
}  // namespace
}  // namespace ckv

extern "C" int ckv_chunk_positions(const int64_t* key_pos, int64_t n_key, int64_t key_shift, const int64_t* sink_pos,
                                   int64_t n_sink, int64_t q_len, int64_t* q_pos, void* stream_) {
    if (!q_pos) return CKV_ERR_NULL;
    if (q_len <= 0 || n_key < 0 || n_sink < 0) return CKV_ERR_SHAPE;
    if (n_key == 0) key_pos = nullptr;
    if (n_sink == 0) sink_pos = nullptr;
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    hipLaunchKernelGGL(ckv::chunk_positions_kernel, dim3(1), dim3(1024), 0, stream, key_pos, key_pos ? n_key : 0, key_shift,
                       sink_pos, sink_pos ? n_sink : 0, q_len, q_pos);
    CKV_HIP_TRY(hipGetLastError());
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
        case CKV_ERR_TOO_LARGE: return "sizes exceed the fixed scratch of ckv_update_static (use ckv_update with a workspace)";
        default: return "unknown ckv status";
    }
}

extern "C" int ckv_abi_version(void) { return CKV_ABI_VERSION; }

// struct sizes, so a foreign-language binding can check its mirror of the header
extern "C" int64_t ckv_sizeof_update_args(void) { return (int64_t)sizeof(ckv_update_args); }
extern "C" int64_t ckv_sizeof_attn_args(void) { return (int64_t)sizeof(ckv_attn_args); }
extern "C" int64_t ckv_sizeof_dense_args(void) { return (int64_t)sizeof(ckv_dense_args); }
extern "C" int64_t ckv_sizeof_dense_bwd_args(void) { return (int64_t)sizeof(ckv_dense_bwd_args); }
