// Shared device/host helpers for libckv (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/ckv.h"

#define CKV_WAVE 64

#define CKV_HIP_TRY(expr)                          \
    do {                                           \
        hipError_t err__ = (expr);                 \
        if (err__ != hipSuccess) {                 \
            (void)hipGetLastError();               \
            return CKV_ERR_LAUNCH;                 \
        }                                          \
    } while (0)

namespace ckv {

__host__ __device__ inline int64_t elem_bytes(int dtype) { return dtype == CKV_F32 ? 4 : 2; }

// exact widening of one stored score to fp32
__device__ inline float load_as_float(const void* base, int64_t idx, int dtype) {
    if (dtype == CKV_F32) return reinterpret_cast<const float*>(base)[idx];
    const uint16_t h = reinterpret_cast<const uint16_t*>(base)[idx];
    if (dtype == CKV_BF16) return __uint_as_float(static_cast<uint32_t>(h) << 16);
    return __half2float(__ushort_as_half(h));
}

__device__ inline float bf16_bits_to_float(uint16_t h) { return __uint_as_float(static_cast<uint32_t>(h) << 16); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ inline uint16_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
    static constexpr int code = CKV_F32;
    __device__ static float to_float(float v) { return v; }
    __device__ static float from_float(float v) { return v; }
};
template <>
struct Elem<__hip_bfloat16> {
    static constexpr int code = CKV_BF16;
    __device__ static float to_float(__hip_bfloat16 v) { return __bfloat162float(v); }
    __device__ static __hip_bfloat16 from_float(float v) { return __float2bfloat16(v); }
};
template <>
struct Elem<__half> {
    static constexpr int code = CKV_F16;
    __device__ static float to_float(__half v) { return __half2float(v); }
    __device__ static __half from_float(float v) { return __float2half(v); }
};

// stage timing hooks (ckv_profile_enable / ckv_profile_read); no-ops while disabled
void prof_begin(int stage, hipStream_t stream);
void prof_end(int stage, hipStream_t stream);
// Timing of a single kernel by events attached to its own dispatch (hipExtLaunchKernelGGL): unlike an
// event record in the stream, this puts nothing between the kernel and its neighbours.  Used when only
// the attention main kernels are timed.
bool prof_kernel_events_wanted(int stage);
void prof_kernel_events(int stage, hipEvent_t* start, hipEvent_t* stop);  // both null unless wanted
struct StageScope {
    int stage;
    hipStream_t stream;
    bool own;
    // kernel_events: the stage is a single kernel whose launch site takes its start / stop events from
    // prof_kernel_events; the scope then records nothing itself when only main kernels are timed
    StageScope(int s, hipStream_t st, bool kernel_events = false)
        : stage(s), stream(st), own(!(kernel_events && prof_kernel_events_wanted(s))) {
        if (own) prof_begin(s, st);
    }
    ~StageScope() {
        if (own) prof_end(stage, stream);
    }
};

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Facts about the current device, asked of the runtime once per device and process.
struct DeviceInfo {
    int device;        // ordinal of the current device
    int cus;           // compute units
    int lds_max;       // bytes of LDS one workgroup may use
};
int current_device_info(DeviceInfo* info);  // CKV_OK or CKV_ERR_LAUNCH
// Raises the dynamic LDS limit of `func` on the current device to at least `bytes`; the runtime is asked
// only when the limit this process has already set for (device, func) is smaller.
int ensure_dynamic_lds(const void* func, int bytes);


// sin and cos of an fp32 angle for the 16-bit cache paths: exact range reduction in double (the
// angle is position * frequency, tens of thousands of radians for long contexts), then the hardware
// sin / cos of the remainder, which take revolutions.  Absolute error about 1e-6: three orders below
// the rounding of the rotated values to bf16 / fp16.  The fp32 paths keep sincosf.
__device__ inline void fast_sincos(float x, float* sn, float* cs) {
    const double xd = (double)x;
    const double n = __builtin_rint(xd * 0.15915494309189535);     // x / (2 pi)
    const double r = __builtin_fma(-n, 6.283185307179586, xd);     // |r| <= pi, error ~ n * 2^-52
    const float rev = (float)(r * 0.15915494309189535);
    *sn = __builtin_amdgcn_sinf(rev);
    *cs = __builtin_amdgcn_cosf(rev);
}

// ---------------------------------------------------------------------------------------------
// Rotary embedding on packed 16-bit words with the roundings of the reference's eager path, which evaluates
// x*cos + rotate_half(x)*sin in the tensor dtype (cascade_attention.py:31-35; cos and sin cast to the dtype,
// modeling_llama.py:219-220) and then multiplies queries and keys alike by sqrt(softmax scale)
// (cascade_attention.py:284-291).  w1 holds elements (j, j+1) of a row, w2 their rotation partners (j+64, j+65);
// RopeWord carries the rounded cos / sin of the two pairs in the form the arithmetic consumes.  Every product of
// two 16-bit values and every sum of two 16-bit values is exact in fp32, so each conversion to the tensor dtype
// is one of the reference's roundings: the four products, the two sums, and the products with `post`.
// ---------------------------------------------------------------------------------------------
typedef __bf16 ckv_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 ckv_f16x2 __attribute__((ext_vector_type(2)));
typedef float ckv_f32x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct RopeWord;
// bfloat16 has no packed arithmetic on this chip, but v_dot2_f32_bf16 multiplies both halves of a word without
// unpacking them: with (c, 0) or (0, c) as the other operand it returns one exact product, with (1, -1) or (1, 1)
// the exact difference or sum of a packed pair.
template <>
struct RopeWord<__hip_bfloat16> {
    uint32_t c_lo, c_hi, s_lo, s_hi;  // (c0, 0), (0, c1), (s0, 0), (0, s1)
    __device__ static uint32_t pack2(float a, float b) {
        ckv_f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, ckv_bf16x2));
    }
    __device__ static float lo(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    __device__ static RopeWord make(float c0, float s0, float c1, float s1) {
        return RopeWord{pack2(c0, 0.f), pack2(0.f, c1), pack2(s0, 0.f), pack2(0.f, s1)};
    }
    __device__ static float dot(uint32_t a, uint32_t b) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ckv_bf16x2, a), __builtin_bit_cast(ckv_bf16x2, b), 0.f, false);
    }
    // scaled == false: the rotation alone
    __device__ void rotate(uint32_t w1, uint32_t w2, float post, bool scaled, uint32_t& o1, uint32_t& o2) const {
        const uint32_t p0 = pack2(dot(w1, c_lo), dot(w2, s_lo)), q0 = pack2(dot(w2, c_lo), dot(w1, s_lo));
        const uint32_t p1 = pack2(dot(w1, c_hi), dot(w2, s_hi)), q1 = pack2(dot(w2, c_hi), dot(w1, s_hi));
        constexpr uint32_t kOneMinusOne = 0xbf803f80u, kOneOne = 0x3f803f80u;  // (1, -1), (1, 1)
        o1 = pack2(dot(p0, kOneMinusOne), dot(p1, kOneMinusOne));
        o2 = pack2(dot(q0, kOneOne), dot(q1, kOneOne));
        if (scaled) {
            o1 = pack2(lo(o1) * post, hi(o1) * post);
            o2 = pack2(lo(o2) * post, hi(o2) * post);
        }
    }
};
// float16: the packed multiply, subtract and add round each result to float16, which is the reference's arithmetic
template <>
struct RopeWord<__half> {
    uint32_t c, s;  // (c0, c1), (s0, s1)
    __device__ static uint32_t pack2(float a, float b) {
        ckv_f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, ckv_f16x2));
    }
    __device__ static float lo(uint32_t w) { return (float)__builtin_bit_cast(ckv_f16x2, w)[0]; }
    __device__ static float hi(uint32_t w) { return (float)__builtin_bit_cast(ckv_f16x2, w)[1]; }
    __device__ static RopeWord make(float c0, float s0, float c1, float s1) { return RopeWord{pack2(c0, c1), pack2(s0, s1)}; }
    __device__ void rotate(uint32_t w1, uint32_t w2, float post, bool scaled, uint32_t& o1, uint32_t& o2) const {
#pragma clang fp contract(off)  // a fused multiply-add would skip the rounding of the product
        const ckv_f16x2 x1 = __builtin_bit_cast(ckv_f16x2, w1), x2 = __builtin_bit_cast(ckv_f16x2, w2);
        const ckv_f16x2 cc = __builtin_bit_cast(ckv_f16x2, c), ss = __builtin_bit_cast(ckv_f16x2, s);
        const ckv_f16x2 a1 = x1 * cc, b1 = x2 * ss, a2 = x2 * cc, b2 = x1 * ss;
        const ckv_f16x2 r1 = a1 - b1, r2 = a2 + b2;
        o1 = __builtin_bit_cast(uint32_t, r1);
        o2 = __builtin_bit_cast(uint32_t, r2);
        if (scaled) {
            o1 = pack2(lo(o1) * post, hi(o1) * post);
            o2 = pack2(lo(o2) * post, hi(o2) * post);
        }
    }
};

__device__ inline const void* uniform_ptr(const void* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
}

// Asynchronous global -> LDS copy of one 16-byte piece per lane (gfx950 global_load_lds_dwordx4):
// the wavefront's 64 pieces land contiguously at LDS byte address `lds_wave_base` (uniform, goes
// to M0), lane i at +16*i; the source is `sbase` (uniform, SGPR pair) + `voff` (per lane).
// Inline assembly on purpose: the compiler keeps no scoreboard entry for the copy, so it cannot
// force it to complete before unrelated LDS reads; completion is awaited explicitly with
// s_waitcnt vmcnt(n) (copies retire in issue order).  M0 is written without being declared: the compiler
// reserves it and loads it itself right before each of its own instructions that read it.
__device__ inline void async_copy16(const void* sbase, uint32_t voff, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)), "v"(voff), "s"(uniform_ptr(sbase))
                 : "memory");
}

__device__ inline uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

}  // namespace ckv
