// Single-token decode attention (Q == 1, head_dim 128): bandwidth-bound kernels.
//
//   decode_q      rotate the B*H query rows, fold softmax scale * log2(e) in, keep them as fp32.
//   decode_main   grid (key tiles of 128, groups of (batch, kv-head)).  A workgroup computes the
//                 cos/sin of its 128 keys ONCE (registers) and then streams the K and V rows of
//                 every (batch, kv-head) of its group: each row is read exactly once, 16 lanes per
//                 row with 8-byte pieces, K is rotated in registers, the G query heads of the
//                 group share the row.  Outputs: raw logits (log2 domain) per key and head, and one
//                 (max, sum, weighted V) partial per (head, tile).
//   decode_stream 16-bit caches with shared positions and up to 8 query heads per kv head (the usual case): the
//                 (128-key tile, batch x kv-head) items are dealt out in equal runs over one workgroup per
//                 compute unit; rows travel global -> LDS as asynchronous copies one item ahead; logits and P.V
//                 on the matrix pipe; per item one result chunk (fp16 probabilities relative to the tile
//                 maximum, the tile's weighted V average, maximum and sum).  decode_stream_wide: 5 to 8 heads.
//   decode_tail   combine the partials of a row: out, log-sum-exp.
//   decode_scores P = exp2(logit - lse) exactly, head reduction, score EMA of every slot and the
//                 new token's own score (cascade_attention.py:315-330 with q_len == 1).
#include "ckv_attn_internal.h"

#include <algorithm>
#include <type_traits>

namespace ckv {
namespace {

constexpr int kD = 128;
constexpr int kTK = 128;     // keys per workgroup tile
constexpr int kSteps = 8;    // a wavefront covers 32 keys as 8 steps of 4 keys (16 lanes per key)
constexpr int kStreamWaves = 8;          // streaming kernel: wavefronts per workgroup, 16 keys each
constexpr int kSK = 16 * kStreamWaves;   // streaming kernel: keys per tile

template <typename T>
__device__ inline float round_t(float v) {
    return Elem<T>::to_float(Elem<T>::from_float(v));
}

// One rotation pair with the roundings of the eager path, which evaluates x*cos + rotate_half(x)*sin in the tensor
// dtype (cascade_attention.py:31-35; cos and sin cast to the dtype, modeling_llama.py:219-220) and then multiplies
// queries and keys alike by sqrt(softmax scale) (cascade_attention.py:284-291): every product and every sum is
// rounded on its own (no fused multiply-add), `c` and `s` arrive rounded, `post` is the sqrt(scale) factor.
template <typename T>
__device__ inline void rope_ref(float x1, float x2, float c, float s, float post, float& r1, float& r2) {
    r1 = round_t<T>(__fadd_rn(round_t<T>(__fmul_rn(x1, c)), round_t<T>(__fmul_rn(-x2, s))));
    r2 = round_t<T>(__fadd_rn(round_t<T>(__fmul_rn(x2, c)), round_t<T>(__fmul_rn(x1, s))));
    r1 = round_t<T>(__fmul_rn(r1, post));
    r2 = round_t<T>(__fmul_rn(r2, post));
}

// all-reduce (sum) inside each row of 16 lanes with DPP: quad xor 1, quad xor 2, half mirror, mirror
__device__ inline float row16_sum(float x) {
    int v = __float_as_int(x);
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));
    v = __float_as_int(x);
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));
    v = __float_as_int(x);
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));
    v = __float_as_int(x);
    x += __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));
    return x;
}

// 4 consecutive elements of a row: raw load now, widening to fp32 later
template <typename T>
struct Piece;
template <>
struct Piece<float> {
    using Raw = float4;
    __device__ static void unpack(const Raw& v, float out[4]) { out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w; }
};
template <>
struct Piece<__hip_bfloat16> {
    using Raw = uint2;
    __device__ static void unpack(const Raw& v, float out[4]) {
        out[0] = __uint_as_float(v.x << 16); out[1] = __uint_as_float(v.x & 0xffff0000u);
        out[2] = __uint_as_float(v.y << 16); out[3] = __uint_as_float(v.y & 0xffff0000u);
    }
};
template <>
struct Piece<__half> {
    using Raw = uint2;
    __device__ static void unpack(const Raw& v, float out[4]) {
        const float2 fa = __half22float2(*reinterpret_cast<const __half2*>(&v.x));
        const float2 fb = __half22float2(*reinterpret_cast<const __half2*>(&v.y));
        out[0] = fa.x; out[1] = fa.y; out[2] = fb.x; out[3] = fb.y;
    }
};

struct DecodeParams {
    ckv_attn_args a;
    float* qrot;       // (B, H, 128) rotated, pre-scaled queries
    void* qrot_t;      // (B, H, 128) rotated queries in the tensor dtype (MFMA operand)
    float* logits;     // (B, KVH, N, G) log2-domain logits, -inf for hidden keys
    // The streaming kernel instead (same memory): one chunk per (tile, b, kvh) item, G rows of kSK fp16
    // values 2^(logit - maximum of the head's logits in the tile), then G rows of 128 per-tile weighted V
    // averages in the tensor dtype.  Chunks are laid out by time: chunk (i, w) is the i-th item of
    // workgroup w, and the chunks of equal i sit side by side, so that what the workgroups store at about
    // the same time is one stretch of memory.
    unsigned char* chunks;
    int64_t Np;        // the keys rounded up to whole tiles of the streaming kernel
    int stream_wgs;    // workgroups of the streaming kernel
    float* part_ml;    // (B, H, tiles, 2); after the streaming kernel (chunk, G, 2)
    float* part_o;     // (B, H, tiles, 128)
    float* lse2;       // (B, H)
    int64_t N;         // num_sink + S + 1
    int tiles;
    int shared_pos;
    float key_scale;   // sqrt(softmax scale): rotated queries and keys both carry it, rounded in (see rope_ref)
    float scale_log2;  // what the logits are still multiplied by: log2(e)
    // Streaming kernel: items exist only for tiles that can hold a visible key, numbered in tile order: the
    // first `tiles_pre` tiles (sinks and the cache slots below the caller's `filled_slots` bound) and the tile
    // of the new token (`tiles - 1`) when it is not one of them.  A cache that is still filling is mostly hidden.
    int tiles_pre;
    int n_vis;         // tiles_pre, or tiles_pre + 1
};

// the j-th tile with items; the rank of a tile among those (-1: the tile has no items, its keys are all hidden)
__device__ inline int stream_tile_of(const DecodeParams& p, int j) { return j < p.tiles_pre ? j : p.tiles - 1; }
__device__ inline int stream_rank_of(const DecodeParams& p, int tile) {
    return tile < p.tiles_pre ? tile : (tile == p.tiles - 1 ? p.n_vis - 1 : -1);
}

// Items (tile-major: item = tile * B * KVH + b * KVH + kvh) are dealt out in equal contiguous runs:
// workgroup w takes [total * w / wgs, total * (w + 1) / wgs).  Chunk index of an item.
__device__ inline int64_t stream_chunk_of(int64_t item, int64_t total, int64_t wgs) {
    int64_t w, first;
    if ((total + 1) * wgs < ((int64_t)1 << 32)) {  // 32-bit division: a fraction of the cost
        w = (int64_t)(((uint32_t)(item + 1) * (uint32_t)wgs - 1u) / (uint32_t)total);
        first = (int64_t)((uint32_t)total * (uint32_t)w / (uint32_t)wgs);
    } else {
        w = ((item + 1) * wgs - 1) / total;
        first = total * w / wgs;
    }
    return (item - first) * wgs + w;
}

template <typename T>
__global__ void decode_q_kernel(DecodeParams p) {
    const ckv_attn_args& a = p.a;
    const int64_t row = blockIdx.x;  // b * H + h
    const int j = threadIdx.x;       // 0..63: rotation pair
    const int64_t b = row / a.H, h = row % a.H;
    const T* q = (const T*)a.q + b * a.q_stride[0] + h * a.q_stride[1];
    const float f = a.inv_freq ? a.inv_freq[j] : 1.0f / powf(a.rope_theta, (float)(2 * j) / (float)kD);
    float sn, cs;
    sincosf(__fmul_rn((float)a.q_pos[0], f), &sn, &cs);
    const float x1 = Elem<T>::to_float(q[j * a.q_stride[3]]), x2 = Elem<T>::to_float(q[(j + 64) * a.q_stride[3]]);
    float r1, r2;
    rope_ref<T>(x1, x2, round_t<T>(cs), round_t<T>(sn), p.key_scale, r1, r2);
    p.qrot[row * kD + j] = r1 * p.scale_log2;
    p.qrot[row * kD + 64 + j] = r2 * p.scale_log2;
    ((T*)p.qrot_t)[row * kD + j] = Elem<T>::from_float(r1);
    ((T*)p.qrot_t)[row * kD + 64 + j] = Elem<T>::from_float(r2);
}

// source row of key n: sink, cache slot or the new token
template <typename T>
__device__ inline bool key_source(const ckv_attn_args& a, int64_t n, int64_t b, int64_t kvh, const T*& kp, const T*& vp,
                                  int64_t& pos) {
    const int64_t NS = a.num_sink, S = a.S;
    if (n < NS) {
        const int64_t off = b * a.sink_stride[0] + kvh * a.sink_stride[1] + n * a.sink_stride[2];
        kp = (const T*)a.sink_k + off;
        vp = (const T*)a.sink_v + off;
        pos = a.sink_pos[b * a.sink_pos_stride[0] + kvh * a.sink_pos_stride[1] + n];
        return a.sink_mask[n] == 0;
    }
    if (n < NS + S) {
        const int64_t slot = n - NS;
        const int64_t off = b * a.cache_stride[0] + kvh * a.cache_stride[1] + slot * a.cache_stride[2];
        kp = (const T*)a.cache_k + off;
        vp = (const T*)a.cache_v + off;
        pos = a.pos[b * a.pos_stride[0] + kvh * a.pos_stride[1] + slot] + a.pos_shift;
        return a.mask[slot] == 0;
    }
    const int64_t off = b * a.kv_new_stride[0] + kvh * a.kv_new_stride[1];
    kp = (const T*)a.k_new + off;
    vp = (const T*)a.v_new + off;
    pos = a.q_pos[0];
    return true;
}

template <typename T, int G>
__global__ void __launch_bounds__(256) decode_main_kernel(DecodeParams p) {
    extern __shared__ __align__(16) float red[];  // [16][G][128] weighted-V partials, [16][G] max, [16][G] sum
    float* red_o = red;
    float* red_m = red + 16 * G * kD;
    float* red_l = red_m + 16 * G;
    using Raw = typename Piece<T>::Raw;
    const ckv_attn_args& a = p.a;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int kg = lane >> 4, j = lane & 15;       // key within a step, piece index inside the row
    const int grp = wave * 4 + kg;                 // 16-lane group id, 0..15
    const int64_t tile = blockIdx.x;
    const int64_t nbh = a.B * a.KVH;

    // cos/sin of this lane's 8 keys x 4 frequencies, computed once when every (b, kvh) shares them
    float cs[kSteps][4], sn[kSteps][4];
    if (p.shared_pos) {
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const int64_t n = tile * kTK + wave * (4 * kSteps) + s * 4 + kg;
            const T *kp, *vp;
            int64_t pos = 0;
            if (n < p.N) key_source<T>(a, n, 0, 0, kp, vp, pos);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int f = 4 * j + e;
                const float fr = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                sincosf(__fmul_rn((float)pos, fr), &sn[s][e], &cs[s][e]);
                sn[s][e] = round_t<T>(sn[s][e]);
                cs[s][e] = round_t<T>(cs[s][e]);
            }
        }
    }

    for (int64_t bh = blockIdx.y; bh < nbh; bh += gridDim.y) {
        const int64_t b = bh / a.KVH, kvh = bh % a.KVH;
        // ---- issue every row read of this (b, kvh) up front: 8 keys x (K, V) x 2 pieces
        Raw kraw[kSteps][2], vraw[kSteps][2];
        bool vis[kSteps];
        int64_t posv[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const int64_t n = tile * kTK + wave * (4 * kSteps) + s * 4 + kg;
            const T *kp = nullptr, *vp = nullptr;
            posv[s] = 0;
            vis[s] = n < p.N && key_source<T>(a, n, b, kvh, kp, vp, posv[s]);
            if (vis[s]) {
                kraw[s][0] = *reinterpret_cast<const Raw*>(kp + 4 * j);
                kraw[s][1] = *reinterpret_cast<const Raw*>(kp + 64 + 4 * j);
                vraw[s][0] = *reinterpret_cast<const Raw*>(vp + 4 * j);
                vraw[s][1] = *reinterpret_cast<const Raw*>(vp + 64 + 4 * j);
            }
        }
        // this lane's 8 dims of the G rotated queries: [4j, 4j+4) and [64+4j, 64+4j+4)
        float qa[G][4], qb[G][4];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float* qr = p.qrot + ((b * a.H) + kvh * G + g) * kD;
            const float4 va = *reinterpret_cast<const float4*>(qr + 4 * j);
            const float4 vb = *reinterpret_cast<const float4*>(qr + 64 + 4 * j);
            qa[g][0] = va.x; qa[g][1] = va.y; qa[g][2] = va.z; qa[g][3] = va.w;
            qb[g][0] = vb.x; qb[g][1] = vb.y; qb[g][2] = vb.z; qb[g][3] = vb.w;
        }
        // ---- phase 1: logits of the 8 keys of this 16-lane group
        float sreg[kSteps][G];
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            float ka[4] = {0.f, 0.f, 0.f, 0.f}, kb[4] = {0.f, 0.f, 0.f, 0.f};
            if (vis[s]) {
                Piece<T>::unpack(kraw[s][0], ka);
                Piece<T>::unpack(kraw[s][1], kb);
            }
            float acc[G];
#pragma unroll
            for (int g = 0; g < G; g++) acc[g] = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float c_ = cs[s][e], s_ = sn[s][e];
                if (!p.shared_pos) {
                    const int f = 4 * j + e;
                    const float fr = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                    sincosf(__fmul_rn((float)posv[s], fr), &s_, &c_);
                    s_ = round_t<T>(s_);
                    c_ = round_t<T>(c_);
                }
                float ra, rb;
                rope_ref<T>(ka[e], kb[e], c_, s_, p.key_scale, ra, rb);
#pragma unroll
                for (int g = 0; g < G; g++) acc[g] = fmaf(ra, qa[g][e], fmaf(rb, qb[g][e], acc[g]));
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float tot = row16_sum(acc[g]);
                sreg[s][g] = vis[s] ? tot : -INFINITY;
            }
            const int64_t n = tile * kTK + wave * (4 * kSteps) + s * 4 + kg;
            if (j == 0 && n < p.N) {
                float* lg = p.logits + ((b * a.KVH + kvh) * p.N + n) * G;
#pragma unroll
                for (int g = 0; g < G; g++) lg[g] = sreg[s][g];
            }
        }
        // ---- phase 2: softmax partial of the group and its weighted V sum
        float mg[G], lgp[G], o[G][8];
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m = sreg[0][g];
#pragma unroll
            for (int s = 1; s < kSteps; s++) m = fmaxf(m, sreg[s][g]);
            mg[g] = m;
            lgp[g] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) o[g][e] = 0.f;
        }
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            if (!vis[s]) continue;
            float va[4], vb[4];
            Piece<T>::unpack(vraw[s][0], va);
            Piece<T>::unpack(vraw[s][1], vb);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float pe = __builtin_amdgcn_exp2f(sreg[s][g] - mg[g]);  // mg is finite: the key is visible
                lgp[g] += pe;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o[g][e] = fmaf(pe, va[e], o[g][e]);
                    o[g][4 + e] = fmaf(pe, vb[e], o[g][4 + e]);
                }
            }
        }
        // ---- combine the 16 groups of the workgroup
        __syncthreads();  // the previous (b, kvh) has been written out
        if (j == 0) {
#pragma unroll
            for (int g = 0; g < G; g++) red_m[grp * G + g] = mg[g];
        }
        __syncthreads();
        float mt[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m = red_m[g];
#pragma unroll
            for (int r = 1; r < 16; r++) m = fmaxf(m, red_m[r * G + g]);
            mt[g] = m;
            const float sc = mg[g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mg[g] - m);
            if (j == 0) red_l[grp * G + g] = lgp[g] * sc;
            float* ro = red_o + (grp * G + g) * kD;
            *reinterpret_cast<float4*>(ro + 4 * j) = make_float4(o[g][0] * sc, o[g][1] * sc, o[g][2] * sc, o[g][3] * sc);
            *reinterpret_cast<float4*>(ro + 64 + 4 * j) =
                make_float4(o[g][4] * sc, o[g][5] * sc, o[g][6] * sc, o[g][7] * sc);
        }
        __syncthreads();
        for (int i = tid; i < G * kD; i += 256) {
            const int g = i / kD, d = i % kD;
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) acc += red_o[(r * G + g) * kD + d];
            p.part_o[(((b * a.H) + kvh * G + g) * p.tiles + tile) * kD + d] = acc;
        }
        if (tid < G) {
            float l = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) l += red_l[r * G + tid];
            float* ml = p.part_ml + (((b * a.H) + kvh * G + tid) * p.tiles + tile) * 2;
            ml[0] = mt[tid];
            ml[1] = l;
        }
    }
}

// ---- 16-bit dtypes: the logits come from v_mfma_f32_16x16x32 (16 head rows, G real, x 16 keys),
// so the dot products cost no vector ALU work and need no cross-lane reduction.  Lane
// (key = lane % 16, kq = lane / 16) holds dims 32*ks + 8*kq + [0, 8) of its key for ks = 0..3:
// the rotation partner of dim d (d + 64) is the same lane's ks + 2 piece.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));

template <typename T>
struct Mma16;
template <>
struct Mma16<__hip_bfloat16> {
    __device__ static f32x4 mma(uint4 a, uint4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                       0, 0, 0);
    }
    __device__ static float lo(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    __device__ static uint32_t pack2(float a, float b) {
        f32x2_t f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
    }
    // 16x16x16: four 16-bit values per lane and operand
    __device__ static f32x4 mma_k16(uint2 a, uint2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c, 0,
                                                         0, 0);
    }
};
template <>
struct Mma16<__half> {
    __device__ static f32x4 mma(uint4 a, uint4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                      0, 0);
    }
    __device__ static float lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[0]; }
    __device__ static float hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[1]; }
    __device__ static uint32_t pack2(float a, float b) {
        f32x2_t f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2_t));
    }
    __device__ static f32x4 mma_k16(uint2 a, uint2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
};

// cos / sin of the two rotation pairs a word covers, at the given angles
template <typename T>
__device__ inline RopeWord<T> rope_word_at(float angle0, float angle1) {
    float s0, c0, s1, c1;
    fast_sincos(angle0, &s0, &c0);
    fast_sincos(angle1, &s1, &c1);
    return RopeWord<T>::make(c0, s0, c1, s1);
}

template <typename T, int G>
__global__ void __launch_bounds__(256, 2) decode_main_mfma_kernel(DecodeParams p) {
    extern __shared__ __align__(16) float red[];  // [16][G][128] partials, [16][G] max, [16][G] sum, [4][32][8] logits
    float* red_o = red;
    float* red_m = red + 16 * G * kD;
    float* red_l = red_m + 16 * G;
    float* s_lds = red_l + 16 * G;
    using Raw = typename Piece<T>::Raw;
    const ckv_attn_args& a = p.a;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int kg = lane >> 4, j = lane & 15;  // phase 2: key within a step, piece index inside the row
    const int grp = wave * 4 + kg;
    const int key16 = lane & 15, kq = lane >> 4;  // phase 1: MFMA column (key) and k-quarter
    const int64_t tile = blockIdx.x;
    const int64_t nbh = a.B * a.KVH;
    const int64_t n_wave = tile * kTK + wave * 32;  // first key of this wavefront
    float* s_wave = s_lds + wave * 32 * 8;

    // phase-1 keys of this lane: n_wave + 16*gi + key16; their source row offset (shared by every
    // (b, kvh) up to the segment base), visibility and rotation factors
    int64_t koff1[2];
    int seg1[2];
    bool vis1[2];
    RopeWord<T> rw[2][2][4];  // [key of this lane][ks][word]
#pragma unroll
    for (int gi = 0; gi < 2; gi++) {
        const int64_t n = n_wave + 16 * gi + key16;
        const int64_t NS = a.num_sink, S = a.S;
        int64_t pos = 0;
        seg1[gi] = 0;
        koff1[gi] = 0;
        vis1[gi] = false;
        if (n < NS) {
            seg1[gi] = 0; koff1[gi] = n * a.sink_stride[2]; vis1[gi] = a.sink_mask[n] == 0;
            if (p.shared_pos) pos = a.sink_pos[n];
        } else if (n < NS + S) {
            seg1[gi] = 1; koff1[gi] = (n - NS) * a.cache_stride[2]; vis1[gi] = a.mask[n - NS] == 0;
            if (p.shared_pos) pos = a.pos[n - NS] + a.pos_shift;
        } else if (n < p.N) {
            seg1[gi] = 2; koff1[gi] = 0; vis1[gi] = true;
            pos = a.q_pos[0];
        }
        if (p.shared_pos) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const int f = 32 * ks + 8 * kq + 2 * w;
                    const float f0 = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                    const float f1 = a.inv_freq ? a.inv_freq[f + 1] : 1.0f / powf(a.rope_theta, (float)(2 * f + 2) / (float)kD);
                    rw[gi][ks][w] = rope_word_at<T>(__fmul_rn((float)pos, f0), __fmul_rn((float)pos, f1));
                }
        }
    }
    // phase-2 keys of this lane: n_wave + 4*s + kg
    int64_t koff2[kSteps];
    int seg2[kSteps];
    bool vis2[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; s++) {
        const int64_t n = n_wave + 4 * s + kg;
        const int64_t NS = a.num_sink, S = a.S;
        seg2[s] = 0; koff2[s] = 0; vis2[s] = false;
        if (n < NS) { seg2[s] = 0; koff2[s] = n * a.sink_stride[2]; vis2[s] = a.sink_mask[n] == 0; }
        else if (n < NS + S) { seg2[s] = 1; koff2[s] = (n - NS) * a.cache_stride[2]; vis2[s] = a.mask[n - NS] == 0; }
        else if (n < p.N) { seg2[s] = 2; koff2[s] = 0; vis2[s] = true; }
    }

    for (int64_t bh = blockIdx.y; bh < nbh; bh += gridDim.y) {
        const int64_t b = bh / a.KVH, kvh = bh % a.KVH;
        const T* kseg[3] = {(const T*)a.sink_k + b * a.sink_stride[0] + kvh * a.sink_stride[1],
                            (const T*)a.cache_k + b * a.cache_stride[0] + kvh * a.cache_stride[1],
                            (const T*)a.k_new + b * a.kv_new_stride[0] + kvh * a.kv_new_stride[1]};
        const T* vseg[3] = {(const T*)a.sink_v + b * a.sink_stride[0] + kvh * a.sink_stride[1],
                            (const T*)a.cache_v + b * a.cache_stride[0] + kvh * a.cache_stride[1],
                            (const T*)a.v_new + b * a.kv_new_stride[0] + kvh * a.kv_new_stride[1]};
        // ---- issue every row read of this (b, kvh) up front
        uint4 kraw[2][4];
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const T* kp = kseg[seg1[gi]] + koff1[gi];
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
                kraw[gi][ks] = vis1[gi] ? *reinterpret_cast<const uint4*>(kp + 32 * ks + 8 * kq) : make_uint4(0, 0, 0, 0);
        }
        Raw vraw[kSteps][2];
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            if (vis2[s]) {
                const T* vp = vseg[seg2[s]] + koff2[s];
                vraw[s][0] = *reinterpret_cast<const Raw*>(vp + 4 * j);
                vraw[s][1] = *reinterpret_cast<const Raw*>(vp + 64 + 4 * j);
            }
        }
        // A operand: rotated queries of the group's heads (rows >= G are zero)
        uint4 qop[4];
        {
            const T* qr = (const T*)p.qrot_t + ((b * a.H) + kvh * G + key16) * kD;
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
                qop[ks] = key16 < G ? *reinterpret_cast<const uint4*>(qr + 32 * ks + 8 * kq) : make_uint4(0, 0, 0, 0);
        }
        // ---- phase 1: rotate K in registers, logits by MFMA, share them through LDS
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            if (!p.shared_pos && vis1[gi]) {
                const int64_t n = n_wave + 16 * gi + key16;
                int64_t pos;
                if (seg1[gi] == 0) pos = a.sink_pos[b * a.sink_pos_stride[0] + kvh * a.sink_pos_stride[1] + n];
                else if (seg1[gi] == 1)
                    pos = a.pos[b * a.pos_stride[0] + kvh * a.pos_stride[1] + (n - a.num_sink)] + a.pos_shift;
                else pos = a.q_pos[0];
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        const int f = 32 * ks + 8 * kq + 2 * w;
                        const float f0 = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                        const float f1 = a.inv_freq ? a.inv_freq[f + 1] : 1.0f / powf(a.rope_theta, (float)(2 * f + 2) / (float)kD);
                        rw[gi][ks][w] = rope_word_at<T>(__fmul_rn((float)pos, f0), __fmul_rn((float)pos, f1));
                    }
            }
            uint4 kop[4];
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&kraw[gi][ks]);
                const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&kraw[gi][ks + 2]);
                uint32_t o1[4], o2[4];
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    rw[gi][ks][w].rotate(w1[w], w2[w], p.key_scale, true, o1[w], o2[w]);
                }
                kop[ks] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
                kop[ks + 2] = make_uint4(o2[0], o2[1], o2[2], o2[3]);
            }
            f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ks++) sacc = Mma16<T>::mma(qop[ks], kop[ks], sacc);
            // lane holds heads 4*kq + v of key (16*gi + key16)
            const int64_t n = n_wave + 16 * gi + key16;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int g = 4 * kq + v;
                if (g < G) {
                    const float sv = vis1[gi] ? sacc[v] * p.scale_log2 : -INFINITY;
                    s_wave[(16 * gi + key16) * 8 + g] = sv;
                    if (n < p.N) p.logits[((b * a.KVH + kvh) * p.N + n) * G + g] = sv;
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS writes are done
        __builtin_amdgcn_wave_barrier();
        // ---- phase 2: softmax partial of each 16-lane group and its weighted V sum
        float sreg[kSteps][G];
#pragma unroll
        for (int s = 0; s < kSteps; s++)
#pragma unroll
            for (int g = 0; g < G; g++) sreg[s][g] = s_wave[(4 * s + kg) * 8 + g];
        float mg[G], lgp[G], o[G][8];
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m = sreg[0][g];
#pragma unroll
            for (int s = 1; s < kSteps; s++) m = fmaxf(m, sreg[s][g]);
            mg[g] = m;
            lgp[g] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) o[g][e] = 0.f;
        }
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            if (!vis2[s]) continue;
            float va[4], vb[4];
            Piece<T>::unpack(vraw[s][0], va);
            Piece<T>::unpack(vraw[s][1], vb);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float pe = __builtin_amdgcn_exp2f(sreg[s][g] - mg[g]);  // mg is finite: the key is visible
                lgp[g] += pe;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o[g][e] = fmaf(pe, va[e], o[g][e]);
                    o[g][4 + e] = fmaf(pe, vb[e], o[g][4 + e]);
                }
            }
        }
        // ---- combine the 16 groups of the workgroup
        __syncthreads();  // the previous (b, kvh) has been written out
        if (j == 0) {
#pragma unroll
            for (int g = 0; g < G; g++) red_m[grp * G + g] = mg[g];
        }
        __syncthreads();
        float mt[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m = red_m[g];
#pragma unroll
            for (int r = 1; r < 16; r++) m = fmaxf(m, red_m[r * G + g]);
            mt[g] = m;
            const float sc = mg[g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mg[g] - m);
            if (j == 0) red_l[grp * G + g] = lgp[g] * sc;
            float* ro = red_o + (grp * G + g) * kD;
            *reinterpret_cast<float4*>(ro + 4 * j) = make_float4(o[g][0] * sc, o[g][1] * sc, o[g][2] * sc, o[g][3] * sc);
            *reinterpret_cast<float4*>(ro + 64 + 4 * j) =
                make_float4(o[g][4] * sc, o[g][5] * sc, o[g][6] * sc, o[g][7] * sc);
        }
        __syncthreads();
        for (int i = tid; i < G * kD; i += 256) {
            const int g = i / kD, d = i % kD;
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) acc += red_o[(r * G + g) * kD + d];
            p.part_o[(((b * a.H) + kvh * G + g) * p.tiles + tile) * kD + d] = acc;
        }
        if (tid < G) {
            float l = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) l += red_l[r * G + tid];
            float* ml = p.part_ml + (((b * a.H) + kvh * G + tid) * p.tiles + tile) * 2;
            ml[0] = mt[tid];
            ml[1] = l;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Streaming variant of the main kernel (16-bit caches, shared positions, G <= 4).
//
// The (64-key tile, batch x kv-head) items are dealt out in equal contiguous runs over as many
// workgroups as the chip holds at once (two per CU), so the launch has no tail.  A workgroup is four
// wavefronts; each stages 16 key rows of an item.  The rows travel global -> LDS as asynchronous
// copies one item ahead (two LDS stages), swizzled on the way by the choice of each lane's source
// piece, so no register holds data in flight and the loads of the next item overlap the arithmetic
// of this one.  Per item: (1) every wavefront rotates its 16 K rows in registers (cos / sin of the
// tile's positions stay in registers for all (b, kvh) of the tile) and gets their logits from the
// matrix pipe; (2) after the item's only workgroup barrier every wavefront normalises all 64 logits
// of each head (redundantly: 4 values per lane) and (3) multiplies P by a 32-dim slice of all 64 V
// rows on the matrix pipe, so the tile's partial result is complete in registers and needs no
// combination across wavefronts.  It is written out at the top of the next item, off the critical
// path.
// ---------------------------------------------------------------------------------------------
constexpr int kStreamThreads = 64 * kStreamWaves;
constexpr int kStreamWgPerCu = 8 / kStreamWaves;  // eight wavefronts per CU
constexpr int kStreamDimBlocks = 8 / kStreamWaves;  // 16-dim blocks of the output a wavefront owns
constexpr int kStreamStage = 2 * kSK * 256;       // K rows then V rows of one tile (16-bit, 256 B per row)
// two stages | two 1 KiB query blocks | two [4 heads][kSK keys] logit planes | per wavefront [4][kSK] probabilities
constexpr int kStreamQ = 2 * kStreamStage, kStreamS = kStreamQ + 2 * 1024, kStreamP = kStreamS + 2 * 4 * kSK * 4;
constexpr int kStreamPPitch = kSK * 2 + 32;        // bytes per head row of the probabilities: the pad puts the four heads on different banks
constexpr int kStreamLds = kStreamP + kStreamWaves * 4 * kStreamPPitch;

// sum / max over the four 16-lane rows of a wavefront (lanes l, l^16, l^32, l^48)
__device__ inline float rows4_sum(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    const auto q = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}
__device__ inline float rows4_max(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const auto q = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
}
// all-reduce over lanes l, l+4, l+8, l+12 of every 16-lane row, then over the four rows: the 16 lanes with equal l % 4
__device__ inline float mod4_max(float m) {
    m = fmaxf(m, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(m), 0x124, 0xF, 0xF, true)));  // row_ror:4
    m = fmaxf(m, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(m), 0x128, 0xF, 0xF, true)));  // row_ror:8
    return rows4_max(m);
}
__device__ inline float mod4_sum(float l) {
    l += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(l), 0x124, 0xF, 0xF, true));
    l += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(l), 0x128, 0xF, 0xF, true));
    return rows4_sum(l);
}

// the byte offsets of the rows inside a (b, kvh) slab must fit the 32-bit lane offsets of the copies
inline bool stream_offsets_fit(const ckv_attn_args& a) {
    const int64_t lim = (int64_t)1 << 31, es = 2;
    return a.S * a.cache_stride[2] * es + 256 < lim && a.num_sink * a.sink_stride[2] * es + 256 < lim;
}

constexpr int kStreamMaxWgs = 1024;  // the result chunks are sized for at most this many workgroups
constexpr int kStreamProbWave = 1;  // the wavefront that stores the tile's probabilities (wavefront 0 stores maximum and sum)
static_assert(kSK / 16 == 8, "a lane's probabilities of a tile are stored as one 16-byte piece");

template <typename T, int G>
__global__ void __launch_bounds__(kStreamThreads, kStreamWgPerCu) decode_stream_kernel(DecodeParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t lds_base = lds_address(smem);
    const ckv_attn_args& a = p.a;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int key16 = lane & 15, kq = lane >> 4;  // logits: MFMA column (key) and k-quarter
    const int pg = lane & 3, kgrp = lane >> 2;    // softmax: head and group of kKpl keys
    constexpr int kKpl = kSK / 16, kDb = kStreamDimBlocks;
    const int64_t nbh = a.B * a.KVH, total = (int64_t)p.n_vis * nbh;
    const int64_t item0 = total * blockIdx.x / gridDim.x, item1 = total * (blockIdx.x + 1) / gridDim.x;
    const int64_t NS = a.num_sink, S = a.S;
    const int KVH = (int)a.KVH;
    constexpr int kEs = (int)sizeof(T);

    // LDS offsets inside a stage.  K row r keeps source piece c at slot c ^ (r & 15), which makes the
    // 16-byte operand reads conflict free.  V row r keeps piece c at slot c ^ ((r & 7) << 1): the
    // transposing reads below take 32 bytes from each of four rows, and this puts the rows on
    // different banks.
    int kaddr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) kaddr[ks] = (wave * 16 + key16) * 256 + (((4 * ks + kq) ^ key16) << 4);
    // P.V on the matrix pipe, 16x16x16: A = V^T block (16 dims x 16 keys), B = P^T (16 keys x 16 heads).
    // ds_read_b64_tr_b16 hands lane i of a 16-lane group element [4e + i/4][i%4] (e = 0..3) of the
    // 16 x 4 matrix whose row r is the 8 bytes lane r points at.  With lane r of group q pointing at
    // dims 16 blk + 4 (r%4) .. +3 of key 4q + r/4, lane i receives dim 16 blk + i of keys 4q .. 4q+3:
    // the A operand.  This wavefront owns kDb blocks of 16 dims (blk = kDb wave ..); the keys of
    // contraction step ks are 16 rows further per step.
    int vt_addr[kDb];
    {
        const int r_l = lane & 15, key = 4 * (lane >> 4) + (r_l >> 2);
#pragma unroll
        for (int b2 = 0; b2 < kDb; b2++) {
            vt_addr[b2] = kSK * 256 + key * 256 + 32 * ((kDb * wave + b2) ^ (key & 7)) + 16 * ((r_l & 3) >> 1) + 8 * (r_l & 1);
        }
    }
    // query block of an item: head g at g * 256, its 16-byte piece c in slot c ^ g (the heads' rows would
    // otherwise sit on the same banks); lanes of idle MFMA rows read head 0 (their results are not used)
    const int q_row = key16 < G ? key16 : 0;
    const int q_off = kStreamQ + q_row * 256 + ((kq ^ q_row) << 4);
    float* s_all = reinterpret_cast<float*>(smem + kStreamS);                                   // [2][4][kSK]
    unsigned char* p_wave = smem + kStreamP + wave * (4 * kStreamPPitch);                       // [4][kSK] 16-bit, padded rows

    for (int64_t item = item0; item < item1;) {
        const int64_t jt = item / nbh, bh0 = item % nbh;  // jt: the tile's rank among the visible ones
        const int64_t tile = stream_tile_of(p, (int)jt);
        const int64_t bh1 = (jt + 1) * nbh > item1 ? item1 - jt * nbh : nbh;
        item = jt * nbh + bh1;
        const int64_t n_wave = tile * kSK + wave * 16;  // first key of this wavefront

        // ---- per-tile constants (the same for every (b, kvh): positions are shared)
        bool vis1 = false;
        RopeWord<T> rw[2][4];  // [ks][word]: dims 32 ks + 8 kq + 2 w, + 1 and their partners 64 further
        {
            const int64_t n = n_wave + key16;
            int64_t pos = 0;
            if (n < NS) { vis1 = a.sink_mask[n] == 0; pos = a.sink_pos[n]; }
            else if (n < NS + S) { vis1 = a.mask[n - NS] == 0; pos = a.pos[n - NS] + a.pos_shift; }
            else if (n < p.N) { vis1 = true; pos = a.q_pos[0]; }
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const int f = 32 * ks + 8 * kq + 2 * w;
                    const float f0 = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                    const float f1 = a.inv_freq ? a.inv_freq[f + 1] : 1.0f / powf(a.rope_theta, (float)(2 * f + 2) / (float)kD);
                    rw[ks][w] = rope_word_at<T>(__fmul_rn((float)pos, f0), __fmul_rn((float)pos, f1));
                }
        }
        // Rows of hidden slots may hold anything (their probability is zero, but 0 * NaN is not), so
        // they are zeroed on the way into the P.V product: masks of this lane's operand keys
        // 16 ks + 4 kq .. + 3, two 16-bit values per word.
        uint32_t m01[kKpl], m23[kKpl];
#pragma unroll
        for (int half = 0; half < kSK / 64; half++) {
            const int64_t n = tile * kSK + 64 * half + lane;
            bool v = false;
            if (n < NS) v = a.sink_mask[n] == 0;
            else if (n < NS + S) v = a.mask[n - NS] == 0;
            else if (n < p.N) v = true;
            const unsigned long long vis64 = __builtin_amdgcn_ballot_w64(v);
#pragma unroll
            for (int k4 = 0; k4 < 4; k4++) {
                const int ks = 4 * half + k4;
                const uint32_t vk = (uint32_t)(vis64 >> (16 * k4 + 4 * kq)) & 0xfu;
                m01[ks] = ((vk & 1u) ? 0x0000ffffu : 0u) | ((vk & 2u) ? 0xffff0000u : 0u);
                m23[ks] = ((vk & 4u) ? 0x0000ffffu : 0u) | ((vk & 8u) ? 0xffff0000u : 0u);
            }
        }
        // Copies: block jb of a wavefront brings rows 4 jb .. 4 jb + 3 of its 16 (1 KiB: lane i lands at
        // +16 i, i.e. row 4 jb + i / 16, slot i % 16, and fetches the source piece that belongs there).
        // seg: 0 sink, 1 cache, 2 the new token (rows past the end repeat it and stay hidden).
        int seg_c[4];
        uint32_t relk[4], relv[4];  // byte offsets inside the (b, kvh) slab of the row's segment
        bool cache_only[4];         // every row of the block is a cache slot: one copy with the slab as base
#pragma unroll
        for (int jb = 0; jb < 4; jb++) {
            const int r = 4 * jb + (lane >> 4);
            const int64_t n = n_wave + r;
            int64_t row_off;
            if (n < NS) { seg_c[jb] = 0; row_off = n * a.sink_stride[2]; }
            else if (n < NS + S) { seg_c[jb] = 1; row_off = (n - NS) * a.cache_stride[2]; }
            else { seg_c[jb] = 2; row_off = 0; }
            relk[jb] = (uint32_t)(row_off * kEs) + ((((uint32_t)lane & 15u) ^ ((uint32_t)r & 15u)) << 4);
            relv[jb] = (uint32_t)(row_off * kEs) + ((((uint32_t)lane & 15u) ^ (((uint32_t)r & 7u) << 1)) << 4);
            cache_only[jb] = __builtin_amdgcn_ballot_w64(seg_c[jb] == 1) == ~0ull;
        }
        // slab pointers of (b, kvh)
        auto slabs = [&](int b, int kvh, const char* (&kb)[3], const char* (&vb)[3]) {
            const int64_t o0 = ((int64_t)b * a.sink_stride[0] + (int64_t)kvh * a.sink_stride[1]) * kEs;
            const int64_t o1 = ((int64_t)b * a.cache_stride[0] + (int64_t)kvh * a.cache_stride[1]) * kEs;
            const int64_t o2 = ((int64_t)b * a.kv_new_stride[0] + (int64_t)kvh * a.kv_new_stride[1]) * kEs;
            kb[0] = (const char*)a.sink_k + o0; vb[0] = (const char*)a.sink_v + o0;
            kb[1] = (const char*)a.cache_k + o1; vb[1] = (const char*)a.cache_v + o1;
            kb[2] = (const char*)a.k_new + o2; vb[2] = (const char*)a.v_new + o2;
        };
        // four copies, at least one per block whatever the segments (the waits below count on that)
        auto copy_rows = [&](const char* (&base)[3], const uint32_t(&rel)[4], uint32_t dst) {
#pragma unroll
            for (int jb = 0; jb < 4; jb++) {
                if (cache_only[jb]) {
                    async_copy16(base[1], rel[jb], dst + jb * 1024);
                } else {
#pragma unroll
                    for (int sgm = 0; sgm < 3; sgm++)
                        if (seg_c[jb] == sgm) async_copy16(base[sgm], rel[jb], dst + jb * 1024);
                }
            }
        };
        // the query block of (b, kvh) into stage `st` (one per workgroup, copied by wavefront 0: lane i fills slot
        // i % 16 of head i / 16 with the piece that belongs there), then this wavefront's K rows.  The query copy
        // goes first: whoever waits for the four K copies behind it has waited for it too, and the item's barrier
        // makes it visible to the other wavefronts.
        auto copy_kq = [&](int b, int kvh, int st) {
            if (wave == 0) {
                const char* qsrc = (const char*)p.qrot_t + ((int64_t)b * a.H + (int64_t)kvh * G) * (kD * kEs);
                if ((lane >> 4) < G)
                    async_copy16(qsrc, (lane >> 4) * 256 + (((lane & 15) ^ (lane >> 4)) << 4), lds_base + kStreamQ + st * 1024);
            }
            const char *kb[3], *vb[3];
            slabs(b, kvh, kb, vb);
            copy_rows(kb, relk, lds_base + st * kStreamStage + wave * 4096);
        };
        // V rows: four copies
        auto copy_v = [&](int b, int kvh, int st) {
            const char *kb[3], *vb[3];
            slabs(b, kvh, kb, vb);
            copy_rows(vb, relv, lds_base + st * kStreamStage + kSK * 256 + wave * 4096);
        };

        int b = (int)(bh0 / KVH), kvh = (int)(bh0 % KVH);
        // results of the previous item, stored at the top of the next one
        bool pending = false;
        int pend_b = 0, pend_kvh = 0;
        uint2 pend_o[kDb];  // the tile's weighted V average (sum / l) of this lane's four dims, in the tensor dtype
        float pend_m = 0.f, pend_l = 0.f;
        uint4 pend_e = make_uint4(0u, 0u, 0u, 0u);  // the storing wavefront's probabilities: head pg, keys kKpl kgrp ..
#pragma unroll
        for (int b2 = 0; b2 < kDb; b2++) pend_o[b2] = make_uint2(0u, 0u);
        // Stores share the counter of the copies and retire in order with them.  All stores of an item are
        // issued together, right after the copies of the next item's K rows; every wavefront issues kDb
        // of them (two wavefronts one more each), and none before the first item of a run has results.
        auto flush = [&]() {
            if (!pending) return;
            const int64_t pend_item = jt * nbh + (int64_t)pend_b * KVH + pend_kvh;
            const int64_t chunk_i = (pend_item - item0) * gridDim.x + blockIdx.x;
            unsigned char* chunk = p.chunks + chunk_i * (G * (kSK + kD) * 2);
            if (wave == kStreamProbWave && pg < G)  // every wavefront holds all of them: one stores, 16 bytes a lane
                *reinterpret_cast<uint4*>(chunk + (pg * kSK + kKpl * kgrp) * 2) = pend_e;
            if (key16 < G) {
#pragma unroll
                for (int b2 = 0; b2 < kDb; b2++)
                    *reinterpret_cast<uint2*>(chunk + (G * kSK + key16 * kD + 16 * (kDb * wave + b2) + 4 * kq) * 2) = pend_o[b2];
            }
            if (wave == 0 && kgrp == 0 && pg < G)  // maximum and sum: G pairs per chunk, in chunk order
                *reinterpret_cast<float2*>(p.part_ml + (chunk_i * G + pg) * 2) = make_float2(pend_m, pend_l);
        };

        // Loads and stores retire in issue order, so "at most n operations outstanding" with n younger
        // ones issued after the wanted copies means the wanted ones are done.  Per item the order is
        // [wavefront 0: the query block of the next item,] K rows of the next item (4), stores of the previous
        // one (kDb and up, once there is one), V rows of the next item (4).
        copy_kq(b, kvh, 0);
        copy_v(b, kvh, 0);
        // the first query block of the run must have landed for every wavefront (younger: the four V copies)
        __builtin_amdgcn_s_waitcnt(0x0F74);
        __builtin_amdgcn_s_barrier();
        int st = 0;
        // stores this wavefront issued in the latest flush(): kDb partial averages, the probabilities
        // from one wavefront, maximum and sum from another
        const int my_stores = kDb + (wave == kStreamProbWave ? 1 : 0) + (wave == 0 ? 1 : 0);
        int stored = 0;
        auto wait_copies = [&](int younger, bool lds_too) {  // vmcnt(younger) [, lgkmcnt(0)]: the count is an immediate
            if (lds_too) {
                switch (younger) {
                    case 4: __builtin_amdgcn_s_waitcnt(0x0074); break;
                    case 5: __builtin_amdgcn_s_waitcnt(0x0075); break;
                    case 6: __builtin_amdgcn_s_waitcnt(0x0076); break;
                    case 7: __builtin_amdgcn_s_waitcnt(0x0077); break;
                    case 8: __builtin_amdgcn_s_waitcnt(0x0078); break;
                    default: __builtin_amdgcn_s_waitcnt(0x0070); break;
                }
            } else {
                switch (younger) {
                    case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
                    case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
                    case 6: __builtin_amdgcn_s_waitcnt(0x0F76); break;
                    case 7: __builtin_amdgcn_s_waitcnt(0x0F77); break;
                    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
                }
            }
        };
        static_assert(kDb <= 2, "wait_copies covers up to kDb + 2 stores");
        for (int64_t bh = bh0; bh < bh1; bh++) {
            int b_nx = b, kvh_nx = kvh;
            if (bh + 1 < bh1) {  // the last item of a run copies itself again: cheaper than a different path
                kvh_nx = kvh + 1 == KVH ? 0 : kvh + 1;
                b_nx = kvh + 1 == KVH ? b + 1 : b;
            }
            // this wavefront's K rows of the item are in LDS (younger: the stores issued after them and the four V
            // copies of this item); the item's query block was complete before the previous barrier
            wait_copies(4 + stored, false);
            copy_kq(b_nx, kvh_nx, st ^ 1);
            stored = pending ? my_stores : 0;
            flush();
            const unsigned char* stage = smem + st * kStreamStage;

            // ---- rotate K in registers, logits by MFMA, shared through LDS
            {
                uint4 kraw[4], qop[4];
#pragma unroll
                for (int ks = 0; ks < 4; ks++) kraw[ks] = *reinterpret_cast<const uint4*>(stage + kaddr[ks]);
#pragma unroll
                for (int ks = 0; ks < 4; ks++) qop[ks] = *reinterpret_cast<const uint4*>(smem + q_off + st * 1024 + ks * 64);
                uint4 kop[4];
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&kraw[ks]);
                    const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&kraw[ks + 2]);
                    uint32_t o1[4], o2[4];
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        rw[ks][w].rotate(w1[w], w2[w], p.key_scale, true, o1[w], o2[w]);
                    }
                    kop[ks] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
                    kop[ks + 2] = make_uint4(o2[0], o2[1], o2[2], o2[3]);
                }
                f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 4; ks++) sacc = Mma16<T>::mma(qop[ks], kop[ks], sacc);
                // lane holds heads 4 kq + v of key key16: with G <= 4 only the lanes of kq == 0 hold heads
                if (kq == 0) {
#pragma unroll
                    for (int v = 0; v < G; v++)
                        s_all[(st * 4 + v) * kSK + wave * 16 + key16] = vis1 ? sacc[v] * p.scale_log2 : -INFINITY;
                }
            }
            // this wavefront's V rows of the item and (wavefront 0) the next query block have landed (younger: the
            // four K copies of the next item and the stores of flush()); its logits are in LDS
            wait_copies(4 + stored, true);
            __builtin_amdgcn_s_barrier();
            // every wavefront is past the previous item: its V stage can be refilled
            copy_v(b_nx, kvh_nx, st ^ 1);

            // ---- softmax over the tile's keys, done by every wavefront: lane = (head, kKpl keys)
            float m_t, l_t;
            uint4 e_half = make_uint4(0u, 0u, 0u, 0u);
            {
                float x[kKpl];
#pragma unroll
                for (int e = 0; e < kKpl; e += 4) {
                    float4 x4 = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
                    if (pg < G) x4 = *reinterpret_cast<const float4*>(s_all + (st * 4 + pg) * kSK + kKpl * kgrp + e);
                    x[e] = x4.x; x[e + 1] = x4.y; x[e + 2] = x4.z; x[e + 3] = x4.w;
                }
                float mloc = x[0];
#pragma unroll
                for (int e = 1; e < kKpl; e++) mloc = fmaxf(mloc, x[e]);
                const float m = mod4_max(mloc);
                const float ms = m == -INFINITY ? 0.f : m;
                float lloc = 0.f;
#pragma unroll
                for (int e = 0; e < kKpl; e += 4) {
                    const float e0 = __builtin_amdgcn_exp2f(x[e] - ms), e1 = __builtin_amdgcn_exp2f(x[e + 1] - ms);
                    const float e2 = __builtin_amdgcn_exp2f(x[e + 2] - ms), e3 = __builtin_amdgcn_exp2f(x[e + 3] - ms);
                    lloc += (e0 + e1) + (e2 + e3);
                    // probabilities in the tensor dtype, [head][kSK keys] (hidden keys and idle lanes: 0)
                    const uint2 pk = make_uint2(Mma16<T>::pack2(e0, e1), Mma16<T>::pack2(e2, e3));
                    *reinterpret_cast<uint2*>(p_wave + pg * kStreamPPitch + (kKpl * kgrp + e) * 2) = pk;
                    // the copy that goes to memory for the score kernel is fp16 whatever the tensor dtype
                    uint2 hk = pk;
                    if constexpr (!std::is_same<T, __half>::value) {
                        if (wave == kStreamProbWave) hk = make_uint2(Mma16<__half>::pack2(e0, e1), Mma16<__half>::pack2(e2, e3));
                    }
                    if (e == 0) { e_half.x = hk.x; e_half.y = hk.y; } else { e_half.z = hk.x; e_half.w = hk.y; }
                }
                m_t = m;
                l_t = mod4_sum(lloc);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
            __builtin_amdgcn_wave_barrier();
            // ---- weighted V sum on the matrix pipe: this wavefront's dims over all keys of the tile.  Lane
            //      16 q + g (g < G) ends up with dims 16 (kDb wave + b2) + 4 q .. + 3 of head g.
            f32x4 acc[kDb];
#pragma unroll
            for (int b2 = 0; b2 < kDb; b2++) acc[b2] = f32x4{0.f, 0.f, 0.f, 0.f};
            {
                const uint32_t vbase = lds_base + st * kStreamStage;
#pragma unroll
                for (int ks = 0; ks < kKpl; ks++) {
                    uint2 pb = make_uint2(0u, 0u);
                    if (key16 < G) pb = *reinterpret_cast<const uint2*>(p_wave + key16 * kStreamPPitch + ks * 32 + kq * 8);
#pragma unroll
                    for (int b2 = 0; b2 < kDb; b2++) {
                        const s16x4_t va = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) s16x4_t*)(uintptr_t)(vbase + vt_addr[b2] + ks * 4096));
                        uint2 av = __builtin_bit_cast(uint2, va);
                        av.x &= m01[ks];
                        av.y &= m23[ks];
                        acc[b2] = Mma16<T>::mma_k16(av, pb, acc[b2]);
                    }
                }
            }
            {
                // lanes 16 q + g hold head g, and g == pg there: l_t is that head's sum (0: the tile is hidden)
                const float inv_l = l_t > 0.f ? 1.0f / l_t : 0.f;
#pragma unroll
                for (int b2 = 0; b2 < kDb; b2++)
                    pend_o[b2] = make_uint2(Mma16<T>::pack2(acc[b2][0] * inv_l, acc[b2][1] * inv_l),
                                            Mma16<T>::pack2(acc[b2][2] * inv_l, acc[b2][3] * inv_l));
            }
            pend_m = m_t;
            pend_l = l_t;
            pend_e = e_half;
            pending = true;
            pend_b = b;
            pend_kvh = kvh;
            b = b_nx;
            kvh = kvh_nx;
            st ^= 1;
        }
        flush();
        // the repeated copies of the last item must land, and every wavefront be done with the stages,
        // before the next run of items refills them
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __builtin_amdgcn_s_barrier();
    }
}

// ---------------------------------------------------------------------------------------------
// The streaming kernel for 5 to 8 query heads per kv head (Qwen2-7B has 7).  The item stream, the row copies,
// the waits and the result chunks are those of the kernel above; what differs: the query block of an item
// (8 heads x 256 bytes) is one per workgroup and stage, copied by wavefronts 0 and 1 one item ahead and made
// visible by that item's barrier; the logits of 8 heads go through LDS; and every wavefront normalises them
// directly in the layout of the P.V operand (lane = (head, quarter) holds 32 keys of its head), so the
// probabilities never go through LDS.  Wavefront w stores the 16 keys 16 w .. of every head's probabilities.
// ---------------------------------------------------------------------------------------------
constexpr int kWideQ = 2 * kStreamStage;            // two query blocks [8 heads][256 bytes]
constexpr int kWideS = kWideQ + 2 * 2048;           // two [8 heads] logit planes, rows of kWidePitch floats
constexpr int kWidePitch = kSK + 16;                // the pad spreads the heads over the banks
constexpr int kWideLds = kWideS + 2 * 8 * kWidePitch * 4;

__device__ inline void wait_vm(int n, bool lds_too) {  // s_waitcnt vmcnt(n) [lgkmcnt(0)]: the count is an immediate
    if (lds_too) {
        switch (n) {
            case 4: __builtin_amdgcn_s_waitcnt(0x0074); break;
            case 5: __builtin_amdgcn_s_waitcnt(0x0075); break;
            case 6: __builtin_amdgcn_s_waitcnt(0x0076); break;
            case 7: __builtin_amdgcn_s_waitcnt(0x0077); break;
            default: __builtin_amdgcn_s_waitcnt(0x0070); break;
        }
    } else {
        switch (n) {
            case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
            case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
            case 6: __builtin_amdgcn_s_waitcnt(0x0F76); break;
            case 7: __builtin_amdgcn_s_waitcnt(0x0F77); break;
            default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
        }
    }
}

template <typename T, int G>
__global__ void __launch_bounds__(kStreamThreads, kStreamWgPerCu) decode_stream_wide_kernel(DecodeParams p) {
    static_assert(G > 4 && G <= 8, "the query block and the logit planes hold 8 heads");
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t lds_base = lds_address(smem);
    const ckv_attn_args& a = p.a;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int key16 = lane & 15, kq = lane >> 4;  // logits: MFMA column (key) and k-quarter; softmax and P.V: head and key quarter
    constexpr int kPv = kSK / 16, kDb = kStreamDimBlocks;   // contraction steps of 16 keys
    const int64_t nbh = a.B * a.KVH, total = (int64_t)p.n_vis * nbh;
    const int64_t item0 = total * blockIdx.x / gridDim.x, item1 = total * (blockIdx.x + 1) / gridDim.x;
    const int64_t NS = a.num_sink, S = a.S;
    const int KVH = (int)a.KVH;
    constexpr int kEs = (int)sizeof(T);

    int kaddr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) kaddr[ks] = (wave * 16 + key16) * 256 + (((4 * ks + kq) ^ key16) << 4);
    int vt_addr[kDb];
    {
        const int r_l = lane & 15, key = 4 * (lane >> 4) + (r_l >> 2);
#pragma unroll
        for (int b2 = 0; b2 < kDb; b2++) {
            vt_addr[b2] = kSK * 256 + key * 256 + 32 * ((kDb * wave + b2) ^ (key & 7)) + 16 * ((r_l & 3) >> 1) + 8 * (r_l & 1);
        }
    }
    // query operand: head row key16 (rows past G read head 0, their results are not used), 16-byte piece
    // 4 ks + kq kept in slot (4 ks + kq) ^ head
    const int q_row = key16 < G ? key16 : 0;
    int q_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) q_off[ks] = kWideQ + q_row * 256 + (((4 * ks + kq) ^ q_row) << 4);
    float* s_all = reinterpret_cast<float*>(smem + kWideS);  // [2][8][kWidePitch]
    const bool head_ok = key16 < G;

    for (int64_t item = item0; item < item1;) {
        const int64_t jt = item / nbh, bh0 = item % nbh;  // jt: the tile's rank among those with items
        const int64_t tile = stream_tile_of(p, (int)jt);
        const int64_t bh1 = (jt + 1) * nbh > item1 ? item1 - jt * nbh : nbh;
        item = jt * nbh + bh1;
        const int64_t n_wave = tile * kSK + wave * 16;  // first key of this wavefront

        // ---- per-tile constants (the same for every (b, kvh): positions are shared)
        bool vis1 = false;
        RopeWord<T> rw[2][4];  // [ks][word]: dims 32 ks + 8 kq + 2 w, + 1 and their partners 64 further
        {
            const int64_t n = n_wave + key16;
            int64_t pos = 0;
            if (n < NS) { vis1 = a.sink_mask[n] == 0; pos = a.sink_pos[n]; }
            else if (n < NS + S) { vis1 = a.mask[n - NS] == 0; pos = a.pos[n - NS] + a.pos_shift; }
            else if (n < p.N) { vis1 = true; pos = a.q_pos[0]; }
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const int f = 32 * ks + 8 * kq + 2 * w;
                    const float f0 = a.inv_freq ? a.inv_freq[f] : 1.0f / powf(a.rope_theta, (float)(2 * f) / (float)kD);
                    const float f1 = a.inv_freq ? a.inv_freq[f + 1] : 1.0f / powf(a.rope_theta, (float)(2 * f + 2) / (float)kD);
                    rw[ks][w] = rope_word_at<T>(__fmul_rn((float)pos, f0), __fmul_rn((float)pos, f1));
                }
        }
        // rows of hidden slots are zeroed on the way into the P.V product (0 * NaN): masks of this lane's
        // operand keys 16 ks + 4 kq .. + 3, two 16-bit values per word
        uint32_t m01[kPv], m23[kPv];
#pragma unroll
        for (int half = 0; half < kSK / 64; half++) {
            const int64_t n = tile * kSK + 64 * half + lane;
            bool v = false;
            if (n < NS) v = a.sink_mask[n] == 0;
            else if (n < NS + S) v = a.mask[n - NS] == 0;
            else if (n < p.N) v = true;
            const unsigned long long vis64 = __builtin_amdgcn_ballot_w64(v);
#pragma unroll
            for (int k4 = 0; k4 < 4; k4++) {
                const int ks = 4 * half + k4;
                const uint32_t vk = (uint32_t)(vis64 >> (16 * k4 + 4 * kq)) & 0xfu;
                m01[ks] = ((vk & 1u) ? 0x0000ffffu : 0u) | ((vk & 2u) ? 0xffff0000u : 0u);
                m23[ks] = ((vk & 4u) ? 0x0000ffffu : 0u) | ((vk & 8u) ? 0xffff0000u : 0u);
            }
        }
        // copies: block jb of a wavefront brings rows 4 jb .. 4 jb + 3 of its 16; seg: 0 sink, 1 cache, 2 the new token
        int seg_c[4];
        uint32_t relk[4], relv[4];
        bool cache_only[4];
#pragma unroll
        for (int jb = 0; jb < 4; jb++) {
            const int r = 4 * jb + (lane >> 4);
            const int64_t n = n_wave + r;
            int64_t row_off;
            if (n < NS) { seg_c[jb] = 0; row_off = n * a.sink_stride[2]; }
            else if (n < NS + S) { seg_c[jb] = 1; row_off = (n - NS) * a.cache_stride[2]; }
            else { seg_c[jb] = 2; row_off = 0; }
            relk[jb] = (uint32_t)(row_off * kEs) + ((((uint32_t)lane & 15u) ^ ((uint32_t)r & 15u)) << 4);
            relv[jb] = (uint32_t)(row_off * kEs) + ((((uint32_t)lane & 15u) ^ (((uint32_t)r & 7u) << 1)) << 4);
            cache_only[jb] = __builtin_amdgcn_ballot_w64(seg_c[jb] == 1) == ~0ull;
        }
        auto slabs = [&](int b, int kvh, const char* (&kb)[3], const char* (&vb)[3]) {
            const int64_t o0 = ((int64_t)b * a.sink_stride[0] + (int64_t)kvh * a.sink_stride[1]) * kEs;
            const int64_t o1 = ((int64_t)b * a.cache_stride[0] + (int64_t)kvh * a.cache_stride[1]) * kEs;
            const int64_t o2 = ((int64_t)b * a.kv_new_stride[0] + (int64_t)kvh * a.kv_new_stride[1]) * kEs;
            kb[0] = (const char*)a.sink_k + o0; vb[0] = (const char*)a.sink_v + o0;
            kb[1] = (const char*)a.cache_k + o1; vb[1] = (const char*)a.cache_v + o1;
            kb[2] = (const char*)a.k_new + o2; vb[2] = (const char*)a.v_new + o2;
        };
        auto copy_rows = [&](const char* (&base)[3], const uint32_t(&rel)[4], uint32_t dst) {  // four copies
#pragma unroll
            for (int jb = 0; jb < 4; jb++) {
                if (cache_only[jb]) {
                    async_copy16(base[1], rel[jb], dst + jb * 1024);
                } else {
#pragma unroll
                    for (int sgm = 0; sgm < 3; sgm++)
                        if (seg_c[jb] == sgm) async_copy16(base[sgm], rel[jb], dst + jb * 1024);
                }
            }
        };
        // the query block of (b, kvh) into stage `st` (wavefronts 0 and 1, four heads each: lane i fills slot
        // i % 16 of head 4 wave + i / 16 with the piece that belongs there), then this wavefront's K rows.  The
        // query copy goes first: whoever waits for the four K copies behind it has waited for it too.
        auto copy_kq = [&](int b, int kvh, int st) {
            if (wave < 2) {
                const char* qsrc = (const char*)p.qrot_t + ((int64_t)b * a.H + (int64_t)kvh * G) * (kD * kEs);
                const int h = 4 * wave + (lane >> 4);
                if (h < G) async_copy16(qsrc, h * 256 + (((lane & 15) ^ h) << 4), lds_base + kWideQ + st * 2048 + wave * 1024);
            }
            const char *kb[3], *vb[3];
            slabs(b, kvh, kb, vb);
            copy_rows(kb, relk, lds_base + st * kStreamStage + wave * 4096);
        };
        auto copy_v = [&](int b, int kvh, int st) {
            const char *kb[3], *vb[3];
            slabs(b, kvh, kb, vb);
            copy_rows(vb, relv, lds_base + st * kStreamStage + kSK * 256 + wave * 4096);
        };

        int b = (int)(bh0 / KVH), kvh = (int)(bh0 % KVH);
        // results of the previous item, stored at the top of the next one
        bool pending = false;
        int pend_b = 0, pend_kvh = 0;
        uint2 pend_o[kDb];
        float pend_m = 0.f, pend_l = 0.f;
        uint2 pend_e = make_uint2(0u, 0u);  // fp16 probabilities of head key16, keys 16 wave + 4 kq .. + 3
#pragma unroll
        for (int b2 = 0; b2 < kDb; b2++) pend_o[b2] = make_uint2(0u, 0u);
        auto flush = [&]() {
            if (!pending) return;
            const int64_t pend_item = jt * nbh + (int64_t)pend_b * KVH + pend_kvh;
            const int64_t chunk_i = (pend_item - item0) * gridDim.x + blockIdx.x;
            unsigned char* chunk = p.chunks + chunk_i * (G * (kSK + kD) * 2);
            if (head_ok) {
                *reinterpret_cast<uint2*>(chunk + (key16 * kSK + 16 * wave + 4 * kq) * 2) = pend_e;
#pragma unroll
                for (int b2 = 0; b2 < kDb; b2++)
                    *reinterpret_cast<uint2*>(chunk + (G * kSK + key16 * kD + 16 * (kDb * wave + b2) + 4 * kq) * 2) = pend_o[b2];
            }
            if (wave == 0 && kq == 0 && head_ok)  // maximum and sum: G pairs per chunk, in chunk order
                *reinterpret_cast<float2*>(p.part_ml + (chunk_i * G + key16) * 2) = make_float2(pend_m, pend_l);
        };
        // Per item a wavefront issues, in this order: [the query copy of the next item,] four K copies of the
        // next item, the stores of the previous item's results, and after the barrier four V copies of the next
        // item.  Loads and stores retire in issue order.
        const int my_stores = kDb + 1 + (wave == 0 ? 1 : 0);
        int stored = 0;
        copy_kq(b, kvh, 0);
        copy_v(b, kvh, 0);
        // the first query block of the run must have landed for every wavefront (younger: the four V copies)
        __builtin_amdgcn_s_waitcnt(0x0F74);
        __builtin_amdgcn_s_barrier();
        int st = 0;
        for (int64_t bh = bh0; bh < bh1; bh++) {
            int b_nx = b, kvh_nx = kvh;
            if (bh + 1 < bh1) {  // the last item of a run copies itself again: cheaper than a different path
                kvh_nx = kvh + 1 == KVH ? 0 : kvh + 1;
                b_nx = kvh + 1 == KVH ? b + 1 : b;
            }
            // this wavefront's K rows of the item are in LDS (younger: the stores issued after them and the four V
            // copies of this item); its query block was complete before the previous barrier
            wait_vm(4 + stored, false);
            copy_kq(b_nx, kvh_nx, st ^ 1);
            stored = pending ? my_stores : 0;
            flush();
            const unsigned char* stage = smem + st * kStreamStage;

            // ---- rotate K in registers, logits by MFMA, shared through LDS
            {
                uint4 kraw[4], qop[4];
#pragma unroll
                for (int ks = 0; ks < 4; ks++) kraw[ks] = *reinterpret_cast<const uint4*>(stage + kaddr[ks]);
#pragma unroll
                for (int ks = 0; ks < 4; ks++) qop[ks] = *reinterpret_cast<const uint4*>(smem + q_off[ks] + st * 2048);
                uint4 kop[4];
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&kraw[ks]);
                    const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&kraw[ks + 2]);
                    uint32_t o1[4], o2[4];
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        rw[ks][w].rotate(w1[w], w2[w], p.key_scale, true, o1[w], o2[w]);
                    }
                    kop[ks] = make_uint4(o1[0], o1[1], o1[2], o1[3]);
                    kop[ks + 2] = make_uint4(o2[0], o2[1], o2[2], o2[3]);
                }
                f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 4; ks++) sacc = Mma16<T>::mma(qop[ks], kop[ks], sacc);
                // lane holds heads 4 kq + v of key key16
                if (kq < 2) {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (4 * kq + v < G)
                            s_all[(st * 8 + 4 * kq + v) * kWidePitch + wave * 16 + key16] = vis1 ? sacc[v] * p.scale_log2 : -INFINITY;
                }
            }
            // this wavefront's V rows of the item and (wavefronts 0, 1) its part of the next query block have landed
            // (younger: the four K copies of the next item and the stores of flush()); its logits are in LDS
            wait_vm(4 + stored, true);
            __builtin_amdgcn_s_barrier();
            // every wavefront is past the previous item: its V stage can be refilled
            copy_v(b_nx, kvh_nx, st ^ 1);

            // ---- softmax of head key16 over the tile, by every wavefront, in the layout of the P.V operand:
            //      this lane holds keys 16 ks + 4 kq .. + 3 (ks = 0 .. 7); lanes l, l ^ 16, l ^ 32, l ^ 48 share a head
            float m_t, l_t;
            uint2 pb[kPv];
            uint2 e_mine = make_uint2(0u, 0u);
            {
                float x[kPv][4];
                float mloc = -INFINITY;
#pragma unroll
                for (int ks = 0; ks < kPv; ks++) {
                    float4 x4 = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
                    if (head_ok) x4 = *reinterpret_cast<const float4*>(s_all + (st * 8 + key16) * kWidePitch + 16 * ks + 4 * kq);
                    x[ks][0] = x4.x; x[ks][1] = x4.y; x[ks][2] = x4.z; x[ks][3] = x4.w;
                    mloc = fmaxf(fmaxf(mloc, fmaxf(x4.x, x4.y)), fmaxf(x4.z, x4.w));
                }
                const float m = rows4_max(mloc);
                const float ms = m == -INFINITY ? 0.f : m;
                float lloc = 0.f;
#pragma unroll
                for (int ks = 0; ks < kPv; ks++) {
                    const float e0 = __builtin_amdgcn_exp2f(x[ks][0] - ms), e1 = __builtin_amdgcn_exp2f(x[ks][1] - ms);
                    const float e2 = __builtin_amdgcn_exp2f(x[ks][2] - ms), e3 = __builtin_amdgcn_exp2f(x[ks][3] - ms);
                    lloc += (e0 + e1) + (e2 + e3);
                    pb[ks] = make_uint2(Mma16<T>::pack2(e0, e1), Mma16<T>::pack2(e2, e3));  // hidden keys and idle rows: 0
                    if (ks == wave) {  // the piece this wavefront hands to the score kernel, fp16 whatever the tensor dtype
                        e_mine = make_uint2(Mma16<__half>::pack2(e0, e1), Mma16<__half>::pack2(e2, e3));
                    }
                }
                m_t = m;
                l_t = rows4_sum(lloc);
            }
            // ---- weighted V sum on the matrix pipe: this wavefront's dims over all keys of the tile.  Lane
            //      16 q + g (g < G) ends up with dims 16 (kDb wave + b2) + 4 q .. + 3 of head g.
            f32x4 acc[kDb];
#pragma unroll
            for (int b2 = 0; b2 < kDb; b2++) acc[b2] = f32x4{0.f, 0.f, 0.f, 0.f};
            {
                const uint32_t vbase = lds_base + st * kStreamStage;
#pragma unroll
                for (int ks = 0; ks < kPv; ks++) {
#pragma unroll
                    for (int b2 = 0; b2 < kDb; b2++) {
                        const s16x4_t va = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) s16x4_t*)(uintptr_t)(vbase + vt_addr[b2] + ks * 4096));
                        uint2 av = __builtin_bit_cast(uint2, va);
                        av.x &= m01[ks];
                        av.y &= m23[ks];
                        acc[b2] = Mma16<T>::mma_k16(av, pb[ks], acc[b2]);
                    }
                }
            }
            {
                // lanes 16 q + g hold head g = key16: l_t is that head's sum (0: the tile is hidden)
                const float inv_l = l_t > 0.f ? 1.0f / l_t : 0.f;
#pragma unroll
                for (int b2 = 0; b2 < kDb; b2++)
                    pend_o[b2] = make_uint2(Mma16<T>::pack2(acc[b2][0] * inv_l, acc[b2][1] * inv_l),
                                            Mma16<T>::pack2(acc[b2][2] * inv_l, acc[b2][3] * inv_l));
            }
            pend_m = m_t;
            pend_l = l_t;
            pend_e = e_mine;
            pending = true;
            pend_b = b;
            pend_kvh = kvh;
            b = b_nx;
            kvh = kvh_nx;
            st ^= 1;
        }
        flush();
        // the repeated copies of the last item must land, and every wavefront be done with the stages,
        // before the next run of items refills them
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __builtin_amdgcn_s_barrier();
    }
}

// one workgroup per (b, h): 16 groups of 32 threads walk every 16th tile, eight tiles in flight, then merge
// through LDS (the fp32 partial sums of the kernels that take a tile per workgroup)
template <typename T>
__global__ void __launch_bounds__(512) decode_tail_kernel(DecodeParams p) {
    __shared__ float sh_m[8], sh_l[16];
    __shared__ float4 sh_o[16][32];
    const ckv_attn_args& a = p.a;
    const int64_t row = blockIdx.x;  // b * H + h
    const int tid = threadIdx.x, d4 = tid & 31, grp = tid >> 5;  // 16 groups of 32 threads, 4 dims per thread
    const float* ml = p.part_ml + row * p.tiles * 2;
    float M = -INFINITY;
    for (int t = tid; t < p.tiles; t += 512) M = fmaxf(M, ml[2 * t]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
    if ((tid & 63) == 0) sh_m[tid >> 6] = M;
    __syncthreads();
    M = sh_m[tid & 7];
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
    // every tile's partial is written by the main kernel (zeros when the tile is hidden), so the
    // loop needs no branch; the loads of eight tiles are in flight together
    float L = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4* po = reinterpret_cast<const float4*>(p.part_o + row * p.tiles * kD) + d4;
    constexpr int kBatch = 8;
    for (int t0 = grp; t0 < p.tiles; t0 += 16 * kBatch) {
        float4 v[kBatch];
        float2 w[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            const int t = t0 + 16 * u;
            const bool ok = t < p.tiles;
            v[u] = ok ? po[(int64_t)t * (kD / 4)] : make_float4(0.f, 0.f, 0.f, 0.f);
            w[u] = ok ? *reinterpret_cast<const float2*>(ml + 2 * t) : make_float2(-INFINITY, 0.f);
        }
#pragma unroll
        for (int u = 0; u < kBatch; u++) {
            const float sc = w[u].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(w[u].x - M);
            L = fmaf(w[u].y, sc, L);
            o.x = fmaf(v[u].x, sc, o.x);
            o.y = fmaf(v[u].y, sc, o.y);
            o.z = fmaf(v[u].z, sc, o.z);
            o.w = fmaf(v[u].w, sc, o.w);
        }
    }
    sh_o[grp][d4] = o;
    if (d4 == 0) sh_l[grp] = L;
    __syncthreads();
    if (tid >= kD) return;
    const int d = tid;
    float od = 0.f;
    L = 0.f;
#pragma unroll
    for (int g = 0; g < 16; g++) {
        od += reinterpret_cast<const float*>(&sh_o[g][0])[d];
        L += sh_l[g];
    }
    const int64_t b = row / a.H, h = row % a.H;
    T* out = (T*)a.out + b * a.out_stride[0] + h * a.out_stride[1];
    out[d * a.out_stride[3]] = Elem<T>::from_float(od / L);
    if (d == 0) {
        const float l2 = M + __builtin_amdgcn_logf(L);
        p.lse2[row] = l2;
        if (a.lse) a.lse[row] = l2 * 0.6931471805599453f;
    }
}

// The same for the streaming kernel's results (per-tile averages in the tensor dtype, one (max, sum) pair per head
// and item) in as few trips to memory as the tiles allow: 32 groups of 16 lanes, a lane owns 8 dims (one 16-byte
// piece of an average), a group walks every 32nd tile with kTailBatch tiles requested at once and keeps a running
// (max, sum, weighted average) of its own, so no pass over the maxima comes first; the groups merge through LDS.
// 513 tiles (a 64K cache) are two batches per group, 257 tiles one.
constexpr int kTailBatch = 9;

template <typename T>
__global__ void __launch_bounds__(512) decode_tail_stream_kernel(DecodeParams p) {
    __shared__ float sh_m[32], sh_l[32];
    __shared__ float sh_o[32][kD];
    const ckv_attn_args& a = p.a;
    const int64_t row = blockIdx.x;  // b * H + h
    const int tid = threadIdx.x, d8 = tid & 15, grp = tid >> 4;
    const int n_vis = p.n_vis;  // the items are numbered over the tiles that can hold a visible key
    const int64_t nbh = a.B * a.KVH, total = (int64_t)n_vis * nbh;
    const int G = (int)(a.H / a.KVH), g = (int)((row % a.H) % G);
    const int64_t bh = (row / a.H) * a.KVH + (row % a.H) / G;
    const int64_t chunk_bytes = (int64_t)G * (kSK + kD) * 2;
    const int64_t in_chunk = ((int64_t)G * kSK + g * kD) * 2 + d8 * 16;
    float M = -INFINITY, L = 0.f;
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = 0.f;
    for (int t0 = grp; t0 < n_vis; t0 += 32 * kTailBatch) {
        // chunk of tile t0 + 32 u: worked out by lane u of the group (two divisions) and handed round
        int64_t ck_mine = 0;
        {
            const int t = t0 + 32 * d8;
            if (d8 < kTailBatch && t < n_vis) ck_mine = stream_chunk_of((int64_t)t * nbh + bh, total, p.stream_wgs);
        }
        uint4 v[kTailBatch];
        float2 w[kTailBatch];
#pragma unroll
        for (int u = 0; u < kTailBatch; u++) {
            const int64_t ck = __shfl(ck_mine, (tid & 48) + u);
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            w[u] = make_float2(-INFINITY, 0.f);
            if (t0 + 32 * u < n_vis) {
                v[u] = *reinterpret_cast<const uint4*>(p.chunks + ck * chunk_bytes + in_chunk);
                w[u] = *reinterpret_cast<const float2*>(p.part_ml + (ck * G + g) * 2);
            }
        }
        float bm = M;
#pragma unroll
        for (int u = 0; u < kTailBatch; u++) bm = fmaxf(bm, w[u].x);
        if (bm == -INFINITY) continue;  // nothing visible so far
        const float keep = M == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M - bm);
        M = bm;
        L *= keep;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] *= keep;
#pragma unroll
        for (int u = 0; u < kTailBatch; u++) {
            const float sc = w[u].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(w[u].x - M) * w[u].y;
            L += sc;
            const uint32_t r[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                o[2 * e] = fmaf(Mma16<T>::lo(r[e]), sc, o[2 * e]);
                o[2 * e + 1] = fmaf(Mma16<T>::hi(r[e]), sc, o[2 * e + 1]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) sh_o[grp][d8 * 8 + e] = o[e];
    if (d8 == 0) {
        sh_m[grp] = M;
        sh_l[grp] = L;
    }
    __syncthreads();
    if (tid >= kD) return;
    float Mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < 32; k++) Mx = fmaxf(Mx, sh_m[k]);
    float od = 0.f;
    L = 0.f;
#pragma unroll
    for (int k = 0; k < 32; k++) {
        const float f = sh_m[k] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sh_m[k] - Mx);
        od = fmaf(sh_o[k][tid], f, od);
        L = fmaf(sh_l[k], f, L);
    }
    const int64_t b = row / a.H, h = row % a.H;
    T* out = (T*)a.out + b * a.out_stride[0] + h * a.out_stride[1];
    out[tid * a.out_stride[3]] = Elem<T>::from_float(od / L);
    if (tid == 0) {
        const float l2 = Mx + __builtin_amdgcn_logf(L);
        p.lse2[row] = l2;
        if (a.lse) a.lse[row] = l2 * 0.6931471805599453f;
    }
}

template <typename T, int G>
__device__ inline float reduce_group(const float* v, int n, int mode) {
    if (mode == CKV_REDUCE_MAX) {
        float r = v[0];
        for (int i = 1; i < n; i++) r = fmaxf(r, v[i]);
        return r;
    }
    if (mode == CKV_REDUCE_MEAN) {
        float r = 0.f;
        for (int i = 0; i < n; i++) r = __fadd_rn(r, v[i]);
        return round_t<T>(r / (float)n);
    }
    float tmp[128];
    for (int i = 0; i < n; i++) {
        const float x = v[i];
        int k = i;
        while (k > 0 && tmp[k - 1] > x) {
            tmp[k] = tmp[k - 1];
            k--;
        }
        tmp[k] = x;
    }
    return tmp[(n - 1) / 2];
}

// one thread per (b, kvh, key): P of the G (or all H) heads, dtype rounding like the eager path
// (cascade_attention.py:319-323 with a single query row), head reduction, EMA / new-token score
template <typename T, int G, bool HOMO, bool PROBS>
__global__ void __launch_bounds__(256) decode_scores_kernel(DecodeParams p, float w_one, float beta_pow) {
    const ckv_attn_args& a = p.a;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t per = a.S + 1;
    if (idx >= a.B * a.KVH * per) return;
    const int64_t i = idx % per, kvh = (idx / per) % a.KVH, b = idx / (per * a.KVH);
    const int64_t n = a.num_sink + i;
    const bool is_new = i == a.S;
    // per kv head the G values stay in registers; only the all-heads reduction needs the long array
    float vals[HOMO ? 128 : G];
    int cnt = 0;
    const int64_t kv0 = HOMO ? 0 : kvh, kv1 = HOMO ? a.KVH : kvh + 1;
    for (int64_t kv = kv0; kv < kv1; kv++) {
        const float* lg = p.logits + ((b * a.KVH + kv) * p.N + n) * G;
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int64_t row = b * a.H + kv * G + g;
            float pt;
            if constexpr (PROBS) {  // 2^(logit - tile maximum) from the streaming kernel, and that maximum
                const int jt = stream_rank_of(p, (int)(n / kSK));  // -1: no key of the tile is visible
                pt = 0.f;
                if (jt >= 0) {
                    const int64_t ck = stream_chunk_of((int64_t)jt * (a.B * a.KVH) + b * a.KVH + kv,
                                                       (int64_t)p.n_vis * (a.B * a.KVH), p.stream_wgs);
                    const float e = (float)reinterpret_cast<const _Float16*>(p.chunks + ck * (G * (kSK + kD) * 2))[g * kSK + n % kSK];
                    const float m = p.part_ml[(ck * G + g) * 2];
                    pt = e == 0.f ? 0.f : round_t<T>(e * __builtin_amdgcn_exp2f(m - p.lse2[row]));
                }
            } else {
                pt = round_t<T>(__builtin_amdgcn_exp2f(lg[g] - p.lse2[row]));
            }
            // cached slots: fp32 product, cast; the new token: product in the tensor dtype
            vals[cnt++] = round_t<T>(__fmul_rn(pt, is_new ? round_t<T>(w_one) : w_one));
        }
    }
    float red;
    if (HOMO) {
        red = reduce_group<T, G>(vals, cnt, a.head_reduction);
    } else if (a.head_reduction == CKV_REDUCE_MAX) {
        red = vals[0];
#pragma unroll
        for (int g = 1; g < G; g++) red = fmaxf(red, vals[g]);
    } else if (a.head_reduction == CKV_REDUCE_MEAN) {
        red = 0.f;
#pragma unroll
        for (int g = 0; g < G; g++) red = __fadd_rn(red, vals[g]);
        red = round_t<T>(red / (float)G);
    } else {  // lower median: rank by counting, no indexed array
        red = vals[0];
#pragma unroll
        for (int g = 0; g < G; g++) {
            int below = 0, equal = 0;
#pragma unroll
            for (int h = 0; h < G; h++) {
                below += vals[h] < vals[g];
                equal += vals[h] == vals[g];
            }
            if (below <= (G - 1) / 2 && (G - 1) / 2 < below + equal) red = vals[g];
        }
    }
    if (is_new) {
        if (a.new_scores)
            *((T*)a.new_scores + b * a.new_scores_stride[0] + kvh * a.new_scores_stride[1]) = Elem<T>::from_float(red);
    } else if (a.cache_s) {
        T* cs = (T*)a.cache_s + b * a.cache_s_stride[0] + kvh * a.cache_s_stride[1] + i * a.cache_s_stride[2];
        const float decayed = round_t<T>(__fmul_rn(beta_pow, Elem<T>::to_float(*cs)));
        *cs = Elem<T>::from_float(__fadd_rn(decayed, red));
    }
}

// The same after the streaming kernel, per kv head: one thread per (b, kvh, 8 consecutive keys), which are one
// 16-byte piece of each head's fp16 probabilities and share the tile maximum.
template <typename T, int G>
__global__ void __launch_bounds__(256) decode_scores_probs_kernel(DecodeParams p, float w_one, float beta_pow) {
    const ckv_attn_args& a = p.a;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t per = p.Np / 8;
    if (idx >= a.B * a.KVH * per) return;
    const int64_t n0 = (idx % per) * 8, kvh = (idx / per) % a.KVH, b = idx / (per * a.KVH);
    if (n0 + 8 <= a.num_sink || n0 >= p.N) return;  // sinks keep no score; padding
    float pr[G][8];
    const int jt = stream_rank_of(p, (int)(n0 / kSK));  // -1: no key of the tile is visible, all probabilities are 0
    const int64_t ck = jt < 0 ? 0 : stream_chunk_of((int64_t)jt * (a.B * a.KVH) + b * a.KVH + kvh,
                                                    (int64_t)p.n_vis * (a.B * a.KVH), p.stream_wgs);
    const unsigned char* chunk = p.chunks + ck * (G * (kSK + kD) * 2);
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int64_t row = b * a.H + kvh * G + g;
        uint4 raw = make_uint4(0u, 0u, 0u, 0u);
        float c = 0.f;
        if (jt >= 0) {
            raw = *reinterpret_cast<const uint4*>(chunk + (g * kSK + n0 % kSK) * 2);
            c = __builtin_amdgcn_exp2f(p.part_ml[(ck * G + g) * 2] - p.lse2[row]);
        }
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float e = (float)__builtin_bit_cast(f16x2_t, w[k >> 1])[k & 1];
            pr[g][k] = e == 0.f ? 0.f : round_t<T>(e * c);
        }
    }
    const float w_new = round_t<T>(w_one);
    float red[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const bool is_new = n0 + k == p.N - 1;
        float vals[G];
        // cached slots: fp32 product, cast; the new token: product in the tensor dtype
#pragma unroll
        for (int g = 0; g < G; g++) vals[g] = round_t<T>(__fmul_rn(pr[g][k], is_new ? w_new : w_one));
        float r;
        if (a.head_reduction == CKV_REDUCE_MAX) {
            r = vals[0];
#pragma unroll
            for (int g = 1; g < G; g++) r = fmaxf(r, vals[g]);
        } else if (a.head_reduction == CKV_REDUCE_MEAN) {
            r = 0.f;
#pragma unroll
            for (int g = 0; g < G; g++) r = __fadd_rn(r, vals[g]);
            r = round_t<T>(r / (float)G);
        } else {  // lower median: rank by counting
            r = vals[0];
#pragma unroll
            for (int g = 0; g < G; g++) {
                int below = 0, equal = 0;
#pragma unroll
                for (int h = 0; h < G; h++) {
                    below += vals[h] < vals[g];
                    equal += vals[h] == vals[g];
                }
                if (below <= (G - 1) / 2 && (G - 1) / 2 < below + equal) r = vals[g];
            }
        }
        red[k] = r;
    }
    const int64_t i0 = n0 - a.num_sink;
    T* cs = a.cache_s ? (T*)a.cache_s + b * a.cache_s_stride[0] + kvh * a.cache_s_stride[1] : nullptr;
    if (cs && i0 >= 0 && i0 + 8 <= a.S && a.cache_s_stride[2] == 1 && (reinterpret_cast<uintptr_t>(cs + i0) & 15) == 0) {
        uint4 old = *reinterpret_cast<const uint4*>(cs + i0);
        T* o = reinterpret_cast<T*>(&old);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float decayed = round_t<T>(__fmul_rn(beta_pow, Elem<T>::to_float(o[k])));
            o[k] = Elem<T>::from_float(__fadd_rn(decayed, red[k]));
        }
        *reinterpret_cast<uint4*>(cs + i0) = old;
        return;
    }
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int64_t i = i0 + k;
        if (i < 0 || i > a.S) continue;
        if (i == a.S) {
            if (a.new_scores)
                *((T*)a.new_scores + b * a.new_scores_stride[0] + kvh * a.new_scores_stride[1]) = Elem<T>::from_float(red[k]);
        } else if (cs) {
            T* c1 = cs + i * a.cache_s_stride[2];
            const float decayed = round_t<T>(__fmul_rn(beta_pow, Elem<T>::to_float(*c1)));
            *c1 = Elem<T>::from_float(__fadd_rn(decayed, red[k]));
        }
    }
}

// All heads reduced together (cascade_attention.py:240-242) after a streaming kernel: one thread per (batch, key),
// a workgroup per 128-key tile, so that the factor 2^(tile maximum - normaliser) of every head is worked out once
// per workgroup.  The thread walks the H heads in order (kv head major, as repeat_kv lays them out), keeps a running
// sum or maximum, or parks the H values in its LDS column and finds the lower median by counting, and writes the
// result to the score row of every kv head.
constexpr int kHomoMaxHeads = 64;

template <typename T, int G>
__global__ void __launch_bounds__(kSK) decode_scores_homo_kernel(DecodeParams p, float w_one, float beta_pow) {
    __shared__ float sh_c[kHomoMaxHeads];
    __shared__ int64_t sh_ck[kHomoMaxHeads / G + 1];
    __shared__ float sh_v[kHomoMaxHeads][kSK];   // median only
    const ckv_attn_args& a = p.a;
    const int tile = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int H = (int)a.H, KVH = (int)a.KVH;
    const int64_t n = (int64_t)tile * kSK + tid;
    const int jt = stream_rank_of(p, tile);  // -1: no key of the tile is visible, every probability is 0
    if (tid < H) {
        const int kv = tid / G, g = tid % G;
        float c = 0.f;
        if (jt >= 0) {
            const int64_t ck = stream_chunk_of((int64_t)jt * (a.B * KVH) + (int64_t)b * KVH + kv, (int64_t)p.n_vis * (a.B * KVH),
                                               p.stream_wgs);
            c = __builtin_amdgcn_exp2f(p.part_ml[(ck * G + g) * 2] - p.lse2[(int64_t)b * H + tid]);
            if (g == 0) sh_ck[kv] = ck;
        }
        sh_c[tid] = c;
    }
    __syncthreads();
    if (n < a.num_sink || n >= p.N) return;  // sinks keep no score; padding of the last tile
    const bool is_new = n == p.N - 1;
    const float w = is_new ? round_t<T>(w_one) : w_one;  // the new token's weight is built in the tensor dtype
    const int mode = a.head_reduction;
    float acc = mode == CKV_REDUCE_MAX ? -INFINITY : 0.f;
    for (int h = 0; h < H; h++) {
        float pt = 0.f;
        if (jt >= 0) {
            const unsigned char* chunk = p.chunks + sh_ck[h / G] * (G * (kSK + kD) * 2);
            const float e = (float)reinterpret_cast<const _Float16*>(chunk)[(h % G) * kSK + tid];
            pt = e == 0.f ? 0.f : round_t<T>(e * sh_c[h]);
        }
        const float v = round_t<T>(__fmul_rn(pt, w));
        if (mode == CKV_REDUCE_MAX) acc = h == 0 ? v : fmaxf(acc, v);
        else if (mode == CKV_REDUCE_MEAN) acc = __fadd_rn(acc, v);
        else sh_v[h][tid] = v;
    }
    float red;
    if (mode == CKV_REDUCE_MAX) {
        red = acc;
    } else if (mode == CKV_REDUCE_MEAN) {
        red = round_t<T>(acc / (float)H);
    } else {  // lower median: the value with at most (H-1)/2 values below it and more than that below or equal
        red = sh_v[0][tid];
        const int k = (H - 1) / 2;
        for (int i = 0; i < H; i++) {
            const float x = sh_v[i][tid];
            int below = 0, equal = 0;
            for (int j = 0; j < H; j++) {
                const float y = sh_v[j][tid];
                below += y < x;
                equal += y == x;
            }
            if (below <= k && k < below + equal) red = x;
        }
    }
    if (is_new) {
        if (a.new_scores)
            for (int kv = 0; kv < KVH; kv++)
                *((T*)a.new_scores + b * a.new_scores_stride[0] + kv * a.new_scores_stride[1]) = Elem<T>::from_float(red);
    } else if (a.cache_s) {
        const int rows = a.cache_s_stride[1] == 0 ? 1 : KVH;  // one shared row or one per kv head
        const int64_t i = n - a.num_sink;
        for (int kv = 0; kv < rows; kv++) {
            T* cs = (T*)a.cache_s + b * a.cache_s_stride[0] + kv * a.cache_s_stride[1] + i * a.cache_s_stride[2];
            const float decayed = round_t<T>(__fmul_rn(beta_pow, Elem<T>::to_float(*cs)));
            *cs = Elem<T>::from_float(__fadd_rn(decayed, red));
        }
    }
}

template <typename T, int G>
int run_decode(const DecodeParams& p_in, hipStream_t stream) {
    DecodeParams p = p_in;
    const ckv_attn_args& a = p.a;
    const bool use_stream =
        !std::is_same<T, float>::value && G <= 8 && p.shared_pos && stream_offsets_fit(a);
    if (use_stream) {
        p.tiles = (int)((p.N + kSK - 1) / kSK);  // the streaming kernel has its own tile size
        // keys that can be visible: the sinks, the leading `filled_slots` cache slots (all S when the caller gives
        // no bound) and the new token
        const int64_t filled = a.filled_slots > 0 && a.filled_slots < a.S ? a.filled_slots : a.S;
        p.tiles_pre = (int)std::min<int64_t>((a.num_sink + filled + kSK - 1) / kSK, p.tiles);
        p.n_vis = p.tiles_pre < p.tiles ? p.tiles_pre + 1 : p.tiles_pre;
    }
    p.Np = (int64_t)p.tiles * kSK;
    {
        StageScope sc(CKV_STAGE_PREP, stream);
        hipLaunchKernelGGL(decode_q_kernel<T>, dim3((unsigned)(a.B * a.H)), dim3(64), 0, stream, p);
        CKV_HIP_TRY(hipGetLastError());
    }
    {
        StageScope sc(CKV_STAGE_DECODE, stream, use_stream);
        const int64_t nbh = a.B * a.KVH;
        // enough workgroups to fill the chip, few enough that cos/sin are amortised over many rows
        int64_t groups = p.shared_pos ? (2048 + p.tiles - 1) / p.tiles : nbh;
        if (groups < 1) groups = 1;
        if (groups > nbh) groups = nbh;
        const int lds = (16 * G * kD + 32 * G + 4 * 32 * 8) * (int)sizeof(float);
        if constexpr (std::is_same<T, float>::value) {
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(decode_main_kernel<T, G>), lds)) return rc;
            hipLaunchKernelGGL((decode_main_kernel<T, G>), dim3((unsigned)p.tiles, (unsigned)groups), dim3(256), lds,
                               stream, p);
        } else if (use_stream) {
            // streaming kernel: as many workgroups as run at once, items dealt out evenly
            if constexpr (G <= 8) {
                constexpr int lds_s = G <= 4 ? kStreamLds : kWideLds;
                const void* kernel;
                if constexpr (G <= 4) kernel = reinterpret_cast<const void*>(decode_stream_kernel<T, G>);
                else kernel = reinterpret_cast<const void*>(decode_stream_wide_kernel<T, G>);
                if (int rc = ensure_dynamic_lds(kernel, lds_s)) return rc;
                DeviceInfo di;
                if (int rc = current_device_info(&di)) return rc;
                int64_t wgs = (di.cus > 0 ? di.cus : 256) * kStreamWgPerCu;
                if (wgs > kStreamMaxWgs) wgs = kStreamMaxWgs;
                if (wgs > p.n_vis * nbh) wgs = p.n_vis * nbh;
                p.stream_wgs = (int)wgs;
                hipEvent_t ev0, ev1;
                prof_kernel_events(CKV_STAGE_DECODE, &ev0, &ev1);
                if constexpr (G <= 4) {
                    if (ev0)
                        hipExtLaunchKernelGGL((decode_stream_kernel<T, G>), dim3((unsigned)wgs), dim3(kStreamThreads),
                                              (uint32_t)lds_s, stream, ev0, ev1, 0u, p);
                    else
                        hipLaunchKernelGGL((decode_stream_kernel<T, G>), dim3((unsigned)wgs), dim3(kStreamThreads), lds_s, stream, p);
                } else {
                    if (ev0)
                        hipExtLaunchKernelGGL((decode_stream_wide_kernel<T, G>), dim3((unsigned)wgs), dim3(kStreamThreads),
                                              (uint32_t)lds_s, stream, ev0, ev1, 0u, p);
                    else
                        hipLaunchKernelGGL((decode_stream_wide_kernel<T, G>), dim3((unsigned)wgs), dim3(kStreamThreads), lds_s,
                                           stream, p);
                }
            }
        } else {
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(decode_main_mfma_kernel<T, G>), lds)) return rc;
            hipLaunchKernelGGL((decode_main_mfma_kernel<T, G>), dim3((unsigned)p.tiles, (unsigned)groups), dim3(256), lds,
                               stream, p);
        }
        CKV_HIP_TRY(hipGetLastError());
    }
    {
        StageScope sc(CKV_STAGE_DECODE_TAIL, stream);
        bool launched = false;
        if constexpr (G <= 8 && !std::is_same<T, float>::value) {
            if (use_stream) {
                hipLaunchKernelGGL(decode_tail_stream_kernel<T>, dim3((unsigned)(a.B * a.H)), dim3(512), 0, stream, p);
                launched = true;
            }
        }
        if (!launched) hipLaunchKernelGGL(decode_tail_kernel<T>, dim3((unsigned)(a.B * a.H)), dim3(512), 0, stream, p);
        CKV_HIP_TRY(hipGetLastError());
        if (a.cache_s || a.new_scores) {
            // w_ema[0] == w_new[0] == (1 - beta) for a single query row; the new token's weight is
            // built in the tensor dtype (cascade_attention.py:270-276)
            const float w_one = (float)(1.0 - a.beta);
            const int64_t items = a.B * a.KVH * (a.S + 1);
            const dim3 grid((unsigned)((items + 255) / 256));
            if (a.homogeneous_heads && use_stream && a.H <= kHomoMaxHeads) {
                if constexpr (G <= 8 && !std::is_same<T, float>::value)
                    hipLaunchKernelGGL((decode_scores_homo_kernel<T, G>), dim3((unsigned)p.tiles, (unsigned)a.B), dim3(kSK), 0, stream,
                                       p, w_one, (float)a.beta);
            } else if (a.homogeneous_heads && use_stream)
                hipLaunchKernelGGL((decode_scores_kernel<T, G, true, true>), grid, dim3(256), 0, stream, p, w_one, (float)a.beta);
            else if (a.homogeneous_heads)
                hipLaunchKernelGGL((decode_scores_kernel<T, G, true, false>), grid, dim3(256), 0, stream, p, w_one, (float)a.beta);
            else if (use_stream) {
                if constexpr (G <= 8 && !std::is_same<T, float>::value) {
                    const int64_t groups8 = a.B * a.KVH * (p.Np / 8);
                    hipLaunchKernelGGL((decode_scores_probs_kernel<T, G>), dim3((unsigned)((groups8 + 255) / 256)), dim3(256), 0,
                                       stream, p, w_one, (float)a.beta);
                }
            }
            else
                hipLaunchKernelGGL((decode_scores_kernel<T, G, false, false>), grid, dim3(256), 0, stream, p, w_one, (float)a.beta);
            CKV_HIP_TRY(hipGetLastError());
        }
    }
    return CKV_OK;
}

template <typename T>
int run_decode_g(const DecodeParams& p, int G, hipStream_t stream) {
    switch (G) {
        case 1: return run_decode<T, 1>(p, stream);
        case 2: return run_decode<T, 2>(p, stream);
        case 4: return run_decode<T, 4>(p, stream);
        case 7: return run_decode<T, 7>(p, stream);
        case 8: return run_decode<T, 8>(p, stream);
        default: return CKV_ERR_UNSUPPORTED;
    }
}

inline bool aligned(const void* p, int64_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace

bool decode_supported(const ckv_attn_args& a) {
    if (a.Q != 1 || a.D != kD) return false;
    const int64_t G = a.H / a.KVH;
    if (!(G == 1 || G == 2 || G == 4 || G == 7 || G == 8)) return false;
    if ((a.homogeneous_heads ? a.H : G) > 128) return false;
    const int64_t es = elem_bytes(a.dtype), vec = 16;
    // rows are read as 16-byte (K of 16-bit caches, all of float32) or 8-byte vectors
    if (a.cache_stride[3] != 1 || a.kv_new_stride[3] != 1 || (a.num_sink > 0 && a.sink_stride[3] != 1)) return false;
    if (!aligned(a.cache_k, vec) || !aligned(a.cache_v, vec) || !aligned(a.k_new, vec) || !aligned(a.v_new, vec)) return false;
    if (a.num_sink > 0 && (!aligned(a.sink_k, vec) || !aligned(a.sink_v, vec))) return false;
    for (int i = 0; i < 3; i++) {
        if ((a.cache_stride[i] * es) % vec || (a.kv_new_stride[i] * es) % vec) return false;
        if (a.num_sink > 0 && (a.sink_stride[i] * es) % vec) return false;
    }
    return true;
}

constexpr int64_t kMinTile = kSK < kTK ? kSK : kTK;  // the partial results are sized for the smaller tile

// fp32 logits per (head, key), or the streaming kernel's result chunks: (kSK + 128) 16-bit values per head and
// item, for up to one item per workgroup more than there are items (runs differ by one in length)
inline int64_t logits_area_bytes(int64_t B, int64_t H, int64_t KVH, int64_t N) {
    const int64_t tiles = (N + kSK - 1) / kSK, items = tiles * B * KVH, G = H / KVH;
    const int64_t chunks = items + std::min<int64_t>(items, kStreamMaxWgs);
    return align_up(std::max(B * H * N * 4, chunks * G * (kSK + kD) * 2), 256);
}

// (maximum, sum) pairs: one per head and tile, or per head and result chunk of the streaming kernels (up to one
// chunk per workgroup more than there are items)
inline int64_t ml_area_bytes(int64_t B, int64_t H, int64_t KVH, int64_t tiles) {
    return align_up((B * H * tiles + std::min<int64_t>(tiles * B * KVH, kStreamMaxWgs) * (H / KVH)) * 2 * 4, 256);
}

int64_t decode_workspace_bytes(int64_t B, int64_t H, int64_t KVH, int64_t num_sink, int64_t S) {
    const int64_t N = num_sink + S + 1, tiles = (N + kMinTile - 1) / kMinTile;
    return 2 * align_up(B * H * kD * 4, 256) + logits_area_bytes(B, H, KVH, N) + ml_area_bytes(B, H, KVH, tiles) +
           align_up(B * H * tiles * kD * 4, 256) + align_up(B * H * 4, 256);
}

int launch_decode(const ckv_attn_args& a, hipStream_t stream) {
    DecodeParams p;
    p.a = a;
    p.N = a.num_sink + a.S + 1;
    p.tiles = (int)((p.N + kTK - 1) / kTK);
    const int64_t G = a.H / a.KVH;
    char* w = reinterpret_cast<char*>(a.workspace);
    p.qrot = reinterpret_cast<float*>(w); w += align_up(a.B * a.H * kD * 4, 256);
    p.qrot_t = w; w += align_up(a.B * a.H * kD * 4, 256);
    p.logits = reinterpret_cast<float*>(w);
    p.chunks = reinterpret_cast<unsigned char*>(w);
    p.stream_wgs = 0;
    p.tiles_pre = 0;
    p.n_vis = 0;
    w += logits_area_bytes(a.B, a.H, a.KVH, p.N);
    const int64_t tiles_max = (p.N + kMinTile - 1) / kMinTile;
    p.part_ml = reinterpret_cast<float*>(w); w += ml_area_bytes(a.B, a.H, a.KVH, tiles_max);
    p.part_o = reinterpret_cast<float*>(w); w += align_up(a.B * a.H * tiles_max * kD * 4, 256);
    p.lse2 = reinterpret_cast<float*>(w);
    p.shared_pos = a.sink_pos_stride[0] == 0 && a.sink_pos_stride[1] == 0 && a.pos_stride[0] == 0 && a.pos_stride[1] == 0;
    p.key_scale = sqrtf(a.scale);
    p.scale_log2 = 1.4426950408889634f;  // queries and keys each carry sqrt(scale)
    switch (a.dtype) {
        case CKV_F32: return run_decode_g<float>(p, (int)G, stream);
        case CKV_F16: return run_decode_g<__half>(p, (int)G, stream);
        case CKV_BF16: return run_decode_g<__hip_bfloat16>(p, (int)G, stream);
        default: return CKV_ERR_DTYPE;
    }
}

}  // namespace ckv
