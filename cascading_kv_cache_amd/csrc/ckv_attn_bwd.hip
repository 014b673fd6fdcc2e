// Backward of the dense-input attention operator (cascade/models/flash_attention.py:279-537, 654-710):
// dq, dk, dv of  out = softmax(scale * q k^T + masks) v  with the cache mask on the first n_kv - n_ctx keys
// and the causal mask on the last n_ctx.  Only training reaches it (the inference path never differentiates).
// The kernels in this file are plain fp32-math kernels for every dtype and head size up to 192, tiled through
// LDS; 16-bit tensors with head_dim 128 go to the matrix-core kernels of ckv_attn_bwd_mfma.hip after the delta
// kernel.  The probabilities are recomputed from the row normalisers the forward pass returns.
//
//   delta   delta[m] = sum_d out[m, d] * dout[m, d]                      (flash_attention.py:279-294)
//   dq      one workgroup = 16 query rows of a head, key tiles of 64 stream through LDS:
//           p = exp(scale s - lse), ds = p (dp - delta) scale, dq += ds k
//   dkdv    one workgroup = 16 keys of a head, query tiles of 64 stream through LDS:
//           dv += p^T dout, dk += ds^T q
#include "ckv_attn_internal.h"

namespace ckv {
namespace {

constexpr int kMaxD = 192;  // two 64-row tiles and two 16-row tiles of fp32 rows must fit the LDS
constexpr int kOwn = 16;     // rows (dq) or keys (dkdv) a workgroup owns
constexpr int kTile = 64;    // keys (dq) or rows (dkdv) per LDS tile
constexpr int kThreads = 256;

struct BwdParams {
    ckv_dense_bwd_args a;
    float* delta;  // (B, H, n_ctx)
};

template <typename T>
__global__ void __launch_bounds__(kThreads) bwd_delta_kernel(BwdParams p) {
    const ckv_dense_bwd_args& a = p.a;
    const int wave = threadIdx.x / CKV_WAVE, lane = threadIdx.x % CKV_WAVE;
    const int64_t rows = a.B * a.H * a.n_ctx;
    const int64_t row = (int64_t)blockIdx.x * (kThreads / CKV_WAVE) + wave;
    if (row >= rows) return;
    const int64_t m = row % a.n_ctx, h = (row / a.n_ctx) % a.H, b = row / (a.n_ctx * a.H);
    const T* o = (const T*)a.out + b * a.out_stride[0] + h * a.out_stride[1] + m * a.out_stride[2];
    const T* g = (const T*)a.dout + b * a.dout_stride[0] + h * a.dout_stride[1] + m * a.dout_stride[2];
    float acc = 0.f;
    for (int64_t d = lane; d < a.D; d += CKV_WAVE)
        acc = fmaf(Elem<T>::to_float(o[d * a.out_stride[3]]), Elem<T>::to_float(g[d * a.dout_stride[3]]), acc);
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) p.delta[row] = acc;
}

// row-major tile of `rows` rows x D floats in LDS with an odd pitch (a lane per row reads without conflicts)
template <typename T>
__device__ inline void load_tile(float* dst, int pitch, const T* src, int64_t row_stride, int64_t d_stride, int64_t first,
                                 int64_t limit, int rows, int64_t D) {
    for (int64_t idx = threadIdx.x; idx < rows * D; idx += kThreads) {
        const int r = (int)(idx / D);
        const int64_t d = idx % D;
        const int64_t n = first + r;
        dst[r * pitch + d] = n < limit ? Elem<T>::to_float(src[n * row_stride + d * d_stride]) : 0.f;
    }
}

template <typename T>
__global__ void __launch_bounds__(kThreads) bwd_dq_kernel(BwdParams p) {
    extern __shared__ float lds[];
    const ckv_dense_bwd_args& a = p.a;
    const int64_t D = a.D, n_ctx = a.n_ctx, n_kv = a.n_kv, n_cached = n_kv - n_ctx;
    const int pitch = (int)D + 1;
    float* k_t = lds;                        // [kTile][D + 1]
    float* v_t = k_t + kTile * pitch;        // [kTile][D + 1]
    float* q_s = v_t + kTile * pitch;        // [kOwn][D + 1]
    float* g_s = q_s + kOwn * pitch;         // [kOwn][D + 1]
    float* ds_s = g_s + kOwn * pitch;        // [kOwn][kTile + 1]
    const int tid = threadIdx.x;
    const int r = tid / 16, c16 = tid % 16;  // the row of the block this thread works on, its lane in the row
    const int64_t bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const int64_t m0 = (int64_t)blockIdx.x * kOwn;
    const T* qb = (const T*)a.q + b * a.q_stride[0] + h * a.q_stride[1];
    const T* gb = (const T*)a.dout + b * a.dout_stride[0] + h * a.dout_stride[1];
    const T* kb = (const T*)a.k + b * a.kv_stride[0] + h * a.kv_stride[1];
    const T* vb = (const T*)a.v + b * a.kv_stride[0] + h * a.kv_stride[1];
    load_tile<T>(q_s, pitch, qb, a.q_stride[2], a.q_stride[3], m0, n_ctx, kOwn, D);
    load_tile<T>(g_s, pitch, gb, a.dout_stride[2], a.dout_stride[3], m0, n_ctx, kOwn, D);
    const int64_t m = m0 + r;
    const bool row_ok = m < n_ctx;
    const float lse = row_ok ? a.lse[bh * n_ctx + m] : 0.f;
    const float delta = row_ok ? p.delta[bh * n_ctx + m] : 0.f;
    float dq[kMaxD / 16];
#pragma unroll
    for (int u = 0; u < kMaxD / 16; u++) dq[u] = 0.f;
    // keys past the diagonal of the block's last row are visible to none of its rows
    int64_t m_last = m0 + kOwn - 1;
    if (m_last > n_ctx - 1) m_last = n_ctx - 1;
    const int64_t n_end = n_cached + m_last + 1;
    for (int64_t n0 = 0; n0 < n_end; n0 += kTile) {
        __syncthreads();  // the tiles of the step before are no longer read
        load_tile<T>(k_t, pitch, kb, a.kv_stride[2], a.kv_stride[3], n0, n_kv, kTile, D);
        load_tile<T>(v_t, pitch, vb, a.kv_stride[2], a.kv_stride[3], n0, n_kv, kTile, D);
        __syncthreads();
        // logits and dp of this thread's four keys of the tile
        float s[4] = {0.f, 0.f, 0.f, 0.f}, dp[4] = {0.f, 0.f, 0.f, 0.f};
        for (int64_t d = 0; d < D; d++) {
            const float qv = q_s[r * pitch + d], gv = g_s[r * pitch + d];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int j = c16 + 16 * u;
                s[u] = fmaf(qv, k_t[j * pitch + d], s[u]);
                dp[u] = fmaf(gv, v_t[j * pitch + d], dp[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = c16 + 16 * u;
            const int64_t n = n0 + j;
            bool vis = row_ok && n < n_kv;
            if (vis) vis = n < n_cached ? a.mask[n] == 0 : (n - n_cached) <= m;
            const float pe = vis ? expf(s[u] * a.scale - lse) : 0.f;
            ds_s[r * (kTile + 1) + j] = pe * (dp[u] - delta) * a.scale;
        }
        __syncthreads();
        // dq[r, d] += sum_j ds[r, j] k[j, d] for this thread's dims d = c16 + 16 u
        for (int j = 0; j < kTile; j++) {
            const float w = ds_s[r * (kTile + 1) + j];
#pragma unroll
            for (int u = 0; u < kMaxD / 16; u++) {
                const int64_t d = c16 + 16 * u;
                if (d < D) dq[u] = fmaf(w, k_t[j * pitch + d], dq[u]);
            }
        }
    }
    if (row_ok) {
        T* out = (T*)a.dq + b * a.dq_stride[0] + h * a.dq_stride[1] + m * a.dq_stride[2];
#pragma unroll
        for (int u = 0; u < kMaxD / 16; u++) {
            const int64_t d = c16 + 16 * u;
            if (d < D) out[d * a.dq_stride[3]] = Elem<T>::from_float(dq[u]);
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kThreads) bwd_dkdv_kernel(BwdParams p) {
    extern __shared__ float lds[];
    const ckv_dense_bwd_args& a = p.a;
    const int64_t D = a.D, n_ctx = a.n_ctx, n_kv = a.n_kv, n_cached = n_kv - n_ctx;
    const int pitch = (int)D + 1;
    float* q_t = lds;                        // [kTile][D + 1]
    float* g_t = q_t + kTile * pitch;        // [kTile][D + 1]
    float* k_s = g_t + kTile * pitch;        // [kOwn][D + 1]
    float* v_s = k_s + kOwn * pitch;         // [kOwn][D + 1]
    float* p_s = v_s + kOwn * pitch;         // [kOwn][kTile + 1]
    float* ds_s = p_s + kOwn * (kTile + 1);  // [kOwn][kTile + 1]
    float* lse_s = ds_s + kOwn * (kTile + 1);  // [kTile]
    float* del_s = lse_s + kTile;              // [kTile]
    const int tid = threadIdx.x;
    const int c = tid / 16, c16 = tid % 16;  // the key of the block this thread works on, its lane in the key
    const int64_t bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const int64_t n0 = (int64_t)blockIdx.x * kOwn;
    const T* qb = (const T*)a.q + b * a.q_stride[0] + h * a.q_stride[1];
    const T* gb = (const T*)a.dout + b * a.dout_stride[0] + h * a.dout_stride[1];
    const T* kb = (const T*)a.k + b * a.kv_stride[0] + h * a.kv_stride[1];
    const T* vb = (const T*)a.v + b * a.kv_stride[0] + h * a.kv_stride[1];
    load_tile<T>(k_s, pitch, kb, a.kv_stride[2], a.kv_stride[3], n0, n_kv, kOwn, D);
    load_tile<T>(v_s, pitch, vb, a.kv_stride[2], a.kv_stride[3], n0, n_kv, kOwn, D);
    const int64_t n = n0 + c;
    bool key_ok = n < n_kv;
    if (key_ok && n < n_cached) key_ok = a.mask[n] == 0;  // a masked slot receives no gradient
    const int64_t first_row = n < n_cached ? 0 : n - n_cached;  // the first row that sees this key
    float dk[kMaxD / 16], dv[kMaxD / 16];
#pragma unroll
    for (int u = 0; u < kMaxD / 16; u++) dk[u] = dv[u] = 0.f;
    // rows before the first one that sees the block's first key see none of its keys
    int64_t m_begin = n0 < n_cached ? 0 : n0 - n_cached;
    m_begin = m_begin / kTile * kTile;
    for (int64_t m0 = m_begin; m0 < n_ctx; m0 += kTile) {
        __syncthreads();
        load_tile<T>(q_t, pitch, qb, a.q_stride[2], a.q_stride[3], m0, n_ctx, kTile, D);
        load_tile<T>(g_t, pitch, gb, a.dout_stride[2], a.dout_stride[3], m0, n_ctx, kTile, D);
        if (tid < kTile) {
            const int64_t m = m0 + tid;
            lse_s[tid] = m < n_ctx ? a.lse[bh * n_ctx + m] : 0.f;
            del_s[tid] = m < n_ctx ? p.delta[bh * n_ctx + m] : 0.f;
        }
        __syncthreads();
        float s[4] = {0.f, 0.f, 0.f, 0.f}, dp[4] = {0.f, 0.f, 0.f, 0.f};
        for (int64_t d = 0; d < D; d++) {
            const float kv = k_s[c * pitch + d], vv = v_s[c * pitch + d];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int j = c16 + 16 * u;
                s[u] = fmaf(kv, q_t[j * pitch + d], s[u]);
                dp[u] = fmaf(vv, g_t[j * pitch + d], dp[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = c16 + 16 * u;
            const int64_t m = m0 + j;
            const bool vis = key_ok && m < n_ctx && m >= first_row;
            const float pe = vis ? expf(s[u] * a.scale - lse_s[j]) : 0.f;
            p_s[c * (kTile + 1) + j] = pe;
            ds_s[c * (kTile + 1) + j] = pe * (dp[u] - del_s[j]) * a.scale;
        }
        __syncthreads();
        for (int j = 0; j < kTile; j++) {
            const float pw = p_s[c * (kTile + 1) + j], dw = ds_s[c * (kTile + 1) + j];
#pragma unroll
            for (int u = 0; u < kMaxD / 16; u++) {
                const int64_t d = c16 + 16 * u;
                if (d < D) {
                    dv[u] = fmaf(pw, g_t[j * pitch + d], dv[u]);
                    dk[u] = fmaf(dw, q_t[j * pitch + d], dk[u]);
                }
            }
        }
    }
    if (n < n_kv) {
        T* ok = (T*)a.dk + b * a.dkv_stride[0] + h * a.dkv_stride[1] + n * a.dkv_stride[2];
        T* ov = (T*)a.dv + b * a.dkv_stride[0] + h * a.dkv_stride[1] + n * a.dkv_stride[2];
#pragma unroll
        for (int u = 0; u < kMaxD / 16; u++) {
            const int64_t d = c16 + 16 * u;
            if (d < D) {
                ok[d * a.dkv_stride[3]] = Elem<T>::from_float(dk[u]);
                ov[d * a.dkv_stride[3]] = Elem<T>::from_float(dv[u]);
            }
        }
    }
}

template <typename T>
int run_bwd(const BwdParams& p, hipStream_t stream) {
    const ckv_dense_bwd_args& a = p.a;
    const int64_t rows = a.B * a.H * a.n_ctx;
    const int pitch = (int)a.D + 1;
    const size_t lds_dq = sizeof(float) * ((size_t)(2 * kTile + 2 * kOwn) * pitch + (size_t)kOwn * (kTile + 1));
    {
        // both kernels stage fp32 tiles of D + 1 columns: a device whose workgroups get less LDS than they ask
        // for is told so before anything is launched
        const size_t lds_kv_ = sizeof(float) * ((size_t)(2 * kTile + 2 * kOwn) * pitch + (size_t)2 * kOwn * (kTile + 1) + 2 * kTile);
        DeviceInfo di;
        if (int rc = current_device_info(&di)) return rc;
        if (lds_dq > (size_t)di.lds_max || lds_kv_ > (size_t)di.lds_max) return CKV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(bwd_delta_kernel<T>, dim3((unsigned)((rows + 3) / 4)), dim3(kThreads), 0, stream, p);
    CKV_HIP_TRY(hipGetLastError());
    if (bwd_mfma_supported(a)) return launch_bwd_mfma(a, p.delta, stream);
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(bwd_dq_kernel<T>), (int)lds_dq)) return rc;
    hipLaunchKernelGGL(bwd_dq_kernel<T>, dim3((unsigned)((a.n_ctx + kOwn - 1) / kOwn), (unsigned)(a.B * a.H)), dim3(kThreads),
                       lds_dq, stream, p);
    CKV_HIP_TRY(hipGetLastError());
    const size_t lds_kv =
        sizeof(float) * ((size_t)(2 * kTile + 2 * kOwn) * pitch + (size_t)2 * kOwn * (kTile + 1) + 2 * kTile);
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(bwd_dkdv_kernel<T>), (int)lds_kv)) return rc;
    hipLaunchKernelGGL(bwd_dkdv_kernel<T>, dim3((unsigned)((a.n_kv + kOwn - 1) / kOwn), (unsigned)(a.B * a.H)), dim3(kThreads),
                       lds_kv, stream, p);
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

}  // namespace
}  // namespace ckv

extern "C" int64_t ckv_dense_bwd_workspace_bytes(int64_t B, int64_t H, int64_t n_ctx) {
    if (B <= 0 || H <= 0 || n_ctx <= 0) return 0;
    return ckv::align_up(B * H * n_ctx * (int64_t)sizeof(float), 256);
}

extern "C" int ckv_attn_dense_bwd(const ckv_dense_bwd_args* args, void* stream_) {
    using namespace ckv;
    if (!args) return CKV_ERR_NULL;
    const ckv_dense_bwd_args& a = *args;
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (a.dtype != CKV_F32 && a.dtype != CKV_F16 && a.dtype != CKV_BF16) return CKV_ERR_DTYPE;
    if (a.B <= 0 || a.H <= 0 || a.n_ctx <= 0 || a.n_kv < a.n_ctx || a.D <= 0) return CKV_ERR_SHAPE;
    if (a.D > kMaxD) return CKV_ERR_UNSUPPORTED;
    if (a.D % 16 != 0) return CKV_ERR_UNSUPPORTED;  // the kernels deal the head dims out in steps of 16
    if (a.B * a.H > 65535) return CKV_ERR_UNSUPPORTED;
    if (!a.q || !a.k || !a.v || !a.out || !a.lse || !a.dout || !a.dq || !a.dk || !a.dv) return CKV_ERR_NULL;
    if (a.n_kv > a.n_ctx && !a.mask) return CKV_ERR_NULL;
    if (!a.workspace || a.workspace_bytes < ckv_dense_bwd_workspace_bytes(a.B, a.H, a.n_ctx)) return CKV_ERR_WORKSPACE;
    BwdParams p;
    p.a = a;
    p.delta = reinterpret_cast<float*>(a.workspace);
    switch (a.dtype) {
        case CKV_F32: return run_bwd<float>(p, stream);
        case CKV_F16: return run_bwd<__half>(p, stream);
        default: return run_bwd<__hip_bfloat16>(p, stream);
    }
}
