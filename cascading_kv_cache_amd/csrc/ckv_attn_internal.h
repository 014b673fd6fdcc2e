// Internal interfaces between the attention entry points and the kernel families.
#pragma once

#include "ckv_common.h"

namespace ckv {

// Attention over keys that are already rotated and laid out as [cached | chunk]:
//   out[b,h,m]  = softmax_n(scale * q[b,h,m] . k[b,h/G,n] + mask) v[b,h/G,n]
//   cached key n < n_cached is masked iff kmasked[n]; chunk key n is visible iff n-n_cached <= m
//   colsum[b,h,n] = sum_m weight(m,n) * P[m,n]   (optional)
//     weight = w_ema[m]                         for cached keys, and for chunk keys if !new_mode
//     weight = w_new[m - (n - n_cached)]        for chunk keys if new_mode (m >= n - n_cached)
struct CoreProblem {
    const void* q;
    int64_t q_stride[4];      // (B, H, Q, D)
    const void* k;
    const void* v;
    int64_t kv_stride[4];     // (B, KVH, N, D)
    const uint8_t* kmasked;   // (n_cached,) 1 = masked; may be null when n_cached == 0
    void* out;
    int64_t out_stride[4];    // (B, H, Q, D)
    float* lse;               // (B, H, Q) natural-log normaliser of every row
    float* colsum;            // (B, H, N) or null
    const float* w_ema;       // (Q,)
    const float* w_new;       // (Q,)
    int new_mode;
    int64_t B, H, KVH, Q, N, D;
    float scale;
    int dtype;
};

// fp32-math kernels for every dtype and head size (<= 256): the parity path for float32 caches
// and the fallback for shapes the MFMA kernels do not cover.
int launch_core_generic(const CoreProblem& p, hipStream_t stream);

// weights of the score sums (cascade_attention.py:270-282, 315-317), rounded like the eager path
// w_ema gets 64 trailing zeros (slack read by the MFMA column pass)
int launch_weights(float* w_ema, float* w_new, int64_t Q, double beta, int dtype, hipStream_t stream);

int launch_cast_scores(const float* colsum, void* scores, const int64_t* stride, int64_t B, int64_t H, int64_t N,
                       int dtype, hipStream_t stream);

struct PrepProblem {
    const ckv_attn_args* a;
    void* qr;        // (B, H, Q, D) rotated queries
    void* kr;        // (B, KVH, N, D) rotated keys, [sink | cache | chunk]
    void* vc;        // (B, KVH, N, D) values in the same order
    uint8_t* kmasked;  // (num_sink + S,)
};
int launch_prep_generic(const PrepProblem& p, hipStream_t stream);

struct FinishProblem {
    const float* colsum;   // (B, H, N)
    int64_t N;
    void* cache_s;         // (B, KVH, S) strides below; may be null
    int64_t cache_s_stride[3];
    void* new_scores;      // (B, KVH, Q); may be null
    int64_t new_scores_stride[3];
    int64_t B, H, KVH, Q, S, num_sink;
    float beta_pow_q;      // beta^Q rounded to fp32
    int head_reduction, homogeneous, dtype;
};
int launch_finish(const FinishProblem& p, hipStream_t stream);

// rows of slack behind the staged queries, their normalisers and weights: the column pass reads whole
// tiles of this many query rows
constexpr int64_t kColSlack = 128;

// ---- bf16/fp16 MFMA family (head_dim 128) ----
struct MfmaSegment {
    const void* k;
    const void* v;
    int64_t stride[4];     // (B, KVH, len, D)
    const int64_t* pos;    // null: keys are already rotated
    int64_t pos_stride[2];
    int64_t pos_shift;
    const uint8_t* masked; // null: all visible
    int64_t len;
};

struct MfmaProblem {
    MfmaSegment seg[3];    // keys in order; the LAST Q keys overall are the causal chunk
    const void* q;
    int64_t q_stride[4];
    const int64_t* q_pos;  // null: queries are already rotated
    const float* inv_freq;
    float theta;
    int shared_pos;
    void *qr, *kr, *vt;
    unsigned long long* tile_vis;
    void* out;
    int64_t out_stride[4];
    float* lse;            // (B, H, Q) natural log
    float* lse2;           // (B*H*Q + kColSlack) scratch: minus the log2-domain normaliser, for the column pass
    float* colsum;         // (B, H, n) or null
    float* part_o;         // (mfma_fwd_splits, B*H*Q, D) and
    float* part_l2;        // (mfma_fwd_splits, B*H*Q): the forward kernel's shares, when it splits the keys
    const float* w_ema;
    const float* w_new;
    double beta;           // the EMA factor the weights were built from
    int new_mode;
    int64_t B, H, KVH, Q, n, n_pad;
    float scale;
    float key_scale;       // keys with position ids are multiplied by this after rotation and rounded again, the
                           // queries carry scale / key_scale: sqrt(scale) for the cascade path, which follows the
                           // eager arm (cascade_attention.py:284-291); 1 for keys that arrive rotated
    int dtype;
};

bool mfma_supported(int dtype, int64_t D, int64_t H, int64_t KVH, int64_t Q);
int64_t mfma_n_pad(int64_t n);
// shares of the key tiles per query tile on a chip of `cus` compute units; what a workspace must hold
int mfma_fwd_splits(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t n, int cus);
int mfma_fwd_splits_for_workspace(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t n);
int mfma_device_cus();  // compute units of the current device (256 where none can be asked)
bool mfma_fits(int64_t n);  // the per-tile bookkeeping of n keys fits in LDS
int launch_mfma(const MfmaProblem& p, hipStream_t stream);

// ---- backward of the dense operator on the matrix cores (16-bit, head_dim 128, 16-byte addressable rows) ----
bool bwd_mfma_supported(const ckv_dense_bwd_args& a);
int launch_bwd_mfma(const ckv_dense_bwd_args& a, const float* delta, hipStream_t stream);  // delta: (B, H, n_ctx)

// ---- single-token decode family (Q == 1, head_dim 128) ----
bool decode_supported(const ckv_attn_args& a);
int64_t decode_workspace_bytes(int64_t B, int64_t H, int64_t KVH, int64_t num_sink, int64_t S);
int launch_decode(const ckv_attn_args& a, hipStream_t stream);

}  // namespace ckv
