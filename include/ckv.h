/*
 * libckv — C ABI of the MI355X (gfx950) Cascading-KV-Cache attention hot path.
 *
 * Two operators of the reference are replaced, each behind plain pointers,
 * element strides and sizes (no torch types cross this boundary):
 *
 *   ckv_update        <- sink_cache(...) / SinkCacheFunc.forward / _update_kv_cache
 *                        (cascade/models/cascading_cache.py:145-299, 302-774, 780-901, 962-1028)
 *   ckv_attn          <- CascadeAttention.forward_cascade prologue + cascade_attn_eager /
 *                        cascade_attn_flash + calc_scores + the score-EMA tail
 *                        (cascade/models/cascade_attention.py:82-340), which in the reference
 *                        bottoms out in attention(q,k,v,causal,sm_scale,mask,beta)
 *                        (cascade/models/flash_attention.py:540-652, 713)
 *   ckv_attn_dense    <- attention(q,k,v,causal,sm_scale,mask,beta) itself, for callers that
 *                        already hold rotated, GQA-expanded, concatenated K/V
 *                        (cascade/models/flash_attention.py:543-652)
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - strides are in ELEMENTS of the pointed-to type, outermost first;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all work is
 *     stream-ordered, nothing synchronises the host;
 *   - functions return CKV_OK (0) or a negative ckv_status; nothing throws;
 *   - the library owns no memory: scratch comes in through `workspace`
 *     (size from the matching *_workspace_bytes call) and is free for reuse once the
 *     stream has passed the call.
 */
#ifndef CKV_H_
#define CKV_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CKV_ABI_VERSION 2

typedef enum ckv_dtype {
    CKV_F32 = 0,
    CKV_F16 = 1,
    CKV_BF16 = 2
} ckv_dtype;

typedef enum ckv_status {
    CKV_OK = 0,
    CKV_ERR_NULL = -1,        /* a required pointer is NULL */
    CKV_ERR_SHAPE = -2,       /* sizes inconsistent (e.g. max_seq_len % window_size != 0) */
    CKV_ERR_STRIDE = -3,      /* layout the kernels cannot address (innermost stride != 1 ...) */
    CKV_ERR_DTYPE = -4,       /* unknown dtype */
    CKV_ERR_WORKSPACE = -5,   /* workspace missing or too small */
    CKV_ERR_UNSUPPORTED = -6, /* valid request outside what the kernels implement */
    CKV_ERR_LAUNCH = -7,      /* the HIP runtime rejected a launch */
    CKV_ERR_TOO_LARGE = -8    /* sizes beyond the fixed scratch of ckv_update_static */
} ckv_status;

typedef enum ckv_head_reduction {
    CKV_REDUCE_MEAN = 0,   /* torch.mean   (cascade_attention.py:235) */
    CKV_REDUCE_MAX = 1,    /* torch.amax   (cascade_attention.py:236) */
    CKV_REDUCE_MEDIAN = 2  /* torch.median(...).values, lower median (cascade_attention.py:237) */
} ckv_head_reduction;

/* ------------------------------------------------------------------------------------------
 * Cache update.  Mirrors the argument list of sink_cache (cascading_cache.py:962-985): the
 * same 3 inputs and 13 tensors mutated in place, the same scalars.  `s` may have more than H
 * heads (only its strides are used, cascade_attention.py:332).
 * ---------------------------------------------------------------------------------------- */
typedef struct ckv_update_args {
    const void* k;                 /* (N, H, K, HID) incoming keys, un-rotated            */
    const void* v;                 /* (N, H, K, HID) incoming values, same strides as k   */
    int64_t kv_stride[4];
    const void* s;                 /* (N, >=H, K) incoming scores, cache dtype            */
    int64_t s_stride[3];

    void* sink_k;                  /* (N, H, num_sink, HID)                               */
    void* sink_v;
    int64_t sink_stride[4];
    void* cache_k;                 /* (N, H, max_seq_len, HID)                            */
    void* cache_v;
    int64_t cache_stride[4];
    void* cache_s;                 /* (N, H, max_seq_len) score EMA per slot              */
    int64_t cache_s_stride[3];

    uint8_t* sink_mask;            /* (N, H, num_sink) bool, 1 = empty                    */
    int64_t sink_mask_stride[3];
    uint8_t* mask;                 /* (N, H, max_seq_len) bool, 1 = empty                 */
    int64_t mask_stride[3];
    int64_t* sink_pos;             /* (N, H, num_sink)                                    */
    int64_t sink_pos_stride[3];
    int64_t* pos;                  /* (N, H, max_seq_len) compact position ids            */
    int64_t pos_stride[3];
    int64_t* og_pos;               /* (N, H, max_seq_len) 1-based global token index      */
    int64_t og_pos_stride[3];

    int64_t* stored_sinks;         /* (N, H)                                              */
    int64_t stored_sinks_stride[2];
    int64_t* stored_tokens;        /* (N, H, cascades)                                    */
    int64_t* start_indices;        /* (N, H, cascades), same strides                      */
    int64_t tracker_stride[3];

    const int64_t* do_cache_every_n; /* (cascades,) contiguous acceptance periods          */
    const int64_t* real_token_idx;   /* 0-dim: tokens consumed before this call            */

    int64_t N, H, K, HID;
    int64_t num_sink;
    int64_t window_size;           /* slots per cascade                                   */
    int64_t max_seq_len;           /* cascades * window_size                              */
    int32_t cascades;
    int32_t eager_fill;
    int32_t dtype;                 /* ckv_dtype of k, v, s, sink_*, cache_*               */
    int32_t reserved;

    void* workspace;
    int64_t workspace_bytes;
} ckv_update_args;

/* bytes of scratch ckv_update needs for these sizes (0 is never returned for valid sizes) */
int64_t ckv_update_workspace_bytes(int64_t N, int64_t H, int64_t K, int64_t max_seq_len,
                                   int32_t cascades);

/* Replaces sink_cache(...) (cascading_cache.py:962-1028): scatters the K incoming rows of
 * every (n, h) across the sink and the cascades exactly as the serial per-token loop of
 * _update_kv_cache_inner (cascading_cache.py:381-774) would, and rewrites `pos`.  The caller
 * adds K to its token counter afterwards (cascading_cache.py:1346). */
int ckv_update(const ckv_update_args* args, void* stream);

/* ckv_update for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels and
 * same results as ckv_update, except that `workspace` / `workspace_bytes` are ignored: the scratch is a
 * fixed array inside the library (ckv_update_static_scratch_bytes() = 32 MiB per device, held until the
 * process ends), so the call allocates nothing and needs no workspace from the caller.  Sizes whose
 * ckv_update_workspace_bytes(...) exceeds that array are refused with CKV_ERR_TOO_LARGE.  All calls on
 * one device share the array: calls that overlap in time on one device (different streams, or different
 * host threads) race on it; calls on one stream are ordered and safe.  The first call on a device looks the
 * array's address and the device's limits up (runtime queries that must not be recorded): a caller that captures
 * the call into a HIP graph makes one ordinary call on that device first. */
int64_t ckv_update_static_scratch_bytes(void);
int ckv_update_static(const ckv_update_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention over [sink | cascades | current chunk] with RoPE from the cache's position ids,
 * GQA, exact softmax, and the score-EMA tail.  One call covers what forward_cascade does
 * between the q/k/v projections and cache.update (cascade_attention.py:114-200, 250-340):
 *   - rotates q and k_new at q_pos, sink keys at sink_pos, cached keys at pos + pos_shift
 *     (cascade_attention.py:150-166; HF half rotation, modeling_llama.py:199-220, 248-252);
 *   - out = softmax(scale * q k^T + masks) v with the sink/cache masks of row [0,0] and a
 *     causal mask inside the chunk (cascade_attention.py:284-313);
 *   - cache_s <- beta^Q * cache_s + reduce_heads(sum_m (1-beta) beta^(Q-1-m) P[m, slot])
 *     (cascade_attention.py:315-330, 231-248);
 *   - new_scores[b, kvh, n] = reduce_heads(sum_{m>=n} (1-beta) beta^(m-n) P[m, chunk n])
 *     (cascade_attention.py:270-282, 322-327).
 * Q == 1 takes the bandwidth-bound decode kernels, Q > 1 the MFMA prefill kernels.
 * ---------------------------------------------------------------------------------------- */
typedef struct ckv_attn_args {
    const void* q;                 /* (B, H, Q, D) un-rotated queries                     */
    int64_t q_stride[4];
    const void* k_new;             /* (B, KVH, Q, D) un-rotated keys of the chunk         */
    const void* v_new;
    int64_t kv_new_stride[4];
    const void* sink_k;            /* (B, KVH, num_sink, D) un-rotated                    */
    const void* sink_v;
    int64_t sink_stride[4];
    const void* cache_k;           /* (B, KVH, S, D) un-rotated                           */
    const void* cache_v;
    int64_t cache_stride[4];

    const uint8_t* sink_mask;      /* (num_sink,) row [0,0] of the bool mask, 1 = empty   */
    const uint8_t* mask;           /* (S,)        row [0,0] of the bool mask, 1 = empty   */
    const int64_t* q_pos;          /* (Q,) position ids of the chunk                      */
    const int64_t* sink_pos;       /* (num_sink,) or per-(b,kvh) with the strides below   */
    int64_t sink_pos_stride[2];    /* batch, kv-head strides; 0,0 = shared row            */
    const int64_t* pos;            /* (S,) or per-(b,kvh): position id of every slot      */
    int64_t pos_stride[2];
    int64_t pos_shift;             /* added to every pos entry (cascading_cache.py:1282-1292) */

    void* cache_s;                 /* (B, KVH or 1, S) score EMA, updated in place; NULL = skip */
    int64_t cache_s_stride[3];
    void* out;                     /* (B, H, Q, D)                                        */
    int64_t out_stride[4];
    void* new_scores;              /* (B, KVH, Q) in the cache dtype; NULL = skip         */
    int64_t new_scores_stride[3];
    float* lse;                    /* optional (B, H, Q) natural-log row normalisers      */

    int64_t B, H, KVH, Q, D;
    int64_t num_sink, S;
    float scale;                   /* softmax scale (1/sqrt(D) in the reference)          */
    float rope_theta;              /* base of the rotary frequencies                      */
    const float* inv_freq;         /* optional (D/2,) table overriding rope_theta         */
    double beta;
    int32_t head_reduction;        /* ckv_head_reduction                                  */
    int32_t homogeneous_heads;     /* reduce over all H heads (cascade_attention.py:240-242) */
    int32_t dtype;                 /* ckv_dtype of every floating tensor above            */
    int32_t filled_slots;          /* optional hint, never a second mask: the caller promises that every cache slot
                                      at or past this index is masked in `mask` (the cache fills from slot 0 up,
                                      cascading_cache.py:381-726, so the tokens stored so far bound it); 0 = no
                                      promise.  Kernels may then skip such slots without reading `mask` (the 16-bit
                                      single-token kernels skip whole 128-key tiles of a cache that is still
                                      filling) or ignore the hint altogether; visibility is decided by `mask` alone,
                                      so with a hint that keeps its promise the results do not depend on it, and a
                                      hint that contradicts `mask` gives unspecified results for the slots it
                                      covers. */

    void* workspace;
    int64_t workspace_bytes;
} ckv_attn_args;

int64_t ckv_attn_workspace_bytes(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t D,
                                 int64_t num_sink, int64_t S, int32_t dtype);

int ckv_attn(const ckv_attn_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dense-input attention with the signature of the reference operator
 * attention(q, k, v, causal, sm_scale, mask, beta) -> (o, scores) (flash_attention.py:543-652):
 * keys are already rotated, expanded to H heads and concatenated as [cached | chunk];
 * `mask` covers the first n_kv - n_ctx keys, the last n_ctx keys are causal.
 * scores[b, h, n] = sum_m (1-beta) beta^(n_ctx-1-m) P[m, n] (the exact value the reference
 * kernel approximates, flash_attention.py:73-100).
 * ---------------------------------------------------------------------------------------- */
typedef struct ckv_dense_args {
    const void* q;                 /* (B, H, n_ctx, D) */
    int64_t q_stride[4];
    const void* k;                 /* (B, H, n_kv, D)  */
    const void* v;
    int64_t kv_stride[4];
    const uint8_t* mask;           /* (n_kv - n_ctx,) bool, 1 = masked; may be NULL if that is 0 */
    void* out;                     /* (B, H, n_ctx, D) */
    int64_t out_stride[4];
    void* scores;                  /* (B, H, n_kv) in q's dtype; NULL = skip */
    int64_t scores_stride[3];
    int64_t B, H, n_ctx, n_kv, D;
    float scale;
    double beta;
    int32_t causal;
    int32_t dtype;
    void* workspace;
    int64_t workspace_bytes;
    float* lse;                    /* optional (B, H, n_ctx) contiguous: natural-log row normalisers, what the
                                      backward pass needs (the reference keeps M, flash_attention.py:272-276) */
} ckv_dense_args;

int64_t ckv_dense_workspace_bytes(int64_t B, int64_t H, int64_t n_ctx, int64_t n_kv, int64_t D,
                                  int32_t dtype);

int ckv_attn_dense(const ckv_dense_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Backward of ckv_attn_dense: replaces _attention.backward -> _attn_bwd_preprocess / _attn_bwd
 * (flash_attention.py:279-537, 654-710).  Given the forward's inputs, its output and row normalisers and the
 * gradient of the output, writes dq, dk, dv (dtype and shapes of q, k, v); the scores carry no gradient, as
 * in the reference.  Masked cached keys receive zero gradients.  head_dim: a multiple of 16, up to 192 (anything
 * else, or a device whose workgroups get less LDS than the fp32 tiles of head_dim + 1 columns need, is refused with
 * CKV_ERR_UNSUPPORTED before anything is launched).  bf16 / fp16 tensors with head_dim 128, unit stride along the
 * head dim, every other stride a multiple of 8 elements and 16-byte aligned base addresses run on the matrix cores
 * (probabilities and dS rounded to the tensor dtype for the products, fp32 accumulation); everything else runs
 * fp32-math kernels.
 * ---------------------------------------------------------------------------------------- */
typedef struct ckv_dense_bwd_args {
    const void* q;                 /* (B, H, n_ctx, D) */
    int64_t q_stride[4];
    const void* k;                 /* (B, H, n_kv, D)  */
    const void* v;
    int64_t kv_stride[4];
    const uint8_t* mask;           /* (n_kv - n_ctx,) bool, 1 = masked; may be NULL if that is 0 */
    const void* out;               /* (B, H, n_ctx, D) forward output */
    int64_t out_stride[4];
    const float* lse;              /* (B, H, n_ctx) contiguous, from ckv_dense_args.lse */
    const void* dout;              /* (B, H, n_ctx, D) gradient of out */
    int64_t dout_stride[4];
    void* dq;                      /* (B, H, n_ctx, D) */
    int64_t dq_stride[4];
    void* dk;                      /* (B, H, n_kv, D)  */
    void* dv;
    int64_t dkv_stride[4];
    int64_t B, H, n_ctx, n_kv, D;
    float scale;
    int32_t dtype;
    void* workspace;
    int64_t workspace_bytes;
} ckv_dense_bwd_args;

int64_t ckv_dense_bwd_workspace_bytes(int64_t B, int64_t H, int64_t n_ctx);

int ckv_attn_dense_bwd(const ckv_dense_bwd_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Position ids of an incoming chunk (cascade_attention.py:114-150): q_pos[i] = i on the first call
 * of a sequence (key_pos and sink_pos NULL), otherwise i + 1 + max(max(key_pos[0..n_key)) + key_shift,
 * max(sink_pos[0..n_sink))) - stale and masked entries included, as in the reference.  One small
 * kernel on `stream`, no host synchronisation (the reference reads the maxima back to the host).
 * key_pos is the cache's position row (or its og_pos tensor with key_shift 0); either array may be
 * NULL / empty.
 * ---------------------------------------------------------------------------------------- */
int ckv_chunk_positions(const int64_t* key_pos, int64_t n_key, int64_t key_shift, const int64_t* sink_pos,
                        int64_t n_sink, int64_t q_len, int64_t* q_pos, void* stream);

/* ------------------------------------------------------------------------------------------
 * Stage timing (the reference's BENCHMARK=True switch, cascading_cache.py:986-1026, extended to
 * every kernel stage).  While enabled, each stage of ckv_attn / ckv_update is bracketed by HIP
 * events on the caller's stream; ckv_profile_read waits for them, ADDS the elapsed milliseconds
 * and launch counts per stage into the caller's arrays (length CKV_STAGE_COUNT) and forgets
 * them.  Process-wide and not thread-safe: a measurement aid, off by default.
 * ---------------------------------------------------------------------------------------- */
typedef enum ckv_stage {
    CKV_STAGE_PREP = 0,        /* rotate + gather prologue                      */
    CKV_STAGE_FWD = 1,         /* prefill attention forward (QK^T, softmax, PV) */
    CKV_STAGE_SCORES = 2,      /* prefill score sums (column pass)              */
    CKV_STAGE_FINISH = 3,      /* head reduction + EMA epilogue                 */
    CKV_STAGE_DECODE = 4,      /* decode attention main kernel                  */
    CKV_STAGE_DECODE_TAIL = 5, /* decode combine + scores                       */
    CKV_STAGE_PLAN = 6,        /* cache update: plan                            */
    CKV_STAGE_APPLY = 7,       /* cache update: apply                           */
    CKV_STAGE_COUNT = 8
} ckv_stage;

/* on: 0 = off, 1 = every stage bracketed by event records in the stream, 2 = only the attention main kernels
 * (CKV_STAGE_FWD, CKV_STAGE_DECODE), 3 = only the kernels of the cache update (CKV_STAGE_PLAN, CKV_STAGE_APPLY),
 * 4 = as 2, but only the first and then every fourth launch of each of the two kernels is timed (a timed dispatch
 * still costs a few microseconds around the kernel; `launches` counts the timed ones).
 * Levels 2 to 4 attach the events to the kernels' own dispatches: nothing is put between a kernel and its
 * neighbours, and the figures are kernel durations, fit for timing inside a throughput measurement. */
int ckv_profile_enable(int on);                       /* returns the previous setting */
int ckv_profile_read(double* ms, int64_t* launches);  /* both arrays CKV_STAGE_COUNT long */

/* human-readable text for a ckv_status (static storage, never NULL) */
const char* ckv_strerror(int status);

/* CKV_ABI_VERSION the library was built with */
int ckv_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* CKV_H_ */
