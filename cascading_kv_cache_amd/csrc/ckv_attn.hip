// ckv_attn / ckv_attn_dense: argument checking, workspace carving and kernel-family dispatch.
#include "ckv_attn_internal.h"

#include <math.h>

namespace ckv {
namespace {

struct Carver {
    char* base;
    int64_t off = 0;
    explicit Carver(void* b) : base(reinterpret_cast<char*>(b)) {}
    void* take(int64_t bytes) {
        void* p = base ? base + off : nullptr;
        off += align_up(bytes, 256);
        return p;
    }
};

struct AttnWorkspace {
    void *qr, *kr, *vc;
    unsigned long long* tile_vis;
    uint8_t* kmasked;
    float *lse, *lse2, *colsum, *w_ema, *w_new, *part_o, *part_l2;
    int64_t bytes;
};

AttnWorkspace carve_attn(void* base, int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t D, int64_t NS, int64_t S,
                         int dtype) {
    const int64_t es = elem_bytes(dtype), N = NS + S + Q, n_pad = mfma_n_pad(N);
    Carver c(base);
    AttnWorkspace w;
    w.qr = c.take((B * H * Q + kColSlack) * D * es);  // rows of slack for the MFMA column pass
    w.kr = c.take(B * KVH * n_pad * D * es);   // padded to whole key tiles for the MFMA family
    w.vc = c.take(B * KVH * n_pad * D * es);
    w.tile_vis = (unsigned long long*)c.take(n_pad / 64 * 8);
    w.kmasked = (uint8_t*)c.take(NS + S);
    w.lse = (float*)c.take(B * H * Q * 4);
    w.lse2 = (float*)c.take((B * H * Q + kColSlack) * 4);
    w.colsum = (float*)c.take(B * H * N * 4);
    w.w_ema = (float*)c.take((Q + kColSlack) * 4);
    w.w_new = (float*)c.take(Q * 4);
    // shares of the forward kernel when few query rows would leave the chip idle
    const int splits = mfma_supported(dtype, D, H, KVH, Q) && Q > 1 ? mfma_fwd_splits_for_workspace(B, H, KVH, Q, N) : 1;
    w.part_o = splits > 1 ? (float*)c.take(splits * B * H * Q * D * 4) : nullptr;
    w.part_l2 = splits > 1 ? (float*)c.take(splits * B * H * Q * 4) : nullptr;
    w.bytes = c.off;
    return w;
}

void contiguous_strides(int64_t* st, int64_t d1, int64_t d2, int64_t d3) {
    st[0] = d1 * d2 * d3;
    st[1] = d2 * d3;
    st[2] = d3;
    st[3] = 1;
}

}  // namespace
}  // namespace ckv

extern "C" int64_t ckv_attn_workspace_bytes(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t D, int64_t num_sink,
                                            int64_t S, int32_t dtype) {
    if (B <= 0 || H <= 0 || KVH <= 0 || Q <= 0 || D <= 0 || num_sink < 0 || S < 0) return 0;
    int64_t bytes = ckv::carve_attn(nullptr, B, H, KVH, Q, D, num_sink, S, dtype).bytes;
    if (Q == 1 && D == 128) {
        const int64_t dec = ckv::decode_workspace_bytes(B, H, KVH, num_sink, S);
        if (dec > bytes) bytes = dec;
    }
    return bytes;
}

extern "C" int ckv_attn(const ckv_attn_args* args, void* stream_) {
    using namespace ckv;
    if (!args) return CKV_ERR_NULL;
    const ckv_attn_args& a = *args;
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (a.dtype != CKV_F32 && a.dtype != CKV_F16 && a.dtype != CKV_BF16) return CKV_ERR_DTYPE;
    if (a.B <= 0 || a.H <= 0 || a.KVH <= 0 || a.Q <= 0 || a.D <= 0 || a.num_sink < 0 || a.S < 0) return CKV_ERR_SHAPE;
    if (a.H % a.KVH != 0 || a.D % 2 != 0) return CKV_ERR_SHAPE;
    if (a.head_reduction < CKV_REDUCE_MEAN || a.head_reduction > CKV_REDUCE_MEDIAN) return CKV_ERR_SHAPE;
    if ((a.homogeneous_heads ? a.H : a.H / a.KVH) > 128) return CKV_ERR_UNSUPPORTED;
    if (!a.q || !a.k_new || !a.v_new || !a.out || !a.q_pos) return CKV_ERR_NULL;
    if (a.num_sink > 0 && (!a.sink_k || !a.sink_v || !a.sink_mask || !a.sink_pos)) return CKV_ERR_NULL;
    if (a.S > 0 && (!a.cache_k || !a.cache_v || !a.mask || !a.pos)) return CKV_ERR_NULL;
    if (!(a.beta > 0.0) || !(a.beta <= 1.0)) return CKV_ERR_SHAPE;
    if (!(a.scale > 0.f)) return CKV_ERR_SHAPE;  // queries and keys are each multiplied by its square root
    if (!a.workspace || a.workspace_bytes < ckv_attn_workspace_bytes(a.B, a.H, a.KVH, a.Q, a.D, a.num_sink, a.S, a.dtype))
        return CKV_ERR_WORKSPACE;
    if (decode_supported(a)) return launch_decode(a, stream);
    AttnWorkspace w = carve_attn(a.workspace, a.B, a.H, a.KVH, a.Q, a.D, a.num_sink, a.S, a.dtype);

    const int64_t N = a.num_sink + a.S + a.Q;
    const bool want_scores = a.cache_s || a.new_scores;
    int rc;
    if (want_scores) {
        rc = launch_weights(w.w_ema, w.w_new, a.Q, a.beta, a.dtype, stream);
        if (rc) return rc;
    }
    const bool use_mfma = mfma_supported(a.dtype, a.D, a.H, a.KVH, a.Q) && a.Q > 1 && mfma_fits(N);
    if (use_mfma) {
        MfmaProblem mp;
        mp.seg[0] = MfmaSegment{a.sink_k, a.sink_v, {a.sink_stride[0], a.sink_stride[1], a.sink_stride[2], a.sink_stride[3]},
                                a.sink_pos, {a.sink_pos_stride[0], a.sink_pos_stride[1]}, 0, a.sink_mask, a.num_sink};
        mp.seg[1] = MfmaSegment{a.cache_k, a.cache_v,
                                {a.cache_stride[0], a.cache_stride[1], a.cache_stride[2], a.cache_stride[3]},
                                a.pos, {a.pos_stride[0], a.pos_stride[1]}, a.pos_shift, a.mask, a.S};
        mp.seg[2] = MfmaSegment{a.k_new, a.v_new,
                                {a.kv_new_stride[0], a.kv_new_stride[1], a.kv_new_stride[2], a.kv_new_stride[3]},
                                a.q_pos, {0, 0}, 0, nullptr, a.Q};
        mp.q = a.q;
        for (int i = 0; i < 4; i++) { mp.q_stride[i] = a.q_stride[i]; mp.out_stride[i] = a.out_stride[i]; }
        mp.q_pos = a.q_pos;
        mp.inv_freq = a.inv_freq;
        mp.theta = a.rope_theta;
        mp.shared_pos = a.sink_pos_stride[0] == 0 && a.sink_pos_stride[1] == 0 && a.pos_stride[0] == 0 &&
                        a.pos_stride[1] == 0;
        mp.qr = w.qr; mp.kr = w.kr; mp.vt = w.vc; mp.tile_vis = w.tile_vis;
        mp.out = a.out;
        mp.lse = w.lse;
        mp.lse2 = w.lse2;
        mp.colsum = want_scores ? w.colsum : nullptr;
        mp.part_o = w.part_o; mp.part_l2 = w.part_l2;
        mp.w_ema = w.w_ema; mp.w_new = w.w_new;
        mp.beta = a.beta;
        mp.new_mode = 1;
        mp.B = a.B; mp.H = a.H; mp.KVH = a.KVH; mp.Q = a.Q; mp.n = N; mp.n_pad = mfma_n_pad(N);
        mp.scale = a.scale;
        mp.key_scale = sqrtf(a.scale);
        mp.dtype = a.dtype;
        rc = launch_mfma(mp, stream);
        if (rc) return rc;
    } else {
        PrepProblem pp{&a, w.qr, w.kr, w.vc, w.kmasked};
        rc = launch_prep_generic(pp, stream);
        if (rc) return rc;

        CoreProblem cp;
        cp.q = w.qr;
        contiguous_strides(cp.q_stride, a.H, a.Q, a.D);
        cp.k = w.kr;
        cp.v = w.vc;
        contiguous_strides(cp.kv_stride, a.KVH, N, a.D);
        cp.kmasked = (a.num_sink + a.S) > 0 ? w.kmasked : nullptr;
        cp.out = a.out;
        for (int i = 0; i < 4; i++) cp.out_stride[i] = a.out_stride[i];
        cp.lse = w.lse;
        cp.colsum = want_scores ? w.colsum : nullptr;
        cp.w_ema = w.w_ema;
        cp.w_new = w.w_new;
        cp.new_mode = 1;
        cp.B = a.B; cp.H = a.H; cp.KVH = a.KVH; cp.Q = a.Q; cp.N = N; cp.D = a.D;
        cp.scale = 1.f;  // the staged queries and keys each carry sqrt(scale), rounded in as the eager path does
        cp.dtype = a.dtype;
        rc = launch_core_generic(cp, stream);
        if (rc) return rc;
    }
    if (a.lse) {
        CKV_HIP_TRY(hipMemcpyAsync(a.lse, w.lse, a.B * a.H * a.Q * sizeof(float), hipMemcpyDeviceToDevice, stream));
    }
    if (want_scores) {
        FinishProblem fp;
        fp.colsum = w.colsum;
        fp.N = N;
        fp.cache_s = a.S > 0 ? a.cache_s : nullptr;
        fp.new_scores = a.new_scores;
        for (int i = 0; i < 3; i++) {
            fp.cache_s_stride[i] = a.cache_s_stride[i];
            fp.new_scores_stride[i] = a.new_scores_stride[i];
        }
        fp.B = a.B; fp.H = a.H; fp.KVH = a.KVH; fp.Q = a.Q; fp.S = a.S; fp.num_sink = a.num_sink;
        fp.beta_pow_q = (float)pow(a.beta, (double)a.Q);
        fp.head_reduction = a.head_reduction;
        fp.homogeneous = a.homogeneous_heads;
        fp.dtype = a.dtype;
        rc = launch_finish(fp, stream);
        if (rc) return rc;
    }
    return CKV_OK;
}

namespace ckv {
// 16-bit, head_dim 128, more than one query row: the dense operator runs on the MFMA kernels too
static bool dense_uses_mfma(int dtype, int64_t D, int64_t H, int64_t n_ctx, int64_t n_kv) {
    return n_ctx > 1 && mfma_supported(dtype, D, H, H, n_ctx) && mfma_fits(n_kv);
}
}  // namespace ckv

extern "C" int64_t ckv_dense_workspace_bytes(int64_t B, int64_t H, int64_t n_ctx, int64_t n_kv, int64_t D,
                                             int32_t dtype) {
    if (B <= 0 || H <= 0 || n_ctx <= 0 || n_kv < n_ctx) return 0;
    using ckv::align_up;
    if (ckv::dense_uses_mfma(dtype, D, H, n_ctx, n_kv))  // staged Q / K / V^T and the column pass's scratch
        return ckv::carve_attn(nullptr, B, H, H, n_ctx, D, 0, n_kv - n_ctx, dtype).bytes;
    return align_up(B * H * n_ctx * 4, 256) + align_up(B * H * n_kv * 4, 256) + 2 * align_up((n_ctx + ckv::kColSlack) * 4, 256);
}

extern "C" int ckv_attn_dense(const ckv_dense_args* args, void* stream_) {
    using namespace ckv;
    if (!args) return CKV_ERR_NULL;
    const ckv_dense_args& a = *args;
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    if (a.dtype != CKV_F32 && a.dtype != CKV_F16 && a.dtype != CKV_BF16) return CKV_ERR_DTYPE;
    if (a.B <= 0 || a.H <= 0 || a.n_ctx <= 0 || a.n_kv < a.n_ctx || a.D <= 0) return CKV_ERR_SHAPE;
    if (!a.q || !a.k || !a.v || !a.out) return CKV_ERR_NULL;
    if (a.n_kv > a.n_ctx && !a.mask) return CKV_ERR_NULL;
    if (!(a.beta > 0.0) || !(a.beta <= 1.0)) return CKV_ERR_SHAPE;
    const int64_t need = ckv_dense_workspace_bytes(a.B, a.H, a.n_ctx, a.n_kv, a.D, a.dtype);
    if (!a.workspace || a.workspace_bytes < need) return CKV_ERR_WORKSPACE;
    if (dense_uses_mfma(a.dtype, a.D, a.H, a.n_ctx, a.n_kv)) {
        // keys and queries arrive rotated (no position ids); every head is its own kv head
        const int64_t n_cache = a.n_kv - a.n_ctx;
        AttnWorkspace w = carve_attn(a.workspace, a.B, a.H, a.H, a.n_ctx, a.D, 0, n_cache, a.dtype);
        int rc;
        if (a.scores) {
            rc = launch_weights(w.w_ema, w.w_new, a.n_ctx, a.beta, a.dtype, stream);
            if (rc) return rc;
        }
        const int64_t es = a.dtype == CKV_F32 ? 4 : 2;
        MfmaProblem mp;
        const MfmaSegment none{nullptr, nullptr, {0, 0, 0, 0}, nullptr, {0, 0}, 0, nullptr, 0};
        mp.seg[0] = MfmaSegment{a.k, a.v, {a.kv_stride[0], a.kv_stride[1], a.kv_stride[2], a.kv_stride[3]},
                                nullptr, {0, 0}, 0, n_cache > 0 ? a.mask : nullptr, n_cache};
        mp.seg[1] = none;
        mp.seg[2] = MfmaSegment{(const char*)a.k + n_cache * a.kv_stride[2] * es, (const char*)a.v + n_cache * a.kv_stride[2] * es,
                                {a.kv_stride[0], a.kv_stride[1], a.kv_stride[2], a.kv_stride[3]},
                                nullptr, {0, 0}, 0, nullptr, a.n_ctx};
        mp.q = a.q;
        for (int i = 0; i < 4; i++) { mp.q_stride[i] = a.q_stride[i]; mp.out_stride[i] = a.out_stride[i]; }
        mp.q_pos = nullptr;
        mp.inv_freq = nullptr;
        mp.theta = 1.f;
        mp.shared_pos = 1;
        mp.qr = w.qr; mp.kr = w.kr; mp.vt = w.vc; mp.tile_vis = w.tile_vis;
        mp.out = a.out;
        mp.lse = w.lse;
        mp.lse2 = w.lse2;
        mp.colsum = a.scores ? w.colsum : nullptr;
        mp.part_o = w.part_o; mp.part_l2 = w.part_l2;
        mp.w_ema = w.w_ema; mp.w_new = w.w_new;
        mp.beta = a.beta;
        mp.new_mode = 0;  // every key is weighted by the query row alone (flash_attention.py:73-77)
        mp.B = a.B; mp.H = a.H; mp.KVH = a.H; mp.Q = a.n_ctx; mp.n = a.n_kv; mp.n_pad = mfma_n_pad(a.n_kv);
        mp.scale = a.scale;
        mp.key_scale = 1.f;
        mp.dtype = a.dtype;
        rc = launch_mfma(mp, stream);
        if (rc) return rc;
        if (a.scores) {
            rc = launch_cast_scores(w.colsum, a.scores, a.scores_stride, a.B, a.H, a.n_kv, a.dtype, stream);
            if (rc) return rc;
        }
        if (a.lse) {
            CKV_HIP_TRY(hipMemcpyAsync(a.lse, w.lse, a.B * a.H * a.n_ctx * sizeof(float), hipMemcpyDeviceToDevice, stream));
        }
        return CKV_OK;
    }
    Carver c(a.workspace);
    float* lse = (float*)c.take(a.B * a.H * a.n_ctx * 4);
    if (a.lse) lse = a.lse;  // the forward kernel writes the caller's array directly
    float* colsum = (float*)c.take(a.B * a.H * a.n_kv * 4);
    float* w_ema = (float*)c.take((a.n_ctx + kColSlack) * 4);
    float* w_new = (float*)c.take(a.n_ctx * 4);
    int rc;
    if (a.scores) {
        rc = launch_weights(w_ema, w_new, a.n_ctx, a.beta, a.dtype, stream);
        if (rc) return rc;
    }
    CoreProblem cp;
    cp.q = a.q;
    cp.k = a.k;
    cp.v = a.v;
    for (int i = 0; i < 4; i++) {
        cp.q_stride[i] = a.q_stride[i];
        cp.kv_stride[i] = a.kv_stride[i];
        cp.out_stride[i] = a.out_stride[i];
    }
    cp.kmasked = a.n_kv > a.n_ctx ? a.mask : nullptr;
    cp.out = a.out;
    cp.lse = lse;
    cp.colsum = a.scores ? colsum : nullptr;
    cp.w_ema = w_ema;
    cp.w_new = w_new;
    cp.new_mode = 0;  // every key is weighted by the query row alone (flash_attention.py:73-77)
    cp.B = a.B; cp.H = a.H; cp.KVH = a.H; cp.Q = a.n_ctx; cp.N = a.n_kv; cp.D = a.D;
    cp.scale = a.scale;
    cp.dtype = a.dtype;
    rc = launch_core_generic(cp, stream);
    if (rc) return rc;
    if (a.scores) {
        rc = launch_cast_scores(colsum, a.scores, a.scores_stride, a.B, a.H, a.n_kv, a.dtype, stream);
        if (rc) return rc;
    }
    return CKV_OK;
}
