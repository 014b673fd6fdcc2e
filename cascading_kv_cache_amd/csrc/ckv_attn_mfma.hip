// bf16 / fp16 MFMA attention for head_dim 128 on gfx950 (CDNA4, wave64, v_mfma_f32_32x32x16).
//
// Stages (all stream-ordered):
//   stage_keys   rotate K on the way into a padded row-major buffer Kr, transpose V into 64-key
//                tiles Vt[tile][d][key'] (key' = the order the PV MFMA consumes), build one 64-bit
//                visibility word per key tile.  cos/sin are computed once per key and reused for
//                every (batch, kv-head) that shares the position row.
//   stage_q      rotate Q and fold the softmax scale (times log2 e) in.
//   fwd          flash forward, software pipelined.  One workgroup = one kv head x 256 (head,
//                position) rows, so the G query heads of a group share every K/V tile staged in
//                LDS.  S^T = K Q^T keeps a query in one lane pair: the row max / sum need a single
//                cross-half exchange and exp2(S^T) is already laid out as the B operand of
//                O^T += V^T P^T.  The softmax of tile i runs beside the logits of tile i+1 and the
//                P.V product of tile i-1.
//   colsum       exact score sums.  One workgroup = one head x 256 keys held in registers; the
//                queries stream through LDS, the accumulators start from minus the final
//                normaliser so the matrix pipe returns log2 P, and the weighted column sums stay
//                inside a lane (S = Q K^T orientation).
#include "ckv_attn_internal.h"

#include <cstring>
#include <type_traits>

namespace ckv {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kD = 128;    // head dim
constexpr int kBN = 64;    // keys per tile

constexpr int kRows = 256;    // (head, position) rows per forward workgroup

template <typename T>
struct Mma;
template <>
struct Mma<__hip_bfloat16> {
    __device__ static f32x16 mma(uint4 a, uint4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
    __device__ static uint32_t pack2(float lo, float hi) {
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    __device__ static float round1(float v) {
        f32x2 f = {v, 0.f};
        const uint32_t u = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
        return __uint_as_float(u << 16);
    }
    // the two elements of a packed pair as floats
    __device__ static float lo_f(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static float hi_f(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    // acc + both halves of a packed pair (one v_dot2c with a pair of ones)
    __device__ static float sum2(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
    }
};
template <>
struct Mma<__half> {
    __device__ static f32x16 mma(uint4 a, uint4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    __device__ static uint32_t pack2(float lo, float hi) {
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    __device__ static float round1(float v) { return (float)(_Float16)v; }
    __device__ static float lo_f(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
    __device__ static float hi_f(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
    __device__ static float sum2(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), __builtin_bit_cast(f16x2, 0x3c003c00u), acc, false);
    }
};

// position of key `k` (0..63) of a tile inside a V^T row: the PV contraction step s covers keys
// 16s..16s+15; lane half h supplies keys 16s + 8a + 4h + e (a = 0,1; e = 0..3) as elements 4a+e
__host__ __device__ inline int vt_slot(int k) {
    const int s = k >> 4, a = (k >> 3) & 1, h = (k >> 2) & 1, e = k & 3;
    return 16 * s + 8 * h + 4 * a + e;
}

// ---------------------------------------------------------------------------------------------
// staging
// ---------------------------------------------------------------------------------------------
struct KeySegment {
    const void* k;
    const void* v;
    int64_t stride[4];       // (B, KVH, len, D)
    const int64_t* pos;      // position ids, or null when keys are already rotated
    int64_t pos_stride[2];
    int64_t pos_shift;
    const uint8_t* masked;   // 1 = masked, or null (all visible)
    int64_t len;
};

struct StageParams {
    KeySegment seg[3];
    const float* inv_freq;
    float theta;
    float key_scale;         // rotated keys are multiplied by this and rounded again (1: they are not)
    int shared_pos;          // every (b, kvh) uses position row [0, 0]
    void* kr;                // (B*KVH, n_pad/64) K tile images, see k_image_off
    void* vt;                // (B*KVH, n_pad/64) V^T tile images, see v_image_off
    unsigned long long* tile_vis;  // (n_pad/64,)
    int64_t B, KVH, n, n_pad;
};

__device__ inline int find_segment(const StageParams& p, int64_t n, int64_t& local) {
    if (n < p.seg[0].len) { local = n; return 0; }
    n -= p.seg[0].len;
    if (n < p.seg[1].len) { local = n; return 1; }
    local = n - p.seg[1].len;
    return 2;
}

// The staged K and V of one 64-key tile are 16 KiB images in exactly the order the forward kernel
// keeps them in LDS, so a tile reaches LDS as a straight copy and the 64 lanes of an operand read
// touch 1 KiB made of two contiguous halves (no bank conflicts, one base address per lane):
//   K image:   16-byte piece c (elements 8c .. 8c+7) of key row r at  (c/2)*2048 + (c%2)*1024 + r*16
//   V^T image: 16-byte piece c (key slots 8c .. 8c+7) of dim row d at (c/2)*4096 + (c%2)*2048 + d*16
// Key slot 16s + 8h + 4a + e of a V^T row holds key 16s + 8a + 4h + e of the tile: the order in
// which the logits leave the matrix pipe.
__device__ __host__ inline int k_image_off(int r, int c) { return (c >> 1) * 2048 + (c & 1) * 1024 + r * 16; }
__device__ __host__ inline int v_image_off(int d, int c) { return (c >> 1) * 4096 + (c & 1) * 2048 + d * 16; }

// One block of 256 threads stages key tile `tile_i` for the (b, kvh) units split_i, split_i + n_split, ...:
// thread = (key = tid/4, quarter = tid%4) owns rotation pairs j = 8q .. 8q+7 and 32+8q .. 32+8q+7, i.e. the
// 16-byte pieces q, 4+q, 8+q and 12+q of its row: the four threads of a row read (and, for queries, write)
// 64 contiguous bytes per instruction.
__device__ inline int stage_pair(int quarter, int i) { return i < 8 ? 8 * quarter + i : 24 + 8 * quarter + i; }
template <typename T>
__device__ inline void stage_keys_block(const StageParams& p, int tile_i, int split_i, int n_split, uint32_t (*v_lds)[kD / 2 + 1]) {
    const int tid = threadIdx.x;
    const int key = tid >> 2, quarter = tid & 3;
    const int64_t tile = tile_i;
    const int64_t n = tile * kBN + key;
    int64_t local = 0;
    const int sidx = n < p.n ? find_segment(p, n, local) : -1;

    if (split_i == 0 && tid < kBN) {  // visibility word of this tile
        const int64_t nn = tile * kBN + tid;
        bool vis = nn < p.n;
        if (vis) {
            int64_t loc;
            const int si = find_segment(p, nn, loc);
            if (p.seg[si].masked) vis = p.seg[si].masked[loc] == 0;
        }
        const unsigned long long bal = __ballot(vis);
        if (tid == 0) p.tile_vis[tile] = bal;
    }

    // cos / sin of this thread's 16 rotation pairs, two per word, rounded to the tensor dtype (see RopeWord)
    RopeWord<T> rw[8];
    auto trig_at = [&](int64_t pos) {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            float sn[2], cs[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int j = stage_pair(quarter, 2 * k + e);
                const float f = p.inv_freq ? p.inv_freq[j] : 1.0f / powf(p.theta, (float)(2 * j) / (float)kD);
                fast_sincos(__fmul_rn((float)pos, f), &sn[e], &cs[e]);
            }
            rw[k] = RopeWord<T>::make(cs[0], sn[0], cs[1], sn[1]);
        }
    };
    const bool rotate = sidx >= 0 && p.seg[sidx].pos != nullptr;
    if (rotate && p.shared_pos) trig_at(p.seg[sidx].pos[local] + p.seg[sidx].pos_shift);
    const bool key_scaled = p.key_scale != 1.0f;
    const int64_t nbh = p.B * p.KVH;
    // the rows of unit bh as this thread's eight 16-byte pieces (zeros past the last key)
    struct Rows {
        uint4 lo[2], hi[2], vlo[2], vhi[2];
    };
    auto load_rows = [&](int64_t bh, Rows& r) {
        r.lo[0] = r.lo[1] = r.hi[0] = r.hi[1] = r.vlo[0] = r.vlo[1] = r.vhi[0] = r.vhi[1] = make_uint4(0, 0, 0, 0);
        if (sidx < 0 || bh >= nbh) return;
        const int64_t b = bh / p.KVH, kvh = bh % p.KVH;
        const KeySegment& sg = p.seg[sidx];
        const int64_t off = b * sg.stride[0] + kvh * sg.stride[1] + local * sg.stride[2];
        const T* kp = (const T*)sg.k + off;
        const T* vp = (const T*)sg.v + off;
        if (sg.stride[3] == 1 && ((reinterpret_cast<uintptr_t>(kp) | reinterpret_cast<uintptr_t>(vp)) & 15) == 0) {
            r.lo[0] = *reinterpret_cast<const uint4*>(kp + 8 * quarter);
            r.lo[1] = *reinterpret_cast<const uint4*>(kp + 32 + 8 * quarter);
            r.hi[0] = *reinterpret_cast<const uint4*>(kp + 64 + 8 * quarter);
            r.hi[1] = *reinterpret_cast<const uint4*>(kp + 96 + 8 * quarter);
            r.vlo[0] = *reinterpret_cast<const uint4*>(vp + 8 * quarter);
            r.vlo[1] = *reinterpret_cast<const uint4*>(vp + 32 + 8 * quarter);
            r.vhi[0] = *reinterpret_cast<const uint4*>(vp + 64 + 8 * quarter);
            r.vhi[1] = *reinterpret_cast<const uint4*>(vp + 96 + 8 * quarter);
        } else {
            T* l0 = reinterpret_cast<T*>(r.lo);
            T* h0 = reinterpret_cast<T*>(r.hi);
            T* vl = reinterpret_cast<T*>(r.vlo);
            T* vh = reinterpret_cast<T*>(r.vhi);
            for (int i = 0; i < 16; i++) {
                l0[i] = kp[stage_pair(quarter, i) * sg.stride[3]];
                h0[i] = kp[(64 + stage_pair(quarter, i)) * sg.stride[3]];
                vl[i] = vp[stage_pair(quarter, i) * sg.stride[3]];
                vh[i] = vp[(64 + stage_pair(quarter, i)) * sg.stride[3]];
            }
        }
    };
    // The rows of the next unit are requested before this unit's rotation, transposition and stores, so
    // the workgroup always has loads in flight.
    Rows nxt;
    load_rows(split_i, nxt);
    for (int64_t bh = split_i; bh < nbh; bh += n_split) {
        const int64_t b = bh / p.KVH, kvh = bh % p.KVH;
        Rows cur = nxt;
        load_rows(bh + n_split, nxt);
        uint4(&lo)[2] = cur.lo;
        uint4(&hi)[2] = cur.hi;
        uint4(&vlo)[2] = cur.vlo;
        uint4(&vhi)[2] = cur.vhi;
        if (sidx >= 0) {
            const KeySegment& sg = p.seg[sidx];
            if (rotate) {
                if (!p.shared_pos)
                    trig_at(sg.pos[b * sg.pos_stride[0] + kvh * sg.pos_stride[1] + local] + sg.pos_shift);
                uint32_t* lw = reinterpret_cast<uint32_t*>(lo);
                uint32_t* hw = reinterpret_cast<uint32_t*>(hi);
#pragma unroll
                for (int k = 0; k < 8; k++) rw[k].rotate(lw[k], hw[k], p.key_scale, key_scaled, lw[k], hw[k]);
            }
        }
        char* kimg = (char*)p.kr + (bh * (p.n_pad / kBN) + tile) * (int64_t)(kD * kBN * sizeof(T));
        *reinterpret_cast<uint4*>(kimg + k_image_off(key, quarter)) = lo[0];
        *reinterpret_cast<uint4*>(kimg + k_image_off(key, 4 + quarter)) = lo[1];
        *reinterpret_cast<uint4*>(kimg + k_image_off(key, 8 + quarter)) = hi[0];
        *reinterpret_cast<uint4*>(kimg + k_image_off(key, 12 + quarter)) = hi[1];

        // V: through LDS into the transposed tile.  A thread holds elements j and j + 64 of its key row for
        // the same 16 values of j, so the two travel as one dword: 16 four-byte LDS writes per thread, and on
        // the way out thread (j, group of 16 key slots) reads 16 dwords and owns 32 bytes of dim row j and of
        // dim row j + 64, which the 64 lanes of a wavefront store as 1 KiB runs of the image.
        __syncthreads();
        {
            const uint16_t* vl = reinterpret_cast<const uint16_t*>(vlo);
            const uint16_t* vh = reinterpret_cast<const uint16_t*>(vhi);
#pragma unroll
            for (int i = 0; i < 16; i++) v_lds[key][stage_pair(quarter, i)] = (uint32_t)vl[i] | ((uint32_t)vh[i] << 16);
        }
        __syncthreads();
        char* vimg = (char*)p.vt + (bh * (p.n_pad / kBN) + tile) * (int64_t)(kD * kBN * sizeof(T));
        {
            const int j = tid & 63, g = tid >> 6;
            uint32_t w[16];
#pragma unroll
            for (int sl = 0; sl < 16; sl++) {
                // inverse of vt_slot: slot = 16g + 8h + 4a + e  ->  key = 16g + 8a + 4h + e
                const int h = (sl >> 3) & 1, a = (sl >> 2) & 1, e = sl & 3;
                w[sl] = v_lds[16 * g + 8 * a + 4 * h + e][j];
            }
            uint32_t lo_row[8], hi_row[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                lo_row[k] = (w[2 * k] & 0xffffu) | (w[2 * k + 1] << 16);
                hi_row[k] = (w[2 * k] >> 16) | (w[2 * k + 1] & 0xffff0000u);
            }
#pragma unroll
            for (int i = 0; i < 2; i++) {
                *reinterpret_cast<uint4*>(vimg + v_image_off(j, 2 * g + i)) =
                    make_uint4(lo_row[4 * i], lo_row[4 * i + 1], lo_row[4 * i + 2], lo_row[4 * i + 3]);
                *reinterpret_cast<uint4*>(vimg + v_image_off(j + 64, 2 * g + i)) =
                    make_uint4(hi_row[4 * i], hi_row[4 * i + 1], hi_row[4 * i + 2], hi_row[4 * i + 3]);
            }
        }
    }
}

struct StageQParams {
    const void* q;
    int64_t stride[4];
    const int64_t* q_pos;    // null: copy only
    const float* inv_freq;
    float theta;
    void* qr;                // (B*H, Q, D) contiguous
    int64_t rows;            // B*H*Q
    int64_t H, Q;
    float qscale;            // folded into the staged queries: softmax scale * log2(e), over the factor the keys carry
    int vec;                 // source rows can be read 16 bytes at a time
};

// thread = (position m, quarter of the rotation pairs); the cos/sin of the position are computed once
// and reused for the batch x head rows share_i, share_i + n_share, ...; a block of 256 threads covers
// positions 64 blk .. 64 blk + 63
template <typename T>
__device__ inline void stage_q_block(const StageQParams& p, int blk, int share_i, int n_share) {
    const int64_t idx = (int64_t)blk * 256 + threadIdx.x;
    const int64_t m = idx >> 2;
    const int quarter = idx & 3;
    if (m >= p.Q) return;
    RopeWord<T> rw[8];
    if (p.q_pos) {
        const int64_t pos = p.q_pos[m];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            float sn[2], cs[2];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int j = stage_pair(quarter, 2 * k + e);
                const float f = p.inv_freq ? p.inv_freq[j] : 1.0f / powf(p.theta, (float)(2 * j) / (float)kD);
                fast_sincos(__fmul_rn((float)pos, f), &sn[e], &cs[e]);
            }
            rw[k] = RopeWord<T>::make(cs[0], sn[0], cs[1], sn[1]);
        }
    }
    const int64_t nbh = p.rows / p.Q;
    struct Row {
        T lo[16], hi[16];
    };
    auto load_row = [&](int64_t bh, Row& r) {
        if (bh >= nbh) return;
        const int64_t b = bh / p.H, h = bh % p.H;
        const T* src = (const T*)p.q + b * p.stride[0] + h * p.stride[1] + m * p.stride[2];
        if (p.vec) {  // unit stride and 16-byte aligned rows
            reinterpret_cast<uint4*>(r.lo)[0] = *reinterpret_cast<const uint4*>(src + 8 * quarter);
            reinterpret_cast<uint4*>(r.lo)[1] = *reinterpret_cast<const uint4*>(src + 32 + 8 * quarter);
            reinterpret_cast<uint4*>(r.hi)[0] = *reinterpret_cast<const uint4*>(src + 64 + 8 * quarter);
            reinterpret_cast<uint4*>(r.hi)[1] = *reinterpret_cast<const uint4*>(src + 96 + 8 * quarter);
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                r.lo[i] = src[stage_pair(quarter, i) * p.stride[3]];
                r.hi[i] = src[(64 + stage_pair(quarter, i)) * p.stride[3]];
            }
        }
    };
    // the softmax scale (times log2 e) rides on the staged queries, so the attention kernels exponentiate the
    // products as they come out of the matrix pipe: rotated with the eager path's roundings, then one rounding
    // of the product with qscale (the eager path rounds the product with sqrt(scale) there; log2 e has to ride
    // on one of the two operands, and noise on a query averages out over the rows a score sums)
    auto finish_row = [&](int64_t bh, Row& r) {
        if (bh >= nbh) return;
        uint32_t* lw = reinterpret_cast<uint32_t*>(r.lo);
        uint32_t* hw = reinterpret_cast<uint32_t*>(r.hi);
#pragma unroll
        for (int k = 0; k < 8; k++) {  // on packed pairs, as in stage_keys_block
            if (p.q_pos) {
                rw[k].rotate(lw[k], hw[k], p.qscale, true, lw[k], hw[k]);
            } else {
                lw[k] = Mma<T>::pack2(Mma<T>::lo_f(lw[k]) * p.qscale, Mma<T>::hi_f(lw[k]) * p.qscale);
                hw[k] = Mma<T>::pack2(Mma<T>::lo_f(hw[k]) * p.qscale, Mma<T>::hi_f(hw[k]) * p.qscale);
            }
        }
        T* dst = (T*)p.qr + (bh * p.Q + m) * kD;
        *reinterpret_cast<uint4*>(dst + 8 * quarter) = reinterpret_cast<uint4*>(r.lo)[0];
        *reinterpret_cast<uint4*>(dst + 32 + 8 * quarter) = reinterpret_cast<uint4*>(r.lo)[1];
        *reinterpret_cast<uint4*>(dst + 64 + 8 * quarter) = reinterpret_cast<uint4*>(r.hi)[0];
        *reinterpret_cast<uint4*>(dst + 96 + 8 * quarter) = reinterpret_cast<uint4*>(r.hi)[1];
    };
    // two rows per trip, both requested before either is rotated: a block is a chain of trips to
    // memory, and this halves it
    for (int64_t bh = share_i; bh < nbh; bh += 2 * n_share) {
        Row r0, r1;
        load_row(bh, r0);
        load_row(bh + n_share, r1);
        finish_row(bh, r0);
        finish_row(bh + n_share, r1);
    }
}

// One launch stages queries and keys: the two are independent.  1-D grid: the key blocks (k_bx x k_by)
// first, then the query blocks (q_bx x q_by), which are short and fill the ragged end of the key blocks.
struct StageGrid {
    int q_bx, q_by, k_bx, k_by;
};
template <typename T>
__global__ void __launch_bounds__(256) stage_kernel(StageParams sp, StageQParams sq, StageGrid g) {
    __shared__ uint32_t v_lds[kBN][kD / 2 + 1];  // (d, d + 64) pairs of a key row, odd pitch
    const int nk = g.k_bx * g.k_by;
    int id = blockIdx.x;
    if (id < nk) {
        stage_keys_block<T>(sp, id % g.k_bx, id / g.k_bx, g.k_by, v_lds);
    } else {
        id -= nk;
        stage_q_block<T>(sq, id % g.q_bx, id / g.q_bx, g.q_by);
    }
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
struct FwdParams {
    const void* qr;   // (B*H, Q, D)
    const void* kr;   // (B*KVH, n_pad/64) K tile images
    const void* vt;   // (B*KVH, n_pad/64) V^T tile images
    const unsigned long long* tile_vis;
    void* out;
    int64_t out_stride[4];
    float* lse;       // (B*H, Q) natural log
    float* lse2;      // (B*H, Q) minus the log2-domain normaliser, consumed by the column pass
    int64_t B, H, KVH, Q, N, Nc, n_pad;
    int G;            // heads per kv head: a workgroup takes 256 consecutive rows of the kv head's (position, head) pairs, position-major
    float scale_log2; // softmax scale * log2(e)
    int n_qt, xcd_aware;  // query tiles per kv head; 1-D XCD-aware block order
    // Few query rows (short chunks, one stream) would leave most of the chip idle: the key tiles of a query tile
    // are then dealt out over n_split workgroups, each of which leaves a partial result (its rows normalised by
    // its own sums, fp32) and the log2-domain normaliser of its share; a small kernel merges them.
    int n_split;
    float* part_o;    // (n_split, B*H*Q, D)
    float* part_l2;   // (n_split, B*H*Q): m_ref + log2(l) of the share, -inf when it holds no visible key
};

// LDS tile of 256-byte rows taken from a row-major matrix (the query tile of the column pass): unpadded
// (the async copy writes 1 KiB per wavefront contiguously); bank conflicts are avoided by XOR-swizzling
// the 16-byte piece index with the row: piece c of row r lives at r*256 + ((c ^ (r & 15)) << 4)
__device__ inline int k_lds_off(int r, int c) { return r * 256 + ((c ^ (r & 15)) << 4); }

// max over the two lane halves (lane l and lane l ^ 32) without a trip through LDS
__device__ inline float half_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// Software-pipelined forward: eight wavefronts, 32 (head, position) rows each.  Iteration i runs
// the softmax of tile i on the vector ALU while the matrix pipe adds the P.V product of tile i-1
// and computes the logits of tile i+1; neither depends on the softmax in flight, so the two pipes
// overlap inside one wavefront.  LDS: three K stages and four V^T stages.  Iteration i copies K
// tile i+3 and V^T tile i+2, which are first read in iteration i+2: the barrier between two
// iterations waits only for the copies of the iteration before the last one (those of the last one
// stay in flight across it), and the first operands of an iteration can be fetched before its barrier.
constexpr int kPipeStage = 16384;
constexpr int kKStages = 3, kVStages = 4;
constexpr int kPipeLds = (kKStages + kVStages) * kPipeStage;   // K0 K1 K2 V0 V1 V2 V3
// stages, one visibility word and one work-list entry per key tile, the list length
inline int64_t pipe_lds_bytes(int64_t n_pad) { return kPipeLds + (n_pad / kBN) * 12 + 16; }
constexpr int64_t kLdsLimit = 160 * 1024;

template <typename T>
__global__ void __launch_bounds__(512) fwd_pipe_kernel(FwdParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int kThreads = 512, kBlocksPerWave = 2, kAhead = 3;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, half = lane >> 5;
    int bkv_i = blockIdx.y, qt_i = blockIdx.x;
    // With 8 | B * KVH the grid is 1-D: workgroup ids go round the 8 XCDs, and all query tiles of a kv
    // head are put on one XCD, so its K / V^T stream is fetched from HBM into one L2 instead of eight
    // (same run time, a fifth of the HBM reads).
    if (p.xcd_aware) {
        const int id = blockIdx.x, jq = id >> 3, per = p.n_qt * p.n_split;
        bkv_i = (id & 7) + 8 * (jq / per);
        qt_i = jq % per;
    }
    const int split_i = qt_i % p.n_split;   // this workgroup's share of the query tile's key tiles
    qt_i /= p.n_split;
    // Later query tiles see more chunk keys, so they go first: the compute units that finish the light
    // tiles of one round early pick up the heavy tiles of the next (two rounds of workgroups then cost
    // light + heavy everywhere instead of heavy + heavy on the slowest unit).
    qt_i = p.n_qt - 1 - qt_i;
    const int64_t bkv = bkv_i;
    const int64_t b = bkv / p.KVH, kvh = bkv % p.KVH;
    // rows of a kv head are its (position, head) pairs, position-major: row rf = position * G + head.  A workgroup
    // takes 256 consecutive ones whatever G is (7 heads per kv head: 36 4/7 positions), so every wavefront has
    // 32 real rows and the number of workgroups is Q * G / 256, not Q / floor(256 / G).
    const int m0 = qt_i * kRows / p.G;
    int m_hi = (qt_i * kRows + kRows - 1) / p.G;
    if (m_hi > (int)p.Q - 1) m_hi = (int)p.Q - 1;
    const int n_tiles = (int)((p.Nc + m_hi) / kBN) + 1;
    const int tiles_cap = (int)(p.n_pad / kBN);
    unsigned long long* vis_lds = reinterpret_cast<unsigned long long*>(smem + kPipeLds);
    int* list_lds = reinterpret_cast<int*>(smem + kPipeLds + 8 * tiles_cap);
    const uint32_t smem_addr = lds_address(smem);

    // ---- work list: tiles with at least one visible key; bit 31 marks tiles that need masking
    for (int i = tid; i < n_tiles; i += kThreads) vis_lds[i] = p.tile_vis[i];
    __syncthreads();
    if (wave == 0) {
        int cnt = 0;
        for (int base = 0; base < n_tiles; base += 64) {
            const int t = base + lane;
            const unsigned long long v = t < n_tiles ? vis_lds[t] : 0ull;
            const unsigned long long bal = __ballot(v != 0ull);
            if (v != 0ull) {
                const bool partial = (v != ~0ull) || (t * kBN + kBN - 1 - (int)p.Nc > m0);
                list_lds[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = t | (partial ? (int)0x80000000 : 0);
            }
            cnt += __popcll(bal);
        }
        if (lane == 0) list_lds[tiles_cap] = cnt;
    }
    __syncthreads();
    const int n_work_all = __builtin_amdgcn_readfirstlane(list_lds[tiles_cap]);
    const int j_first = n_work_all * split_i / p.n_split;
    const int n_work = n_work_all * (split_i + 1) / p.n_split - j_first;
    list_lds += j_first;

    // ---- the query row this lane owns as MFMA column `col`
    int row_m;
    uint4 qreg[8];
    {
        const int rf = qt_i * kRows + wave * 32 + col;
        const int g = rf % p.G;
        row_m = rf / p.G;
        const int64_t row_h = kvh * p.G + g;
        const bool row_ok = row_m < p.Q;
        const T* qrow = (const T*)p.qr + ((b * p.H + row_h) * p.Q + row_m) * kD;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            qreg[kk] = row_ok ? *reinterpret_cast<const uint4*>(qrow + 16 * kk + 8 * half) : make_uint4(0, 0, 0, 0);
        }
    }
    f32x16 oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[dt][v] = 0.f;
    // m_ref: the reference the row's logits and sums are relative to; m_run: running maximum relative to it
    // (-inf until the row has seen a key); l_run: partial over this lane's keys, halves are added at the end
    float m_ref = 0.f, m_run = -INFINITY, l_run = 0.f;
    f32x16 cinit;  // -m_ref in every element: what the matrix pipe starts a tile's logits from
#pragma unroll
    for (int v = 0; v < 16; v++) cinit[v] = 0.f;
    constexpr float kShiftAt = 10.f;  // probabilities stay below 2^10 between two moves of the reference

    // ---- LDS byte offset of this lane's operand pieces inside the stage being read (pieces of later
    // contraction steps / row blocks are at compile-time distances); moved from stage to stage in place.
    // k_base: key row `col` of the K stage with the next logits' tile; v_base: dim row `col` of the V^T
    // stage with the tile to multiply.
    int k_base = k_image_off(col, half);
    int v_base = v_image_off(col, half) + (kKStages + kVStages - 1) * kPipeStage;
    int k_rd = 0, v_rd = kVStages - 1;  // the stages k_base / v_base point at
    auto advance_k = [&]() {
        k_base += k_rd == kKStages - 1 ? -(kKStages - 1) * kPipeStage : kPipeStage;
        k_rd = k_rd == kKStages - 1 ? 0 : k_rd + 1;
    };
    auto advance_v = [&]() {
        v_base += v_rd == kVStages - 1 ? -(kVStages - 1) * kPipeStage : kPipeStage;
        v_rd = v_rd == kVStages - 1 ? 0 : v_rd + 1;
    };
    // K piece (kk, ks): contraction step kk of key rows 32ks ..; V^T piece (s, dt): step s of dim rows 32dt ..
    auto k_piece = [&](int kk, int ks) { return *reinterpret_cast<const uint4*>(smem + k_base + kk * 2048 + ks * 512); };
    auto v_piece = [&](int s_, int dt) { return *reinterpret_cast<const uint4*>(smem + v_base + s_ * 4096 + dt * 512); };
    const uint32_t copy_off = lane * 16;  // a wavefront copies 1 KiB blocks of an image as they are
    const char* kbase = (const char*)uniform_ptr((const char*)p.kr + bkv * p.n_pad * kD * (int64_t)sizeof(T));
    const char* vbase = (const char*)uniform_ptr((const char*)p.vt + bkv * p.n_pad * kD * (int64_t)sizeof(T));
    constexpr int kTileBytes = kBN * kD * (int)sizeof(T);

    // one 1 KiB block (j = 0, 1) of a tile into K stage `stage` / V^T stage `stage`
    auto copy_k = [&](int t, int stage, int j) {
        const int blk = (wave * kBlocksPerWave + j) * 1024;
        async_copy16(kbase + (int64_t)t * kTileBytes + blk, copy_off, smem_addr + stage * kPipeStage + blk);
    };
    auto copy_v = [&](int t, int stage, int j) {
        const int blk = (wave * kBlocksPerWave + j) * 1024;
        async_copy16(vbase + (int64_t)t * kTileBytes + blk, copy_off, smem_addr + (kKStages + stage) * kPipeStage + blk);
    };
    auto work = [&](int j) { return __builtin_amdgcn_readfirstlane(list_lds[j < n_work ? j : n_work - 1]); };

    // logits of the K tile k_base points at: s[ks][v] = key 32ks + 8(v/4) + 4half + v%4, query column col
    auto qk = [&](f32x16(&s)[2]) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++) s[ks] = cinit;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                s[ks] = Mma<T>::mma(k_piece(kk, ks), qreg[kk], s[ks]);
            }
        }
    };
    uint32_t pk[4][4];  // P^T of one tile as the B operands of the four P.V contraction steps
    // O^T += V^T P^T with the V^T tile v_base points at
    auto pv = [&]() {
#pragma unroll
        for (int s = 0; s < 4; s++) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const uint4 a = v_piece(s, dt);
                const uint4 bq = make_uint4(pk[s][0], pk[s][1], pk[s][2], pk[s][3]);
                oacc[dt] = Mma<T>::mma(a, bq, oacc[dt]);
            }
        }
    };
    // One 64-bit word per lane says which keys of the tile its query row may see (visible slot and not
    // later than the row); it is shifted once so that the bit of every element sits at a compile-time
    // position.  Few live values: this path must not push the loop's registers into scratch.
    auto mask_tile = [&](int entry, f32x16(&s)[2]) {
        const int t = entry & 0x7fffffff;
        unsigned long long allowed = vis_lds[t];
        const int limit = row_m - (t * kBN - (int)p.Nc);  // last key index of the tile the row may see, if it is a chunk tile
        if (t * kBN + kBN - 1 >= (int)p.Nc) {             // the tile holds chunk keys
            const int first_chunk = (int)p.Nc - t * kBN;  // <= 0 when the whole tile is chunk
            unsigned long long causal = limit >= 63 ? ~0ull : (limit < 0 ? 0ull : ((2ull << limit) - 1ull));
            if (first_chunk > 0) causal |= (1ull << first_chunk) - 1ull;  // cached keys in front of the chunk: always allowed
            allowed &= causal;
        }
        allowed >>= 4 * half;
        const uint32_t lo = (uint32_t)allowed, hi = (uint32_t)(allowed >> 32);
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int bit = 8 * (v >> 2) + (v & 3);  // key 32 ks + bit + 4 half
                const bool ok = ((ks ? hi : lo) >> bit) & 1u;
                s[ks][v] = ok ? s[ks][v] : -INFINITY;
            }
    };
    float alpha = 1.f;  // rescale of the accumulator owed since the last softmax
    // the running maximum settles after a few tiles: rescale only when some row of the wavefront moved
    auto rescale = [&]() {
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0ull) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int v = 0; v < 16; v++) oacc[dt][v] *= alpha;
        }
    };

    // Iteration i, written in issue order: 32 slots, each one matrix instruction (slots 0..15: P.V of
    // tile i-1 out of the V^T stage at v_base, slots 16..31: logits of tile i+1 out of the K stage at
    // k_base), the LDS read of the operand kAhead slots ahead, and a slice of the softmax of tile i.
    // Scheduling barriers keep the slots as written, so matrix and vector instructions alternate
    // inside the wavefront.  The probabilities of tile i overwrite those of tile i-1 piece by piece,
    // each after its last use by the P.V product.  The copies (V^T tile t_v = i+2 into stage v_wr, K
    // tile t_k = i+3 into stage k_wr, both last read in iteration i-1) go out one at a time, a quarter
    // of the slots apart.
    // pre[]: on entry the operands of slots 0..kAhead-1, read before the barrier; on exit those
    // of the next iteration.
    // fetch_idx / fetched: the work-list entry four tiles ahead is read from LDS in the middle of the
    // slots, so its latency is never waited for.
    auto iteration = [&](auto with_pv, int entry, int t_v, int t_k, f32x16(&s_cur)[2], f32x16(&s_nxt)[2],
                         uint4(&pre)[kAhead], int fetch_idx, int& fetched) {
        constexpr bool kPV = decltype(with_pv)::value;
        constexpr int kSlots = kPV ? 32 : 16, kQk0 = kPV ? 16 : 0;
        constexpr int kCopyStep = kSlots / 4;
        const int v_wr = v_rd == 0 ? kVStages - 1 : v_rd - 1;   // (v_rd + 3) % 4
        const int k_wr = k_rd == 0 ? kKStages - 1 : k_rd - 1;   // (k_rd + 2) % 3
        if (entry < 0) mask_tile(entry, s_cur);
        rescale();  // tile i-2 is in the accumulator; tile i-1, scaled for the newer reference, is added below
        auto operand = [&](int k) -> uint4 {
            if (k >= kQk0) {
                const int j = k - kQk0;  // K piece (kk, ks) = (j % 8, j / 8): one 32-key block after the other
                return k_piece(j & 7, j >> 3);
            }
            return v_piece(k >> 2, k & 3);
        };
        uint4 ops[kSlots];
        if (kPV) {
#pragma unroll
            for (int k = 0; k < kAhead; k++) ops[k] = pre[k];
        }
        float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        float shift = 0.f, rs = 0.f;
        // Softmax schedule.  With P.V: slots 0..7 running maxima (the last one also reduces them), then one
        // pair of probabilities per slot: the first 32-key block of the tile is consumed by slot 15 and the
        // second by slot 23, just before the matrix pipe starts to overwrite them with the next tile's
        // logits (slots 16..23 and 24..31), so one set of logit registers serves both tiles.
        constexpr int kMaxSlots = kPV ? 8 : 4;             // slots with running maxima
        constexpr int kMaxPer = 32 / kMaxSlots;            // logits per such slot
        constexpr int kExpFirst = kMaxSlots;               // first slot with probabilities
        constexpr int kExpPer = kPV ? 1 : 2;               // pairs per slot
        float q0[kExpPer], q1[kExpPer];                    // exponentials of the previous slot, packed one slot later
        int raw_entry = 0;
        bool moved = true;                                 // some row of the wavefront takes a new reference
        auto slot = [&](int k) {
            if (kPV && k + kAhead < kSlots) ops[k + kAhead] = operand(k + kAhead);
            if (k % kCopyStep == 1) {
                const int q = k / kCopyStep;               // 0, 1: V^T blocks; 2, 3: K blocks
                if (q < 2) copy_v(t_v, v_wr, q);
                else copy_k(t_k, k_wr, q - 2);
            }
            if (k == 4) raw_entry = list_lds[fetch_idx];
            if (!kPV) {
                // the first iteration of a workgroup: the next tile's logits follow the slots (below)
            } else if (k >= kQk0) {
                const int j = k - kQk0;
                s_nxt[j >> 3] = Mma<T>::mma(ops[k], qreg[j & 7], (j & 7) == 0 ? cinit : s_nxt[j >> 3]);
            } else {
                const int st = k >> 2, dt = k & 3;
                const uint4 bq = make_uint4(pk[st][0], pk[st][1], pk[st][2], pk[st][3]);
                oacc[dt] = Mma<T>::mma(ops[k], bq, oacc[dt]);
            }
            if (k < kMaxSlots) {
#pragma unroll
                for (int e = 0; e < kMaxPer; e++) {
                    const int idx = k * kMaxPer + e;
                    mx[e & 3] = fmaxf(mx[e & 3], s_cur[idx >> 4][idx & 15]);
                }
                if (k == kMaxSlots - 1) {
                    // The logits are relative to the row's reference m_ref (it rides on the accumulator
                    // initialisation of the matrix pipe), m_run is the running maximum relative to it.
                    // The reference moves only when the maximum has outgrown it by kShiftAt, or with the
                    // first visible key of a row; until then a probability is a bare exponential.
                    float m = fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3]));
                    m = half_max(m);
                    const float m_new = fmaxf(m_run, m);
                    const bool first = m_run == -INFINITY && m != -INFINITY;
                    const bool sh = first || m_new > kShiftAt;
                    moved = __builtin_amdgcn_ballot_w64(sh) != 0ull;
                    shift = sh ? m_new : 0.f;
                    alpha = sh ? (first ? 0.f : __builtin_amdgcn_exp2f(-shift)) : 1.f;
                    m_run = m_new - shift;
                    m_ref += shift;
                }
            } else {
#pragma unroll
                for (int r = 0; r < kExpPer; r++) {
                    const int prev = (k - 1 - kExpFirst) * kExpPer + r;  // pair computed one slot ago
                    if (prev >= 0 && prev < 16) {
                        const int ks = prev >> 3, v = 2 * (prev & 7);
                        const uint32_t w = Mma<T>::pack2(q0[r], q1[r]);
                        rs = Mma<T>::sum2(w, rs);              // the row sum takes the rounded values the product uses
                        pk[2 * ks + (v >> 3)][(v & 7) >> 1] = w;
                    }
                    const int pair = (k - kExpFirst) * kExpPer + r;      // (ks, v) = (pair / 8, 2 * (pair % 8))
                    if (pair < 16) {
                        const int ks = pair >> 3, v = 2 * (pair & 7);
                        q0[r] = __builtin_amdgcn_exp2f(s_cur[ks][v]);
                        q1[r] = __builtin_amdgcn_exp2f(s_cur[ks][v + 1]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        };
#pragma unroll
        for (int k = 0; k < kMaxSlots; k++) slot(k);
        if (moved) {
            // rare after the first tiles: this tile's logits come down to the new reference here, the later
            // ones through the accumulator initialisation
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int v = 0; v < 16; v++) s_cur[ks][v] -= shift;
#pragma unroll
            for (int v = 0; v < 16; v++) cinit[v] = -m_ref;
        }
#pragma unroll
        for (int k = kMaxSlots; k < kSlots; k++) slot(k);
        l_run = l_run * alpha + rs;
        fetched = __builtin_amdgcn_readfirstlane(raw_entry);
        if (!kPV) qk(s_nxt);  // once per workgroup, not interleaved: the logits of tile 1
        // on to the stages of tiles i and i+2; first operands of the next iteration: V^T tile i,
        // complete since the last barrier
        advance_v();
        advance_k();
#pragma unroll
        for (int k = 0; k < kAhead; k++) pre[k] = v_piece(k >> 2, k & 3);
        // keep the packed probabilities in this region (they are next read after the barrier)
#pragma unroll
        for (int st = 0; st < 4; st++) asm volatile("" ::"v"(pk[st][0]), "v"(pk[st][1]), "v"(pk[st][2]), "v"(pk[st][3]));
    };

    f32x16 sA[2], sB[2];
    uint4 pre[kAhead];
    if (n_work > 0) {
#pragma unroll
        for (int j = 0; j < kBlocksPerWave; j++) {
            copy_k(work(0) & 0x7fffffff, 0, j);
            copy_k(work(1) & 0x7fffffff, 1, j);
            copy_k(work(2) & 0x7fffffff, 2, j);
            copy_v(work(0) & 0x7fffffff, 0, j);
            copy_v(work(1) & 0x7fffffff, 1, j);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        qk(sA);
        advance_k();
        // iteration 0: nothing to multiply by V yet.  e0 .. e3: work-list entries of tiles i .. i+3
        auto clamp_idx = [&](int j) { return j < n_work ? j : n_work - 1; };
        int e0 = work(0), e1 = work(1), e2 = work(2), e3 = work(3), e4 = 0;
        __syncthreads();                     // every wavefront is done with K stage 0
        iteration(std::false_type{}, e0, e2 & 0x7fffffff, e3 & 0x7fffffff, sA, sB, pre, clamp_idx(4), e4);
        // all copies but the four of the iteration just finished have landed
        constexpr int kWaitOlder = 0x0F74;   // vmcnt(4)
        for (int i = 1; i < n_work; i += 2) {
            e0 = e1; e1 = e2; e2 = e3; e3 = e4;
            __builtin_amdgcn_s_waitcnt(kWaitOlder);
            __syncthreads();
            iteration(std::true_type{}, e0, e2 & 0x7fffffff, e3 & 0x7fffffff, sB, sA, pre, clamp_idx(i + 4), e4);
            if (i + 1 < n_work) {
                e0 = e1; e1 = e2; e2 = e3; e3 = e4;
                __builtin_amdgcn_s_waitcnt(kWaitOlder);
                __syncthreads();
                iteration(std::true_type{}, e0, e2 & 0x7fffffff, e3 & 0x7fffffff, sA, sB, pre, clamp_idx(i + 5), e4);
            }
        }
        // the P.V product of the last tile; the copies still in flight are repeats that nobody reads
        rescale();
        pv();
        __builtin_amdgcn_s_waitcnt(0x0F70);
    }

    // epilogue: lane owns d = 32dt + 8(v/4) + 4half + v%4 of its query row
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (p.n_split > 1) {
        // a share of the key tiles: the row normalised by the share's own sum, and the share's normaliser
        const int rf_p = qt_i * kRows + wave * 32 + col;
        const int64_t row_p = (b * p.H + kvh * p.G + rf_p % p.G) * p.Q + row_m;
        if (row_m < p.Q) {
            const bool any = l_tot > 0.f;
            const float inv_p = any ? 1.f / l_tot : 0.f;
            float* po = p.part_o + ((int64_t)split_i * p.B * p.H * p.Q + row_p) * kD;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int v4 = 0; v4 < 4; v4++)
                    *reinterpret_cast<float4*>(po + 32 * dt + 8 * v4 + 4 * half) =
                        make_float4(oacc[dt][4 * v4] * inv_p, oacc[dt][4 * v4 + 1] * inv_p, oacc[dt][4 * v4 + 2] * inv_p,
                                    oacc[dt][4 * v4 + 3] * inv_p);
            if (half == 0)
                p.part_l2[(int64_t)split_i * p.B * p.H * p.Q + row_p] = any ? m_ref + __builtin_amdgcn_logf(l_tot) : -INFINITY;
        }
        return;
    }
    const int g_row = (qt_i * kRows + wave * 32 + col) % p.G;
    const int64_t row_h = kvh * p.G + g_row;
    const bool row_ok = row_m < p.Q;
    const float inv = 1.f / l_tot;
    const bool rows16 = p.out_stride[3] == 1 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0 && p.out_stride[0] % 8 == 0 &&
                        p.out_stride[1] % 8 == 0 && p.out_stride[2] % 8 == 0;
    if (rows16) {
        // through LDS, so that a row leaves as 16-byte pieces of 16 neighbouring lanes (a lane's own
        // 8-byte pieces would reach memory as partly filled 32-byte sectors)
        constexpr int kRowPitch = 256 + 16;  // bytes; the pad spreads the banks
        __syncthreads();                      // the tile stages are no longer read
        unsigned char* ow = smem + wave * (32 * kRowPitch);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                uint2 w;
                w.x = Mma<T>::pack2(oacc[dt][4 * v4] * inv, oacc[dt][4 * v4 + 1] * inv);
                w.y = Mma<T>::pack2(oacc[dt][4 * v4 + 2] * inv, oacc[dt][4 * v4 + 3] * inv);
                *reinterpret_cast<uint2*>(ow + col * kRowPitch + (32 * dt + 8 * v4 + 4 * half) * (int)sizeof(T)) = w;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_wave_barrier();
        // 4 rows per pass: lane = (row in the pass, 16-byte piece)
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int r = 4 * pass + (lane >> 4), piece = lane & 15;
            const int rr = qt_i * kRows + wave * 32 + r;
            const int g_r = rr % p.G, m_r = rr / p.G;
            if (m_r < p.Q) {
                const uint4 v = *reinterpret_cast<const uint4*>(ow + r * kRowPitch + piece * 16);
                T* dst = (T*)p.out + b * p.out_stride[0] + (kvh * p.G + g_r) * p.out_stride[1] + m_r * p.out_stride[2];
                *reinterpret_cast<uint4*>(dst + piece * 8) = v;
            }
        }
    } else if (row_ok) {
        T* orow = (T*)p.out + b * p.out_stride[0] + row_h * p.out_stride[1] + row_m * p.out_stride[2];
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                const int d = 32 * dt + 8 * v4 + 4 * half;
#pragma unroll
                for (int e = 0; e < 4; e++) orow[(d + e) * p.out_stride[3]] = Elem<T>::from_float(oacc[dt][4 * v4 + e] * inv);
            }
        }
    }
    if (row_ok) {
        if (half == 0) {
            const float l2 = m_ref + __builtin_amdgcn_logf(l_tot);  // v_log_f32 is log2
            p.lse[(b * p.H + row_h) * p.Q + row_m] = l2 * 0.6931471805599453f;
            p.lse2[(b * p.H + row_h) * p.Q + row_m] = -l2;
        }
    }
}

// Merge of the forward kernel's shares: one row per 32 lanes (4 dims each), 8 rows per workgroup.
template <typename T>
__global__ void __launch_bounds__(256) fwd_combine_kernel(FwdParams p) {
    const int64_t rows = p.B * p.H * p.Q;
    const int64_t row = (int64_t)blockIdx.x * 8 + threadIdx.x / 32;
    if (row >= rows) return;
    const int d4 = threadIdx.x % 32;
    float M = -INFINITY;
    for (int s_ = 0; s_ < p.n_split; s_++) M = fmaxf(M, p.part_l2[s_ * rows + row]);
    float L = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s_ = 0; s_ < p.n_split; s_++) {
        const float l2 = p.part_l2[s_ * rows + row];
        if (l2 == -INFINITY) continue;
        const float w = __builtin_amdgcn_exp2f(l2 - M);
        const float4 v = *reinterpret_cast<const float4*>(p.part_o + (s_ * rows + row) * kD + 4 * d4);
        L += w;
        o.x = fmaf(v.x, w, o.x); o.y = fmaf(v.y, w, o.y); o.z = fmaf(v.z, w, o.z); o.w = fmaf(v.w, w, o.w);
    }
    const float inv = 1.f / L;
    const int64_t m = row % p.Q, h = (row / p.Q) % p.H, b = row / (p.Q * p.H);
    T* dst = (T*)p.out + b * p.out_stride[0] + h * p.out_stride[1] + m * p.out_stride[2];
    dst[(4 * d4) * p.out_stride[3]] = Elem<T>::from_float(o.x * inv);
    dst[(4 * d4 + 1) * p.out_stride[3]] = Elem<T>::from_float(o.y * inv);
    dst[(4 * d4 + 2) * p.out_stride[3]] = Elem<T>::from_float(o.z * inv);
    dst[(4 * d4 + 3) * p.out_stride[3]] = Elem<T>::from_float(o.w * inv);
    if (d4 == 0) {
        const float l2 = M + __builtin_amdgcn_logf(L);  // v_log_f32 is log2
        p.lse[row] = l2 * 0.6931471805599453f;
        p.lse2[row] = -l2;
    }
}

// ---------------------------------------------------------------------------------------------
// score sums
// ---------------------------------------------------------------------------------------------
struct ColsumParams {
    const void* qr;       // (B*H*Q + kColSlack rows, D)
    const void* kr;
    const unsigned long long* tile_vis;
    const float* lse2;    // (B*H*Q + kColSlack) minus the log2-domain row normalisers
    const float* w_ema;   // (Q + kColSlack), zero beyond Q
    const float* w_new;   // (Q)
    float* colsum;        // (B*H, N)
    int64_t B, H, KVH, Q, N, Nc, n_pad;
    int G;
    int new_mode;
    float scale_log2;
    int nkb, first_chunk_blk, nbkv, xcd_aware, gsplit;  // block order and head split, see the kernel
    int wnew_uniform;     // every entry of w_new has the value wnew_value (beta rounds to one in the tensor dtype)
    float wnew_value;
};

constexpr int kQT2 = 128;                     // query rows per LDS tile of the column pass
constexpr int kCsSub = kQT2 / 32;             // 32-row subtiles of a tile
constexpr int kCsStage = kQT2 * 256 + 2 * kQT2 * 4;   // Q tile + its lse2 + its weights

// One workgroup = one kv head x 256 keys (64 per wavefront, held in registers as the B operand of
// S = Q K^T).  The (head, query-tile) sequence streams through a double-buffered LDS stage filled
// by asynchronous copies; lane (col, half) owns key column `col` of each 32-key subtile, so the
// weighted column sums never leave the lane.
template <typename T>
__global__ void __launch_bounds__(256, 2) colsum_mfma_kernel(ColsumParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    float* wnew_lds = reinterpret_cast<float*>(smem + 2 * kCsStage);
    const uint32_t smem_addr = lds_address(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, half = lane >> 5;
    // Block order.  Key blocks that hold chunk keys cost the most per step (masking on the
    // diagonal, per-element weights), so they are handed out first and never form the tail of
    // the launch.  Workgroup ids go round the 8 XCDs; when the kv heads divide evenly, every
    // block of one kv head runs on one XCD so that head's query stream stays in that XCD's L2.
    // A key block is shared out over gsplit workgroups, each taking G / gsplit heads: units small
    // enough that the last round of workgroups costs little.
    int bkv_i, kb_i, g_first;
    const int g_cnt = p.G / p.gsplit;
    {
        const int nkb = p.nkb * p.gsplit, cb0 = p.first_chunk_blk * p.gsplit, heavy = nkb - cb0;
        int id = blockIdx.x, nb = p.nbkv, first = 0, stride = 1;
        if (p.xcd_aware) {
            first = id & 7;
            stride = 8;
            id >>= 3;
            nb >>= 3;
        }
        int i;
        if (id < nb * heavy) {
            i = id / heavy;
            kb_i = cb0 + id % heavy;
        } else {
            id -= nb * heavy;
            i = id / cb0;
            kb_i = id % cb0;
        }
        bkv_i = first + stride * i;
        g_first = (kb_i % p.gsplit) * g_cnt;
        kb_i /= p.gsplit;
    }
    const int64_t bkv = bkv_i;
    const int64_t b = bkv / p.KVH, kvh = bkv % p.KVH;
    const int Q = (int)p.Q;
    const int64_t key_blk = (int64_t)kb_i * 256;          // first key of the workgroup
    const int64_t key_w = key_blk + wave * 64;            // first key of this wavefront

    uint4 kreg[2][8];
    const char* kbase = (const char*)p.kr + bkv * p.n_pad * kD * (int64_t)sizeof(T);
    bool live[2];
    int nrel[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        const int64_t n = key_w + 32 * ks + col;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            kreg[ks][kk] = n < p.n_pad ? *reinterpret_cast<const uint4*>(kbase + (n / kBN) * (int64_t)(kBN * kD * sizeof(T)) +
                                                                         k_image_off((int)(n % kBN), 2 * kk + half))
                                       : make_uint4(0, 0, 0, 0);
        }
        live[ks] = n < p.N && ((p.tile_vis[n / kBN] >> (n % kBN)) & 1ull);
        nrel[ks] = (int)(n - p.Nc);
    }
    // first query tile that can see any key of the workgroup
    int m_first = (int)(key_blk - p.Nc);
    if (m_first < 0) m_first = 0;
    m_first = m_first / kQT2 * kQT2;
    const bool chunk_keys = key_blk + 255 >= p.Nc;  // some key of the workgroup belongs to the chunk
    const int last_nrel = (int)(key_blk + 255 - p.Nc);
    const bool new_chunk = chunk_keys && p.new_mode;
    const bool pure_chunk = key_blk >= p.Nc;        // no cached key in the workgroup
    // the weights of chunk keys by distance: a table in LDS, unless every entry is the same value (then the
    // launch reserves no LDS for it, and two workgroups fit a compute unit whatever the chunk length)
    if (new_chunk && !p.wnew_uniform) {
        for (int i = tid; i < Q; i += 256) wnew_lds[i] = p.w_new[i];
    }
    auto wnew_at = [&](int i) -> float { return p.wnew_uniform ? p.wnew_value : wnew_lds[i]; };
    const int nmt = (Q - m_first + kQT2 - 1) / kQT2;  // query tiles per head
    const int n_steps = nmt * g_cnt;

    // async copy assignments: the Q tile is kQT2 / 4 blocks of 1 KiB (a quarter per wavefront); wavefront 0
    // also brings the tile's normalisers, wavefront 1 its weights (kQT2 / 4 lanes x 16 bytes each)
    constexpr int kQBlocks = kQT2 / 16;   // per wavefront
    uint32_t q_src[kQBlocks];
#pragma unroll
    for (int j = 0; j < kQBlocks; j++) {
        const int pos = (wave * kQBlocks + j) * 64 + lane;
        const int r = pos >> 4, c = (pos & 15) ^ (r & 15);
        q_src[j] = r * 256 + c * 16;
    }
    int q_off[8];  // query row `col` of the tile (+32 rows = +8192 B)
#pragma unroll
    for (int kk = 0; kk < 8; kk++) q_off[kk] = k_lds_off(col, 2 * kk + half);
    const int64_t head_row0 = (b * p.H + kvh * p.G) * p.Q;
    // (head, query tile) of a step are tracked incrementally: integer division per step would
    // cost more scalar instructions than the step's matrix work leaves room for
    auto issue = [&](int g, int mt, int stage) {
        const int64_t row0 = head_row0 + (int64_t)g * p.Q + mt;
        const char* qt = (const char*)p.qr + row0 * (kD * (int64_t)sizeof(T));
        const uint32_t st = smem_addr + stage * kCsStage;
#pragma unroll
        for (int j = 0; j < kQBlocks; j++) async_copy16(qt, q_src[j], st + (wave * kQBlocks + j) * 1024);
        if (wave < 2 && lane < kQT2 / 4) {
            const char* src = wave ? (const char*)(p.w_ema + mt) : (const char*)(p.lse2 + row0);
            async_copy16(src, lane * 16, st + kQT2 * 256 + wave * (kQT2 * 4));
        }
    };

    float acc[2] = {0.f, 0.f};
    auto tile_step = [&](auto stage_tag, int g, int mt) {
        constexpr int ST = decltype(stage_tag)::value;
        const unsigned char* q_lds = smem + ST * kCsStage;
        const float* lse_lds = reinterpret_cast<const float*>(q_lds + kQT2 * 256);
        const float* w_lds = lse_lds + kQT2;
        const bool tail = mt + kQT2 > Q;                       // rows past the chunk end
        const bool diag = chunk_keys && mt <= last_nrel;       // tile may cross the diagonal
        // Accumulators start from minus the row normaliser, so the matrix pipe hands back log2 P (the
        // softmax scale is already on the staged queries).  Element (c, v) of a 32-row subtile c:
        // query row mt + 32c + 8(v/4) + 4half + v%4, key column of this lane.
        auto row_init = [&](int c) {
            f32x16 init;
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                const float4 l4 = *reinterpret_cast<const float4*>(lse_lds + 32 * c + 8 * v4 + 4 * half);
                init[4 * v4] = l4.x;
                init[4 * v4 + 1] = l4.y;
                init[4 * v4 + 2] = l4.z;
                init[4 * v4 + 3] = l4.w;
            }
            return init;
        };
        auto load_weights = [&](int c, float(&ws)[16]) {
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                const float4 w4 = *reinterpret_cast<const float4*>(w_lds + 32 * c + 8 * v4 + 4 * half);
                ws[4 * v4] = w4.x; ws[4 * v4 + 1] = w4.y; ws[4 * v4 + 2] = w4.z; ws[4 * v4 + 3] = w4.w;
            }
        };
        if (!tail && !diag && !new_chunk) {
            // The common case, written in issue order: the logits of subtile c go through the matrix
            // pipe while the vector ALU turns subtile c-1 into weighted probabilities.
            f32x16 sq[2][2];  // [c & 1][ks]
            sq[0][0] = sq[0][1] = row_init(0);
#pragma unroll
            for (int kk = 0; kk < 8; kk++) {
                const uint4 a = *reinterpret_cast<const uint4*>(q_lds + q_off[kk]);
                sq[0][0] = Mma<T>::mma(a, kreg[0][kk], sq[0][0]);
                sq[0][1] = Mma<T>::mma(a, kreg[1][kk], sq[0][1]);
            }
#pragma unroll
            for (int c = 1; c < kCsSub; c++) {
                sq[c & 1][0] = sq[c & 1][1] = row_init(c);
                uint4 a1[8];
#pragma unroll
                for (int kk = 0; kk < 8; kk++) a1[kk] = *reinterpret_cast<const uint4*>(q_lds + q_off[kk] + c * 8192);
                float ws[16];
                load_weights(c - 1, ws);
                __builtin_amdgcn_sched_barrier(0);
                // an exponential is consumed one slot after it was issued, so no wavefront waits for the
                // transcendental unit
                float pe_prev[2] = {0.f, 0.f};
#pragma unroll
                for (int slot = 0; slot < 16; slot++) {
                    const int kk = slot >> 1, ks = slot & 1;
                    sq[c & 1][ks] = Mma<T>::mma(a1[kk], kreg[ks][kk], sq[c & 1][ks]);
                    float pe[2];
#pragma unroll
                    for (int r = 0; r < 2; r++) {
                        const int j = 2 * slot + r, ksv = j >> 4, v = j & 15;
                        pe[r] = __builtin_amdgcn_exp2f(sq[(c - 1) & 1][ksv][v]);
                    }
                    if (slot > 0) {
#pragma unroll
                        for (int r = 0; r < 2; r++) {
                            const int j = 2 * (slot - 1) + r, ksv = j >> 4, v = j & 15;
                            acc[ksv] = fmaf(ws[v], pe_prev[r], acc[ksv]);
                        }
                    }
                    pe_prev[0] = pe[0];
                    pe_prev[1] = pe[1];
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int r = 0; r < 2; r++) {
                    const int j = 30 + r, ksv = j >> 4, v = j & 15;
                    acc[ksv] = fmaf(ws[v], pe_prev[r], acc[ksv]);
                }
            }
            {
                float ws[16];
                load_weights(kCsSub - 1, ws);
#pragma unroll
                for (int v = 0; v < 16; v++) {
#pragma unroll
                    for (int ks = 0; ks < 2; ks++) {
                        const float pe = __builtin_amdgcn_exp2f(sq[(kCsSub - 1) & 1][ks][v]);
                        acc[ks] = fmaf(ws[v], pe, acc[ks]);
                    }
                }
            }
        } else {
            // special cases, one 32-row subtile at a time
            const bool fast_new = !tail && !diag;   // new_chunk holds: every row is later than every key of the block
            bool chunk_lane[2];
#pragma unroll
            for (int ks = 0; ks < 2; ks++) chunk_lane[ks] = nrel[ks] >= 0;
            // a chunk key takes the weight of its distance m - n; a cached key (only in the block that
            // straddles the chunk start) takes the row's EMA weight
            auto weight_of = [&](int ks, int r) -> float {
                return chunk_lane[ks] ? wnew_at(mt + 4 * half - nrel[ks] + r) : w_lds[4 * half + r];
            };
#pragma unroll 1
            for (int c = 0; c < kCsSub; c++) {
                f32x16 sacc[2];
                sacc[0] = sacc[1] = row_init(c);
#pragma unroll
                for (int kk = 0; kk < 8; kk++) {
                    const uint4 a = *reinterpret_cast<const uint4*>(q_lds + q_off[kk] + c * 8192);
                    sacc[0] = Mma<T>::mma(a, kreg[0][kk], sacc[0]);
                    sacc[1] = Mma<T>::mma(a, kreg[1][kk], sacc[1]);
                }
                if (fast_new && p.wnew_uniform && __builtin_amdgcn_ballot_w64(!(chunk_lane[0] && chunk_lane[1])) == 0ull) {
                    // every key of the wavefront is a chunk key and all of them weigh the same: P and the
                    // products are rounded to the tensor dtype two at a time by the packed conversions, and
                    // the rounded products join the sum through a dot product with a pair of ones
                    const float wu = p.wnew_value;
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
#pragma unroll
                        for (int ks = 0; ks < 2; ks++) {
                            const uint32_t u = Mma<T>::pack2(__builtin_amdgcn_exp2f(sacc[ks][v]),
                                                             __builtin_amdgcn_exp2f(sacc[ks][v + 1]));
                            acc[ks] = Mma<T>::sum2(Mma<T>::pack2(Mma<T>::lo_f(u) * wu, Mma<T>::hi_f(u) * wu), acc[ks]);
                        }
                    }
                } else if (fast_new) {
                    // no masks; the eager path holds P and the products of chunk keys in the tensor dtype
#pragma unroll
                    for (int v4 = 0; v4 < 4; v4++) {
                        const int r0 = 32 * c + 8 * v4;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
#pragma unroll
                            for (int ks = 0; ks < 2; ks++) {
                                const float pe = __builtin_amdgcn_exp2f(sacc[ks][4 * v4 + e]);
                                const float w = weight_of(ks, r0 + e);
                                if (pure_chunk) {
                                    acc[ks] += Mma<T>::round1(Mma<T>::round1(pe) * w);
                                } else {
                                    const float prod = (chunk_lane[ks] ? Mma<T>::round1(pe) : pe) * w;
                                    acc[ks] += chunk_lane[ks] ? Mma<T>::round1(prod) : prod;
                                }
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int r = 32 * c + 8 * (v >> 2) + 4 * half + (v & 3);
                        const int m = mt + r;
                        const bool row_in = m < Q;
                        const float we = w_lds[r];
#pragma unroll
                        for (int ks = 0; ks < 2; ks++) {
                            float pe = __builtin_amdgcn_exp2f(sacc[ks][v]);
                            const bool is_chunk = nrel[ks] >= 0;
                            const bool vis = row_in && (!is_chunk || m >= nrel[ks]);
                            pe = vis ? pe : 0.f;
                            if (is_chunk && p.new_mode) {
                                // the eager path holds P and the products in the tensor dtype
                                const float w = vis ? wnew_at(m - nrel[ks]) : 0.f;
                                acc[ks] += Mma<T>::round1(Mma<T>::round1(pe) * w);
                            } else {
                                acc[ks] = fmaf(row_in ? we : 0.f, pe, acc[ks]);
                            }
                        }
                    }
                }
            }
        }
        if (mt + kQT2 >= Q) {  // head finished: combine the two lane halves and store
            const int64_t h = kvh * p.G + g;
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const float tot = acc[ks] + __shfl_xor(acc[ks], 32);
                const int64_t n = key_w + 32 * ks + col;
                if (half == 0 && n < p.N) p.colsum[(b * p.H + h) * p.N + n] = live[ks] ? tot : 0.f;
                acc[ks] = 0.f;
            }
        }
    };

    // two steps per trip: while stage s is consumed the copy of the next step fills stage s^1
    int g_cur = g_first, mt_cur = m_first;    // step being consumed
    auto advance = [&](int& g, int& mt) {
        mt += kQT2;
        if (mt >= Q) {
            mt = m_first;
            g++;
        }
    };
    if (n_steps > 0) issue(g_first, m_first, 0);
    for (int step = 0; step < n_steps; step += 2) {
        int g_n = g_cur, mt_n = mt_cur;
        advance(g_n, mt_n);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        if (step + 1 < n_steps) issue(g_n, mt_n, 1);
        tile_step(std::integral_constant<int, 0>{}, g_cur, mt_cur);
        if (step + 1 < n_steps) {
            int g_n2 = g_n, mt_n2 = mt_n;
            advance(g_n2, mt_n2);
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            if (step + 2 < n_steps) issue(g_n2, mt_n2, 0);
            tile_step(std::integral_constant<int, 1>{}, g_n, mt_n);
            g_cur = g_n2;
            mt_cur = mt_n2;
        }
    }
    if (n_steps == 0) {  // no query can see these keys (only possible for padding blocks)
        for (int g = g_first; g < g_first + g_cnt; g++)
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const int64_t n = key_w + 32 * ks + col;
                if (half == 0 && n < p.N) p.colsum[(b * p.H + kvh * p.G + g) * p.N + n] = 0.f;
            }
    }
}

template <typename T>
int run_mfma(const MfmaProblem& mp, hipStream_t stream) {
    const int64_t n = mp.n, n_pad = mp.n_pad;
    const float scale_log2 = mp.scale * 1.4426950408889634f;
    const int cus = mfma_device_cus();
    {
        StageScope sc(CKV_STAGE_PREP, stream);
        StageParams sp;
        for (int i = 0; i < 3; i++) {
            sp.seg[i].k = mp.seg[i].k;
            sp.seg[i].v = mp.seg[i].v;
            for (int j = 0; j < 4; j++) sp.seg[i].stride[j] = mp.seg[i].stride[j];
            sp.seg[i].pos = mp.seg[i].pos;
            sp.seg[i].pos_stride[0] = mp.seg[i].pos_stride[0];
            sp.seg[i].pos_stride[1] = mp.seg[i].pos_stride[1];
            sp.seg[i].pos_shift = mp.seg[i].pos_shift;
            sp.seg[i].masked = mp.seg[i].masked;
            sp.seg[i].len = mp.seg[i].len;
        }
        sp.inv_freq = mp.inv_freq;
        sp.theta = mp.theta;
        sp.key_scale = mp.key_scale;
        sp.shared_pos = mp.shared_pos;
        sp.kr = mp.kr;
        sp.vt = mp.vt;
        sp.tile_vis = mp.tile_vis;
        sp.B = mp.B; sp.KVH = mp.KVH; sp.n = n; sp.n_pad = n_pad;
        const int64_t nbh = mp.B * mp.KVH;
        // shared positions: a block walks several (b, kvh) units with one set of cos/sin, the next unit's rows
        // always on their way
        int64_t splits = nbh;
        if (mp.shared_pos) {  // about two workgroups per compute unit
            const int64_t tiles = n_pad / kBN;
            splits = (2 * cus + tiles - 1) / tiles;
            if (splits < 2) splits = 2;
            if (splits > nbh) splits = nbh;
        }
        if (splits > 65535) splits = 65535;
        StageQParams sq;
        sq.q = mp.q;
        for (int j = 0; j < 4; j++) sq.stride[j] = mp.q_stride[j];
        sq.q_pos = mp.q_pos;
        sq.inv_freq = mp.inv_freq;
        sq.theta = mp.theta;
        sq.qr = mp.qr;
        sq.rows = mp.B * mp.H * mp.Q;
        sq.H = mp.H; sq.Q = mp.Q;
        sq.qscale = mp.q_pos ? scale_log2 / mp.key_scale : scale_log2;  // rotated keys carry key_scale
        sq.vec = mp.q_stride[3] == 1 && reinterpret_cast<uintptr_t>(mp.q) % 16 == 0 && mp.q_stride[0] % 8 == 0 &&
                 mp.q_stride[1] % 8 == 0 && mp.q_stride[2] % 8 == 0;
        {
            // about four query blocks (64 positions each) per compute unit; the rest of batch x heads is looped
            // over inside, sharing cos/sin
            const int64_t bx = (mp.Q + 63) / 64, nbh_q = mp.B * mp.H;
            int64_t by = (4 * cus + bx - 1) / bx;
            if (by > nbh_q) by = nbh_q;
            if (by < 1) by = 1;
            StageGrid g;
            g.q_bx = (int)bx; g.q_by = (int)by; g.k_bx = (int)(n_pad / kBN); g.k_by = (int)splits;
            const int64_t blocks = bx * by + (n_pad / kBN) * splits;
            if (blocks > 0x7fffffff) return CKV_ERR_UNSUPPORTED;
            hipLaunchKernelGGL(stage_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, sp, sq, g);
        }
        CKV_HIP_TRY(hipGetLastError());
    }
    const int G = (int)(mp.H / mp.KVH);
    {
        StageScope sc(CKV_STAGE_FWD, stream, true);
        FwdParams fp;
        fp.qr = mp.qr; fp.kr = mp.kr; fp.vt = mp.vt; fp.tile_vis = mp.tile_vis;
        fp.out = mp.out;
        for (int j = 0; j < 4; j++) fp.out_stride[j] = mp.out_stride[j];
        fp.lse = mp.lse;
        fp.lse2 = mp.lse2;
        fp.B = mp.B; fp.H = mp.H; fp.KVH = mp.KVH; fp.Q = mp.Q; fp.N = n; fp.Nc = n - mp.Q; fp.n_pad = n_pad;
        fp.G = G;
        fp.scale_log2 = 1.f;  // already on the staged queries
        fp.n_qt = (int)((mp.Q * G + kRows - 1) / kRows);
        fp.n_split = mfma_fwd_splits(mp.B, mp.H, mp.KVH, mp.Q, n, cus);
        fp.part_o = mp.part_o;
        fp.part_l2 = mp.part_l2;
        if (fp.n_split > 1 && (!fp.part_o || !fp.part_l2)) return CKV_ERR_WORKSPACE;
        const dim3 grid((unsigned)(fp.n_qt * fp.n_split), (unsigned)(mp.B * mp.KVH));
        const int lds = pipe_lds_bytes(n_pad);
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fwd_pipe_kernel<T>), lds)) return rc;
        fp.xcd_aware = grid.y % 8 == 0;
        hipEvent_t ev0, ev1;
        prof_kernel_events(CKV_STAGE_FWD, &ev0, &ev1);
        const dim3 launch_grid = fp.xcd_aware ? dim3(grid.x * grid.y) : grid;
        if (ev0) hipExtLaunchKernelGGL(fwd_pipe_kernel<T>, launch_grid, dim3(512), (uint32_t)lds, stream, ev0, ev1, 0u, fp);
        else hipLaunchKernelGGL(fwd_pipe_kernel<T>, launch_grid, dim3(512), lds, stream, fp);
        CKV_HIP_TRY(hipGetLastError());
        if (fp.n_split > 1) {
            const int64_t rows = mp.B * mp.H * mp.Q;
            hipLaunchKernelGGL(fwd_combine_kernel<T>, dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, stream, fp);
            CKV_HIP_TRY(hipGetLastError());
        }
    }
    if (mp.colsum) {
        StageScope sc(CKV_STAGE_SCORES, stream);
        ColsumParams cp;
        cp.qr = mp.qr; cp.kr = mp.kr; cp.tile_vis = mp.tile_vis; cp.lse2 = mp.lse2;
        cp.w_ema = mp.w_ema; cp.w_new = mp.w_new; cp.colsum = mp.colsum;
        cp.B = mp.B; cp.H = mp.H; cp.KVH = mp.KVH; cp.Q = mp.Q; cp.N = n; cp.Nc = n - mp.Q; cp.n_pad = n_pad;
        cp.G = G;
        cp.new_mode = mp.new_mode;
        {
            // w_new[k] = round((1 - beta) * round(round(beta)^k)) in the tensor dtype: one value for every k when
            // beta rounds to one there (0.9999999 does in both 16-bit formats)
            auto round_t_host = [](float v) -> float {
                if (std::is_same<T, __half>::value) return (float)(_Float16)v;
                uint32_t u;
                memcpy(&u, &v, 4);
                u += 0x7fffu + ((u >> 16) & 1u);  // to nearest even on the upper 16 bits (finite values)
                u &= 0xffff0000u;
                float r;
                memcpy(&r, &u, 4);
                return r;
            };
            cp.wnew_uniform = round_t_host((float)mp.beta) == 1.0f ? 1 : 0;
            cp.wnew_value = round_t_host((float)(1.0 - mp.beta));
        }
        cp.scale_log2 = 1.f;  // already on the staged queries
        cp.nkb = (int)((n + 255) / 256);
        cp.first_chunk_blk = (int)(cp.Nc / 256);
        cp.nbkv = (int)(mp.B * mp.KVH);
        cp.xcd_aware = cp.nbkv % 8 == 0;
        // two heads per workgroup where the group allows it: the keys a workgroup holds in registers and its
        // pipeline start serve twice the work, and the units stay small enough for an even last round
        cp.gsplit = (G % 2 == 0 && G >= 4) ? G / 2 : G;
        const dim3 grid((unsigned)(cp.nkb * cp.nbkv * cp.gsplit));
        const int lds = 2 * kCsStage + (cp.wnew_uniform ? 0 : (int)mp.Q * 4);
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(colsum_mfma_kernel<T>), lds)) return rc;
        hipLaunchKernelGGL(colsum_mfma_kernel<T>, grid, dim3(256), lds, stream, cp);
        CKV_HIP_TRY(hipGetLastError());
    }
    return CKV_OK;
}

}  // namespace

bool mfma_supported(int dtype, int64_t D, int64_t H, int64_t KVH, int64_t Q) {
    if (dtype != CKV_BF16 && dtype != CKV_F16) return false;
    if (D != kD) return false;
    if (Q > 16384) return false;  // the column pass keeps a Q-long weight table in LDS beside its two stages
    const int64_t G = H / KVH;
    return G >= 1 && G <= kRows / 32;  // at least 32 positions per workgroup
}

int64_t mfma_n_pad(int64_t n) { return align_up(n, 256); }

// Shares of a query tile's key tiles (1: no splitting) on a chip of `cus` compute units, each of which holds one
// workgroup of the forward kernel at a time: launches with fewer workgroups than that are topped up to about two per
// compute unit, with at least 16 key tiles per share and at most 8 shares.
int mfma_fwd_splits(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t n, int cus) {
    const int64_t G = H / KVH;
    const int64_t wgs = ((Q * G + kRows - 1) / kRows) * B * KVH, tiles = (n + kBN - 1) / kBN;
    if (wgs >= cus) return 1;
    int64_t s_ = 2 * (int64_t)cus / wgs;
    if (s_ > tiles / 16) s_ = tiles / 16;
    if (s_ > 8) s_ = 8;
    return s_ < 1 ? 1 : (int)s_;
}

// compute units of the current device; 256 (one MI355X) where no device can be asked, e.g. when a workspace is
// sized on a host without one
int mfma_device_cus() {
    DeviceInfo di;
    if (current_device_info(&di) != CKV_OK || di.cus <= 0) return 256;
    return di.cus;
}

// what a workspace is sized for: the shares the current device would use, and never fewer than a 256-unit chip's,
// so that a size computed where no device is visible also serves the launch
int mfma_fwd_splits_for_workspace(int64_t B, int64_t H, int64_t KVH, int64_t Q, int64_t n) {
    const int here = mfma_fwd_splits(B, H, KVH, Q, n, mfma_device_cus());
    const int base = mfma_fwd_splits(B, H, KVH, Q, n, 256);
    return here > base ? here : base;
}

// the forward kernel keeps per-tile bookkeeping of all N keys in LDS
bool mfma_fits(int64_t n) { return pipe_lds_bytes(mfma_n_pad(n)) <= kLdsLimit; }


int launch_mfma(const MfmaProblem& mp, hipStream_t stream) {
    if (mp.dtype == CKV_BF16) return run_mfma<__hip_bfloat16>(mp, stream);
    if (mp.dtype == CKV_F16) return run_mfma<__half>(mp, stream);
    return CKV_ERR_DTYPE;
}

}  // namespace ckv
