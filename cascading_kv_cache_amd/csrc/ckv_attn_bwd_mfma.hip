// Backward of the dense-input attention operator on the matrix cores (cascade/models/flash_attention.py:279-537):
// bf16 / fp16, head_dim 128, v_mfma_f32_32x32x16.  Two kernels, as in the reference (_attn_bwd_dq, _attn_bwd_dkdv),
// so that no gradient is accumulated with atomics; both recompute the probabilities from the row normalisers of
// the forward pass and take delta[m] = sum_d out[m, d] dout[m, d] from the caller.
//
//   dq     a wavefront owns 32 query rows, a workgroup 128; 32-key blocks of K and V stream through LDS.
//          S^T = K Q^T and dP^T = V dO^T keep a query in one lane (its normaliser and delta are one value per
//          lane), dS^T = P^T (dP^T - delta) scale is, packed, directly the B operand of dQ^T += K^T dS^T.
//   dkdv   a wavefront owns 32 keys, a workgroup 128; 32-row blocks of Q and dO stream through LDS.
//          S = Q K^T and dP = dO V^T keep a key in one lane; P and dS are the B operands of
//          dV^T += dO^T P and dK^T += Q^T dS.
//
// The A operands K^T, Q^T and dO^T are read from the row-major tiles in LDS with the transposing read
// ds_read_b64_tr_b16: lane i of a 16-lane group receives element [4e + i/4][i%4] (e = 0..3) of the 16 x 4 matrix
// whose row r is the 8 bytes lane r points at; with lane r pointing at dims 4 (r%4) .. +3 of row r/4 of a
// 4-row group, lane i receives dim i of the four rows.  Rows are 256 bytes; the 16-byte piece c of row r sits in
// slot c ^ (((r & 3) << 2) | ((r >> 2) & 3)), which keeps both the 16-byte row reads (32 rows, one piece) and the
// transposing reads (4 rows x 64 bytes) off each other's banks.
#include "ckv_attn_internal.h"

namespace ckv {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

constexpr int kHD = 128;              // head dim
constexpr int kBlk = 32;              // rows of a streamed block
constexpr int kWaves = 4;             // wavefronts of a workgroup, 32 stationary rows each
constexpr int kThreads = kWaves * CKV_WAVE;
constexpr int kOwn = kWaves * 32;     // stationary rows of a workgroup
constexpr int kRowBytes = kHD * 2;    // 256
constexpr int kTile = kBlk * kRowBytes;  // 8 KiB
constexpr float kLog2e = 1.4426950408889634f;
// dynamic LDS of the dk/dv kernel: two stages of (Q, dO) tiles, the per-row scalars of both stages, V^T operands
constexpr int kDkdvRowv = 2 * 2 * kTile;
constexpr int kDkdvV = kDkdvRowv + 2 * 2 * kBlk * (int)sizeof(float);
constexpr int kDkdvLds = kDkdvV + kWaves * (kHD / 16) * CKV_WAVE * 16;

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
};

struct BwdMfmaParams {
    ckv_dense_bwd_args a;
    const float* delta;  // (B, H, n_ctx)
};

__device__ inline int swz(int row, int piece) { return piece ^ (((row & 3) << 2) | ((row >> 2) & 3)); }

// A 32-row block of a (rows, 128) tensor into a tile, global -> LDS without registers: wavefront w copies rows
// 8 w .. 8 w + 7 with two instructions of 64 x 16 bytes; lane i fills slot i % 16 of row 4 (2 w + j) + i / 16 with
// the piece that belongs there.  Rows at or past `limit` repeat row limit - 1 (finite values; whatever is
// computed from them is masked).  The caller waits with vmcnt(0) before the barrier that publishes the tile.
__device__ inline void copy_block(const char* base, int64_t row_bytes, int64_t first, int64_t limit, uint32_t tile_lds,
                                  int wave, int lane) {
    const char* blk = base + first * row_bytes;  // uniform
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int row = 4 * (2 * wave + j) + (lane >> 4);
        int64_t rr = row;
        if (first + rr > limit - 1) rr = limit - 1 - first;
        const uint32_t voff = (uint32_t)(rr * row_bytes) + (uint32_t)(swz(row, lane & 15) << 4);
        async_copy16(blk, voff, tile_lds + (uint32_t)(4 * (2 * wave + j) * kRowBytes));
    }
}

// A operand of a product that contracts over the head dims: row lane%32 of the tile, dims 16 ds + 8 (lane/32) .. +7
__device__ inline uint4 row_operand(const unsigned char* tile, int lane, int ds) {
    const int row = lane & 31;
    return *reinterpret_cast<const uint4*>(tile + row * kRowBytes + swz(row, 2 * ds + (lane >> 5)) * 16);
}

// A operand of a product that contracts over the rows of the tile: dim 32 db + lane%32 of rows
// 16 s + 8 a + 4 (lane/32) + e (elements 4 a + e), the order in which the packed B operand holds them.
// `tr_base[a]` is the lane's address for db = 0, s = 0; blocks of 32 dims flip bits 2-3 of the slot.
__device__ inline uint4 col_operand(uint32_t tile_lds, const int (&tr_base)[2], int s, int db) {
    uint4 r;
#pragma unroll
    for (int a = 0; a < 2; a++) {
        const uint32_t addr = tile_lds + (uint32_t)((tr_base[a] ^ (db << 6)) + s * 16 * kRowBytes);
        const s16x4_t v =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(uintptr_t)addr);
        const uint2 u = __builtin_bit_cast(uint2, v);
        if (a == 0) {
            r.x = u.x;
            r.y = u.y;
        } else {
            r.z = u.x;
            r.w = u.y;
        }
    }
    return r;
}

__device__ inline void col_operand_setup(int lane, int (&tr_base)[2]) {
    const int h = lane >> 5, g16 = (lane >> 4) & 1, rl = lane & 15;
#pragma unroll
    for (int a = 0; a < 2; a++) {
        const int row = 8 * a + 4 * h + (rl >> 2);             // + 16 s
        const int piece = 2 * g16 + ((rl & 3) >> 1);           // + 4 db
        tr_base[a] = row * kRowBytes + swz(row, piece) * 16 + 8 * (rl & 1);
    }
}

template <typename T>
__device__ inline uint4 pack8(const f32x16& v, int s) {
    return make_uint4(Mma<T>::pack2(v[8 * s + 0], v[8 * s + 1]), Mma<T>::pack2(v[8 * s + 2], v[8 * s + 3]),
                      Mma<T>::pack2(v[8 * s + 4], v[8 * s + 5]), Mma<T>::pack2(v[8 * s + 6], v[8 * s + 7]));
}

// bits [0, n) set, for 0 <= n <= 32
__device__ inline uint32_t low_bits(int n) { return n >= 32 ? 0xffffffffu : ((1u << n) - 1u); }

// v if bit `bit` of `word` is set, else +0: a sign-extended one-bit field and a bitwise and
__device__ inline float keep_if_bit(float v, uint32_t word, int bit) {
    const int32_t m = (int32_t)(word << (31 - bit)) >> 31;
    return __uint_as_float(__float_as_uint(v) & (uint32_t)m);
}

__device__ inline f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; i++) z[i] = 0.f;
    return z;
}

// ---------------------------------------------------------------------------------------------
// dq
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(kThreads, 2) bwd_mfma_dq_kernel(BwdMfmaParams p) {
    __shared__ __attribute__((aligned(16))) unsigned char smem[2][2][kTile];  // [stage][K, V]
    const ckv_dense_bwd_args& a = p.a;
    const int tid = threadIdx.x, wave = tid / CKV_WAVE, lane = tid % CKV_WAVE, h = lane >> 5;
    const int64_t n_ctx = a.n_ctx, n_kv = a.n_kv, n_cached = n_kv - n_ctx;
    const int64_t bh = blockIdx.y, b = bh / a.H, hd = bh % a.H;
    const int64_t m_wg = (int64_t)blockIdx.x * kOwn;
    const int64_t m_lane = m_wg + wave * 32 + (lane & 31);  // this lane's query
    const char* kb = reinterpret_cast<const char*>(a.k) + (b * a.kv_stride[0] + hd * a.kv_stride[1]) * 2;
    const char* vb = reinterpret_cast<const char*>(a.v) + (b * a.kv_stride[0] + hd * a.kv_stride[1]) * 2;
    const int64_t kv_row = a.kv_stride[2] * 2;

    // stationary B operands: Q^T and dO^T of this lane's query, dims 16 ds + 8 h .. +7
    uint4 qreg[kHD / 16], greg[kHD / 16];
    {
        const char* qrow = reinterpret_cast<const char*>(a.q) +
                           (b * a.q_stride[0] + hd * a.q_stride[1] + m_lane * a.q_stride[2]) * 2;
        const char* grow = reinterpret_cast<const char*>(a.dout) +
                           (b * a.dout_stride[0] + hd * a.dout_stride[1] + m_lane * a.dout_stride[2]) * 2;
#pragma unroll
        for (int ds = 0; ds < kHD / 16; ds++) {
            qreg[ds] = greg[ds] = make_uint4(0u, 0u, 0u, 0u);
            if (m_lane < n_ctx) {
                qreg[ds] = *reinterpret_cast<const uint4*>(qrow + (16 * ds + 8 * h) * 2);
                greg[ds] = *reinterpret_cast<const uint4*>(grow + (16 * ds + 8 * h) * 2);
            }
        }
    }
    const bool row_ok = m_lane < n_ctx;
    const float nlse2 = row_ok ? -a.lse[bh * n_ctx + m_lane] * kLog2e : 0.f;
    const float delta = row_ok ? p.delta[bh * n_ctx + m_lane] : 0.f;
    const float c2 = a.scale * kLog2e;

    int tr_base[2];
    col_operand_setup(lane, tr_base);
    const uint32_t lds0 = lds_address(&smem[0][0][0]);

    f32x16 dq[kHD / 32];
#pragma unroll
    for (int db = 0; db < kHD / 32; db++) dq[db] = zero16();

    // keys past the diagonal of the workgroup's last row are visible to none of its rows
    int64_t m_last = m_wg + kOwn - 1;
    if (m_last > n_ctx - 1) m_last = n_ctx - 1;
    const int64_t n_end = n_cached + m_last + 1;
    const int nblk = (int)((n_end + kBlk - 1) / kBlk);

    // which keys of a block any query may see: inside the tensor, and not masked if cached.  The mask byte of the
    // block after this one is requested before that block's copies and looked at after this block's work, so
    // that nothing in between waits for memory.
    auto mask_byte = [&](int64_t n0) -> uint32_t {
        const int64_t n = n0 + (lane & 31);
        return n < n_kv ? (n < n_cached ? (uint32_t)a.mask[n] : 0u) : 1u;
    };
    uint32_t vis = (uint32_t)__ballot(mask_byte(0) == 0u);
    copy_block(kb, kv_row, 0, n_kv, lds0, wave, lane);
    copy_block(vb, kv_row, 0, n_kv, lds0 + kTile, wave, lane);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    for (int blk = 0; blk < nblk; blk++) {
        const int st = blk & 1;
        const int64_t n0 = (int64_t)blk * kBlk;
        uint32_t mb_next = 1u;
        if (blk + 1 < nblk) {  // the other stage was last read before the barrier that ended the step before
            mb_next = mask_byte(n0 + kBlk);
            __builtin_amdgcn_sched_barrier(0);
            copy_block(kb, kv_row, n0 + kBlk, n_kv, lds0 + (uint32_t)((st ^ 1) * 2 * kTile), wave, lane);
            copy_block(vb, kv_row, n0 + kBlk, n_kv, lds0 + (uint32_t)((st ^ 1) * 2 * kTile + kTile), wave, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        // keys of this block that are chunk keys past this wavefront's last row: nothing to do for it
        const bool chunk_part = n0 + kBlk > n_cached;
        // chunk key r of the block is visible to this lane's query iff r <= r_last (every r when the block is cached)
        int64_t r_last64 = m_lane + n_cached - n0;
        if (r_last64 > kBlk) r_last64 = kBlk;
        if (r_last64 < -1) r_last64 = -1;
        const int r_last = (int)r_last64;
        const int r_cached = n_cached - n0 >= kBlk ? kBlk : (n_cached > n0 ? (int)(n_cached - n0) : 0);  // r < r_cached: cached
        const int64_t wave_last = m_wg + wave * 32 + 31;
        const bool dead = vis == 0u || (n0 >= n_cached && n0 - n_cached > wave_last);
        if (!dead) {
            const unsigned char* kt = smem[st][0];
            const unsigned char* vt = smem[st][1];
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int ds = 0; ds < kHD / 16; ds++) {
                s = Mma<T>::mma(row_operand(kt, lane, ds), qreg[ds], s);
                if ((ds & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int ds = 0; ds < kHD / 16; ds++) {
                dp = Mma<T>::mma(row_operand(vt, lane, ds), greg[ds], dp);
                if ((ds & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
            // A lane is a query: a row past the end spoils only its own accumulators, which are never stored, so
            // no element tests its row.  A cached block with every key visible tests nothing at all.
            f32x16 dsv;
            if (vis == 0xffffffffu && !chunk_part) {
#pragma unroll
                for (int i = 0; i < 16; i++) dsv[i] = __builtin_amdgcn_exp2f(fmaf(s[i], c2, nlse2)) * (dp[i] - delta) * a.scale;
            } else {
                // bit r of `allow`: key r of the block is visible to this lane's query
                uint32_t allow = vis;
                if (chunk_part) allow &= low_bits(r_cached) | low_bits(r_last + 1);
                allow >>= 4 * h;  // element i looks at key 8 (i / 4) + 4 h + i % 4
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const float pe = keep_if_bit(__builtin_amdgcn_exp2f(fmaf(s[i], c2, nlse2)), allow, 8 * (i / 4) + (i % 4));
                    dsv[i] = pe * (dp[i] - delta) * a.scale;
                }
            }
            const uint32_t kt_lds = lds0 + (uint32_t)(st * 2 * kTile);
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const uint4 bop = pack8<T>(dsv, s2);
#pragma unroll
                for (int db = 0; db < kHD / 32; db++) {
                    dq[db] = Mma<T>::mma(col_operand(kt_lds, tr_base, s2, db), bop, dq[db]);
                    if (db & 1) __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's copies of the next block have landed
        vis = (uint32_t)__ballot(mb_next == 0u);
        __syncthreads();
    }
    if (row_ok) {
        char* out = reinterpret_cast<char*>(a.dq) + (b * a.dq_stride[0] + hd * a.dq_stride[1] + m_lane * a.dq_stride[2]) * 2;
#pragma unroll
        for (int db = 0; db < kHD / 32; db++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int d = 32 * db + 8 * j + 4 * h;
                *reinterpret_cast<uint2*>(out + d * 2) = make_uint2(Mma<T>::pack2(dq[db][4 * j], dq[db][4 * j + 1]),
                                                                    Mma<T>::pack2(dq[db][4 * j + 2], dq[db][4 * j + 3]));
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dk, dv
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(kThreads, 2) bwd_mfma_dkdv_kernel(BwdMfmaParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_smem[];
    typedef unsigned char (*TilePtr)[2][kTile];
    typedef float (*RowPtr)[2][kBlk];
    TilePtr smem = reinterpret_cast<TilePtr>(dyn_smem);                                  // [stage][Q, dO]
    RowPtr rowv = reinterpret_cast<RowPtr>(dyn_smem + kDkdvRowv);                        // [stage][-lse log2 e, delta]
    // the V^T operands of a wavefront's 32 keys, in operand order: [wave][ds][lane] 16 bytes each
    uint4* vstat = reinterpret_cast<uint4*>(dyn_smem + kDkdvV) + (threadIdx.x / CKV_WAVE) * (kHD / 16) * CKV_WAVE;
    const ckv_dense_bwd_args& a = p.a;
    const int tid = threadIdx.x, wave = tid / CKV_WAVE, lane = tid % CKV_WAVE, h = lane >> 5;
    const int64_t n_ctx = a.n_ctx, n_kv = a.n_kv, n_cached = n_kv - n_ctx;
    const int64_t bh = blockIdx.y, b = bh / a.H, hd = bh % a.H;
    const int64_t n_wg = (int64_t)blockIdx.x * kOwn;
    const int64_t n_lane = n_wg + wave * 32 + (lane & 31);  // this lane's key
    const char* qb = reinterpret_cast<const char*>(a.q) + (b * a.q_stride[0] + hd * a.q_stride[1]) * 2;
    const char* gb = reinterpret_cast<const char*>(a.dout) + (b * a.dout_stride[0] + hd * a.dout_stride[1]) * 2;
    const int64_t q_row = a.q_stride[2] * 2, g_row = a.dout_stride[2] * 2;
    const float* lse = a.lse + bh * n_ctx;
    const float* dl = p.delta + bh * n_ctx;

    // stationary B operands: K^T of this lane's key in registers, V^T in LDS (the registers go to the accumulators)
    uint4 kreg[kHD / 16];
    {
        const int64_t off = (b * a.kv_stride[0] + hd * a.kv_stride[1] + n_lane * a.kv_stride[2]) * 2;
        const char* krow = reinterpret_cast<const char*>(a.k) + off;
        const char* vrow = reinterpret_cast<const char*>(a.v) + off;
#pragma unroll
        for (int ds = 0; ds < kHD / 16; ds++) {
            kreg[ds] = make_uint4(0u, 0u, 0u, 0u);
            uint4 vv = make_uint4(0u, 0u, 0u, 0u);
            if (n_lane < n_kv) {
                kreg[ds] = *reinterpret_cast<const uint4*>(krow + (16 * ds + 8 * h) * 2);
                vv = *reinterpret_cast<const uint4*>(vrow + (16 * ds + 8 * h) * 2);
            }
            vstat[ds * CKV_WAVE + lane] = vv;
        }
    }
    bool key_ok = n_lane < n_kv;
    if (key_ok && n_lane < n_cached) key_ok = a.mask[n_lane] == 0;
    const int64_t first_row = n_lane < n_cached ? 0 : n_lane - n_cached;  // the first query that sees this key
    const float c2 = a.scale * kLog2e;

    int tr_base[2];
    col_operand_setup(lane, tr_base);
    const uint32_t lds0 = lds_address(dyn_smem);

    f32x16 dk[kHD / 32], dv[kHD / 32];
#pragma unroll
    for (int db = 0; db < kHD / 32; db++) dk[db] = dv[db] = zero16();

    // the first query block any key of the workgroup can be seen from
    const int64_t m_first = n_wg < n_cached ? 0 : n_wg - n_cached;
    const int blk0 = (int)(m_first / kBlk);
    const int nblk = (int)((n_ctx + kBlk - 1) / kBlk);
    // does any key of this wavefront exist and pass its mask?
    const bool wave_alive = __ballot(key_ok) != 0ull;
    const int64_t wave_first_key = n_wg + wave * 32;

    auto load_rowv = [&](int st, int64_t m0) {
        if (tid < 2 * kBlk) {
            const int64_t m = m0 + (tid & (kBlk - 1));
            float v = 0.f;
            if (m < n_ctx) v = tid < kBlk ? -lse[m] * kLog2e : dl[m];
            rowv[st][tid / kBlk][tid & (kBlk - 1)] = v;
        }
    };
    if (blk0 < nblk) {
        copy_block(qb, q_row, (int64_t)blk0 * kBlk, n_ctx, lds0 + (uint32_t)((blk0 & 1) * 2 * kTile), wave, lane);
        copy_block(gb, g_row, (int64_t)blk0 * kBlk, n_ctx, lds0 + (uint32_t)((blk0 & 1) * 2 * kTile + kTile), wave, lane);
        load_rowv(blk0 & 1, (int64_t)blk0 * kBlk);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    for (int blk = blk0; blk < nblk; blk++) {
        const int st = blk & 1;
        const int64_t m0 = (int64_t)blk * kBlk;
        const bool more = blk + 1 < nblk;
        float rv_next = 0.f;  // this thread's per-row scalar of the next block: requested first, parked in LDS last
        if (more) {  // the other stage was last read before the barrier that ended the step before
            if (tid < 2 * kBlk) {
                const int64_t m = m0 + kBlk + (tid & (kBlk - 1));
                if (m < n_ctx) rv_next = tid < kBlk ? lse[m] : dl[m];
            }
            __builtin_amdgcn_sched_barrier(0);
            copy_block(qb, q_row, m0 + kBlk, n_ctx, lds0 + (uint32_t)((st ^ 1) * 2 * kTile), wave, lane);
            copy_block(gb, g_row, m0 + kBlk, n_ctx, lds0 + (uint32_t)((st ^ 1) * 2 * kTile + kTile), wave, lane);
        }
        // rows before the first chunk key of the wavefront's keys see none of them when all its keys are chunk keys
        const bool dead = !wave_alive || (wave_first_key >= n_cached && wave_first_key - n_cached > m0 + kBlk - 1);
        if (!dead) {
            const unsigned char* qt = smem[st][0];
            const unsigned char* gt = smem[st][1];
            // rows r of the block with r_lo <= r < r_hi see this lane's key
            int64_t lo64 = first_row - m0, hi64 = n_ctx - m0;
            if (lo64 < 0) lo64 = 0;
            if (lo64 > kBlk) lo64 = kBlk;
            if (hi64 > kBlk) hi64 = kBlk;
            // A lane is a key: a masked or absent key spoils only its own accumulators, which are stored as zeros.
            const int r_lo = (int)lo64, r_hi = (int)hi64;
            const bool plain = __ballot(r_lo > 0) == 0ull && r_hi == kBlk;  // every row of the block sees every key
            // bit r of `allow`: row r of the block sees this lane's key; element i looks at row 8 (i / 4) + 4 h + i % 4
            const uint32_t allow = (low_bits(r_hi) & ~low_bits(r_lo)) >> (4 * h);
            const uint32_t qt_lds = lds0 + (uint32_t)(st * 2 * kTile), gt_lds = qt_lds + kTile;
            // The phases are fenced so that the compiler keeps their registers apart: P, then dV, then dP and dS, then dK.
            f32x16 pv = zero16();
#pragma unroll
            for (int ds = 0; ds < kHD / 16; ds++) {
                pv = Mma<T>::mma(row_operand(qt, lane, ds), kreg[ds], pv);
                if ((ds & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 nl = *reinterpret_cast<const float4*>(&rowv[st][0][8 * j + 4 * h]);
                const float nls[4] = {nl.x, nl.y, nl.z, nl.w};
#pragma unroll
                for (int e = 0; e < 4; e++) pv[4 * j + e] = __builtin_amdgcn_exp2f(fmaf(pv[4 * j + e], c2, nls[e]));
            }
            if (!plain) {
#pragma unroll
                for (int i = 0; i < 16; i++) pv[i] = keep_if_bit(pv[i], allow, 8 * (i / 4) + (i % 4));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const uint4 pb = pack8<T>(pv, s2);
#pragma unroll
                for (int db = 0; db < kHD / 32; db++) {
                    dv[db] = Mma<T>::mma(col_operand(gt_lds, tr_base, s2, db), pb, dv[db]);
                    if (db & 1) __builtin_amdgcn_sched_barrier(0);
                }
            }
            f32x16 dp = zero16();
#pragma unroll
            for (int ds = 0; ds < kHD / 16; ds++) {
                dp = Mma<T>::mma(row_operand(gt, lane, ds), vstat[ds * CKV_WAVE + lane], dp);
                if (ds & 1) __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 de = *reinterpret_cast<const float4*>(&rowv[st][1][8 * j + 4 * h]);
                const float des[4] = {de.x, de.y, de.z, de.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int i = 4 * j + e;
                    dp[i] = pv[i] * (dp[i] - des[e]) * a.scale;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                const uint4 db_ = pack8<T>(dp, s2);
#pragma unroll
                for (int db = 0; db < kHD / 32; db++) {
                    dk[db] = Mma<T>::mma(col_operand(qt_lds, tr_base, s2, db), db_, dk[db]);
                    if (db & 1) __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's copies of the next block have landed
        if (more && tid < 2 * kBlk) rowv[st ^ 1][tid / kBlk][tid & (kBlk - 1)] = tid < kBlk ? -rv_next * kLog2e : rv_next;
        __syncthreads();
    }
    if (!key_ok) {
#pragma unroll
        for (int db = 0; db < kHD / 32; db++) dk[db] = dv[db] = zero16();
    }
    if (n_lane < n_kv) {
        const int64_t off = (b * a.dkv_stride[0] + hd * a.dkv_stride[1] + n_lane * a.dkv_stride[2]) * 2;
        char* ok_ = reinterpret_cast<char*>(a.dk) + off;
        char* ov_ = reinterpret_cast<char*>(a.dv) + off;
#pragma unroll
        for (int db = 0; db < kHD / 32; db++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int d = 32 * db + 8 * j + 4 * h;
                *reinterpret_cast<uint2*>(ok_ + d * 2) = make_uint2(Mma<T>::pack2(dk[db][4 * j], dk[db][4 * j + 1]),
                                                                    Mma<T>::pack2(dk[db][4 * j + 2], dk[db][4 * j + 3]));
                *reinterpret_cast<uint2*>(ov_ + d * 2) = make_uint2(Mma<T>::pack2(dv[db][4 * j], dv[db][4 * j + 1]),
                                                                    Mma<T>::pack2(dv[db][4 * j + 2], dv[db][4 * j + 3]));
            }
        }
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// unit stride along the head dim, 16-byte addressable rows, and 32 rows apart still within a 32-bit byte offset
inline bool rows_ok(const int64_t* st) {
    return st[3] == 1 && st[2] % 8 == 0 && st[1] % 8 == 0 && st[0] % 8 == 0 && st[2] > 0 && st[2] < (1 << 24);
}

template <typename T>
int run(const BwdMfmaParams& p, hipStream_t stream) {
    const ckv_dense_bwd_args& a = p.a;
    hipLaunchKernelGGL(bwd_mfma_dq_kernel<T>, dim3((unsigned)((a.n_ctx + kOwn - 1) / kOwn), (unsigned)(a.B * a.H)),
                       dim3(kThreads), 0, stream, p);
    CKV_HIP_TRY(hipGetLastError());
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(bwd_mfma_dkdv_kernel<T>), kDkdvLds)) return rc;
    hipLaunchKernelGGL(bwd_mfma_dkdv_kernel<T>, dim3((unsigned)((a.n_kv + kOwn - 1) / kOwn), (unsigned)(a.B * a.H)),
                       dim3(kThreads), kDkdvLds, stream, p);
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

}  // namespace

bool bwd_mfma_supported(const ckv_dense_bwd_args& a) {
    if (a.dtype != CKV_F16 && a.dtype != CKV_BF16) return false;
    if (a.D != kHD) return false;
    if (!rows_ok(a.q_stride) || !rows_ok(a.kv_stride) || !rows_ok(a.dout_stride) || !rows_ok(a.dq_stride) ||
        !rows_ok(a.dkv_stride))
        return false;
    return aligned16(a.q) && aligned16(a.k) && aligned16(a.v) && aligned16(a.dout) && aligned16(a.dq) &&
           aligned16(a.dk) && aligned16(a.dv);
}

int launch_bwd_mfma(const ckv_dense_bwd_args& a, const float* delta, hipStream_t stream) {
    BwdMfmaParams p;
    p.a = a;
    p.delta = delta;
    return a.dtype == CKV_F16 ? run<__half>(p, stream) : run<__hip_bfloat16>(p, stream);
}

}  // namespace ckv
