// fp32-math attention kernels for every dtype: the parity path for float32 caches and the
// fallback for shapes the MFMA kernels do not take.  Also the small shared stages: score-sum
// weights, the rotate+gather prologue, and the head-reduction / EMA epilogue.
#include "ckv_attn_internal.h"

namespace ckv {
namespace {

template <typename T>
__device__ inline float round_t(float v) {
    return Elem<T>::to_float(Elem<T>::from_float(v));
}

// ---------------------------------------------------------------------------------------------
// weights: w_ema[m] = (1-beta) * beta^(Q-1-m) as fp32 (cascade_attention.py:315-317);
//          w_new[k] = (1-beta) * beta^k built in the tensor dtype (cascade_attention.py:270-276)
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void weights_kernel(float* w_ema, float* w_new, int64_t Q, double beta) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Q + kColSlack) return;
    if (i >= Q) {  // slack read (and multiplied by zero) by the MFMA column pass
        w_ema[i] = 0.f;
        return;
    }
    const float omb = (float)(1.0 - beta);
    const float b32 = (float)beta;
    w_ema[i] = __fmul_rn(omb, powf(b32, (float)(Q - 1 - i)));
    const float bt = round_t<T>(b32);
    const float pw = round_t<T>(powf(bt, round_t<T>((float)i)));
    w_new[i] = round_t<T>(__fmul_rn(omb, pw));
}

// ---------------------------------------------------------------------------------------------
// prologue: rotate and gather.  One thread per (row, rotation pair).
// Rotation is evaluated in the tensor dtype exactly like x*cos + rotate_half(x)*sin
// (cascade_attention.py:31-35) with cos/sin from fp32 angles cast to the dtype
// (modeling_llama.py:205-220); the rotated row is then multiplied by sqrt(softmax scale) and rounded
// again, as the eager path does to queries and keys alike (cascade_attention.py:284-291).
// ---------------------------------------------------------------------------------------------
template <typename T>
__device__ inline void rotate_pair(const T* src, int64_t sd, T* dst, int64_t j, int64_t half, int64_t pos,
                                   const float* inv_freq, float theta, int64_t D, float post) {
    const float f = inv_freq ? inv_freq[j] : 1.0f / powf(theta, (float)(2 * j) / (float)D);
    const float ang = __fmul_rn((float)pos, f);
    float sn, cs;
    sincosf(ang, &sn, &cs);
    cs = round_t<T>(cs);
    sn = round_t<T>(sn);
    const float x1 = Elem<T>::to_float(src[j * sd]);
    const float x2 = Elem<T>::to_float(src[(j + half) * sd]);
    // out[j] = x1*cos + (-x2)*sin ; out[j+half] = x2*cos + x1*sin, each product rounded first
    const float o1 = round_t<T>(__fadd_rn(round_t<T>(__fmul_rn(x1, cs)), round_t<T>(__fmul_rn(-x2, sn))));
    const float o2 = round_t<T>(__fadd_rn(round_t<T>(__fmul_rn(x2, cs)), round_t<T>(__fmul_rn(x1, sn))));
    dst[j] = Elem<T>::from_float(__fmul_rn(o1, post));
    dst[j + half] = Elem<T>::from_float(__fmul_rn(o2, post));
}

template <typename T>
__global__ void prep_generic_kernel(ckv_attn_args a, T* qr, T* kr, T* vc, uint8_t* kmasked, float post) {
    const int64_t D = a.D, half = D / 2, NS = a.num_sink, S = a.S, Q = a.Q;
    const int64_t N = NS + S + Q;
    const int64_t n_key_items = a.B * a.KVH * N * half;
    const int64_t n_q_items = a.B * a.H * Q * half;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < NS + S) kmasked[idx] = idx < NS ? a.sink_mask[idx] : a.mask[idx - NS];
    if (idx < n_key_items) {
        const int64_t j = idx % half;
        const int64_t n = (idx / half) % N;
        const int64_t kvh = (idx / (half * N)) % a.KVH;
        const int64_t b = idx / (half * N * a.KVH);
        const T *ks, *vs;
        int64_t sd, pos;
        if (n < NS) {
            const int64_t off = b * a.sink_stride[0] + kvh * a.sink_stride[1] + n * a.sink_stride[2];
            ks = (const T*)a.sink_k + off;
            vs = (const T*)a.sink_v + off;
            sd = a.sink_stride[3];
            pos = a.sink_pos[b * a.sink_pos_stride[0] + kvh * a.sink_pos_stride[1] + n];
        } else if (n < NS + S) {
            const int64_t slot = n - NS;
            const int64_t off = b * a.cache_stride[0] + kvh * a.cache_stride[1] + slot * a.cache_stride[2];
            ks = (const T*)a.cache_k + off;
            vs = (const T*)a.cache_v + off;
            sd = a.cache_stride[3];
            pos = a.pos[b * a.pos_stride[0] + kvh * a.pos_stride[1] + slot] + a.pos_shift;
        } else {
            const int64_t m = n - NS - S;
            const int64_t off = b * a.kv_new_stride[0] + kvh * a.kv_new_stride[1] + m * a.kv_new_stride[2];
            ks = (const T*)a.k_new + off;
            vs = (const T*)a.v_new + off;
            sd = a.kv_new_stride[3];
            pos = a.q_pos[m];
        }
        T* kd = kr + ((b * a.KVH + kvh) * N + n) * D;
        T* vd = vc + ((b * a.KVH + kvh) * N + n) * D;
        rotate_pair<T>(ks, sd, kd, j, half, pos, a.inv_freq, a.rope_theta, D, post);
        vd[j] = vs[j * sd];
        vd[j + half] = vs[(j + half) * sd];
    }
    if (idx < n_q_items) {
        const int64_t j = idx % half;
        const int64_t m = (idx / half) % Q;
        const int64_t h = (idx / (half * Q)) % a.H;
        const int64_t b = idx / (half * Q * a.H);
        const T* qs = (const T*)a.q + b * a.q_stride[0] + h * a.q_stride[1] + m * a.q_stride[2];
        T* qd = qr + ((b * a.H + h) * Q + m) * D;
        rotate_pair<T>(qs, a.q_stride[3], qd, j, half, a.q_pos[m], a.inv_freq, a.rope_theta, D, post);
    }
}

// ---------------------------------------------------------------------------------------------
// forward: one wavefront per query row, lanes = keys for the logits, lanes = dims for P.V.  The four rows of a
// workgroup are consecutive; when they belong to one (batch, kv head) the workgroup stages each chunk of 64 keys
// in LDS once for all four (K rows 16-byte aligned at a pitch of D + 4 floats, V as is), otherwise every
// wavefront reads its own rows from memory.  Either way a row sees the same operands in the same order, and
// every sum is one chain of fused multiply-adds in ascending order of its index, so the result does not depend
// on the path.  DS > 0: the head size, known at compile time (the query row then lives in registers).
// ---------------------------------------------------------------------------------------------
constexpr int kMaxD = 256;

// element e of a 16-byte piece of a row of T, as a float
template <typename T>
__device__ inline float piece_elem(const uint32_t (&w)[4], int e) {
    if constexpr (sizeof(T) == 4) {
        return __uint_as_float(w[e]);
    } else {
        const uint16_t bits = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
        return Elem<T>::to_float(__builtin_bit_cast(T, bits));
    }
}

template <typename T, int DS>
__global__ void __launch_bounds__(256) fwd_generic_kernel(CoreProblem p) {
    extern __shared__ __attribute__((aligned(16))) float kv_tile[];  // K [64][D + 4], V [64][D]
    __shared__ __attribute__((aligned(16))) float q_lds[4][kMaxD];
    __shared__ __attribute__((aligned(16))) float pe_lds[4][CKV_WAVE];
    __shared__ int64_t n_end_lds[4];
    const int wave = threadIdx.x / CKV_WAVE, lane = threadIdx.x % CKV_WAVE;
    const int64_t rows = p.B * p.H * p.Q;
    const int64_t row0 = (int64_t)blockIdx.x * 4;
    int64_t row = row0 + wave;
    const bool active = row < rows;
    if (!active) row = rows - 1;
    const int64_t m = row % p.Q;
    const int64_t h = (row / p.Q) % p.H;
    const int64_t b = row / (p.Q * p.H);
    const int64_t G = p.H / p.KVH, kvh = h / G;
    const int64_t D = DS > 0 ? DS : p.D, N = p.N, Nc = N - p.Q;
    const T* qrow = (const T*)p.q + b * p.q_stride[0] + h * p.q_stride[1] + m * p.q_stride[2];
    for (int64_t d = lane; d < D; d += CKV_WAVE) q_lds[wave][d] = Elem<T>::to_float(qrow[d * p.q_stride[3]]);
    const int64_t n_end = Nc + m + 1;  // keys past the diagonal are never visible
    if (lane == 0) n_end_lds[wave] = active ? n_end : 0;
    __syncthreads();
    // one (batch, kv head) for the whole workgroup?  Rows are ordered (batch, head, position), so the first and
    // the last row decide.
    const int64_t row3 = row0 + 3 < rows ? row0 + 3 : rows - 1;
    const bool shared_kv = row0 / (p.Q * p.H) == row3 / (p.Q * p.H) &&
                           ((row0 / p.Q) % p.H) / G == ((row3 / p.Q) % p.H) / G;
    int64_t n_end_wg = n_end_lds[0];
    for (int w = 1; w < 4; w++) n_end_wg = n_end_lds[w] > n_end_wg ? n_end_lds[w] : n_end_wg;
    const T* kbase = (const T*)p.k + b * p.kv_stride[0] + kvh * p.kv_stride[1];
    const T* vbase = (const T*)p.v + b * p.kv_stride[0] + kvh * p.kv_stride[1];
    const int64_t pitch = D + 4;
    float* k_t = kv_tile;
    float* v_t = kv_tile + CKV_WAVE * pitch;
    float qreg[DS > 0 ? DS : 1];
    if (DS > 0) {
#pragma unroll
        for (int d = 0; d < DS; d += 4) {
            const float4 q4 = *reinterpret_cast<const float4*>(&q_lds[wave][d]);
            qreg[d] = q4.x;
            qreg[d + 1] = q4.y;
            qreg[d + 2] = q4.z;
            qreg[d + 3] = q4.w;
        }
    }

    float m_run = -INFINITY, l_run = 0.f;
    float o[kMaxD / CKV_WAVE] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t base = 0; base < n_end_wg; base += CKV_WAVE) {
        if (shared_kv) {
            __syncthreads();  // the chunk before is no longer read
            for (int64_t i = threadIdx.x; i < CKV_WAVE * D; i += 256) {
                const int64_t r = i / D, d = i % D, nn = base + r;
                float kx = 0.f, vx = 0.f;
                if (nn < n_end_wg) {
                    kx = Elem<T>::to_float(kbase[nn * p.kv_stride[2] + d * p.kv_stride[3]]);
                    vx = Elem<T>::to_float(vbase[nn * p.kv_stride[2] + d * p.kv_stride[3]]);
                }
                k_t[r * pitch + d] = kx;
                v_t[r * D + d] = vx;
            }
            __syncthreads();
        }
        if (!active || base >= n_end) continue;
        const int64_t n = base + lane;
        bool valid = n < n_end;
        if (valid && n < Nc && p.kmasked) valid = p.kmasked[n] == 0;
        float s = -INFINITY;
        if (valid) {
            float acc = 0.f;
            if (shared_kv) {
                const float* kr = k_t + lane * pitch;
                if (DS > 0) {
#pragma unroll
                    for (int d = 0; d < DS; d += 4) {
                        const float4 k4 = *reinterpret_cast<const float4*>(kr + d);
                        acc = fmaf(qreg[d], k4.x, acc);
                        acc = fmaf(qreg[d + 1], k4.y, acc);
                        acc = fmaf(qreg[d + 2], k4.z, acc);
                        acc = fmaf(qreg[d + 3], k4.w, acc);
                    }
                } else {
                    for (int64_t d = 0; d < D; d++) acc = fmaf(q_lds[wave][d], kr[d], acc);
                }
            } else {
                const T* kr = kbase + n * p.kv_stride[2];
                for (int64_t d = 0; d < D; d++) acc = fmaf(q_lds[wave][d], Elem<T>::to_float(kr[d * p.kv_stride[3]]), acc);
            }
            s = acc * p.scale;
        }
        float cmax = s;
        for (int off = 32; off > 0; off >>= 1) cmax = fmaxf(cmax, __shfl_xor(cmax, off));
        if (cmax == -INFINITY) continue;  // nothing visible in this chunk
        const float m_new = fmaxf(m_run, cmax);
        const float pe = valid ? expf(s - m_new) : 0.f;
        float csum = pe;
        for (int off = 32; off > 0; off >>= 1) csum += __shfl_xor(csum, off);
        const float alpha = m_run == -INFINITY ? 0.f : expf(m_run - m_new);
        l_run = l_run * alpha + csum;
        m_run = m_new;
#pragma unroll
        for (int r = 0; r < kMaxD / CKV_WAVE; r++) o[r] *= alpha;
        const int64_t cnt = n_end - base < CKV_WAVE ? n_end - base : CKV_WAVE;
        // the probabilities of the chunk go through LDS: every lane reads them all, four at a time (the wavefront's
        // own row of pe_lds: written and read by the same wavefront, in program order)
        pe_lds[wave][lane] = pe;
        for (int j4 = 0; j4 < cnt; j4 += 4) {
            const float4 p4 = *reinterpret_cast<const float4*>(&pe_lds[wave][j4]);
            const float pj4[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int j = j4 + e;
                const float pj = pj4[e];
                if (j >= cnt || pj == 0.f) continue;  // a hidden key's V row is never touched (it may hold anything)
                if (shared_kv) {
                    const float* vr = v_t + j * D;
#pragma unroll
                    for (int r = 0; r < kMaxD / CKV_WAVE; r++) {
                        const int64_t d = lane + r * CKV_WAVE;
                        if (d < D) o[r] = fmaf(pj, vr[d], o[r]);
                    }
                } else {
                    const T* vr = vbase + (base + j) * p.kv_stride[2];
#pragma unroll
                    for (int r = 0; r < kMaxD / CKV_WAVE; r++) {
                        const int64_t d = lane + r * CKV_WAVE;
                        if (d < D) o[r] = fmaf(pj, Elem<T>::to_float(vr[d * p.kv_stride[3]]), o[r]);
                    }
                }
            }
        }
    }
    if (!active) return;
    const float inv = 1.f / l_run;
    T* orow = (T*)p.out + b * p.out_stride[0] + h * p.out_stride[1] + m * p.out_stride[2];
#pragma unroll
    for (int r = 0; r < kMaxD / CKV_WAVE; r++) {
        const int64_t d = lane + r * CKV_WAVE;
        if (d < D) orow[d * p.out_stride[3]] = Elem<T>::from_float(o[r] * inv);
    }
    if (lane == 0 && p.lse) p.lse[row] = m_run + logf(l_run);
}

// ---------------------------------------------------------------------------------------------
// forward, several rows per wavefront: the same arithmetic as fwd_generic_kernel, row by row, for head sizes known
// at compile time and chunks whose length is a multiple of the 4 x R rows of a workgroup (so that a workgroup never
// straddles two heads).  A staged chunk of 64 keys then serves 4 x R rows, and a K or V element read from LDS
// serves R of them: the one-row kernel is bound by what its workgroups re-read through the L2.
// ---------------------------------------------------------------------------------------------
template <typename T, int DS, int R>
__global__ void __launch_bounds__(256) fwd_generic_rows_kernel(CoreProblem p) {
    extern __shared__ __attribute__((aligned(16))) float kv_tile[];  // K [64][DS + 4], V [64][DS]
    __shared__ __attribute__((aligned(16))) float q_lds[4 * R][DS];
    __shared__ __attribute__((aligned(16))) float pe_lds[4][R][CKV_WAVE];
    const int wave = threadIdx.x / CKV_WAVE, lane = threadIdx.x % CKV_WAVE;
    const int64_t row0 = (int64_t)blockIdx.x * (4 * R);   // all rows exist and share (b, h): Q % (4 R) == 0
    const int64_t m0 = row0 % p.Q;
    const int64_t h = (row0 / p.Q) % p.H;
    const int64_t b = row0 / (p.Q * p.H);
    const int64_t G = p.H / p.KVH, kvh = h / G;
    const int64_t N = p.N, Nc = N - p.Q;
    constexpr int pitch = DS + 4;
    {
        const T* qrows = (const T*)p.q + b * p.q_stride[0] + h * p.q_stride[1];
        for (int i = threadIdx.x; i < 4 * R * DS; i += 256) {
            const int r = i / DS, d = i % DS;
            q_lds[r][d] = Elem<T>::to_float(qrows[(m0 + r) * p.q_stride[2] + d * p.q_stride[3]]);
        }
    }
    const T* kbase = (const T*)p.k + b * p.kv_stride[0] + kvh * p.kv_stride[1];
    const T* vbase = (const T*)p.v + b * p.kv_stride[0] + kvh * p.kv_stride[1];
    float* k_t = kv_tile;
    float* v_t = kv_tile + CKV_WAVE * pitch;
    const int64_t n_end_wg = Nc + m0 + 4 * R;  // what the last row of the workgroup sees
    float m_run[R], l_run[R], o[R][DS / CKV_WAVE];
#pragma unroll
    for (int i = 0; i < R; i++) {
        m_run[i] = -INFINITY;
        l_run[i] = 0.f;
#pragma unroll
        for (int r = 0; r < DS / CKV_WAVE; r++) o[i][r] = 0.f;
    }
    for (int64_t base = 0; base < n_end_wg; base += CKV_WAVE) {
        __syncthreads();  // the chunk before is no longer read (the first time: the queries are in place)
        for (int i = threadIdx.x; i < CKV_WAVE * DS; i += 256) {
            const int r = i / DS, d = i % DS;
            const int64_t nn = base + r;
            float kx = 0.f, vx = 0.f;
            if (nn < n_end_wg) {
                kx = Elem<T>::to_float(kbase[nn * p.kv_stride[2] + d * p.kv_stride[3]]);
                vx = Elem<T>::to_float(vbase[nn * p.kv_stride[2] + d * p.kv_stride[3]]);
            }
            k_t[r * pitch + d] = kx;
            v_t[r * DS + d] = vx;
        }
        __syncthreads();
        const int64_t n = base + lane;
        const bool key_ok = !(n < Nc && p.kmasked && p.kmasked[n < Nc ? n : 0] != 0);
        // logits of this lane's key for the R rows: one pass over the key row, R chains
        float acc[R];
#pragma unroll
        for (int i = 0; i < R; i++) acc[i] = 0.f;
        const float* kr = k_t + lane * pitch;
#pragma unroll 8
        for (int d = 0; d < DS; d += 4) {
            const float4 k4 = *reinterpret_cast<const float4*>(kr + d);
#pragma unroll
            for (int i = 0; i < R; i++) {
                const float4 q4 = *reinterpret_cast<const float4*>(&q_lds[wave * R + i][d]);
                acc[i] = fmaf(q4.x, k4.x, acc[i]);
                acc[i] = fmaf(q4.y, k4.y, acc[i]);
                acc[i] = fmaf(q4.z, k4.z, acc[i]);
                acc[i] = fmaf(q4.w, k4.w, acc[i]);
            }
        }
        int cnt[R];
        bool upd[R];
#pragma unroll
        for (int i = 0; i < R; i++) {
            const int64_t n_end = Nc + m0 + wave * R + i + 1;
            cnt[i] = 0;
            upd[i] = false;
            if (base >= n_end) continue;
            const bool valid = n < n_end && key_ok;
            const float s = valid ? acc[i] * p.scale : -INFINITY;
            float cmax = s;
            for (int off = 32; off > 0; off >>= 1) cmax = fmaxf(cmax, __shfl_xor(cmax, off));
            if (cmax == -INFINITY) continue;  // nothing visible in this chunk
            const float m_new = fmaxf(m_run[i], cmax);
            const float pe = valid ? expf(s - m_new) : 0.f;
            float csum = pe;
            for (int off = 32; off > 0; off >>= 1) csum += __shfl_xor(csum, off);
            const float alpha = m_run[i] == -INFINITY ? 0.f : expf(m_run[i] - m_new);
            l_run[i] = l_run[i] * alpha + csum;
            m_run[i] = m_new;
#pragma unroll
            for (int r = 0; r < DS / CKV_WAVE; r++) o[i][r] *= alpha;
            cnt[i] = n_end - base < CKV_WAVE ? (int)(n_end - base) : CKV_WAVE;
            upd[i] = true;
            pe_lds[wave][i][lane] = pe;
        }
        int cnt_max = 0;
#pragma unroll
        for (int i = 0; i < R; i++) cnt_max = cnt[i] > cnt_max ? cnt[i] : cnt_max;
        // P.V: a V element read once serves the R rows; per row the keys are added in ascending order, a key with
        // probability 0 (hidden, or past the row's diagonal) is not touched
        for (int j4 = 0; j4 < cnt_max; j4 += 4) {
            float pj[R][4];
#pragma unroll
            for (int i = 0; i < R; i++) {
                float4 p4 = make_float4(0.f, 0.f, 0.f, 0.f);
                if (upd[i]) p4 = *reinterpret_cast<const float4*>(&pe_lds[wave][i][j4]);
                pj[i][0] = p4.x;
                pj[i][1] = p4.y;
                pj[i][2] = p4.z;
                pj[i][3] = p4.w;
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int j = j4 + e;
                const float* vr = v_t + j * DS;
                float vv[DS / CKV_WAVE];
#pragma unroll
                for (int r = 0; r < DS / CKV_WAVE; r++) vv[r] = vr[lane + r * CKV_WAVE];
#pragma unroll
                for (int i = 0; i < R; i++) {
                    if (j >= cnt[i] || pj[i][e] == 0.f) continue;
#pragma unroll
                    for (int r = 0; r < DS / CKV_WAVE; r++) o[i][r] = fmaf(pj[i][e], vv[r], o[i][r]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
        const int64_t m = m0 + wave * R + i;
        const float inv = 1.f / l_run[i];
        T* orow = (T*)p.out + b * p.out_stride[0] + h * p.out_stride[1] + m * p.out_stride[2];
#pragma unroll
        for (int r = 0; r < DS / CKV_WAVE; r++) orow[(lane + r * CKV_WAVE) * p.out_stride[3]] = Elem<T>::from_float(o[i][r] * inv);
        if (lane == 0 && p.lse) p.lse[row0 + wave * R + i] = m_run[i] + logf(l_run[i]);
    }
}

// ---------------------------------------------------------------------------------------------
// score sums: one wavefront per (b, h, 64 keys); lanes = keys, loop over the query rows.  DS > 0: the head size,
// known at compile time: the query rows then pass through LDS and four of them share each read of the key row.
// ---------------------------------------------------------------------------------------------
constexpr int kColQTile = 32;  // query rows per LDS tile of the score kernel (a multiple of 4)

template <typename T, int DS>
__global__ void __launch_bounds__(CKV_WAVE) colsum_generic_kernel(CoreProblem p) {
    extern __shared__ __attribute__((aligned(16))) float k_lds[];  // K [64][D + 1]; with DS > 0: K [64][DS + 4], Q [kColQTile][DS]
    const int lane = threadIdx.x;
    const int64_t D = DS > 0 ? DS : p.D, N = p.N, Q = p.Q, Nc = N - Q;
    const int64_t chunks = (N + CKV_WAVE - 1) / CKV_WAVE;
    const int64_t c = blockIdx.x % chunks;
    const int64_t h = (blockIdx.x / chunks) % p.H;
    const int64_t b = blockIdx.x / (chunks * p.H);
    const int64_t G = p.H / p.KVH, kvh = h / G;
    const int64_t n = c * CKV_WAVE + lane;
    const T* kbase = (const T*)p.k + b * p.kv_stride[0] + kvh * p.kv_stride[1];
    const int64_t pitch = DS > 0 ? D + 4 : D + 1;  // rows of 16-byte pieces when the head size is built in
    for (int64_t i = lane; i < CKV_WAVE * D; i += CKV_WAVE) {
        const int64_t r = i / D, d = i % D;
        const int64_t nn = c * CKV_WAVE + r;
        k_lds[r * pitch + d] = nn < N ? Elem<T>::to_float(kbase[nn * p.kv_stride[2] + d * p.kv_stride[3]]) : 0.f;
    }
    __syncthreads();
    bool live = n < N;
    if (live && n < Nc && p.kmasked) live = p.kmasked[n] == 0;
    const int64_t nrel = n - Nc;  // >= 0 for chunk keys
    // first query row that can see any key of this chunk of keys
    int64_t m0 = c * CKV_WAVE - Nc;
    if (m0 < 0) m0 = 0;
    const T* qbase = (const T*)p.q + b * p.q_stride[0] + h * p.q_stride[1];
    const float* lse = p.lse + (b * p.H + h) * Q;
    float acc = 0.f;
    // what one visible (row, key) pair adds, rows in ascending order
    auto add_row = [&](int64_t m, float s) {
        const bool vis = live && (n < Nc || nrel <= m);
        if (vis) {
            // the eager path holds P in the tensor dtype (softmax output) before weighting it;
            // chunk-key products are rounded to the dtype as well (cascade_attention.py:319-323)
            const float pt = round_t<T>(expf(s * p.scale - lse[m]));
            if (n >= Nc && p.new_mode) {
                acc = __fadd_rn(acc, round_t<T>(__fmul_rn(pt, p.w_new[m - nrel])));
            } else {
                acc = fmaf(p.w_ema[m], pt, acc);
            }
        }
    };
    if constexpr (DS > 0) {
        // Query rows pass through LDS in tiles of kColQTile; the logits of four rows are worked out together (four
        // independent chains over the head dims, each in ascending order; a piece of the lane's key row read from
        // LDS serves all four), then the rows are added in order.
        float* q_t = k_lds + CKV_WAVE * (DS + 4);   // [kColQTile][DS]
        const float* krow = k_lds + lane * (DS + 4);
        for (int64_t mt = m0; mt < Q; mt += kColQTile) {
            __syncthreads();  // the tile before is no longer read
#pragma unroll 8
            for (int i = lane; i < kColQTile * DS; i += CKV_WAVE) {
                const int r = i / DS, d = i % DS;
                q_t[i] = mt + r < Q ? Elem<T>::to_float(qbase[(mt + r) * p.q_stride[2] + d * p.q_stride[3]]) : 0.f;
            }
            __syncthreads();
            const int rows_here = Q - mt < kColQTile ? (int)(Q - mt) : kColQTile;
            for (int mi = 0; mi < rows_here; mi += 4) {
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
                for (int d = 0; d < DS; d += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(krow + d);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float4 q4 = *reinterpret_cast<const float4*>(q_t + (mi + i) * DS + d);
                        s4[i] = fmaf(q4.x, k4.x, s4[i]);
                        s4[i] = fmaf(q4.y, k4.y, s4[i]);
                        s4[i] = fmaf(q4.z, k4.z, s4[i]);
                        s4[i] = fmaf(q4.w, k4.w, s4[i]);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (mi + i < rows_here) add_row(mt + mi + i, s4[i]);
            }
        }
    } else {
        for (int64_t m = m0; m < Q; m++) {
            const T* qr = qbase + m * p.q_stride[2];
            float s = 0.f;
            for (int64_t d = 0; d < D; d++) s = fmaf(Elem<T>::to_float(qr[d * p.q_stride[3]]), k_lds[lane * pitch + d], s);
            add_row(m, s);
        }
    }
    if (n < N) p.colsum[(b * p.H + h) * N + n] = acc;
}

// ---------------------------------------------------------------------------------------------
// epilogue: per-head sums -> dtype -> head reduction -> EMA / new-token scores
// (cascade_attention.py:231-248, 319-330)
// ---------------------------------------------------------------------------------------------
template <typename T>
__device__ inline float reduce_heads(const float* colsum, int64_t b, int64_t h0, int64_t nh, int64_t H, int64_t N,
                                     int64_t n, int mode) {
    const float* base = colsum + (b * H + h0) * N + n;
    if (mode == CKV_REDUCE_MAX) {
        float r = round_t<T>(base[0]);
        for (int64_t g = 1; g < nh; g++) r = fmaxf(r, round_t<T>(base[g * N]));
        return r;
    }
    if (mode == CKV_REDUCE_MEAN) {
        float r = 0.f;
        for (int64_t g = 0; g < nh; g++) r = __fadd_rn(r, round_t<T>(base[g * N]));
        return round_t<T>(r / (float)nh);
    }
    float vals[128];  // lower median (torch.median): element (nh-1)/2 of the sorted values
    for (int64_t g = 0; g < nh; g++) {
        const float x = round_t<T>(base[g * N]);
        int64_t i = g;
        while (i > 0 && vals[i - 1] > x) {
            vals[i] = vals[i - 1];
            i--;
        }
        vals[i] = x;
    }
    return vals[(nh - 1) / 2];
}

template <typename T>
__global__ void finish_kernel(FinishProblem p) {
    const int64_t per = p.S + p.Q;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= p.B * p.KVH * per) return;
    const int64_t i = idx % per;
    const int64_t kvh = (idx / per) % p.KVH;
    const int64_t b = idx / (per * p.KVH);
    const int64_t G = p.H / p.KVH;
    const int64_t h0 = p.homogeneous ? 0 : kvh * G;
    const int64_t nh = p.homogeneous ? p.H : G;
    if (i < p.S) {
        if (!p.cache_s) return;
        const float red = reduce_heads<T>(p.colsum, b, h0, nh, p.H, p.N, p.num_sink + i, p.head_reduction);
        T* cs = (T*)p.cache_s + b * p.cache_s_stride[0] + kvh * p.cache_s_stride[1] + i * p.cache_s_stride[2];
        const float decayed = round_t<T>(__fmul_rn(p.beta_pow_q, Elem<T>::to_float(*cs)));
        *cs = Elem<T>::from_float(__fadd_rn(decayed, red));
    } else {
        if (!p.new_scores) return;
        const int64_t m = i - p.S;
        const float red = reduce_heads<T>(p.colsum, b, h0, nh, p.H, p.N, p.num_sink + p.S + m, p.head_reduction);
        T* ns = (T*)p.new_scores + b * p.new_scores_stride[0] + kvh * p.new_scores_stride[1] +
                m * p.new_scores_stride[2];
        *ns = Elem<T>::from_float(red);
    }
}

template <typename T>
__global__ void cast_scores_kernel(const float* colsum, T* scores, int64_t s0, int64_t s1, int64_t s2, int64_t B,
                                   int64_t H, int64_t N) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * H * N) return;
    const int64_t n = idx % N, h = (idx / N) % H, b = idx / (N * H);
    scores[b * s0 + h * s1 + n * s2] = Elem<T>::from_float(colsum[idx]);
}

template <typename T, int DS>
int core_generic_d(const CoreProblem& p, hipStream_t stream) {
    const int64_t rows = p.B * p.H * p.Q;
    {
        const size_t lds_f = (size_t)CKV_WAVE * (2 * p.D + 4) * sizeof(float);
        constexpr int kRowsPerWave = 4;
        if constexpr (DS > 0) {
            if (p.Q % (4 * kRowsPerWave) == 0) {
                const void* fn = reinterpret_cast<const void*>(fwd_generic_rows_kernel<T, DS, kRowsPerWave>);
                if (int rc = ensure_dynamic_lds(fn, (int)lds_f)) return rc;
                StageScope sc(CKV_STAGE_FWD, stream);
                hipLaunchKernelGGL((fwd_generic_rows_kernel<T, DS, kRowsPerWave>), dim3((unsigned)(rows / (4 * kRowsPerWave))),
                                   dim3(256), lds_f, stream, p);
                CKV_HIP_TRY(hipGetLastError());
                goto scores;
            }
        }
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fwd_generic_kernel<T, DS>), (int)lds_f)) return rc;
        StageScope sc(CKV_STAGE_FWD, stream);
        hipLaunchKernelGGL((fwd_generic_kernel<T, DS>), dim3((unsigned)((rows + 3) / 4)), dim3(256), lds_f, stream, p);
    }
scores:
    CKV_HIP_TRY(hipGetLastError());
    if (p.colsum) {
        const int64_t chunks = (p.N + CKV_WAVE - 1) / CKV_WAVE;
        // K tile (padded to a multiple of 16 bytes so that the query tile behind it is aligned), then the query tile
        const size_t lds = DS > 0 ? ((size_t)CKV_WAVE * (DS + 4) + (size_t)kColQTile * DS) * sizeof(float)
                                  : (size_t)CKV_WAVE * (p.D + 1) * sizeof(float);
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(colsum_generic_kernel<T, DS>), (int)lds)) return rc;
        {
            StageScope sc(CKV_STAGE_SCORES, stream);
            hipLaunchKernelGGL((colsum_generic_kernel<T, DS>), dim3((unsigned)(p.B * p.H * chunks)), dim3(CKV_WAVE), lds,
                               stream, p);
        }
        CKV_HIP_TRY(hipGetLastError());
    }
    return CKV_OK;
}

// the two head sizes models use get kernels with the size built in; every other size the general ones
template <typename T>
int core_generic_t(const CoreProblem& p, hipStream_t stream) {
    if (p.D == 128) return core_generic_d<T, 128>(p, stream);
    if (p.D == 64) return core_generic_d<T, 64>(p, stream);
    return core_generic_d<T, 0>(p, stream);
}

}  // namespace

int launch_core_generic(const CoreProblem& p, hipStream_t stream) {
    if (p.D > kMaxD) return CKV_ERR_UNSUPPORTED;
    switch (p.dtype) {
        case CKV_F32: return core_generic_t<float>(p, stream);
        case CKV_F16: return core_generic_t<__half>(p, stream);
        case CKV_BF16: return core_generic_t<__hip_bfloat16>(p, stream);
        default: return CKV_ERR_DTYPE;
    }
}

int launch_cast_scores(const float* colsum, void* scores, const int64_t* stride, int64_t B, int64_t H, int64_t N,
                       int dtype, hipStream_t stream) {
    const dim3 grid((unsigned)((B * H * N + 255) / 256)), block(256);
    switch (dtype) {
        case CKV_F32:
            hipLaunchKernelGGL(cast_scores_kernel<float>, grid, block, 0, stream, colsum, (float*)scores, stride[0],
                               stride[1], stride[2], B, H, N);
            break;
        case CKV_F16:
            hipLaunchKernelGGL(cast_scores_kernel<__half>, grid, block, 0, stream, colsum, (__half*)scores, stride[0],
                               stride[1], stride[2], B, H, N);
            break;
        case CKV_BF16:
            hipLaunchKernelGGL(cast_scores_kernel<__hip_bfloat16>, grid, block, 0, stream, colsum,
                               (__hip_bfloat16*)scores, stride[0], stride[1], stride[2], B, H, N);
            break;
        default: return CKV_ERR_DTYPE;
    }
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

int launch_weights(float* w_ema, float* w_new, int64_t Q, double beta, int dtype, hipStream_t stream) {
    const dim3 grid((unsigned)((Q + kColSlack + 255) / 256)), block(256);
    switch (dtype) {
        case CKV_F32: hipLaunchKernelGGL(weights_kernel<float>, grid, block, 0, stream, w_ema, w_new, Q, beta); break;
        case CKV_F16: hipLaunchKernelGGL(weights_kernel<__half>, grid, block, 0, stream, w_ema, w_new, Q, beta); break;
        case CKV_BF16:
            hipLaunchKernelGGL(weights_kernel<__hip_bfloat16>, grid, block, 0, stream, w_ema, w_new, Q, beta);
            break;
        default: return CKV_ERR_DTYPE;
    }
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

int launch_prep_generic(const PrepProblem& p, hipStream_t stream) {
    StageScope sc(CKV_STAGE_PREP, stream);
    const ckv_attn_args& a = *p.a;
    const int64_t half = a.D / 2;
    const int64_t N = a.num_sink + a.S + a.Q;
    int64_t items = a.B * a.KVH * N * half;
    const int64_t qitems = a.B * a.H * a.Q * half;
    if (qitems > items) items = qitems;
    if (a.num_sink + a.S > items) items = a.num_sink + a.S;
    const dim3 grid((unsigned)((items + 255) / 256)), block(256);
    const float post = sqrtf(a.scale);  // on queries and keys: the caller's core kernel multiplies by nothing more
    switch (a.dtype) {
        case CKV_F32:
            hipLaunchKernelGGL(prep_generic_kernel<float>, grid, block, 0, stream, a, (float*)p.qr, (float*)p.kr,
                               (float*)p.vc, p.kmasked, post);
            break;
        case CKV_F16:
            hipLaunchKernelGGL(prep_generic_kernel<__half>, grid, block, 0, stream, a, (__half*)p.qr, (__half*)p.kr,
                               (__half*)p.vc, p.kmasked, post);
            break;
        case CKV_BF16:
            hipLaunchKernelGGL(prep_generic_kernel<__hip_bfloat16>, grid, block, 0, stream, a,
                               (__hip_bfloat16*)p.qr, (__hip_bfloat16*)p.kr, (__hip_bfloat16*)p.vc, p.kmasked, post);
            break;
        default: return CKV_ERR_DTYPE;
    }
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

int launch_finish(const FinishProblem& p, hipStream_t stream) {
    StageScope sc(CKV_STAGE_FINISH, stream);
    const int64_t items = p.B * p.KVH * (p.S + p.Q);
    const dim3 grid((unsigned)((items + 255) / 256)), block(256);
    switch (p.dtype) {
        case CKV_F32: hipLaunchKernelGGL(finish_kernel<float>, grid, block, 0, stream, p); break;
        case CKV_F16: hipLaunchKernelGGL(finish_kernel<__half>, grid, block, 0, stream, p); break;
        case CKV_BF16: hipLaunchKernelGGL(finish_kernel<__hip_bfloat16>, grid, block, 0, stream, p); break;
        default: return CKV_ERR_DTYPE;
    }
    CKV_HIP_TRY(hipGetLastError());
    return CKV_OK;
}

}  // namespace ckv
