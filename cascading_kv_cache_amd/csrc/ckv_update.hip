// ckv_update: the cascading cache update as a plan + apply pair of gfx950 kernels.
//
// Replaces the serial per-token Triton program of the reference
// (cascade/models/cascading_cache.py:145-299 token loop, 302-774 body) with
//
//   plan   one workgroup per (batch, kv-head).  Walks the cascades in order; at every cascade
//          the arrivals of the whole call are classified (insert / challenger), numbered with a
//          ballot prefix sum, the challengers of each group are reduced to the group's winner
//          ("later wins iff score >=", cascading_cache.py:699), and the tokens the cascade evicts
//          become the arrival list of the next cascade.  Everything lives in LDS.  The result is
//          a forest of disjoint move chains in global memory:
//              first[t]   = slot the incoming token t finally lands in (-1: dropped)
//              next_of[d] = slot the OLD content of slot d finally lands in (-1: dropped)
//          plus the updated trackers.
//   apply  one lane group per incoming token.  Follows the chain of its token from the head,
//          carrying a whole row (K, V, score, original index) in registers with 16-byte lanes:
//          read the displaced row, write the carried one, move on.  Chains are vertex-disjoint
//          and only ever move towards higher cascades, so groups never touch each other's slots.
//          The same launch writes the position ids in closed form from the updated trackers
//          (cascading_cache.py:112-142, 728-774) with extra blocks at the end of its grid.
//
// Why this equals the serial loop: within one cascade the n-th insert of a call always lands in
// ring position (start + stored + n) mod W whatever the scores are; only WHICH arrival owns a
// slot depends on scores, and that is decided inside the group of arrivals between two inserts.
#include "ckv_common.h"

#include <mutex>

namespace ckv {
namespace {

constexpr int kMaxCascades = 64;
constexpr int kPlanMaxTokens = 8192;   // incoming tokens one plan launch takes at most
constexpr int kRingPer = 8;            // kPlanMaxTokens / 1024 threads, and enough for 256 tokens on 256 threads

struct UpdateParams {
    ckv_update_args a;
    int64_t token_offset;  // first incoming token handled by this launch
    int32_t k_sub;         // tokens handled by this launch
    int32_t do_pos;        // run the position pass (last launch of a call only)
    int32_t* first;        // [N*H][K]
    int32_t* next_of;      // [N*H][S]
    int32_t* pos_flag;     // [N*H]: the call put a token into the cascades, so the position ids change
    int32_t* mode;         // [N*H]: 1 = planned by the steady-state kernel: the new ring starts wait in start_new
    int32_t* start_new;    // [N*H][cascades]: ring starts after the call, committed by the apply kernel
    int32_t apply_blocks;  // blocks along x that move rows; the blocks behind them write position ids
};

// exclusive prefix sum of one flag per thread over the whole workgroup; returns the block total
__device__ inline int block_flag_scan(bool flag, int* wave_tot, int& exclusive) {
    const unsigned long long bal = __ballot(flag);
    const int lane = threadIdx.x & (CKV_WAVE - 1);
    const int wave = threadIdx.x / CKV_WAVE;
    const int nwaves = (blockDim.x + CKV_WAVE - 1) / CKV_WAVE;
    const int in_wave = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_tot[wave] = __popcll(bal);
    __syncthreads();
    int before = 0, total = 0;
    for (int w = 0; w < nwaves; w++) {
        const int c = wave_tot[w];
        if (w < wave) before += c;
        total += c;
    }
    __syncthreads();  // wave_tot is reused by the next call
    exclusive = before + in_wave;
    return total;
}

__device__ inline void emit_move(int32_t* first, int32_t* next_of, int dst, int src) {
    next_of[dst] = -1;
    if (src < 0) {
        first[-1 - src] = dst;
    } else {
        next_of[src] = dst;
    }
}

__global__ void ckv_update_plan_kernel(UpdateParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const ckv_update_args& A = p.a;
    const int tid = threadIdx.x, T = blockDim.x;
    const int64_t bh = blockIdx.x;
    if (p.mode[bh]) return;  // the steady-state kernel has planned this unit
    const int64_t n = bh / A.H, h = bh % A.H;
    const int cap = p.k_sub;
    const int C = A.cascades;
    const int64_t W = A.window_size, S = A.max_seq_len, NS = A.num_sink;

    int32_t* a_src[2];
    uint16_t* a_trig[2];   // index of the token whose arrival set the entry moving: below kPlanMaxTokens
    float* a_score[2];
    unsigned char* ptr = smem;
    // per cascade, fetched once up front so that no cascade waits for global memory on their account:
    // the acceptance period and the score of the newest slot left by earlier calls
    int64_t* per_l = reinterpret_cast<int64_t*>(ptr); ptr += 8 * kMaxCascades;
    float* lead_l = reinterpret_cast<float*>(ptr); ptr += 4 * kMaxCascades;
    for (int i = 0; i < 2; i++) {
        a_src[i] = reinterpret_cast<int32_t*>(ptr); ptr += 4 * (size_t)cap;
        a_score[i] = reinterpret_cast<float*>(ptr); ptr += 4 * (size_t)cap;
    }
    uint32_t* eflag = reinterpret_cast<uint32_t*>(ptr); ptr += 4 * (size_t)cap;
    float* ring_l = reinterpret_cast<float*>(ptr); ptr += 4 * (size_t)cap;  // scores of the oldest ring entries
    int32_t* w_src = reinterpret_cast<int32_t*>(ptr); ptr += 4 * (size_t)(cap + 1);
    float* w_score = reinterpret_cast<float*>(ptr); ptr += 4 * (size_t)(cap + 1);
    int32_t* st_l = reinterpret_cast<int32_t*>(ptr); ptr += 4 * kMaxCascades;
    int32_t* sx_l = reinterpret_cast<int32_t*>(ptr); ptr += 4 * kMaxCascades;
    int* wave_tot = reinterpret_cast<int*>(ptr); ptr += 64 * sizeof(int);
    for (int i = 0; i < 2; i++) {
        a_trig[i] = reinterpret_cast<uint16_t*>(ptr); ptr += 2 * (size_t)((cap + 1) & ~1);
    }

    int64_t* g_stored = A.stored_tokens + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    int64_t* g_start = A.start_indices + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    int64_t* g_sinks = A.stored_sinks + n * A.stored_sinks_stride[0] + h * A.stored_sinks_stride[1];
    const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int32_t* first = p.first + bh * A.K + p.token_offset;
    int32_t* next_of = p.next_of + bh * S;

    const int64_t seen = *A.real_token_idx + p.token_offset;  // tokens before token 0 of this launch
    const int64_t sinks0 = *g_sinks;
    int64_t room = NS - sinks0;
    if (room < 0) room = 0;
    const int n_sink_new = room < cap ? (int)room : cap;

    for (int i = tid; i < C; i += T) {
        const int32_t st = (int32_t)g_stored[i * A.tracker_stride[2]];
        const int32_t sx = (int32_t)g_start[i * A.tracker_stride[2]];
        st_l[i] = st;
        sx_l[i] = sx;
        per_l[i] = A.do_cache_every_n[i];
        // the plan never writes scores, so the newest slot's score can be read before its cascade's turn
        lead_l[i] = st > 0 ? load_as_float(A.cache_s, cs_base + ((int64_t)i * W + (sx - 1 + st) % st) * A.cache_s_stride[2],
                                           A.dtype)
                           : 0.f;
    }
    // level-0 arrivals: the non-sink tokens of this launch, in order (cascading_cache.py:447-462)
    for (int t = tid; t < cap; t += T) {
        if (t < n_sink_new) {
            first[t] = (int32_t)(S + sinks0 + t);
        } else {
            first[t] = -1;
            const int a = t - n_sink_new;
            a_src[0][a] = -1 - t;
            a_trig[0][a] = (uint16_t)t;
            a_score[0][a] = load_as_float(
                A.s, n * A.s_stride[0] + h * A.s_stride[1] + (p.token_offset + t) * A.s_stride[2], A.dtype);
        }
    }
    __syncthreads();
    if (tid == 0 && n_sink_new > 0) *g_sinks = sinks0 + n_sink_new;

    // 64-bit division per arrival is what this kernel would spend its time on: token indices, periods
    // and the window fit 32 bits in every realistic call, and both divisors are usually powers of two
    const bool small = seen + cap + S + NS < (1ll << 31) && W < (1ll << 31);
    const bool w_pow2 = (W & (W - 1)) == 0;
    auto mod_w = [&](int64_t x) -> int {  // x >= 0
        if (w_pow2) return (int)(x & (W - 1));
        if (small) return (int)((uint32_t)x % (uint32_t)W);
        return (int)(x % W);
    };

    int nA = cap - n_sink_new;
    int cur = 0;
    for (int i = 0; i < C && nA > 0; i++) {
        const int64_t l = (int64_t)i * W;
        const int stored0 = st_l[i], start0 = sx_l[i];
        const int64_t per = per_l[i];
        const bool per_small = small && per > 0 && per < (1ll << 31);
        const bool per_pow2 = per > 0 && (per & (per - 1)) == 0;
        const int32_t* Asrc = a_src[cur];
        const uint16_t* Atrig = a_trig[cur];
        const float* Ascore = a_score[cur];

        // Scores of the ring entries this call can evict (the oldest ones, at most one per arrival beyond
        // the free room): requested here, parked in LDS after pass 2, read in pass 3, so their way from
        // memory runs beside passes 1 and 2.
        int n_ring = stored0 + nA - (int)W;
        if (n_ring > stored0 - 1) n_ring = stored0 - 1;
        if (i + 1 >= C) n_ring = 0;
        float ring_pre[kRingPer];
#pragma unroll
        for (int r = 0; r < kRingPer; r++) {
            const int j = r * T + tid;
            ring_pre[r] = j < n_ring ? load_as_float(A.cache_s, cs_base + (l + mod_w(start0 + (int64_t)j)) * A.cache_s_stride[2],
                                                     A.dtype)
                                     : 0.f;
        }

        // ---- pass 1: insert flags (accept, or the first arrival of an empty cascade:
        //      cascading_cache.py:471-478, 606) and their running index
        int E = 0;
        for (int base = 0; base < nA; base += T) {
            const int a = base + tid;
            bool f = false;
            if (a < nA) {
                const int64_t gidx = seen + Atrig[a];  // 0-based global index of the triggering token
                const int64_t rel = gidx - NS;  // >= 0: sink tokens never arrive here
                const bool on_period = per_pow2 ? (rel & (per - 1)) == 0
                                                : (per_small ? ((uint32_t)rel % (uint32_t)per) == 0 : (rel % per) == 0);
                const bool acc = (A.eager_fill && gidx <= S + NS) || on_period;
                f = acc || (stored0 == 0 && a == 0);
            }
            int ex;
            const int tot = block_flag_scan(f, wave_tot, ex);
            if (a < nA) eflag[a] = (uint32_t)(E + ex) | (f ? 0x80000000u : 0u);
            E += tot;
        }
        __syncthreads();

        // ---- pass 2: the winner of every group.  Slot 0 of w_* is the newest slot left by
        //      earlier calls (cascading_cache.py:676-680), slot e+1 belongs to insert e.
        const int p_lead = (int)l + (stored0 > 0 ? (start0 - 1 + stored0) % stored0 : 0);
        if (tid == 0 && stored0 > 0) {
            int ws = p_lead;
            float wv = lead_l[i];
            for (int b = 0; b < nA && !(eflag[b] & 0x80000000u); b++) {
                if (Ascore[b] >= wv) { ws = Asrc[b]; wv = Ascore[b]; }
            }
            w_src[0] = ws;
            w_score[0] = wv;
        }
        for (int a = tid; a < nA; a += T) {
            const uint32_t ef = eflag[a];
            if (!(ef & 0x80000000u)) continue;
            int ws = Asrc[a];
            float wv = Ascore[a];
            for (int b = a + 1; b < nA && !(eflag[b] & 0x80000000u); b++) {
                if (Ascore[b] >= wv) { ws = Asrc[b]; wv = Ascore[b]; }
            }
            const int e = (int)(ef & 0x7fffffffu);
            w_src[e + 1] = ws;
            w_score[e + 1] = wv;
        }
#pragma unroll
        for (int r = 0; r < kRingPer; r++) {
            const int j = r * T + tid;
            if (j < n_ring) ring_l[j] = ring_pre[r];
        }
        __syncthreads();

        // ---- pass 3: evictions feed the next cascade; surviving slots become moves
        const int room_i = (int)W - stored0;          // inserts that still append
        const bool has_next = (i + 1 < C);
        int32_t* Bsrc = a_src[cur ^ 1];
        uint16_t* Btrig = a_trig[cur ^ 1];
        float* Bscore = a_score[cur ^ 1];
        for (int a = tid; a < nA; a += T) {
            const uint32_t ef = eflag[a];
            if (!(ef & 0x80000000u)) continue;
            const int e = (int)(ef & 0x7fffffffu);
            if (e >= room_i && has_next) {  // full: the oldest entry leaves (cascading_cache.py:542-604)
                const int mv = e - room_i;  // index of the evicted entry in [old ring | inserts]
                int ns;
                float nv;
                if (mv < stored0 - 1) {     // an old ring entry nobody touched in this call
                    ns = (int)l + mod_w(start0 + (int64_t)mv);
                    nv = ring_l[mv];
                } else {
                    ns = w_src[mv - stored0 + 1];
                    nv = w_score[mv - stored0 + 1];
                }
                Bsrc[mv] = ns;
                Bscore[mv] = nv;
                Btrig[mv] = Atrig[a];
            }
            if (e >= E - (int)W) {  // not evicted again before the call ends
                const int phys = (int)l + mod_w((int64_t)start0 + stored0 + e);
                emit_move(first, next_of, phys, w_src[e + 1]);
            }
        }
        if (tid == 0 && stored0 > 0 && E <= (int)W - 1 && w_src[0] != p_lead) {
            emit_move(first, next_of, p_lead, w_src[0]);
        }
        const int n_ev = (stored0 + E > (int)W) ? stored0 + E - (int)W : 0;
        __syncthreads();
        if (tid == 0) {
            const int st_new = stored0 + E < (int)W ? stored0 + E : (int)W;
            const int sx_new = mod_w((int64_t)start0 + n_ev);
            st_l[i] = st_new;
            sx_l[i] = sx_new;
            g_stored[i * A.tracker_stride[2]] = st_new;
            g_start[i * A.tracker_stride[2]] = sx_new;
        }
        nA = has_next ? n_ev : 0;
        cur ^= 1;
    }
    __syncthreads();

    // the position ids change only when the last token of the call went to the cascades
    if (p.do_pos && tid == 0) p.pos_flag[bh] = cap > n_sink_new ? 1 : 0;
}

// Steady-state plan: every cascade of the unit is full, no token of the call is accepted by the eager-fill rule,
// and every acceptance period divides the next one (the power schedules).  Then which arrivals a cascade sees,
// which of them are inserted and where, is a closed form of the token counter: the arrivals of cascade i are
// the tokens whose index is a multiple of period i-1, every (period i / period i-1)-th of them is inserted,
// the n-th insert lands n slots behind the ring start and pushes the n-th oldest entry on to cascade i+1.
// As long as a cascade evicts only entries the call has not touched, its arrivals can be read straight from
// the cache as it was before the call, so every cascade is planned by workgroups of its own, side by side:
// one thread per insert folds the arrivals up to the next insert into the group's winner ("later wins iff
// score >=", cascading_cache.py:699) and writes where every member of the group ends up.  Every chain entry
// has one writer: the workgroups of cascade i own the pointers of cascade i's arrivals.  The ring starts after
// the call go to scratch (the neighbours still read the old ones); the apply kernel commits them.
// A unit that does not meet the conditions is left to the general kernel (mode 0).
constexpr int kSteadyParts = 4;   // workgroups per cascade and unit
constexpr int kSteadyThreads = 256;

struct SteadyCascade {
    int64_t per_prev, r;   // period of the cascade before, inserts every r-th arrival
    int64_t a0;            // first token of the call that arrives at this cascade
    int32_t nA, kf, E;     // arrivals, index of the first inserted arrival, inserts
    int32_t sx;            // ring start before the call
};

__global__ void __launch_bounds__(kSteadyThreads) ckv_update_plan_steady_kernel(UpdateParams p) {
    __shared__ SteadyCascade sc[kMaxCascades];
    __shared__ int64_t st_s[kMaxCascades], sx_s[kMaxCascades], per_s[kMaxCascades], seen_s, sinks_s;
    __shared__ int fast_s;
    const ckv_update_args& A = p.a;
    const int tid = threadIdx.x;
    const int64_t bh = blockIdx.y;
    const int i = blockIdx.x / kSteadyParts, part = blockIdx.x % kSteadyParts;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int C = A.cascades;
    const int64_t W = A.window_size, S = A.max_seq_len, NS = A.num_sink;
    const int cap = (int)A.K;  // the whole call is planned at once
    const int64_t* g_stored = A.stored_tokens + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    const int64_t* g_start = A.start_indices + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    // the trackers of all cascades travel together; one thread then works out the closed forms
    if (tid < C) {
        st_s[tid] = g_stored[tid * A.tracker_stride[2]];
        sx_s[tid] = g_start[tid * A.tracker_stride[2]];
        per_s[tid] = A.do_cache_every_n[tid];
    } else if (tid == kMaxCascades) {
        seen_s = *A.real_token_idx;
    } else if (tid == kMaxCascades + 1) {
        sinks_s = A.stored_sinks[n * A.stored_sinks_stride[0] + h * A.stored_sinks_stride[1]];
    }
    __syncthreads();
    // one thread per cascade works out that cascade's closed forms (they depend on the token counter and the
    // periods only); 32-bit division when everything fits, which it does outside pathological streams
    __shared__ int ok_s[kMaxCascades];
    if (tid < C) {
        const int j = tid;
        const int64_t seen = seen_s, sinks0 = sinks_s;
        const int64_t rel0 = seen - NS;
        const int64_t per = per_s[j], per_prev = j == 0 ? 1 : per_s[j - 1];
        const int64_t st = st_s[j], sx = sx_s[j];
        bool ok = sinks0 >= NS && rel0 >= 0 && !(A.eager_fill && seen <= S + NS) && W >= 2 && W < (1ll << 30) &&
                  cap < (1 << 30) && per > 0 && per_prev > 0 && st == W && sx >= 0 && sx < W;
        SteadyCascade c;
        c.per_prev = per_prev;
        c.r = 1;
        c.nA = c.kf = c.E = 0;
        c.sx = (int32_t)sx;
        c.a0 = 0;
        if (ok) {
            const bool small = rel0 < (1ll << 31) && per < (1ll << 31);
            auto mod = [&](int64_t x, int64_t y) -> int64_t { return small ? (int64_t)((uint32_t)x % (uint32_t)y) : x % y; };
            auto div = [&](int64_t x, int64_t y) -> int64_t { return small ? (int64_t)((uint32_t)x / (uint32_t)y) : x / y; };
            ok = mod(per, per_prev) == 0;
            if (ok) {
                c.r = div(per, per_prev);
                const int64_t a0 = mod(per_prev - mod(rel0, per_prev), per_prev);   // first token that arrives here
                c.a0 = a0;
                c.nA = a0 < cap ? (int32_t)div(cap - a0 + per_prev - 1, per_prev) : 0;
                const int64_t q0 = div(rel0 + a0, per_prev);                       // arrival k is inserted iff (q0 + k) % r == 0
                c.kf = (int32_t)mod(c.r - mod(q0, c.r), c.r);
                c.E = c.nA > c.kf ? (int32_t)div((int64_t)c.nA - c.kf + c.r - 1, c.r) : 0;
                // what the cascade evicts must be entries the call has not touched: at most all but the newest
                // old entry; or all of them when no arrival challenges that entry before the first insert; cascade
                // 0 with period 1 has no challengers at all, and what it evicts beyond its old entries are the
                // call's own tokens in order
                const bool untouched = c.E <= W - 1 || (c.E <= W && c.kf == 0) || (j == 0 && per == 1);
                ok = j + 1 < C ? untouched : (c.E <= W || (j == 0 && per == 1));
            }
        }
        sc[j] = c;
        ok_s[j] = ok ? 1 : 0;
    }
    __syncthreads();
    if (tid == 0) {
        bool ok = true;
        for (int j = 0; j < C; j++) {
            ok = ok && ok_s[j];
            if (j >= 1 && sc[j - 1].E != sc[j].nA) ok = false;  // evictions of a full cascade = its inserts
        }
        fast_s = ok ? 1 : 0;
    }
    __syncthreads();
    const bool fast = fast_s != 0;
    if (blockIdx.x == 0 && tid == 0) {
        p.mode[bh] = fast ? 1 : 0;
        if (fast) p.pos_flag[bh] = 1;
    }
    if (!fast) return;
    const SteadyCascade c = sc[i];
    const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int32_t* first = p.first + bh * A.K;
    int32_t* next_of = p.next_of + bh * S;
    const int l = (int)((int64_t)i * W);
    const int Wi = (int)W;
    const bool prev_passes_tokens = i == 1 && sc[0].per_prev == 1 && sc[0].r == 1;  // cascade 0 has period 1
    const int sx_prev = i >= 1 ? sc[i - 1].sx : 0;
    // arrival k of this cascade: where it comes from (-1 - token, or the slot of the cascade before) and its score
    auto arrival = [&](int k, int& src, float& score) {
        if (i == 0) {
            const int64_t t = c.a0 + (int64_t)k * c.per_prev;
            src = -1 - (int)t;
            score = load_as_float(A.s, n * A.s_stride[0] + h * A.s_stride[1] + t * A.s_stride[2], A.dtype);
        } else if (prev_passes_tokens && k >= Wi) {
            const int t = k - Wi;  // evicted by cascade 0 after it had been placed there in this call
            src = -1 - t;
            score = load_as_float(A.s, n * A.s_stride[0] + h * A.s_stride[1] + (int64_t)t * A.s_stride[2], A.dtype);
        } else {
            int ring = sx_prev + k;
            if (ring >= Wi) ring -= Wi;
            src = l - Wi + ring;
            score = load_as_float(A.cache_s, cs_base + (int64_t)src * A.cache_s_stride[2], A.dtype);
        }
    };
    auto point = [&](int src, int dst) {  // the arrival that came from `src` ends up in slot dst (-1: nowhere)
        if (src < 0) first[-1 - src] = dst;
        else next_of[src] = dst;
    };
    if (part == 0 && tid == 0) {
        int sx_new = c.sx + (int)(c.E % Wi);
        if (sx_new >= Wi) sx_new -= Wi;
        p.start_new[bh * C + i] = sx_new;
        // arrivals before the first insert challenge the newest entry earlier calls left
        const int lead_n = c.kf < c.nA ? c.kf : c.nA;
        if (lead_n > 0) {
            const int p_lead = l + (c.sx == 0 ? Wi - 1 : c.sx - 1);
            int ws = p_lead;
            float wv = load_as_float(A.cache_s, cs_base + (int64_t)p_lead * A.cache_s_stride[2], A.dtype);
            bool held = true;  // the old entry still holds the slot
            for (int k = 0; k < lead_n; k++) {
                int src;
                float score;
                arrival(k, src, score);
                if (score >= wv) {
                    if (!held) point(ws, -1);
                    held = false;
                    ws = src;
                    wv = score;
                } else {
                    point(src, -1);
                }
            }
            // with W inserts in the call the slot is taken again by the last of them (only behind the last
            // cascade: elsewhere such a call is left to the general kernel), and the group's winner is dropped
            const bool survives = c.E <= Wi - 1;
            if (!held) {
                if (survives) {
                    point(ws, p_lead);
                    next_of[p_lead] = -1;  // the old entry is dropped
                } else {
                    point(ws, -1);
                }
            }
        }
    }
    const int drop_before = c.E > Wi ? c.E - Wi : 0;  // inserts whose slot is taken again later in the call
    for (int g = part * kSteadyThreads + tid; g < c.E; g += kSteadyParts * kSteadyThreads) {
        const int k0 = c.kf + (int)((int64_t)g * c.r);
        int k1 = k0 + (int)c.r;
        if (k1 > c.nA) k1 = c.nA;
        if (g < drop_before) {
            // placed and pushed out again within the call: cascade 1 owns the pointer (it sees the token as an
            // arrival of its own); behind the last cascade the members are dropped
            if (i + 1 >= C) {
                for (int k = k0; k < k1; k++) {
                    int src;
                    float score;
                    arrival(k, src, score);
                    point(src, -1);
                }
            }
            continue;
        }
        int ring = c.sx + (g % Wi);
        if (ring >= Wi) ring -= Wi;
        const int phys = l + ring;
        int ws;
        float wv;
        arrival(k0, ws, wv);
        for (int k = k0 + 1; k < k1; k++) {
            int src;
            float score;
            arrival(k, src, score);
            if (score >= wv) {
                point(ws, -1);
                ws = src;
                wv = score;
            } else {
                point(src, -1);
            }
        }
        point(ws, phys);
        if (i + 1 >= C) next_of[phys] = -1;  // what the last cascade evicts is dropped
    }
}

// The plan of a single incoming token (the decode step): one wavefront per (batch, kv head), no workgroup
// barriers.  Lane i fetches what cascade i may need (trackers, period, the scores of its oldest and its newest
// slot) so that all cascades' loads travel together; the walk over the cascades then runs on values handed
// round by shuffles, identical in every lane, and lane 0 writes the chain.  Same semantics as the general
// kernel (cascading_cache.py:381-726 for one token).
__global__ void __launch_bounds__(CKV_WAVE) ckv_update_plan1_kernel(UpdateParams p) {
    const ckv_update_args& A = p.a;
    const int lane = threadIdx.x;
    const int64_t bh = blockIdx.x;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int C = A.cascades;
    const int64_t W = A.window_size, S = A.max_seq_len, NS = A.num_sink;
    int64_t* g_stored = A.stored_tokens + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    int64_t* g_start = A.start_indices + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    int64_t* g_sinks = A.stored_sinks + n * A.stored_sinks_stride[0] + h * A.stored_sinks_stride[1];
    const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int32_t* first = p.first + bh * A.K + p.token_offset;
    int32_t* next_of = p.next_of + bh * S;

    const int64_t gidx = *A.real_token_idx + p.token_offset;  // 0-based global index of the token
    const int64_t sinks0 = *g_sinks;
    const float tok_score = load_as_float(A.s, n * A.s_stride[0] + h * A.s_stride[1] + p.token_offset * A.s_stride[2], A.dtype);
    // lane i: cascade i
    int32_t st = 0, sx = 0;
    int64_t per = 1;
    float oldest = 0.f, newest = 0.f;
    if (lane < C) {
        st = (int32_t)g_stored[lane * A.tracker_stride[2]];
        sx = (int32_t)g_start[lane * A.tracker_stride[2]];
        per = A.do_cache_every_n[lane];
        const int64_t l = (int64_t)lane * W;
        if (st > 0) {
            oldest = load_as_float(A.cache_s, cs_base + (l + sx) * A.cache_s_stride[2], A.dtype);
            newest = load_as_float(A.cache_s, cs_base + (l + (sx - 1 + st) % st) * A.cache_s_stride[2], A.dtype);
        }
    }
    if (lane == 0) p.mode[bh] = 0;  // the trackers are written here, not left in scratch
    if (sinks0 < NS) {  // the token is a sink (cascading_cache.py:399-431): no position pass
        if (lane == 0) {
            first[0] = (int32_t)(S + sinks0);
            *g_sinks = sinks0 + 1;
            if (p.do_pos) p.pos_flag[bh] = 0;
        }
        return;
    }
    int carry_src = -1;          // -1 - token index, or the slot whose old content is carried
    float carry_score = tok_score;
    int32_t first_val = -1;      // where the token lands (-1: dropped)
    const int64_t rel = gidx - NS;
    const bool eager = A.eager_fill && gidx <= S + NS;
    for (int i = 0; i < C; i++) {
        const int32_t st_i = __shfl(st, i), sx_i = __shfl(sx, i);
        const int64_t per_i = __shfl(per, i);
        const int l = (int)((int64_t)i * W);
        const bool acc = eager || (rel % per_i) == 0;
        if (acc || st_i == 0) {
            const int phys = l + (int)(((int64_t)sx_i + st_i) % W);
            if (st_i < (int32_t)W) {  // append (or the first entry of an empty cascade)
                if (lane == 0) {
                    next_of[phys] = -1;
                    if (carry_src < 0) first_val = phys; else next_of[carry_src] = phys;
                    g_stored[i * A.tracker_stride[2]] = st_i + 1;
                }
                break;
            }
            // full: the oldest entry (at the ring start) leaves for the next cascade, or is dropped
            if (lane == 0) {
                next_of[phys] = -1;
                if (carry_src < 0) first_val = phys; else next_of[carry_src] = phys;
                g_start[i * A.tracker_stride[2]] = (int64_t)((sx_i + 1) % (int32_t)W);
            }
            carry_src = phys;
            carry_score = __shfl(oldest, i);
            continue;
        }
        // not accepted: the newest slot keeps its token unless the arrival's score is at least as large
        if (carry_score >= __shfl(newest, i)) {
            const int p_lead = l + (sx_i - 1 + st_i) % st_i;
            if (lane == 0) {
                next_of[p_lead] = -1;
                if (carry_src < 0) first_val = p_lead; else next_of[carry_src] = p_lead;
            }
        }
        break;
    }
    if (lane == 0) {
        first[0] = first_val;
        if (p.do_pos) p.pos_flag[bh] = 1;
    }
}

// Position pass (cascading_cache.py:728-774, 129-142) after the plan kernel has updated the trackers:
// slot j of cascade i gets ((j + seg - start) mod seg) + ub - seg, where seg is the number of stored
// tokens and ub the ids still to hand out (all stored tokens, less a window per earlier cascade).
// One 256-thread block per kPosChunk slots of a cascade and (batch, kv head), so the whole chip writes; the
// blocks ride at the end of the apply kernels' grid (they need the plan's trackers, not the moved rows).
constexpr int kPosChunk = 2048;

__device__ inline void update_positions_block(const UpdateParams& p, int blk) {
    const ckv_update_args& A = p.a;
    const int64_t bh = blockIdx.y;
    if (!p.pos_flag[bh]) return;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int C = A.cascades;
    const int W = (int)A.window_size;
    const int per_c = (W + kPosChunk - 1) / kPosChunk;
    const int i = blk / per_c, j0 = (blk % per_c) * kPosChunk;
    const int64_t* g_stored = A.stored_tokens + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    const int64_t* g_start = A.start_indices + n * A.tracker_stride[0] + h * A.tracker_stride[1];
    // a unit planned by the steady-state kernel: every cascade is full, and the ring starts after the call are
    // still in scratch (this launch commits them, so the trackers themselves are not read here)
    const bool steady = p.mode[bh] != 0;
    int64_t ub = 0;
    for (int c = 0; c < C; c++) ub += steady ? (int64_t)W : g_stored[c * A.tracker_stride[2]];
    // cascade i is written only if every earlier one holds tokens and ids are left
    for (int c = 0; c < i; c++) {
        if (!steady && g_stored[c * A.tracker_stride[2]] <= 0) return;
        ub -= W;
        if (ub <= 0) return;
    }
    const int64_t st = steady ? (int64_t)W : g_stored[i * A.tracker_stride[2]];
    const uint32_t seg = (uint32_t)(st < W ? st : W);
    if (seg == 0) return;
    const uint32_t sx_now = steady ? (uint32_t)p.start_new[bh * C + i] : (uint32_t)g_start[i * A.tracker_stride[2]];
    const uint32_t add = seg - sx_now;  // start < seg or start == 0
    const int64_t base = ub - seg;
    auto id_of = [&](int j) -> int64_t {
        uint32_t x = (uint32_t)j + add;
        if (x >= seg) x -= seg;
        if (x >= seg) x %= seg;  // slots past the stored tokens of a cascade that is not full
        return (int64_t)x + base;
    };
    int64_t* pos = A.pos + n * A.pos_stride[0] + h * A.pos_stride[1] + (int64_t)i * W * A.pos_stride[2];
    const int tid = threadIdx.x;
    if (A.pos_stride[2] == 1 && (reinterpret_cast<uintptr_t>(pos) & 15u) == 0 && (W & 1) == 0) {
#pragma unroll
        for (int it = 0; it < kPosChunk / 512; it++) {
            const int j = j0 + it * 512 + 2 * tid;
            if (j < W) *reinterpret_cast<longlong2*>(pos + j) = make_longlong2(id_of(j), id_of(j + 1));
        }
    } else {
        for (int j = j0 + tid; j < j0 + kPosChunk && j < W; j += 256) pos[(int64_t)j * A.pos_stride[2]] = id_of(j);
    }
}

// One 16-byte piece of a row per lane.
struct RowPiece {
    uint4 k, v;
};

template <int LANES>
__global__ void ckv_update_apply_vec_kernel(UpdateParams p) {
    const ckv_update_args& A = p.a;
    constexpr int kGroups = 256 / LANES;
    if (blockIdx.x == 0 && p.do_pos && p.mode[blockIdx.y] && (int)threadIdx.x < A.cascades) {
        // commit the ring starts the steady-state plan left in scratch (nobody reads the trackers in this launch)
        const int64_t bh_c = blockIdx.y;
        A.start_indices[(bh_c / A.H) * A.tracker_stride[0] + (bh_c % A.H) * A.tracker_stride[1] +
                        threadIdx.x * A.tracker_stride[2]] = p.start_new[bh_c * A.cascades + threadIdx.x];
    }
    if ((int)blockIdx.x >= p.apply_blocks) {
        update_positions_block(p, (int)blockIdx.x - p.apply_blocks);
        return;
    }
    const int g = blockIdx.x * kGroups + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    if (g >= p.k_sub) return;
    const int64_t bh = blockIdx.y;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int64_t S = A.max_seq_len;
    const int32_t* first = p.first + bh * A.K + p.token_offset;
    const int32_t* next_of = p.next_of + bh * S;
    int d = first[g];
    if (d < 0) return;  // the token entered and left the cache inside this call

    const int es = (int)elem_bytes(A.dtype);
    const int chunks = (int)(A.HID * es / 16);
    const bool active = lane < chunks;
    const int64_t t_in = p.token_offset + g;

    const char* kin = reinterpret_cast<const char*>(A.k) +
                      (n * A.kv_stride[0] + h * A.kv_stride[1] + t_in * A.kv_stride[2]) * es;
    const char* vin = reinterpret_cast<const char*>(A.v) +
                      (n * A.kv_stride[0] + h * A.kv_stride[1] + t_in * A.kv_stride[2]) * es;
    RowPiece carry;
    carry.k = make_uint4(0, 0, 0, 0);
    carry.v = make_uint4(0, 0, 0, 0);
    if (active) {
        carry.k = reinterpret_cast<const uint4*>(kin)[lane];
        carry.v = reinterpret_cast<const uint4*>(vin)[lane];
    }

    if (d >= S) {  // sink slot (cascading_cache.py:61-109)
        const int64_t j = d - S;
        const int64_t so = (n * A.sink_stride[0] + h * A.sink_stride[1] + j * A.sink_stride[2]) * es;
        if (active) {
            reinterpret_cast<uint4*>(reinterpret_cast<char*>(A.sink_k) + so)[lane] = carry.k;
            reinterpret_cast<uint4*>(reinterpret_cast<char*>(A.sink_v) + so)[lane] = carry.v;
        }
        if (lane == 0) {
            A.sink_pos[n * A.sink_pos_stride[0] + h * A.sink_pos_stride[1] + j * A.sink_pos_stride[2]] = j;
            A.sink_mask[n * A.sink_mask_stride[0] + h * A.sink_mask_stride[1] + j * A.sink_mask_stride[2]] = 0;
        }
        return;
    }

    // scalars that travel with the row: score bits and original token index (lane 0 only)
    uint32_t c_score = 0;
    int64_t c_og = 0;
    if (lane == 0) {
        const int64_t so = n * A.s_stride[0] + h * A.s_stride[1] + t_in * A.s_stride[2];
        c_score = es == 4 ? reinterpret_cast<const uint32_t*>(A.s)[so] : reinterpret_cast<const uint16_t*>(A.s)[so];
        c_og = *A.real_token_idx + t_in + 1;  // cascading_cache.py:388
    }
    char* ck = reinterpret_cast<char*>(A.cache_k) + (n * A.cache_stride[0] + h * A.cache_stride[1]) * es;
    char* cv = reinterpret_cast<char*>(A.cache_v) + (n * A.cache_stride[0] + h * A.cache_stride[1]) * es;
    const int64_t row_bytes = A.cache_stride[2] * es;
    const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int64_t* og = A.og_pos + n * A.og_pos_stride[0] + h * A.og_pos_stride[1];
    uint8_t* mask = A.mask + n * A.mask_stride[0] + h * A.mask_stride[1];

    // A chain is walked kHops slots at a time.  First only its slot numbers (4-byte loads that depend on
    // each other, served by the L2 the plan kernel has just written them to); then every displaced row of
    // the stretch is requested at once, so the rows cost one trip to memory instead of one per hop; then
    // the stretch is written: slot 0 takes the carried row, slot j the row displaced from slot j - 1.
    constexpr int kHops = 4;
    for (int round = 0; round * kHops <= A.cascades; round++) {  // a chain visits each cascade at most once
        int sl[kHops];
        int nx = d;
#pragma unroll
        for (int j = 0; j < kHops; j++) {
            sl[j] = nx;
            nx = nx >= 0 ? next_of[nx] : -1;
        }
        RowPiece old[kHops];
        uint32_t o_score[kHops];
        int64_t o_og[kHops];
#pragma unroll
        for (int j = 0; j < kHops; j++) {
            const int succ = j + 1 < kHops ? sl[j + 1] : nx;
            old[j].k = old[j].v = make_uint4(0, 0, 0, 0);
            o_score[j] = 0;
            o_og[j] = 0;
            if (sl[j] >= 0 && succ >= 0) {  // the displaced row lives on elsewhere: pick it up
                if (active) {
                    old[j].k = reinterpret_cast<const uint4*>(ck + (int64_t)sl[j] * row_bytes)[lane];
                    old[j].v = reinterpret_cast<const uint4*>(cv + (int64_t)sl[j] * row_bytes)[lane];
                }
                if (lane == 0) {
                    const int64_t sidx = cs_base + (int64_t)sl[j] * A.cache_s_stride[2];
                    o_score[j] = es == 4 ? reinterpret_cast<const uint32_t*>(A.cache_s)[sidx]
                                         : reinterpret_cast<const uint16_t*>(A.cache_s)[sidx];
                    o_og[j] = og[(int64_t)sl[j] * A.og_pos_stride[2]];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kHops; j++) {
            if (sl[j] < 0) continue;
            const RowPiece& src = j == 0 ? carry : old[j - 1];
            const uint32_t w_score = j == 0 ? c_score : o_score[j - 1];
            const int64_t w_og = j == 0 ? c_og : o_og[j - 1];
            if (active) {
                reinterpret_cast<uint4*>(ck + (int64_t)sl[j] * row_bytes)[lane] = src.k;
                reinterpret_cast<uint4*>(cv + (int64_t)sl[j] * row_bytes)[lane] = src.v;
            }
            if (lane == 0) {
                const int64_t sidx = cs_base + (int64_t)sl[j] * A.cache_s_stride[2];
                if (es == 4) {
                    reinterpret_cast<uint32_t*>(A.cache_s)[sidx] = w_score;
                } else {
                    reinterpret_cast<uint16_t*>(A.cache_s)[sidx] = (uint16_t)w_score;
                }
                og[(int64_t)sl[j] * A.og_pos_stride[2]] = w_og;
                mask[(int64_t)sl[j] * A.mask_stride[2]] = 0;
            }
        }
        if (nx < 0) break;
        carry = old[kHops - 1];
        c_score = o_score[kHops - 1];
        c_og = o_og[kHops - 1];
        d = nx;
    }
}

// The whole update of a single incoming token (the decode step) in one launch.  One workgroup owns everything
// of its (batch, kv head): wavefront 0 plans as the single-token plan kernel does (the chain of slots stays in
// LDS: the token lands in chain[0], the old content of chain[j] in chain[j + 1], the last entry's old content is
// dropped), writes the trackers and leaves their values after the call in LDS; then wavefront j moves the row
// that ends in chain[j] (all rows are read before any is written) while every thread writes position ids from
// the trackers in LDS.  No order between workgroups is needed, so plan, moves and position ids share a launch.
// Same semantics as cascading_cache.py:381-774 for one token.  Needs 16-byte row pieces and at most kOneWaves
// cascades.
constexpr int kOneThreads = 1024, kOneWaves = kOneThreads / CKV_WAVE;
// One workgroup writes all position ids of its unit, which takes as long with 8 units as with 128; the two-launch
// path spreads them over the chip and is faster while the units are few (8 units of 64K slots: 9.4 + a launch gap
// against 13.4 us; 128 units of 32K slots: 18 against 12.5 us).
constexpr int kOneMinUnits = 32;

__global__ void __launch_bounds__(kOneThreads) ckv_update_one_kernel(UpdateParams p) {
    __shared__ int sh_chain[kOneWaves];
    __shared__ int sh_n, sh_pos;
    __shared__ int sh_write[kOneWaves];                     // position ids of the cascade are written
    __shared__ unsigned sh_seg[kOneWaves], sh_add[kOneWaves];
    __shared__ long long sh_base[kOneWaves];
    const ckv_update_args& A = p.a;
    const int tid = threadIdx.x, lane = tid % CKV_WAVE, wave = tid / CKV_WAVE;
    const int64_t bh = blockIdx.x;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int C = A.cascades;
    const int64_t W = A.window_size, S = A.max_seq_len, NS = A.num_sink;
    const int es = (int)elem_bytes(A.dtype);

    if (wave == 0) {
        int64_t* g_stored = A.stored_tokens + n * A.tracker_stride[0] + h * A.tracker_stride[1];
        int64_t* g_start = A.start_indices + n * A.tracker_stride[0] + h * A.tracker_stride[1];
        int64_t* g_sinks = A.stored_sinks + n * A.stored_sinks_stride[0] + h * A.stored_sinks_stride[1];
        const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
        const int64_t gidx = *A.real_token_idx;  // 0-based global index of the token
        const int64_t sinks0 = *g_sinks;
        const float tok_score = load_as_float(A.s, n * A.s_stride[0] + h * A.s_stride[1], A.dtype);
        // lane i: cascade i; all cascades' loads travel together
        int32_t st = 0, sx = 0;
        int64_t per = 1;
        float oldest = 0.f, newest = 0.f;
        if (lane < C) {
            st = (int32_t)g_stored[lane * A.tracker_stride[2]];
            sx = (int32_t)g_start[lane * A.tracker_stride[2]];
            per = A.do_cache_every_n[lane];
            const int64_t l = (int64_t)lane * W;
            if (st > 0) {
                oldest = load_as_float(A.cache_s, cs_base + (l + sx) * A.cache_s_stride[2], A.dtype);
                newest = load_as_float(A.cache_s, cs_base + (l + (sx - 1 + st) % st) * A.cache_s_stride[2], A.dtype);
            }
        }
        int n_chain = 0, do_pos = 1;
        int st_new = st, sx_new = sx;  // lane i: trackers of cascade i after the call
        if (sinks0 < NS) {  // the token is a sink (cascading_cache.py:399-431): no position pass
            if (lane == 0) {
                sh_chain[0] = (int)(S + sinks0);
                *g_sinks = sinks0 + 1;
            }
            n_chain = 1;
            do_pos = 0;
        } else {
            float carry_score = tok_score;
            const int64_t rel = gidx - NS;
            const bool eager = A.eager_fill && gidx <= S + NS;
            for (int i = 0; i < C; i++) {
                const int32_t st_i = __shfl(st, i), sx_i = __shfl(sx, i);
                const int64_t per_i = __shfl(per, i);
                const int l = (int)((int64_t)i * W);
                const bool acc = eager || (rel % per_i) == 0;
                if (acc || st_i == 0) {
                    const int phys = l + (int)(((int64_t)sx_i + st_i) % W);
                    if (lane == 0) sh_chain[n_chain] = phys;
                    n_chain++;
                    if (st_i < (int32_t)W) {  // append (or the first entry of an empty cascade)
                        if (lane == i) st_new = st_i + 1;
                        if (lane == 0) g_stored[i * A.tracker_stride[2]] = st_i + 1;
                        break;
                    }
                    // full: the oldest entry (at the ring start) leaves for the next cascade, or is dropped
                    if (lane == i) sx_new = (sx_i + 1) % (int32_t)W;
                    if (lane == 0) g_start[i * A.tracker_stride[2]] = (int64_t)((sx_i + 1) % (int32_t)W);
                    carry_score = __shfl(oldest, i);
                    continue;
                }
                // not accepted: the newest slot keeps its token unless the arrival's score is at least as large
                if (carry_score >= __shfl(newest, i)) {
                    if (lane == 0) sh_chain[n_chain] = l + (sx_i - 1 + st_i) % st_i;
                    n_chain++;
                }
                break;
            }
        }
        // ---- parameters of the position ids (cascading_cache.py:728-774, 129-142) from the trackers after the
        //      call, which lane i holds for cascade i: the same closed form as the position blocks of the apply
        //      kernel.  Cascade i is written while every earlier cascade holds tokens and ids are left for it.
        {
            long long tot = lane < C ? (long long)st_new : 0;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) tot += __shfl_xor(tot, off);
            const unsigned long long empty = __builtin_amdgcn_ballot_w64(lane < C && st_new <= 0);
            const int first_empty = empty ? __builtin_ctzll(empty) : C;
            if (lane < C) {
                const long long ub = tot - (long long)lane * W;   // ids still to hand out when cascade `lane` is reached
                const unsigned seg = (unsigned)((long long)st_new < W ? st_new : (int32_t)W);
                sh_write[lane] = (lane <= first_empty && (lane == 0 || ub > 0) && seg != 0) ? 1 : 0;
                sh_seg[lane] = seg;
                sh_add[lane] = seg - (unsigned)sx_new;  // start < seg or start == 0
                sh_base[lane] = ub - (long long)seg;
            }
        }
        if (lane == 0) {
            sh_n = n_chain;
            sh_pos = do_pos;
        }
    }
    __syncthreads();
    const int n_chain = sh_n;
    const bool do_pos = sh_pos != 0;

    // ---- rows: wavefront j takes the row that ends in chain[j] (the token, or the old content of chain[j - 1])
    const int chunks = (int)(A.HID * es / 16);
    uint4 rk = make_uint4(0, 0, 0, 0), rv = make_uint4(0, 0, 0, 0);
    uint32_t r_score = 0;
    int64_t r_og = 0;
    const bool mover = wave < n_chain;
    const bool piece = lane < chunks;
    char* ck = reinterpret_cast<char*>(A.cache_k) + (n * A.cache_stride[0] + h * A.cache_stride[1]) * es;
    char* cv = reinterpret_cast<char*>(A.cache_v) + (n * A.cache_stride[0] + h * A.cache_stride[1]) * es;
    const int64_t row_bytes = A.cache_stride[2] * es;
    const int64_t cs_base = n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int64_t* og = A.og_pos + n * A.og_pos_stride[0] + h * A.og_pos_stride[1];
    if (mover) {
        if (wave == 0) {
            const int64_t in_off = (n * A.kv_stride[0] + h * A.kv_stride[1]) * es;
            if (piece) {
                rk = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.k) + in_off)[lane];
                rv = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(A.v) + in_off)[lane];
            }
            if (lane == 0) {
                const int64_t so = n * A.s_stride[0] + h * A.s_stride[1];
                r_score = es == 4 ? reinterpret_cast<const uint32_t*>(A.s)[so] : reinterpret_cast<const uint16_t*>(A.s)[so];
                r_og = *A.real_token_idx + 1;  // cascading_cache.py:388
            }
        } else {
            const int src = sh_chain[wave - 1];
            if (piece) {
                rk = reinterpret_cast<const uint4*>(ck + (int64_t)src * row_bytes)[lane];
                rv = reinterpret_cast<const uint4*>(cv + (int64_t)src * row_bytes)[lane];
            }
            if (lane == 0) {
                const int64_t sidx = cs_base + (int64_t)src * A.cache_s_stride[2];
                r_score = es == 4 ? reinterpret_cast<const uint32_t*>(A.cache_s)[sidx] : reinterpret_cast<const uint16_t*>(A.cache_s)[sidx];
                r_og = og[(int64_t)src * A.og_pos_stride[2]];
            }
        }
    }
    // ---- position ids: they need the plan alone, so their stores go out while the displaced rows are on their way
    if (do_pos) {
        int64_t* pos = A.pos + n * A.pos_stride[0] + h * A.pos_stride[1];
        auto id_of = [&](int i, unsigned j) -> int64_t {
            const unsigned seg = sh_seg[i];
            unsigned x = j + sh_add[i];
            if (x >= seg) x -= seg;
            if (x >= seg) x %= seg;  // slots past the stored tokens of a cascade that is not full
            return (int64_t)x + sh_base[i];
        };
        if (A.pos_stride[2] == 1 && (reinterpret_cast<uintptr_t>(pos) & 15u) == 0 && (W & 1) == 0) {
            for (int i = 0; i < C; i++) {
                if (!sh_write[i]) continue;
                int64_t* pc = pos + (int64_t)i * W;
                for (int64_t j = 2 * (int64_t)tid; j < W; j += 2 * kOneThreads)
                    *reinterpret_cast<longlong2*>(pc + j) = make_longlong2(id_of(i, (unsigned)j), id_of(i, (unsigned)j + 1));
            }
        } else {
            for (int i = 0; i < C; i++) {
                if (!sh_write[i]) continue;
                for (int64_t j = tid; j < W; j += kOneThreads) pos[((int64_t)i * W + j) * A.pos_stride[2]] = id_of(i, (unsigned)j);
            }
        }
    }
    __syncthreads();  // every displaced row is in registers
    if (mover) {
        const int d = sh_chain[wave];
        if (d >= S) {  // sink slot (cascading_cache.py:61-109); only the token itself gets here
            const int64_t j = d - S;
            const int64_t so = (n * A.sink_stride[0] + h * A.sink_stride[1] + j * A.sink_stride[2]) * es;
            if (piece) {
                reinterpret_cast<uint4*>(reinterpret_cast<char*>(A.sink_k) + so)[lane] = rk;
                reinterpret_cast<uint4*>(reinterpret_cast<char*>(A.sink_v) + so)[lane] = rv;
            }
            if (lane == 0) {
                A.sink_pos[n * A.sink_pos_stride[0] + h * A.sink_pos_stride[1] + j * A.sink_pos_stride[2]] = j;
                A.sink_mask[n * A.sink_mask_stride[0] + h * A.sink_mask_stride[1] + j * A.sink_mask_stride[2]] = 0;
            }
        } else {
            if (piece) {
                reinterpret_cast<uint4*>(ck + (int64_t)d * row_bytes)[lane] = rk;
                reinterpret_cast<uint4*>(cv + (int64_t)d * row_bytes)[lane] = rv;
            }
            if (lane == 0) {
                const int64_t sidx = cs_base + (int64_t)d * A.cache_s_stride[2];
                if (es == 4) reinterpret_cast<uint32_t*>(A.cache_s)[sidx] = r_score;
                else reinterpret_cast<uint16_t*>(A.cache_s)[sidx] = (uint16_t)r_score;
                og[(int64_t)d * A.og_pos_stride[2]] = r_og;
                (A.mask + n * A.mask_stride[0] + h * A.mask_stride[1])[(int64_t)d * A.mask_stride[2]] = 0;
            }
        }
    }
}

// Layouts the vector kernel cannot address (innermost stride != 1, rows not a multiple of 16
// bytes, unaligned bases): one wavefront per token, one element at a time.
template <typename U>
__global__ void ckv_update_apply_elem_kernel(UpdateParams p) {
    const ckv_update_args& A = p.a;
    constexpr int kPerLane = 8;
    if (blockIdx.x == 0 && p.do_pos && p.mode[blockIdx.y] && (int)threadIdx.x < A.cascades) {
        // commit the ring starts the steady-state plan left in scratch (nobody reads the trackers in this launch)
        const int64_t bh_c = blockIdx.y;
        A.start_indices[(bh_c / A.H) * A.tracker_stride[0] + (bh_c % A.H) * A.tracker_stride[1] +
                        threadIdx.x * A.tracker_stride[2]] = p.start_new[bh_c * A.cascades + threadIdx.x];
    }
    if ((int)blockIdx.x >= p.apply_blocks) {
        update_positions_block(p, (int)blockIdx.x - p.apply_blocks);
        return;
    }
    const int g = blockIdx.x * (256 / CKV_WAVE) + threadIdx.x / CKV_WAVE;
    const int lane = threadIdx.x % CKV_WAVE;
    if (g >= p.k_sub) return;
    const int64_t bh = blockIdx.y;
    const int64_t n = bh / A.H, h = bh % A.H;
    const int64_t S = A.max_seq_len;
    const int32_t* first = p.first + bh * A.K + p.token_offset;
    const int32_t* next_of = p.next_of + bh * S;
    int d = first[g];
    if (d < 0) return;
    const int64_t t_in = p.token_offset + g;
    const U* kin = reinterpret_cast<const U*>(A.k) + n * A.kv_stride[0] + h * A.kv_stride[1] + t_in * A.kv_stride[2];
    const U* vin = reinterpret_cast<const U*>(A.v) + n * A.kv_stride[0] + h * A.kv_stride[1] + t_in * A.kv_stride[2];
    U ck_[kPerLane], cv_[kPerLane], ok_[kPerLane], ov_[kPerLane];
#pragma unroll
    for (int r = 0; r < kPerLane; r++) {
        const int64_t e = lane + (int64_t)r * CKV_WAVE;
        if (e < A.HID) {
            ck_[r] = kin[e * A.kv_stride[3]];
            cv_[r] = vin[e * A.kv_stride[3]];
        }
    }
    if (d >= S) {
        const int64_t j = d - S;
        U* sk = reinterpret_cast<U*>(A.sink_k) + n * A.sink_stride[0] + h * A.sink_stride[1] + j * A.sink_stride[2];
        U* sv = reinterpret_cast<U*>(A.sink_v) + n * A.sink_stride[0] + h * A.sink_stride[1] + j * A.sink_stride[2];
#pragma unroll
        for (int r = 0; r < kPerLane; r++) {
            const int64_t e = lane + (int64_t)r * CKV_WAVE;
            if (e < A.HID) {
                sk[e * A.sink_stride[3]] = ck_[r];
                sv[e * A.sink_stride[3]] = cv_[r];
            }
        }
        if (lane == 0) {
            A.sink_pos[n * A.sink_pos_stride[0] + h * A.sink_pos_stride[1] + j * A.sink_pos_stride[2]] = j;
            A.sink_mask[n * A.sink_mask_stride[0] + h * A.sink_mask_stride[1] + j * A.sink_mask_stride[2]] = 0;
        }
        return;
    }
    U c_score = reinterpret_cast<const U*>(A.s)[n * A.s_stride[0] + h * A.s_stride[1] + t_in * A.s_stride[2]];
    int64_t c_og = *A.real_token_idx + t_in + 1;
    U* ck = reinterpret_cast<U*>(A.cache_k) + n * A.cache_stride[0] + h * A.cache_stride[1];
    U* cv = reinterpret_cast<U*>(A.cache_v) + n * A.cache_stride[0] + h * A.cache_stride[1];
    U* cs = reinterpret_cast<U*>(A.cache_s) + n * A.cache_s_stride[0] + h * A.cache_s_stride[1];
    int64_t* og = A.og_pos + n * A.og_pos_stride[0] + h * A.og_pos_stride[1];
    uint8_t* mask = A.mask + n * A.mask_stride[0] + h * A.mask_stride[1];
    for (int hop = 0; hop <= A.cascades; hop++) {
        const int nd = next_of[d];
        U* kd = ck + (int64_t)d * A.cache_stride[2];
        U* vd = cv + (int64_t)d * A.cache_stride[2];
        U o_score = c_score;
        int64_t o_og = 0;
        if (nd >= 0) {
#pragma unroll
            for (int r = 0; r < kPerLane; r++) {
                const int64_t e = lane + (int64_t)r * CKV_WAVE;
                if (e < A.HID) {
                    ok_[r] = kd[e * A.cache_stride[3]];
                    ov_[r] = vd[e * A.cache_stride[3]];
                }
            }
            o_score = cs[(int64_t)d * A.cache_s_stride[2]];
            o_og = og[(int64_t)d * A.og_pos_stride[2]];
        }
#pragma unroll
        for (int r = 0; r < kPerLane; r++) {
            const int64_t e = lane + (int64_t)r * CKV_WAVE;
            if (e < A.HID) {
                kd[e * A.cache_stride[3]] = ck_[r];
                vd[e * A.cache_stride[3]] = cv_[r];
            }
        }
        if (lane == 0) {
            cs[(int64_t)d * A.cache_s_stride[2]] = c_score;
            og[(int64_t)d * A.og_pos_stride[2]] = c_og;
            mask[(int64_t)d * A.mask_stride[2]] = 0;
        }
        if (nd < 0) break;
#pragma unroll
        for (int r = 0; r < kPerLane; r++) {
            ck_[r] = ok_[r];
            cv_[r] = ov_[r];
        }
        c_score = o_score;
        c_og = o_og;
        d = nd;
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline size_t plan_lds_bytes(int cap) {
    return (size_t)cap * 24 + (size_t)(cap + 1) * 8 + (size_t)(cap + 2) * 4 + kMaxCascades * 20 + 64 * sizeof(int) + 64;
}

}  // namespace
}  // namespace ckv

extern "C" int64_t ckv_update_workspace_bytes(int64_t N, int64_t H, int64_t K, int64_t max_seq_len,
                                              int32_t cascades) {
    if (N <= 0 || H <= 0 || K < 0 || max_seq_len <= 0 || cascades <= 0) return 0;
    // move chains (first, next_of), then per unit: position flag, plan mode, ring starts after the call
    return ckv::align_up(N * H * (K + max_seq_len) * (int64_t)sizeof(int32_t), 256) +
           2 * ckv::align_up(N * H * (int64_t)sizeof(int32_t), 256) +
           ckv::align_up(N * H * cascades * (int64_t)sizeof(int32_t), 256) + 256;
}

// Scratch of the entry point that allocates nothing (ckv_update_static): one array per device, part of the
// code object, held until the process ends.  In host code its name is a stand-in, not a device address:
// the address is looked up once per device (static_scratch below) and only that address is ever handed to
// kernels.
constexpr int64_t kStaticScratchBytes = (int64_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace ckv {
namespace {

constexpr int kScratchDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kScratchDevices];

int static_scratch(void** out) {
    int dev = 0;
    CKV_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kScratchDevices) return CKV_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        CKV_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));  // the current device's copy of the array
        if (!ptr) return CKV_ERR_LAUNCH;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return CKV_OK;
}

// launch with the stage's timing: events attached to the dispatch when single kernels are timed, else the
// stream bracket of StageScope
template <typename Kernel>
void launch_timed(int stage, Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const UpdateParams& p) {
    StageScope sc(stage, stream, true);
    hipEvent_t ev0, ev1;
    prof_kernel_events(stage, &ev0, &ev1);
    if (ev0) hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, stream, ev0, ev1, 0u, p);
    else hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
}

int run_update(const ckv_update_args& A, void* workspace, hipStream_t stream) {
    const int es = (int)elem_bytes(A.dtype);
    const bool vec = A.kv_stride[3] == 1 && A.cache_stride[3] == 1 && (A.num_sink == 0 || A.sink_stride[3] == 1) &&
                     (A.HID * es) % 16 == 0 && A.HID * es <= 16 * 64 && aligned16(A.k) && aligned16(A.v) &&
                     aligned16(A.cache_k) && aligned16(A.cache_v) &&
                     (A.num_sink == 0 || (aligned16(A.sink_k) && aligned16(A.sink_v))) &&
                     (A.kv_stride[0] * es) % 16 == 0 && (A.kv_stride[1] * es) % 16 == 0 &&
                     (A.kv_stride[2] * es) % 16 == 0 && (A.cache_stride[0] * es) % 16 == 0 &&
                     (A.cache_stride[1] * es) % 16 == 0 && (A.cache_stride[2] * es) % 16 == 0 &&
                     (A.sink_stride[0] * es) % 16 == 0 && (A.sink_stride[1] * es) % 16 == 0 &&
                     (A.sink_stride[2] * es) % 16 == 0;
    if (!vec && A.HID > 8 * CKV_WAVE) return CKV_ERR_UNSUPPORTED;

    DeviceInfo di;
    if (int rc = current_device_info(&di)) return rc;
    const int lds_max = di.lds_max;
    int qmax = (int)((lds_max - 4096) / 36);
    qmax = qmax / 64 * 64;
    if (qmax > kPlanMaxTokens) qmax = kPlanMaxTokens;
    if (qmax < 64) return CKV_ERR_UNSUPPORTED;

    UpdateParams p;
    p.a = A;
    p.first = reinterpret_cast<int32_t*>(workspace);
    p.next_of = p.first + A.N * A.H * A.K;
    p.pos_flag = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) +
                                            align_up(A.N * A.H * (A.K + A.max_seq_len) * (int64_t)sizeof(int32_t), 256));
    p.mode = p.pos_flag + align_up(A.N * A.H * (int64_t)sizeof(int32_t), 256) / 4;
    p.start_new = p.mode + align_up(A.N * A.H * (int64_t)sizeof(int32_t), 256) / 4;
    p.token_offset = 0;
    p.k_sub = 0;
    p.do_pos = 0;
    p.apply_blocks = 0;
    if (A.K == 1 && vec && A.cascades <= kOneWaves && A.HID * es / 16 <= CKV_WAVE && A.N * A.H >= kOneMinUnits) {
        // the decode step of many streams: plan, moves and position ids of a unit by one workgroup, one launch
        launch_timed(CKV_STAGE_APPLY, ckv_update_one_kernel, dim3((unsigned)(A.N * A.H)), dim3(kOneThreads), 0, stream, p);
        CKV_HIP_TRY(hipGetLastError());
        return CKV_OK;
    }
    if (A.K >= 2) {
        // every unit first gets the chance of the steady-state plan (whole call, all cascades side by side); it
        // marks the units it has planned, the general kernel below takes the others
        launch_timed(CKV_STAGE_PLAN, ckv_update_plan_steady_kernel,
                     dim3((unsigned)(A.cascades * kSteadyParts), (unsigned)(A.N * A.H)), dim3(kSteadyThreads), 0, stream, p);
        CKV_HIP_TRY(hipGetLastError());
    }

    for (int64_t off = 0; off < A.K; off += qmax) {
        const int ksub = (int)((A.K - off < qmax) ? (A.K - off) : qmax);
        p.token_offset = off;
        p.k_sub = ksub;
        p.do_pos = (off + ksub == A.K) ? 1 : 0;
        if (A.K == 1) {  // the decode step: one wavefront per unit
            launch_timed(CKV_STAGE_PLAN, ckv_update_plan1_kernel, dim3((unsigned)(A.N * A.H)), dim3(CKV_WAVE), 0, stream, p);
        } else {
            const int T = ksub <= 256 ? 256 : 1024;  // few tokens: a small block plans them
            const size_t lds = plan_lds_bytes(ksub);
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(ckv_update_plan_kernel), (int)lds)) return rc;
            launch_timed(CKV_STAGE_PLAN, ckv_update_plan_kernel, dim3((unsigned)(A.N * A.H)), dim3(T), lds, stream, p);
        }
        CKV_HIP_TRY(hipGetLastError());
        // the position ids of the last launch of a call are written by extra blocks of the apply grid
        const unsigned pos_blocks =
            p.do_pos ? (unsigned)(((A.window_size + kPosChunk - 1) / kPosChunk) * A.cascades) : 0u;

        if (vec) {
            const int chunks = (int)(A.HID * es / 16);
            int lanes = 1;
            while (lanes < chunks) lanes *= 2;
            const dim3 block(256);
            p.apply_blocks = (ksub + 256 / lanes - 1) / (256 / lanes);
            const dim3 grid((unsigned)p.apply_blocks + pos_blocks, (unsigned)(A.N * A.H));
            switch (lanes) {
                case 1: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<1>, grid, block, 0, stream, p); break;
                case 2: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<2>, grid, block, 0, stream, p); break;
                case 4: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<4>, grid, block, 0, stream, p); break;
                case 8: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<8>, grid, block, 0, stream, p); break;
                case 16: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<16>, grid, block, 0, stream, p); break;
                case 32: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<32>, grid, block, 0, stream, p); break;
                default: launch_timed(CKV_STAGE_APPLY, ckv_update_apply_vec_kernel<64>, grid, block, 0, stream, p); break;
            }
        } else {
            const dim3 block(256);
            p.apply_blocks = (ksub + 3) / 4;
            const dim3 grid((unsigned)p.apply_blocks + pos_blocks, (unsigned)(A.N * A.H));
            if (es == 4) {
                launch_timed(CKV_STAGE_APPLY, ckv_update_apply_elem_kernel<uint32_t>, grid, block, 0, stream, p);
            } else {
                launch_timed(CKV_STAGE_APPLY, ckv_update_apply_elem_kernel<uint16_t>, grid, block, 0, stream, p);
            }
        }
        CKV_HIP_TRY(hipGetLastError());
    }
    return CKV_OK;
}

// everything ckv_update checks before it looks at the scratch; *empty: nothing to do
int check_update_args(const ckv_update_args* args, bool* empty) {
    *empty = false;
    if (!args) return CKV_ERR_NULL;
    const ckv_update_args& A = *args;
    if (A.dtype != CKV_F32 && A.dtype != CKV_F16 && A.dtype != CKV_BF16) return CKV_ERR_DTYPE;
    if (A.N <= 0 || A.H <= 0 || A.K < 0 || A.HID <= 0 || A.num_sink < 0) return CKV_ERR_SHAPE;
    if (A.window_size <= 0 || A.cascades <= 0 || A.cascades > kMaxCascades) return CKV_ERR_SHAPE;
    if ((int64_t)A.cascades * A.window_size != A.max_seq_len) return CKV_ERR_SHAPE;
    if (A.max_seq_len + A.num_sink >= (int64_t)1 << 30 || A.K >= (int64_t)1 << 30) return CKV_ERR_SHAPE;
    if (A.N * A.H > 65535) return CKV_ERR_UNSUPPORTED;
    if (!A.cache_k || !A.cache_v || !A.cache_s || !A.mask || !A.pos || !A.og_pos || !A.stored_tokens ||
        !A.start_indices || !A.stored_sinks || !A.do_cache_every_n || !A.real_token_idx)
        return CKV_ERR_NULL;
    if (A.num_sink > 0 && (!A.sink_k || !A.sink_v || !A.sink_mask || !A.sink_pos)) return CKV_ERR_NULL;
    if (A.K == 0) {
        *empty = true;
        return CKV_OK;
    }
    if (!A.k || !A.v || !A.s) return CKV_ERR_NULL;
    return CKV_OK;
}

}  // namespace
}  // namespace ckv

extern "C" int ckv_update(const ckv_update_args* args, void* stream_) {
    using namespace ckv;
    bool empty;
    if (int rc = check_update_args(args, &empty)) return rc;
    if (empty) return CKV_OK;
    const ckv_update_args& A = *args;
    const int64_t need = ckv_update_workspace_bytes(A.N, A.H, A.K, A.max_seq_len, A.cascades);
    if (!A.workspace || A.workspace_bytes < need) return CKV_ERR_WORKSPACE;
    return run_update(A, A.workspace, reinterpret_cast<hipStream_t>(stream_));
}

extern "C" int64_t ckv_update_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int ckv_update_static(const ckv_update_args* args, void* stream_) {
    using namespace ckv;
    bool empty;
    if (int rc = check_update_args(args, &empty)) return rc;
    if (empty) return CKV_OK;
    const ckv_update_args& A = *args;
    if (ckv_update_workspace_bytes(A.N, A.H, A.K, A.max_seq_len, A.cascades) > kStaticScratchBytes) return CKV_ERR_TOO_LARGE;
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    // Nothing in the scratch has to start at zero: the plan kernel writes every chain entry and flag the
    // apply kernel reads, whatever the last call left there.
    return run_update(A, ws, reinterpret_cast<hipStream_t>(stream_));
}
