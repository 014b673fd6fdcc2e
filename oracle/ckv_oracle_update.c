/*
 * TEST INFRASTRUCTURE — CPU oracle of the cascading cache update.  Never shipped, never a
 * fallback: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it.
 *
 * A literal, serial, per-token restatement of the reference's update kernel for host memory:
 *   _update_kv_cache        cascade/models/cascading_cache.py:145-299  (token loop, :223)
 *   _update_kv_cache_inner  cascade/models/cascading_cache.py:302-774
 *   _update_sink_cache      cascade/models/cascading_cache.py:22-109
 *   _update_positional_idx  cascade/models/cascading_cache.py:112-142
 * It has an argument block of its own (`oracle_update_desc` below: one {pointer, strides} record
 * per tensor, filled by oracle/update.py) and shares no header and no marshalling code with the
 * library under test, so a wrong stride or field on the product's side cannot reach both sides.
 *
 * Pinned by tests/test_oracle_update.py (closed forms for sinks and metadata, the C=1
 * StreamingLLM special case, the eager-fill rule, split-call invariance, a restatement of the
 * reference's independent per-token CascadingKVCacheSlow, and a group-maximum closed form for
 * the score tournament).
 */
#include <stdint.h>
#include <string.h>

/* dtype codes and status values of the oracle (its own; the Python face maps torch dtypes to them) */
enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 };
enum { ORACLE_OK = 0, ORACLE_ERR_NULL = 1, ORACLE_ERR_DTYPE = 2, ORACLE_ERR_SHAPE = 3 };

/* a host tensor: base pointer and element strides, outermost dimension first (unused entries 0) */
typedef struct oracle_tensor {
    void* ptr;
    int64_t stride[4];
} oracle_tensor;

/* the arguments of sink_cache (cascading_cache.py:962-985) in the order of that signature */
typedef struct oracle_update_desc {
    oracle_tensor k, v, s;                         /* (N, H, K, HID) x2, (N, >=H, K)              */
    oracle_tensor sink_k, sink_v;                  /* (N, H, num_sink, HID)                       */
    oracle_tensor sink_mask, sink_pos;             /* (N, H, num_sink) bool / int64               */
    oracle_tensor cache_k, cache_v, cache_s;       /* (N, H, S, HID) x2, (N, H, S)                */
    oracle_tensor mask, pos, og_pos;               /* (N, H, S) bool / int64 / int64              */
    oracle_tensor do_cache_every_n;                /* (cascades,) int64                           */
    oracle_tensor stored_tokens, start_indices;    /* (N, H, cascades) int64                      */
    oracle_tensor stored_sinks;                    /* (N, H) int64                                */
    int64_t num_sink, window_size, real_token_idx, max_seq_len;
    int64_t eager_fill;
    int64_t n, h, k_len, hid, cascades;            /* sizes of k and of the trackers              */
    int64_t dtype;                                 /* ORACLE_F32 / F16 / BF16                     */
} oracle_update_desc;

/* The body below is written against flat names; this view gives them from the per-tensor records. */
typedef struct oracle_view {
    const void *k, *v, *s;
    void *sink_k, *sink_v, *cache_k, *cache_v, *cache_s;
    uint8_t *sink_mask, *mask;
    int64_t *sink_pos, *pos, *og_pos, *stored_sinks, *stored_tokens, *start_indices;
    const int64_t* do_cache_every_n;
    const int64_t *kv_stride, *s_stride, *sink_stride, *cache_stride, *cache_s_stride, *sink_mask_stride,
        *mask_stride, *sink_pos_stride, *pos_stride, *og_pos_stride, *stored_sinks_stride, *tracker_stride;
    int64_t every_n_stride;
    int64_t N, H, K, HID, num_sink, window_size, max_seq_len, cascades, seen;
    int eager_fill, dtype;
} oracle_view;

static float oracle_load_score(const void* base, int64_t idx, int dtype) {
    if (dtype == ORACLE_F32) {
        return ((const float*)base)[idx];
    }
    uint16_t h = ((const uint16_t*)base)[idx];
    uint32_t bits;
    if (dtype == ORACLE_BF16) {
        bits = (uint32_t)h << 16;
    } else { /* IEEE binary16 -> binary32, exact */
        uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
        uint32_t exp = (h >> 10) & 0x1fu;
        uint32_t man = h & 0x3ffu;
        if (exp == 0) {
            if (man == 0) {
                bits = sign;
            } else {
                int e = -1;
                do {
                    man <<= 1;
                    e++;
                } while ((man & 0x400u) == 0);
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
            }
        } else if (exp == 31) {
            bits = sign | 0x7f800000u | (man << 13);
        } else {
            bits = sign | ((exp + 112u) << 23) | (man << 13);
        }
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static int64_t elem_size(int dtype) { return dtype == ORACLE_F32 ? 4 : 2; }

/* one row of HID elements, arbitrary strides */
static void copy_row(void* dst, int64_t dst_off, int64_t dst_sh, const void* src, int64_t src_off,
                     int64_t src_sh, int64_t hid, int64_t es) {
    for (int64_t d = 0; d < hid; d++) {
        memcpy((char*)dst + (dst_off + d * dst_sh) * es, (const char*)src + (src_off + d * src_sh) * es,
               (size_t)es);
    }
}

int ckv_oracle_update(const oracle_update_desc* d) {
    if (!d) return ORACLE_ERR_NULL;
    oracle_view view;
    view.k = d->k.ptr; view.v = d->v.ptr; view.s = d->s.ptr;
    view.sink_k = d->sink_k.ptr; view.sink_v = d->sink_v.ptr;
    view.cache_k = d->cache_k.ptr; view.cache_v = d->cache_v.ptr; view.cache_s = d->cache_s.ptr;
    view.sink_mask = (uint8_t*)d->sink_mask.ptr; view.mask = (uint8_t*)d->mask.ptr;
    view.sink_pos = (int64_t*)d->sink_pos.ptr; view.pos = (int64_t*)d->pos.ptr; view.og_pos = (int64_t*)d->og_pos.ptr;
    view.stored_sinks = (int64_t*)d->stored_sinks.ptr;
    view.stored_tokens = (int64_t*)d->stored_tokens.ptr; view.start_indices = (int64_t*)d->start_indices.ptr;
    view.do_cache_every_n = (const int64_t*)d->do_cache_every_n.ptr;
    view.every_n_stride = d->do_cache_every_n.stride[0];
    /* k and v, the two sink tensors, the two cache tensors and the two trackers are each walked with one
     * set of strides, as the reference kernel does (cascading_cache.py:846-891 passes k's, sink_k's,
     * cache_k's and stored_tokens' strides only); the Python face refuses pairs that differ */
    view.kv_stride = d->k.stride; view.s_stride = d->s.stride; view.sink_stride = d->sink_k.stride;
    view.cache_stride = d->cache_k.stride; view.cache_s_stride = d->cache_s.stride;
    view.sink_mask_stride = d->sink_mask.stride; view.mask_stride = d->mask.stride;
    view.sink_pos_stride = d->sink_pos.stride; view.pos_stride = d->pos.stride; view.og_pos_stride = d->og_pos.stride;
    view.stored_sinks_stride = d->stored_sinks.stride; view.tracker_stride = d->stored_tokens.stride;
    view.N = d->n; view.H = d->h; view.K = d->k_len; view.HID = d->hid;
    view.num_sink = d->num_sink; view.window_size = d->window_size; view.max_seq_len = d->max_seq_len;
    view.cascades = d->cascades; view.seen = d->real_token_idx;
    view.eager_fill = d->eager_fill != 0; view.dtype = (int)d->dtype;
    const oracle_view* a = &view;
    if (a->dtype != ORACLE_F32 && a->dtype != ORACLE_F16 && a->dtype != ORACLE_BF16) return ORACLE_ERR_DTYPE;
    const int64_t es = elem_size(a->dtype);
    const int64_t W = a->window_size, C = a->cascades, NS = a->num_sink, S = a->max_seq_len;
    if (W <= 0 || C <= 0 || C * W != S || a->HID <= 0 || a->HID > 4096) return ORACLE_ERR_SHAPE;
    const int64_t seen = a->seen;

    /* the carried row lives here between cascades (cascading_cache.py:589-593) */
    char ck[4096 * 4], cv[4096 * 4], tk[4096 * 4], tv[4096 * 4], cs[4], ts[4];

    for (int64_t n = 0; n < a->N; n++) {
        for (int64_t h = 0; h < a->H; h++) {
            int64_t* p_sinks = a->stored_sinks + n * a->stored_sinks_stride[0] + h * a->stored_sinks_stride[1];
            int64_t* stored = a->stored_tokens + n * a->tracker_stride[0] + h * a->tracker_stride[1];
            int64_t* start = a->start_indices + n * a->tracker_stride[0] + h * a->tracker_stride[1];
            const int64_t st_c = a->tracker_stride[2];
            const int64_t ck_base = n * a->cache_stride[0] + h * a->cache_stride[1];
            const int64_t cs_base = n * a->cache_s_stride[0] + h * a->cache_s_stride[1];
            const int64_t op_base = n * a->og_pos_stride[0] + h * a->og_pos_stride[1];
            const int64_t m_base = n * a->mask_stride[0] + h * a->mask_stride[1];
            int last_was_cache = 0;

            for (int64_t t = 0; t < a->K; t++) { /* cascading_cache.py:223 */
                const int64_t rti = seen + t + 1; /* cascading_cache.py:388 */
                const int64_t in_off = n * a->kv_stride[0] + h * a->kv_stride[1] + t * a->kv_stride[2];
                last_was_cache = 0;
                if (*p_sinks < NS) { /* cascading_cache.py:399-431, 61-109 */
                    const int64_t j = *p_sinks;
                    const int64_t so = n * a->sink_stride[0] + h * a->sink_stride[1] + j * a->sink_stride[2];
                    copy_row(a->sink_k, so, a->sink_stride[3], a->k, in_off, a->kv_stride[3], a->HID, es);
                    copy_row(a->sink_v, so, a->sink_stride[3], a->v, in_off, a->kv_stride[3], a->HID, es);
                    a->sink_pos[n * a->sink_pos_stride[0] + h * a->sink_pos_stride[1] + j * a->sink_pos_stride[2]] = j;
                    a->sink_mask[n * a->sink_mask_stride[0] + h * a->sink_mask_stride[1] + j * a->sink_mask_stride[2]] = 0;
                    *p_sinks = j + 1;
                    continue;
                }
                last_was_cache = 1;
                const int always = a->eager_fill && (rti - 1 <= S + NS); /* cascading_cache.py:471 */
                /* carry = incoming token (cascading_cache.py:447-462) */
                copy_row(ck, 0, 1, a->k, in_off, a->kv_stride[3], a->HID, es);
                copy_row(cv, 0, 1, a->v, in_off, a->kv_stride[3], a->HID, es);
                memcpy(cs, (const char*)a->s + (n * a->s_stride[0] + h * a->s_stride[1] + t * a->s_stride[2]) * es,
                       (size_t)es);
                int64_t og = rti;

                int64_t i = 0;
                while (i < C) { /* cascading_cache.py:466 */
                    const int64_t l = i * W;
                    int accept = always;
                    if (!accept) { /* cascading_cache.py:474-478 */
                        accept = ((rti - 1 - NS) % a->do_cache_every_n[i * a->every_n_stride]) == 0;
                    }
                    const int64_t st = stored[i * st_c], sx = start[i * st_c];
                    int64_t slot;
                    if (accept && st >= W) { /* evict the oldest, carry it down: :542-604 */
                        slot = l + sx;
                        const int64_t ko = ck_base + slot * a->cache_stride[2];
                        copy_row(tk, 0, 1, a->cache_k, ko, a->cache_stride[3], a->HID, es);
                        copy_row(tv, 0, 1, a->cache_v, ko, a->cache_stride[3], a->HID, es);
                        memcpy(ts, (char*)a->cache_s + (cs_base + slot * a->cache_s_stride[2]) * es, (size_t)es);
                        const int64_t tog = a->og_pos[op_base + slot * a->og_pos_stride[2]];
                        copy_row(a->cache_k, ko, a->cache_stride[3], ck, 0, 1, a->HID, es);
                        copy_row(a->cache_v, ko, a->cache_stride[3], cv, 0, 1, a->HID, es);
                        memcpy((char*)a->cache_s + (cs_base + slot * a->cache_s_stride[2]) * es, cs, (size_t)es);
                        a->og_pos[op_base + slot * a->og_pos_stride[2]] = og;
                        memcpy(ck, tk, (size_t)(a->HID * es));
                        memcpy(cv, tv, (size_t)(a->HID * es));
                        memcpy(cs, ts, (size_t)es);
                        og = tog;
                        start[i * st_c] = (sx + 1) % W;
                        i += 1;
                        continue; /* falling off the last cascade drops the carry */
                    }
                    if (accept || st == 0) { /* append (:492-540) or "eager add" (:606-665) */
                        slot = l + sx + st;
                        const int64_t ko = ck_base + slot * a->cache_stride[2];
                        copy_row(a->cache_k, ko, a->cache_stride[3], ck, 0, 1, a->HID, es);
                        copy_row(a->cache_v, ko, a->cache_stride[3], cv, 0, 1, a->HID, es);
                        memcpy((char*)a->cache_s + (cs_base + slot * a->cache_s_stride[2]) * es, cs, (size_t)es);
                        a->og_pos[op_base + slot * a->og_pos_stride[2]] = og;
                        a->mask[m_base + slot * a->mask_stride[2]] = 0;
                        stored[i * st_c] = st + 1;
                        break;
                    }
                    /* not accepting and non-empty: compete with the NEWEST slot (:667-726);
                     * (start - 1) floor-mod stored, the formula written at :676 */
                    int64_t r = (sx - 1) % st;
                    if (r < 0) r += st;
                    slot = l + r;
                    const float mine = oracle_load_score(cs, 0, a->dtype);
                    const float old = oracle_load_score(a->cache_s, cs_base + slot * a->cache_s_stride[2], a->dtype);
                    if (mine >= old) { /* :699 */
                        const int64_t ko = ck_base + slot * a->cache_stride[2];
                        copy_row(a->cache_k, ko, a->cache_stride[3], ck, 0, 1, a->HID, es);
                        copy_row(a->cache_v, ko, a->cache_stride[3], cv, 0, 1, a->HID, es);
                        memcpy((char*)a->cache_s + (cs_base + slot * a->cache_s_stride[2]) * es, cs, (size_t)es);
                        a->og_pos[op_base + slot * a->og_pos_stride[2]] = og;
                    }
                    break;
                }
            }

            if (a->K > 0 && last_was_cache) { /* position pass: cascading_cache.py:728-774 */
                int64_t ub = 0;
                for (int64_t i = 0; i < C; i++) ub += stored[i * st_c];
                const int64_t p_base = n * a->pos_stride[0] + h * a->pos_stride[1];
                for (int64_t i = 0; i < C; i++) {
                    const int64_t st = stored[i * st_c], sx = start[i * st_c];
                    const int64_t seg = st < W ? st : W; /* :130 */
                    if (seg <= 0) return ORACLE_ERR_SHAPE;   /* the reference would divide by zero */
                    for (int64_t j = 0; j < W; j++) {     /* :132-142 */
                        a->pos[p_base + (i * W + j) * a->pos_stride[2]] = ((j + seg - sx) % seg) + ub - seg;
                    }
                    ub -= W; /* :770 */
                    if (ub <= 0) break;
                }
            }
        }
    }
    return ORACLE_OK;
}

/* lets the Python face check that its ctypes mirror of oracle_update_desc has the same size */
int64_t ckv_oracle_sizeof_desc(void) { return (int64_t)sizeof(oracle_update_desc); }
