/* CPU oracle for the second cache format — TEST INFRASTRUCTURE, NOT PRODUCT.
 * See v4cache_oracle.h for scope and for what pins each function.
 * Build: with kvcache_oracle.c into libkvoracle.so (oracle/Makefile). */
#include "v4cache_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "kvcache_oracle.h"

static inline uint32_t bits_of(float x) {
    uint32_t b;
    memcpy(&b, &x, sizeof b);
    return b;
}
static inline float float_of(uint32_t b) {
    float x;
    memcpy(&x, &b, sizeof x);
    return x;
}

/* numerics.rs:92-94: past the half always up, at the half only off an odd mantissa. */
static inline int rne_up_f(float rem, float half, int odd) { return rem > half || (rem == half && odd); }
static inline int rne_up_u(uint32_t rem, uint32_t half, int odd) {
    return rem > half || (rem == half && odd);
}

uint8_t ro_e4m3_encode_rne(float x) {
    if (isnan(x)) return 0x7f;
    uint8_t sign = signbit(x) ? 0x80 : 0x00;
    float a = fabsf(x);
    if (a >= 464.0f) return sign | 0x7e;
    if (a <= 1.0f / 1024.0f) return sign;
    uint32_t bits = bits_of(a);
    int e = (int)((bits >> 23) & 0xff) - 127;
    if (e < -6) {
        /* numerics.rs:104-114: value = m * 2^-9; m == 8 promotes to the smallest normal */
        float scaled = a * 512.0f;
        float m = floorf(scaled);
        float rem = scaled - m;
        if (rne_up_f(rem, 0.5f, ((uint32_t)m & 1u) != 0)) m += 1.0f;
        uint32_t mi = (uint32_t)m;
        return mi >= 8 ? (uint8_t)(sign | 0x08) : (uint8_t)(sign | mi);
    }
    /* numerics.rs:118-135 */
    uint32_t mant = bits & 0x007fffffu;
    uint32_t m3 = mant >> 20;
    uint32_t rem = mant & 0x000fffffu;
    if (rne_up_u(rem, 0x00080000u, (m3 & 1u) != 0)) m3 += 1;
    int exp = e + 7;
    if (m3 == 8) {
        m3 = 0;
        exp += 1;
    }
    if (exp >= 15 && m3 >= 7) return sign | 0x7e;
    return (uint8_t)(sign | (uint8_t)(exp << 3) | (uint8_t)m3);
}

void ro_e4m3_encode_rne_n(const float* x, uint8_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ro_e4m3_encode_rne(x[i]);
}

float ro_fast_round_scale(float amax, float max_inv) {
    uint32_t b = bits_of(amax * max_inv);
    int e = (int)((b >> 23) & 0xff) - 127 + ((b & 0x007fffffu) ? 1 : 0);
    return float_of((uint32_t)(e + 127) << 23);
}

int ro_act_quant_f8_prefix(const float* src, float* dst, int rows, int row_stride, int n,
                           int block) {
    if (rows <= 0 || n <= 0 || block <= 0 || row_stride < n) return 1001;
    if (src != dst && n != row_stride) return 1002;
    if (n % block) return 1004;
    const float fp8_max = 448.0f, max_inv = 1.0f / 448.0f;
    for (int r = 0; r < rows; ++r) {
        for (int b = 0; b < n / block; ++b) {
            const float* seg = src + (size_t)r * row_stride + (size_t)b * block;
            float* out = dst + (size_t)r * row_stride + (size_t)b * block;
            float amax = 1e-4f;
            /* f32::max keeps the other operand when one is a NaN, quiet or signaling; libm's
             * fmaxf turns a signaling one into a NaN result, so the compare is spelled out */
            for (int i = 0; i < block; ++i) {
                float a = fabsf(seg[i]);
                if (a > amax) amax = a;
            }
            float s = ro_fast_round_scale(amax, max_inv);
            for (int i = 0; i < block; ++i) {
                float q = seg[i] / s;
                /* comparisons, so that a NaN stays a NaN (actquant.hpp:90-99) */
                q = q < -fp8_max ? -fp8_max : (q > fp8_max ? fp8_max : q);
                out[i] = ro_e4m3_to_f32(ro_e4m3_encode_rne(q)) * s;
            }
        }
    }
    return 0;
}

/* f32::total_cmp's key: the bits as a sign-magnitude integer made two's complement. */
static inline int32_t total_key(float v) {
    int32_t b = (int32_t)bits_of(v);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

typedef struct {
    int32_t key;
    int32_t idx;
} scored_t;

static int by_score_then_index(const void* pa, const void* pb) {
    const scored_t* a = (const scored_t*)pa;
    const scored_t* b = (const scored_t*)pb;
    if (a->key != b->key) return a->key > b->key ? -1 : 1; /* descending score */
    return a->idx < b->idx ? -1 : (a->idx > b->idx ? 1 : 0);
}
static int by_index(const void* pa, const void* pb) {
    int32_t a = ((const scored_t*)pa)->idx, b = ((const scored_t*)pb)->idx;
    return a < b ? -1 : (a > b ? 1 : 0);
}

int ro_v4_scored_rows(const float* scores, int rows, int n_comp, int ratio, int index_topk,
                      int prefill, int offset, int32_t* out) {
    if (!scores || !out || rows <= 0 || n_comp <= 0 || ratio <= 0 || index_topk <= 0) return -1;
    const int k = index_topk < n_comp ? index_topk : n_comp;
    scored_t* sel = (scored_t*)malloc((size_t)n_comp * sizeof(scored_t));
    for (int t = 0; t < rows; ++t) {
        const float* row = scores + (size_t)t * n_comp;
        int limit = n_comp;
        if (prefill) {
            limit = (t + 1) / ratio;
            if (limit > n_comp) limit = n_comp;
        }
        for (int c = 0; c < limit; ++c) {
            sel[c].key = total_key(row[c]);
            sel[c].idx = c;
        }
        qsort(sel, (size_t)limit, sizeof(scored_t), by_score_then_index);
        int kept = limit < k ? limit : k;
        qsort(sel, (size_t)kept, sizeof(scored_t), by_index);
        int32_t* o = out + (size_t)t * k;
        for (int j = 0; j < kept; ++j) o[j] = sel[j].idx + offset;
        for (int j = kept; j < k; ++j) o[j] = -1;
    }
    free(sel);
    return k;
}

static inline float round_bf16(float x) { return ro_bf16_to_f32(ro_f32_to_bf16(x)); }

/* ------------------------------------------------------------------------------------------
 * Selection rectangles, the ring write, the index-list attention
 * ---------------------------------------------------------------------------------------- */

int ro_sel_shape(int win, int ratio, int index_topk, int seqlen, int start_pos, int* rows,
                 int* cols) {
    if (win <= 0 || seqlen <= 0 || start_pos < 0 || ratio < 0 || index_topk < 0) return 1001;
    const int prefill = start_pos == 0;
    if (!prefill && seqlen != 1) return 1005;
    const int q = prefill ? seqlen : 1;
    const int win_cols = prefill ? (seqlen < win ? seqlen : win) : win;
    int n_comp = 0;
    if (ratio > 0) {
        n_comp = (start_pos + q) / ratio;
        if (ratio == 4 && n_comp > index_topk) return 1006;
    }
    if (rows) *rows = q;
    if (cols) *cols = win_cols + n_comp;
    return 0;
}

/* one window cell: select.rs:195-216 */
static int32_t window_cell(int win, int seqlen, int start_pos, int t, int j) {
    if (start_pos == 0) {
        int first = t - (win - 1);
        if (first < 0) first = 0;
        const int v = first + j;
        return v <= t ? v : -1;
    }
    if (start_pos >= win - 1) return (start_pos % win + 1 + j) % win;
    (void)seqlen;
    return j <= start_pos ? j : -1;
}

static void window_fill(int win, int seqlen, int start_pos, int q, int win_cols, int cols,
                        int32_t* out) {
    for (int t = 0; t < q; ++t)
        for (int j = 0; j < win_cols; ++j)
            out[(size_t)t * cols + j] = window_cell(win, seqlen, start_pos, t, j);
}

int ro_sel_gather(int win, int ratio, int index_topk, int seqlen, int start_pos, int32_t* out) {
    int q, cols;
    const int code = ro_sel_shape(win, ratio, index_topk, seqlen, start_pos, &q, &cols);
    if (code) return code;
    if (!out) return 1001;
    const int prefill = start_pos == 0;
    const int win_cols = prefill ? (seqlen < win ? seqlen : win) : win;
    const int offset = prefill ? seqlen : win;
    window_fill(win, seqlen, start_pos, q, win_cols, cols, out);
    for (int t = 0; t < q; ++t)
        for (int c = 0; c < cols - win_cols; ++c) {
            const int legal = prefill ? c < (t + 1) / ratio : 1;
            out[(size_t)t * cols + win_cols + c] = legal ? c + offset : -1;
        }
    return 0;
}

int ro_sel_gather_scored(const float* scores, int n_comp, int win, int ratio, int index_topk,
                         int seqlen, int start_pos, int32_t* out, int* cols_out) {
    if (win <= 0 || seqlen <= 0 || start_pos < 0 || ratio <= 0 || index_topk < 0 || n_comp < 0)
        return 1001;
    const int prefill = start_pos == 0;
    if (!prefill && seqlen != 1) return 1005;
    if (!out || (n_comp > 0 && !scores)) return 1001;
    const int q = prefill ? seqlen : 1;
    const int win_cols = prefill ? (seqlen < win ? seqlen : win) : win;
    const int k = index_topk < n_comp ? index_topk : n_comp;
    const int cols = win_cols + k;
    if (cols_out) *cols_out = cols;
    window_fill(win, seqlen, start_pos, q, win_cols, cols, out);
    if (k > 0) {
        int32_t* comp = (int32_t*)malloc((size_t)q * k * sizeof(int32_t));
        ro_v4_scored_rows(scores, q, n_comp, ratio, index_topk, prefill, prefill ? seqlen : win,
                          comp);
        for (int t = 0; t < q; ++t)
            memcpy(out + (size_t)t * cols + win_cols, comp + (size_t)t * k, (size_t)k * 4);
        free(comp);
    }
    return 0;
}

int ro_ring_write(const float* kv, float* cache, int win, int hd, int seqlen, int start_pos) {
    if (!kv || !cache || win <= 0 || hd <= 0 || seqlen <= 0 || start_pos < 0) return 1001;
    if (start_pos != 0 && seqlen != 1) return 1005;
    const size_t row = (size_t)hd * sizeof(float);
    if (start_pos != 0) {
        memcpy(cache + (size_t)(start_pos % win) * hd, kv, row);
        return 0;
    }
    if (seqlen <= win) {
        memcpy(cache, kv, (size_t)seqlen * row);
        return 0;
    }
    const int cut = seqlen % win;
    memcpy(cache + (size_t)cut * hd, kv + (size_t)(seqlen - win) * hd, (size_t)(win - cut) * row);
    if (cut > 0) memcpy(cache, kv + (size_t)(seqlen - cut) * hd, (size_t)cut * row);
    return 0;
}

int ro_sparse_attn(const float* q, const float* kv, const float* sink, const int32_t* idxs, int m,
                   int h, int d, int topk, float scale, float* o) {
    if (!q || !kv || !sink || !idxs || !o || m <= 0 || h <= 0 || d <= 0 || topk <= 0) return 1001;
    float* logits = (float*)malloc((size_t)topk * sizeof(float));
    float* acc = (float*)malloc((size_t)d * sizeof(float));
    for (int t = 0; t < m; ++t) {
        const int32_t* ix = idxs + (size_t)t * topk;
        for (int hh = 0; hh < h; ++hh) {
            const float* qh = q + ((size_t)t * h + hh) * d;
            float* dst = o + ((size_t)t * h + hh) * d;
            float mx = -INFINITY;
            for (int j = 0; j < topk; ++j) {
                logits[j] = -INFINITY;
                if (ix[j] < 0) continue;
                const float* k = kv + (size_t)ix[j] * d;
                float a = 0.0f;
                for (int i = 0; i < d; ++i) a += qh[i] * k[i];
                const float l = a * scale;
                if (l > mx) mx = l; /* f32::max: a NaN logit loses */
                logits[j] = l;
            }
            if (!isfinite(mx)) {
                for (int i = 0; i < d; ++i) dst[i] = NAN;
                continue;
            }
            float sum = 0.0f;
            for (int i = 0; i < d; ++i) acc[i] = 0.0f;
            for (int j = 0; j < topk; ++j) {
                if (ix[j] < 0) continue;
                const float e = expf(logits[j] - mx);
                sum += e;
                const float* k = kv + (size_t)ix[j] * d;
                for (int i = 0; i < d; ++i) acc[i] += e * k[i];
            }
            sum += expf(sink[hh] - mx);
            for (int i = 0; i < d; ++i) dst[i] = round_bf16(acc[i] / sum);
        }
    }
    free(logits);
    free(acc);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * The compressor's pooling stage
 * ---------------------------------------------------------------------------------------- */


int ro_compress_guard(const ro_comp_geom* p) {
    if (p->ratio <= 1 || p->d <= 0 || p->rd <= 0 || p->coff < 1 || p->coff > 2) return 1001;
    if (p->rd > p->d || (p->rd & 1)) return 1002;
    if (p->cd != p->coff * p->d || p->ents != p->coff * p->ratio) return 1003;
    if (p->ents > 128) return 1004;
    if ((p->coff == 2) != (p->ratio == 4)) return 1010;
    return 0;
}

int ro_kv_compress_deposit(const float* kv, const float* score, const float* ape, float* kv_state,
                           float* score_state, const ro_comp_geom* p, int s, int slot0) {
    if (!p) return 1000;
    int g = ro_compress_guard(p);
    if (g) return g;
    if (s <= 0) return 1005;
    if (slot0 < 0 || slot0 + s % p->ratio > p->ratio) return 1008;
    const int remainder = s % p->ratio, cutoff = s - remainder;
    const int overlap = p->coff == 2;
    const int state_off = overlap ? p->ratio : 0;
    const size_t cd = (size_t)p->cd;
    if (overlap && cutoff >= p->ratio) {
        /* the last complete block is also the next block's overlap half */
        for (size_t i = 0; i < (size_t)p->ratio * cd; ++i) {
            size_t src = (size_t)(cutoff - p->ratio) * cd + i;
            kv_state[i] = kv[src];
            score_state[i] = score[src] + ape[i];
        }
    }
    for (size_t i = 0; i < (size_t)remainder * cd; ++i) {
        size_t src = (size_t)cutoff * cd + i;
        size_t dst = (size_t)(state_off + slot0) * cd + i;
        kv_state[dst] = kv[src];
        score_state[dst] = score[src] + ape[(size_t)slot0 * cd + i]; /* the slot WITHIN its block */
    }
    return 0;
}

/* kvcompress.hip:117-150: softmax over the entries of one feature, then the weighted sum; a
 * null score pointer is a masked entry; a null ape table means it is already in the score. */
static void pool_row(const float* const* kvp, const float* const* scp, const float* const* apep,
                     int ents, int d, float* outrow) {
    for (int e = 0; e < d; ++e) {
        float mx = -INFINITY;
        for (int j = 0; j < ents; ++j) {
            if (!scp[j]) continue;
            mx = fmaxf(mx, scp[j][e] + (apep ? apep[j][e] : 0.0f));
        }
        if (!isfinite(mx)) {
            outrow[e] = 0.0f;
            continue;
        }
        float sum = 0.0f;
        for (int j = 0; j < ents; ++j) {
            if (!scp[j]) continue;
            sum += expf(scp[j][e] + (apep ? apep[j][e] : 0.0f) - mx);
        }
        float acc = 0.0f;
        for (int j = 0; j < ents; ++j) {
            if (!scp[j]) continue;
            acc += kvp[j][e] * (expf(scp[j][e] + (apep ? apep[j][e] : 0.0f) - mx) / sum);
        }
        outrow[e] = acc;
    }
}

/* kvcompress.hip:176-203: bf16 store, RMSNorm (f32 statistic, weight after the scale, bf16
 * store), adjacent-pair rotation of the last rd dims at `pos`, bf16 store. */
static void finish_row(float* row, const float* norm, const float* freqs, int pos,
                       const ro_comp_geom* p) {
    const int d = p->d, rd = p->rd;
    for (int e = 0; e < d; ++e) row[e] = round_bf16(row[e]);
    float ss = 0.0f;
    for (int e = 0; e < d; ++e) ss += row[e] * row[e];
    const float rs = 1.0f / sqrtf(ss / (float)d + p->eps);
    for (int e = 0; e < d; ++e) row[e] = round_bf16(norm[e] * (row[e] * rs));
    const float* t = freqs + (size_t)pos * rd;
    float* seg = row + (d - rd);
    for (int i = 0; i < rd / 2; ++i) {
        float c = t[2 * i], s = t[2 * i + 1];
        float a = seg[2 * i], b = seg[2 * i + 1];
        seg[2 * i] = a * c - b * s;
        seg[2 * i + 1] = a * s + b * c;
    }
    for (int e = 0; e < d; ++e) row[e] = round_bf16(row[e]);
}

int ro_kv_compress_prefill(const float* kv, const float* score, const float* ape,
                           const float* norm, const float* freqs, float* out,
                           const ro_comp_geom* p, int nblk) {
    if (!p || !norm || !freqs || !out) return 1000;
    int g = ro_compress_guard(p);
    if (g) return g;
    if (nblk <= 0) return 1006;
    const int overlap = p->coff == 2;
    const float* kvp[128];
    const float* scp[128];
    const float* apep[128];
    for (int b = 0; b < nblk; ++b) {
        for (int j = 0; j < p->ents; ++j) {
            int sblk, src_j, half;
            if (!overlap) {
                sblk = b, src_j = j, half = 0;
            } else if (j >= p->ratio) {
                sblk = b, src_j = j - p->ratio, half = p->d; /* the block's own rows, "normal" half */
            } else if (b > 0) {
                sblk = b - 1, src_j = j, half = 0; /* the previous block's rows, "overlap" half */
            } else {
                kvp[j] = scp[j] = apep[j] = NULL; /* block 0 has no previous block */
                continue;
            }
            size_t src = (size_t)(sblk * p->ratio + src_j) * p->cd + half;
            kvp[j] = kv + src;
            scp[j] = score + src;
            apep[j] = ape + (size_t)src_j * p->cd + half;
        }
        float* row = out + (size_t)b * p->d;
        pool_row(kvp, scp, apep, p->ents, p->d, row);
        finish_row(row, norm, freqs, b * p->ratio, p);
    }
    return 0;
}

int ro_kv_compress_decode(float* kv_state, float* score_state, const float* norm,
                          const float* freqs, float* out, const ro_comp_geom* p, int start_pos) {
    if (!p || !norm || !freqs || !out) return 1000;
    int g = ro_compress_guard(p);
    if (g) return g;
    if (start_pos <= 0) return 1007;
    if ((start_pos + 1) % p->ratio != 0) return 1009;
    const int overlap = p->coff == 2;
    const float* kvp[128];
    const float* scp[128];
    for (int j = 0; j < p->ents; ++j) {
        int half = (overlap && j >= p->ratio) ? p->d : 0;
        kvp[j] = kv_state + (size_t)j * p->cd + half;
        scp[j] = score_state + (size_t)j * p->cd + half;
    }
    pool_row(kvp, scp, NULL, p->ents, p->d, out);
    finish_row(out, norm, freqs, (start_pos / p->ratio) * p->ratio, p);
    if (overlap) {
        size_t n = (size_t)p->ratio * p->cd;
        for (size_t i = 0; i < n; ++i) {
            kv_state[i] = kv_state[n + i];
            score_state[i] = score_state[n + i];
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * The indexer's spread (Hadamard + simulated fp4) and its block scorer
 * ---------------------------------------------------------------------------------------- */

/* formats.hpp:285-293 / numerics.rs e2m1_encode: the code is the number of midpoints passed;
 * a tie goes up at an odd-indexed midpoint (to the even mantissa). NaN passes none. */
uint8_t ro_e2m1_encode(float x) {
    static const float mid[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    const float a = fabsf(x);
    unsigned code = 0;
    for (int i = 0; i < 7; ++i) code += (a > mid[i] || (a == mid[i] && (i & 1))) ? 1u : 0u;
    return (uint8_t)((signbit(x) ? 8u : 0u) | code);
}

float ro_e2m1_decode(uint8_t c) {
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    const float m = mag[c & 7u];
    return (c & 8u) ? -m : m;
}

/* numerics.rs:324-353: Sylvester (natural-order) butterflies, h = 1, 2, 4, ..., then one
 * multiply by 1 / sqrt(n) with a correctly rounded square root and a true divide. */
void ro_hadamard_rotate(float* row, int n) {
    for (int h = 1; h < n; h *= 2)
        for (int i = 0; i < n; i += 2 * h)
            for (int j = i; j < i + h; ++j) {
                const float a = row[j], b = row[j + h];
                row[j] = a + b;
                row[j + h] = a - b;
            }
    const float scale = 1.0f / sqrtf((float)n);
    for (int i = 0; i < n; ++i) row[i] *= scale;
}

/* numerics.rs:245-298 with the fp4 constants (actquant.hpp:45-51): block amax floored at
 * 6 * 2^-126, scale rounded up to a power of two, clamp by comparisons, e2m1 round trip. */
void ro_fp4_act_quant_inplace(float* row, int n, int block) {
    const float fp4_max = 6.0f;
    const float floor_amax = fp4_max * float_of(1u << 23);
    for (int b0 = 0; b0 < n; b0 += block) {
        const int len = n - b0 < block ? n - b0 : block;
        float amax = 0.0f;
        for (int i = 0; i < len; ++i) amax = fmaxf(amax, fabsf(row[b0 + i]));
        amax = fmaxf(amax, floor_amax);
        const float s = ro_fast_round_scale(amax, 1.0f / fp4_max);
        for (int i = 0; i < len; ++i) {
            float q = row[b0 + i] / s;
            q = q < -fp4_max ? -fp4_max : (q > fp4_max ? fp4_max : q);
            row[b0 + i] = ro_e2m1_decode(ro_e2m1_encode(q)) * s;
        }
    }
}

/* blockindex.hip:99-136 behind the launcher's guards (:241-262): rotate, store as bf16,
 * quantize in blocks of 32, store as bf16 — the order of kernel_v4_indexer.rs:149-156. */
int ro_act_quant_f4_rotated(float* x, int rows, int d) {
    if (rows <= 0 || d <= 0) return 1001;
    if (d > 256) return 1002;
    if (d & (d - 1)) return 1003;
    if (d % 32) return 1004;
    for (int r = 0; r < rows; ++r) {
        float* row = x + (size_t)r * d;
        ro_hadamard_rotate(row, d);
        for (int i = 0; i < d; ++i) row[i] = round_bf16(row[i]);
        ro_fp4_act_quant_inplace(row, d, 32);
        for (int i = 0; i < d; ++i) row[i] = round_bf16(row[i]);
    }
    return 0;
}

/* blockindex.hip:209-235 (and kernel_v4_indexer.rs:437-462, the same fold on the host) behind
 * the launcher's guards (:264-281). q: [s][heads][hd]; kv: [n_comp][hd]; w: [s][heads];
 * score: [s][n_comp]. Products and sums are separate roundings (this file is built with
 * -ffp-contract=off); the head sum is carried in f32 and rounded to bf16 once. */
int ro_index_score_blocks(const float* q, const float* kv, const float* w, float* score, int s,
                          int n_comp, int heads, int hd) {
    if (s <= 0 || heads <= 0 || hd <= 0) return 1001;
    if (n_comp <= 0) return 1005;
    for (int t = 0; t < s; ++t)
        for (int c = 0; c < n_comp; ++c) {
            const float* kvr = kv + (size_t)c * hd;
            float acc = 0.0f;
            for (int hh = 0; hh < heads; ++hh) {
                const float* qh = q + ((size_t)t * heads + hh) * hd;
                float dot = 0.0f;
                for (int i = 0; i < hd; ++i) {
                    const float prod = qh[i] * kvr[i];
                    dot = dot + prod;
                }
                dot = round_bf16(dot);
                dot = dot > 0.0f ? dot : 0.0f;  /* the sign of a zero cannot reach the output */
                const float term = dot * w[(size_t)t * heads + hh];
                acc = acc + round_bf16(term);
            }
            score[(size_t)t * n_comp + c] = round_bf16(acc);
        }
    return 0;
}
