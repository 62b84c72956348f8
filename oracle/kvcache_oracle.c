/* CPU oracle for the fp8 MLA KV-cache path — TEST INFRASTRUCTURE, NOT PRODUCT.
 * See kvcache_oracle.h for scope and for what pins each function.
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared -pthread (oracle/Makefile). */
#include "kvcache_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f32_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, sizeof b);
    return b;
}
static inline float bits_f32(uint32_t b) {
    float x;
    memcpy(&x, &b, sizeof x);
    return x;
}

/* ------------------------------------------------------------------------------------------
 * Element codecs
 * ---------------------------------------------------------------------------------------- */

/* crates/core/src/num.rs:157-182 (e4m3_normal): a in [2^-6, 448). */
static uint8_t e4m3_normal(float a) {
    uint32_t bits = f32_bits(a);
    int e = (int)((bits >> 23) & 0xff) - 127;
    uint32_t mant = bits & 0x007fffffu;
    uint32_t m3 = mant >> 20;
    uint32_t rem = mant & 0x000fffffu;
    /* nearest even over the 20 dropped bits; 0x80000 is the exact half */
    if (rem > 0x00080000u || (rem == 0x00080000u && (m3 & 1u))) m3 += 1;
    int exp = e + 7;
    if (m3 == 8) {
        m3 = 0;
        exp += 1;
    }
    if (exp >= 15 && m3 >= 7) return 0x7e;
    return (uint8_t)(((uint32_t)exp << 3) | m3);
}

/* crates/core/src/num.rs:128-152. Normals round to nearest even, the subnormal band rounds
 * half AWAY from zero (Rust's f32::round), magnitudes >= 448 saturate to 0x7e, NaN -> 0x7f. */
uint8_t ro_f32_to_e4m3(float x) {
    if (isnan(x)) return 0x7f;
    uint8_t sign = (f32_bits(x) >> 31) ? 0x80 : 0;
    float a = fabsf(x);
    if (a >= 448.0f) return sign | 0x7e;
    if (a < 0.0009765625f) return sign; /* < 2^-10: below half the smallest subnormal */
    if (a < 0.015625f) {                /* < 2^-6: subnormal, value = m/8 * 2^-6 */
        /* a*512 is exact (power-of-two scale of a normal f32); roundf is half-away. */
        uint32_t m = (uint32_t)roundf(a * 512.0f);
        return m >= 8 ? (sign | 0x08) : (uint8_t)(sign | m);
    }
    return sign | e4m3_normal(a);
}

/* crates/core/src/num.rs:189-201. Exact. Both NaN codes give the positive quiet NaN. */
float ro_e4m3_to_f32(uint8_t b) {
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int exp = (b >> 3) & 0x0f;
    float mant = (float)(b & 0x07);
    if (exp == 0) return sign * (mant / 8.0f) * 0.015625f;
    if (exp == 15 && mant == 7.0f) return bits_f32(0x7fc00000u);
    return sign * (1.0f + mant / 8.0f) * ldexpf(1.0f, exp - 7);
}

/* crates/core/src/num.rs:86-88 delegates to crate `half` 2.7.1 (Cargo.lock:477-478, source not
 * vendored). half's published bf16::from_f32: a NaN keeps its high half with the quiet bit
 * forced; otherwise round to nearest even — up iff the round bit is set and (sticky or lsb). */
uint16_t ro_f32_to_bf16(float x) {
    uint32_t b = f32_bits(x);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    uint32_t round_bit = 0x00008000u;
    if ((b & round_bit) != 0 && (b & (3u * round_bit - 1u)) != 0) return (uint16_t)((b >> 16) + 1u);
    return (uint16_t)(b >> 16);
}

/* crates/core/src/num.rs:93-96: bf16 is the high half of an f32. */
float ro_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

void ro_f32_to_e4m3_n(const float* x, uint8_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ro_f32_to_e4m3(x[i]);
}
void ro_e4m3_to_f32_n(const uint8_t* c, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ro_e4m3_to_f32(c[i]);
}
void ro_f32_to_bf16_n(const float* x, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ro_f32_to_bf16(x[i]);
}

uint64_t ro_selftest_bf16_exhaustive(void) {
    uint64_t bad = 0;
    for (uint64_t u = 0; u <= 0xffffffffull; ++u) {
        uint32_t b = (uint32_t)u;
        if ((b & 0x7fffffffu) > 0x7f800000u) continue; /* NaN: not RNE's business */
        uint16_t textbook = (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
        if (ro_f32_to_bf16(bits_f32(b)) != textbook) ++bad;
    }
    return bad;
}

/* ------------------------------------------------------------------------------------------
 * The reference tests' deterministic input stream
 * ---------------------------------------------------------------------------------------- */

/* crates/engine/tests/common/reference.rs:155-161. `as f32` of a u64 < 2^32 rounds to nearest
 * even; u32::MAX as f32 is 2^32. */
float ro_lcg_f(uint64_t* state) {
    *state = *state * 6364136223846793005ull + 1442695040888963407ull;
    float hi = (float)(uint32_t)(*state >> 32);
    return (hi / 4294967296.0f) * 2.0f - 1.0f;
}
void ro_lcg_fill(uint64_t* state, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ro_lcg_f(state);
}

/* ------------------------------------------------------------------------------------------
 * Scale rule and quantization
 * ---------------------------------------------------------------------------------------- */

/* crates/engine/tests/fwd_kernel.rs:164-171: amax = fold(0, max(m, |v|)) — f32::max drops a
 * NaN operand, as fmaxf does; scl = amax > 0 ? amax/448 : 1; code = enc(v / scl). */
void ro_quant_block(const float* v, int n, uint8_t* codes, float* scale) {
    float amax = 0.0f;
    for (int i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(v[i]));
    float scl = amax > 0.0f ? amax / 448.0f : 1.0f;
    *scale = scl;
    for (int i = 0; i < n; ++i) codes[i] = ro_f32_to_e4m3(v[i] / scl);
}

/* crates/backend/kernels/fwd.hip:51-71 + launcher guards :224-229. */
int ro_append_kv(const float* latent, const float* rope, uint8_t* lc8, float* lscale,
                 uint16_t* rc, int pos, int kvl, int ropn, int n_blocks) {
    if (pos < 0 || kvl <= 0 || ropn <= 0 || n_blocks <= 0) return 1001;
    if (kvl > 1024 || kvl < 128 || (kvl % 128) != 0 || ropn > kvl) return 1002;
    for (int b = 0; b < kvl / 128; ++b) {
        ro_quant_block(latent + b * 128, 128, lc8 + (size_t)pos * kvl + b * 128,
                       lscale + (size_t)pos * n_blocks + b);
    }
    for (int i = 0; i < ropn; ++i) rc[(size_t)pos * ropn + i] = ro_f32_to_bf16(rope[i]);
    return 0;
}

/* crates/backend/kernels/indexer.hip:54-58 + guard :270. */
int ro_index_append(const float* k, uint16_t* kcache, int pos, int hd) {
    if (hd <= 0 || pos < 0) return 1001;
    for (int i = 0; i < hd; ++i) kcache[(size_t)pos * hd + i] = ro_f32_to_bf16(k[i]);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Indexer scores
 * ---------------------------------------------------------------------------------------- */

/* One token's score in the host reference's order (crates/engine/tests/indexer_kernel.rs:
 * 240-249): per head a left fold of q*k products, then acc + w*wscale*max(dot*dscale, 0). */
static float score_one(const float* q, const float* w, const uint16_t* krow,
                       const uint32_t* heads, int nact, int hd, float wscale, float dscale) {
    float acc = 0.0f;
    for (int a = 0; a < nact; ++a) {
        int h = heads ? (int)heads[a] : a;
        const float* qh = q + (size_t)h * hd;
        float dot = 0.0f;
        for (int i = 0; i < hd; ++i) dot += qh[i] * ro_bf16_to_f32(krow[i]);
        acc = acc + w[h] * wscale * fmaxf(dot * dscale, 0.0f);
    }
    return acc;
}

int ro_index_score(const float* q, const float* w, const uint16_t* kcache, const uint32_t* heads,
                   int nt, int nh, int nact, int hd, float wscale, float dscale, float* scores) {
    if (nt <= 0 || nh <= 0 || nact <= 0 || nact > nh || hd <= 0) return 1001;
    for (int t = 0; t < nt; ++t)
        scores[t] = score_one(q, w, kcache + (size_t)t * hd, heads, nact, hd, wscale, dscale);
    return 0;
}

int ro_index_append_paged(const float* k, const int32_t* slot_mapping, uint16_t* kpool,
                          int n_tokens, int hd, int page_tokens, int n_pages) {
    int bad = 0;
    for (int t = 0; t < n_tokens; ++t) {
        int32_t slot = slot_mapping[t];
        if (slot < 0) continue;
        if ((int64_t)slot >= (int64_t)n_pages * page_tokens) {
            ++bad;
            continue;
        }
        for (int i = 0; i < hd; ++i)
            kpool[(size_t)slot * hd + i] = ro_f32_to_bf16(k[(size_t)t * hd + i]);
    }
    return bad;
}

typedef struct {
    const float *q, *w;
    const uint16_t* kpool;
    const int32_t *block_table, *nts;
    const uint32_t* heads;
    float* scores;
    int n_queries, max_blocks_per_seq, stride, nh, nact, hd, page_tokens, tid, n_threads;
    float wscale, dscale;
} score_job;

static void* score_worker(void* p) {
    score_job* j = (score_job*)p;
    long item = 0;
    for (int qi = 0; qi < j->n_queries; ++qi) {
        const float* q = j->q + (size_t)qi * j->nh * j->hd;
        const float* w = j->w + (size_t)qi * j->nh;
        for (int t = 0; t < j->nts[qi]; ++t, ++item) {
            if ((item >> 6) % j->n_threads != j->tid) continue; /* 64-token slices per thread */
            int page = j->block_table[(size_t)qi * j->max_blocks_per_seq + t / j->page_tokens];
            size_t slot = (size_t)page * j->page_tokens + (size_t)(t % j->page_tokens);
            j->scores[(size_t)qi * j->stride + t] = score_one(
                q, w, j->kpool + slot * j->hd, j->heads, j->nact, j->hd, j->wscale, j->dscale);
        }
    }
    return NULL;
}

void ro_index_score_paged(const float* q, const float* w, const uint16_t* kpool,
                          const int32_t* block_table, const int32_t* nts, const uint32_t* heads,
                          int n_queries, int max_blocks_per_seq, int stride, int nh, int nact,
                          int hd, int page_tokens, float wscale, float dscale, float* scores,
                          int n_threads) {
    if (n_threads < 1) n_threads = 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n_threads);
    score_job* jobs = (score_job*)malloc(sizeof(score_job) * (size_t)n_threads);
    for (int i = 0; i < n_threads; ++i) {
        score_job j = {q, w, kpool, block_table, nts, heads, scores, n_queries,
                       max_blocks_per_seq, stride, nh, nact, hd, page_tokens, i, n_threads,
                       wscale, dscale};
        jobs[i] = j;
        pthread_create(&th[i], NULL, score_worker, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

/* ------------------------------------------------------------------------------------------
 * Paged cache, one scale per token
 * ---------------------------------------------------------------------------------------- */

size_t ro_kv_page_bytes(int page_tokens, int width) {
    return (size_t)page_tokens * (size_t)width + (size_t)page_tokens * sizeof(float);
}

static void append_range(const uint16_t* rows, const int32_t* slot_mapping, uint8_t* pool,
                         int t0, int t1, int width, int page_tokens, int n_pages, int* bad) {
    size_t page_bytes = ro_kv_page_bytes(page_tokens, width);
    float* v = (float*)malloc((size_t)width * sizeof(float));
    for (int t = t0; t < t1; ++t) {
        int32_t slot = slot_mapping[t];
        if (slot < 0) continue;
        if ((int64_t)slot >= (int64_t)n_pages * page_tokens) {
            ++*bad;
            continue;
        }
        int page = slot / page_tokens, off = slot % page_tokens;
        uint8_t* pg = pool + (size_t)page * page_bytes;
        for (int i = 0; i < width; ++i) v[i] = ro_bf16_to_f32(rows[(size_t)t * width + i]);
        float scl;
        ro_quant_block(v, width, pg + (size_t)off * width, &scl);
        memcpy(pg + (size_t)page_tokens * width + (size_t)off * sizeof(float), &scl, sizeof scl);
    }
    free(v);
}

int ro_kv_append_paged(const uint16_t* rows, const int32_t* slot_mapping, uint8_t* pool,
                       int n_tokens, int width, int page_tokens, int n_pages) {
    int bad = 0;
    append_range(rows, slot_mapping, pool, 0, n_tokens, width, page_tokens, n_pages, &bad);
    return bad;
}

/* One token: crates/backend/kernels/attn.hip:176 (code * scale in f32), then RNE to bf16. */
static inline void dequant_row(const uint8_t* pg, int off, int width, int page_tokens,
                               const float* lut, uint16_t* out) {
    float scl;
    memcpy(&scl, pg + (size_t)page_tokens * width + (size_t)off * sizeof(float), sizeof scl);
    const uint8_t* c = pg + (size_t)off * width;
    for (int i = 0; i < width; ++i) out[i] = ro_f32_to_bf16(lut[c[i]] * scl);
}

static void decode_table(float* lut) {
    for (int c = 0; c < 256; ++c) lut[c] = ro_e4m3_to_f32((uint8_t)c);
}

static void gather_seq_range(const uint8_t* pool, const int32_t* block_table,
                             const int32_t* seq_lens, const int32_t* cu_seqlens, uint16_t* out,
                             int s0, int s1, int max_blocks_per_seq, int width,
                             int page_tokens) {
    float lut[256];
    decode_table(lut);
    size_t page_bytes = ro_kv_page_bytes(page_tokens, width);
    for (int s = s0; s < s1; ++s) {
        for (int t = 0; t < seq_lens[s]; ++t) {
            int page = block_table[(size_t)s * max_blocks_per_seq + t / page_tokens];
            dequant_row(pool + (size_t)page * page_bytes, t % page_tokens, width, page_tokens,
                        lut, out + ((size_t)cu_seqlens[s] + t) * width);
        }
    }
}

void ro_kv_gather_paged(const uint8_t* pool, const int32_t* block_table, const int32_t* seq_lens,
                        const int32_t* cu_seqlens, uint16_t* out, int n_seqs,
                        int max_blocks_per_seq, int width, int page_tokens) {
    gather_seq_range(pool, block_table, seq_lens, cu_seqlens, out, 0, n_seqs,
                     max_blocks_per_seq, width, page_tokens);
}

void ro_kv_gather_rows_paged(const uint8_t* pool, const int32_t* block_table,
                             const uint32_t* rows, const int32_t* n_rows, uint16_t* out,
                             int n_queries, int k, int max_blocks_per_seq, int width,
                             int page_tokens) {
    float lut[256];
    decode_table(lut);
    size_t page_bytes = ro_kv_page_bytes(page_tokens, width);
    for (int q = 0; q < n_queries; ++q) {
        int nr = n_rows ? n_rows[q] : k;
        for (int j = 0; j < nr; ++j) {
            uint32_t t = rows[(size_t)q * k + j];
            int page = block_table[(size_t)q * max_blocks_per_seq + t / (uint32_t)page_tokens];
            dequant_row(pool + (size_t)page * page_bytes, (int)(t % (uint32_t)page_tokens), width,
                        page_tokens, lut, out + ((size_t)q * k + j) * width);
        }
    }
}

/* ---- host-thread fan-out, for timing the CPU path on all cores ---- */

typedef struct {
    const uint8_t* pool;
    const int32_t *block_table, *seq_lens, *cu_seqlens;
    uint16_t* out;
    int n_seqs, max_blocks_per_seq, width, page_tokens, tid, n_threads;
} gather_job;

/* Pages, not sequences, are dealt round-robin so uneven contexts still balance. */
static void* gather_worker(void* p) {
    gather_job* j = (gather_job*)p;
    float lut[256];
    decode_table(lut);
    size_t page_bytes = ro_kv_page_bytes(j->page_tokens, j->width);
    long item = 0;
    for (int s = 0; s < j->n_seqs; ++s) {
        int n_blocks = (j->seq_lens[s] + j->page_tokens - 1) / j->page_tokens;
        for (int b = 0; b < n_blocks; ++b, ++item) {
            if (item % j->n_threads != j->tid) continue;
            int page = j->block_table[(size_t)s * j->max_blocks_per_seq + b];
            int t0 = b * j->page_tokens;
            int t1 = t0 + j->page_tokens < j->seq_lens[s] ? t0 + j->page_tokens : j->seq_lens[s];
            for (int t = t0; t < t1; ++t)
                dequant_row(j->pool + (size_t)page * page_bytes, t - t0, j->width,
                            j->page_tokens, lut,
                            j->out + ((size_t)j->cu_seqlens[s] + t) * j->width);
        }
    }
    return NULL;
}

void ro_kv_gather_paged_mt(const uint8_t* pool, const int32_t* block_table,
                           const int32_t* seq_lens, const int32_t* cu_seqlens, uint16_t* out,
                           int n_seqs, int max_blocks_per_seq, int width, int page_tokens,
                           int n_threads) {
    if (n_threads < 1) n_threads = 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n_threads);
    gather_job* jobs = (gather_job*)malloc(sizeof(gather_job) * (size_t)n_threads);
    for (int i = 0; i < n_threads; ++i) {
        gather_job j = {pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                        max_blocks_per_seq, width, page_tokens, i, n_threads};
        jobs[i] = j;
        pthread_create(&th[i], NULL, gather_worker, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

typedef struct {
    const uint16_t* rows;
    const int32_t* slot_mapping;
    uint8_t* pool;
    int t0, t1, width, page_tokens, n_pages, bad;
} append_job;

static void* append_worker(void* p) {
    append_job* j = (append_job*)p;
    append_range(j->rows, j->slot_mapping, j->pool, j->t0, j->t1, j->width, j->page_tokens,
                 j->n_pages, &j->bad);
    return NULL;
}

void ro_kv_append_paged_mt(const uint16_t* rows, const int32_t* slot_mapping, uint8_t* pool,
                           int n_tokens, int width, int page_tokens, int n_pages,
                           int n_threads) {
    if (n_threads < 1) n_threads = 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n_threads);
    append_job* jobs = (append_job*)malloc(sizeof(append_job) * (size_t)n_threads);
    for (int i = 0; i < n_threads; ++i) {
        long a = (long)n_tokens * i / n_threads, b = (long)n_tokens * (i + 1) / n_threads;
        append_job j = {rows, slot_mapping, pool, (int)a, (int)b, width, page_tokens, n_pages, 0};
        jobs[i] = j;
        pthread_create(&th[i], NULL, append_worker, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

/* ------------------------------------------------------------------------------------------
 * Selection
 * ---------------------------------------------------------------------------------------- */

/* ---- MLA decode attention in latent space ------------------------------------------------
 * The dense two-pass scalar softmax the reference's flash kernel is checked against:
 * crates/engine/tests/kernel_attend.rs:201-226 (attend_reference) with
 * crates/core/src/routing.rs:10-22 (softmax). `lat` is [nr][kvl] and `rk` is [nr][rope], both
 * already widened to f32 the way the kernel widens them; one running f32 sum per score,
 * latent terms then roped ones, times `scale`; out[h][i] += p_t * lat[t][i] in token order. */
void ro_mla_attend_dense(const float* qabs, const float* qrope, const float* lat, const float* rk,
                         int H, int nr, int kvl, int rope, float scale, float* clat) {
    float* scores = (float*)malloc(sizeof(float) * (size_t)(nr > 0 ? nr : 1));
    for (int h = 0; h < H; ++h) {
        const float* qa = qabs + (size_t)h * kvl;
        const float* qr = qrope + (size_t)h * rope;
        float* out = clat + (size_t)h * kvl;
        for (int i = 0; i < kvl; ++i) out[i] = 0.0f;
        float mx = -INFINITY;
        for (int t = 0; t < nr; ++t) {
            float sum = 0.0f;
            for (int i = 0; i < kvl; ++i) sum += qa[i] * lat[(size_t)t * kvl + i];
            for (int d = 0; d < rope; ++d) sum += qr[d] * rk[(size_t)t * rope + d];
            scores[t] = sum * scale;
            if (scores[t] > mx) mx = scores[t];
        }
        float den = 0.0f;
        for (int t = 0; t < nr; ++t) {
            scores[t] = expf(scores[t] - mx);
            den += scores[t];
        }
        if (den > 0.0f)
            for (int t = 0; t < nr; ++t) scores[t] /= den;
        for (int t = 0; t < nr; ++t)
            for (int i = 0; i < kvl; ++i) out[i] += scores[t] * lat[(size_t)t * kvl + i];
    }
    free(scores);
}

/* The reference's cache layout and launcher (crates/backend/kernels/attn.hip:168-183,279-293):
 * latent e4m3 with one f32 scale per 128 values, roped key bf16, token = rows ? rows[j] : j. */
int ro_mla_attend(const float* qabs, const float* qrope, const uint8_t* lc8, const float* lscale,
                  const uint16_t* rc, const uint32_t* rows, int H, int nr, int kvl, int rope,
                  int n_blocks, float scale, float* clat) {
    if (H <= 0 || nr <= 0 || kvl <= 0 || rope <= 0 || n_blocks <= 0) return 1001;
    if (kvl > 512 || kvl % 128) return 1004;
    float* lat = (float*)malloc(sizeof(float) * (size_t)nr * kvl);
    float* rk = (float*)malloc(sizeof(float) * (size_t)nr * rope);
    for (int j = 0; j < nr; ++j) {
        size_t t = rows ? rows[j] : (size_t)j;
        for (int i = 0; i < kvl; ++i)
            lat[(size_t)j * kvl + i] = ro_e4m3_to_f32(lc8[t * kvl + i]) * lscale[t * n_blocks + i / 128];
        for (int d = 0; d < rope; ++d) rk[(size_t)j * rope + d] = ro_bf16_to_f32(rc[t * rope + d]);
    }
    ro_mla_attend_dense(qabs, qrope, lat, rk, H, nr, kvl, rope, scale, clat);
    free(lat);
    free(rk);
    return 0;
}

/* The paged cache of this build: a token is kvl + rope e4m3 codes under ONE f32 scale, so both
 * halves widen as e4m3_to_f32(code) * scale. Sequence s attends rows[s*k + j] for
 * j < n_rows[s] (k when null) if rows is given, else tokens 0..seq_lens[s]-1. */
static void attend_paged_seq(const float* qabs, const float* qrope, const uint8_t* pool,
                             const int32_t* block_table, const int32_t* seq_lens,
                             const uint32_t* rows, const int32_t* n_rows, int k, int s, int H,
                             int max_blocks_per_seq, int kvl, int rope, int page_tokens,
                             float scale, float* clat) {
    const int width = kvl + rope;
    const size_t page_bytes = ro_kv_page_bytes(page_tokens, width);
    const int nr = rows ? (n_rows ? n_rows[s] : k) : seq_lens[s];
    float* out = clat + (size_t)s * H * kvl;
    if (nr <= 0) {
        for (size_t i = 0; i < (size_t)H * kvl; ++i) out[i] = 0.0f;
        return;
    }
    float* lat = (float*)malloc(sizeof(float) * (size_t)nr * kvl);
    float* rk = (float*)malloc(sizeof(float) * (size_t)nr * rope);
    for (int j = 0; j < nr; ++j) {
        uint32_t t = rows ? rows[(size_t)s * k + j] : (uint32_t)j;
        int page = block_table[(size_t)s * max_blocks_per_seq + t / (uint32_t)page_tokens];
        int off = (int)(t % (uint32_t)page_tokens);
        const uint8_t* pg = pool + (size_t)page * page_bytes;
        float scl;
        memcpy(&scl, pg + (size_t)page_tokens * width + (size_t)off * 4, 4);
        const uint8_t* codes = pg + (size_t)off * width;
        for (int i = 0; i < kvl; ++i) lat[(size_t)j * kvl + i] = ro_e4m3_to_f32(codes[i]) * scl;
        for (int d = 0; d < rope; ++d) rk[(size_t)j * rope + d] = ro_e4m3_to_f32(codes[kvl + d]) * scl;
    }
    ro_mla_attend_dense(qabs + (size_t)s * H * kvl, qrope + (size_t)s * H * rope, lat, rk, H, nr,
                        kvl, rope, scale, out);
    free(lat);
    free(rk);
}

typedef struct {
    const float *qabs, *qrope;
    const uint8_t* pool;
    const int32_t *block_table, *seq_lens;
    const uint32_t* rows;
    const int32_t* n_rows;
    int k, n_seqs, H, max_blocks_per_seq, kvl, rope, page_tokens;
    float scale;
    float* clat;
    int tid, n_threads;
} attend_job;

static void* attend_worker(void* p) {
    attend_job* j = (attend_job*)p;
    for (int s = j->tid; s < j->n_seqs; s += j->n_threads)
        attend_paged_seq(j->qabs, j->qrope, j->pool, j->block_table, j->seq_lens, j->rows,
                         j->n_rows, j->k, s, j->H, j->max_blocks_per_seq, j->kvl, j->rope,
                         j->page_tokens, j->scale, j->clat);
    return NULL;
}

void ro_mla_attend_paged(const float* qabs, const float* qrope, const uint8_t* pool,
                         const int32_t* block_table, const int32_t* seq_lens,
                         const uint32_t* rows, const int32_t* n_rows, int k, int n_seqs, int H,
                         int max_blocks_per_seq, int kvl, int rope, int page_tokens, float scale,
                         float* clat, int n_threads) {
    if (n_threads < 1) n_threads = 1;
    if (n_threads > n_seqs) n_threads = n_seqs;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n_threads);
    attend_job* jobs = (attend_job*)malloc(sizeof(attend_job) * (size_t)n_threads);
    for (int i = 0; i < n_threads; ++i) {
        attend_job j = {qabs, qrope, pool, block_table, seq_lens, rows, n_rows, k, n_seqs, H,
                        max_blocks_per_seq, kvl, rope, page_tokens, scale, clat, i, n_threads};
        jobs[i] = j;
        pthread_create(&th[i], NULL, attend_worker, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

/* qsort has no closure argument; selection is only ever run from one thread per array, and
 * the batched form gives each worker its own copy through thread-local storage. */
static __thread const float* g_scores;

/* crates/core/src/routing.rs:50-55: value descending (partial_cmp, so -0.0 == +0.0), index
 * ascending. NaN is out of contract on both sides. */
static int cmp_desc_then_index(const void* pa, const void* pb) {
    uint32_t a = *(const uint32_t*)pa, b = *(const uint32_t*)pb;
    float sa = g_scores[a], sb = g_scores[b];
    if (sb < sa) return -1;
    if (sb > sa) return 1;
    return a < b ? -1 : (a > b ? 1 : 0);
}
static int cmp_u32(const void* pa, const void* pb) {
    uint32_t a = *(const uint32_t*)pa, b = *(const uint32_t*)pb;
    return a < b ? -1 : (a > b ? 1 : 0);
}

/* The comparator is a total order on NaN-free input, so the first-k SET is unique and a full
 * sort selects exactly what select_nth_unstable_by + truncate does. */
int ro_topk(const float* scores, int nt, int k, uint32_t* rows) {
    if (nt <= 0 || k <= 0) return 0;
    if (k > nt) k = nt;
    uint32_t* idx = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)nt);
    for (int i = 0; i < nt; ++i) idx[i] = (uint32_t)i;
    g_scores = scores;
    qsort(idx, (size_t)nt, sizeof(uint32_t), cmp_desc_then_index);
    qsort(idx, (size_t)k, sizeof(uint32_t), cmp_u32);
    memcpy(rows, idx, sizeof(uint32_t) * (size_t)k);
    free(idx);
    return k;
}

typedef struct {
    const float* scores;
    const int32_t* nts;
    uint32_t* rows;
    int n_queries, stride, nt, k, tid, n_threads;
} topk_job;

static void* topk_worker(void* p) {
    topk_job* j = (topk_job*)p;
    for (int q = j->tid; q < j->n_queries; q += j->n_threads)
        ro_topk(j->scores + (size_t)q * j->stride, j->nts ? j->nts[q] : j->nt, j->k,
                j->rows + (size_t)q * j->k);
    return NULL;
}

void ro_topk_batched(const float* scores, int n_queries, int stride, const int32_t* nts, int nt,
                     int k, uint32_t* rows, int n_threads) {
    if (n_threads < 1) n_threads = 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n_threads);
    topk_job* jobs = (topk_job*)malloc(sizeof(topk_job) * (size_t)n_threads);
    for (int i = 0; i < n_threads; ++i) {
        topk_job j = {scores, nts, rows, n_queries, stride, nt, k, i, n_threads};
        jobs[i] = j;
        pthread_create(&th[i], NULL, topk_worker, &jobs[i]);
    }
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
    free(jobs);
    free(th);
}

/* ------------------------------------------------------------------------------------------
 * Content pinning
 * ---------------------------------------------------------------------------------------- */

/* crates/core/src/hash.rs:9-24 */
uint64_t ro_fnv1a(const uint8_t* bytes, size_t n) {
    uint64_t h = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < n; ++i) h = (h ^ (uint64_t)bytes[i]) * 0x00000100000001b3ull;
    return h;
}

/* crates/core/src/hash.rs:52-56 */
uint64_t ro_splitmix_finalize(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* crates/core/src/hash.rs:68-112: XOR over every stride-th 32-bit word of
 * finalize(((i_base + i) << 32) ^ bits), i the element index. */
uint64_t ro_xor_fold(const uint32_t* words, size_t n, uint64_t i_base, size_t stride) {
    uint64_t h = 0;
    if (stride == 0) return 0;
    for (size_t i = 0; i < n; i += stride)
        h ^= ro_splitmix_finalize(((i_base + (uint64_t)i) << 32) ^ (uint64_t)words[i]);
    return h;
}
