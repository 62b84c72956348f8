/* CPU oracle for the fp8 MLA KV-cache path — TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A plain-C restatement of the reference's CPU arithmetic for this path. Only tests, the
 * smoke check and the benchmark's CPU-baseline leg may link or call it; the shipped library
 * never does. Every function names the reference lines it follows (paths are relative to the
 * reference tree).
 *
 * Pinning status (what checks each function besides itself — see tests/test_oracle_*.py):
 *   ro_f32_to_e4m3      KATs crates/core/src/routing.rs:338-362; independent nearest-value
 *                       brute force; enc(dec(c))==c; monotone; subnormal tie KATs
 *   ro_e4m3_to_f32      closed form over all 256 codes; same KATs
 *   ro_f32_to_bf16      KATs crates/core/src/routing.rs:259-284; exhaustive 2^32 vs the
 *                       textbook integer RNE (ro_selftest_bf16_exhaustive)
 *   ro_quant_block      test restatement crates/engine/tests/fwd_kernel.rs:162-171; the
 *                       0xA99E fixture's documented block amaxes (0.9949 / 19.9455);
 *                       invariants (amax -> 0x7e, zero row, power-of-two scaling)
 *   ro_topk             KAT crates/core/src/routing.rs:207-212; brute-force lexsort
 *   ro_xor_fold         published splitmix64 sequence crates/core/src/hash.rs:248-259
 *   ro_fnv1a            published FNV-1a vectors crates/core/src/hash.rs:121-125
 *   ro_lcg_f            documented fixture values (block amaxes above)
 *   paged addressing    NEW in this build (the reference has a linear slab): pinned by
 *                       identity-table equivalence with the linear slab and by permutation
 *                       invariance, not by any reference test
 *   ro_index_score      float64 restatement within 1e-6 of the scale; the reference test's
 *                       own separation property (head subset [5,0,6,2] vs all heads > 1e-2);
 *                       single-head / all-negative closed forms
 *   ro_mla_attend*      float64 restatement (numpy) within 1e-5 of the largest output; closed
 *                       forms (equal scores -> the mean row, one dominant score -> that row,
 *                       one row -> itself); the paged form against the linear form on the
 *                       same widened rows. The reference's own expectation for this kernel
 *                       is computed at test time by this same formula (no stored vectors).
 *   ro_kv_gather_rows   parity unpinned by reference tests (no reference test passes
 *                       rows != null, crates/engine/tests/kernel_attend.rs:114); pinned
 *                       here by gather_rows(rows) == gather_dense()[rows]
 */
#ifndef RIVOLI_KVCACHE_ORACLE_H
#define RIVOLI_KVCACHE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- element codecs: crates/core/src/num.rs:86-201 ---- */
uint8_t ro_f32_to_e4m3(float x);
float ro_e4m3_to_f32(uint8_t b);
uint16_t ro_f32_to_bf16(float x);
float ro_bf16_to_f32(uint16_t b);
void ro_f32_to_e4m3_n(const float* x, uint8_t* out, size_t n);
void ro_e4m3_to_f32_n(const uint8_t* c, float* out, size_t n);
void ro_f32_to_bf16_n(const float* x, uint16_t* out, size_t n);
/* Exhaustive check of ro_f32_to_bf16 against (bits + 0x7fff + lsb) >> 16 over every
 * non-NaN f32; returns the number of mismatches. */
uint64_t ro_selftest_bf16_exhaustive(void);

/* ---- the reference tests' input stream: crates/engine/tests/common/reference.rs:141-162 */
float ro_lcg_f(uint64_t* state);
void ro_lcg_fill(uint64_t* state, float* out, size_t n);

/* ---- scale rule + quantize: crates/backend/kernels/fwd.hip:66-69,
 *      crates/engine/tests/fwd_kernel.rs:162-171 ---- */
void ro_quant_block(const float* v, int n, uint8_t* codes, float* scale);

/* Reference-exact linear slab append (block 128 over the latent, rope as bf16):
 * crates/backend/kernels/fwd.hip:51-71. Returns the launcher's guard code (0/1001/1002). */
int ro_append_kv(const float* latent, const float* rope, uint8_t* lc8, float* lscale,
                 uint16_t* rc, int pos, int kvl, int ropn, int n_blocks);
/* crates/backend/kernels/indexer.hip:54-58 */
int ro_index_append(const float* k, uint16_t* kcache, int pos, int hd);

/* ---- indexer scores: crates/backend/kernels/indexer.hip:60-93, host restatement
 *      crates/engine/tests/indexer_kernel.rs:238-250 (same fold order):
 *      scores[t] = sum over active heads h of w[h]*wscale*max((q_h . k_t)*dscale, 0).
 *      kcache is [nt][hd] bf16; heads (nullable) lists the nact active heads. Returns the
 *      launcher's guard code (crates/backend/kernels/indexer.hip:281). ---- */
int ro_index_score(const float* q, const float* w, const uint16_t* kcache, const uint32_t* heads,
                   int nt, int nh, int nact, int hd, float wscale, float dscale, float* scores);
/* Paged forms (new here): the key cache is [n_pages*page_tokens][hd] bf16 addressed by slot;
 * query qi scores its first nts[qi] tokens through block_table[qi]. */
int ro_index_append_paged(const float* k, const int32_t* slot_mapping, uint16_t* kpool,
                          int n_tokens, int hd, int page_tokens, int n_pages);
void ro_index_score_paged(const float* q, const float* w, const uint16_t* kpool,
                          const int32_t* block_table, const int32_t* nts, const uint32_t* heads,
                          int n_queries, int max_blocks_per_seq, int stride, int nh, int nact,
                          int hd, int page_tokens, float wscale, float dscale, float* scores,
                          int n_threads);

/* ---- paged fp8 cache, one f32 scale per token (block = whole row) ----
 * Page layout: [page_tokens][width] u8 codes, then [page_tokens] f32 scales. */
size_t ro_kv_page_bytes(int page_tokens, int width);
/* rows: [n_tokens][width] bf16; slot = page*page_tokens + offset; slot < 0 skips the token;
 * slot >= n_pages*page_tokens is counted in the return value and never written. */
int ro_kv_append_paged(const uint16_t* rows, const int32_t* slot_mapping, uint8_t* pool,
                       int n_tokens, int width, int page_tokens, int n_pages);
/* Dense gather+dequant (formula crates/backend/kernels/attn.hip:168-177 with rows == null):
 * out[cu_seqlens[s] + t][:] = bf16(e4m3(code) * scale) for t < seq_lens[s]. */
void ro_kv_gather_paged(const uint8_t* pool, const int32_t* block_table, const int32_t* seq_lens,
                        const int32_t* cu_seqlens, uint16_t* out, int n_seqs,
                        int max_blocks_per_seq, int width, int page_tokens);
/* Sparse gather (the `rows` argument of crates/backend/kernels/attn.hip:175):
 * out[(q*k + j)][:] = token rows[q*k + j] of sequence q, for j < n_rows[q] (or k if null). */
void ro_kv_gather_rows_paged(const uint8_t* pool, const int32_t* block_table,
                             const uint32_t* rows, const int32_t* n_rows, uint16_t* out,
                             int n_queries, int k, int max_blocks_per_seq, int width,
                             int page_tokens);
/* Same two gathers split over n_threads host threads (CPU-baseline timing only). */
void ro_kv_gather_paged_mt(const uint8_t* pool, const int32_t* block_table,
                           const int32_t* seq_lens, const int32_t* cu_seqlens, uint16_t* out,
                           int n_seqs, int max_blocks_per_seq, int width, int page_tokens,
                           int n_threads);
void ro_kv_append_paged_mt(const uint16_t* rows, const int32_t* slot_mapping, uint8_t* pool,
                           int n_tokens, int width, int page_tokens, int n_pages,
                           int n_threads);

/* ---- MLA decode attention in latent space: crates/engine/tests/kernel_attend.rs:201-226
 *      (attend_reference, the dense two-pass softmax the flash kernel is checked against),
 *      crates/core/src/routing.rs:10-22 (softmax). lat [nr][kvl], rk [nr][rope] are the
 *      attended rows already widened to f32; clat [H][kvl]. ---- */
void ro_mla_attend_dense(const float* qabs, const float* qrope, const float* lat, const float* rk,
                         int H, int nr, int kvl, int rope, float scale, float* clat);
/* Over the reference's linear slabs (crates/backend/kernels/attn.hip:168-183): e4m3 latent
 * with one f32 scale per 128 values, bf16 roped key, token = rows ? rows[j] : j. Returns the
 * launcher's guard code (crates/backend/kernels/attn.hip:284-293). */
int ro_mla_attend(const float* qabs, const float* qrope, const uint8_t* lc8, const float* lscale,
                  const uint16_t* rc, const uint32_t* rows, int H, int nr, int kvl, int rope,
                  int n_blocks, float scale, float* clat);
/* Over the paged cache (new here): every token is kvl + rope codes under one f32 scale;
 * sequence s attends its first seq_lens[s] tokens, or rows[s*k + j], j < n_rows[s] (k when
 * null) when rows is given. qabs [n_seqs][H][kvl], qrope [n_seqs][H][rope], clat like qabs.
 * Sequences are dealt to n_threads host threads. */
void ro_mla_attend_paged(const float* qabs, const float* qrope, const uint8_t* pool,
                         const int32_t* block_table, const int32_t* seq_lens,
                         const uint32_t* rows, const int32_t* n_rows, int k, int n_seqs, int H,
                         int max_blocks_per_seq, int kvl, int rope, int page_tokens, float scale,
                         float* clat, int n_threads);

/* ---- selection: crates/core/src/routing.rs:42-61 then sort_unstable()
 *      (crates/engine/tests/kernel_vector.rs:126-131). Writes min(k, nt) ascending
 *      indices, returns that count. ---- */
int ro_topk(const float* scores, int nt, int k, uint32_t* rows);
void ro_topk_batched(const float* scores, int n_queries, int stride, const int32_t* nts, int nt,
                     int k, uint32_t* rows, int n_threads);

/* ---- content pinning: crates/core/src/hash.rs ---- */
uint64_t ro_fnv1a(const uint8_t* bytes, size_t n);
uint64_t ro_splitmix_finalize(uint64_t z);
uint64_t ro_xor_fold(const uint32_t* words, size_t n, uint64_t i_base, size_t stride);

#ifdef __cplusplus
}
#endif
#endif
