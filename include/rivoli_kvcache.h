/* rivoli fp8 MLA KV-cache hot path for gfx950 (MI355X) — C ABI.
 *
 * The entry points below are what rivoli's backend FFI binds for this path. They follow the
 * house launcher convention (crates/backend/kernels/fwd.hip:1-4, crates/backend/src/hip.rs:
 * 328-336): return 0 on success, a POSITIVE argument-guard code when the call is refused
 * before anything is launched (1001 non-positive / null argument, 1002 size bound,
 * 1004 divisibility), or -(int)hipError_t from the launch. Launch-only: no allocation, no
 * copy, no synchronisation. Every pointer is a device pointer owned by the caller and must
 * stay live until `stream` (nullptr = the null stream) has drained. The paged entry points
 * move 16 bytes per lane: their row, pool, output, query and scratch buffers must be 16-byte
 * aligned (guard 1004 otherwise). Dims cross as int
 * (the Rust side narrows usize as i32); all byte offsets are formed in 64 bits inside.
 *
 * Paged cache layout ("page"): page_tokens rows of `width` e4m3 codes, then page_tokens f32
 * scales — rivoli_kv_page_bytes(page_tokens, width) bytes, one scale per token (the whole
 * row is one quantization block). A pool is n_pages such pages, contiguous.
 * slot = page * page_tokens + offset_in_page.
 */
#ifndef RIVOLI_KVCACHE_H
#define RIVOLI_KVCACHE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Entry points that keep a reference signature byte for byte (drop-in for gfx950)
 * ---------------------------------------------------------------------------------------- */

/* Replaces crates/backend/kernels/fwd.hip:224-235 (Rust: launch_append_kv,
 * crates/backend/src/hip_attn.rs:137-147). One token into the LINEAR slabs at row `pos`:
 * latent as e4m3 with one f32 scale per 128 values, roped key as bf16. Null stream.
 * Guards: 1001 pos<0 or a non-positive dim; 1002 kvl not a multiple of 128 in [128,1024]
 * or ropn > kvl. */
int rivoli_append_kv(const float* latent, const float* rope, unsigned char* lc8, float* lscale,
                     unsigned short* rc, int pos, int kvl, int ropn, int n_blocks);

/* Replaces crates/backend/kernels/indexer.hip:268-276 (launch_index_append,
 * crates/backend/src/hip_attn.rs:450-455): kcache[pos*hd + i] = bf16(k[i]). */
int rivoli_index_append(const float* k, unsigned short* kcache, int pos, int hd);

/* Replaces crates/backend/kernels/indexer.hip:327-335 (launch_index_topk,
 * crates/backend/src/hip_attn.rs:490-495): rows[0..min(k,nt)) = the k best-scoring token
 * indices (score descending, ties to the lowest index, -0.0 == +0.0), emitted ASCENDING.
 * Entries past min(k,nt) are not written. Guard 1001: nt<=0 or k<=0. Null stream. */
int rivoli_index_topk(const float* scores, int nt, int k, unsigned int* rows);

/* Replaces crates/backend/kernels/fwd.hip:411-427 (launch_hash_rows,
 * crates/backend/src/hip.rs:581-603): XOR-folds splitmix64(((i_base+i)<<32) ^ bits(x[i]))
 * over i = 0, stride, 2*stride, ... < n INTO *out (the caller zeroes it). */
int rivoli_hash_rows(const float* x, int n, int stride, unsigned long long i_base,
                     unsigned long long* out, void* stream);

/* Replaces crates/backend/kernels/attn.hip:100-103,279-308 (Rust: attend_scratch_floats and
 * launch_attend, crates/backend/src/hip_attn.rs:113-128): MLA decode attention for one token
 * over the LINEAR slabs — clat[h] = sum_t softmax_t((qabs_h . L_t + qrope_h . R_t) * scale) *
 * L_t with L_t the e4m3 latent times its per-128 f32 scales, R_t the bf16 roped key, token =
 * rows ? rows[j] : j for j < nr. `partial` is scratch of rivoli_mla_attend_scratch_floats(H,
 * kvl) floats, or null for a single split. Null stream. Guards as the reference: 1001
 * non-positive dim; 1002 (kvl + rope) > 1024; 1004 kvl > 512 or kvl % 128. */
size_t rivoli_mla_attend_scratch_floats(int H, int kvl);
int rivoli_mla_attend(const float* qabs, const float* qrope, const unsigned char* Lc8,
                      const float* Lscale, const unsigned short* Rc, const unsigned int* rows, int H,
                      int nr, int kvl, int rope, int n_blocks, float scale, float* clat,
                      float* partial);

/* Replaces crates/backend/src/hip.rs:339-342's rivoli_device_sync: hipDeviceSynchronize. */
int rivoli_device_sync(void);

/* ------------------------------------------------------------------------------------------
 * New entry points (same convention, trailing stream): the paged, batched path
 * ---------------------------------------------------------------------------------------- */

/* Pure function, like rivoli_mla_attend_scratch_floats (crates/backend/kernels/attn.hip:
 * 100-103): bytes of one page. 64 x 576 -> 37120. */
size_t rivoli_kv_page_bytes(int page_tokens, int width);

/* Quantize-and-append (the paged, many-token form of append_kv, crates/backend/kernels/
 * fwd.hip:51-71 with the block widened to the whole row): for each token t < n_tokens,
 * rows[t*width .. +width) (bf16) -> amax, scale = amax>0 ? amax/448 : 1, codes =
 * e4m3(v/scale), stored at slot_mapping[t]. A negative slot skips the token (padding). A
 * slot >= n_pages*page_tokens is never written; it is counted in *bad_slots when that
 * pointer is non-null.
 * Guards: 1001 null pointer / non-positive dim; 1002 width > 1024; 1004 width % 16 or
 * page_tokens % 4. */
int rivoli_kv_append_paged(const unsigned short* rows, const int* slot_mapping,
                           unsigned char* pool, int n_tokens, int width, int page_tokens,
                           int n_pages, unsigned int* bad_slots, void* stream);

/* Linear-slab append of n_tokens consecutive rows starting at pos0 — rivoli_append_kv for a
 * prefill chunk in ONE launch and on a stream (the reference loops rows on the host,
 * crates/engine/src/glm/attn.rs:135-160). latent is [n_tokens][kvl] f32, rope
 * [n_tokens][ropn] f32. Same guards as rivoli_append_kv plus 1001 for n_tokens <= 0. */
int rivoli_append_kv_rows(const float* latent, const float* rope, unsigned char* lc8,
                          float* lscale, unsigned short* rc, int pos0, int n_tokens, int kvl,
                          int ropn, int n_blocks, void* stream);

/* Block-table gather + dequantize (the tile load of mla_latent_attend with rows == null,
 * crates/backend/kernels/attn.hip:168-177, materialised): for each sequence s < n_seqs and
 * t < seq_lens[s]:
 *   out[(cu_seqlens[s] + t)*width + i] = bf16(e4m3_to_f32(code) * scale)
 * where the token lives in page block_table[s*max_blocks_per_seq + t/page_tokens].
 * cu_seqlens has n_seqs+1 entries (exclusive prefix sum of seq_lens, in tokens). A page id
 * outside [0, n_pages) is skipped and counted in *bad_pages when non-null.
 * Guards: 1001, 1004 as above. */
int rivoli_kv_gather_paged(const unsigned char* pool, const int* block_table,
                           const int* seq_lens, const int* cu_seqlens, unsigned short* out,
                           int n_seqs, int max_blocks_per_seq, int width, int page_tokens,
                           int n_pages, unsigned int* bad_pages, void* stream);

/* rivoli_kv_gather_paged for a caller that knows how many rows the batch holds (it sized
 * `out` by that number): total_tokens >= the sum of seq_lens. Same results. When the batch
 * fills less than 0.7 of what its block tables could address (ragged batches, or tables sized
 * for a context limit above the sequences' lengths), the launch is sized by total_tokens instead of by
 * n_seqs * max_blocks_per_seq pages and each workgroup finds its sequence from the device-side
 * lengths; otherwise this is rivoli_kv_gather_paged. Rows may be left out if total_tokens
 * understates the sum. Guards as above, plus 1001 for total_tokens < 0 and 1002 when
 * total_tokens / 4 does not fit a launch. */
int rivoli_kv_gather_paged_packed(const unsigned char* pool, const int* block_table,
                                  const int* seq_lens, const int* cu_seqlens, unsigned short* out,
                                  int n_seqs, int max_blocks_per_seq, long long total_tokens,
                                  int width, int page_tokens, int n_pages, unsigned int* bad_pages,
                                  void* stream);

/* A decode step's cache work in ONE launch: rivoli_kv_append_paged of one new row per sequence
 * (new_rows [n_seqs][width] bf16, slot_mapping [n_seqs]) followed by rivoli_kv_gather_paged_packed
 * (rivoli_kv_gather_paged when total_tokens < 0) — what the reference runs per layer as
 * append_kv (crates/backend/kernels/fwd.hip:51-71) and then the tile loads of the attend
 * (attn.hip:168-177), one launch each per token. seq_lens ALREADY COUNTS the new token, and
 * slot_mapping[s] must be the slot the block table gives token seq_lens[s] - 1 of sequence s:
 * that token's output row is written from the row just quantized (dequantized from its new
 * codes and scale, so bit-identical to gathering the stored record), every other token is
 * gathered from the pool, and no workgroup reads what another one writes. Under that condition
 * pool and out end up exactly as after the two separate calls. A negative slot is a sequence
 * without a new token (all of it is gathered); a slot >= n_pages * page_tokens is counted in
 * *bad_slots, written nowhere, and the sequence is gathered whole. A slot_mapping that names
 * another token's slot is outside the contract (the separate calls would gather the new row
 * there; this call gathers what the pool held).
 * Guards: those of the two calls (1001 null / non-positive, 1002 width > 1024, 1004 alignment
 * of pool, out and new_rows or a width that is not a multiple of 16). */
int rivoli_kv_append_gather_paged(const unsigned short* new_rows, const int* slot_mapping,
                                  unsigned char* pool, const int* block_table, const int* seq_lens,
                                  const int* cu_seqlens, unsigned short* out, int n_seqs,
                                  int max_blocks_per_seq, long long total_tokens, int width,
                                  int page_tokens, int n_pages, unsigned int* bad_slots,
                                  unsigned int* bad_pages, void* stream);

/* Sparse row gather + dequantize (the `rows` argument of rivoli_mla_attend,
 * crates/backend/kernels/attn.hip:125,175): for query q < n_queries and j < n_rows[q]
 * (k when n_rows is null): out[(q*k + j)*width ..] = dequantized token rows[q*k + j] of
 * sequence q. Row indices >= max_blocks_per_seq*page_tokens or pages outside the pool are
 * skipped and counted in *bad_rows when non-null. */
int rivoli_kv_gather_rows_paged(const unsigned char* pool, const int* block_table,
                                const unsigned int* rows, const int* n_rows,
                                unsigned short* out, int n_queries, int k,
                                int max_blocks_per_seq, int width, int page_tokens, int n_pages,
                                unsigned int* bad_rows, void* stream);

/* Batched rivoli_index_topk: query q reads scores[q*stride .. +nts[q]) (nt for every query
 * when nts is null) and writes rows[q*k .. +min(k, nt_q)), ascending. One call for all
 * queries; the selection rule is the single-query one.
 * `workspace` (nullable) lets the call spread every query over many workgroups instead of
 * one (queries longer than 16384 scores; shorter ones stay on one workgroup either way):
 * rivoli_index_topk_workspace_bytes(n_queries, nt) bytes of 16-byte-aligned device memory that
 * the caller zero-fills ONCE (hipMemset) before its first use; every call puts back to zero
 * whatever has to start at zero, so it can be reused call after call on one stream (calls
 * that share a workspace must not overlap, and a workspace serves one (n_queries, nt) shape).
 * The split form is three launches on the stream and no workgroup waits for another.
 * Guards: 1001 null / non-positive; 1002 stride < nt; 1004 workspace not 16-byte aligned. */
size_t rivoli_index_topk_workspace_bytes(int n_queries, int nt);
int rivoli_index_topk_batched(const float* scores, int n_queries, int stride, const int* nts,
                              int nt, int k, unsigned int* rows, void* workspace, void* stream);

/* The DSA step the reference runs as index_topk followed by an attend over `rows`, with "no
 * D2H, no host top-k, and no device_sync" between them (crates/backend/src/hip_attn.rs:478-495),
 * for a consumer that wants the selected rows as bf16: rivoli_index_topk_batched and
 * rivoli_kv_gather_rows_paged in one call. rows[q*k + j] as the batched top-k writes them, and
 * out[(q*k + j)*width ..] = the dequantized token rows[q*k + j] of sequence q for
 * j < min(k, nt_q), through block_table[q]. With a workspace and a split shape the selection's
 * last launch gathers the rows it has just placed (no separate gather launch, and the gather
 * is dealt evenly whatever the positions of the selected tokens); otherwise the two kernels
 * follow each other on the stream. hist_ready != 0: the workspace's histogram was filled by
 * rivoli_index_score_paged_hist on the same stream with the same (n_queries, nt, nts) — the
 * selection then skips its first launch (1001 when the shape is not a split one).
 * Guards: those of the two calls it stands for. */
int rivoli_dsa_select_gather_paged(const float* scores, int n_queries, int stride, const int* nts,
                                   int nt, int k, unsigned int* rows, void* workspace,
                                   int hist_ready, const unsigned char* pool,
                                   const int* block_table, unsigned short* out,
                                   int max_blocks_per_seq, int width, int page_tokens, int n_pages,
                                   unsigned int* bad_rows, void* stream);

/* rivoli_dsa_select_gather_paged for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference. Same arguments without `workspace` and `hist_ready`, same
 * results bit for bit: the selection's workspace is a 4.5 MiB array inside the library's own
 * device image (one copy per GPU, held until the process ends), and the call makes no
 * hipMalloc / hipFree and calls no allocating routine. Shapes that run split must fit it:
 * n_queries * rivoli_index_topk_workspace_bytes(1, nt) <= 4 718 592 bytes (16 queries of 65536
 * scores do), else 1002; shorter queries (nt <= 16384) need no workspace and are not limited.
 * Every call on a GPU shares that GPU's array, so calls that overlap on one GPU (two streams,
 * two threads) race; calls that follow each other on one stream are fine, whatever their shapes
 * (the call clears what must start at zero with a fill kernel, not a memset). The first call on
 * a device looks the array's address up (hipGetSymbolAddress): make it outside a graph capture.
 * Other guards as rivoli_dsa_select_gather_paged. */
int rivoli_dsa_select_gather_paged_noalloc(const float* scores, int n_queries, int stride,
                                           const int* nts, int nt, int k, unsigned int* rows,
                                           const unsigned char* pool, const int* block_table,
                                           unsigned short* out, int max_blocks_per_seq, int width,
                                           int page_tokens, int n_pages, unsigned int* bad_rows,
                                           void* stream);

/* Replaces crates/backend/kernels/indexer.hip:278-295 (launch_index_score,
 * crates/backend/src/hip_attn.rs:464-476): scores[t] = sum over the active heads h of
 * w[h]*wscale*max((q_h . k_t)*dscale, 0) for t < nt, over the LINEAR bf16 key cache
 * kcache[nt][hd]. q is [nh][hd] f32, w [nh] f32; heads (nullable) lists the nact active
 * heads, null = heads 0..nact-1. Results agree with the reference's within 1e-5 of the
 * largest score (its own test bar), not bit for bit: the dots run on the matrix cores.
 * Guards: the reference's own — 1001 non-positive dims or nact > nh; 1002 more than 1024 active
 * heads, or (hd + the next power of two >= max(nact, 32)) * 4 > 65536. Up to 64 active heads
 * with hd <= 128, hd % 16 == 0 and 16-byte-aligned q and kcache run on the matrix cores; every
 * other accepted shape takes a plain f32 kernel (same bar). Null stream. */
int rivoli_index_score(const float* q, const float* w, const unsigned short* kcache,
                       const unsigned int* heads, int nt, int nh, int nact, int hd, float wscale,
                       float dscale, float* scores);

/* The paged, batched form: query qi (q [n_queries][nh][hd], w [n_queries][nh]) scores its
 * first nts[qi] tokens (nt when nts is null) through block_table[qi] over the paged key
 * cache kpool[n_pages*page_tokens][hd] bf16, into scores[qi*stride + t]. Tokens whose page id
 * is outside [0, n_pages) are not written. Same guards, plus 1002 for stride < nt, for
 * nt > max_blocks_per_seq * page_tokens (a scored token without a block-table entry) or for
 * n_queries > 65535. A page size that is not a multiple of 32 takes the plain f32 kernel. */
int rivoli_index_score_paged(const float* q, const float* w, const unsigned short* kpool,
                             const int* block_table, const int* nts, const unsigned int* heads,
                             int n_queries, int max_blocks_per_seq, int stride, int nt, int nh,
                             int nact, int hd, int page_tokens, int n_pages, float wscale,
                             float dscale, float* scores, void* stream);

/* rivoli_index_score_paged that also does the first step of the selection that follows it
 * (the score -> top-k fusion the reference's design aims at, crates/backend/kernels/
 * indexer.hip:1-13): while a score is still in a register its selection key's top 12 bits are
 * counted into topk_workspace (the rivoli_index_topk_workspace_bytes(n_queries, nt) buffer the
 * selection will be handed, zero-filled as described there), so rivoli_dsa_select_gather_paged
 * (hist_ready = 1) does not sweep the scores for it. A token whose key page is outside the pool
 * is written as -inf here (and counted as such), not left unwritten: the histogram and the
 * scores the selection reads next must describe the same keys. For shapes the selection does not split
 * (nt <= 16384) the workspace is left alone. Guards as rivoli_index_score_paged, plus 1001 for a
 * null workspace and 1004 for one that is not 16-byte aligned. */
int rivoli_index_score_paged_hist(const float* q, const float* w, const unsigned short* kpool,
                                  const int* block_table, const int* nts, const unsigned int* heads,
                                  int n_queries, int max_blocks_per_seq, int stride, int nt, int nh,
                                  int nact, int hd, int page_tokens, int n_pages, float wscale,
                                  float dscale, float* scores, void* topk_workspace, void* stream);

/* Paged form of rivoli_index_append for many tokens: kpool[slot_mapping[t]*hd + i] =
 * bf16(k[t*hd + i]). Negative slots are padding; slots >= n_pages*page_tokens are counted in
 * *bad_slots (nullable) and never written. Guards: 1001; 1004 hd % 8. */
int rivoli_index_append_paged(const float* k, const int* slot_mapping, unsigned short* kpool,
                              int n_tokens, int hd, int page_tokens, int n_pages,
                              unsigned int* bad_slots, void* stream);

/* MLA decode attention in latent space over the PAGED cache — the batched, paged form of
 * rivoli_mla_attend (crates/backend/kernels/attn.hip:279-308; Rust launch_attend,
 * crates/backend/src/hip_attn.rs:113-128), consuming the fp8 pages directly instead of a
 * gathered bf16 copy. For sequence s < n_seqs and head h < H:
 *   clat[s][h][:] = sum_t softmax_t((qabs[s][h] . L_t + qrope[s][h] . R_t) * scale) * L_t
 * with L_t = e4m3_to_f32(codes[0:kvl]) * scale_t and R_t = e4m3_to_f32(codes[kvl:kvl+rope]) *
 * scale_t of the page row. Attended tokens: 0 .. min(seq_lens[s], max_rows)-1 when `rows` is
 * null (dense); otherwise rows[s*max_rows + j] for j < n_rows[s] (max_rows when n_rows is
 * null) — the DSA selection, as rivoli_index_topk_batched emits it with k = max_rows.
 * Tokens whose page id is outside [0, n_pages) are left out of the softmax and counted in
 * *bad_rows when non-null. A sequence with nothing to attend gets zeros.
 * `partial` is caller-owned scratch of rivoli_mla_attend_paged_scratch_floats(n_seqs, H,
 * max_rows) floats (the split-KV partials; may be null when that returns 0). When scratch is
 * used, the 32-token tiles of the whole batch are dealt evenly to the workgroups from the
 * device-side lengths, so ragged batches keep the GPU full; the plan depends only on
 * (n_seqs, H, max_rows) and those lengths: equal calls give bit-equal results.
 * `precise`: 2 carries both q and the softmax weights as bf16 hi + lo (~17 bits) through the
 * matrix cores — the parity mode: results agree with the reference formula far inside its
 * own bar for this kernel (1e-3 of the largest output + 1e-3, crates/engine/tests/common/
 * asserts.rs), though not bit for bit; 1 carries only q that way (weights rounded to bf16
 * once: errors up to ~1e-3 of the SPREAD of the attended rows); 0 rounds q to bf16 once as
 * well (a score is off by ~2^-10 |q||k|: ordinary bf16 flash-attention numerics).
 * 3 and 4 (512 + 64 rows only) run both contractions on the 8-bit matrix instructions, the
 * cache codes going into them untouched and q / the weights as sums of e4m3 terms under
 * power-of-two block scales: 3 = two terms each (the accuracy class of 0), 4 = three terms for
 * q and two for the weights (the class of 1; inside the reference's bar on the test caches).
 * They are the fastest modes: about 30 % less time per launch than 0 / 2.
 * Other row widths (kvl a multiple of 128 up to 512, rope a multiple of 8 up to 64) always run
 * as 2.
 * Guards: 1001 null / non-positive, or a null `partial` when scratch is needed; 1002
 * n_seqs > 65535; 1004 for a latent width that is not a multiple of 128 or above 512, a rope
 * width that is not a multiple of 8 or above 64, or a buffer that is not 16-byte aligned. */
size_t rivoli_mla_attend_paged_scratch_floats(int n_seqs, int H, int max_rows);
int rivoli_mla_attend_paged(const float* qabs, const float* qrope, const unsigned char* pool,
                            const int* block_table, const int* seq_lens,
                            const unsigned int* rows, const int* n_rows, int n_seqs, int H,
                            int max_rows, int max_blocks_per_seq, int kvl, int rope,
                            int page_tokens, int n_pages, float scale, int precise, float* clat,
                            float* partial, unsigned int* bad_rows, void* stream);

/* ---- the second cache format: f32 rows holding simulated-fp8 values, a window ring followed
 * by compressed blocks, and a scored selection of those blocks ---- */

/* Replaces crates/backend/kernels/mla.hip:527-548 (launch_act_quant_f8_prefix,
 * crates/engine/src/v4/attn.rs:288): the fused quantize-then-dequantize of dims [0, n) of every
 * row in blocks of `block`: amax = max(1e-4, |x|) over the block, s = 2^ceil(log2(amax/448))
 * (actquant.hpp:69-81), dst = e4m3_to_f32(rne_e4m3(clamp(src / s, +-448))) * s, nearest even
 * everywhere (formats.hpp:245-264). Dims [n, row_stride) are not touched. src == dst is the
 * in-place form. Guards as the reference's: 1001 non-positive or row_stride < n (also null
 * pointers); 1002 src != dst with n != row_stride (dst rows would be part stale), or more than
 * 2^32 - 1 elements; 1004 n not a multiple of block. Blocks of 16, 32, 64, 128 or 256 with
 * 16-byte-aligned rows take the coalesced kernel; anything else a thread-per-block kernel. */
int rivoli_act_quant_f8_prefix(const float* src, float* dst, int rows, int row_stride, int n,
                               int block, void* stream);

/* Replaces crates/backend/kernels/blockindex.hip:241-262 (launch_act_quant_f4_rotated,
 * crates/backend/src/hip_linalg.rs:620; callers crates/engine/src/v4/blocksel.rs:218 on the
 * indexer's q rows and v4/kvcompress.rs:388 as the indexer compressor's finish): every row of
 * x [rows][d], in place, becomes bf16(fp4(bf16(H x / sqrt(d)))) — H the natural-order
 * (Sylvester) Hadamard matrix, the butterflies in the reference's stage order; fp4 = blocks of
 * 32 with amax floored at 6 * 2^-126, scale 2^ceil(log2(amax / 6)), e2m1 nearest with ties to
 * the even mantissa (actquant.hpp:45-105, formats.hpp:285-293). Bit-identical to the
 * reference's kernel. Guards as the reference's: 1001 non-positive sizes (also a null
 * pointer), 1002 d > 256, 1003 d not a power of two, 1004 d not a multiple of 32 (also x not
 * 16-byte aligned). */
int rivoli_act_quant_f4_rotated(float* x, int rows, int d, void* stream);

/* Replaces crates/backend/kernels/blockindex.hip:264-281 (launch_index_score_blocks,
 * crates/backend/src/hip.rs:497-520; caller v4/blocksel.rs:248): score[t][c] =
 * bf16(sum_h bf16(relu(bf16(q[t][h] . kv[c])) * w[t][h])) for q [s][heads][hd], kv
 * [n_comp][hd], w [s][heads], score [s][n_comp] — what rivoli_index_select_blocks ranks. The
 * dot is a sequential f32 fold of separately rounded products and the head sum a sequential
 * f32 fold rounded once, exactly as the reference's kernel, so the result is bit-identical
 * to it. hd = 128 (the shipped width) with a 16-byte-aligned kv takes the register-resident
 * kernels (one for prefill-sized calls, one that splits the heads of a decode step's single
 * query over a workgroup's waves); any other width a slower one. Guards as the reference's: 1001 non-positive s, heads
 * or hd (also null pointers); 1005 n_comp <= 0 (no block has completed: the caller must not
 * rank an unwritten buffer). */
int rivoli_index_score_blocks(const float* q, const float* kv, const float* w, float* score,
                              int s, int n_comp, int heads, int hd, void* stream);

/* rivoli_index_score_blocks for a prefill (query row t is prompt position t), where the
 * selection ranks block c for row t only when c < (t + 1) / ratio (select.rs:153-188: a block
 * is legal once it has closed): every legal entry of score is written, bit-identical to
 * rivoli_index_score_blocks; an entry whose 64-block group holds no legal block is left
 * untouched, which is about half of the matrix and half of the time. The other entries of a
 * group with a legal block are written too. rivoli_index_select_blocks(prefill = 1) and
 * rivoli_sel_gather_scored read legal entries only. ITS OUTPUT FEEDS A PREFILL SELECTION
 * ONLY: a consumer that ranks whole rows (rivoli_index_select_blocks with prefill = 0, a
 * host-side scored_rows over all n_comp blocks) would rank entries this call never wrote, and
 * nothing in the buffer marks them. No counterpart in the reference, whose kernel scores the
 * whole rectangle. Guards as rivoli_index_score_blocks; ratio <= 0: 1001. */
int rivoli_index_score_blocks_prefill(const float* q, const float* kv, const float* w,
                                      float* score, int s, int n_comp, int heads, int hd, int ratio,
                                      void* stream);

/* The scored block selection that crates/engine/src/v4/select.rs:153-188 (scored_rows) performs
 * on the host after a device-to-host copy of the scores, as one launch on the device. scores is
 * [rows][n_comp] f32 (what launch_index_score_blocks wrote; illegal slots need not be masked).
 * For query row t: limit = prefill ? min((t + 1) / ratio, n_comp) : n_comp, and the
 * k = min(index_topk, n_comp) best of the first `limit` scores under f32 total order
 * (descending; ties to the LOWER block index) are written ascending as block + offset to
 * out[t*k ..], then -1 out to k columns. Where limit <= k the row is offset .. offset+limit-1
 * whatever the scores are. The reference takes one query row at decode; here prefill == 0 with
 * rows > 1 is a batch of decode rows, each over all n_comp blocks.
 * Guards: 1001 null / non-positive / negative offset; 1002 offset + n_comp overflows int. */
int rivoli_index_select_blocks(const float* scores, int rows, int n_comp, int ratio,
                               int index_topk, int prefill, int offset, int* out, void* stream);

/* Selection rectangles (crates/engine/src/v4/select.rs:334-488, Sel::shape / Sel::gather /
 * Sel::gather_scored, which the reference fills on the host and uploads per call): one row per
 * query, [window columns | compressed columns], -1 for a masked cell; the index-list attention
 * below reads it as is. The phase is start_pos == 0 (prefill: seqlen rows, values are absolute
 * positions, the last `win` up to the query's own) or not (decode: one row, values are ring
 * slots oldest first, slot p % win holding position p; slots not yet written are -1).
 * Compressed columns are block + offset with offset = seqlen at prefill and win at decode
 * (select.rs:268-270); at prefill query t may read block c only if c < (t + 1) / ratio.
 * ratio == 0 is a layer without a compressor, ratio == 4 the class with an indexer
 * (crates/engine/src/v4/geometry.rs:86-92,128-130).
 * rivoli_sel_shape is pure host arithmetic: rows, and cols = window columns (min(seqlen, win) at
 * prefill, win at decode) + (start_pos + rows) / ratio. rivoli_sel_gather fills that rectangle
 * with the positional rule (every closed block). rivoli_sel_gather_scored fills the window
 * columns and then the k = min(index_topk, n_comp) columns of rivoli_index_select_blocks over
 * scores [rows][n_comp]; *cols_out (host, optional) receives window columns + k.
 * Guards: 1001 null / win <= 0 / seqlen <= 0 / negative arguments (gather_scored: ratio == 0,
 * nothing to rank); 1002 more than 16 776 960 columns; 1005 decode with seqlen != 1
 * (select.rs:78-86); 1006 positional selection on the indexed class with more closed blocks
 * than index_topk (select.rs:363-383: the scored form is how that is answered). */
int rivoli_sel_shape(int win, int ratio, int index_topk, int seqlen, int start_pos, int* rows,
                     int* cols);
int rivoli_sel_gather(int win, int ratio, int index_topk, int seqlen, int start_pos, int* out,
                      void* stream);
int rivoli_sel_gather_scored(const float* scores, int n_comp, int win, int ratio, int index_topk,
                             int seqlen, int start_pos, int* out, int* cols_out, void* stream);

/* Replaces the device copies of crates/engine/src/v4/attn.rs:343-378 (write_ring) with one
 * launch: cache is the layer's [win][hd] f32 ring, kv the step's rows ([seqlen][hd] at prefill,
 * one row at decode). Decode writes slot start_pos % win; a prompt seeds slot t % win with
 * position t for its last min(seqlen, win) positions. kv and cache must not overlap.
 * Guards: 1001, 1005 as above. Which buffer the attention then indexes is the caller's rule
 * (the prompt's own rows at prefill, the cache at decode). */
int rivoli_kv_ring_write(const float* kv, float* cache, int win, int hd, int seqlen,
                         int start_pos, void* stream);

/* Replaces crates/backend/kernels/attn.hip:446-465 (rivoli_gather_attn_shared_kv; Rust row
 * launch_gather_attn_shared_kv, caller crates/engine/src/v4/attn.rs:304-330), same signature:
 * multi-query attention with one d-wide row serving as key and value for all h heads, over
 * the explicit index list idxs [m][topk] into kv [rows][d] (-1 masks a slot, which is then
 * never dereferenced); sink [h] joins the softmax denominator only, exp(sink - max) after the
 * running-max shift (attn.hip:333-343); a query with no live slot gets NaN (attn.hip:344-351);
 * o [m][h][d] is the quotient rounded to bf16, stored as f32. q is [m][h][d] f32.
 * d == 512 with 16-byte-aligned q / kv / o takes the matrix-core kernel, which reads a query's
 * rows once for all heads and rounds kv to bf16 on the way in — exact for cache rows, which are
 * fp8-simulated or bf16-rounded values (crates/engine/src/v4/attn.rs:288, kvcompress.hip) — and
 * carries q as bf16 hi + lo; any topk. Other shapes take a workgroup per (query, head) under the
 * reference launcher's limits. Parity bar: the reference's for this kernel, 1/128 of the largest
 * expected element (crates/engine/tests/kernel_v4_attend.rs:97-106, ATTEND_TOL).
 * Guards: 1001 null / non-positive; 1002 d > 1024 or m > 65535 on the plain path; 1006 (d + topk)
 * floats of LDS past 64 KiB on the plain path.
 * _bounded: the same with n_kv = rows of kv (an index at or past it is treated as masked instead
 * of read) and `precise` as in rivoli_mla_attend_paged: 2 = q and the softmax weights as
 * bf16 hi + lo (what the plain name uses), 1 = q hi + lo, 0 = single bf16 (exact products when q
 * is bf16-valued, as the model's is after its rotary), 3 = the plain f32 kernel at any width (for
 * kv rows that are not bf16 values and must not be rounded). */
int rivoli_gather_attn_shared_kv(const float* q, const float* kv, const float* sink,
                                 const int* idxs, int m, int h, int d, int topk, float scale,
                                 float* o, void* stream);
int rivoli_gather_attn_shared_kv_bounded(const float* q, const float* kv, const float* sink,
                                         const int* idxs, int m, int h, int d, int topk, int n_kv,
                                         float scale, int precise, float* o, void* stream);
/* _split: the bounded form with a caller-provided partial buffer, for calls whose queries alone
 * cannot fill the GPU (decode: the reference drives one query row, crates/engine/src/v4/select.rs:78-86):
 * a query's list is shared among several workgroups, each writing unnormalised accumulators and
 * (max, sum) to `partial`, and a second launch merges them in ascending order, adds the sink and
 * rounds — the scheme of the reference's mla_attend_combine (attn.hip:235-277) applied to this
 * kernel, which has no such path in the reference. rivoli_gather_attn_scratch_floats is the
 * pure sizing function (0 = this shape is not split and partial may be null), as
 * rivoli_mla_attend_scratch_floats is for the latent attention (attn.hip:100-103). The plan is a
 * function of the shape alone, so equal calls give bit-equal results. 1001 also when the plan
 * needs `partial` and it is null or not 16-byte aligned. */
size_t rivoli_gather_attn_scratch_floats(int m, int h, int d, int topk);
int rivoli_gather_attn_shared_kv_split(const float* q, const float* kv, const float* sink,
                                       const int* idxs, int m, int h, int d, int topk, int n_kv,
                                       float scale, int precise, float* o, float* partial,
                                       void* stream);

/* The compressor's pooling stage (crates/backend/kernels/kvcompress.hip; Rust rows
 * launch_kv_compress_deposit / _prefill / _decode, crates/backend/src/hip_attn.rs:547-605).
 * The two structs cross the boundary by pointer, as in the reference (kvcompress.hip:40-48,
 * :63-67; crates/engine/src/v4/kvcompress.rs GeomAbi / Finish are the same repr(C) layouts). */
typedef struct rivoli_comp_geom {
    int ratio; /* positions pooled into one compressed row */
    int coff;  /* 1 + overlap; overlapping windows exist at ratio 4 only */
    int d;     /* the compressor's head width */
    int cd;    /* coff * d: width of the kv / score projections and of an ape row */
    int ents;  /* coff * ratio: entries in one pooling window, at most 128 */
    int rd;    /* the last rd dims of a pooled row are rotated */
    float eps; /* RMSNorm epsilon */
} rivoli_comp_geom;
typedef struct rivoli_comp_finish {
    const float* norm;  /* [d] the compressor's own RMSNorm weight */
    const float* freqs; /* [positions][rd] (cos, sin) pairs of the COMPRESSED rotation table */
    float* out;         /* [nblk][d] at prefill, one row at decode */
} rivoli_comp_finish;

/* Replaces kvcompress.hip:419-437. kv, score: [s][cd] f32 (this call's projections); ape:
 * [ratio][cd]; the states: [coff*ratio][cd], a sequence starting with kv_state zeroed and
 * score_state -inf. A prefill of s tokens (slot0 = 0) stores its last complete block as the
 * next block's overlap half (overlapping layers) and its s % ratio trailing rows; a decode
 * step (s = 1) stores its row at slot0 = start_pos % ratio. score_state gets score + the ape
 * row of the position within its block. Launch it on every call, also when nothing is emitted.
 * Codes: 1000 null geometry; the geometry guard 1001 (ranges), 1002 (rd), 1003 (cd / ents not
 * the derived values), 1004 (ents > 128), 1010 (overlap and ratio disagree); 1001 null buffer;
 * 1005 s <= 0; 1008 slot0 out of range. */
int rivoli_kv_compress_deposit(const float* kv, const float* score, const float* ape,
                               float* kv_state, float* score_state, const rivoli_comp_geom* pp,
                               int s, int slot0, void* stream);

/* Replaces kvcompress.hip:439-456. For block b < nblk: per feature, softmax over the window's
 * entries of score + ape and the weighted sum of kv (on overlapping layers the window is the
 * previous block's rows, dims [0, d), then the block's own rows, dims [d, 2d); block 0's first
 * half is masked); then bf16 store, RMSNorm (f32 statistic, weight after the scale) with its
 * bf16 store, rotation of adjacent pairs of the last rd dims at position b * ratio, bf16 store;
 * out[b][d] holds bf16 values in f32. Codes as above, plus 1002 d > 8192, 1006 nblk <= 0. */
int rivoli_kv_compress_prefill(const float* kv, const float* score, const float* ape,
                               const rivoli_comp_finish* ff, const rivoli_comp_geom* pp, int nblk,
                               void* stream);

/* Replaces kvcompress.hip:458-478. Pools the completed window out of the state into ff->out[d]
 * (rotated at the block's first position, (start_pos / ratio) * ratio), then slides the window
 * on overlapping layers. One workgroup. Codes as above, plus 1007 start_pos <= 0 and 1009 when
 * start_pos + 1 is not a multiple of ratio. */
int rivoli_kv_compress_decode(float* kv_state, float* score_state, const rivoli_comp_finish* ff,
                              const rivoli_comp_geom* pp, int start_pos, void* stream);

/* Element codecs as launchers (what formats.hpp:42-57,99-106 and fwd.hip:20-45 are to the
 * reference's kernels), for census tests of the device codecs on arbitrary inputs:
 *   e4m3_encode: out[i] = f32_to_e4m3(x[i])            (rule of crates/core/src/num.rs:128-152)
 *   e4m3_dequant_bf16: out[i] = bf16(e4m3_to_f32(c[i]) * scale)
 *   bf16_encode: out[i] = f32_to_bf16(x[i]) */
int rivoli_codec_e4m3_encode(const float* x, unsigned char* out, long long n, void* stream);
int rivoli_codec_e4m3_dequant_bf16(const unsigned char* codes, float scale, unsigned short* out,
                                   long long n, void* stream);
int rivoli_codec_bf16_encode(const float* x, unsigned short* out, long long n, void* stream);

#ifdef __cplusplus
}
#endif
#endif
