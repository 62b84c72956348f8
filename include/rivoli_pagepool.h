/* Host-side page allocator for the paged fp8 KV cache — C ABI.
 *
 * The reference keeps linear per-layer slabs (crates/engine/src/glm/engine.rs:77-83,168-175)
 * and has no KV page allocator; the only free list in its tree is the routed-expert slot
 * arena (crates/core/src/arena.rs). This allocator follows that arena's placement order for
 * one flat tier: a freed page is pushed on a LIFO list (arena.rs:132-135), an allocation pops
 * the most recently freed page first (arena.rs:141) and otherwise grows the frontier
 * (arena.rs:145-149). The arena's frontier retreat and cross-tier compaction have no
 * counterpart: a flat pool of equal pages has nothing to compact.
 *
 * Pure host code: no HIP, no device memory. It produces the block tables and slot mappings
 * the kernels in rivoli_kvcache.h consume. Not thread-safe: one decode thread owns a pool,
 * as one thread issues all launches in the reference (crates/backend/src/gpustream.rs:83-91).
 * Return convention: >= 0 success / value, negative = refusal:
 *   -1001 invalid argument or unknown sequence, -1005 pool exhausted, -1006 out of host memory
 *   (nothing was changed in either case; no C++ exception leaves an entry point).
 */
#ifndef RIVOLI_PAGEPOOL_H
#define RIVOLI_PAGEPOOL_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rivoli_pagepool rivoli_pagepool;

rivoli_pagepool* rivoli_pagepool_create(int n_pages, int page_tokens);
void rivoli_pagepool_destroy(rivoli_pagepool* pool);

/* A new empty sequence; returns its id. Ids of freed sequences are reused. */
int rivoli_pagepool_seq_create(rivoli_pagepool* pool);
/* Returns every page of `seq` to the free list, in block-table order (so the sequence's
 * LAST page is the next one handed out), and retires the id. Returns the pages freed. */
int rivoli_pagepool_seq_free(rivoli_pagepool* pool, int seq);
/* Grows `seq` by n_tokens, allocating pages as its tail page fills. Writes the n_tokens new
 * slot ids (page * page_tokens + offset) to slots_out, which may be null. All or nothing:
 * when the pool cannot supply the pages, returns -1005 and leaves the pool untouched. */
int rivoli_pagepool_seq_extend(rivoli_pagepool* pool, int seq, int n_tokens, int* slots_out);

int rivoli_pagepool_seq_len(const rivoli_pagepool* pool, int seq);
int rivoli_pagepool_seq_blocks(const rivoli_pagepool* pool, int seq);
/* Copies up to max_blocks page ids of `seq` into out; returns the sequence's block count. */
int rivoli_pagepool_block_table(const rivoli_pagepool* pool, int seq, int* out, int max_blocks);

int rivoli_pagepool_pages_free(const rivoli_pagepool* pool);   /* free list + never-used */
int rivoli_pagepool_pages_owned(const rivoli_pagepool* pool);
int rivoli_pagepool_frontier(const rivoli_pagepool* pool);     /* pages ever handed out */

#ifdef __cplusplus
}
#endif
#endif
