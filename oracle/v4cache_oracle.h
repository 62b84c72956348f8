/* CPU oracle for the second cache format (window ring + compressed blocks of simulated-fp8
 * f32 rows) — TEST INFRASTRUCTURE, NOT PRODUCT. Plain-C restatement of the reference's CPU
 * arithmetic; only tests, the smoke check and the benchmark's CPU-baseline leg may call it.
 * Paths are relative to the reference tree.
 *
 * Pinning status (tests/test_oracle_v4.py):
 *   ro_e4m3_encode_rne    nearest-value enumeration over the 127 finite magnitudes with ties to
 *                         the even code (the technique of
 *                         crates/oracles/tests/v4_oracle_codecs.rs:27-57,103-145) on every
 *                         code, every midpoint, their neighbours and random points; saturation
 *                         and NaN KATs of the same test; agreement with ro_f32_to_e4m3
 *                         everywhere except exact subnormal ties, where the two rules are
 *                         stated to differ (crates/oracles/src/v4oracle/numerics.rs:60-67)
 *   ro_fast_round_scale   against ceil(log2) computed exactly (frexp) on powers of two, their
 *                         neighbours and random values; result is a power of two >= amax/448
 *                         and < 2 * that
 *   ro_act_quant_f8_prefix  the reference's own tie fixture restated
 *                         (crates/engine/tests/kernel_v4_quant.rs:283-343: a 448 pins the
 *                         scale, multiples and half multiples of 2^-9 in both signs; the data
 *                         separates RNE from half-away); idempotence; every output is an e4m3
 *                         value times the block's power-of-two scale; the launcher's guards
 *                         (crates/backend/kernels/mla.hip:527-541)
 *   ro_kv_compress_*      closed forms of the pooling (equal scores -> the mean of the window;
 *                         one dominant score -> that entry; block 0's masked overlap half);
 *                         the overlap index map against a literal overlap_transform tensor
 *                         and a float64 softmax (numpy); norm and rotation against float64 /
 *                         complex arithmetic; and the reference's state machine as an
 *                         invariant: a prefill of s tokens followed by single-token decode
 *                         steps emits bit for bit the blocks of one longer prefill
 *                         (crates/oracles/src/v4oracle/compress.rs:62-199 computes both arms
 *                         with the same per-feature fold). The reference's expectation for
 *                         these kernels is computed at test time from seeded weights
 *                         (crates/engine/tests/kernel_v4_compress.rs); it stores no vectors.
 *   ro_e2m1_encode / ro_e2m1_decode  (tests/test_oracle_v4_blockindex.py, as all of this group)
 *                         the seven midpoints as crates/oracles/tests/v4_oracle_codecs.rs:163-180
 *                         writes them, nearest magnitude by enumeration, saturation at +-1e9,
 *                         every code its own nearest (ibid. :181-207)
 *   ro_hadamard_rotate    equality with scipy's Sylvester matrix on integer inputs (exact in
 *                         f32, so a different basis order fails); involution and norm
 *                         (v4_oracle_codecs.rs:387-420)
 *   ro_fp4_act_quant_inplace  scale = smallest power of two >= amax / 6 from frexp; every output
 *                         the nearest of the eight magnitudes times that scale; the floor
 *   ro_act_quant_f4_rotated  the four steps in the order of
 *                         crates/engine/tests/kernel_v4_indexer.rs:149-156 from the parts above
 *                         (the store between rotation and quantization shown to matter);
 *                         power-of-two equivariance over 60 binades (ibid. :246-277); guards
 *                         (:287-320); on the GPU also the reference's own kernel
 *   ro_index_score_blocks the reference's known answer 1.125 (kernel_v4_indexer.rs:689-726);
 *                         closed forms that isolate each bf16 store, the relu and signed
 *                         weights; inputs on which a reordered or fused dot changes the
 *                         bits; guards; on the GPU also the reference's own kernel
 *   ro_v4_scored_rows     the three reference KATs (crates/engine/src/v4/select.rs:645-747:
 *                         below the cap the row is offset+0..limit-1 then -1; three-way tie
 *                         keeps the lower indices; a prefill row cannot take a block that
 *                         closed after it) and a brute-force sort under f32 total order
 *   ro_sel_shape / ro_sel_gather / ro_sel_gather_scored
 *                         the reference's own unit cases (select.rs:514-808: multi-row decode
 *                         refused; full ring read oldest first; ring not yet full padded; the
 *                         prefill causal rule for blocks; the indexed layer's cap; below the
 *                         cap the scored fill equals the positional one byte for byte; the
 *                         rectangle shapes of five layer/phase cases) and a literal per-cell
 *                         restatement in Python
 *   ro_ring_write         the three arms of crates/engine/src/v4/attn.rs:343-378 against the
 *                         rule "slot t % win holds position t" for every live position
 *   ro_sparse_attn        closed forms (one live slot -> the row over 1 + exp(sink - logit);
 *                         equal rows -> that row times the softmax mass; sink = -inf -> the
 *                         plain softmax average), a float64 numpy softmax on random cases,
 *                         masked slots never dereferenced, a fully masked query -> NaN
 *                         (crates/backend/kernels/attn.hip:344-351). The reference's goldens
 *                         for this kernel are captured at test time from its frozen model
 *                         oracle (crates/engine/tests/kernel_v4_attend.rs); it stores none.
 */
#ifndef RIVOLI_V4CACHE_ORACLE_H
#define RIVOLI_V4CACHE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* crates/oracles/src/v4oracle/numerics.rs:68-139 (device twin f2e4m3_rne,
 * crates/backend/kernels/formats.hpp:245-264): nearest even everywhere, subnormals included;
 * |x| >= 464 saturates to 0x7e; |x| <= 2^-10 is signed zero; NaN -> 0x7f. */
uint8_t ro_e4m3_encode_rne(float x);
void ro_e4m3_encode_rne_n(const float* x, uint8_t* out, size_t n);

/* numerics.rs:202-218 (device: crates/backend/kernels/actquant.hpp:69-81): 2^ceil(log2(amax *
 * max_inv)) by exponent-field surgery. */
float ro_fast_round_scale(float amax, float max_inv);

/* crates/backend/kernels/mla.hip:319-338 and its launcher :527-548 (CPU statement:
 * numerics.rs:245-285 act_quant_inplace with round_scale = true). For every row r < rows and
 * block b < n / block: amax = max(1e-4, |src[r*row_stride + b*block + i]|), s =
 * fast_round_scale(amax, 1/448), dst[..] = decode(encode_rne(clamp(src[..] / s, +-448))) * s.
 * Dims [n, row_stride) of a row are not touched. Returns the launcher's guard code (0, 1001,
 * 1002, 1004) and does nothing when it is non-zero. src == dst is the in-place form. */
int ro_act_quant_f8_prefix(const float* src, float* dst, int rows, int row_stride, int n,
                           int block);

/* crates/engine/src/v4/select.rs:153-188 scored_rows: for query row t < rows, limit =
 * prefill ? min((t + 1) / ratio, n_comp) : n_comp; the min(index_topk, n_comp) best of
 * scores[t*n_comp + 0..limit) under f32 total order (descending; ties to the lower index),
 * written ascending as index + offset, then -1 out to k = min(index_topk, n_comp) columns.
 * out is [rows][k]. Returns k, or -1 for a non-positive argument. */
int ro_v4_scored_rows(const float* scores, int rows, int n_comp, int ratio, int index_topk,
                      int prefill, int offset, int32_t* out);

/* crates/engine/src/v4/select.rs:334-400 (Sel::shape, Sel::n_comp): rows = seqlen at prefill
 * (start_pos == 0), 1 at decode; cols = window columns (min(seqlen, win) at prefill, win at
 * decode) + compressed columns ((start_pos + rows) / ratio; none when ratio == 0). Returns 0, or
 * 1001 (win <= 0, seqlen <= 0, negative start_pos / ratio / index_topk), 1005 (decode with
 * seqlen != 1: select.rs:78-86), 1006 (ratio == 4, the indexed class of geometry.rs:86-92,
 * 128-130, with more live blocks than index_topk: the positional rule refuses, select.rs:363-383). */
int ro_sel_shape(int win, int ratio, int index_topk, int seqlen, int start_pos, int* rows,
                 int* cols);
/* select.rs:395-408 Sel::gather = window_rows (:195-216) ‖ compressed_rows (:224-241) at
 * compress_offset (:268-270), row-major [rows][cols] with -1 for masked cells. Returns
 * ro_sel_shape's code and writes nothing when it is non-zero. */
int ro_sel_gather(int win, int ratio, int index_topk, int seqlen, int start_pos, int32_t* out);
/* select.rs:418-434 Sel::gather_scored over scored_rows(scores [rows][n_comp]) : the same window
 * fill, then the min(index_topk, n_comp) scored columns. cols_out receives the row width.
 * Returns 0, 1001 (as above, or ratio == 0: a scored selection needs a compressor), 1005. */
int ro_sel_gather_scored(const float* scores, int n_comp, int win, int ratio, int index_topk,
                         int seqlen, int start_pos, int32_t* out, int* cols_out);

/* crates/engine/src/v4/attn.rs:343-378 write_ring: decode copies kv row 0 into slot
 * start_pos % win; a prompt of s <= win rows seeds slots [0, s); a longer one seeds every slot
 * with the last win positions, position t in slot t % win. cache is [win][hd]. Returns 0 or
 * 1001 / 1005 as ro_sel_shape. */
int ro_ring_write(const float* kv, float* cache, int win, int hd, int seqlen, int start_pos);

/* crates/oracles/src/v4oracle/attention.rs:118-193 sparse_attn / attn_head (device twin
 * gather_attn_shared_kv, crates/backend/kernels/attn.hip:358-443): for query t < m and head
 * hh < h, over the slots j < topk with idxs[t*topk + j] >= 0 in ascending j:
 * logit = (sum_i q[i] * kv[idx][i], ascending i) * scale; mx their maximum;
 * e = expf(logit - mx); sum += e; acc[i] += e * kv[idx][i]; then sum += expf(sink[hh] - mx)
 * and o = bf16_round(acc[i] / sum). A query with no live slot gets NaN (the device kernel's
 * rule; the reference's CPU oracle asserts instead). o is [m][h][d]. Returns 0 or 1001. */
int ro_sparse_attn(const float* q, const float* kv, const float* sink, const int32_t* idxs, int m,
                   int h, int d, int topk, float scale, float* o);

/* ---- the compressor's pooling stage: crates/backend/kernels/kvcompress.hip:103-384 and its
 * launchers :386-478; CPU statement crates/oracles/src/v4oracle/compress.rs:42-199 with
 * rmsnorm / rope_row / softmax_strided of forward.rs:353-383,427-456,557-580 ---- */

/* kvcompress.hip:40-48. cd = coff * d and ents = coff * ratio are derived and checked. */
typedef struct {
    int ratio;
    int coff;
    int d;
    int cd;
    int ents;
    int rd;
    float eps;
} ro_comp_geom;

/* The launchers' shared guard (kvcompress.hip:386-405): 0, 1001, 1002, 1003, 1004 or 1010. */
int ro_compress_guard(const ro_comp_geom* p);

/* kvcompress.hip:227-262 + :419-437. kv, score: [s][cd]; ape: [ratio][cd]; the two states:
 * [coff * ratio][cd]. Returns the launcher's code (1000, the guard's, 1005, 1008, or 0). */
int ro_kv_compress_deposit(const float* kv, const float* score, const float* ape, float* kv_state,
                           float* score_state, const ro_comp_geom* p, int s, int slot0);

/* kvcompress.hip:278-319 + :439-456: nblk pooled, normed and rotated rows into out[nblk][d].
 * norm: [d]; freqs: [positions][rd] as (cos, sin) pairs. Code 1000 / guard / 1006 / 0. */
int ro_kv_compress_prefill(const float* kv, const float* score, const float* ape,
                           const float* norm, const float* freqs, float* out,
                           const ro_comp_geom* p, int nblk);

/* kvcompress.hip:332-382 + :458-478: pool the completed window out of the state into out[d],
 * then slide the window when overlapping. Code 1000 / guard / 1007 / 1009 / 0. */
int ro_kv_compress_decode(float* kv_state, float* score_state, const float* norm,
                          const float* freqs, float* out, const ro_comp_geom* p, int start_pos);

/* ---- the indexer's spread and block scorer (crates/backend/kernels/blockindex.hip) ---- */

/* formats.hpp:285-293 and its decode table {0, .5, 1, 1.5, 2, 3, 4, 6}; bit 3 is the sign. */
uint8_t ro_e2m1_encode(float x);
float ro_e2m1_decode(uint8_t code);

/* crates/oracles/src/v4oracle/numerics.rs:324-353, n a power of two, in place. */
void ro_hadamard_rotate(float* row, int n);

/* numerics.rs:245-298 with actquant.hpp:45-51's constants, in place over n values. */
void ro_fp4_act_quant_inplace(float* row, int n, int block);

/* blockindex.hip:99-136 + :241-262, x: [rows][d] in place. Code 1001-1004 or 0. */
int ro_act_quant_f4_rotated(float* x, int rows, int d);

/* blockindex.hip:209-235 + :264-281. Code 1001, 1005 or 0. */
int ro_index_score_blocks(const float* q, const float* kv, const float* w, float* score, int s,
                          int n_comp, int heads, int hd);

#ifdef __cplusplus
}
#endif
#endif
