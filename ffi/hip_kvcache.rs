//! Rust side of the gfx950 KV-cache library: the rows a maintainer adds to rivoli's backend.
//!
//! Text, not a compiled crate (the build image has no Rust toolchain): drop it next to
//! `crates/backend/src/hip_attn.rs` as `hip_kvcache.rs`, add `mod hip_kvcache;` and
//! `pub use hip_kvcache::*;` beside the existing `hip_attn` lines of `crates/backend/src/hip.rs`,
//! and link `librivoli_kvcache.so` in place of the objects `build.rs` makes from
//! `kernels/{fwd,indexer,attn,mla,kvcompress}.hip`. It uses the backend's own DSL
//! (`launchers!`, `abi_ty!`, `ensure_hip_status`: `crates/backend/src/hip.rs:147-221,328-336`):
//! one row per C entry point, the argument list in the C order, `usize as i32` where the C side
//! takes an `int` count. Every row below is a symbol the reference does not have; the
//! reference's own rows listed at the end bind to this library unchanged.
//!
//! `tests/test_abi_drift.py` parses this file, `include/rivoli_kvcache.h`, the ctypes table in
//! `rivoli_amd/hip.py` and (where the reference tree is mounted) the prototypes in the
//! reference's `kernels/*.hip`, and fails on any difference in argument count, order, name
//! or kind.
use core::ffi::c_void;

use crate::hip::{abi_ty, ensure_hip_status, launchers};
use crate::Result;

launchers! {
    /// Quantize-and-append `n_tokens` bf16 rows into fp8 pages through a slot mapping
    /// (one f32 scale per token). Negative slots are padding.
    ///
    /// # Safety
    /// Device pointers live until `stream` drains: `rows` (`n_tokens*width` bf16),
    /// `slot_mapping` (`n_tokens` i32), `pool` (`n_pages` pages of
    /// [`kv_page_bytes`] bytes, 16-byte aligned), `bad_slots` (one u32 or null).
    launch_kv_append_paged -> rivoli_kv_append_paged, "kv_append_paged" (
        rows: *const u16,
        slot_mapping: *const i32,
        pool: *mut u8,
        n_tokens: usize as i32,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_slots: *mut u32,
        stream: *mut c_void,
    );

    /// `append_kv` for a prefill chunk of consecutive rows, one launch, on a stream.
    launch_append_kv_rows -> rivoli_append_kv_rows, "append_kv_rows" (
        latent: *const f32,
        rope: *const f32,
        lc8: *mut u8,
        lscale: *mut f32,
        rc: *mut u16,
        pos0: usize as i32,
        n_tokens: usize as i32,
        kvl: usize as i32,
        ropn: usize as i32,
        n_blocks: usize as i32,
        stream: *mut c_void,
    );

    /// Block-table gather + dequantize of every sequence's context to packed bf16 rows.
    launch_kv_gather_paged -> rivoli_kv_gather_paged, "kv_gather_paged" (
        pool: *const u8,
        block_table: *const i32,
        seq_lens: *const i32,
        cu_seqlens: *const i32,
        out: *mut u16,
        n_seqs: usize as i32,
        max_blocks_per_seq: usize as i32,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_pages: *mut u32,
        stream: *mut c_void,
    );

    /// rivoli_kv_gather_paged for a caller that knows how many rows the batch holds (it sized `out`
    /// by that number): total_tokens >= the sum of seq_lens.
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_kv_gather_paged_packed -> rivoli_kv_gather_paged_packed, "kv_gather_paged_packed" (
        pool: *const u8,
        block_table: *const i32,
        seq_lens: *const i32,
        cu_seqlens: *const i32,
        out: *mut u16,
        n_seqs: usize as i32,
        max_blocks_per_seq: usize as i32,
        total_tokens: usize as i64,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_pages: *mut u32,
        stream: *mut c_void,
    );

    /// A decode step's cache work in one launch: append one new row per sequence (`seq_lens`
    /// already counts it, `slot_mapping[s]` is that token's slot), then gather every context.
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_kv_append_gather_paged -> rivoli_kv_append_gather_paged, "kv_append_gather_paged" (
        new_rows: *const u16,
        slot_mapping: *const i32,
        pool: *mut u8,
        block_table: *const i32,
        seq_lens: *const i32,
        cu_seqlens: *const i32,
        out: *mut u16,
        n_seqs: usize as i32,
        max_blocks_per_seq: usize as i32,
        total_tokens: usize as i64,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_slots: *mut u32,
        bad_pages: *mut u32,
        stream: *mut c_void,
    );

    /// Sparse row gather + dequantize: `rows[q*k + j]` of sequence `q`, `j < n_rows[q]`.
    launch_kv_gather_rows_paged -> rivoli_kv_gather_rows_paged, "kv_gather_rows_paged" (
        pool: *const u8,
        block_table: *const i32,
        rows: *const u32,
        n_rows: *const i32,
        out: *mut u16,
        n_queries: usize as i32,
        k: usize as i32,
        max_blocks_per_seq: usize as i32,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_rows: *mut u32,
        stream: *mut c_void,
    );

    /// `index_topk` for many queries in one launch: `rows[q*k ..]`, ascending.
    launch_index_topk_batched -> rivoli_index_topk_batched, "index_topk_batched" (
        scores: *const f32,
        n_queries: usize as i32,
        stride: usize as i32,
        nts: *const i32,
        nt: usize as i32,
        k: usize as i32,
        rows: *mut u32,
        workspace: *mut c_void,
        stream: *mut c_void,
    );

    /// The DSA step the reference runs as index_topk followed by an attend over `rows`, with "no
    /// D2H, no host top-k, and no device_sync" between them
    /// (crates/backend/src/hip_attn.rs:478-495), for a consumer that wants the selected rows as
    /// bf16: rivoli_index_topk_batched and rivoli_kv_gather_rows_paged in one call.
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_dsa_select_gather_paged -> rivoli_dsa_select_gather_paged, "dsa_select_gather_paged" (
        scores: *const f32,
        n_queries: usize as i32,
        stride: usize as i32,
        nts: *const i32,
        nt: usize as i32,
        k: usize as i32,
        rows: *mut u32,
        workspace: *mut c_void,
        hist_ready: i32,
        pool: *const u8,
        block_table: *const i32,
        out: *mut u16,
        max_blocks_per_seq: usize as i32,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_rows: *mut u32,
        stream: *mut c_void,
    );

    /// rivoli_dsa_select_gather_paged for callers that cannot allocate device memory (code under
    /// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_dsa_select_gather_paged_noalloc -> rivoli_dsa_select_gather_paged_noalloc, "dsa_select_gather_paged_noalloc" (
        scores: *const f32,
        n_queries: usize as i32,
        stride: usize as i32,
        nts: *const i32,
        nt: usize as i32,
        k: usize as i32,
        rows: *mut u32,
        pool: *const u8,
        block_table: *const i32,
        out: *mut u16,
        max_blocks_per_seq: usize as i32,
        width: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_rows: *mut u32,
        stream: *mut c_void,
    );

    /// The paged, batched form: query qi (q [n_queries][nh][hd], w [n_queries][nh]) scores its
    /// first nts[qi] tokens (nt when nts is null) through block_table[qi] over the paged key cache
    /// kpool[n_pages*page_tokens][hd] bf16, into scores[qi*stride + t].
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_index_score_paged -> rivoli_index_score_paged, "index_score_paged" (
        q: *const f32,
        w: *const f32,
        kpool: *const u16,
        block_table: *const i32,
        nts: *const i32,
        heads: *const u32,
        n_queries: usize as i32,
        max_blocks_per_seq: usize as i32,
        stride: usize as i32,
        nt: usize as i32,
        nh: usize as i32,
        nact: usize as i32,
        hd: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        wscale: f32,
        dscale: f32,
        scores: *mut f32,
        stream: *mut c_void,
    );

    /// rivoli_index_score_paged that also does the first step of the selection that follows it (the
    /// score -> top-k fusion the reference's design aims at, crates/backend/kernels/
    /// indexer.hip:1-13): while a score is still in a register its selection key's top 12 bits are
    /// counted into topk_workspace (the rivoli_index_topk_workspace_bytes(n_queries, nt) buffer the
    /// selection will be handed, zero-filled as described there), so rivoli_dsa_select_gather_paged
    /// (hist_ready = 1) does not sweep the scores for it.
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_index_score_paged_hist -> rivoli_index_score_paged_hist, "index_score_paged_hist" (
        q: *const f32,
        w: *const f32,
        kpool: *const u16,
        block_table: *const i32,
        nts: *const i32,
        heads: *const u32,
        n_queries: usize as i32,
        max_blocks_per_seq: usize as i32,
        stride: usize as i32,
        nt: usize as i32,
        nh: usize as i32,
        nact: usize as i32,
        hd: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        wscale: f32,
        dscale: f32,
        scores: *mut f32,
        topk_workspace: *mut c_void,
        stream: *mut c_void,
    );

    /// Paged form of rivoli_index_append for many tokens: kpool[slot_mapping[t]*hd + i] =
    /// bf16(k[t*hd + i]).
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_index_append_paged -> rivoli_index_append_paged, "index_append_paged" (
        k: *const f32,
        slot_mapping: *const i32,
        kpool: *mut u16,
        n_tokens: usize as i32,
        hd: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        bad_slots: *mut u32,
        stream: *mut c_void,
    );

    /// `launch_attend` for a whole decode batch over the paged fp8 cache, dense (`rows`
    /// null, `seq_lens` given) or over DSA row lists (`rows[s*max_rows + j]`, `j <
    /// n_rows[s]`). `partial`: [`attend_paged_scratch_floats`] floats, or null when that is 0.
    /// `precise`: 2 = q and softmax weights as bf16 hi + lo (parity), 1 = q only, 0 = bf16;
    /// 4 / 3 = both contractions on the 8-bit matrix instructions (q as three / two e4m3 terms):
    /// the fastest modes, 4 inside the reference's bar for this kernel.
    launch_attend_paged -> rivoli_mla_attend_paged, "mla_attend_paged" (
        qabs: *const f32,
        qrope: *const f32,
        pool: *const u8,
        block_table: *const i32,
        seq_lens: *const i32,
        rows: *const u32,
        n_rows: *const i32,
        n_seqs: usize as i32,
        h: usize as i32,
        max_rows: usize as i32,
        max_blocks_per_seq: usize as i32,
        kvl: usize as i32,
        rope: usize as i32,
        page_tokens: usize as i32,
        n_pages: usize as i32,
        scale: f32,
        precise: i32,
        clat: *mut f32,
        partial: *mut f32,
        bad_rows: *mut u32,
        stream: *mut c_void,
    );

    /// The scored block selection of `v4::select::scored_rows`, on the device: no D2H of the
    /// score matrix, no host sort, no upload of the index rectangle.
    ///
    /// # Safety
    /// `scores` is `rows * n_comp` f32 as `launch_index_score_blocks` wrote it; `out` is
    /// `rows * min(index_topk, n_comp)` i32; both live until `stream` drains.
    launch_index_select_blocks -> rivoli_index_select_blocks, "index_select_blocks" (
        scores: *const f32,
        rows: usize as i32,
        n_comp: usize as i32,
        ratio: usize as i32,
        index_topk: usize as i32,
        prefill: i32,
        offset: usize as i32,
        out: *mut i32,
        stream: *mut c_void,
    );

    /// `launch_index_score_blocks` (crates/backend/src/hip.rs:497-520) for a prefill: only the
    /// entries a row's selection can rank (block < (t + 1) / ratio, in groups of 64 blocks) are
    /// computed, bit-identical to the full kernel's; the rest of `score` is left untouched.
    ///
    /// # Safety
    /// As `launch_index_score_blocks`: `q` is `s * heads * hd`, `kv` `n_comp * hd`, `w`
    /// `s * heads`, `score` `s * n_comp` f32; all live until `stream` drains.
    launch_index_score_blocks_prefill -> rivoli_index_score_blocks_prefill, "index_score_blocks_prefill" (
        q: *const f32,
        kv: *const f32,
        w: *const f32,
        score: *mut f32,
        s: usize as i32,
        n_comp: usize as i32,
        heads: usize as i32,
        hd: usize as i32,
        ratio: usize as i32,
        stream: *mut c_void,
    );

    /// `Sel::gather` on the device: the `[window | positional blocks]` rectangle written where the
    /// attend reads it, instead of a host fill plus `upload_selection`. The shape check stays
    /// on the host: `rivoli_sel_shape` is `Sel::shape` (1005 = multi-row decode, 1006 = past the
    /// indexed layer's cap).
    ///
    /// # Safety
    /// `out` is `rows * cols` i32 of `sel_shape`; live until `stream` drains.
    launch_sel_gather -> rivoli_sel_gather, "sel_gather" (
        win: usize as i32,
        ratio: usize as i32,
        index_topk: usize as i32,
        seqlen: usize as i32,
        start_pos: usize as i32,
        out: *mut i32,
        stream: *mut c_void,
    );

    /// `Sel::gather_scored(scored_rows(scores))` on the device, both halves of the rectangle.
    ///
    /// # Safety
    /// `scores` is `rows * n_comp` f32; `out` is `rows * (window columns + min(index_topk,
    /// n_comp))` i32; `cols_out` is a host `i32` or null.
    launch_sel_gather_scored -> rivoli_sel_gather_scored, "sel_gather_scored" (
        scores: *const f32,
        n_comp: usize as i32,
        win: usize as i32,
        ratio: usize as i32,
        index_topk: usize as i32,
        seqlen: usize as i32,
        start_pos: usize as i32,
        out: *mut i32,
        cols_out: *mut i32,
        stream: *mut c_void,
    );

    /// `write_ring`'s one or two `memcpy_dtod_async` calls as one launch.
    ///
    /// # Safety
    /// `cache` holds `win * hd` f32, `kv` the step's rows; distinct allocations.
    launch_kv_ring_write -> rivoli_kv_ring_write, "kv_ring_write" (
        kv: *const f32,
        cache: *mut f32,
        win: usize as i32,
        hd: usize as i32,
        seqlen: usize as i32,
        start_pos: usize as i32,
        stream: *mut c_void,
    );

    /// Replaces crates/backend/kernels/attn.hip:446-465 (rivoli_gather_attn_shared_kv; Rust row
    /// launch_gather_attn_shared_kv, caller crates/engine/src/v4/attn.rs:304-330), same signature:
    /// multi-query attention with one d-wide row serving as key and value for all h heads, over the
    /// explicit index list idxs [m][topk] into kv [rows][d] (-1 masks a slot, which is then never
    /// dereferenced); sink [h] joins the softmax denominator only, exp(sink - max) after the
    /// running-max shift (attn.hip:333-343); a query with no live slot gets NaN (attn.hip:344-351);
    /// o [m][h][d] is the quotient rounded to bf16, stored as f32.
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_gather_attn_shared_kv_bounded -> rivoli_gather_attn_shared_kv_bounded, "gather_attn_shared_kv_bounded" (
        q: *const f32,
        kv: *const f32,
        sink: *const f32,
        idxs: *const i32,
        m: usize as i32,
        h: usize as i32,
        d: usize as i32,
        topk: usize as i32,
        n_kv: usize as i32,
        scale: f32,
        precise: i32,
        o: *mut f32,
        stream: *mut c_void,
    );

    /// `launch_gather_attn_shared_kv` with the rows of `kv` stated (an index at or past `n_kv` is
    /// masked rather than read), a precision mode, and a partial buffer of
    /// `gather_attn_scratch_floats(m, h, d, topk)` f32 that lets one query's list be shared
    /// among workgroups — the decode call, where `m == 1`.
    ///
    /// # Safety
    /// As `launch_gather_attn_shared_kv`; `partial` may be null when the sizing function
    /// returns 0.
    launch_gather_attn_shared_kv_split -> rivoli_gather_attn_shared_kv_split, "gather_attn_shared_kv" (
        q: *const f32,
        kv: *const f32,
        sink: *const f32,
        idxs: *const i32,
        m: usize as i32,
        h: usize as i32,
        d: usize as i32,
        topk: usize as i32,
        n_kv: usize as i32,
        scale: f32,
        precise: i32,
        o: *mut f32,
        partial: *mut f32,
        stream: *mut c_void,
    );

    /// Element codecs as launchers (what formats.hpp:42-57,99-106 and fwd.hip:20-45 are to the
    /// reference's kernels), for census tests of the device codecs on arbitrary inputs:
    /// e4m3_encode: out[i] = f32_to_e4m3(x[i]) (rule of crates/core/src/num.rs:128-152)
    /// e4m3_dequant_bf16: out[i] = bf16(e4m3_to_f32(c[i]) * scale) bf16_encode: out[i] =
    /// f32_to_bf16(x[i]).
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_codec_e4m3_encode -> rivoli_codec_e4m3_encode, "codec_e4m3_encode" (
        x: *const f32,
        out: *mut u8,
        n: usize as i64,
        stream: *mut c_void,
    );

    /// Element codecs as launchers (what formats.hpp:42-57,99-106 and fwd.hip:20-45 are to the
    /// reference's kernels), for census tests of the device codecs on arbitrary inputs:
    /// e4m3_encode: out[i] = f32_to_e4m3(x[i]) (rule of crates/core/src/num.rs:128-152)
    /// e4m3_dequant_bf16: out[i] = bf16(e4m3_to_f32(c[i]) * scale) bf16_encode: out[i] =
    /// f32_to_bf16(x[i]).
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_codec_e4m3_dequant_bf16 -> rivoli_codec_e4m3_dequant_bf16, "codec_e4m3_dequant_bf16" (
        codes: *const u8,
        scale: f32,
        out: *mut u16,
        n: usize as i64,
        stream: *mut c_void,
    );

    /// Element codecs as launchers (what formats.hpp:42-57,99-106 and fwd.hip:20-45 are to the
    /// reference's kernels), for census tests of the device codecs on arbitrary inputs:
    /// e4m3_encode: out[i] = f32_to_e4m3(x[i]) (rule of crates/core/src/num.rs:128-152)
    /// e4m3_dequant_bf16: out[i] = bf16(e4m3_to_f32(c[i]) * scale) bf16_encode: out[i] =
    /// f32_to_bf16(x[i]).
    /// See `include/rivoli_kvcache.h` for the full contract.
    launch_codec_bf16_encode -> rivoli_codec_bf16_encode, "codec_bf16_encode" (
        x: *const f32,
        out: *mut u16,
        n: usize as i64,
        stream: *mut c_void,
    );

}

// Sizing and shape functions: pure host arithmetic, no launch, no status code to map.
unsafe extern "C" {
    fn rivoli_kv_page_bytes(page_tokens: i32, width: i32) -> usize;
    fn rivoli_index_topk_workspace_bytes(n_queries: i32, nt: i32) -> usize;
    fn rivoli_mla_attend_paged_scratch_floats(n_seqs: i32, h: i32, max_rows: i32) -> usize;
    fn rivoli_sel_shape(win: i32, ratio: i32, index_topk: i32, seqlen: i32, start_pos: i32, rows: *mut i32, cols: *mut i32) -> i32;
    fn rivoli_gather_attn_scratch_floats(m: i32, h: i32, d: i32, topk: i32) -> usize;
}

/// Bytes of one page: `page_tokens * width` codes followed by `page_tokens` f32 scales.
pub fn kv_page_bytes(page_tokens: usize, width: usize) -> usize {
    // SAFETY: pure host function, no pointers.
    unsafe { rivoli_kv_page_bytes(page_tokens as i32, width as i32) }
}

/// Bytes of the selection workspace a split top-k of this shape wants (zero-filled once).
pub fn index_topk_workspace_bytes(n_queries: usize, nt: usize) -> usize {
    // SAFETY: pure host function, no pointers.
    unsafe { rivoli_index_topk_workspace_bytes(n_queries as i32, nt as i32) }
}

/// f32 elements of the partial buffer `launch_attend_paged` wants for this shape (0 = none).
pub fn attend_paged_scratch_floats(n_seqs: usize, h: usize, max_rows: usize) -> usize {
    // SAFETY: pure host function, no pointers.
    unsafe { rivoli_mla_attend_paged_scratch_floats(n_seqs as i32, h as i32, max_rows as i32) }
}

/// f32 elements of the partial buffer `launch_gather_attn_shared_kv_split` wants (0 = none).
pub fn gather_attn_scratch_floats(m: usize, h: usize, d: usize, topk: usize) -> usize {
    // SAFETY: pure host function, no pointers.
    unsafe { rivoli_gather_attn_scratch_floats(m as i32, h as i32, d as i32, topk as i32) }
}

/// Rows and columns of a selection rectangle, or the guard code `Sel::shape` would refuse with.
pub fn sel_shape(win: usize, ratio: usize, index_topk: usize, seqlen: usize, start_pos: usize)
                 -> Result<(usize, usize)> {
    let (mut rows, mut cols) = (0i32, 0i32);
    // SAFETY: the two out-pointers are live locals.
    let r = unsafe {
        rivoli_sel_shape(win as i32, ratio as i32, index_topk as i32, seqlen as i32, start_pos as i32,
                         &mut rows, &mut cols)
    };
    ensure_hip_status(r, "sel_shape")?;
    Ok((rows as usize, cols as usize))
}

// The reference's own rows bind to this library unchanged (same symbol, same argument list):
//   rivoli_append_kv                     launch_append_kv, crates/backend/src/hip_attn.rs:137-147
//   rivoli_index_append                  launch_index_append, hip_attn.rs:450-455
//   rivoli_index_topk                    launch_index_topk, hip_attn.rs:490-495
//   rivoli_index_score                   launch_index_score, hip_attn.rs:464-476
//   rivoli_hash_rows                     launch_hash_rows, crates/backend/src/hip.rs:586-604
//   rivoli_mla_attend                    launch_attend, hip_attn.rs:113-128
//   rivoli_mla_attend_scratch_floats     attend_scratch_floats, hip_attn.rs:113-128
//   rivoli_device_sync                   device_sync, hip.rs:339-342
//   rivoli_act_quant_f8_prefix           launch_act_quant_f8_prefix, hip_attn.rs
//   rivoli_gather_attn_shared_kv         launch_gather_attn_shared_kv, hip_attn.rs
//   rivoli_kv_compress_deposit           launch_kv_compress_deposit, hip_attn.rs:547-605
//   rivoli_kv_compress_prefill           launch_kv_compress_prefill, hip_attn.rs:547-605
//   rivoli_kv_compress_decode            launch_kv_compress_decode, hip_attn.rs:547-605
//   rivoli_act_quant_f4_rotated          launch_act_quant_f4_rotated, hip_linalg.rs:620
//   rivoli_index_score_blocks            launch_index_score_blocks, hip.rs:497-520
