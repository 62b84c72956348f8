"""The launcher wall: one `launch_*` per `extern "C" int rivoli_*` entry point.

Host-side mirror of the reference's `launchers!` rows (crates/backend/src/hip.rs:196-221,
crates/backend/src/hip_attn.rs:113-147,450-495): every wrapper narrows its dims to C int,
calls the symbol, and maps the return code the way `ensure_hip_status` does
(crates/backend/src/hip.rs:328-336) — 0 ok, positive = argument guard, negative = HIP error.
Pointers are device addresses: pass a torch tensor (its data_ptr is taken), an int, or None.
There is no fallback: if the HIP library has not been built, importing a launcher fails.
"""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB_PATH

NULL_STREAM = None


class LaunchError(RuntimeError):
    """What `ensure_hip_status` bails with; `.code` keeps the raw launcher return."""

    def __init__(self, name: str, code: int):
        self.name, self.code = name, code
        if code > 0:
            super().__init__(f"{name}: argument guard rejected ({code})")
        else:
            super().__init__(f"{name}: HIP error {-code}")


def ensure_hip_status(code: int, name: str) -> None:
    if code != 0:
        raise LaunchError(name, code)


_LIB = None

_VP, _I, _LL, _ULL, _F = C.c_void_p, C.c_int, C.c_longlong, C.c_ulonglong, C.c_float
_SIGNATURES = {
    "rivoli_append_kv": [_VP] * 5 + [_I] * 4,
    "rivoli_append_kv_rows": [_VP] * 5 + [_I] * 5 + [_VP],
    "rivoli_index_append": [_VP, _VP, _I, _I],
    "rivoli_index_topk": [_VP, _I, _I, _VP],
    "rivoli_index_topk_batched": [_VP, _I, _I, _VP, _I, _I, _VP, _VP, _VP],
    "rivoli_index_score": [_VP] * 4 + [_I] * 4 + [_F, _F, _VP],
    "rivoli_index_score_paged": [_VP] * 6 + [_I] * 9 + [_F, _F, _VP, _VP],
    "rivoli_index_score_paged_hist": [_VP] * 6 + [_I] * 9 + [_F, _F, _VP, _VP, _VP],
    "rivoli_dsa_select_gather_paged": [_VP, _I, _I, _VP, _I, _I, _VP, _VP, _I, _VP, _VP, _VP,
                                       _I, _I, _I, _I, _VP, _VP],
    "rivoli_dsa_select_gather_paged_noalloc": [_VP, _I, _I, _VP, _I, _I, _VP, _VP, _VP, _VP,
                                               _I, _I, _I, _I, _VP, _VP],
    "rivoli_index_append_paged": [_VP, _VP, _VP, _I, _I, _I, _I, _VP, _VP],
    "rivoli_hash_rows": [_VP, _I, _I, _ULL, _VP, _VP],
    "rivoli_device_sync": [],
    "rivoli_kv_append_paged": [_VP, _VP, _VP, _I, _I, _I, _I, _VP, _VP],
    "rivoli_kv_gather_paged": [_VP] * 5 + [_I] * 5 + [_VP, _VP],
    "rivoli_kv_gather_paged_packed": [_VP] * 5 + [_I, _I, _LL] + [_I] * 3 + [_VP, _VP],
    "rivoli_kv_append_gather_paged": [_VP] * 7 + [_I, _I, _LL] + [_I] * 3 + [_VP, _VP, _VP],
    "rivoli_kv_gather_rows_paged": [_VP] * 5 + [_I] * 6 + [_VP, _VP],
    "rivoli_mla_attend": [_VP] * 6 + [_I] * 5 + [_F, _VP, _VP],
    "rivoli_mla_attend_paged": [_VP] * 7 + [_I] * 8 + [_F, _I, _VP, _VP, _VP, _VP],
    "rivoli_act_quant_f8_prefix": [_VP, _VP] + [_I] * 4 + [_VP],
    "rivoli_act_quant_f4_rotated": [_VP, _I, _I, _VP],
    "rivoli_index_score_blocks": [_VP] * 4 + [_I] * 4 + [_VP],
    "rivoli_index_score_blocks_prefill": [_VP] * 4 + [_I] * 5 + [_VP],
    "rivoli_index_select_blocks": [_VP] + [_I] * 6 + [_VP, _VP],
    "rivoli_sel_shape": [_I] * 5 + [_VP, _VP],
    "rivoli_sel_gather": [_I] * 5 + [_VP, _VP],
    "rivoli_sel_gather_scored": [_VP] + [_I] * 6 + [_VP, _VP, _VP],
    "rivoli_kv_ring_write": [_VP, _VP] + [_I] * 4 + [_VP],
    "rivoli_gather_attn_shared_kv": [_VP] * 4 + [_I] * 4 + [_F, _VP, _VP],
    "rivoli_gather_attn_shared_kv_bounded": [_VP] * 4 + [_I] * 5 + [_F, _I, _VP, _VP],
    "rivoli_gather_attn_shared_kv_split": [_VP] * 4 + [_I] * 5 + [_F, _I, _VP, _VP, _VP],
    "rivoli_kv_compress_deposit": [_VP] * 6 + [_I, _I, _VP],
    "rivoli_kv_compress_prefill": [_VP] * 5 + [_I, _VP],
    "rivoli_kv_compress_decode": [_VP] * 4 + [_I, _VP],
    "rivoli_codec_e4m3_encode": [_VP, _VP, _LL, _VP],
    "rivoli_codec_e4m3_dequant_bf16": [_VP, _F, _VP, _LL, _VP],
    "rivoli_codec_bf16_encode": [_VP, _VP, _LL, _VP],
}


# the sizing functions: pure host arithmetic, size_t results
_SIZE_SIGNATURES = {
    "rivoli_kv_page_bytes": [_I, _I],
    "rivoli_index_topk_workspace_bytes": [_I, _I],
    "rivoli_mla_attend_paged_scratch_floats": [_I, _I, _I],
    "rivoli_mla_attend_scratch_floats": [_I, _I],
    "rivoli_gather_attn_scratch_floats": [_I, _I, _I, _I],
}


def lib() -> C.CDLL:
    """The loaded HIP library. Raises if it was never built — there is no other path."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m rivoli_amd.build` "
                "(hipcc, gfx950); this package has no CPU fallback")
        # torch ships its own copy of the HIP runtime. A process must end up with ONE runtime:
        # if this library were loaded first it would bring in the system copy, torch would
        # then load its own beside it, and every launch from here would fail with
        # hipErrorNoDevice (the second runtime never sees the device). So torch, which owns
        # the device buffers these launchers are handed, is loaded first whenever it exists.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = C.CDLL(LIB_PATH)
        for name, args in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = C.c_int, args
        for name, args in _SIZE_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = C.c_size_t, args
        _LIB = handle
    return _LIB


def exported_symbols() -> list[str]:
    return sorted(list(_SIGNATURES) + ["rivoli_kv_page_bytes", "rivoli_index_topk_workspace_bytes",
                                       "rivoli_mla_attend_paged_scratch_floats",
                                       "rivoli_mla_attend_scratch_floats", "rivoli_gather_attn_scratch_floats"])


def _p(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()  # torch tensor


def _s(stream):
    if stream is None:
        return None
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream  # torch.cuda.Stream


def device_sync() -> None:
    ensure_hip_status(lib().rivoli_device_sync(), "device_sync")


def kv_page_bytes(page_tokens: int, width: int) -> int:
    return int(lib().rivoli_kv_page_bytes(page_tokens, width))


# ---- reference-signature launchers --------------------------------------------------------

def launch_append_kv(latent, rope, lc8, lscale, rc, pos, kvl, ropn, n_blocks) -> None:
    ensure_hip_status(lib().rivoli_append_kv(_p(latent), _p(rope), _p(lc8), _p(lscale), _p(rc),
                                             pos, kvl, ropn, n_blocks), "append_kv")


def launch_append_kv_rows(latent, rope, lc8, lscale, rc, pos0, n_tokens, kvl, ropn, n_blocks,
                          stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_append_kv_rows(_p(latent), _p(rope), _p(lc8), _p(lscale),
                                                  _p(rc), pos0, n_tokens, kvl, ropn, n_blocks,
                                                  _s(stream)), "append_kv_rows")


def launch_index_append(k, kcache, pos, hd) -> None:
    ensure_hip_status(lib().rivoli_index_append(_p(k), _p(kcache), pos, hd), "index_append")


def launch_index_topk(scores, nt, k, rows) -> None:
    ensure_hip_status(lib().rivoli_index_topk(_p(scores), nt, k, _p(rows)), "index_topk")


def launch_index_score(q, w, kcache, heads, nt, nh, nact, hd, wscale, dscale, scores) -> None:
    ensure_hip_status(lib().rivoli_index_score(_p(q), _p(w), _p(kcache), _p(heads), nt, nh, nact,
                                               hd, wscale, dscale, _p(scores)), "index_score")


def launch_index_score_paged(q, w, kpool, block_table, nts, heads, n_queries, max_blocks_per_seq,
                             stride, nt, nh, nact, hd, page_tokens, n_pages, wscale, dscale,
                             scores, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_index_score_paged(
        _p(q), _p(w), _p(kpool), _p(block_table), _p(nts), _p(heads), n_queries,
        max_blocks_per_seq, stride, nt, nh, nact, hd, page_tokens, n_pages, wscale, dscale,
        _p(scores), _s(stream)), "index_score_paged")


def launch_index_score_paged_hist(q, w, kpool, block_table, nts, heads, n_queries, max_blocks_per_seq,
                                  stride, nt, nh, nact, hd, page_tokens, n_pages, wscale, dscale,
                                  scores, topk_workspace, stream=NULL_STREAM) -> None:
    """index_score_paged that also counts the selection histogram into the top-k workspace."""
    ensure_hip_status(lib().rivoli_index_score_paged_hist(
        _p(q), _p(w), _p(kpool), _p(block_table), _p(nts), _p(heads), n_queries,
        max_blocks_per_seq, stride, nt, nh, nact, hd, page_tokens, n_pages, wscale, dscale,
        _p(scores), _p(topk_workspace), _s(stream)), "index_score_paged_hist")


def launch_index_append_paged(k, slot_mapping, kpool, n_tokens, hd, page_tokens, n_pages,
                              bad_slots=None, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_index_append_paged(_p(k), _p(slot_mapping), _p(kpool), n_tokens,
                                                      hd, page_tokens, n_pages, _p(bad_slots),
                                                      _s(stream)), "index_append_paged")


def launch_hash_rows(x, n, stride, i_base, out, stream=NULL_STREAM) -> None:
    if n > 2 ** 31 - 1:
        raise LaunchError("hash_rows", 1002)  # exceeds the i32 ABI, crates/backend/src/hip.rs:595-598
    ensure_hip_status(lib().rivoli_hash_rows(_p(x), n, stride, i_base, _p(out), _s(stream)),
                      "hash_rows")


# ---- paged, batched launchers -------------------------------------------------------------

def launch_kv_append_paged(rows, slot_mapping, pool, n_tokens, width, page_tokens, n_pages,
                           bad_slots=None, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_append_paged(_p(rows), _p(slot_mapping), _p(pool), n_tokens,
                                                   width, page_tokens, n_pages, _p(bad_slots),
                                                   _s(stream)), "kv_append_paged")


def launch_kv_gather_paged(pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                           max_blocks_per_seq, width, page_tokens, n_pages, bad_pages=None,
                           stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_gather_paged(_p(pool), _p(block_table), _p(seq_lens),
                                                   _p(cu_seqlens), _p(out), n_seqs,
                                                   max_blocks_per_seq, width, page_tokens, n_pages,
                                                   _p(bad_pages), _s(stream)), "kv_gather_paged")


def launch_kv_gather_paged_packed(pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                                  max_blocks_per_seq, total_tokens, width, page_tokens, n_pages,
                                  bad_pages=None, stream=NULL_STREAM) -> None:
    """launch_kv_gather_paged sized by the batch's real token count (>= sum of seq_lens)."""
    ensure_hip_status(lib().rivoli_kv_gather_paged_packed(
        _p(pool), _p(block_table), _p(seq_lens), _p(cu_seqlens), _p(out), n_seqs, max_blocks_per_seq,
        total_tokens, width, page_tokens, n_pages, _p(bad_pages), _s(stream)), "kv_gather_paged_packed")


def launch_kv_append_gather_paged(new_rows, slot_mapping, pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                                  max_blocks_per_seq, total_tokens, width, page_tokens, n_pages,
                                  bad_slots=None, bad_pages=None, stream=NULL_STREAM) -> None:
    """One launch for a decode step's cache work: append one new row per sequence (seq_lens already
    counts it; slot_mapping[s] is that token's slot), then gather every context."""
    ensure_hip_status(lib().rivoli_kv_append_gather_paged(
        _p(new_rows), _p(slot_mapping), _p(pool), _p(block_table), _p(seq_lens), _p(cu_seqlens), _p(out), n_seqs,
        max_blocks_per_seq, total_tokens, width, page_tokens, n_pages, _p(bad_slots), _p(bad_pages),
        _s(stream)), "kv_append_gather_paged")


def launch_kv_gather_rows_paged(pool, block_table, rows, n_rows, out, n_queries, k,
                                max_blocks_per_seq, width, page_tokens, n_pages, bad_rows=None,
                                stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_gather_rows_paged(_p(pool), _p(block_table), _p(rows),
                                                        _p(n_rows), _p(out), n_queries, k,
                                                        max_blocks_per_seq, width, page_tokens,
                                                        n_pages, _p(bad_rows), _s(stream)),
                      "kv_gather_rows_paged")


def index_topk_workspace_bytes(n_queries: int, nt: int) -> int:
    return int(lib().rivoli_index_topk_workspace_bytes(n_queries, nt))


def launch_index_topk_batched(scores, n_queries, stride, nts, nt, k, rows, workspace=None,
                              stream=NULL_STREAM) -> None:
    """`workspace`: a zero-filled device buffer of index_topk_workspace_bytes(n_queries, nt)
    bytes (left zero-filled by every call), or None for one workgroup per query."""
    ensure_hip_status(lib().rivoli_index_topk_batched(_p(scores), n_queries, stride, _p(nts), nt,
                                                      k, _p(rows), _p(workspace), _s(stream)),
                      "index_topk_batched")


def launch_dsa_select_gather_paged(scores, n_queries, stride, nts, nt, k, rows, workspace, hist_ready,
                                   pool, block_table, out, max_blocks_per_seq, width, page_tokens,
                                   n_pages, bad_rows=None, stream=NULL_STREAM) -> None:
    """Top-k selection and the sparse gather of the selected rows in one call."""
    ensure_hip_status(lib().rivoli_dsa_select_gather_paged(
        _p(scores), n_queries, stride, _p(nts), nt, k, _p(rows), _p(workspace), 1 if hist_ready else 0,
        _p(pool), _p(block_table), _p(out), max_blocks_per_seq, width, page_tokens, n_pages,
        _p(bad_rows), _s(stream)), "dsa_select_gather_paged")


def launch_dsa_select_gather_paged_noalloc(scores, n_queries, stride, nts, nt, k, rows, pool, block_table,
                                           out, max_blocks_per_seq, width, page_tokens, n_pages,
                                           bad_rows=None, stream=NULL_STREAM) -> None:
    """launch_dsa_select_gather_paged over the library's own workspace: allocates nothing."""
    ensure_hip_status(lib().rivoli_dsa_select_gather_paged_noalloc(
        _p(scores), n_queries, stride, _p(nts), nt, k, _p(rows), _p(pool), _p(block_table), _p(out),
        max_blocks_per_seq, width, page_tokens, n_pages, _p(bad_rows), _s(stream)),
        "dsa_select_gather_paged_noalloc")


# ---- attention: the reference's single-token launcher over its linear slabs ----------------

def attend_scratch_floats(H: int, kvl: int) -> int:
    """crates/backend/src/hip_attn.rs: attend_scratch_floats."""
    return int(lib().rivoli_mla_attend_scratch_floats(H, kvl))


def launch_attend(qabs, qrope, lc8, lscale, rc, rows, H, nr, kvl, rope, n_blocks, scale, clat,
                  partial) -> None:
    """crates/backend/src/hip_attn.rs:113-128 (launch_attend -> rivoli_mla_attend)."""
    ensure_hip_status(lib().rivoli_mla_attend(_p(qabs), _p(qrope), _p(lc8), _p(lscale), _p(rc), _p(rows),
                                              H, nr, kvl, rope, n_blocks, scale, _p(clat), _p(partial)),
                      "mla_attend")


# ---- attention over the paged cache -------------------------------------------------------

def mla_attend_paged_scratch_floats(n_seqs: int, H: int, max_rows: int) -> int:
    return int(lib().rivoli_mla_attend_paged_scratch_floats(n_seqs, H, max_rows))


def launch_mla_attend_paged(qabs, qrope, pool, block_table, seq_lens, rows, n_rows, n_seqs, H,
                            max_rows, max_blocks_per_seq, kvl, rope, page_tokens, n_pages, scale,
                            precise, clat, partial, bad_rows=None, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_mla_attend_paged(
        _p(qabs), _p(qrope), _p(pool), _p(block_table), _p(seq_lens), _p(rows), _p(n_rows), n_seqs,
        H, max_rows, max_blocks_per_seq, kvl, rope, page_tokens, n_pages, scale, int(precise),
        _p(clat), _p(partial), _p(bad_rows), _s(stream)), "mla_attend_paged")


# ---- the second cache format: simulated-fp8 rows, scored block selection -------------------

def launch_act_quant_f8_prefix(src, dst, rows, row_stride, n, block, stream=NULL_STREAM) -> None:
    """crates/backend/src/hip_attn.rs launch_act_quant_f8_prefix: quantize-dequantize dims
    [0, n) of every row in blocks of `block`; src may be dst."""
    ensure_hip_status(lib().rivoli_act_quant_f8_prefix(_p(src), _p(dst), rows, row_stride, n, block,
                                                       _s(stream)), "act_quant_f8_prefix")


def launch_act_quant_f4_rotated(x, rows, d, stream=NULL_STREAM) -> None:
    """crates/backend/src/hip_linalg.rs:620 launch_act_quant_f4_rotated: the Hadamard + fp4
    spread of every row of x [rows][d], in place."""
    ensure_hip_status(lib().rivoli_act_quant_f4_rotated(_p(x), rows, d, _s(stream)), "act_quant_f4_rotated")


def launch_index_score_blocks(q, kv, w, score, s, n_comp, heads, hd, stream=NULL_STREAM) -> None:
    """crates/backend/src/hip.rs:497-520 launch_index_score_blocks: block scores [s][n_comp]."""
    ensure_hip_status(lib().rivoli_index_score_blocks(_p(q), _p(kv), _p(w), _p(score), s, n_comp, heads, hd,
                                                      _s(stream)), "index_score_blocks")


def launch_index_score_blocks_prefill(q, kv, w, score, s, n_comp, heads, hd, ratio, stream=NULL_STREAM) -> None:
    """launch_index_score_blocks for a prefill: only entries a row's selection can rank
    (block < (t + 1) / ratio, in groups of 64 blocks) are computed."""
    ensure_hip_status(lib().rivoli_index_score_blocks_prefill(_p(q), _p(kv), _p(w), _p(score), s, n_comp, heads,
                                                              hd, ratio, _s(stream)), "index_score_blocks_prefill")


def launch_index_select_blocks(scores, rows, n_comp, ratio, index_topk, prefill, offset, out,
                               stream=NULL_STREAM) -> None:
    """crates/engine/src/v4/select.rs scored_rows on the device: out is int32
    [rows][min(index_topk, n_comp)]."""
    ensure_hip_status(lib().rivoli_index_select_blocks(_p(scores), rows, n_comp, ratio, index_topk,
                                                       1 if prefill else 0, offset, _p(out),
                                                       _s(stream)), "index_select_blocks")


def sel_shape(win, ratio, index_topk, seqlen, start_pos):
    """crates/engine/src/v4/select.rs Sel::shape: (rows, cols) of the positional rectangle;
    raises LaunchError with the guard code where the reference refuses."""
    rows, cols = C.c_int(0), C.c_int(0)
    ensure_hip_status(lib().rivoli_sel_shape(win, ratio, index_topk, seqlen, start_pos, C.byref(rows),
                                             C.byref(cols)), "sel_shape")
    return rows.value, cols.value


def compress_offset(win, seqlen, start_pos):
    """crates/engine/src/v4/select.rs:268-270: where the compressed region starts in SELECTION
    space — past the prompt at prefill, past the ring at decode."""
    return seqlen if start_pos == 0 else win


def compress_dst(ratio, region_base, seqlen, start_pos):
    """crates/engine/src/v4/select.rs:278-329 (should_compress + compress_dst): the
    (first_row, count) this call's pooled blocks belong at, or None when the call emits none.
    Prefill emits every complete block from the region's base; decode emits one block on the
    position that completes it, at region_base + start_pos // ratio — a function of the
    position, never of how many blocks were emitted before."""
    if ratio <= 0:
        return None
    if start_pos == 0:
        return (region_base, seqlen // ratio) if seqlen >= ratio else None
    return (region_base + start_pos // ratio, 1) if (start_pos + 1) % ratio == 0 else None


def launch_sel_gather(win, ratio, index_topk, seqlen, start_pos, out, stream=NULL_STREAM):
    """Sel::gather on the device: out is int32 [rows][cols] of sel_shape. Returns (rows, cols)."""
    shape = sel_shape(win, ratio, index_topk, seqlen, start_pos)
    ensure_hip_status(lib().rivoli_sel_gather(win, ratio, index_topk, seqlen, start_pos, _p(out), _s(stream)),
                      "sel_gather")
    return shape


def launch_sel_gather_scored(scores, n_comp, win, ratio, index_topk, seqlen, start_pos, out,
                             stream=NULL_STREAM):
    """Sel::gather_scored over scored_rows on the device. Returns (rows, cols)."""
    cols = C.c_int(0)
    ensure_hip_status(lib().rivoli_sel_gather_scored(_p(scores), n_comp, win, ratio, index_topk, seqlen,
                                                     start_pos, _p(out), C.byref(cols), _s(stream)),
                      "sel_gather_scored")
    return (seqlen if start_pos == 0 else 1), cols.value


def launch_kv_ring_write(kv, cache, win, hd, seqlen, start_pos, stream=NULL_STREAM) -> None:
    """crates/engine/src/v4/attn.rs write_ring as one launch."""
    ensure_hip_status(lib().rivoli_kv_ring_write(_p(kv), _p(cache), win, hd, seqlen, start_pos, _s(stream)),
                      "kv_ring_write")


def gather_attn_scratch_floats(m, h, d, topk) -> int:
    """f32 elements of the partial buffer launch_gather_attn_shared_kv(partial=...) needs (0: none)."""
    return int(lib().rivoli_gather_attn_scratch_floats(m, h, d, topk))


def launch_gather_attn_shared_kv(q, kv, sink, idxs, m, h, d, topk, scale, o, stream=NULL_STREAM, *,
                                 n_kv=None, precise=2, partial=None) -> None:
    """crates/backend/src/hip_attn.rs launch_gather_attn_shared_kv. With n_kv (rows of kv) the
    bounded entry point runs: indices at or past it are treated as masked. With partial (a
    buffer of gather_attn_scratch_floats f32) a query's list may be shared among workgroups."""
    if partial is not None:
        code = lib().rivoli_gather_attn_shared_kv_split(_p(q), _p(kv), _p(sink), _p(idxs), m, h, d, topk,
                                                        0x7fffffff if n_kv is None else n_kv, scale, precise,
                                                        _p(o), _p(partial), _s(stream))
    elif n_kv is None and precise == 2:
        code = lib().rivoli_gather_attn_shared_kv(_p(q), _p(kv), _p(sink), _p(idxs), m, h, d, topk, scale, _p(o),
                                                  _s(stream))
    else:
        code = lib().rivoli_gather_attn_shared_kv_bounded(_p(q), _p(kv), _p(sink), _p(idxs), m, h, d, topk,
                                                          0x7fffffff if n_kv is None else n_kv, scale, precise,
                                                          _p(o), _s(stream))
    ensure_hip_status(code, "gather_attn_shared_kv")


class CompGeom(C.Structure):
    """rivoli_comp_geom (crates/engine/src/v4/kvcompress.rs GeomAbi): only `build` derives the
    dependent fields, so a stale cd / ents cannot be handed over."""
    _fields_ = [("ratio", C.c_int), ("coff", C.c_int), ("d", C.c_int), ("cd", C.c_int),
                ("ents", C.c_int), ("rd", C.c_int), ("eps", C.c_float)]

    @classmethod
    def build(cls, ratio: int, d: int, rd: int, eps: float) -> "CompGeom":
        coff = 2 if ratio == 4 else 1        # overlapping windows exist at ratio 4 only
        return cls(ratio, coff, d, coff * d, coff * ratio, rd, eps)


class CompFinish(C.Structure):
    """rivoli_comp_finish: device pointers of the norm weight, the compressed rotation table
    and the output rows."""
    _fields_ = [("norm", C.c_void_p), ("freqs", C.c_void_p), ("out", C.c_void_p)]

    @classmethod
    def of(cls, norm, freqs, out) -> "CompFinish":
        return cls(_p(norm), _p(freqs), _p(out))


def _ref_or_null(struct):
    return None if struct is None else C.byref(struct)


def launch_kv_compress_deposit(kv, score, ape, kv_state, score_state, geom, s, slot0,
                               stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_compress_deposit(
        _p(kv), _p(score), _p(ape), _p(kv_state), _p(score_state), _ref_or_null(geom), s, slot0,
        _s(stream)), "kv_compress_deposit")


def launch_kv_compress_prefill(kv, score, ape, finish, geom, nblk, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_compress_prefill(
        _p(kv), _p(score), _p(ape), _ref_or_null(finish), _ref_or_null(geom), nblk, _s(stream)),
        "kv_compress_prefill")


def launch_kv_compress_decode(kv_state, score_state, finish, geom, start_pos,
                              stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_kv_compress_decode(
        _p(kv_state), _p(score_state), _ref_or_null(finish), _ref_or_null(geom), start_pos,
        _s(stream)), "kv_compress_decode")


# ---- element codecs -----------------------------------------------------------------------

def launch_codec_e4m3_encode(x, out, n, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_codec_e4m3_encode(_p(x), _p(out), n, _s(stream)),
                      "codec_e4m3_encode")


def launch_codec_e4m3_dequant_bf16(codes, scale, out, n, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_codec_e4m3_dequant_bf16(_p(codes), scale, _p(out), n,
                                                           _s(stream)), "codec_e4m3_dequant_bf16")


def launch_codec_bf16_encode(x, out, n, stream=NULL_STREAM) -> None:
    ensure_hip_status(lib().rivoli_codec_bf16_encode(_p(x), _p(out), n, _s(stream)),
                      "codec_bf16_encode")
