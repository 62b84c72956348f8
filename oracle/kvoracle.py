"""ctypes view of the CPU oracle (oracle/libkvoracle.so) — TEST INFRASTRUCTURE, NOT PRODUCT.

Only the tests, the smoke check and the benchmark's CPU-baseline leg import this module. The
shipped package (rivoli_amd) never does. Arrays cross as numpy; every function mirrors one in
kvcache_oracle.h, which carries the reference citations.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libkvoracle.so")
REF_LIB_PATH = os.path.join(HERE, "_ref", "librivoli_ref_kernels.so")


def build(with_ref: bool = True) -> None:
    """Compile the oracle; also the reference's own launchers when its tree is mounted."""
    subprocess.run(["make", "-C", HERE, "-B", "all"], check=True)
    if with_ref and os.path.isdir("/root/reference/crates/backend/kernels"):
        subprocess.run(["make", "-C", HERE, "-B", "ref"], check=True)


def _ptr(a: np.ndarray, ctype):
    return a.ctypes.data_as(C.POINTER(ctype))


def _c(a, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


class CompGeom(C.Structure):
    """crates/backend/kernels/kvcompress.hip:40-48, by value the layout both sides share."""
    _fields_ = [("ratio", C.c_int), ("coff", C.c_int), ("d", C.c_int), ("cd", C.c_int),
                ("ents", C.c_int), ("rd", C.c_int), ("eps", C.c_float)]

    @classmethod
    def attention(cls, ratio: int, d: int = 512, rd: int = 64, eps: float = 1e-6) -> "CompGeom":
        """The attention compressor's geometry: overlapping windows at ratio 4 only."""
        coff = 2 if ratio == 4 else 1
        return cls(ratio, coff, d, coff * d, coff * ratio, rd, eps)


class _V4Mixin:
    """The second cache format (v4cache_oracle.h)."""

    def e4m3_encode_rne(self, x) -> np.ndarray:
        x = _c(x, np.float32)
        out = np.empty(x.shape, np.uint8)
        self.lib.ro_e4m3_encode_rne_n(_ptr(x, C.c_float), _ptr(out, C.c_uint8), x.size)
        return out

    def fast_round_scale(self, amax, max_inv=np.float32(1.0) / np.float32(448.0)) -> np.float32:
        return np.float32(self.lib.ro_fast_round_scale(float(np.float32(amax)), float(np.float32(max_inv))))

    def act_quant_f8_prefix(self, x, n: int, block: int, inplace: bool = True):
        """x is [rows, row_stride] f32. Returns (guard code, result); the input is not modified.
        With inplace=False the source and destination are distinct buffers (n must then cover
        the row) and the destination starts as NaN-free garbage (0x5a bytes)."""
        x = _c(x, np.float32)
        rows, row_stride = x.shape
        if inplace:
            dst = x.copy()
            src = dst
        else:
            src, dst = x, np.frombuffer(b"\x5a" * (x.size * 4), np.float32).reshape(x.shape).copy()
        code = int(self.lib.ro_act_quant_f8_prefix(_ptr(src, C.c_float), _ptr(dst, C.c_float), rows,
                                                   row_stride, n, block))
        return code, dst

    def compress_guard(self, geom: CompGeom) -> int:
        return int(self.lib.ro_compress_guard(C.byref(geom)))

    def kv_compress_deposit(self, kv, score, ape, kv_state, score_state, geom: CompGeom, s: int,
                            slot0: int) -> int:
        """The two states are float32 arrays updated in place."""
        kv, score, ape = _c(kv, np.float32), _c(score, np.float32), _c(ape, np.float32)
        return int(self.lib.ro_kv_compress_deposit(
            _ptr(kv, C.c_float), _ptr(score, C.c_float), _ptr(ape, C.c_float),
            _ptr(kv_state, C.c_float), _ptr(score_state, C.c_float), C.byref(geom), s, slot0))

    def kv_compress_prefill(self, kv, score, ape, norm, freqs, geom: CompGeom, nblk: int):
        """Returns (code, out[nblk, d])."""
        kv, score, ape = _c(kv, np.float32), _c(score, np.float32), _c(ape, np.float32)
        norm, freqs = _c(norm, np.float32), _c(freqs, np.float32)
        out = np.zeros((max(nblk, 1), geom.d), np.float32)
        code = int(self.lib.ro_kv_compress_prefill(
            _ptr(kv, C.c_float), _ptr(score, C.c_float), _ptr(ape, C.c_float), _ptr(norm, C.c_float),
            _ptr(freqs, C.c_float), _ptr(out, C.c_float), C.byref(geom), nblk))
        return code, out[:max(nblk, 0)]

    def e2m1_encode(self, x) -> int:
        return int(self.lib.ro_e2m1_encode(float(np.float32(x))))

    def e2m1_decode(self, code: int) -> np.float32:
        return np.float32(self.lib.ro_e2m1_decode(int(code)))

    def hadamard_rotate(self, row) -> np.ndarray:
        out = _c(row, np.float32).copy()
        self.lib.ro_hadamard_rotate(_ptr(out, C.c_float), out.size)
        return out

    def fp4_act_quant(self, row, block: int = 32) -> np.ndarray:
        out = _c(row, np.float32).copy()
        self.lib.ro_fp4_act_quant_inplace(_ptr(out, C.c_float), out.size, block)
        return out

    def act_quant_f4_rotated(self, x):
        """x: [rows, d] f32. Returns (code, spread rows); the input is not modified."""
        out = _c(x, np.float32).copy()
        rows, d = out.shape
        code = int(self.lib.ro_act_quant_f4_rotated(_ptr(out, C.c_float), rows, d))
        return code, out

    def index_score_blocks(self, q, kv, w):
        """q: [s, heads, hd]; kv: [n_comp, hd]; w: [s, heads]. Returns (code, score[s, n_comp])."""
        q, kv, w = _c(q, np.float32), _c(kv, np.float32), _c(w, np.float32)
        s, heads, hd = q.shape
        n_comp = kv.shape[0]
        score = np.zeros((s, max(n_comp, 1)), np.float32)
        code = int(self.lib.ro_index_score_blocks(_ptr(q, C.c_float), _ptr(kv, C.c_float),
                                                  _ptr(w, C.c_float), _ptr(score, C.c_float), s, n_comp,
                                                  heads, hd))
        return code, score[:, :n_comp]

    def kv_compress_decode(self, kv_state, score_state, norm, freqs, geom: CompGeom, start_pos: int):
        """Returns (code, out[d]); the states are updated in place (the window slides)."""
        norm, freqs = _c(norm, np.float32), _c(freqs, np.float32)
        out = np.zeros(geom.d, np.float32)
        code = int(self.lib.ro_kv_compress_decode(
            _ptr(kv_state, C.c_float), _ptr(score_state, C.c_float), _ptr(norm, C.c_float),
            _ptr(freqs, C.c_float), _ptr(out, C.c_float), C.byref(geom), start_pos))
        return code, out

    def v4_scored_rows(self, scores, ratio: int, index_topk: int, prefill: bool, offset: int):
        """scores is [rows, n_comp] f32. Returns int32 [rows, min(index_topk, n_comp)]."""
        scores = _c(scores, np.float32)
        rows, n_comp = scores.shape
        k = min(index_topk, n_comp)
        out = np.empty((rows, k), np.int32)
        got = int(self.lib.ro_v4_scored_rows(_ptr(scores, C.c_float), rows, n_comp, ratio, index_topk,
                                             1 if prefill else 0, offset, _ptr(out, C.c_int32)))
        assert got == k, got
        return out


    def sel_shape(self, win: int, ratio: int, index_topk: int, seqlen: int, start_pos: int):
        """(code, rows, cols) of a positional selection rectangle."""
        rows, cols = C.c_int(0), C.c_int(0)
        code = int(self.lib.ro_sel_shape(win, ratio, index_topk, seqlen, start_pos, C.byref(rows),
                                         C.byref(cols)))
        return code, rows.value, cols.value

    def sel_gather(self, win: int, ratio: int, index_topk: int, seqlen: int, start_pos: int):
        """(code, int32 [rows, cols]) — window columns then the positional compressed columns."""
        code, rows, cols = self.sel_shape(win, ratio, index_topk, seqlen, start_pos)
        if code:
            return code, None
        out = np.full((rows, cols), -7, np.int32)
        code = int(self.lib.ro_sel_gather(win, ratio, index_topk, seqlen, start_pos, _ptr(out, C.c_int32)))
        return code, out

    def sel_gather_scored(self, scores, win: int, ratio: int, index_topk: int, seqlen: int, start_pos: int):
        """scores is [rows, n_comp] f32 (n_comp may be 0). (code, int32 [rows, cols])."""
        scores = _c(scores, np.float32)
        rows, n_comp = scores.shape
        win_cols = min(seqlen, win) if start_pos == 0 else win
        out = np.full((max(rows, 1), win_cols + min(index_topk, n_comp)), -7, np.int32)
        cols = C.c_int(0)
        code = int(self.lib.ro_sel_gather_scored(_ptr(scores, C.c_float) if n_comp else None, n_comp, win, ratio,
                                                 index_topk, seqlen, start_pos, _ptr(out, C.c_int32),
                                                 C.byref(cols)))
        assert code or cols.value == out.shape[1]
        return code, (None if code else out)

    @staticmethod
    def compress_dst(ratio: int, region_base: int, seqlen: int, start_pos: int):
        """crates/engine/src/v4/select.rs:278-329 restated branch by branch: None when the call
        emits no block, else (first_row, count). Pinned by the reference's unit cases
        (select.rs:556-611) in tests/test_oracle_v4_select.py."""
        if ratio == 0:                                   # LayerKind::Plain: no compressor at all
            return None
        prefill = start_pos == 0
        emits = seqlen >= ratio if prefill else (start_pos + 1) % ratio == 0
        if not emits:
            return None
        return (region_base, seqlen // ratio) if prefill else (region_base + start_pos // ratio, 1)

    def ring_write(self, kv, cache, win: int, seqlen: int, start_pos: int) -> int:
        """Updates cache ([win, hd] f32) in place from kv ([rows, hd] f32)."""
        kv = _c(kv, np.float32)
        assert cache.dtype == np.float32 and cache.flags.c_contiguous and cache.shape == (win, kv.shape[1])
        return int(self.lib.ro_ring_write(_ptr(kv, C.c_float), _ptr(cache, C.c_float), win, kv.shape[1], seqlen,
                                          start_pos))

    def sparse_attn(self, q, kv, sink, idxs, scale: float) -> np.ndarray:
        """q [m, h, d], kv [rows, d], sink [h], idxs int32 [m, topk] -> o [m, h, d] (bf16-valued f32)."""
        q, kv, sink = _c(q, np.float32), _c(kv, np.float32), _c(sink, np.float32)
        idxs = _c(idxs, np.int32)
        m, h, d = q.shape
        assert idxs.shape[0] == m and kv.shape[1] == d and sink.shape == (h,)
        assert idxs.max(initial=-1) < kv.shape[0]
        o = np.empty((m, h, d), np.float32)
        code = int(self.lib.ro_sparse_attn(_ptr(q, C.c_float), _ptr(kv, C.c_float), _ptr(sink, C.c_float),
                                           _ptr(idxs, C.c_int32), m, h, d, idxs.shape[1], scale,
                                           _ptr(o, C.c_float)))
        assert code == 0, code
        return o


class Oracle(_V4Mixin):
    def __init__(self, path: str = LIB_PATH):
        if not os.path.exists(path):
            build(with_ref=False)
        self.lib = lib = C.CDLL(path)
        u8p, u16p, u32p = C.POINTER(C.c_uint8), C.POINTER(C.c_uint16), C.POINTER(C.c_uint32)
        i32p, f32p = C.POINTER(C.c_int32), C.POINTER(C.c_float)
        sig = {
            "ro_f32_to_e4m3": (C.c_uint8, [C.c_float]),
            "ro_e4m3_to_f32": (C.c_float, [C.c_uint8]),
            "ro_f32_to_bf16": (C.c_uint16, [C.c_float]),
            "ro_bf16_to_f32": (C.c_float, [C.c_uint16]),
            "ro_f32_to_e4m3_n": (None, [f32p, u8p, C.c_size_t]),
            "ro_e4m3_to_f32_n": (None, [u8p, f32p, C.c_size_t]),
            "ro_f32_to_bf16_n": (None, [f32p, u16p, C.c_size_t]),
            "ro_selftest_bf16_exhaustive": (C.c_uint64, []),
            "ro_lcg_f": (C.c_float, [C.POINTER(C.c_uint64)]),
            "ro_lcg_fill": (None, [C.POINTER(C.c_uint64), f32p, C.c_size_t]),
            "ro_quant_block": (None, [f32p, C.c_int, u8p, f32p]),
            "ro_append_kv": (C.c_int, [f32p, f32p, u8p, f32p, u16p] + [C.c_int] * 4),
            "ro_index_append": (C.c_int, [f32p, u16p, C.c_int, C.c_int]),
            "ro_index_score": (C.c_int, [f32p, f32p, u16p, u32p] + [C.c_int] * 4 + [C.c_float] * 2 + [f32p]),
            "ro_index_append_paged": (C.c_int, [f32p, i32p, u16p] + [C.c_int] * 4),
            "ro_index_score_paged": (None, [f32p, f32p, u16p, i32p, i32p, u32p] + [C.c_int] * 7
                                     + [C.c_float] * 2 + [f32p, C.c_int]),
            "ro_kv_page_bytes": (C.c_size_t, [C.c_int, C.c_int]),
            "ro_kv_append_paged": (C.c_int, [u16p, i32p, u8p] + [C.c_int] * 4),
            "ro_kv_append_paged_mt": (None, [u16p, i32p, u8p] + [C.c_int] * 5),
            "ro_kv_gather_paged": (None, [u8p, i32p, i32p, i32p, u16p] + [C.c_int] * 4),
            "ro_kv_gather_paged_mt": (None, [u8p, i32p, i32p, i32p, u16p] + [C.c_int] * 5),
            "ro_kv_gather_rows_paged": (None, [u8p, i32p, u32p, i32p, u16p] + [C.c_int] * 5),
            "ro_mla_attend_dense": (None, [f32p] * 4 + [C.c_int] * 4 + [C.c_float, f32p]),
            "ro_mla_attend": (C.c_int, [f32p, f32p, u8p, f32p, u16p, u32p] + [C.c_int] * 5 + [C.c_float, f32p]),
            "ro_mla_attend_paged": (None, [f32p, f32p, u8p, i32p, i32p, u32p, i32p] + [C.c_int] * 7
                                    + [C.c_float, f32p, C.c_int]),
            "ro_topk": (C.c_int, [f32p, C.c_int, C.c_int, u32p]),
            "ro_topk_batched": (None, [f32p, C.c_int, C.c_int, i32p, C.c_int, C.c_int, u32p, C.c_int]),
            "ro_fnv1a": (C.c_uint64, [u8p, C.c_size_t]),
            "ro_splitmix_finalize": (C.c_uint64, [C.c_uint64]),
            "ro_xor_fold": (C.c_uint64, [u32p, C.c_size_t, C.c_uint64, C.c_size_t]),
            "ro_e4m3_encode_rne_n": (None, [f32p, u8p, C.c_size_t]),
            "ro_fast_round_scale": (C.c_float, [C.c_float, C.c_float]),
            "ro_act_quant_f8_prefix": (C.c_int, [f32p, f32p] + [C.c_int] * 4),
            "ro_v4_scored_rows": (C.c_int, [f32p] + [C.c_int] * 6 + [i32p]),
            "ro_sel_shape": (C.c_int, [C.c_int] * 5 + [C.POINTER(C.c_int)] * 2),
            "ro_sel_gather": (C.c_int, [C.c_int] * 5 + [i32p]),
            "ro_sel_gather_scored": (C.c_int, [f32p] + [C.c_int] * 6 + [i32p, C.POINTER(C.c_int)]),
            "ro_ring_write": (C.c_int, [f32p, f32p] + [C.c_int] * 4),
            "ro_sparse_attn": (C.c_int, [f32p, f32p, f32p, i32p] + [C.c_int] * 4 + [C.c_float, f32p]),
            "ro_compress_guard": (C.c_int, [C.POINTER(CompGeom)]),
            "ro_kv_compress_deposit": (C.c_int, [f32p] * 5 + [C.POINTER(CompGeom), C.c_int, C.c_int]),
            "ro_kv_compress_prefill": (C.c_int, [f32p] * 6 + [C.POINTER(CompGeom), C.c_int]),
            "ro_kv_compress_decode": (C.c_int, [f32p] * 5 + [C.POINTER(CompGeom), C.c_int]),
            "ro_e2m1_encode": (C.c_uint8, [C.c_float]),
            "ro_e2m1_decode": (C.c_float, [C.c_uint8]),
            "ro_hadamard_rotate": (None, [f32p, C.c_int]),
            "ro_fp4_act_quant_inplace": (None, [f32p, C.c_int, C.c_int]),
            "ro_act_quant_f4_rotated": (C.c_int, [f32p, C.c_int, C.c_int]),
            "ro_index_score_blocks": (C.c_int, [f32p] * 4 + [C.c_int] * 4),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args

    # ---- codecs -------------------------------------------------------------------------
    def f32_to_e4m3(self, x) -> np.ndarray:
        x = _c(x, np.float32)
        out = np.empty(x.shape, np.uint8)
        self.lib.ro_f32_to_e4m3_n(_ptr(x, C.c_float), _ptr(out, C.c_uint8), x.size)
        return out

    def e4m3_to_f32(self, c) -> np.ndarray:
        c = _c(c, np.uint8)
        out = np.empty(c.shape, np.float32)
        self.lib.ro_e4m3_to_f32_n(_ptr(c, C.c_uint8), _ptr(out, C.c_float), c.size)
        return out

    def f32_to_bf16(self, x) -> np.ndarray:
        x = _c(x, np.float32)
        out = np.empty(x.shape, np.uint16)
        self.lib.ro_f32_to_bf16_n(_ptr(x, C.c_float), _ptr(out, C.c_uint16), x.size)
        return out

    def selftest_bf16_exhaustive(self) -> int:
        return int(self.lib.ro_selftest_bf16_exhaustive())

    # ---- the reference tests' input stream ----------------------------------------------
    def lcg(self, seed: int) -> "Lcg":
        return Lcg(self, seed)

    # ---- quantization -------------------------------------------------------------------
    def quant_block(self, v):
        v = _c(v, np.float32).ravel()
        codes = np.empty(v.size, np.uint8)
        scale = C.c_float()
        self.lib.ro_quant_block(_ptr(v, C.c_float), v.size, _ptr(codes, C.c_uint8), C.byref(scale))
        return codes, np.float32(scale.value)

    def append_kv(self, latent, rope, lc8, lscale, rc, pos, kvl, ropn, n_blocks) -> int:
        latent, rope = _c(latent, np.float32), _c(rope, np.float32)
        return int(self.lib.ro_append_kv(
            _ptr(latent, C.c_float), _ptr(rope, C.c_float), _ptr(lc8, C.c_uint8),
            _ptr(lscale, C.c_float), _ptr(rc, C.c_uint16), pos, kvl, ropn, n_blocks))

    def index_append(self, k, kcache, pos, hd) -> int:
        k = _c(k, np.float32)
        return int(self.lib.ro_index_append(_ptr(k, C.c_float), _ptr(kcache, C.c_uint16), pos, hd))

    # ---- indexer scores -----------------------------------------------------------------
    def index_score(self, q, w, kcache_bf16, heads, nh, hd, wscale, dscale):
        """Returns (guard code, scores[nt])."""
        q, w, kc = _c(q, np.float32), _c(w, np.float32), _c(kcache_bf16, np.uint16)
        nt = kc.size // hd
        hs = None if heads is None else _c(heads, np.uint32)
        nact = nh if hs is None else hs.size
        scores = np.zeros(max(nt, 0), np.float32)
        rc = self.lib.ro_index_score(_ptr(q, C.c_float), _ptr(w, C.c_float), _ptr(kc, C.c_uint16),
                                     None if hs is None else _ptr(hs, C.c_uint32), nt, nh, nact,
                                     hd, wscale, dscale, _ptr(scores, C.c_float))
        return int(rc), scores

    def index_append_paged(self, k, slot_mapping, kpool, hd, page_tokens, n_pages) -> int:
        k, slot_mapping = _c(k, np.float32), _c(slot_mapping, np.int32)
        return int(self.lib.ro_index_append_paged(_ptr(k, C.c_float), _ptr(slot_mapping, C.c_int32),
                                                  _ptr(kpool, C.c_uint16), slot_mapping.size, hd,
                                                  page_tokens, n_pages))

    def index_score_paged(self, q, w, kpool, block_table, nts, heads, stride, hd, page_tokens,
                          wscale, dscale, n_threads: int = 1) -> np.ndarray:
        q, w = _c(q, np.float32), _c(w, np.float32)
        block_table, nts = _c(block_table, np.int32), _c(nts, np.int32)
        n_q, nh = w.shape
        hs = None if heads is None else _c(heads, np.uint32)
        nact = nh if hs is None else hs.size
        scores = np.zeros((n_q, stride), np.float32)
        self.lib.ro_index_score_paged(
            _ptr(q, C.c_float), _ptr(w, C.c_float), _ptr(kpool, C.c_uint16),
            _ptr(block_table, C.c_int32), _ptr(nts, C.c_int32),
            None if hs is None else _ptr(hs, C.c_uint32), n_q, block_table.shape[1], stride, nh,
            nact, hd, page_tokens, wscale, dscale, _ptr(scores, C.c_float), n_threads)
        return scores

    # ---- paged cache --------------------------------------------------------------------
    def kv_page_bytes(self, page_tokens: int, width: int) -> int:
        return int(self.lib.ro_kv_page_bytes(page_tokens, width))

    def kv_append_paged(self, rows_bf16, slot_mapping, pool, width, page_tokens, n_pages,
                        n_threads: int = 0) -> int:
        rows_bf16, slot_mapping = _c(rows_bf16, np.uint16), _c(slot_mapping, np.int32)
        assert pool.dtype == np.uint8 and pool.flags.c_contiguous
        n = slot_mapping.size
        if n_threads > 0:
            self.lib.ro_kv_append_paged_mt(_ptr(rows_bf16, C.c_uint16), _ptr(slot_mapping, C.c_int32),
                                           _ptr(pool, C.c_uint8), n, width, page_tokens, n_pages,
                                           n_threads)
            return 0
        return int(self.lib.ro_kv_append_paged(_ptr(rows_bf16, C.c_uint16),
                                               _ptr(slot_mapping, C.c_int32),
                                               _ptr(pool, C.c_uint8), n, width, page_tokens,
                                               n_pages))

    def kv_gather_paged(self, pool, block_table, seq_lens, width, page_tokens,
                        n_threads: int = 0, out=None) -> np.ndarray:
        block_table, seq_lens = _c(block_table, np.int32), _c(seq_lens, np.int32)
        n_seqs, max_blocks = block_table.shape
        cu = np.zeros(n_seqs + 1, np.int32)
        np.cumsum(seq_lens, out=cu[1:])
        if out is None:
            out = np.zeros((int(cu[-1]), width), np.uint16)
        args = (_ptr(pool, C.c_uint8), _ptr(block_table, C.c_int32), _ptr(seq_lens, C.c_int32),
                _ptr(cu, C.c_int32), _ptr(out, C.c_uint16), n_seqs, max_blocks, width, page_tokens)
        if n_threads > 0:
            self.lib.ro_kv_gather_paged_mt(*args, n_threads)
        else:
            self.lib.ro_kv_gather_paged(*args)
        return out

    def kv_gather_rows_paged(self, pool, block_table, rows, width, page_tokens,
                             n_rows=None) -> np.ndarray:
        block_table, rows = _c(block_table, np.int32), _c(rows, np.uint32)
        n_q, max_blocks = block_table.shape
        k = rows.shape[1]
        out = np.zeros((n_q, k, width), np.uint16)
        nr = None if n_rows is None else _c(n_rows, np.int32)
        self.lib.ro_kv_gather_rows_paged(
            _ptr(pool, C.c_uint8), _ptr(block_table, C.c_int32), _ptr(rows, C.c_uint32),
            None if nr is None else _ptr(nr, C.c_int32), _ptr(out, C.c_uint16), n_q, k,
            max_blocks, width, page_tokens)
        return out

    # ---- attention ----------------------------------------------------------------------
    def mla_attend_dense(self, qabs, qrope, lat, rk, scale) -> np.ndarray:
        """qabs [H][kvl], qrope [H][rope], lat [nr][kvl], rk [nr][rope] (all f32) -> clat [H][kvl]."""
        qabs, qrope, lat, rk = (_c(x, np.float32) for x in (qabs, qrope, lat, rk))
        (H, kvl), rope, nr = qabs.shape, qrope.shape[1], lat.shape[0]
        clat = np.zeros((H, kvl), np.float32)
        self.lib.ro_mla_attend_dense(_ptr(qabs, C.c_float), _ptr(qrope, C.c_float), _ptr(lat, C.c_float),
                                     _ptr(rk, C.c_float), H, nr, kvl, rope, scale, _ptr(clat, C.c_float))
        return clat

    def mla_attend(self, qabs, qrope, lc8, lscale, rc, rows, H, nr, kvl, rope, n_blocks, scale):
        """The reference's linear-slab form. Returns (guard code, clat [H][kvl])."""
        qabs, qrope = _c(qabs, np.float32), _c(qrope, np.float32)
        lc8, lscale, rc = _c(lc8, np.uint8), _c(lscale, np.float32), _c(rc, np.uint16)
        rw = None if rows is None else _c(rows, np.uint32)
        clat = np.zeros((max(H, 0), max(kvl, 0)), np.float32)
        code = self.lib.ro_mla_attend(_ptr(qabs, C.c_float), _ptr(qrope, C.c_float), _ptr(lc8, C.c_uint8),
                                      _ptr(lscale, C.c_float), _ptr(rc, C.c_uint16),
                                      None if rw is None else _ptr(rw, C.c_uint32), H, nr, kvl, rope,
                                      n_blocks, scale, _ptr(clat, C.c_float))
        return int(code), clat

    def mla_attend_paged(self, qabs, qrope, pool, block_table, seq_lens, rows, n_rows, kvl, rope,
                         page_tokens, scale, n_threads: int = 1) -> np.ndarray:
        """qabs [n_seqs][H][kvl], qrope [n_seqs][H][rope]; dense when rows is None."""
        qabs, qrope = _c(qabs, np.float32), _c(qrope, np.float32)
        block_table = _c(block_table, np.int32)
        n_seqs, H = qabs.shape[0], qabs.shape[1]
        lens = None if seq_lens is None else _c(seq_lens, np.int32)
        rw = None if rows is None else _c(rows, np.uint32)
        nr = None if n_rows is None else _c(n_rows, np.int32)
        k = 0 if rw is None else rw.shape[1]
        clat = np.zeros((n_seqs, H, kvl), np.float32)
        self.lib.ro_mla_attend_paged(
            _ptr(qabs, C.c_float), _ptr(qrope, C.c_float), _ptr(pool, C.c_uint8),
            _ptr(block_table, C.c_int32), None if lens is None else _ptr(lens, C.c_int32),
            None if rw is None else _ptr(rw, C.c_uint32), None if nr is None else _ptr(nr, C.c_int32),
            k, n_seqs, H, block_table.shape[1], kvl, rope, page_tokens, scale, _ptr(clat, C.c_float),
            n_threads)
        return clat

    # ---- selection ----------------------------------------------------------------------
    def topk(self, scores, k: int) -> np.ndarray:
        scores = _c(scores, np.float32).ravel()
        rows = np.empty(max(min(k, scores.size), 0), np.uint32)
        n = self.lib.ro_topk(_ptr(scores, C.c_float), scores.size, k, _ptr(rows, C.c_uint32))
        return rows[:n]

    def topk_batched(self, scores, k: int, nts=None, n_threads: int = 1) -> np.ndarray:
        scores = _c(scores, np.float32)
        n_q, stride = scores.shape
        rows = np.full((n_q, k), 0xFFFFFFFF, np.uint32)
        nt_arr = None if nts is None else _c(nts, np.int32)
        self.lib.ro_topk_batched(_ptr(scores, C.c_float), n_q, stride,
                                 None if nt_arr is None else _ptr(nt_arr, C.c_int32), stride, k,
                                 _ptr(rows, C.c_uint32), n_threads)
        return rows

    # ---- content pinning ----------------------------------------------------------------
    def fnv1a(self, data: bytes) -> int:
        buf = np.frombuffer(data, np.uint8) if len(data) else np.zeros(0, np.uint8)
        return int(self.lib.ro_fnv1a(_ptr(buf, C.c_uint8) if buf.size else None, buf.size))

    def splitmix_finalize(self, z: int) -> int:
        return int(self.lib.ro_splitmix_finalize(C.c_uint64(z)))

    def xor_fold(self, buf, i_base: int = 0, stride: int = 1) -> int:
        """Fold over the buffer's 32-bit words (its byte length must be a multiple of 4)."""
        words = np.ascontiguousarray(buf).view(np.uint8).ravel().view(np.uint32)
        return int(self.lib.ro_xor_fold(_ptr(words, C.c_uint32), words.size, i_base, stride))


class Lcg:
    """crates/engine/tests/common/reference.rs:141-162 — uniform in [-1, 1)."""

    def __init__(self, oracle: Oracle, seed: int):
        self._o = oracle
        self._state = C.c_uint64(seed)

    def f(self) -> np.float32:
        return np.float32(self._o.lib.ro_lcg_f(C.byref(self._state)))

    def fill(self, n: int) -> np.ndarray:
        out = np.empty(n, np.float32)
        self._o.lib.ro_lcg_fill(C.byref(self._state), _ptr(out, C.c_float), n)
        return out


_ORACLE = None


def oracle() -> Oracle:
    global _ORACLE
    if _ORACLE is None:
        _ORACLE = Oracle()
    return _ORACLE
