"""The second cache format's pieces driven in the order the reference's attention sublayer
drives them (crates/engine/src/v4/attn.rs:272-330, kvcompress.rs:263-392,406-520): quantize the
step's cache entries, write the ring, run the compressor (deposit; pool when a block closes;
quantize the pooled rows; place them by position), build the selection rectangle, attend — a
prefill and then one token at a time, on the device and through the oracle side by side.

What is compared at every step: the ring and the rectangle bit for bit; the pooled rows to the
compressor's bar (2 bf16 codes, tests/test_gpu_v4_compress.py); the attention, computed by
the oracle from the DEVICE's own cache so that both see identical rows, to the attention's bar
(1/128 of the largest element)."""
import numpy as np
import pytest

from oracle.kvoracle import CompGeom as OracleGeom
from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros
from tests.v4_cases import bf16_round, compress_gap, compress_inputs

pytestmark = pytest.mark.gpu
ATTEND_TOL, CLEAN_ULP = 1.0 / 128.0, 2


class DeviceLayer:
    """One layer's persistent state on the device: [ring | compressed] cache, compressor state."""

    def __init__(self, win, ratio, d, rd, heads, max_ctx, ape, norm, freqs, sink, index_topk):
        self.win, self.ratio, self.d, self.rd, self.heads, self.cap = win, ratio, d, rd, heads, index_topk
        self.geom = hip.CompGeom.build(ratio, d, rd, 1e-6) if ratio else None
        self.cache = dzeros((win + (max_ctx // ratio if ratio else 0)) * d * 4)
        if ratio:
            n = self.geom.coff * ratio * self.geom.cd
            self.state_kv = dev(np.zeros(n, np.float32))
            self.state_score = dev(np.full(n, -np.inf, np.float32))
            self.ape, self.norm, self.freqs = dev(ape), dev(norm), dev(freqs)
        self.sink = dev(sink)
        self.scale = d ** -0.5

    def step(self, kv_entry, q, ckv, cscore, scores, seqlen, start_pos):
        """kv_entry [rows, d], q [rows, heads, d], ckv / cscore [rows, cd] (the compressor's
        projections), scores [rows, n_comp] or None (positional selection). Returns the
        attention output, the rectangle, and the pooled rows this call emitted (or None)."""
        win, ratio, d, rd = self.win, self.ratio, self.d, self.rd
        prefill = start_pos == 0
        rows = seqlen if prefill else 1
        n_comp_sel = (start_pos + rows) // ratio if ratio else 0
        # attention scratch at prefill: [prompt rows | pooled rows]; the ring cache at decode
        kv_d = dzeros((rows + n_comp_sel) * d * 4)
        kv_d[: rows * d * 4] = dev(kv_entry)
        hip.launch_act_quant_f8_prefix(kv_d, kv_d, rows, d, d - rd, 64)      # the cache entry's quantization
        hip.launch_kv_ring_write(kv_d, self.cache, win, d, seqlen, start_pos)
        emitted = None
        if ratio:
            hip.launch_kv_compress_deposit(dev(ckv), dev(cscore), self.ape, self.state_kv, self.state_score,
                                           self.geom, rows, start_pos % ratio)
            dst = hip.compress_dst(ratio, win, seqlen, start_pos)
            if dst is not None:
                first, count = dst
                out = dzeros(count * d * 4)
                fin = hip.CompFinish.of(self.norm, self.freqs, out)
                if prefill:
                    hip.launch_kv_compress_prefill(dev(ckv), dev(cscore), self.ape, fin, self.geom, count)
                else:
                    hip.launch_kv_compress_decode(self.state_kv, self.state_score, fin, self.geom, start_pos)
                pooled = back(out, np.float32).reshape(count, d).copy()
                hip.launch_act_quant_f8_prefix(out, out, count, d, d - rd, 64)
                self.cache[first * d * 4:(first + count) * d * 4] = out        # persistent home, by position
                if prefill:                                                     # and the scratch's tail
                    sel_first, _ = hip.compress_dst(ratio, hip.compress_offset(win, seqlen, start_pos), seqlen, 0)
                    kv_d[sel_first * d * 4:(sel_first + count) * d * 4] = out
                emitted = (pooled, back(out, np.float32).reshape(count, d).copy())
        src = kv_d if prefill else self.cache
        if scores is None:
            shape = hip.sel_shape(win, ratio, self.cap, seqlen, start_pos)
            idx = dzeros(shape[0] * shape[1] * 4, 0xEE)
            hip.launch_sel_gather(win, ratio, self.cap, seqlen, start_pos, idx)
        else:
            idx = dzeros(rows * (win + scores.shape[1]) * 4, 0xEE)
            shape = hip.launch_sel_gather_scored(dev(scores), scores.shape[1], win, ratio, self.cap, seqlen,
                                                 start_pos, idx)
        o = dzeros(rows * self.heads * d * 4)
        part = dzeros(max(hip.gather_attn_scratch_floats(rows, self.heads, d, shape[1]), 4) * 4)
        hip.launch_gather_attn_shared_kv(dev(q), src, self.sink, idx, rows, self.heads, d, shape[1], self.scale, o,
                                         partial=part)
        rect = back(idx, np.int32)[: shape[0] * shape[1]].reshape(shape).copy()
        return (back(o, np.float32).reshape(rows, self.heads, d).copy(), rect, emitted,
                back(src, np.float32).reshape(-1, d).copy())


@pytest.mark.parametrize("win,ratio,d,rd,heads,prompt,steps,cap", [
    (8, 4, 512, 64, 64, 21, 12, 512),      # the indexed class, matrix-core attention, positional selection
    (8, 4, 512, 64, 64, 21, 12, 3),        # the same past a cap of 3 blocks: scored selection
    (16, 8, 128, 64, 8, 40, 20, 512),      # an unindexed ratio, toy width: the plain attention kernel
    (8, 0, 512, 64, 64, 5, 14, 512),       # no compressor; the prompt fits the ring, which then fills and wraps
])
def test_prefill_then_decode(oracle, win, ratio, d, rd, heads, prompt, steps, cap):
    total = prompt + steps
    rng = np.random.default_rng(win * 100 + ratio + d)
    kv_all = bf16_round(rng.standard_normal((total, d)).astype(np.float32))
    q_all = bf16_round(rng.standard_normal((total, heads, d)).astype(np.float32))
    sink = rng.standard_normal(heads).astype(np.float32)
    if ratio:
        og = OracleGeom.attention(ratio, d, rd)
        ckv, cscore, ape, norm, freqs = compress_inputs(og, total, seed=7, positions=total)
        o_state = [np.zeros((og.coff * ratio, og.cd), np.float32), np.full((og.coff * ratio, og.cd), -np.inf, np.float32)]
    else:
        og, ckv, cscore, ape, norm, freqs = None, None, None, None, None, None
    layer = DeviceLayer(win, ratio, d, rd, heads, total + 8, ape, norm, freqs, sink, cap)
    o_cache = np.zeros((win + ((total + 8) // ratio if ratio else 0), d), np.float32)
    scored = ratio == 4 and cap < 512

    for seqlen, start in [(prompt, 0)] + [(1, p) for p in range(prompt, total)]:
        prefill = start == 0
        rows = seqlen if prefill else 1
        sl = slice(0, prompt) if prefill else slice(start, start + 1)
        n_comp = (start + rows) // ratio if ratio else 0
        scores = rng.standard_normal((rows, n_comp)).astype(np.float32) if scored and n_comp else None
        if scored and scores is None:
            scores = np.zeros((rows, 0), np.float32)
        got_o, got_rect, got_emit, got_src = layer.step(kv_all[sl], q_all[sl], ckv[sl] if ratio else None,
                                                        cscore[sl] if ratio else None, scores, seqlen, start)
        # ---- the oracle's twin of the same step ----
        code, entry = oracle.act_quant_f8_prefix(kv_all[sl], d - rd, 64)
        assert code == 0 and oracle.ring_write(entry, o_cache[:win], win, seqlen, start) == 0
        want_emit = None
        if ratio:
            assert oracle.kv_compress_deposit(ckv[sl], cscore[sl], ape, o_state[0], o_state[1], og, rows,
                                              start % ratio) == 0
            dst = oracle.compress_dst(ratio, win, seqlen, start)
            if dst is not None:
                first, count = dst
                if prefill:
                    code, pooled = oracle.kv_compress_prefill(ckv[sl], cscore[sl], ape, norm, freqs, og, count)
                else:
                    code, pooled = oracle.kv_compress_decode(o_state[0], o_state[1], norm, freqs, og, start)
                    pooled = pooled.reshape(1, d)
                assert code == 0
                code, want_emit = oracle.act_quant_f8_prefix(pooled, d - rd, 64)
                o_cache[first:first + count] = want_emit
        what = f"seqlen {seqlen} start {start}"
        # ring: bit for bit
        ring = back(layer.cache, np.float32).reshape(-1, d)[:win]
        assert np.array_equal(ring.view(np.uint32), o_cache[:win].view(np.uint32)), what
        # pooled rows: which call emits, where, and the values to the compressor's bar
        assert (got_emit is None) == (want_emit is None), what
        if want_emit is not None:
            got_pooled, got_quant = got_emit
            gap = compress_gap(oracle, got_pooled, pooled, rd)
            assert gap.max() <= CLEAN_ULP and np.mean(gap > 0) < 0.01, (what, int(gap.max()))
            # after the block quantization a pooled value one code off may sit on the next fp8
            # step (1/8 of the value), or move its block's power-of-two scale: rare, and bounded
            off = np.abs(got_quant - want_emit) > 0
            assert np.mean(off) < 0.02, (what, float(np.mean(off)))
            assert np.all(np.abs(got_quant - want_emit) <= 0.126 * np.maximum(np.abs(want_emit), np.abs(got_quant))
                          + 2.0 ** -9 * np.abs(want_emit).max()), what
        # rectangle: bit for bit
        if scores is None:
            code, want_rect = oracle.sel_gather(win, ratio, cap, seqlen, start)
        else:
            code, want_rect = oracle.sel_gather_scored(scores, win, ratio, cap, seqlen, start)
        assert code == 0 and np.array_equal(got_rect, want_rect), what
        assert got_rect.max() < got_src.shape[0], what             # every index names a row of the buffer attended
        # attention: the oracle over the device's own rows
        want_o = oracle.sparse_attn(q_all[sl], got_src, sink, got_rect, d ** -0.5)
        err = float(np.max(np.abs(got_o - want_o)) / np.max(np.abs(want_o)))
        assert err <= ATTEND_TOL, (what, err)
    if ratio:
        # every block that closed sits at its position's row; nothing else was written
        closed = total // ratio
        tail = back(layer.cache, np.float32).reshape(-1, d)[win:]
        assert np.abs(tail[:closed]).max() > 0 and not tail[closed:].any()
