"""Pins the oracle's compressor pooling (deposit, prefill, decode) by restatements that share
no line with it and by the reference's own state machine as an invariant."""
import numpy as np
import pytest

from oracle.kvoracle import CompGeom
from tests.v4_cases import bf16_gap, compress_inputs, literal_finish, literal_pooling


@pytest.mark.parametrize("ratio,d,rd,s", [(4, 512, 64, 64), (4, 64, 16, 23), (128, 512, 64, 384), (8, 32, 8, 40)])
def test_prefill_against_a_literal_float64_restatement(oracle, ratio, d, rd, s):
    g = CompGeom.attention(ratio, d, rd)
    kv, score, ape, norm, freqs = compress_inputs(g, s, seed=ratio * 1000 + d)
    nblk = s // ratio
    code, got = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, g, nblk)
    assert code == 0
    want = literal_finish(oracle, g, literal_pooling(g, kv, score, ape, nblk), norm, freqs, 0)
    gap = bf16_gap(oracle, got, want)
    # float32 against float64 arithmetic can land on the other side of a bf16 rounding, once per
    # store: two stores downstream of the pooling
    assert gap.max() <= 2 and np.mean(gap > 0) < 0.02, (gap.max(), np.mean(gap > 0))


def test_pooling_closed_forms(oracle):
    g = CompGeom.attention(4, 64, 16)
    kv, score, ape, norm, freqs = compress_inputs(g, 16, seed=5)
    one = np.ones(g.d, np.float32)
    flat = np.zeros_like(freqs)
    flat[:, 0::2] = 1.0                                  # cos 1, sin 0: no rotation
    # equal scores -> the mean of the window's entries (block 0: its own four rows only)
    code, got = oracle.kv_compress_prefill(kv, np.zeros_like(score), np.zeros_like(ape), one, flat, g, 4)
    own = kv.reshape(4, 4, g.cd)[:, :, g.d:]             # [block, row, normal half]
    prev = kv.reshape(4, 4, g.cd)[:, :, :g.d]            # [block, row, overlap half]
    mean = np.empty((4, g.d))
    mean[0] = own[0].astype(np.float64).mean(axis=0)
    for b in range(1, 4):
        mean[b] = np.concatenate([prev[b - 1], own[b]]).astype(np.float64).mean(axis=0)
    want = literal_finish(oracle, g, mean, one, flat, 0)
    assert code == 0 and bf16_gap(oracle, got, want).max() <= 2
    # one dominant score -> that entry alone: row 2 of the previous block, overlap half
    sc = np.zeros_like(score)
    sc[4 + 2, :g.d] = 80.0
    code, got = oracle.kv_compress_prefill(kv, sc, np.zeros_like(ape), one, flat, g, 3)
    want = literal_finish(oracle, g, kv[6:7, :g.d].astype(np.float64), one, flat, 0)
    assert bf16_gap(oracle, got[2:3], want).max() <= 1
    # ... and the rotation really depends on the block's FIRST position (block 2 -> position 8)
    code, rot = oracle.kv_compress_prefill(kv, sc, np.zeros_like(ape), one, freqs, g, 3)
    want = literal_finish(oracle, g, kv[6:7, :g.d].astype(np.float64), one, freqs[8:], 0)
    assert bf16_gap(oracle, rot[2:3], want).max() <= 1 and not np.array_equal(rot[2], got[2])


def run_decode_continuation(oracle, g, kv, score, ape, norm, freqs, s0):
    """Prefill s0 tokens, then feed the rest one token at a time; returns every emitted block."""
    s = kv.shape[0]
    # the state a sequence starts with (crates/engine/src/v4/kvcompress.rs:222): kv zeroed, scores
    # -inf, so a window that was never filled weighs nothing
    states = [np.zeros((g.coff * g.ratio, g.cd), np.float32),
              np.full((g.coff * g.ratio, g.cd), -np.inf, np.float32)]
    assert oracle.kv_compress_deposit(kv[:s0], score[:s0], ape, states[0], states[1], g, s0, 0) == 0
    blocks = []
    if s0 >= g.ratio:
        code, out = oracle.kv_compress_prefill(kv[:s0], score[:s0], ape, norm, freqs, g, s0 // g.ratio)
        assert code == 0
        blocks += list(out)
    for pos in range(s0, s):
        assert oracle.kv_compress_deposit(kv[pos:pos + 1], score[pos:pos + 1], ape, states[0], states[1],
                                          g, 1, pos % g.ratio) == 0
        if (pos + 1) % g.ratio == 0:
            code, out = oracle.kv_compress_decode(states[0], states[1], norm, freqs, g, pos)
            assert code == 0
            blocks.append(out)
    return np.array(blocks)


@pytest.mark.parametrize("ratio,d,rd,s,s0", [(4, 64, 16, 41, 13), (4, 64, 16, 40, 12), (4, 32, 8, 30, 2),
                                              (128, 64, 16, 400, 130), (8, 32, 8, 50, 19), (4, 512, 64, 24, 8)])
def test_prefill_then_decode_emits_the_blocks_of_one_long_prefill(oracle, ratio, d, rd, s, s0):
    g = CompGeom.attention(ratio, d, rd)
    kv, score, ape, norm, freqs = compress_inputs(g, s, seed=s * 7 + ratio)
    code, whole = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, g, s // ratio)
    assert code == 0
    stepped = run_decode_continuation(oracle, g, kv, score, ape, norm, freqs, s0)
    assert stepped.shape == whole.shape
    assert np.array_equal(stepped.view(np.uint32), whole.view(np.uint32))


def test_deposit_fills_the_state_as_the_reference_describes(oracle):
    """crates/backend/kernels/kvcompress.hip:205-262: a prefill of s tokens leaves the last
    complete block in slots [0, ratio) (overlapping layers) and the s % ratio trailing rows from
    slot state_off; the scores carry the embedding of the row's slot WITHIN its block."""
    g = CompGeom.attention(4, 32, 8)
    kv, score, ape, _, _ = compress_inputs(g, 11, seed=3)
    st_kv, st_sc = np.full((8, g.cd), 7.0, np.float32), np.full((8, g.cd), 7.0, np.float32)
    assert oracle.kv_compress_deposit(kv, score, ape, st_kv, st_sc, g, 11, 0) == 0
    assert np.array_equal(st_kv[:4], kv[4:8]) and np.array_equal(st_sc[:4], score[4:8] + ape)
    assert np.array_equal(st_kv[4:7], kv[8:11]) and np.array_equal(st_sc[4:7], score[8:11] + ape[:3])
    assert np.all(st_kv[7] == 7.0) and np.all(st_sc[7] == 7.0)
    # decode: one row into slot state_off + pos % ratio, embedding of pos % ratio
    assert oracle.kv_compress_deposit(kv[:1], score[:1], ape, st_kv, st_sc, g, 1, 3) == 0
    assert np.array_equal(st_kv[7], kv[0]) and np.array_equal(st_sc[7], score[0] + ape[3])
    # without overlap the state is one window from slot 0
    g8 = CompGeom.attention(8, 32, 8)
    kv, score, ape, _, _ = compress_inputs(g8, 21, seed=4)
    st_kv, st_sc = np.zeros((8, g8.cd), np.float32), np.zeros((8, g8.cd), np.float32)
    assert oracle.kv_compress_deposit(kv, score, ape, st_kv, st_sc, g8, 21, 0) == 0
    assert np.array_equal(st_kv[:5], kv[16:21]) and np.array_equal(st_sc[:5], score[16:21] + ape[:5])


def test_compress_guards(oracle):
    """crates/backend/kernels/kvcompress.hip:386-478."""
    ok = CompGeom.attention(4, 32, 8)
    bad = [(CompGeom(1, 1, 32, 32, 1, 8, 1e-6), 1001), (CompGeom(4, 3, 32, 96, 12, 8, 1e-6), 1001),
           (CompGeom(4, 2, 32, 64, 8, 7, 1e-6), 1002), (CompGeom(4, 2, 32, 64, 8, 34, 1e-6), 1002),
           (CompGeom(4, 2, 32, 32, 8, 8, 1e-6), 1003), (CompGeom(4, 2, 32, 64, 4, 8, 1e-6), 1003),
           (CompGeom(256, 1, 32, 32, 256, 8, 1e-6), 1004), (CompGeom(128, 2, 32, 64, 256, 8, 1e-6), 1004),
           (CompGeom(8, 2, 32, 64, 16, 8, 1e-6), 1010), (CompGeom(4, 1, 32, 32, 4, 8, 1e-6), 1010)]
    for geom, code in bad:
        assert oracle.compress_guard(geom) == code, (geom.ratio, geom.coff)
    kv, score, ape, norm, freqs = compress_inputs(ok, 8, seed=1)
    st = [np.zeros((8, ok.cd), np.float32) for _ in range(2)]
    assert oracle.kv_compress_deposit(kv, score, ape, st[0], st[1], ok, 0, 0) == 1005
    assert oracle.kv_compress_deposit(kv, score, ape, st[0], st[1], ok, 3, 2) == 1008
    assert oracle.kv_compress_deposit(kv, score, ape, st[0], st[1], ok, 1, -1) == 1008
    assert oracle.kv_compress_prefill(kv, score, ape, norm, freqs, ok, 0)[0] == 1006
    assert oracle.kv_compress_decode(st[0], st[1], norm, freqs, ok, 0)[0] == 1007
    assert oracle.kv_compress_decode(st[0], st[1], norm, freqs, ok, 5)[0] == 1009
    assert oracle.kv_compress_decode(st[0], st[1], norm, freqs, ok, 7)[0] == 0
