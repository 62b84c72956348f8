"""Pins the oracle's functions for the second cache format (simulated-fp8 rows, scored block
selection) against the reference's own known-answer tests and against checks that share no
line with them."""
import math
import struct

import numpy as np

from tests.test_oracle_codecs import all_e4m3_values

FP8_MAX = np.float32(448.0)


def nearest_ties_even(x: np.ndarray) -> np.ndarray:
    """Nearest finite e4m3 magnitude by enumeration, ties to the even code, float64 distances
    (the technique of crates/oracles/tests/v4_oracle_codecs.rs:27-57)."""
    mags = all_e4m3_values()[:0x7F]
    a = np.abs(x.astype(np.float64))
    d = np.abs(a[..., None] - mags[None, :])
    best = d.min(axis=-1, keepdims=True)
    is_best = d == best
    lo = is_best.argmax(axis=-1)
    hi = 0x7E - is_best[..., ::-1].argmax(axis=-1)
    code = np.where(lo % 2 == 0, lo, hi)          # one candidate: lo == hi; two: the even one
    sign = np.where(np.signbit(x), 0x80, 0)
    return (code | sign).astype(np.uint8)


def rne_probe_set():
    vals = all_e4m3_values()[:0x7F].astype(np.float32)
    mids = ((all_e4m3_values()[:0x7E] + all_e4m3_values()[1:0x7F]) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))])
    rng = np.random.default_rng(0xE4)
    band = np.exp(rng.uniform(np.log(2.0 ** -13), np.log(463.0), 60000)).astype(np.float32)
    x = np.concatenate([vals, mids, near, band])
    return np.concatenate([x, -x])


def test_rne_encoder_is_nearest_ties_to_even(oracle):
    x = rne_probe_set()
    got, want = oracle.e4m3_encode_rne(x), nearest_ties_even(x)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, [(x[i], hex(got[i]), hex(want[i])) for i in bad[:8]]
    # saturation and NaN, crates/oracles/tests/v4_oracle_codecs.rs:136-141
    assert oracle.e4m3_encode_rne(np.array([1e30, -1e30, 464.0, np.inf], np.float32)).tolist() == \
        [0x7E, 0xFE, 0x7E, 0x7E]
    assert oracle.e4m3_encode_rne(np.array([np.nan], np.float32))[0] == 0x7F
    # idempotent on every finite code, :143-150
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    assert np.array_equal(oracle.e4m3_encode_rne(oracle.e4m3_to_f32(codes)), codes)


def test_rne_and_half_away_differ_exactly_on_subnormal_ties(oracle):
    """crates/oracles/src/v4oracle/numerics.rs:60-67: the two rules differ by one code on exact
    halfway subnormals and nowhere else."""
    x = rne_probe_set()
    rne, away = oracle.e4m3_encode_rne(x), oracle.f32_to_e4m3(x)
    differ = rne != away
    q = np.float32(2.0 ** -10)
    ties = np.isin(np.abs(x), np.array([1, 5, 9, 13], np.float32) * q)   # odd multiples whose lower neighbour is even
    assert np.array_equal(differ, ties)
    assert oracle.e4m3_encode_rne(np.array([1, 3, 5, 7, 9, 11, 13, 15], np.float32) * q).tolist() == \
        [0, 2, 2, 4, 4, 6, 6, 8]


def test_round_scale_is_the_next_power_of_two(oracle):
    rng = np.random.default_rng(7)
    probes = [np.float32(2.0) ** e for e in range(-30, 31)]
    probes += [np.nextafter(p, np.float32(0)) for p in probes] + [np.nextafter(p, np.float32(1e30)) for p in probes]
    probes += list(np.exp(rng.uniform(np.log(1e-6), np.log(1e6), 4000)).astype(np.float32))
    one = np.float32(1.0)
    for y in probes:
        got = oracle.fast_round_scale(y, one)                       # max_inv = 1: the scale of y itself
        m, e = math.frexp(float(y))                                  # y = m * 2^e, 0.5 <= m < 1, exact
        want = 2.0 ** (e - 1) if m == 0.5 else 2.0 ** e
        assert float(got) == want, (y, got, want)
    # with the format's ceiling: a power of two, >= amax/448 as the device computes it, < twice that
    inv = one / FP8_MAX
    for amax in np.exp(rng.uniform(np.log(1e-4), np.log(1e5), 2000)).astype(np.float32):
        s = oracle.fast_round_scale(amax, inv)
        y = np.float32(amax) * inv
        assert math.frexp(float(s))[0] == 0.5 and y <= s < 2 * y
    assert oracle.fast_round_scale(448.0) == 1.0 and oracle.fast_round_scale(449.0) == 2.0


def reference_tie_block():
    """crates/engine/tests/kernel_v4_quant.rs:283-296."""
    q = np.float32(1.0 / 512.0)
    row = np.zeros(64, np.float32)
    row[0] = FP8_MAX
    i = np.arange(63)
    m = (i % 16).astype(np.float32) * np.float32(0.5)
    row[1:] = np.where(i % 2 == 0, m * q, -m * q)
    return row


def test_act_quant_on_the_reference_tie_fixture(oracle):
    row = reference_tie_block()
    code, got = oracle.act_quant_f8_prefix(row[None, :], 64, 64)
    assert code == 0
    got = got[0]
    # the expectation written out by hand: scale 1, every value is a multiple or a half multiple
    # of 2^-9; halves go to the even neighbour
    q = 2.0 ** -9
    mult = np.abs(row[1:].astype(np.float64)) / q
    lo = np.floor(mult)
    want = np.where(mult - lo == 0.5, np.where(lo % 2 == 0, lo, lo + 1), lo) * q * np.sign(row[1:])
    assert got[0] == 448.0 and np.array_equal(got[1:].astype(np.float64), want)
    assert np.array_equal(np.signbit(got), np.signbit(row))          # -0.0 keeps its sign
    # the reference test's two anti-vacuity checks (:300-322)
    assert np.count_nonzero((got != 0) & (np.abs(got) < 0.015625)) >= 8
    half_away = oracle.e4m3_to_f32(oracle.f32_to_e4m3(np.clip(row, -FP8_MAX, FP8_MAX)))
    assert not np.array_equal(half_away, got)


def test_act_quant_structure_and_guards(oracle):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((37, 512)) * np.exp(rng.uniform(-6, 6, (37, 1)))).astype(np.float32)
    x[3, 64:128] = 0.0                                               # all-zero block: the 1e-4 floor
    x[5, 7] = 3e4
    code, y = oracle.act_quant_f8_prefix(x, 448, 64)
    assert code == 0
    assert np.array_equal(y[:, 448:], x[:, 448:])                    # the tail is left alone
    blocks_in, blocks_out = x[:, :448].reshape(37, 7, 64), y[:, :448].reshape(37, 7, 64)
    amax = np.maximum(np.abs(blocks_in).max(axis=2), np.float32(1e-4))
    s = np.array([[oracle.fast_round_scale(a) for a in r] for r in amax], np.float32)
    ratio = blocks_out / s[:, :, None]
    grid = set(all_e4m3_values()[:0x7F].tolist())
    assert all(abs(v) in grid for v in ratio.ravel().tolist())       # e4m3 value x power of two
    assert np.all(np.abs(blocks_out - blocks_in) <= np.maximum(np.abs(blocks_in) / 16, s[:, :, None] * 2.0 ** -10))
    assert np.array_equal(blocks_out[3, 1], np.zeros(64, np.float32))
    # quantizing again changes nothing
    code, z = oracle.act_quant_f8_prefix(y, 448, 64)
    assert code == 0 and np.array_equal(z.view(np.uint32), y.view(np.uint32))
    # block 128 over the whole row into a second buffer
    code, w = oracle.act_quant_f8_prefix(x, 512, 128, inplace=False)
    assert code == 0 and not np.array_equal(w[:, :128], y[:, :128])
    # guards, crates/backend/kernels/mla.hip:529-541
    assert oracle.act_quant_f8_prefix(x, 448, 64, inplace=False)[0] == 1002
    assert oracle.act_quant_f8_prefix(x, 448, 60)[0] == 1004
    assert oracle.act_quant_f8_prefix(x, 0, 64)[0] == 1001
    assert oracle.act_quant_f8_prefix(x, 576, 64)[0] == 1001


def total_order_key(v) -> int:
    b = struct.unpack("<i", struct.pack("<f", v))[0]
    return b ^ 0x7FFFFFFF if b < 0 else b


def brute_force_rows(scores, ratio, index_topk, prefill, offset):
    rows, n_comp = scores.shape
    k = min(index_topk, n_comp)
    out = np.full((rows, k), -1, np.int32)
    for t in range(rows):
        limit = min((t + 1) // ratio, n_comp) if prefill else n_comp
        order = sorted(range(limit), key=lambda c: (-total_order_key(float(scores[t, c])), c))
        kept = sorted(order[:k])
        out[t, :len(kept)] = np.array(kept, np.int32) + offset
    return out


def test_scored_rows_reference_cases(oracle):
    """crates/engine/src/v4/select.rs:645-747."""
    # below the cap the scores do not matter: decode with 5 live blocks, prefill of 12 rows
    inc = np.arange(5, dtype=np.float32)[None, :]
    assert oracle.v4_scored_rows(inc, 4, 512, False, 128).tolist() == [[128, 129, 130, 131, 132]]
    pre = np.arange(36, dtype=np.float32).reshape(12, 3)
    got = oracle.v4_scored_rows(pre, 4, 512, True, 12)
    for t in range(12):
        live = (t + 1) // 4
        assert got[t].tolist() == [12 + c for c in range(live)] + [-1] * (3 - live)
    # above the cap: three-way tie keeps the lower indices; a bump moves the set
    s = np.array([[1.0, 1.0, 9.0, 0.5, 1.0]], np.float32)
    assert oracle.v4_scored_rows(s, 4, 3, False, 100).tolist() == [[100, 101, 102]]
    s[0, 4] = 2.0
    assert oracle.v4_scored_rows(s, 4, 3, False, 100).tolist() == [[100, 102, 104]]
    # a prefill row cannot take a block that closed after it
    s = np.tile(np.array([0.1, 9.0], np.float32), (8, 1))
    assert oracle.v4_scored_rows(s, 4, 1, True, 10).ravel().tolist() == [-1, -1, -1, 10, 10, 10, 10, 11]


def test_scored_rows_against_a_brute_force_total_order_sort(oracle):
    rng = np.random.default_rng(0x5E1)
    for rows, n_comp, ratio, topk, prefill in ((1, 300, 4, 64, False), (40, 9, 4, 3, True),
                                               (130, 2, 128, 1, True), (3, 50, 4, 50, False),
                                               (17, 33, 4, 40, True)):
        s = rng.standard_normal((rows, n_comp)).astype(np.float32)
        s[rng.random(s.shape) < 0.3] = np.float32(0.5)               # heavy ties
        s.ravel()[::7] = np.float32(-0.0)
        s.ravel()[3::11] = np.float32(0.0)                           # -0 sorts strictly below +0 here
        s.ravel()[5::13] = np.float32(-np.inf)
        s.ravel()[1::29] = np.float32(np.inf)
        want = brute_force_rows(s, ratio, topk, prefill, 1000)
        assert np.array_equal(oracle.v4_scored_rows(s, ratio, topk, prefill, 1000), want)
    # the zero signs matter under total order: with k = 1 the +0.0 wins over an earlier -0.0
    z = np.array([[-0.0, 0.0, -0.0]], np.float32)
    assert oracle.v4_scored_rows(z, 4, 1, False, 0).tolist() == [[1]]
