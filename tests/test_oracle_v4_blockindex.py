"""Pins the oracle's restatement of the indexer's spread (Hadamard + simulated fp4) and of its
block scorer (crates/backend/kernels/blockindex.hip) against the reference's own known-answer
tests and against checks that share no line with the restatement: an explicitly built
Sylvester matrix, an enumeration of the eight fp4 magnitudes, exact power-of-two arithmetic,
closed forms of the score chain."""
import math

import numpy as np
import pytest
import scipy.linalg

from tests.util import bf16_to_f32, f32_to_bf16_rne

MAGS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def bf16_round(x):
    return bf16_to_f32(f32_to_bf16_rne(np.ascontiguousarray(x, np.float32)))


# ---- e2m1 -------------------------------------------------------------------------------------

def test_e2m1_ties_go_to_the_even_mantissa(oracle):
    """crates/oracles/tests/v4_oracle_codecs.rs:163-180, the seven midpoints as written there."""
    for probe, want in [(0.25, 0.0), (0.75, 1.0), (1.25, 1.0), (1.75, 2.0), (2.5, 2.0), (3.5, 4.0),
                        (5.0, 4.0)]:
        assert oracle.e2m1_decode(oracle.e2m1_encode(probe)) == want
        assert oracle.e2m1_decode(oracle.e2m1_encode(-probe)) == -want


def test_e2m1_is_nearest_saturates_and_round_trips(oracle):
    """v4_oracle_codecs.rs:181-207: nearest magnitude by enumeration, +-1e9 -> +-6, every code
    its own nearest."""
    rng = np.random.default_rng(0xE2)
    for a in (rng.random(4000) * 8.0).astype(np.float32):
        got = abs(float(oracle.e2m1_decode(oracle.e2m1_encode(a))))
        dist = np.abs(MAGS - min(float(a), 6.0))
        assert abs(got - min(float(a), 6.0)) == dist.min(), a
    assert oracle.e2m1_decode(oracle.e2m1_encode(1e9)) == 6.0
    assert oracle.e2m1_decode(oracle.e2m1_encode(-1e9)) == -6.0
    for c in range(16):
        assert oracle.e2m1_encode(oracle.e2m1_decode(c)) == c
    assert [float(oracle.e2m1_decode(c)) for c in range(8)] == list(MAGS)


# ---- Hadamard ---------------------------------------------------------------------------------

@pytest.mark.parametrize("n", [2, 8, 32, 128, 256])
def test_hadamard_is_the_sylvester_matrix_in_natural_order(oracle, n):
    """The basis order is what a restatement gets wrong silently (every order is orthogonal):
    small integers make H x exact in f32, so the butterflies must equal the product with
    scipy's Sylvester construction — the contract the reference settles on
    (blockindex.hip:45-55) — up to the one closing multiply."""
    rng = np.random.default_rng(n)
    x = rng.integers(-8, 9, n).astype(np.float32)
    want = (scipy.linalg.hadamard(n).astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    scale = np.float32(1.0) / np.sqrt(np.float32(n))
    np.testing.assert_array_equal(oracle.hadamard_rotate(x), want * scale)
    # a sequency-ordered (Walsh) matrix differs on the same input: the check can fail
    walsh = scipy.linalg.hadamard(n)[np.argsort([(np.diff(r) != 0).sum() for r in scipy.linalg.hadamard(n)])]
    if n > 2:
        assert not np.array_equal(walsh @ x.astype(np.float64), want.astype(np.float64))


def test_hadamard_is_its_own_inverse_and_keeps_the_norm(oracle):
    """v4_oracle_codecs.rs:387-420."""
    rng = np.random.default_rng(7)
    for n in (2, 8, 128):
        x = rng.random(n).astype(np.float32)
        y = oracle.hadamard_rotate(x)
        assert not np.array_equal(x, y)
        np.testing.assert_allclose(oracle.hadamard_rotate(y), x, atol=1e-5)
        assert abs(float((x * x).sum()) - float((y * y).sum())) < 1e-4 * max(float((x * x).sum()), 1.0)


# ---- fp4 block quantization -------------------------------------------------------------------

def exact_pow2_scale(amax: float) -> float:
    """The smallest power of two >= amax / 6, from the exact mantissa/exponent split."""
    y = float(np.float32(amax) * (np.float32(1.0) / np.float32(6.0)))
    m, e = math.frexp(y)            # y = m * 2^e, 0.5 <= m < 1
    return math.ldexp(1.0, e - 1) if m == 0.5 else math.ldexp(1.0, e)


def test_fp4_quant_lands_on_the_grid_of_its_own_power_of_two_scale(oracle):
    rng = np.random.default_rng(0xF4)
    for trial in range(200):
        binade = int(rng.integers(-40, 40))
        x = (rng.standard_normal(64) * 2.0 ** binade).astype(np.float32)
        got = oracle.fp4_act_quant(x, 32)
        for b in range(2):
            seg, out = x[32 * b:32 * b + 32], got[32 * b:32 * b + 32]
            s = exact_pow2_scale(float(np.abs(seg).max()))
            q = np.clip(seg.astype(np.float64) / s, -6.0, 6.0)
            dist = np.abs(np.abs(q)[:, None] - MAGS[None, :])
            # nearest magnitude; at a tie the reference's table decides, checked separately
            ok = np.isclose(np.abs(out.astype(np.float64)) / s, MAGS[dist.argmin(axis=1)]) | \
                (np.sort(dist, axis=1)[:, 0] == np.sort(dist, axis=1)[:, 1])
            assert ok.all(), (trial, b)
            assert (np.signbit(out) == np.signbit(seg)).all()
            assert np.abs(seg).max() <= 6.0 * s < 2.0 * max(np.abs(seg).max(), 6.0 * 2.0 ** -126) * (1 + 1e-6)


def test_fp4_quant_zero_block_uses_the_floor_and_stays_zero(oracle):
    got = oracle.fp4_act_quant(np.zeros(32, np.float32), 32)
    assert (got == 0).all()
    tiny = np.full(32, 2.0 ** -126, np.float32)  # below the floor 6 * 2^-126: scale 2^-126
    assert (oracle.fp4_act_quant(tiny, 32) == np.float32(2.0 ** -126)).all()


# ---- the spread as a whole --------------------------------------------------------------------

def test_spread_is_the_four_steps_in_the_reference_order(oracle):
    """crates/engine/tests/kernel_v4_indexer.rs:149-156: rotate, store bf16, quantize, store
    bf16. Dropping the store between rotation and quantization changes block scales; the
    composition here is built from the separately pinned parts."""
    rng = np.random.default_rng(11)
    x = bf16_round(rng.standard_normal((9, 128)).astype(np.float32))
    code, got = oracle.act_quant_f4_rotated(x)
    assert code == 0
    differs_without_store = False
    for r in range(9):
        rot = oracle.hadamard_rotate(x[r])
        want = bf16_round(oracle.fp4_act_quant(bf16_round(rot), 32))
        np.testing.assert_array_equal(got[r], want)
        differs_without_store |= not np.array_equal(bf16_round(oracle.fp4_act_quant(rot, 32)), want)
    assert differs_without_store  # the store between the two steps is visible on this input
    # 60 binades (kernel_v4_indexer.rs:246-277): every row lands on its own scale
    base = bf16_round(rng.standard_normal((60, 128)).astype(np.float32))
    wide = bf16_round(base * (2.0 ** (np.arange(60) - 30))[:, None].astype(np.float32))
    code, spread = oracle.act_quant_f4_rotated(wide)
    assert code == 0
    np.testing.assert_array_equal(spread, (oracle.act_quant_f4_rotated(base)[1] *
                                           (2.0 ** (np.arange(60) - 30))[:, None]).astype(np.float32))


def test_spread_guards(oracle):
    """blockindex.hip:241-257 and kernel_v4_indexer.rs:287-320."""
    z = lambda r, d: np.zeros((r, d), np.float32)
    assert oracle.act_quant_f4_rotated(z(1, 128))[0] == 0
    assert oracle.act_quant_f4_rotated(z(1, 512))[0] == 1002
    assert oracle.act_quant_f4_rotated(z(1, 96))[0] == 1003
    assert oracle.act_quant_f4_rotated(z(1, 16))[0] == 1004
    assert oracle.lib.ro_act_quant_f4_rotated(None, 0, 128) == 1001


# ---- the block scorer -------------------------------------------------------------------------

def test_score_accumulates_in_f32_and_rounds_once(oracle):
    """kernel_v4_indexer.rs:689-726: one unit term and 63 terms of 2^-9 give 1.125; a bf16
    running fold would give 1.0."""
    heads, hd = 64, 128
    kv = np.zeros((1, hd), np.float32)
    kv[0, 0] = 1.0
    q = np.zeros((1, heads, hd), np.float32)
    q[0, :, 0] = 2.0 ** -9
    q[0, 0, 0] = 1.0
    code, got = oracle.index_score_blocks(q, kv, np.ones((1, heads), np.float32))
    assert code == 0 and got.shape == (1, 1)
    assert got[0, 0] == np.float32(1.125)


def test_score_chain_closed_forms(oracle):
    """One live dim per head makes every fold a single term, so each store and the relu are
    visible one at a time: score = bf16(sum_h bf16(relu(bf16(q_h k)) * w_h)) with the sum exact."""
    heads, hd = 4, 32
    q = np.zeros((1, heads, hd), np.float32)
    kv = np.zeros((2, hd), np.float32)
    q[0, :, 5] = [1.0, -2.0, 1.0 + 2.0 ** -9, 3.0]      # head 2's product needs the first store
    kv[0, 5], kv[1, 5] = 1.0, -1.0
    w = np.array([[0.5, 4.0, 1.0, -0.25]], np.float32)   # signed weights
    code, got = oracle.index_score_blocks(q, kv, w)
    assert code == 0
    # block 0: dots 1, -2 (relu -> 0), bf16(1 + 2^-9) = 1, 3 -> 0.5 + 0 + 1 - 0.75
    assert got[0, 0] == np.float32(0.75)
    # block 1: dots -1, 2, -1, -3 -> only head 1 survives: 2 * 4
    assert got[0, 1] == np.float32(8.0)


def test_score_dot_is_a_sequential_f32_fold_without_fusion(oracle):
    """Three terms chosen so that the order of the additions and a fused multiply-add each
    change the bits: (2^24 + 1*1) loses the 1 unless it is added last; a * b with a = b =
    1 + 2^-12 rounds before the add."""
    hd = 4
    a = np.float32(1.0 + 2.0 ** -12)
    q = np.zeros((1, 1, hd), np.float32)
    kv = np.zeros((1, hd), np.float32)
    q[0, 0, :3] = [2.0 ** 24, 1.0, -(2.0 ** 24)]
    kv[0, :3] = [1.0, 1.0, 1.0]
    code, got = oracle.index_score_blocks(q, kv, np.ones((1, 1), np.float32))
    assert got[0, 0] == 0.0            # ((2^24 + 1) - 2^24) = 0 in sequence; 1 in any other order
    q[0, 0, :3] = [a, -1.0, 0.0]
    kv[0, :3] = [a, np.float32(1.0 + 2.0 ** -11), 0.0]
    code, got = oracle.index_score_blocks(q, kv, np.full((1, 1), 2.0 ** 30, np.float32))
    # a * a rounds to 1 + 2^-11 (the 2^-24 is lost); fused, the 2^-24 would survive the subtraction
    assert got[0, 0] == 0.0


def test_score_guards(oracle):
    """blockindex.hip:264-275."""
    q, kv, w = np.zeros((1, 2, 8), np.float32), np.zeros((0, 8), np.float32), np.zeros((1, 2), np.float32)
    assert oracle.index_score_blocks(q, kv, w)[0] == 1005
    assert oracle.lib.ro_index_score_blocks(None, None, None, None, 0, 1, 1, 1) == 1001
