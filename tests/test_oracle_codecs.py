"""Pins the oracle's element codecs against the reference's own known-answer tests and against
checks that share no line with the encoder (nearest-value brute force, closed forms)."""
import numpy as np


def all_e4m3_values():
    """Closed form for the 256 codes, written from the format (1-4-3, bias 7, no inf)."""
    vals = np.zeros(256, np.float64)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e, m = (c >> 3) & 0xF, c & 7
        if e == 0:
            vals[c] = s * m * 2.0 ** -9
        elif e == 15 and m == 7:
            vals[c] = np.nan
        else:
            vals[c] = s * (1 + m / 8) * 2.0 ** (e - 7)
    return vals


def brute_force_e4m3(x: np.ndarray) -> np.ndarray:
    """Nearest finite e4m3 magnitude; ties -> even mantissa for |x| >= 2^-6, away from zero
    below; |x| >= 448 saturates; |x| < 2^-10 is zero; NaN -> 0x7f."""
    mags = all_e4m3_values()[:0x7F]  # codes 0x00..0x7e, ascending
    out = np.zeros(x.shape, np.uint8)
    a = np.abs(x.astype(np.float64))
    sign = np.where(np.signbit(x), 0x80, 0).astype(np.uint8)
    d = np.abs(a[..., None] - mags[None, :])
    best = d.min(axis=-1, keepdims=True)
    is_best = d == best
    lo = is_best.argmax(axis=-1)
    hi = 0x7E - is_best[..., ::-1].argmax(axis=-1)
    tie = hi != lo
    even = np.where(lo % 2 == 0, lo, hi)
    code = np.where(tie, np.where(a >= 2.0 ** -6, even, hi), lo)
    code = np.where(a >= 448.0, 0x7E, code)
    code = np.where(a < 2.0 ** -10, 0, code)
    out = (code.astype(np.uint8) | sign)
    out = np.where(np.isnan(x), 0x7F, out).astype(np.uint8)
    return out


def test_e4m3_decode_closed_form(oracle):
    got = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    want = all_e4m3_values()
    assert np.isnan(got[0x7F]) and np.isnan(got[0xFF])
    fin = ~np.isnan(want)
    assert np.array_equal(got[fin], want[fin])
    # the sign of zero is carried
    assert np.signbit(oracle.e4m3_to_f32(np.array([0x80], np.uint8)))[0]


def test_e4m3_reference_known_values(oracle):
    """crates/core/src/routing.rs:338-362."""
    rt = lambda v: oracle.e4m3_to_f32(oracle.f32_to_e4m3(np.array([v], np.float32)))[0]
    for x in (0.0, 1.0, -2.0, 448.0, 1.5, 0.0625):
        assert rt(x) == np.float32(x)
    assert rt(1000.0) == 448.0 and rt(-1000.0) == -448.0
    for x in (0.3, -1.7, 12.5, 100.0, 0.011, -55.0):
        assert abs(rt(x) - x) <= abs(x) * 0.07 + 1e-3
    assert oracle.f32_to_e4m3(np.array([np.nan], np.float32))[0] == 0x7F
    assert np.isnan(rt(np.nan))


def test_e4m3_subnormal_ties_round_away(oracle):
    """The cache quantizer is half-AWAY in the subnormal band (crates/core/src/num.rs:143-150);
    round-to-nearest-even would give {0,2,4,6} here."""
    q = np.float32(2.0 ** -10)
    x = np.array([1, 5, 9, 13, 15, 3, 7, 11], np.float32) * q
    assert oracle.f32_to_e4m3(x).tolist() == [1, 3, 5, 7, 0x08, 2, 4, 6]
    assert oracle.f32_to_e4m3(-x).tolist() == [0x81, 0x83, 0x85, 0x87, 0x88, 0x82, 0x84, 0x86]
    # and RNE on the normal side: 1 + 1/16 ties to the even mantissa 0 (0x38), 1 + 3/16 to 2
    assert oracle.f32_to_e4m3(np.array([1.0625, 1.1875], np.float32)).tolist() == [0x38, 0x3A]


def test_e4m3_encode_roundtrips_every_finite_code(oracle):
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], np.uint8)
    assert np.array_equal(oracle.f32_to_e4m3(oracle.e4m3_to_f32(codes)), codes)


def test_e4m3_encode_matches_brute_force(oracle):
    vals = all_e4m3_values()[:0x7F]
    mids = (vals[:-1] + vals[1:]) / 2  # every tie, exactly representable in f32
    rng = np.random.default_rng(0xE4B3)
    nudged = np.concatenate([np.nextafter(mids.astype(np.float32), np.float32(0)),
                             np.nextafter(mids.astype(np.float32), np.float32(1e9))])
    rand = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 100,
        (rng.random(20000).astype(np.float32) - 0.5) * 0.06,   # subnormal band
        np.exp(rng.uniform(np.log(2.0 ** -12), np.log(600.0), 20000)).astype(np.float32),
    ])
    edge = np.array([447.99, 448.0, 464.0, 1e30, np.inf, 2.0 ** -10, 2.0 ** -6,
                     np.nextafter(np.float32(2.0 ** -10), np.float32(0)),
                     np.nextafter(np.float32(2.0 ** -6), np.float32(0)), 0.0, np.nan], np.float32)
    x = np.concatenate([vals.astype(np.float32), mids.astype(np.float32), nudged, rand, edge])
    x = np.concatenate([x, -x])
    got, want = oracle.f32_to_e4m3(x), brute_force_e4m3(x)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]
    # anti-vacuity: the probe set really contains ties of both kinds
    assert np.count_nonzero(np.isin(np.abs(x), mids.astype(np.float32))) >= 2 * len(mids)


def test_e4m3_encode_is_monotone(oracle):
    x = np.sort(np.random.default_rng(7).uniform(-500, 500, 100000).astype(np.float32))
    v = oracle.e4m3_to_f32(oracle.f32_to_e4m3(x))
    assert np.all(np.diff(v) >= 0)


def test_bf16_reference_known_values(oracle):
    """crates/core/src/routing.rs:259-284."""
    cases = [(0.0, 0x0000), (1.0, 0x3F80), (-2.0, 0xC000), (1.0 + 2.0 ** -8, 0x3F80),
             (1.0 + 2.0 ** -8 + 2.0 ** -16, 0x3F81), (np.inf, 0x7F80)]
    x = np.array([c[0] for c in cases], np.float32)
    assert oracle.f32_to_bf16(x).tolist() == [c[1] for c in cases]
    for bits, want in ((0x3F80, 1.0), (0xC000, -2.0), (0x7F80, np.inf)):
        assert oracle.lib.ro_bf16_to_f32(bits) == want
    nan16 = int(oracle.f32_to_bf16(np.array([np.nan], np.float32))[0])
    assert np.isnan(oracle.lib.ro_bf16_to_f32(nan16))


def test_bf16_matches_torch_on_random_bits(oracle):
    """An independent library's RNE: torch's float32 -> bfloat16 cast on the CPU."""
    import torch

    bits = np.random.default_rng(11).integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)


def test_bf16_exhaustive_vs_textbook_rne(oracle):
    assert oracle.selftest_bf16_exhaustive() == 0
