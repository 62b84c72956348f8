"""Quantize-and-append on the device against the CPU oracle (bit-exact codes, scales, bf16
keys), on the reference's own fixture, on benchmark configurations 1 and 2, and on rows built to sit
on the quantizer's rounding ties."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.test_oracle_quant import fixture_a99e
from tests.util import f32_to_bf16_rne, make_rows_bf16, shuffled_block_tables, slots_for

pytestmark = pytest.mark.gpu
W, PT = 576, 64


def test_append_kv_reference_fixture(oracle):
    """crates/engine/tests/fwd_kernel.rs:139-214 — five-row slabs, row 3 written."""
    rows, kvl, ropn, pos, nb = 5, 256, 64, 3, 2
    latent, rope = fixture_a99e(oracle)
    want = [np.zeros(rows * kvl, np.uint8), np.zeros(rows * nb, np.float32),
            np.zeros(rows * ropn, np.uint16)]
    assert oracle.append_kv(latent, rope, *want, pos, kvl, ropn, nb) == 0
    c8, ls, rc = dzeros(rows * kvl), dzeros(rows * nb * 4), dzeros(rows * ropn * 2)
    hip.launch_append_kv(dev(latent), dev(rope), c8, ls, rc, pos, kvl, ropn, nb)
    assert np.count_nonzero(want[0]) > kvl // 2
    assert np.array_equal(back(c8), want[0])
    assert np.array_equal(back(ls, np.uint32), want[1].view(np.uint32))
    assert np.array_equal(back(rc, np.uint16), want[2])


def test_reference_append_kv_agrees_with_the_oracle(oracle):
    """The reference's own kernel (fwd.hip compiled for this GPU) on the same fixture."""
    ref = need_ref("rivoli_append_kv")
    rows, kvl, ropn, pos, nb = 5, 256, 64, 3, 2
    latent, rope = fixture_a99e(oracle)
    want = [np.zeros(rows * kvl, np.uint8), np.zeros(rows * nb, np.float32),
            np.zeros(rows * ropn, np.uint16)]
    assert oracle.append_kv(latent, rope, *want, pos, kvl, ropn, nb) == 0
    r8, rs, rr = dzeros(rows * kvl), dzeros(rows * nb * 4), dzeros(rows * ropn * 2)
    lat_d, rope_d = dev(latent), dev(rope)
    assert ref.rivoli_append_kv(lat_d.data_ptr(), rope_d.data_ptr(), r8.data_ptr(),
                                rs.data_ptr(), rr.data_ptr(), pos, kvl, ropn, nb) == 0
    assert np.array_equal(back(r8), want[0])
    assert np.array_equal(back(rs, np.uint32), want[1].view(np.uint32))
    assert np.array_equal(back(rr, np.uint16), want[2])


def test_append_kv_guards():
    b = dzeros(4096)
    for args, code in (((-1, 256, 64, 2), 1001), ((0, 0, 64, 2), 1001), ((0, 192, 64, 2), 1002),
                       ((0, 2048, 64, 16), 1002), ((0, 128, 256, 1), 1002)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_append_kv(b, b, b, b, b, *args)
        assert e.value.code == code
    assert str(e.value) == "append_kv: argument guard rejected (1002)"


def test_append_kv_rows_matches_per_token_oracle(oracle):
    """GLM dims (kvl 512, rope 64, 4 block scales), 37 tokens from pos 5, in one launch."""
    n, kvl, ropn, nb, pos0, rows = 37, 512, 64, 4, 5, 50
    rng = np.random.default_rng(12)
    latent = (rng.standard_normal((n, kvl)) * rng.choice([0.01, 1, 30], (n, 1))).astype(np.float32)
    latent[3, 128:256] = 0.0                      # an all-zero block: scale 1.0, codes 0
    rope = rng.standard_normal((n, ropn)).astype(np.float32)
    want = [np.full(rows * kvl, 0xEE, np.uint8), np.full(rows * nb, 7.0, np.float32),
            np.full(rows * ropn, 0xABCD, np.uint16)]
    for t in range(n):
        oracle.append_kv(latent[t], rope[t], *want, pos0 + t, kvl, ropn, nb)
    c8, ls, rc = dev(np.full(rows * kvl, 0xEE, np.uint8)), dev(np.full(rows * nb, 7.0, np.float32)), \
        dev(np.full(rows * ropn, 0xABCD, np.uint16))
    hip.launch_append_kv_rows(dev(latent), dev(rope), c8, ls, rc, pos0, n, kvl, ropn, nb)
    assert np.array_equal(back(c8), want[0])
    assert np.array_equal(back(ls, np.uint32), want[1].view(np.uint32))
    assert np.array_equal(back(rc, np.uint16), want[2])


def test_index_append_reference_fixture(oracle):
    """crates/engine/tests/indexer_kernel.rs:119-140 — seven-row slab, row 5."""
    rows, hd, pos = 7, 128, 5
    k = oracle.lcg(0xC0DE).fill(hd) * np.float32(8.0)
    want = np.zeros(rows * hd, np.uint16)
    oracle.index_append(k, want, pos, hd)
    cache = dzeros(rows * hd * 2)
    hip.launch_index_append(dev(k), cache, pos, hd)
    assert np.array_equal(back(cache, np.uint16), want)
    with pytest.raises(hip.LaunchError):
        hip.launch_index_append(dev(k), cache, -1, hd)


def test_reference_index_append_agrees_with_the_oracle(oracle):
    """The reference's own kernel (indexer.hip compiled for this GPU) on the same fixture."""
    ref = need_ref("rivoli_index_append")
    rows, hd, pos = 7, 128, 5
    k = oracle.lcg(0xC0DE).fill(hd) * np.float32(8.0)
    want = np.zeros(rows * hd, np.uint16)
    oracle.index_append(k, want, pos, hd)
    rcache, kd = dzeros(rows * hd * 2), dev(k)
    assert ref.rivoli_index_append(kd.data_ptr(), rcache.data_ptr(), pos, hd) == 0
    assert np.array_equal(back(rcache, np.uint16), want)


def paged_append_both(oracle, rows, slots, n_pages, fill=0xA5):
    page_bytes = oracle.kv_page_bytes(PT, W)
    assert hip.kv_page_bytes(PT, W) == page_bytes
    want = np.full(n_pages * page_bytes, fill, np.uint8)
    bad_want = oracle.kv_append_paged(rows, slots, want, W, PT, n_pages)
    pool, bad = dzeros(n_pages * page_bytes, fill), dzeros(4)
    hip.launch_kv_append_paged(dev(rows), dev(slots), pool, slots.size, W, PT, n_pages, bad)
    return back(pool), want, int(back(bad, np.uint32)[0]), bad_want


def test_config1_append_one_token_after_4095(oracle):
    """benchmark configuration 1: 4095 cached tokens, block table = seeded permutation of 64 pages,
    append the 4096th."""
    table = shuffled_block_tables(1, 64, 64, seed=0x5EED0001)[0]
    rows = make_rows_bf16(4096, W, seed=0x5EED0001)
    slots = slots_for(table, np.arange(4096))
    got, want, bad, bad_want = paged_append_both(oracle, rows[:4095], slots[:4095], 64)
    assert np.array_equal(got, want) and bad == bad_want == 0
    # now the decode step: one token into the live pool
    pool = dev(got)
    hip.launch_kv_append_paged(dev(rows[4095:]), dev(slots[4095:]), pool, 1, W, PT, 64)
    oracle.kv_append_paged(rows[4095:], slots[4095:], want, W, PT, 64)
    assert np.array_equal(back(pool), want)


def test_config2_prefill_bulk_append_with_outlier_rows(oracle):
    """benchmark configuration 2: 8192 rows, 0.5% of rows x50, 128 shuffled pages."""
    table = shuffled_block_tables(1, 128, 128, seed=0x5EED0002)[0]
    rows = make_rows_bf16(8192, W, seed=0x5EED0002, outlier_frac=0.005, outlier_mul=50.0)
    slots = slots_for(table, np.arange(8192))
    got, want, bad, _ = paged_append_both(oracle, rows, slots, 128)
    assert bad == 0
    mism = np.flatnonzero(got != want)
    assert mism.size == 0, mism[:10]
    scales = got.reshape(128, -1)[:, PT * W:].copy().view(np.float32)
    assert scales.max() / np.median(scales) > 20      # the outlier rows really moved the scale


def special_rows():
    """19 rows that meet every branch of the quantizer: subnormal and normal ties, zeros, tiny
    and huge scales, outliers, NaNs and infinities."""
    f32 = np.zeros((19, W), np.float32)
    q = np.float32(2.0 ** -10)
    # row 0: a 448 pins scale == 1; the rest are multiples and half-multiples of the subnormal
    # quantum in both signs, so exact subnormal ties reach the encoder
    f32[0, 0] = 448.0
    m = (np.arange(1, W) % 32).astype(np.float32) * q
    f32[0, 1:] = np.where(np.arange(1, W) % 2 == 0, m, -m)
    # row 1: normal-range ties (k + 1/2 mantissa steps) under scale 1
    f32[1, 0] = -448.0
    f32[1, 1:] = (1.0 + (np.arange(1, W) % 16) / 16.0) * np.where(np.arange(1, W) % 3 == 0, -4.0, 0.25)
    f32[2] = 0.0                                           # all zero -> scale 1.0
    f32[3, ::2] = -0.0                                     # signed zeros only
    f32[4] = np.random.default_rng(1).standard_normal(W) * 1e-38   # denormal-range amax
    f32[5] = np.random.default_rng(2).standard_normal(W) * 1e37    # huge
    f32[6] = np.random.default_rng(3).standard_normal(W)
    f32[6, 17] *= 200.0                                    # one outlier crushes the rest
    f32[7, 5] = 3.0                                        # single non-zero
    f32[8] = np.random.default_rng(4).standard_normal(W) * 200.0   # the x200 outlier-token case
    f32[9:16] = np.random.default_rng(5).standard_normal((7, W)) * np.float32(2.0) ** np.arange(-60, 61, 20)[:, None]
    # NaNs do not take part in the row maximum and encode as 0x7f; an infinity makes the scale
    # infinite (finite values -> 0, the infinity itself -> NaN -> 0x7f)
    f32[16:19] = np.random.default_rng(6).standard_normal((3, W))
    f32[16, [3, 200, 575]] = np.nan
    f32[17, 40] = np.inf
    f32[18, 7], f32[18, 300] = -np.inf, np.nan
    return f32_to_bf16_rne(f32)


def test_append_rounding_ties_saturation_and_special_rows(oracle):
    rows = special_rows()
    slots = np.arange(19, dtype=np.int32) * 3
    got, want, bad, _ = paged_append_both(oracle, rows, slots, 1)
    assert bad == 0 and np.array_equal(got, want)
    nan_row = want[16 * 3 * W: (16 * 3 + 1) * W]
    assert (nan_row[[3, 200, 575]] & 0x7F).tolist() == [0x7F] * 3 and (nan_row == 0x7E).any() | (nan_row == 0xFE).any()
    codes0 = want[: W]
    assert {1, 3, 5, 7}.issubset(set(codes0.tolist()))      # half-away results are present
    # anti-vacuity: nearest-even on those ties would have produced a different row
    assert np.count_nonzero(codes0 & 0x7F) > W // 2


def census_rows():
    """Every bf16 amax mantissa (at seven exponents) against every bf16 magnitude in the 18
    binades below it, both signs; the row's first element is the amax."""
    amax_bits, span = [], 18 * 128
    for e in (-118, -60, -9, 0, 8, 61, 120):
        amax_bits += [((e + 127) << 7) | m for m in range(128)]
    per = W - 1
    n_rows_each = -(-(2 * (span + 1)) // per)
    rows = np.zeros((len(amax_bits) * n_rows_each, W), np.uint16)
    for i, ab in enumerate(amax_bits):
        mags = np.arange(max(ab - span, 0), ab + 1, dtype=np.uint16)
        vals = np.concatenate([mags, mags | 0x8000])
        block = np.zeros(n_rows_each * per, np.uint16)
        block[: vals.size] = vals
        rows[i * n_rows_each:(i + 1) * n_rows_each, 0] = ab
        rows[i * n_rows_each:(i + 1) * n_rows_each, 1:] = block.reshape(n_rows_each, per)
    return rows


def test_append_every_amax_mantissa_against_every_value_below_it(oracle):
    """The quotient x / scale depends only on the two mantissas and the exponent gap (powers of
    two are exact), so every bf16 amax mantissa against every bf16 magnitude in the 18 binades
    below it, both signs, is every quotient the quantizer can meet away from the ends of the
    f32 range; a few exponents near those ends cover the rest."""
    rows = census_rows()
    n_pages = -(-rows.shape[0] // PT)
    slots = np.arange(rows.shape[0], dtype=np.int32)
    got, want, bad, _ = paged_append_both(oracle, rows, slots, n_pages)
    assert bad == 0
    mism = np.flatnonzero(got != want)
    assert mism.size == 0, [(int(j), hex(got[j]), hex(want[j])) for j in mism[:8]]
    assert np.unique(want[: PT * W]).size > 200            # nearly every code is produced


def test_append_padding_bad_slots_and_guards(oracle):
    rows = make_rows_bf16(6, W, seed=8)
    slots = np.array([5, -1, 128, 2 ** 31 - 1, 64, -7], np.int32)
    got, want, bad, bad_want = paged_append_both(oracle, rows, slots, 2, fill=0)
    assert bad == bad_want == 2 and np.array_equal(got, want)
    b = dzeros(4096)
    for args, code in (((0, W, PT, 1), 1001), ((1, 0, PT, 1), 1001), ((1, W, PT, 0), 1001),
                       ((1, 2048, PT, 1), 1002), ((1, 570, PT, 1), 1004), ((1, W, 6, 1), 1004)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_kv_append_paged(b, b, b, *args)
        assert e.value.code == code, args
    with pytest.raises(hip.LaunchError) as e:
        hip.launch_kv_append_paged(None, b, b, 1, W, PT, 1)
    assert e.value.code == 1001


def test_append_other_widths(oracle):
    """Non-flagship shapes: width 512 (one step per lane), 128, 1024; page of 16 tokens."""
    for width, pt in ((512, 64), (128, 16), (1024, 32), (64, 4)):
        n, n_pages = 100, 8 * 64 // pt
        rows = make_rows_bf16(n, width, seed=width)
        slots = np.random.default_rng(width).permutation(n_pages * pt)[:n].astype(np.int32)
        pb = oracle.kv_page_bytes(pt, width)
        want = np.zeros(n_pages * pb, np.uint8)
        oracle.kv_append_paged(rows, slots, want, width, pt, n_pages)
        pool = dzeros(n_pages * pb)
        hip.launch_kv_append_paged(dev(rows), dev(slots), pool, n, width, pt, n_pages)
        assert np.array_equal(back(pool), want), (width, pt)


def test_large_batch_kernel_on_the_census_and_the_special_rows(oracle):
    """Large batches (20 480 tokens and more at this width) take the eight-rows-per-wave kernel, which has its own
    row maxima (packed 16-bit integer maxima, float maxima when a row holds a NaN) and its own
    per-row record: the same census and special rows, interleaved so that NaN rows share a wave
    with ordinary ones, repeated up to 40 000 tokens into shuffled slots."""
    base = np.concatenate([special_rows(), census_rows()])
    base = base[np.random.default_rng(11).permutation(base.shape[0])]
    rows = np.concatenate([base] * (-(-40000 // base.shape[0])))[:40000]
    n_pages = -(-rows.shape[0] // PT) + 3
    slots = np.random.default_rng(12).permutation(n_pages * PT)[:rows.shape[0]].astype(np.int32)
    page_bytes = oracle.kv_page_bytes(PT, W)
    want = np.full(n_pages * page_bytes, 0xA5, np.uint8)
    assert oracle.kv_append_paged(rows, slots, want, W, PT, n_pages, n_threads=8) == 0
    pool, bad = dzeros(n_pages * page_bytes, 0xA5), dzeros(4)
    hip.launch_kv_append_paged(dev(rows), dev(slots), pool, slots.size, W, PT, n_pages, bad)
    got = back(pool)
    mism = np.flatnonzero(got != want)
    assert int(back(bad, np.uint32)[0]) == 0 and mism.size == 0, [(int(j), hex(got[j]), hex(want[j])) for j in mism[:8]]


def test_each_batch_size_class_on_the_census_and_the_special_rows(oracle):
    """kv_append_paged picks its kernel by the batch's size: a wave per token below 512 tokens,
    576 threads per 8 tokens from 512 up to the large-batch kernel's 20 480. The census and the
    special rows, shuffled, go through the first in batches of 500 and through the second in
    batches of 4 001 (not a multiple of eight) with padding tokens in between; the pool must
    equal the oracle's after every batch."""
    base = np.concatenate([special_rows(), census_rows()])
    base = np.concatenate([base, base])[np.random.default_rng(21).permutation(2 * base.shape[0])]
    n_pages = -(-base.shape[0] // PT) + 2
    page_bytes = oracle.kv_page_bytes(PT, W)
    for batch in (500, 4001, 9000, 13001):      # (the second kernel in its three shapes)
        slots = np.random.default_rng(batch).permutation(n_pages * PT)[: base.shape[0]].astype(np.int32)
        slots[::131] = -1
        want = np.full(n_pages * page_bytes, 0xA5, np.uint8)
        pool, bad = dzeros(n_pages * page_bytes, 0xA5), dzeros(4)
        rows_d, slots_d = dev(base), dev(slots)
        for at in range(0, base.shape[0], batch):
            n = min(batch, base.shape[0] - at)
            assert oracle.kv_append_paged(base[at: at + n], slots[at: at + n], want, W, PT, n_pages) == 0
            hip.launch_kv_append_paged(rows_d[at * W * 2:], slots_d[at * 4:], pool, n, W, PT, n_pages, bad)
        got = back(pool)
        mism = np.flatnonzero(got != want)
        assert int(back(bad, np.uint32)[0]) == 0 and mism.size == 0, \
            (batch, [(int(j), hex(got[j]), hex(want[j])) for j in mism[:8]])


def test_large_batch_kernel_other_widths(oracle):
    """The eight-rows-per-wave kernel's generic-width form, with padding tokens and a batch that
    is not a multiple of eight."""
    for width, pt in ((512, 64), (128, 16), (1024, 32), (64, 4), (592, 64)):
        n = 33001
        n_pages = -(-n // pt) + 2
        rows = make_rows_bf16(n, width, seed=width + 1, outlier_frac=0.01, outlier_mul=200.0)
        slots = np.random.default_rng(width).permutation(n_pages * pt)[:n].astype(np.int32)
        slots[::97] = -1                                   # padding tokens
        pb = oracle.kv_page_bytes(pt, width)
        want = np.full(n_pages * pb, 0x5A, np.uint8)
        oracle.kv_append_paged(rows, slots, want, width, pt, n_pages, n_threads=8)
        pool = dzeros(n_pages * pb, 0x5A)
        hip.launch_kv_append_paged(dev(rows), dev(slots), pool, n, width, pt, n_pages)
        assert np.array_equal(back(pool), want), (width, pt)
