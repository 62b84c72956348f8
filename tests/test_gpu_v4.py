"""The second cache format on the device against the CPU oracle, bit for bit: the block
quantize-dequantize of cache rows and the scored block selection."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.test_oracle_v4 import brute_force_rows, reference_tie_block

pytestmark = pytest.mark.gpu


def same_bits(got: np.ndarray, want: np.ndarray) -> np.ndarray:
    """Positions where two f32 arrays differ, NaN payloads aside."""
    g, w = got.view(np.uint32).ravel(), want.view(np.uint32).ravel()
    both_nan = np.isnan(got.ravel()) & np.isnan(want.ravel())
    return np.flatnonzero((g != w) & ~both_nan)


def device_act_quant(x: np.ndarray, n: int, block: int, inplace: bool = True, launch=None) -> np.ndarray:
    rows, row_stride = x.shape
    src = dev(x)
    dst = src if inplace else dzeros(x.size * 4, 0x5A)
    if launch is None:
        hip.launch_act_quant_f8_prefix(src, dst, rows, row_stride, n, block)
    else:
        assert launch(src.data_ptr(), dst.data_ptr(), rows, row_stride, n, block, None) == 0
    return back(dst, np.float32).reshape(x.shape)


def check_act_quant(oracle, x, n, block, inplace=True, what=""):
    code, want = oracle.act_quant_f8_prefix(x, n, block, inplace=inplace)
    assert code == 0
    got = device_act_quant(x, n, block, inplace)
    bad = same_bits(got, want)
    assert bad.size == 0, (what, [(int(i), x.ravel()[i], got.ravel()[i], want.ravel()[i]) for i in bad[:6]])
    return got


def test_act_quant_reference_tie_fixture(oracle):
    """crates/engine/tests/kernel_v4_quant.rs:283-343: subnormal ties, rounded to even."""
    row = reference_tie_block()[None, :]
    got = check_act_quant(oracle, row, 64, 64, what="tie block")
    assert np.count_nonzero((got != 0) & (np.abs(got) < 0.015625)) >= 8


def test_reference_act_quant_agrees_with_the_oracle(oracle):
    """The reference's own kernel (mla.hip compiled for this GPU): the tie fixture against the
    oracle, 300 cache rows against the oracle and this library."""
    ref = need_ref("rivoli_act_quant_f8_prefix")
    row = reference_tie_block()[None, :]
    theirs = device_act_quant(row, 64, 64, launch=ref.rivoli_act_quant_f8_prefix)
    assert same_bits(theirs, oracle.act_quant_f8_prefix(row, 64, 64)[1]).size == 0
    x = cache_rows(300, seed=64)
    theirs = device_act_quant(x, 448, 64, launch=ref.rivoli_act_quant_f8_prefix)
    assert same_bits(theirs, oracle.act_quant_f8_prefix(x, 448, 64)[1]).size == 0
    assert same_bits(theirs, device_act_quant(x, 448, 64)).size == 0


def cache_rows(rows, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, 512)) * np.exp(rng.uniform(-8, 8, (rows, 1)))).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= np.float32(200.0)               # outliers crush their block
    x[3, 64:128] = 0.0                                               # all zero: the amax floor
    x[4, :64] = np.float32(-0.0)
    x[5, 128:192] = np.float32(1e-5)                                 # below the floor
    x[6, 7] = np.float32(3e38)
    x[7, :64] = rng.standard_normal(64).astype(np.float32) * np.float32(1e-41)   # denormals
    x[8, 100] = np.inf
    x[9, 200] = np.nan
    x[10, 64:128] = np.float32(448.0) * np.float32(2.0) ** rng.integers(-20, 20, 64)
    return x


def test_act_quant_cache_rows_block_64_prefix(oracle):
    """The cache entry's shape: 448 of 512 dims at block 64, in place, tail untouched."""
    x = cache_rows(3001, seed=64)
    got = check_act_quant(oracle, x, 448, 64, what="kv rows")
    assert np.array_equal(got[:, 448:].view(np.uint32), x[:, 448:].view(np.uint32))


def test_act_quant_block_128_into_a_second_buffer(oracle):
    """The quantized Linear's shape: whole rows at block 128, source kept."""
    x = cache_rows(777, seed=128)
    check_act_quant(oracle, x, 512, 128, inplace=False, what="block 128")


def test_act_quant_every_rounding_class(oracle):
    """Every sign, exponent and top-8 mantissa bits, with the low bits at zero, one, just under
    the half, the half, just over it and all ones: every rounding decision the encoder can
    take at any exponent, under a block scale pinned to 1 by a 448."""
    hi = np.arange(1 << 17, dtype=np.uint32) << 15
    low = np.array([0, 1, 0x3FFF, 0x4000, 0x4001, 0x7FFF], np.uint32)
    probes = (hi[:, None] | low[None, :]).ravel().view(np.float32)
    pad = (-probes.size) % 63
    probes = np.concatenate([probes, np.zeros(pad, np.float32)]).reshape(-1, 63)
    x = np.concatenate([np.full((probes.shape[0], 1), 448.0, np.float32), probes], axis=1)
    check_act_quant(oracle, x, 64, 64, what="rounding classes")


@pytest.mark.parametrize("block,n,stride", [(16, 64, 64), (32, 96, 128), (256, 512, 512), (24, 48, 50),
                                            (7, 21, 21), (64, 64, 66), (4, 8, 8)])
def test_act_quant_other_blocks_and_the_unaligned_path(oracle, block, n, stride):
    rng = np.random.default_rng(block)
    x = (rng.standard_normal((130, stride)) * np.exp(rng.uniform(-3, 3, (130, 1)))).astype(np.float32)
    check_act_quant(oracle, x, n, block, what=f"block {block}")
    if n == stride:
        check_act_quant(oracle, x, n, block, inplace=False, what=f"block {block} copy")


def test_act_quant_guards():
    b = dzeros(4096)
    other = dzeros(4096)
    for args, code in (((b, b, 0, 64, 64, 64), 1001), ((b, b, 1, 64, 0, 64), 1001),
                       ((b, b, 1, 64, 64, 0), 1001), ((b, b, 1, 32, 64, 64), 1001),
                       ((b, other, 1, 128, 64, 64), 1002), ((b, b, 1, 128, 100, 64), 1004),
                       ((None, b, 1, 64, 64, 64), 1001), ((b, None, 1, 64, 64, 64), 1001)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_act_quant_f8_prefix(*args)
        assert e.value.code == code, args


# ---- scored block selection -------------------------------------------------------------------

def device_select(scores, ratio, index_topk, prefill, offset):
    rows, n_comp = scores.shape
    k = min(index_topk, n_comp)
    out = dzeros(rows * k * 4, 0xEE)
    hip.launch_index_select_blocks(dev(scores), rows, n_comp, ratio, index_topk, prefill, offset, out)
    return back(out, np.int32).reshape(rows, k)


def test_select_reference_cases(oracle):
    """crates/engine/src/v4/select.rs:645-747."""
    inc = np.arange(5, dtype=np.float32)[None, :]
    assert device_select(inc, 4, 512, False, 128).tolist() == [[128, 129, 130, 131, 132]]
    pre = np.arange(36, dtype=np.float32).reshape(12, 3)
    got = device_select(pre, 4, 512, True, 12)
    for t in range(12):
        live = (t + 1) // 4
        assert got[t].tolist() == [12 + c for c in range(live)] + [-1] * (3 - live)
    s = np.array([[1.0, 1.0, 9.0, 0.5, 1.0]], np.float32)
    assert device_select(s, 4, 3, False, 100).tolist() == [[100, 101, 102]]
    s[0, 4] = 2.0
    assert device_select(s, 4, 3, False, 100).tolist() == [[100, 102, 104]]
    s = np.tile(np.array([0.1, 9.0], np.float32), (8, 1))
    assert device_select(s, 4, 1, True, 10).ravel().tolist() == [-1, -1, -1, 10, 10, 10, 10, 11]
    z = np.array([[-0.0, 0.0, -0.0]], np.float32)                    # total order: +0 above -0
    assert device_select(z, 4, 1, False, 0).tolist() == [[1]]


def adversarial_scores(rows, n_comp, seed):
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((rows, n_comp)).astype(np.float32)
    s[rng.random(s.shape) < 0.3] = np.float32(0.5)
    flat = s.ravel()
    flat[::7] = np.float32(-0.0)
    flat[3::11] = np.float32(0.0)
    flat[5::13] = -np.inf
    flat[1::29] = np.inf
    flat[2::31] = np.nan                                             # ordered above +inf
    flat[4::37] = np.float32(-np.nan)                                # and below -inf
    return s


@pytest.mark.parametrize("rows,n_comp,ratio,topk,prefill", [
    (1, 300, 4, 64, False), (40, 9, 4, 3, True), (130, 2, 128, 1, True), (3, 50, 4, 50, False),
    (700, 160, 4, 40, True),                                          # prefill rows of growing limit
    (1, 16384, 4, 2048, False),                                       # a 64K context at ratio 4
    (5, 3000, 4, 512, False), (2, 70000, 4, 2048, False), (1, 1025, 4, 1024, False),
    # one case per remaining dispatch width: 4 waves, 16 waves, the 64-keys-per-thread select
    (2, 6000, 4, 512, False), (2, 20000, 4, 2048, False), (2, 50000, 4, 700, False), (3, 8192, 4, 8000, False)])
def test_select_matches_oracle(oracle, rows, n_comp, ratio, topk, prefill):
    s = adversarial_scores(rows, n_comp, seed=rows * 131 + n_comp)
    want = oracle.v4_scored_rows(s, ratio, topk, prefill, 4096)
    got = device_select(s, ratio, topk, prefill, 4096)
    assert np.array_equal(got, want), np.argwhere(got != want)[:5]
    if rows * n_comp <= 40000:
        assert np.array_equal(want, brute_force_rows(s, ratio, topk, prefill, 4096))


def test_select_prefill_at_scale(oracle):
    """A 8192-token prefill at ratio 4 with a cap of 512: rows below the cap are positional,
    rows above it ranked; every row is ascending, legal, and -1 padded only at its tail."""
    rows, ratio, topk = 8192, 4, 512
    n_comp = rows // ratio
    s = adversarial_scores(rows, n_comp, seed=8192)
    got = device_select(s, ratio, topk, True, 128)
    assert np.array_equal(got, oracle.v4_scored_rows(s, ratio, topk, True, 128))
    limit = np.minimum((np.arange(rows) + 1) // ratio, n_comp)
    kept = (got >= 0).sum(axis=1)
    assert np.array_equal(kept, np.minimum(limit, topk))
    for t in (3, 100, 2047, 2051, 8191):
        r = got[t, :kept[t]]
        assert np.all(np.diff(r) > 0) and (r.size == 0 or r[-1] < 128 + limit[t])


def test_select_guards():
    b = dzeros(4096)
    for args, code in (((None, 1, 8, 4, 2, 0, 0, b), 1001), ((b, 1, 8, 4, 2, 0, 0, None), 1001),
                       ((b, 0, 8, 4, 2, 0, 0, b), 1001), ((b, 1, 0, 4, 2, 0, 0, b), 1001),
                       ((b, 1, 8, 0, 2, 1, 0, b), 1001), ((b, 1, 8, 4, 0, 0, 0, b), 1001),
                       ((b, 1, 8, 4, 2, 0, -1, b), 1001), ((b, 1, 8, 4, 2, 0, 2 ** 31 - 4, b), 1002)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_index_select_blocks(*args)
        assert e.value.code == code, args
