"""The second cache format's block indexer on the device against the CPU oracle and against
the reference's own kernels, bit for bit: the Hadamard + fp4 spread and the block scorer."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.test_gpu_v4 import same_bits
from tests.test_oracle_v4_blockindex import bf16_round

pytestmark = pytest.mark.gpu


def device_spread(x: np.ndarray, launch=None) -> np.ndarray:
    rows, d = x.shape
    buf = dev(x)
    if launch is None:
        hip.launch_act_quant_f4_rotated(buf, rows, d)
    else:
        assert launch(buf.data_ptr(), rows, d, None) == 0
    return back(buf, np.float32).reshape(x.shape)


def spread_rows(rows, d, seed):
    """bf16-valued rows (the reference's input dtype) over a wide range of magnitudes, with the
    special blocks: all zero, negative zero, below the amax floor, one outlier per block."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, d)) * np.exp(rng.uniform(-6, 6, (rows, 1)))).astype(np.float32)
    if rows > 8:
        x[1] = 0.0
        x[2] = np.float32(-0.0)
        x[3] = np.float32(1e-38)
        x[4, ::32] *= np.float32(300.0)
        x[5] = np.float32(3.0)         # a constant row: one spike after the rotation
        x[6] = rng.standard_normal(d).astype(np.float32) * np.float32(1e-40)   # denormals: below the amax floor
        x[7] = rng.standard_normal(d).astype(np.float32) * np.float32(1e30)    # sums stay finite
    return bf16_round(x)


@pytest.mark.parametrize("rows,d", [(1, 128), (9, 128), (60, 128), (1000, 128), (7, 32), (33, 64), (129, 256),
                                    (4097, 128)])
def test_spread_matches_the_oracle(oracle, rows, d):
    x = spread_rows(rows, d, rows * 1000 + d)
    code, want = oracle.act_quant_f4_rotated(x)
    assert code == 0
    got = device_spread(x)
    bad = same_bits(got, want)
    assert bad.size == 0, [(int(i) // d, int(i) % d, got.ravel()[i], want.ravel()[i]) for i in bad[:6]]


def sixty_binades():
    rng = np.random.default_rng(60)
    base = bf16_round(rng.standard_normal((60, 128)).astype(np.float32))
    return bf16_round(base * (2.0 ** (np.arange(60) - 30))[:, None].astype(np.float32))


def test_spread_over_sixty_binades(oracle):
    """crates/engine/tests/kernel_v4_indexer.rs:246-277: row r scaled into binade r - 30, so the
    block scale lands on 60 powers of two."""
    x = sixty_binades()
    code, want = oracle.act_quant_f4_rotated(x)
    assert same_bits(device_spread(x), want).size == 0
    scales = {float(np.abs(r[r != 0]).min()) for r in want if (r != 0).any()}
    assert len(scales) >= 55


def test_reference_spread_agrees_with_the_oracle_and_this_library(oracle):
    """The reference's own kernel (blockindex.hip compiled for this GPU): the sixty binades
    against the oracle, other widths against this library."""
    ref = need_ref("rivoli_act_quant_f4_rotated")
    x = sixty_binades()
    want = oracle.act_quant_f4_rotated(x)[1]
    assert same_bits(device_spread(x, launch=ref.rivoli_act_quant_f4_rotated), want).size == 0
    for rows, d in ((333, 256), (77, 128), (19, 64), (11, 32)):
        wide = spread_rows(rows, d, 5)
        assert same_bits(device_spread(wide, launch=ref.rivoli_act_quant_f4_rotated),
                         device_spread(wide)).size == 0, (rows, d)


def test_spread_guards():
    """blockindex.hip:241-257; kernel_v4_indexer.rs:287-320."""
    buf = dzeros(512 * 4)
    lib = hip.lib()
    call = lambda rows, d: lib.rivoli_act_quant_f4_rotated(buf.data_ptr(), rows, d, None)
    assert call(1, 128) == 0
    assert call(0, 128) == 1001 and call(1, 0) == 1001
    assert call(1, 512) == 1002
    assert call(1, 96) == 1003
    assert call(1, 16) == 1004
    assert lib.rivoli_act_quant_f4_rotated(None, 1, 128, None) == 1001
    assert lib.rivoli_act_quant_f4_rotated(buf.data_ptr() + 4, 1, 128, None) == 1004


# ---- the block scorer -------------------------------------------------------------------------

def device_score(q, kv, w, launch=None) -> np.ndarray:
    s, heads, hd = q.shape
    n_comp = kv.shape[0]
    qd, kd, wd = dev(q), dev(kv), dev(w)
    out = dzeros(s * n_comp * 4, 0x5A)
    if launch is None:
        hip.launch_index_score_blocks(qd, kd, wd, out, s, n_comp, heads, hd)
    else:
        assert launch(qd.data_ptr(), kd.data_ptr(), wd.data_ptr(), out.data_ptr(), s, n_comp, heads, hd, None) == 0
    return back(out, np.float32).reshape(s, n_comp)


def score_case(s, n_comp, heads, hd, seed, spread=None):
    """Arbitrary f32 operands make every addition round, so a reordered or fused dot shows;
    spread operands (oracle-made) are what the engine feeds."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((s, heads, hd)).astype(np.float32)
    kv = rng.standard_normal((n_comp, hd)).astype(np.float32)
    if spread is not None:
        q = spread.act_quant_f4_rotated(bf16_round(q).reshape(-1, hd))[1].reshape(s, heads, hd)
        kv = spread.act_quant_f4_rotated(bf16_round(kv))[1]
    w = bf16_round((rng.standard_normal((s, heads)) * hd ** -0.5).astype(np.float32))  # signed
    return q, kv, w


@pytest.mark.parametrize("s,n_comp,heads,hd,spread", [
    (1, 1, 64, 128, False), (2, 300, 64, 128, False), (33, 70, 8, 128, True), (5, 513, 64, 128, True),
    (3, 5, 4, 32, False), (2, 130, 3, 64, True), (1, 257, 2, 256, False), (40, 64, 64, 128, False),
    (1, 200, 128, 128, False), (1, 70, 130, 128, False), (2, 65, 5, 128, True), (300, 520, 3, 128, False),
])
def test_score_matches_the_oracle(oracle, s, n_comp, heads, hd, spread):
    q, kv, w = score_case(s, n_comp, heads, hd, s * 31 + n_comp, oracle if spread else None)
    code, want = oracle.index_score_blocks(q, kv, w)
    assert code == 0
    got = device_score(q, kv, w)
    bad = same_bits(got, want)
    assert bad.size == 0, [(int(i) // n_comp, int(i) % n_comp, got.ravel()[i], want.ravel()[i]) for i in bad[:6]]
    assert np.count_nonzero(want) > 0 or n_comp * s < 4


def test_score_known_answer(oracle):
    """kernel_v4_indexer.rs:689-726 (f32 accumulation, one bf16 round: 1.125, not 1.0)."""
    heads, hd = 64, 128
    kv = np.zeros((1, hd), np.float32)
    kv[0, 0] = 1.0
    q = np.zeros((1, heads, hd), np.float32)
    q[0, :, 0] = 2.0 ** -9
    q[0, 0, 0] = 1.0
    got = device_score(q, kv, np.ones((1, heads), np.float32))
    assert got[0, 0] == np.float32(1.125)


def test_reference_scorer_agrees_with_the_oracle_and_this_library(oracle):
    """The reference's own kernel (blockindex.hip compiled for this GPU) on rounding-sensitive
    operands."""
    ref = need_ref("rivoli_index_score_blocks")
    for shape in [(4, 200, 64, 128), (3, 77, 5, 64)]:
        q, kv, w = score_case(*shape, seed=9)
        theirs = device_score(q, kv, w, launch=ref.rivoli_index_score_blocks)
        assert same_bits(theirs, oracle.index_score_blocks(q, kv, w)[1]).size == 0
        assert same_bits(theirs, device_score(q, kv, w)).size == 0


def test_score_guards():
    """blockindex.hip:264-275."""
    buf = dzeros(4096)
    p = buf.data_ptr()
    lib = hip.lib()
    assert lib.rivoli_index_score_blocks(p, p, p, p, 1, 1, 1, 8, None) == 0
    assert lib.rivoli_index_score_blocks(p, p, p, p, 0, 1, 1, 8, None) == 1001
    assert lib.rivoli_index_score_blocks(p, p, p, p, 1, 1, 0, 8, None) == 1001
    assert lib.rivoli_index_score_blocks(p, p, p, p, 1, 1, 1, 0, None) == 1001
    assert lib.rivoli_index_score_blocks(p, p, p, p, 1, 0, 1, 8, None) == 1005
    assert lib.rivoli_index_score_blocks(None, p, p, p, 1, 1, 1, 8, None) == 1001


def test_prefill_sized_scores_on_sampled_rows_and_the_selection_they_feed(oracle):
    """A prefill chunk's worth (256 queries x 2048 blocks x 64 heads x 128): the oracle checks
    sampled query rows; then the chain the engine runs (crates/engine/src/v4/blocksel.rs:218-248
    followed by select.rs:153-188) — spread q, score, select — against the oracle's chain."""
    s, n_comp, heads, hd, k = 256, 2048, 64, 128, 512
    rng = np.random.default_rng(2048)
    q_raw = bf16_round(rng.standard_normal((s * heads, hd)).astype(np.float32))
    kv = oracle.act_quant_f4_rotated(bf16_round(rng.standard_normal((n_comp, hd)).astype(np.float32)))[1]
    w = bf16_round((rng.standard_normal((s, heads)) * hd ** -0.5).astype(np.float32))
    qd, kd, wd = dev(q_raw), dev(kv), dev(w)
    hip.launch_act_quant_f4_rotated(qd, s * heads, hd)
    score = dzeros(s * n_comp * 4, 0x5A)
    hip.launch_index_score_blocks(qd, kd, wd, score, s, n_comp, heads, hd)
    got = back(score, np.float32).reshape(s, n_comp)
    q = back(qd, np.float32).reshape(s, heads, hd)
    for t in (0, 1, 100, 255):
        want_q = oracle.act_quant_f4_rotated(q_raw.reshape(s, heads, hd)[t])[1]
        assert same_bits(q[t], want_q).size == 0
        code, want = oracle.index_score_blocks(want_q[None], kv, w[t:t + 1])
        assert same_bits(got[t:t + 1], want).size == 0, t
    sel = dzeros(s * k * 4)
    hip.launch_index_select_blocks(score, s, n_comp, 4, k, False, 0, sel)   # decode rule: every row ranks all blocks
    got_sel = back(sel, np.int32).reshape(s, k)
    for t in (0, 100, 255):
        want_sel = oracle.v4_scored_rows(got[t:t + 1], 4, k, False, 0)
        np.testing.assert_array_equal(got_sel[t], want_sel[0])


@pytest.mark.parametrize("s,n_comp,heads,hd,ratio", [(700, 175, 4, 128, 4), (300, 300, 2, 128, 1), (520, 130, 3, 64, 4),
                                                     (64, 16, 8, 128, 4), (1030, 100, 2, 128, 4)])
def test_prefill_form_writes_every_legal_entry_and_skips_whole_groups(oracle, s, n_comp, heads, hd, ratio):
    """score[t][c] for c < (t + 1) / ratio equals the full kernel's bit for bit; a 64-block group
    with no legal block for row t keeps the buffer's fill; the selection built on it is the one
    built on the full matrix."""
    q, kv, w = score_case(s, n_comp, heads, hd, s + ratio)
    full = device_score(q, kv, w)
    qd, kd, wd = dev(q), dev(kv), dev(w)
    out = dzeros(s * n_comp * 4, 0x5A)
    hip.launch_index_score_blocks_prefill(qd, kd, wd, out, s, n_comp, heads, hd, ratio)
    got = back(out, np.float32).reshape(s, n_comp)
    fill = np.frombuffer(b"\x5a" * 4, np.uint32)[0]
    limit = np.minimum((np.arange(s) + 1) // ratio, n_comp)
    cols = np.arange(n_comp)
    legal = cols[None, :] < limit[:, None]
    group_live = (cols[None, :] // 64) * 64 < limit[:, None]
    assert np.array_equal(got.view(np.uint32)[legal], full.view(np.uint32)[legal])
    assert np.array_equal(got.view(np.uint32)[group_live], full.view(np.uint32)[group_live])
    assert (got.view(np.uint32)[~group_live] == fill).all()
    assert (~group_live).any() and legal.any()
    k = min(32, n_comp)
    sel_a, sel_b = dzeros(s * k * 4), dzeros(s * k * 4)
    hip.launch_index_select_blocks(out, s, n_comp, ratio, k, True, 0, sel_a)
    hip.launch_index_select_blocks(dev(full), s, n_comp, ratio, k, True, 0, sel_b)
    assert np.array_equal(back(sel_a, np.int32), back(sel_b, np.int32))
    assert hip.lib().rivoli_index_score_blocks_prefill(qd.data_ptr(), kd.data_ptr(), wd.data_ptr(), out.data_ptr(),
                                                       s, n_comp, heads, hd, 0, None) == 1001
