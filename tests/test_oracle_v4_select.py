"""Pins the oracle's selection rectangles, ring write and index-list attention: the reference's
own unit cases (crates/engine/src/v4/select.rs:514-808) as known answers, a literal per-cell
restatement, and closed forms / float64 arithmetic for the attention."""
import numpy as np
import pytest

from tests.v4_cases import literal_sel_gather, sparse_attn_f64

WIN, TOPK = 8, 512   # select.rs:496-505 (BASE)


def test_multi_row_decode_is_refused(oracle):
    """select.rs:514-529."""
    assert oracle.sel_shape(WIN, 0, TOPK, 3, 5)[0] == 1005
    assert oracle.sel_shape(WIN, 0, TOPK, 3, 0) == (0, 3, 3)
    assert oracle.sel_shape(WIN, 0, TOPK, 1, 5) == (0, 1, 8)
    assert oracle.sel_shape(0, 0, TOPK, 1, 5)[0] == 1001


def test_ring_is_read_oldest_first(oracle):
    """select.rs:533-538: win 4, position 6 -> slot 2 holds position 6, the oldest live slot is 3;
    not yet full: live slots, then padding to the ring's width."""
    assert oracle.sel_gather(4, 0, TOPK, 1, 6)[1].tolist() == [[3, 0, 1, 2]]
    assert oracle.sel_gather(4, 0, TOPK, 1, 2)[1].tolist() == [[0, 1, 2, -1]]
    # position win - 1 fills the ring for the first time
    assert oracle.sel_gather(4, 0, TOPK, 1, 3)[1].tolist() == [[0, 1, 2, 3]]


def test_prefill_blocks_are_causal(oracle):
    """select.rs:542-553: 6 positions, ratio 2 -> 3 blocks; query t reads blocks below (t+1)/2.
    The compressed columns start at offset = seqlen."""
    code, out = oracle.sel_gather(100, 2, TOPK, 6, 0)
    comp = out[:, 6:]
    assert code == 0 and comp.shape == (6, 3)
    assert comp[0].tolist() == [-1, -1, -1] and comp[1].tolist() == [6, -1, -1]
    assert comp[3].tolist() == [6, 7, -1] and comp[5].tolist() == [6, 7, 8]
    # and the window part of a prompt that fits is the causal triangle of absolute positions
    assert out[:, :6].tolist() == [[j if j <= t else -1 for j in range(6)] for t in range(6)]


def test_prefill_window_slides_over_long_prompts(oracle):
    out = oracle.sel_gather(4, 0, TOPK, 7, 0)[1]
    assert out.tolist() == [[0, -1, -1, -1], [0, 1, -1, -1], [0, 1, 2, -1], [0, 1, 2, 3], [1, 2, 3, 4],
                            [2, 3, 4, 5], [3, 4, 5, 6]]


def test_indexed_layer_refuses_past_its_cap(oracle):
    """select.rs:613-641: topk 2 -> limit 12; an unindexed ratio never refuses."""
    assert oracle.sel_shape(WIN, 4, 2, 1, 10)[0] == 0
    assert oracle.sel_shape(WIN, 4, 2, 1, 12)[0] == 1006
    assert oracle.sel_shape(WIN, 2, 2, 1, 48)[0] == 0


@pytest.mark.parametrize("seqlen,start", [(1, 19), (12, 0)])
def test_below_the_cap_scored_equals_positional(oracle, seqlen, start):
    """select.rs:645-677, with its adversarial strictly increasing scores."""
    code, pos = oracle.sel_gather(WIN, 4, TOPK, seqlen, start)
    rows, cols = pos.shape
    n_comp = cols - (min(seqlen, WIN) if start == 0 else WIN)
    scores = np.arange(rows * n_comp, dtype=np.float32).reshape(rows, n_comp)
    code2, scr = oracle.sel_gather_scored(scores, WIN, 4, TOPK, seqlen, start)
    assert code == 0 and code2 == 0 and np.array_equal(pos, scr)


def test_rectangle_shapes(oracle):
    """select.rs:790-808."""
    for ratio, seqlen, start in ((0, 5, 0), (0, 1, 9), (4, 12, 0), (4, 1, 19), (128, 1, 300)):
        code, rows, cols = oracle.sel_shape(WIN, ratio, TOPK, seqlen, start)
        code2, out = oracle.sel_gather(WIN, ratio, TOPK, seqlen, start)
        assert code == 0 and code2 == 0 and out.shape == (rows, cols)
        assert np.array_equal(out, literal_sel_gather(WIN, ratio, seqlen, start)), (ratio, seqlen, start)
        assert (out != -7).all()


def test_gather_matches_literal_restatement(oracle):
    rng = np.random.default_rng(5)
    for _ in range(200):
        win = int(rng.integers(1, 20))
        ratio = int(rng.choice([0, 2, 4, 8, 128]))
        if rng.random() < 0.5:
            seqlen, start = int(rng.integers(1, 70)), 0
        else:
            seqlen, start = 1, int(rng.integers(1, 400))
        code, out = oracle.sel_gather(win, ratio, 10 ** 6, seqlen, start)
        assert code == 0
        assert np.array_equal(out, literal_sel_gather(win, ratio, seqlen, start)), (win, ratio, seqlen, start)


def test_scored_gather_above_the_cap(oracle):
    """select.rs:681-710 through the assembled rectangle: offset is the window at decode."""
    scores = np.array([[1.0, 1.0, 9.0, 0.5, 1.0]], np.float32)
    code, out = oracle.sel_gather_scored(scores, 4, 4, 3, 1, 19)
    assert code == 0 and out.tolist() == [[0, 1, 2, 3, 4 + 0, 4 + 1, 4 + 2]]
    scores[0, 4] = 2.0
    assert oracle.sel_gather_scored(scores, 4, 4, 3, 1, 19)[1][0, 4:].tolist() == [4, 6, 8]
    assert oracle.sel_gather_scored(scores, 4, 0, 3, 1, 19)[0] == 1001     # no compressor, nothing to rank
    assert oracle.sel_gather_scored(np.zeros((2, 5), np.float32), 4, 4, 3, 2, 19)[0] == 1005


@pytest.mark.parametrize("win,hd,seqlen,start", [(8, 6, 1, 5), (8, 6, 1, 21), (8, 6, 5, 0), (8, 6, 8, 0),
                                                  (8, 6, 19, 0), (8, 6, 16, 0), (128, 512, 300, 0)])
def test_ring_write_puts_position_t_in_slot_t_mod_win(oracle, win, hd, seqlen, start):
    """crates/engine/src/v4/attn.rs:343-378."""
    rng = np.random.default_rng(seqlen * 7 + start)
    kv = rng.standard_normal((seqlen, hd)).astype(np.float32)
    cache = np.full((win, hd), 123.0, np.float32)
    assert oracle.ring_write(kv, cache, win, seqlen, start) == 0
    if start:
        live = {start % win: kv[0]}
    else:
        live = {t % win: kv[t] for t in range(max(0, seqlen - win), seqlen)}
    for slot in range(win):
        want = live.get(slot, np.full(hd, 123.0, np.float32))
        assert np.array_equal(cache[slot], want), slot
    assert oracle.ring_write(kv, cache, win, 2, 3) == 1005


def test_compress_dst_reference_cases(oracle):
    """select.rs:556-611: cache space starts at the window, selection space past the prompt; the
    decode bases coincide; the decode row is a function of the position (3, 7 for positions 15
    and 31), not a count of blocks emitted (0, 1)."""
    from rivoli_amd import hip

    for dst, off in ((oracle.compress_dst, hip.compress_offset), (hip.compress_dst, hip.compress_offset)):
        win, prompt = 128, 16
        assert dst(4, win, prompt, 0) == (win, 4)
        assert dst(4, off(win, prompt, 0), prompt, 0) == (prompt, 4)
        assert dst(4, win, 1, 47) == (win + 11, 1) and dst(4, off(win, 1, 47), 1, 47) == (win + 11, 1)
        assert [dst(4, 0, 1, pos)[0] for pos in (15, 31)] == [3, 7]
        assert dst(4, 0, 1, 16) is None and dst(4, 0, 3, 0) is None and dst(0, 0, 50, 0) is None
        assert dst(128, 128, 1, 127) == (128, 1) and dst(128, 128, 1, 128) is None


def test_sparse_attn_closed_forms(oracle):
    rng = np.random.default_rng(3)
    h, d = 3, 16
    kv = rng.standard_normal((9, d)).astype(np.float32)
    q = rng.standard_normal((2, h, d)).astype(np.float32)
    sink = np.array([0.3, -1.0, 2.0], np.float32)
    scale = d ** -0.5
    # one live slot: the row over 1 + exp(sink - logit)
    idx = np.array([[-1, 4, -1], [7, -1, -1]], np.int32)
    o = oracle.sparse_attn(q, kv, sink, idx, scale)
    for t, row in ((0, 4), (1, 7)):
        for hh in range(h):
            logit = float(np.dot(q[t, hh].astype(np.float64), kv[row].astype(np.float64))) * scale
            want = kv[row].astype(np.float64) / (1.0 + np.exp(float(sink[hh]) - logit))
            assert np.allclose(o[t, hh], want, rtol=2 ** -8, atol=1e-7)
    # the same row in every slot: that row times the softmax mass outside the sink
    idx = np.full((2, 5), 2, np.int32)
    o = oracle.sparse_attn(q, kv, sink, idx, scale)
    for t in range(2):
        for hh in range(h):
            logit = float(np.dot(q[t, hh].astype(np.float64), kv[2].astype(np.float64))) * scale
            want = kv[2].astype(np.float64) * 5.0 / (5.0 + np.exp(float(sink[hh]) - logit))
            assert np.allclose(o[t, hh], want, rtol=2 ** -8, atol=1e-7)
    # outputs are bf16 values
    assert not (o.view(np.uint32) & 0xFFFF).any()
    # a fully masked query is NaN, the other query is not touched by it
    idx = np.array([[-1, -1], [1, 3]], np.int32)
    o = oracle.sparse_attn(q, kv, sink, idx, scale)
    assert np.isnan(o[0]).all() and np.isfinite(o[1]).all()
    # sink = -inf is the plain softmax average; masked slots are never dereferenced (index -1
    # would read before the buffer)
    o = oracle.sparse_attn(q, kv, np.full(h, -np.inf, np.float32), np.array([[0, -1, 8], [8, 0, -1]], np.int32), scale)
    assert np.array_equal(o[0], o[0]) and np.allclose(o, sparse_attn_f64(q, kv, np.full(h, -np.inf), np.array([[0, -1, 8], [8, 0, -1]]), scale), rtol=2 ** -7, atol=1e-6)


@pytest.mark.parametrize("m,h,d,topk,rows", [(5, 4, 32, 12, 40), (3, 8, 128, 70, 50), (2, 64, 512, 40, 64)])
def test_sparse_attn_matches_float64(oracle, m, h, d, topk, rows):
    rng = np.random.default_rng(m * 100 + d)
    kv = rng.standard_normal((rows, d)).astype(np.float32)
    q = (rng.standard_normal((m, h, d)) * 2).astype(np.float32)
    sink = rng.standard_normal(h).astype(np.float32)
    idx = rng.integers(-1, rows, (m, topk)).astype(np.int32)
    idx[:, 0] = 1                                           # at least one live slot
    got = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    want = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
    # half a bf16 ulp of the element plus the f32 fold's error
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-5)
    # the softmax is over a set: permuting a query's slots moves nothing beyond f32 rounding
    perm = rng.permutation(topk)
    again = oracle.sparse_attn(q, kv, sink, idx[:, perm], d ** -0.5)
    assert np.all(np.abs(got - again) <= 2.0 ** -7 * np.abs(want) + 1e-5)
