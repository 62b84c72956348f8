"""The index-list attention on the device against the CPU oracle. Floating point with reductions
in a different order, so not bit-exact: the bar is the reference's own for this kernel, 1/128 of
the largest expected element (crates/engine/tests/kernel_v4_attend.rs:97-106, ATTEND_TOL); the
observed error on cache-like inputs is held to a far smaller figure beside it."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.v4_cases import attend_inputs, sparse_attn_f64

pytestmark = pytest.mark.gpu
ATTEND_TOL = 1.0 / 128.0


def device_attend(q, kv, sink, idx, scale, launch=None, **kw):
    m, h, d = q.shape
    out = dzeros(m * h * d * 4 + 64, 0xEE)
    bufs = [dev(a) for a in (q, kv, sink, idx)]
    if launch is None:
        hip.launch_gather_attn_shared_kv(*bufs, m, h, d, idx.shape[1], scale, out, **kw)
    else:
        assert launch(*(b.data_ptr() for b in bufs), m, h, d, idx.shape[1], scale, out.data_ptr(), None) == 0
    raw = back(out, np.float32)
    assert (raw[m * h * d:].view(np.uint32) == 0xEEEEEEEE).all()
    return raw[:m * h * d].reshape(m, h, d)


def worst_rel(got, want):
    """The reference's metric: the largest difference over the largest expected magnitude."""
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


def random_lists(rng, m, topk, rows, masked=0.2):
    idx = rng.integers(0, rows, (m, topk)).astype(np.int32)
    idx[rng.random((m, topk)) < masked] = -1
    idx[:, topk // 2] = rng.integers(0, rows, m)            # every query keeps a live slot
    return idx


@pytest.mark.parametrize("m,h,topk,rows,cache_like,precise", [
    (3, 64, 640, 900, True, 2), (5, 64, 128, 200, True, 0), (4, 64, 70, 100, False, 2), (2, 64, 33, 64, False, 1),
    (2, 8, 40, 64, True, 2), (2, 100, 96, 128, True, 2), (1, 64, 1, 8, True, 2), (3, 128, 200, 300, True, 0), (3, 128, 200, 300, False, 1)])
def test_matrix_core_kernel_matches_oracle(oracle, m, h, topk, rows, cache_like, precise):
    d = 512
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=m * 1000 + topk, cache_like=cache_like)
    idx = random_lists(np.random.default_rng(topk), m, topk, rows)
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    got = device_attend(q, kv, sink, idx, d ** -0.5, precise=precise)
    err = worst_rel(got, want)
    assert err <= ATTEND_TOL, err
    assert not (got.view(np.uint32) & 0xFFFF).any()          # bf16 values
    if cache_like:
        # against float64 on the same inputs: one bf16 rounding of the result plus little else
        exact = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
        assert np.all(np.abs(got - exact) <= 2.0 ** -8 * np.abs(exact) + 2.0 ** -10 * np.abs(exact).max()), \
            float(np.max(np.abs(got - exact)))


def test_queries_with_and_without_a_bf16_remainder_in_one_call(oracle):
    """A wave whose 16 heads x 256 dims of q are bf16 values leaves the remainder's products out;
    its partner on the other half of the dims, or its neighbour on other heads, may not. Heads 5
    and 40 get a remainder on dims 0..255 only, head 20 on all dims, query 1 on every head."""
    d, m, h, topk, rows = 512, 3, 64, 200, 300
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=77, cache_like=True)
    rng = np.random.default_rng(7)
    noise = (rng.standard_normal(q.shape) * 2.0 ** -12).astype(np.float32)
    q = q.copy()
    q[0, 5, :256] += noise[0, 5, :256]
    q[0, 40, :256] += noise[0, 40, :256]
    q[0, 20] += noise[0, 20]
    q[1] += noise[1]
    idx = random_lists(rng, m, topk, rows)
    exact = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
    got = device_attend(q, kv, sink, idx, d ** -0.5, precise=2)
    assert worst_rel(got, oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)) <= ATTEND_TOL
    assert np.all(np.abs(got - exact) <= 2.0 ** -8 * np.abs(exact) + 2.0 ** -10 * np.abs(exact).max()), \
        float(np.max(np.abs(got - exact)))


def test_peaked_and_flat_softmax(oracle):
    """Logits far apart (one slot holds the whole softmax; the lazily moved maximum must move)
    and logits all equal."""
    d, h, m, rows = 512, 64, 2, 300
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=7, q_scale=12.0)
    idx = random_lists(np.random.default_rng(1), m, 256, rows, masked=0.0)
    idx[0] = np.sort(idx[0])                                  # any order
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    assert worst_rel(device_attend(q, kv, sink, idx, d ** -0.5), want) <= ATTEND_TOL
    q[:] = 0.0                                                # every logit 0: the mean of the rows, less the sink's share
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    assert worst_rel(device_attend(q, kv, sink, idx, d ** -0.5), want) <= ATTEND_TOL / 8


def test_sink_extremes_and_masked_queries(oracle):
    d, h, m, rows = 512, 64, 4, 64
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=9)
    idx = random_lists(np.random.default_rng(2), m, 48, rows)
    idx[1] = -1                                               # query 1 attends to nothing
    idx[2, 1:] = -1                                           # query 2 has exactly one live slot
    idx[2, 0] = 5
    sink[:8] = -np.inf                                        # no leak
    sink[8:16] = 60.0                                         # almost everything leaks
    sink[16:24] = 200.0                                       # the sink's weight overflows: zeros
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    got = device_attend(q, kv, sink, idx, d ** -0.5)
    assert np.isnan(got[1]).all() and np.isnan(want[1]).all()
    live = [0, 2, 3]
    assert np.isfinite(got[live]).all()
    assert worst_rel(got[live], want[live]) <= ATTEND_TOL
    assert np.allclose(got[live][:, 8:16], want[live][:, 8:16], rtol=2 ** -7, atol=1e-30)   # tiny values keep their ratio
    assert (got[live][:, 16:24] == 0).all()


def test_masked_slots_are_never_read_and_bounds_hold(oracle):
    """A -1 slot and (bounded form) an index past the buffer contribute nothing: the rows they
    would name hold NaN."""
    d, h, m, rows = 512, 64, 2, 40
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=11)
    kv_nan = np.concatenate([kv, np.full((8, d), np.nan, np.float32)])
    idx = random_lists(np.random.default_rng(3), m, 64, rows)
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    wild = idx.copy()
    wild[idx < 0] = rows + 3                                  # past n_kv: masked by the bounded form
    got = device_attend(q, kv_nan, sink, wild, d ** -0.5, n_kv=rows)
    assert np.isfinite(got).all() and worst_rel(got, want) <= ATTEND_TOL
    small = dict(m=2, h=4, d=48)
    q2, kv2, sink2 = attend_inputs(oracle, 2, 4, 48, rows, seed=12, cache_like=False)
    kv2_nan = np.concatenate([kv2, np.full((8, 48), np.nan, np.float32)])
    idx2 = random_lists(np.random.default_rng(4), 2, 20, rows)
    wild2 = idx2.copy()
    wild2[idx2 < 0] = rows + 1
    got2 = device_attend(q2, kv2_nan, sink2, wild2, 48 ** -0.5, n_kv=rows)
    assert worst_rel(got2, oracle.sparse_attn(q2, kv2, sink2, idx2, 48 ** -0.5)) <= ATTEND_TOL, small


@pytest.mark.parametrize("m,h,d,topk,rows", [(12, 4, 64, 8, 12), (3, 5, 48, 37, 50), (2, 8, 128, 300, 400),
                                             (2, 3, 1024, 20, 30), (2, 2, 130, 9, 16)])
def test_plain_kernel_matches_oracle(oracle, m, h, d, topk, rows):
    """Every width but 512: toy heads, widths that are no multiple of the wave, the launcher's cap."""
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=d + topk, cache_like=False)
    idx = random_lists(np.random.default_rng(d), m, topk, rows)
    idx[0, :] = -1
    idx[0, -1] = 0
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    got = device_attend(q, kv, sink, idx, d ** -0.5)
    assert worst_rel(got, want) <= ATTEND_TOL / 4
    exact = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
    assert np.all(np.abs(got - exact) <= 2.0 ** -8 * np.abs(exact) + 1e-5)


def test_random_shapes(oracle):
    """40 random (queries, heads, width, list length) shapes: both kernels, odd widths, lists
    shorter and longer than a tile, with and without a partial buffer."""
    rng = np.random.default_rng(0xA77)
    for case in range(40):
        wide = rng.random() < 0.4
        d = 512 if wide else int(rng.integers(1, 300))
        h = int(rng.integers(1, 70)) if wide else int(rng.integers(1, 9))
        m, topk, rows = int(rng.integers(1, 5)), int(rng.integers(1, 200)), int(rng.integers(1, 120))
        q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=case, cache_like=wide)
        idx = random_lists(rng, m, topk, rows)
        want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
        partial = None
        if rng.random() < 0.5:
            partial = dzeros(max(hip.gather_attn_scratch_floats(m, h, d, topk), 4) * 4)
        got = device_attend(q, kv, sink, idx, d ** -0.5, partial=partial)
        assert worst_rel(got, want) <= ATTEND_TOL, (case, m, h, d, topk, rows)


def test_window_selection_feeds_the_attention(oracle):
    """The reference's own drive of this kernel (kernel_v4_attend.rs:167-213): a prefill whose
    prompt outruns the window, selection from the engine's rule, rows = the prompt's own kv."""
    win, prompt, h, d = 8, 12, 64, 512
    q, kv, sink = attend_inputs(oracle, prompt, h, d, prompt, seed=21)
    rows, cols = hip.sel_shape(win, 0, 0, prompt, 0)
    d_idx = dzeros(rows * cols * 4)
    hip.launch_sel_gather(win, 0, 0, prompt, 0, d_idx)
    idx = back(d_idx, np.int32).reshape(rows, cols)
    assert (idx < 0).any()
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    out = dzeros(prompt * h * d * 4)
    hip.launch_gather_attn_shared_kv(dev(q), dev(kv), dev(sink), d_idx, prompt, h, d, cols, d ** -0.5, out)
    assert worst_rel(back(out, np.float32).reshape(prompt, h, d), want) <= ATTEND_TOL


def test_reference_kernel_agrees_with_the_oracle(oracle):
    """The reference's own kernel compiled for this GPU, where that build exists: it and the
    oracle follow the same folds, so they agree far inside the bar."""
    ref = need_ref("rivoli_gather_attn_shared_kv")
    for (m, h, d, topk, rows) in ((3, 8, 512, 40, 64), (2, 4, 64, 8, 12)):
        q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=31 + d)
        idx = random_lists(np.random.default_rng(5), m, topk, rows)
        want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
        theirs = device_attend(q, kv, sink, idx, d ** -0.5, launch=ref.rivoli_gather_attn_shared_kv)
        assert worst_rel(theirs, want) <= ATTEND_TOL / 16
        ours = device_attend(q, kv, sink, idx, d ** -0.5)
        assert worst_rel(ours, theirs) <= ATTEND_TOL


@pytest.mark.parametrize("m,h,topk,precise", [(1, 64, 640, 2), (1, 64, 128, 0), (3, 64, 1000, 2), (2, 128, 333, 1),
                                              (1, 8, 64, 2), (40, 64, 640, 2)])
def test_split_plan_matches_oracle_and_the_unsplit_kernel(oracle, m, h, topk, precise):
    """Decode-shaped calls: a query's list shared among workgroups through the caller's partial
    buffer. Same bar against the oracle; against the one-workgroup plan the only difference is
    where the softmax was re-associated."""
    d, rows = 512, 1500
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=m + topk)
    idx = random_lists(np.random.default_rng(topk + 1), m, topk, rows)
    idx[0, : topk // 2] = -1                                   # whole shares of query 0 masked
    n = hip.gather_attn_scratch_floats(m, h, d, topk)
    assert (n > 0) == (m * ((h + 63) // 64) < 256 and topk > 96)
    partial = dzeros(max(n, 4) * 4, 0xEE)
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    got = device_attend(q, kv, sink, idx, d ** -0.5, precise=precise, partial=partial)
    assert worst_rel(got, want) <= ATTEND_TOL
    exact = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
    assert np.all(np.abs(got - exact) <= 2.0 ** -8 * np.abs(exact) + 2.0 ** -10 * np.abs(exact).max())
    whole = device_attend(q, kv, sink, idx, d ** -0.5, precise=precise)
    assert worst_rel(got, whole) <= 2.0 ** -7                  # one bf16 code where a rounding flipped
    again = device_attend(q, kv, sink, idx, d ** -0.5, precise=precise, partial=partial)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))      # the plan depends on the shape alone
    if n > 0:
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_gather_attn_shared_kv(dev(q), dev(kv), dev(sink), dev(idx), m, h, d, topk, d ** -0.5,
                                             dzeros(m * h * d * 4), partial=dzeros(0))
        assert e.value.code == 1001


def test_split_plan_with_a_fully_masked_query(oracle):
    d, h, rows, topk = 512, 64, 200, 320
    q, kv, sink = attend_inputs(oracle, 2, h, d, rows, seed=77)
    idx = random_lists(np.random.default_rng(8), 2, topk, rows)
    idx[1] = -1
    partial = dzeros(hip.gather_attn_scratch_floats(2, h, d, topk) * 4)
    got = device_attend(q, kv, sink, idx, d ** -0.5, partial=partial)
    want = oracle.sparse_attn(q, kv, sink, idx, d ** -0.5)
    assert np.isnan(got[1]).all() and worst_rel(got[0], want[0]) <= ATTEND_TOL


def test_plain_kernel_on_request_keeps_f32_rows(oracle):
    """precise = 3: rows that are not bf16 values are not rounded, at width 512 too."""
    d, h, m, rows = 512, 8, 2, 64
    q, kv, sink = attend_inputs(oracle, m, h, d, rows, seed=41, cache_like=False)
    idx = random_lists(np.random.default_rng(6), m, 40, rows)
    got = device_attend(q, kv, sink, idx, d ** -0.5, precise=3)
    exact = sparse_attn_f64(q, kv, sink, idx, d ** -0.5)
    assert np.all(np.abs(got - exact) <= 2.0 ** -8 * np.abs(exact) + 1e-5)


def test_attend_guards():
    b = dzeros(1 << 16)

    def code_of(*args, **kw):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_gather_attn_shared_kv(*args, **kw)
        return e.value.code

    assert code_of(None, b, b, b, 1, 1, 512, 4, 1.0, b) == 1001
    assert code_of(b, b, b, b, 0, 1, 512, 4, 1.0, b) == 1001
    assert code_of(b, b, b, b, 1, 1, 512, 0, 1.0, b) == 1001
    assert code_of(b, b, b, b, 1, 1, 1025, 4, 1.0, b) == 1002
    assert code_of(b, b, b, b, 1, 1, 64, 20000, 1.0, b) == 1006
    assert code_of(b, b, b, b, 1, 1, 64, 4, 1.0, b, n_kv=0) == 1001
