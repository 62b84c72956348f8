"""The DSA step as one call: selection plus the sparse gather of the selected rows, and the
indexer's score kernel doing the selection's histogram on the way. Bit-exact against the
oracle's top-k followed by its sparse gather (the sparse gather itself is pinned by
gather_rows(rows) == gather_dense()[rows], the reference having no test with rows != null)."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.churn import token_rows
from tests.gpu_util import back, dev, dzeros
from tests.util import shuffled_block_tables

pytestmark = pytest.mark.gpu
SENTINEL = 0xFFFFFFFF
W, PT = 576, 64


def paged_cache(oracle, rng, n_q, nt, width=W, pt=PT, spare=3):
    """A fragmented pool holding nt tokens for each of n_q sequences (host and device copies)."""
    blocks = -(-nt // pt)
    n_pages = n_q * blocks + spare
    tables = shuffled_block_tables(n_q, blocks, n_pages, seed=int(rng.integers(1 << 30)))
    page_bytes = oracle.kv_page_bytes(pt, width)
    pool_h = np.zeros(n_pages * page_bytes, np.uint8)
    pos = np.arange(nt)
    for s in range(n_q):
        rows = token_rows(rng, nt) if width == W else token_rows(rng, nt)[:, :width].copy()
        slots = (tables[s][pos // pt] * pt + pos % pt).astype(np.int32)
        oracle.kv_append_paged(np.ascontiguousarray(rows), slots, pool_h, width, pt, n_pages)
    return tables, n_pages, pool_h


def run_fused(scores, nts, k, tables, n_pages, pool_d, width=W, pt=PT, split=True, hist_ready=False, ws=None):
    n_q, stride = scores.shape
    if ws is None and split:
        ws = dzeros(hip.index_topk_workspace_bytes(n_q, stride))
    rows = dzeros(n_q * k * 4, 0xFF)
    out = dzeros(n_q * k * width * 2, 0xEE)
    bad = dzeros(4)
    hip.launch_dsa_select_gather_paged(dev(scores), n_q, stride, None if nts is None else dev(np.asarray(nts, np.int32)),
                                       stride, k, rows, ws, hist_ready, pool_d, dev(tables), out, tables.shape[1],
                                       width, pt, n_pages, bad)
    return (back(rows, np.uint32).reshape(n_q, k), back(out, np.uint16).reshape(n_q, k, width),
            int(back(bad, np.uint32)[0]))


def check_against_oracle(oracle, scores, nts, k, tables, pool_h, got_rows, got_out, width=W, pt=PT):
    n_q = scores.shape[0]
    for q in range(n_q):
        nt_q = scores.shape[1] if nts is None else int(nts[q])
        want = oracle.topk(scores[q, :nt_q], k) if nt_q > 0 else np.zeros(0, np.uint32)
        assert np.array_equal(got_rows[q, : want.size], want), q
        assert np.all(got_rows[q, want.size:] == SENTINEL), q
        if want.size:
            want_out = oracle.kv_gather_rows_paged(pool_h, tables[q: q + 1], want[None, :], width, pt)[0]
            assert np.array_equal(got_out[q, : want.size], want_out), q
        assert np.all(got_out[q, want.size:] == 0xEEEE), q      # nothing written past the selection


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("nt,k", [(20000, 2048), (16385, 100), (65536, 2048), (70000, 129), (3000, 256)])
def test_select_gather_matches_topk_then_sparse_gather(oracle, nt, k, split):
    rng = np.random.default_rng(nt + k)
    n_q = 3
    tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
    s = rng.standard_normal((n_q, nt), dtype=np.float32)
    s[:, -64:] += np.float32(4.0)
    s[1, ::3] = np.float32(0.25)                 # tie-heavy: the pivot bin cannot be listed
    s[2, : nt // 2] = np.float32(-5.0)           # every selected token in the second half
    pool_d = dev(pool_h)
    ws = dzeros(hip.index_topk_workspace_bytes(n_q, nt)) if split else None
    for _ in range(2):                           # the second call reuses what the first left in the workspace
        got_rows, got_out, bad = run_fused(s, None, k, tables, n_pages, pool_d, split=split, ws=ws)
        assert bad == 0
        check_against_oracle(oracle, s, None, k, tables, pool_h, got_rows, got_out)


def test_select_gather_ragged_lengths_and_bad_pages(oracle):
    rng = np.random.default_rng(77)
    n_q, stride, k = 5, 40000, 512
    tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, stride)
    nts = np.array([40000, 17000, 0, 300, 39999], np.int32)
    s = rng.standard_normal((n_q, stride), dtype=np.float32)
    got_rows, got_out, bad = run_fused(s, nts, k, tables, n_pages, dev(pool_h))
    assert bad == 0
    check_against_oracle(oracle, s, nts, k, tables, pool_h, got_rows, got_out)
    # page ids outside the pool: their selected rows are skipped and counted, the others are right
    broken = tables.copy()
    broken[0, 5:45] = n_pages + 9
    got_rows, got_out, bad = run_fused(s, nts, k, broken, n_pages, dev(pool_h))
    want = oracle.topk(s[0, : nts[0]], k)
    hit = ((want // PT) >= 5) & ((want // PT) < 45)
    assert bad == int(hit.sum()) and hit.any()
    want_out = oracle.kv_gather_rows_paged(pool_h, tables[:1], want[None, :], W, PT)[0]
    assert np.array_equal(got_out[0, : want.size][~hit], want_out[~hit])
    assert np.all(got_out[0, : want.size][hit] == 0xEEEE)


def test_select_gather_other_page_geometry(oracle):
    rng = np.random.default_rng(5)
    n_q, nt, k, width, pt = 2, 18000, 300, 64, 16
    tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, nt, width, pt)
    s = rng.standard_normal((n_q, nt), dtype=np.float32)
    got_rows, got_out, bad = run_fused(s, None, k, tables, n_pages, dev(pool_h), width, pt)
    assert bad == 0
    check_against_oracle(oracle, s, None, k, tables, pool_h, got_rows, got_out, width, pt)


def test_select_gather_guards(oracle):
    b = dzeros(1 << 20)
    ws = dzeros(hip.index_topk_workspace_bytes(1, 20000))
    def call(**kw):
        a = dict(scores=b, n_queries=1, stride=20000, nts=None, nt=20000, k=8, rows=b, workspace=ws, hist_ready=False,
                 pool=b, block_table=b, out=b, max_blocks_per_seq=400, width=W, page_tokens=PT, n_pages=10)
        a.update(kw)
        hip.launch_dsa_select_gather_paged(**a)
    for kw, code in ((dict(pool=None), 1001), (dict(out=None), 1001), (dict(k=0), 1001), (dict(stride=100), 1002),
                     (dict(width=100), 1004), (dict(nt=3000, stride=3000, hist_ready=True), 1001),
                     (dict(workspace=None, hist_ready=True), 1001), (dict(workspace=ws.data_ptr() + 4), 1004)):
        with pytest.raises(hip.LaunchError) as e:
            call(**kw)
        assert e.value.code == code, kw


@pytest.mark.parametrize("nh", [32, 72])
def test_score_kernel_fills_the_selection_histogram(oracle, nh):
    """index_score_paged_hist -> select (hist_ready) gives the rows that the plain score kernel
    followed by the full selection gives on the same device scores, and the oracle's rows for
    those scores. 72 heads are past the matrix-core kernel: the f32 kernel fills the histogram."""
    hd, pt, nt, k, n_q = 128, 64, 20000, 700, 3
    rng = np.random.default_rng(31)
    blocks = -(-nt // pt)
    n_pages = n_q * blocks
    tables = shuffled_block_tables(n_q, blocks, n_pages, seed=9)
    kpool_h = np.zeros((n_pages * pt, hd), np.uint16)
    for qi in range(n_q):
        keys = rng.standard_normal((nt, hd), dtype=np.float32)
        slots = (tables[qi][np.arange(nt) // pt] * pt + np.arange(nt) % pt).astype(np.int32)
        oracle.index_append_paged(keys, slots, kpool_h, hd, pt, n_pages)
    q = rng.standard_normal((n_q, nh, hd), dtype=np.float32)
    w = np.abs(rng.standard_normal((n_q, nh), dtype=np.float32))
    nts = np.array([nt, 16500, nt - 1], np.int32)
    kv_tables, kv_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
    pool_d, kpool = dev(pool_h), dev(kpool_h)
    ws = dzeros(hip.index_topk_workspace_bytes(n_q, nt))
    for ntd in (None, nts):
        sc = dzeros(n_q * nt * 4)
        rows = dzeros(n_q * k * 4, 0xFF)
        out = dzeros(n_q * k * W * 2, 0xEE)
        nt_dev = None if ntd is None else dev(ntd)
        hip.launch_index_score_paged_hist(dev(q), dev(w), kpool, dev(tables), nt_dev, None, n_q, blocks, nt, nt, nh,
                                          nh, hd, pt, n_pages, 0.1, 0.1, sc, ws)
        hist = back(ws, np.uint32).reshape(n_q, -1)[:, :4096].copy()
        hip.launch_dsa_select_gather_paged(sc, n_q, nt, nt_dev, nt, k, rows, ws, True, pool_d, dev(kv_tables), out,
                                           kv_tables.shape[1], W, PT, kv_pages)
        got_rows, got_out = back(rows, np.uint32).reshape(n_q, k), back(out, np.uint16).reshape(n_q, k, W)
        scores = back(sc, np.float32).reshape(n_q, nt)
        for qi in range(n_q):           # the histogram counts exactly the scored tokens, by key
            n = nt if ntd is None else int(ntd[qi])
            assert int(hist[qi].sum()) == n
            b = scores[qi, :n].view(np.uint32).copy()
            b[scores[qi, :n] == 0] = 0
            key = np.where(b >> 31, ~b, b | np.uint32(0x80000000))
            assert np.array_equal(hist[qi], np.bincount(key >> 20, minlength=4096))
        check_against_oracle(oracle, scores, ntd, k, kv_tables, pool_h, got_rows, got_out)
        assert not back(ws, np.uint32).reshape(n_q, -1)[:, :4096].any()


@pytest.mark.parametrize("nh", [32, 72])
def test_a_key_page_outside_the_pool_scores_minus_infinity_in_the_histogram_form(oracle, nh):
    """A block-table entry of the key cache that is not a page of the pool: the score kernel
    that also fills the selection histogram writes -inf for that page's tokens and counts them,
    so the histogram, the scores and the selection that follows (hist_ready) agree; the plain
    score kernel leaves those tokens unwritten."""
    hd, pt, nt, k, n_q = 128, 64, 20000, 700, 2
    rng = np.random.default_rng(77)
    blocks = -(-nt // pt)
    n_pages = n_q * blocks
    tables = shuffled_block_tables(n_q, blocks, n_pages, seed=3)
    kpool_h = (rng.standard_normal((n_pages * pt, hd), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
    tables[0, 5] = n_pages + 7                       # tokens 320..383 of query 0
    tables[1, blocks - 1] = -1                       # the last (partial) page of query 1
    q = rng.standard_normal((n_q, nh, hd), dtype=np.float32)
    w = np.abs(rng.standard_normal((n_q, nh), dtype=np.float32))
    kv_tables, kv_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
    ws = dzeros(hip.index_topk_workspace_bytes(n_q, nt))
    sc = dev(np.full((n_q, nt), 123.0, np.float32))
    rows, out = dzeros(n_q * k * 4, 0xFF), dzeros(n_q * k * W * 2, 0xEE)
    hip.launch_index_score_paged_hist(dev(q), dev(w), dev(kpool_h), dev(tables), None, None, n_q, blocks, nt, nt, nh,
                                      nh, hd, pt, n_pages, 0.1, 0.1, sc, ws)
    hist = back(ws, np.uint32).reshape(n_q, -1)[:, :4096].copy()
    scores = back(sc, np.float32).reshape(n_q, nt).copy()
    lost0, lost1 = slice(5 * pt, 6 * pt), slice((blocks - 1) * pt, nt)
    assert np.all(np.isneginf(scores[0, lost0])) and np.all(np.isneginf(scores[1, lost1]))
    assert np.isfinite(np.delete(scores[0], np.r_[lost0])).all() and int(hist[0].sum()) == nt == int(hist[1].sum())
    hip.launch_dsa_select_gather_paged(sc, n_q, nt, None, nt, k, rows, ws, True, dev(pool_h), dev(kv_tables), out,
                                       kv_tables.shape[1], W, PT, kv_pages)
    got_rows, got_out = back(rows, np.uint32).reshape(n_q, k), back(out, np.uint16).reshape(n_q, k, W)
    check_against_oracle(oracle, scores, None, k, kv_tables, pool_h, got_rows, got_out)
    plain = dev(np.full((n_q, nt), 123.0, np.float32))
    hip.launch_index_score_paged(dev(q), dev(w), dev(kpool_h), dev(tables), None, None, n_q, blocks, nt, nt, nh, nh,
                                 hd, pt, n_pages, 0.1, 0.1, plain)
    plain_h = back(plain, np.float32).reshape(n_q, nt)
    assert np.all(plain_h[0, lost0] == 123.0) and np.all(plain_h[1, lost1] == 123.0)
    keep = np.ones((n_q, nt), bool)
    keep[0, lost0] = keep[1, lost1] = False
    assert np.array_equal(plain_h[keep], scores[keep])


def test_config4_layer_fused(oracle):
    """benchmark configuration 4's layer: 16 queries x 65536 scores, k = 2048, fragmented pages."""
    rng = np.random.default_rng(0x5EED0004)
    n_q, nt, k = 16, 65536, 2048
    tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
    s = rng.standard_normal((n_q, nt), dtype=np.float32)
    s[:, -64:] += np.float32(4.0)
    got_rows, got_out, bad = run_fused(s, None, k, tables, n_pages, dev(pool_h))
    assert bad == 0
    want = oracle.topk_batched(s, k, n_threads=8)
    assert np.array_equal(got_rows, want)
    want_out = oracle.kv_gather_rows_paged(pool_h, tables, want, W, PT)
    assert np.array_equal(got_out, want_out)
