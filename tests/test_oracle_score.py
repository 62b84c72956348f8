"""Pins the oracle's indexer score against a float64 restatement and the properties the
reference's own test relies on (crates/engine/tests/indexer_kernel.rs:200-366)."""
import numpy as np

from tests.util import bf16_to_f32


def score_case(oracle, nt=64, nh=64, hd=128):
    """The reference's ScoreCase: one Lcg(0x5C04) stream drawn as q, w, then the key cache
    rounded through bf16 (crates/engine/tests/indexer_kernel.rs:213-236)."""
    r = oracle.lcg(0x5C04)
    q = r.fill(nh * hd).reshape(nh, hd)
    w = r.fill(nh)
    kbits = oracle.f32_to_bf16(r.fill(nt * hd)).reshape(nt, hd)
    return q, w, kbits, np.float32(0.75), np.float32(0.125)


def score_f64(q, w, kbits, heads, wscale, dscale):
    k = bf16_to_f32(kbits).astype(np.float64)
    qa = q.astype(np.float64)[heads]
    dots = k @ qa.T                                              # [nt, nact]
    return (np.maximum(dots * float(dscale), 0.0) * (w.astype(np.float64)[heads] * float(wscale))).sum(axis=1)


def rel(a, b):
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def test_index_score_matches_float64_and_separates_head_sets(oracle):
    q, w, kbits, wscale, dscale = score_case(oracle)
    all_heads = np.arange(64)
    subset = np.array([5, 0, 6, 2])
    rc, got_all = oracle.index_score(q, w, kbits, None, 64, 128, wscale, dscale)
    assert rc == 0
    rc, got_sub = oracle.index_score(q, w, kbits, subset, 64, 128, wscale, dscale)
    assert rc == 0
    assert rel(got_all, score_f64(q, w, kbits, all_heads, wscale, dscale)) < 1e-6
    assert rel(got_sub, score_f64(q, w, kbits, subset, wscale, dscale)) < 1e-6
    # the reference's anti-vacuity: the two head sets really score differently
    assert rel(got_sub, got_all) > 1e-2
    # a prefix list [0,1,2,3] is NOT what [5,0,6,2] computes
    _, got_prefix = oracle.index_score(q, w, kbits, np.arange(4), 64, 128, wscale, dscale)
    assert rel(got_prefix, got_sub) > 1e-2


def test_index_score_closed_forms_and_guards(oracle):
    hd, nt = 16, 5
    q = np.zeros((2, hd), np.float32)
    q[0, 3] = 2.0
    q[1, 3] = -2.0
    w = np.array([0.5, 4.0], np.float32)
    k = np.zeros((nt, hd), np.float32)
    k[:, 3] = np.array([1.0, -1.0, 0.0, 3.0, -0.5], np.float32)
    kbits = oracle.f32_to_bf16(k)
    _, got = oracle.index_score(q, w, kbits, None, 2, hd, 1.0, 1.0)
    # head 0 passes positive products (x0.5), head 1 the negated ones (x4): ReLU picks one each
    want = np.array([0.5 * 2, 4 * 2, 0, 0.5 * 6, 4 * 1], np.float32)
    assert np.array_equal(got, want)
    rc, _ = oracle.index_score(q, w, np.zeros(0, np.uint16), None, 2, hd, 1.0, 1.0)   # nt == 0
    assert rc == 1001
    rc, _ = oracle.index_score(q, w, kbits, np.arange(3), 2, hd, 1.0, 1.0)   # nact > nh
    assert rc == 1001


def test_paged_score_equals_linear_score_through_any_table(oracle):
    hd, pt, n_pages, nh = 128, 64, 12, 8
    rng = np.random.default_rng(3)
    q = rng.standard_normal((2, nh, hd), dtype=np.float32)
    w = rng.standard_normal((2, nh), dtype=np.float32)
    nts = np.array([300, 130], np.int32)
    tables = rng.permutation(n_pages)[:10].reshape(2, 5).astype(np.int32)
    keys = [rng.standard_normal((n, hd), dtype=np.float32) for n in nts]
    kpool = np.zeros((n_pages * pt, hd), np.uint16)
    for qi in range(2):
        t = np.arange(nts[qi])
        slots = (tables[qi][t // pt] * pt + t % pt).astype(np.int32)
        assert oracle.index_append_paged(keys[qi], slots, kpool, hd, pt, n_pages) == 0
    got = oracle.index_score_paged(q, w, kpool, tables, nts, None, 320, hd, pt, 0.75, 0.125, n_threads=3)
    for qi in range(2):
        _, lin = oracle.index_score(q[qi], w[qi], oracle.f32_to_bf16(keys[qi]), None, nh, hd, 0.75, 0.125)
        assert np.array_equal(got[qi, : nts[qi]], lin)
        assert not got[qi, nts[qi]:].any()
    assert oracle.index_append_paged(keys[0][:2], np.array([-1, n_pages * pt], np.int32), kpool, hd, pt, n_pages) == 1
