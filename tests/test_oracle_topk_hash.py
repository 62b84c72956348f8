"""Pins the oracle's selection and content hashes."""
import numpy as np

from tests.topk_cases import brute_force_topk, reference_topk_cases


def test_topk_reference_kat(oracle):
    """crates/core/src/routing.rs:207-212: score order [1,3,2] -> emitted ascending [1,2,3];
    k beyond n clamps."""
    s = np.array([0.1, 0.9, 0.5, 0.9], np.float32)
    assert oracle.topk(s, 3).tolist() == [1, 2, 3]
    assert oracle.topk(s, 10).tolist() == [0, 1, 2, 3]
    assert oracle.topk(s, 1).tolist() == [1]   # the tie goes to the LOWER index
    assert oracle.topk(s, 0).size == 0


def test_topk_reference_cases_match_brute_force(oracle):
    for name, scores, k in reference_topk_cases(oracle):
        got = oracle.topk(scores, k)
        assert got.size == min(k, scores.size), name
        assert np.array_equal(got, brute_force_topk(scores, k)), name
        assert np.all(np.diff(got.astype(np.int64)) > 0), name


def test_topk_case_shapes_are_what_the_reference_describes(oracle):
    cases = {n: (s, k) for n, s, k in reference_topk_cases(oracle)}
    # the ReLU-sparse answer is an index prefix, the scattered one is not
    s, k = cases["ReLU-sparse (prefix answer)"]
    assert np.array_equal(oracle.topk(s, k), np.arange(2048))
    s, k = cases["scattered zeros (non-prefix answer)"]
    got = oracle.topk(s, k)
    assert not np.array_equal(got, np.arange(2048)) and np.count_nonzero(s[got]) == 300
    # signed zeros all tie: the lowest 2048 indices win, whatever their sign bit
    s, k = cases["mixed +0.0/-0.0"]
    assert np.array_equal(oracle.topk(s, k), np.arange(2048))
    # heavy ties really are heavy: at most 8 distinct values
    assert np.unique(cases["heavy ties"][0]).size <= 8


def test_topk_random_vs_brute_force_and_monotone_relabel(oracle):
    rng = np.random.default_rng(99)
    for n, k in ((1, 1), (7, 3), (64, 64), (1000, 17), (4097, 2048), (65536, 2048)):
        s = rng.standard_normal(n).astype(np.float32)
        s[rng.integers(0, n, n // 4)] = np.float32(0.5)   # ties
        assert np.array_equal(oracle.topk(s, k), brute_force_topk(s, k))
    # spreading the same scores over a longer array (others -inf) relabels the set monotonically
    s = rng.standard_normal(500).astype(np.float32)
    pos = np.sort(rng.choice(5000, 500, replace=False))
    wide = np.full(5000, -np.inf, np.float32)
    wide[pos] = s
    assert np.array_equal(oracle.topk(wide, 100), pos[oracle.topk(s, 100)])


def test_topk_batched_matches_single(oracle):
    rng = np.random.default_rng(5)
    s = rng.standard_normal((5, 3000)).astype(np.float32)
    nts = np.array([3000, 10, 2999, 1, 512], np.int32)
    rows = oracle.topk_batched(s, 256, nts=nts, n_threads=3)
    for q in range(5):
        want = oracle.topk(s[q, : nts[q]], 256)
        assert np.array_equal(rows[q, : want.size], want)
        assert np.all(rows[q, want.size:] == 0xFFFFFFFF)


def test_fnv1a_published_vectors(oracle):
    """crates/core/src/hash.rs:121-125."""
    assert oracle.fnv1a(b"") == 0xCBF29CE484222325
    assert oracle.fnv1a(b"a") == 0xAF63DC4C8601EC8C
    assert oracle.fnv1a(b"foobar") == 0x85944171F73967E8


def test_splitmix_published_sequence_and_fold_properties(oracle):
    """crates/core/src/hash.rs:147-149,248-259 and :171-236."""
    assert oracle.splitmix_finalize(0) == 0
    state, gamma = 0, 0x9E3779B97F4A7C15
    for want in (0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F):
        state = (state + gamma) & (2 ** 64 - 1)
        assert oracle.splitmix_finalize(state) == want
    x = (np.arange(1000, dtype=np.float32) * np.float32(0.5) - np.float32(250.0))
    base = oracle.xor_fold(x)
    assert base != 0
    ulp = x.copy()
    ulp.view(np.uint32)[617] ^= 1
    assert oracle.xor_fold(ulp) != base
    sw = x.copy()
    sw[[4, 900]] = sw[[900, 4]]
    assert oracle.xor_fold(sw) != base
    assert oracle.xor_fold(x, 1) != base
    assert oracle.xor_fold(x[:400]) ^ oracle.xor_fold(x[400:], 400) == base
    sweep = oracle.xor_fold(x, 0, 32)
    want = 0
    for i in range(0, 1000, 32):
        want ^= oracle.xor_fold(x[i:i + 1], i)
    assert sweep == want and sweep != base
    # definition, written out once in Python integers
    m = 2 ** 64 - 1
    h = 0
    for i, b in enumerate(x.view(np.uint32).tolist()):
        z = ((i << 32) ^ b) & m
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        h ^= z ^ (z >> 31)
    assert h == base
