"""Device row selection and the XOR fold against the CPU oracle (and, where it was built,
against the reference's own kernels compiled for this GPU)."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.topk_cases import brute_force_topk, reference_topk_cases

pytestmark = pytest.mark.gpu
SENTINEL = 0xFFFFFFFF


def check_topk_case(name, scores, k, want, launch):
    """crates/engine/tests/kernel_vector.rs:174-212: sentinel-filled buffer, tail untouched,
    strictly ascending."""
    n = scores.size
    written = min(k, n)
    rows = dzeros(max(n, k) * 4, 0xFF)
    launch(dev(scores), n, k, rows)
    got = back(rows, np.uint32)
    assert want.size == written, name
    assert np.array_equal(got[:written], want), name
    assert np.all(got[written:] == SENTINEL), f"wrote past min(k,nt) on {name}"
    assert np.all(np.diff(got[:written].astype(np.int64)) > 0), name


def test_index_topk_reference_cases(oracle):
    for name, scores, k in reference_topk_cases(oracle):
        want = oracle.topk(scores, k)
        check_topk_case(name, scores, k, want, hip.launch_index_topk)


def test_reference_index_topk_agrees_with_the_oracle(oracle):
    """The reference's own kernel (indexer.hip compiled for this GPU) on its own cases."""
    ref = need_ref("rivoli_index_topk")
    for name, scores, k in reference_topk_cases(oracle):
        check_topk_case("ref:" + name, scores, k, oracle.topk(scores, k),
                        lambda s, n, kk, r: ref.rivoli_index_topk(s.data_ptr(), n, kk, r.data_ptr()))


def test_index_topk_guards():
    b = dzeros(64)
    for nt, k in ((0, 4), (4, 0), (-1, 4)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_index_topk(b, nt, k, b)
        assert e.value.code == 1001
    with pytest.raises(hip.LaunchError) as e:
        hip.launch_index_topk_batched(b, 2, 4, None, 8, 2, b)   # stride < nt
    assert e.value.code == 1002


def batched_topk(scores, nts, k, split):
    """Runs the batched entry point without (one workgroup per query) or with a workspace
    (each query split over the chip), twice in the latter case on the SAME workspace so the
    second call sees what the first one left behind."""
    n_q, stride = scores.shape
    sd = dev(scores)
    ntd = None if nts is None else dev(np.asarray(nts, np.int32))
    ws = dzeros(hip.index_topk_workspace_bytes(n_q, stride)) if split else None
    got = None
    for _ in range(2 if split else 1):
        rows = dzeros(n_q * k * 4, 0xFF)
        hip.launch_index_topk_batched(sd, n_q, stride, ntd, stride, k, rows, ws)
        got = back(rows, np.uint32).reshape(n_q, k)
    if split:   # the per-query histogram is back to zero
        assert not back(ws, np.uint32).reshape(n_q, -1)[:, :4096].any()
    return got


def dsa_scores(n_q, nt, seed):
    """benchmark configuration 4's score shape: N(0,1) plus a boost on the last 64 tokens."""
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((n_q, nt), dtype=np.float32)
    s[:, -64:] += np.float32(4.0)
    return s


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("nt", [1, 63, 64, 65, 1023, 1024, 1025, 4096, 4097, 5185, 8192, 16384,
                                16385, 65535, 65536, 65537, 200_000, 300_000])
def test_batched_topk_sizes(oracle, nt, split):
    """Every register-resident variant's boundary, the streaming path past 65536, and the
    segment boundaries of the split form."""
    n_q, k = 3, 2048
    s = dsa_scores(n_q, nt, seed=nt)
    s[1, :: 3] = np.float32(0.25)               # a tie-heavy query (overflows the candidate cache)
    got = batched_topk(s, None, k, split)
    for q in range(n_q):
        want = oracle.topk(s[q], k)
        assert np.array_equal(got[q, : want.size], want), (nt, q)
        assert np.all(got[q, want.size:] == SENTINEL)
    if nt <= 5185:
        assert np.array_equal(got[0, : min(k, nt)], brute_force_topk(s[0], k))


@pytest.mark.parametrize("split", [False, True])
def test_config4_shape_16_queries_of_65536(oracle, split):
    n_q, nt, k = 16, 65536, 2048
    s = dsa_scores(n_q, nt, seed=0x5EED0004)
    got = batched_topk(s, None, k, split)
    want = oracle.topk_batched(s, k, n_threads=8)
    assert np.array_equal(got, want)
    assert np.all(np.isin(np.arange(nt - 64, nt), got[0]))   # the recency window is selected


@pytest.mark.parametrize("split", [False, True])
def test_batched_topk_per_query_lengths_and_strides(oracle, split):
    n_q, stride, k = 6, 9000, 512
    s = dsa_scores(n_q, stride, seed=4)
    nts = np.array([9000, 1, 0, 511, 512, 8999], np.int32)
    got = batched_topk(s, nts, k, split)
    for q in range(n_q):
        want = oracle.topk(s[q, : nts[q]], k)
        assert np.array_equal(got[q, : want.size], want), q
        assert np.all(got[q, want.size:] == SENTINEL), q


@pytest.mark.parametrize("split", [False, True])
def test_topk_adversarial_values(oracle, split):
    nt, k = 70000, 2048
    rng = np.random.default_rng(8)
    cases = {
        "all equal": np.full(nt, 1.5, np.float32),
        "all zero mixed sign": np.where(rng.random(nt) < 0.5, np.float32(-0.0), np.float32(0.0)),
        "infinities": rng.choice(np.array([-np.inf, np.inf, 0.0, 1.0], np.float32), nt),
        "denormals": (rng.integers(-50, 50, nt) * np.float32(1e-45)).astype(np.float32),
        "low-byte ties": (np.float32(1.0) + (rng.integers(0, 4, nt) * np.float32(2.0 ** -23))).astype(np.float32),
        "descending": np.arange(nt, 0, -1).astype(np.float32),
        "ascending": np.arange(nt).astype(np.float32),
    }
    for name, s in cases.items():
        for n in (nt, 65536, 3000):
            got = batched_topk(np.ascontiguousarray(s[None, :n]), None, k, split)[0]
            assert np.array_equal(got, oracle.topk(s[:n], k)), (name, n)


@pytest.mark.parametrize("split", [False, True])
def test_topk_small_k_and_k_beyond_nt(oracle, split):
    rng = np.random.default_rng(15)
    s = rng.standard_normal((4, 20000)).astype(np.float32)
    for k in (1, 2, 63, 64, 4095, 4096, 4097, 20000, 25000):
        got = batched_topk(s, None, k, split)
        for q in range(4):
            want = oracle.topk(s[q], k)
            assert np.array_equal(got[q, : want.size], want), (k, q)
            assert np.all(got[q, want.size:] == SENTINEL), (k, q)


def test_hash_rows_matches_the_host_fold(oracle):
    """crates/engine/tests/fwd_kernel.rs:313-384: n = 1000 from Lcg(0x8AD5)."""
    n = 1000
    x = oracle.lcg(0x8AD5).fill(n)

    def fold(v, stride=1, i_base=0, launch=hip.launch_hash_rows):
        out = dzeros(8)
        launch(dev(v), v.size, stride, i_base, out)
        return int(back(out, np.uint64)[0])

    want = oracle.xor_fold(x)
    assert fold(x) == want
    ulp = x.copy()
    ulp.view(np.uint32)[617] ^= 1
    assert oracle.xor_fold(ulp) != want and fold(ulp) == oracle.xor_fold(ulp)
    sw = x.copy()
    sw[[4, 900]] = sw[[900, 4]]
    assert fold(sw) != want
    assert fold(x, stride=32) == oracle.xor_fold(x, 0, 32)
    assert fold(x, i_base=400) == oracle.xor_fold(x, 400)
    xd, twice = dev(x), dzeros(8)
    for _ in range(2):
        hip.launch_hash_rows(xd, n, 1, 0, twice)
    assert int(back(twice, np.uint64)[0]) == 0
    big = np.random.default_rng(1).integers(0, 2 ** 32, 3_000_001, dtype=np.uint64).astype(np.uint32)
    assert fold(big.view(np.float32)) == oracle.xor_fold(big)
    with pytest.raises(hip.LaunchError):
        hip.launch_hash_rows(xd, 0, 1, 0, twice)


def test_reference_hash_rows_agrees_with_the_host_fold(oracle):
    """The reference's own kernel (compiled for this GPU) on the same 1000 values."""
    ref = need_ref("rivoli_hash_rows")
    n = 1000
    x = oracle.lcg(0x8AD5).fill(n)
    xd, out = dev(x), dzeros(8)
    assert ref.rivoli_hash_rows(xd.data_ptr(), n, 1, 0, out.data_ptr(), None) == 0
    assert int(back(out, np.uint64)[0]) == oracle.xor_fold(x)
