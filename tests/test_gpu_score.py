"""Device indexer scores and the paged indexer key cache against the CPU oracle. The key
cache is bit-exact (one rounding per element); scores carry the reference's own bar for this
kernel: 1e-5 of the largest score (crates/engine/tests/indexer_kernel.rs:336-366)."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros
from tests.test_oracle_score import rel, score_case

pytestmark = pytest.mark.gpu
TOL = 1e-5


def gpu_score(q, w, kbits, heads, nh, hd, wscale, dscale):
    nt = kbits.size // hd
    out = dzeros(nt * 4, 0x7F)
    nact = nh if heads is None else len(heads)
    hip.launch_index_score(dev(q), dev(w), dev(kbits), None if heads is None else dev(np.asarray(heads, np.uint32)),
                           nt, nh, nact, hd, float(wscale), float(dscale), out)
    return back(out, np.float32)


def test_index_score_reference_fixture_both_head_modes(oracle):
    """crates/engine/tests/indexer_kernel.rs:314-366: nt 64, nh 64, hd 128; all heads (DSA) and
    the non-prefix list [5, 0, 6, 2] (MISA)."""
    q, w, kbits, wscale, dscale = score_case(oracle)
    _, want_all = oracle.index_score(q, w, kbits, None, 64, 128, wscale, dscale)
    _, want_sub = oracle.index_score(q, w, kbits, [5, 0, 6, 2], 64, 128, wscale, dscale)
    got_all = gpu_score(q, w, kbits, None, 64, 128, wscale, dscale)
    got_sub = gpu_score(q, w, kbits, [5, 0, 6, 2], 64, 128, wscale, dscale)
    assert rel(got_all, want_all) < TOL, rel(got_all, want_all)
    assert rel(got_sub, want_sub) < TOL, rel(got_sub, want_sub)
    assert rel(got_sub, want_all) > 1e-2       # the head list is honoured, not ignored


def test_index_score_head_weights_land_on_the_right_heads(oracle):
    """One head active at a time with a distinctive weight: a wrong accumulator-to-head map
    would move a weight onto another head's dot."""
    nh, hd, nt = 64, 128, 96
    rng = np.random.default_rng(5)
    q = rng.standard_normal((nh, hd), dtype=np.float32)
    kbits = oracle.f32_to_bf16(rng.standard_normal((nt, hd), dtype=np.float32))
    for h in (0, 1, 3, 4, 7, 8, 31, 32, 36, 63):
        w = np.zeros(nh, np.float32)
        w[h] = np.float32(1.0 + h)
        _, want = oracle.index_score(q, w, kbits, None, nh, hd, 1.0, 0.25)
        got = gpu_score(q, w, kbits, None, nh, hd, 1.0, 0.25)
        assert rel(got, want) < TOL, h
        assert np.abs(want).max() > 0


@pytest.mark.parametrize("nt,nh,nact,hd", [(1, 8, 8, 16), (31, 32, 32, 64), (33, 32, 17, 128),
                                           (513, 64, 64, 128), (2000, 40, 33, 96), (512, 4, 4, 32),
                                           # beyond the matrix-core kernel: more than 64 active heads,
                                           # wider heads, a width that is not a multiple of 16, and
                                           # the reference's own upper limits (1024 heads; 64 KiB of LDS)
                                           (300, 128, 128, 128), (200, 8, 8, 256), (100, 8, 5, 24),
                                           (70, 100, 65, 40), (9, 1024, 1024, 16), (5, 4, 4, 16000),
                                           (130, 200, 200, 128)])
def test_index_score_shapes(oracle, nt, nh, nact, hd):
    rng = np.random.default_rng(nt)
    q = rng.standard_normal((nh, hd), dtype=np.float32)
    w = rng.standard_normal(nh, dtype=np.float32)
    kbits = oracle.f32_to_bf16(rng.standard_normal((nt, hd), dtype=np.float32))
    heads = None if nact == nh else rng.permutation(nh)[:nact]
    _, want = oracle.index_score(q, w, kbits, heads, nh, hd, 0.75, 0.125)
    got = gpu_score(q, w, kbits, heads, nh, hd, 0.75, 0.125)
    assert rel(got, want) < TOL


def test_index_score_guards():
    b = dzeros(1 << 16)
    for args, code in (((0, 8, 8, 16), 1001), ((4, 8, 9, 16), 1001), ((4, 0, 0, 16), 1001),
                       ((4, 2048, 1025, 16), 1002), ((4, 8, 8, 16384), 1002)):     # the reference's own limits
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_index_score(b, b, b, None, *args, 1.0, 1.0, b)
        assert e.value.code == code, args
    # paged: every scored token needs a block-table entry (here 2 blocks x 64 tokens < nt = 129)
    with pytest.raises(hip.LaunchError) as e:
        hip.launch_index_score_paged(b, b, b, b, None, None, 1, 2, 129, 129, 8, 8, 16, 64, 4, 1.0, 1.0, b)
    assert e.value.code == 1002


@pytest.mark.parametrize("pt,n_pages,blocks,nh", [(64, 40, 12, 32), (16, 160, 48, 32), (64, 40, 12, 96)])
def test_paged_index_append_and_score(oracle, pt, n_pages, blocks, nh):
    """Keys appended through a slot mapping into a fragmented pool, then scored through the
    block tables for three queries of different lengths (pages of 16 tokens and 96 heads take
    the plain kernel)."""
    hd = 128
    rng = np.random.default_rng(8)
    nts = np.array([760, 64, 300], np.int32)
    tables = rng.permutation(n_pages)[:3 * blocks].reshape(3, blocks).astype(np.int32)
    q = rng.standard_normal((3, nh, hd), dtype=np.float32)
    w = rng.standard_normal((3, nh), dtype=np.float32)
    want_pool = np.full((n_pages * pt, hd), 0x1234, np.uint16)
    kpool = dev(want_pool)
    bad = dzeros(4)
    for qi in range(3):
        t = np.arange(nts[qi])
        keys = rng.standard_normal((nts[qi], hd), dtype=np.float32) * np.float32(3.0)
        slots = (tables[qi][t // pt] * pt + t % pt).astype(np.int32)
        slots_pad = np.concatenate([slots, [-1, n_pages * pt + 5]]).astype(np.int32)
        keys_pad = np.concatenate([keys, np.ones((2, hd), np.float32)])
        assert oracle.index_append_paged(keys_pad, slots_pad, want_pool, hd, pt, n_pages) == 1
        hip.launch_index_append_paged(dev(keys_pad), dev(slots_pad), kpool, slots_pad.size, hd, pt,
                                      n_pages, bad)
    assert int(back(bad, np.uint32)[0]) == 3
    assert np.array_equal(back(kpool, np.uint16).reshape(-1, hd), want_pool)   # bit-exact keys
    stride = 768
    out = dzeros(3 * stride * 4, 0x7F)
    hip.launch_index_score_paged(dev(q), dev(w), kpool, dev(tables), dev(nts), None, 3, blocks, stride,
                                 stride, nh, nh, hd, pt, n_pages, 0.75, 0.125, out)
    got = back(out, np.float32).reshape(3, stride)
    want = oracle.index_score_paged(q, w, want_pool, tables, nts, None, stride, hd, pt, 0.75, 0.125,
                                    n_threads=4)
    fill = np.frombuffer(b"\x7f" * 4, np.float32)[0]
    for qi in range(3):
        assert rel(got[qi, : nts[qi]], want[qi, : nts[qi]]) < TOL, qi
        assert np.all(got[qi, nts[qi]:] == fill)            # nothing written past nts[qi]


def test_scores_feed_topk_like_the_oracle_chain(oracle):
    """score -> top-k on the device selects what the oracle's score -> top-k selects, except
    where two scores sit within the score tolerance of the k-th one."""
    hd, pt, nh, nt, k = 128, 64, 32, 8192, 512
    rng = np.random.default_rng(21)
    n_pages = nt // pt
    table = rng.permutation(n_pages).astype(np.int32)[None, :]
    keys = rng.standard_normal((nt, hd), dtype=np.float32)
    slots = (table[0][np.arange(nt) // pt] * pt + np.arange(nt) % pt).astype(np.int32)
    kpool_h = np.zeros((n_pages * pt, hd), np.uint16)
    oracle.index_append_paged(keys, slots, kpool_h, hd, pt, n_pages)
    q = rng.standard_normal((1, nh, hd), dtype=np.float32)
    w = np.abs(rng.standard_normal((1, nh), dtype=np.float32))
    want_scores = oracle.index_score_paged(q, w, kpool_h, table, [nt], None, nt, hd, pt, 0.1, 0.1)
    kpool = dzeros(kpool_h.nbytes)
    hip.launch_index_append_paged(dev(keys), dev(slots), kpool, nt, hd, pt, n_pages)
    sc = dzeros(nt * 4)
    hip.launch_index_score_paged(dev(q), dev(w), kpool, dev(table), None, None, 1, n_pages, nt, nt,
                                 nh, nh, hd, pt, n_pages, 0.1, 0.1, sc)
    rows = dzeros(k * 4, 0xFF)
    hip.launch_index_topk_batched(sc, 1, nt, None, nt, k, rows)
    got = back(rows, np.uint32)
    want = oracle.topk(want_scores[0], k)
    differ = np.setxor1d(got, want)
    kth = np.sort(want_scores[0])[-k]
    tol = TOL * np.abs(want_scores).max() * 4
    assert np.all(np.abs(want_scores[0][differ] - kth) <= tol), differ
    # and on the device's own scores the selection is exactly the oracle's rule
    assert np.array_equal(got, oracle.topk(back(sc, np.float32), k))
