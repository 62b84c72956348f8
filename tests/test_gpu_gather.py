"""Block-table gather + dequantize and the sparse row gather against the CPU oracle: every
bf16 bit equal (the bar is 1 ulp; the kernels meet 0)."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros
from tests.util import make_rows_bf16, shuffled_block_tables, slots_for

pytestmark = pytest.mark.gpu
W, PT = 576, 64


def build_pool(oracle, seq_lens, n_pages, seed, width=W, pt=PT, outlier_frac=0.0, outlier_mul=1.0):
    """Oracle-side pool with every sequence appended through a shuffled global block table."""
    n_seqs = len(seq_lens)
    max_blocks = -(-max(seq_lens) // pt)
    tables = shuffled_block_tables(n_seqs, max_blocks, n_pages, seed)
    pool = np.zeros(n_pages * oracle.kv_page_bytes(pt, width), np.uint8)
    for s, ln in enumerate(seq_lens):
        rows = make_rows_bf16(ln, width, seed=seed * 1000 + s, outlier_frac=outlier_frac,
                              outlier_mul=outlier_mul)
        oracle.kv_append_paged(rows, slots_for(tables[s], np.arange(ln), pt), pool, width, pt,
                               n_pages)
    return pool, tables


def gpu_gather(pool, tables, seq_lens, width=W, pt=PT, n_pages=None, fill=0x5A):
    """The gather through both entry points — the grid over what the block tables could hold and
    the one sized by the batch's token count (exact, and overstated) — which must agree byte
    for byte, fill included."""
    seq_lens = np.asarray(seq_lens, np.int32)
    cu = np.zeros(seq_lens.size + 1, np.int32)
    np.cumsum(seq_lens, out=cu[1:])
    n_pages = n_pages or pool.size // (pt * (width + 4))
    pool_d, tables_d, lens_d, cu_d = dev(pool), dev(tables), dev(seq_lens), dev(cu)
    total = int(np.minimum(np.maximum(seq_lens, 0), tables.shape[1] * pt).sum())
    # the same tables with four times as many (unused) columns: a batch that fills less than
    # 0.7 of its tables takes the launch sized by the token count
    wide = np.full((tables.shape[0], 4 * tables.shape[1] + 1), -1, np.int32)
    wide[:, : tables.shape[1]] = tables
    wide_d = dev(wide)
    results = []
    for form in ("grid", "packed", "packed-wide", "packed-wide+slack"):
        out = dzeros(max(int(cu[-1]), 1) * width * 2, fill)
        bad = dzeros(4)
        if form == "grid":
            hip.launch_kv_gather_paged(pool_d, tables_d, lens_d, cu_d, out, seq_lens.size,
                                       tables.shape[1], width, pt, n_pages, bad)
        else:
            t_d, t = (wide_d, wide) if "wide" in form else (tables_d, tables)
            hip.launch_kv_gather_paged_packed(pool_d, t_d, lens_d, cu_d, out, seq_lens.size, t.shape[1],
                                              total + (37 if form.endswith("slack") else 0),
                                              width, pt, n_pages, bad)
        results.append((back(out, np.uint16).reshape(-1, width), int(back(bad, np.uint32)[0])))
    for got, bad in results[1:]:
        assert bad == results[0][1]
        assert np.array_equal(got, results[0][0])
    return results[0]


def test_config1_gather_full_context(oracle):
    """benchmark configuration 1: batch 1, ctx 4096, block table a seeded permutation of 64 pages."""
    pool, tables = build_pool(oracle, [4096], 64, seed=0x5EED0001 % 10007)
    want = oracle.kv_gather_paged(pool, tables, [4096], W, PT)
    got, bad = gpu_gather(pool, tables, [4096])
    assert bad == 0 and np.array_equal(got, want)
    assert np.count_nonzero(want) > want.size * 0.9


def test_ragged_batch_with_partial_pages_and_outliers(oracle):
    seq_lens = [1, 63, 64, 65, 700, 1024, 2049, 5]
    pool, tables = build_pool(oracle, seq_lens, 320, seed=31, outlier_frac=0.01, outlier_mul=200.0)
    want = oracle.kv_gather_paged(pool, tables, seq_lens, W, PT)
    got, bad = gpu_gather(pool, tables, seq_lens)
    assert bad == 0 and np.array_equal(got, want)


def test_zero_length_sequences_and_untouched_tail(oracle):
    seq_lens = [0, 130, 0, 64]
    pool, tables = build_pool(oracle, [1, 130, 1, 64], 16, seed=5)
    want = oracle.kv_gather_paged(pool, tables, seq_lens, W, PT)
    got, _ = gpu_gather(pool, tables, seq_lens)
    assert got.shape == want.shape and np.array_equal(got, want)
    # a larger output buffer keeps its fill past the last token
    cu_total = sum(seq_lens)
    out = dzeros((cu_total + 3) * W * 2, 0x5A)
    sl = np.asarray(seq_lens, np.int32)
    cu = np.concatenate([[0], np.cumsum(sl)]).astype(np.int32)
    hip.launch_kv_gather_paged(dev(pool), dev(tables), dev(sl), dev(cu), out, 4, tables.shape[1],
                               W, PT, 16)
    assert np.all(back(out)[cu_total * W * 2:] == 0x5A)


def test_many_uneven_sequences(oracle):
    """More sequences than a wave has lanes, lengths from 0 to a few pages, block tables mostly
    empty: the token-count-sized launch scans the lengths in several rounds."""
    rng = np.random.default_rng(150)
    seq_lens = [int(x) for x in rng.integers(0, 300, size=150)]
    seq_lens[0], seq_lens[63], seq_lens[64], seq_lens[149] = 0, 299, 1, 17
    pool, tables = build_pool(oracle, [max(n, 1) for n in seq_lens], 150 * 5 + 7, seed=150)
    want = oracle.kv_gather_paged(pool, tables, seq_lens, W, PT)
    got, bad = gpu_gather(pool, tables, seq_lens)
    assert bad == 0 and np.array_equal(got, want)


def test_gather_is_invariant_under_page_permutation(oracle):
    """Same tokens through two different block tables give the same rows."""
    outs = []
    for seed in (3, 4):
        rows = make_rows_bf16(1000, W, seed=77)
        table = shuffled_block_tables(1, 16, 32, seed)
        pool = np.zeros(32 * oracle.kv_page_bytes(PT, W), np.uint8)
        oracle.kv_append_paged(rows, slots_for(table[0], np.arange(1000)), pool, W, PT, 32)
        outs.append(gpu_gather(pool, table, [1000])[0])
    assert np.array_equal(outs[0], outs[1])


def test_bad_page_ids_are_skipped_and_counted(oracle):
    pool, tables = build_pool(oracle, [200, 200], 8, seed=9)
    tables = tables.copy()
    tables[0, 1] = 8          # one past the pool
    tables[1, 0] = -3
    got, bad = gpu_gather(pool, tables, [200, 200], n_pages=8, fill=0x5A)
    assert bad == 2
    want = oracle.kv_gather_paged(pool, np.where((tables < 0) | (tables >= 8), 0, tables),
                                  [200, 200], W, PT)
    ok = np.ones(400, bool)
    ok[64:128] = False
    ok[200:264] = False
    assert np.array_equal(got[ok], want[ok])
    assert np.all(got[~ok] == 0x5A5A)


def test_gather_other_shapes(oracle):
    for width, pt, lens in ((512, 64, [300, 70]), (128, 16, [100, 33, 16]), (1024, 32, [65]),
                            (64, 4, [9, 4, 1])):
        n_pages = 64
        pool, tables = build_pool(oracle, lens, n_pages, seed=width, width=width, pt=pt)
        want = oracle.kv_gather_paged(pool, tables, lens, width, pt)
        got, bad = gpu_gather(pool, tables, lens, width=width, pt=pt, n_pages=n_pages)
        assert bad == 0 and np.array_equal(got, want), (width, pt)


def test_gather_guards():
    b = dzeros(4096)
    for args, code in (((0, 1, W, PT, 1), 1001), ((1, 0, W, PT, 1), 1001), ((1, 1, W, PT, 0), 1001),
                       ((1, 1, 570, PT, 1), 1004), ((1, 1, W, 6, 1), 1004),
                       ((70000, 1, W, PT, 1), 1002)):
        with pytest.raises(hip.LaunchError) as e:
            hip.launch_kv_gather_paged(b, b, b, b, b, *args)
        assert e.value.code == code, args
    with pytest.raises(hip.LaunchError):
        hip.launch_kv_gather_rows_paged(b, b, None, None, b, 1, 1, 1, W, PT, 1)


def gpu_gather_rows(pool, tables, rows, n_rows=None, width=W, pt=PT, fill=0x5A):
    n_q, k = rows.shape
    out, bad = dzeros(n_q * k * width * 2, fill), dzeros(4)
    n_pages = pool.size // (pt * (width + 4))
    hip.launch_kv_gather_rows_paged(dev(pool), dev(tables), dev(rows),
                                    None if n_rows is None else dev(np.asarray(n_rows, np.int32)),
                                    out, n_q, k, tables.shape[1], width, pt, n_pages, bad)
    return back(out, np.uint16).reshape(n_q, k, width), int(back(bad, np.uint32)[0])


def test_sparse_rows_equal_dense_gather_indexed(oracle):
    """The reference has no test with rows != null (crates/engine/tests/kernel_attend.rs:114);
    the sparse gather is pinned by gather_rows(rows) == gather_dense()[rows]."""
    ctx, n_q, k = 3000, 3, 500
    pool, tables = build_pool(oracle, [ctx] * n_q, 160, seed=13, outlier_frac=0.01, outlier_mul=50.0)
    rng = np.random.default_rng(2)
    rows = np.stack([np.sort(rng.choice(ctx, k, replace=False)) for _ in range(n_q)]).astype(np.uint32)
    dense, _ = gpu_gather(pool, tables, [ctx] * n_q)
    dense = dense.reshape(n_q, ctx, W)
    got, bad = gpu_gather_rows(pool, tables, rows)
    want = oracle.kv_gather_rows_paged(pool, tables, rows, W, PT)
    assert bad == 0 and np.array_equal(got, want)
    for q in range(n_q):
        assert np.array_equal(got[q], dense[q][rows[q]])
    # unsorted and repeated indices are legal: the gather is a pure function of each row id
    rows2 = rng.integers(0, ctx, (n_q, k)).astype(np.uint32)
    got2, _ = gpu_gather_rows(pool, tables, rows2)
    assert np.array_equal(got2, oracle.kv_gather_rows_paged(pool, tables, rows2, W, PT))


def test_sparse_rows_short_lists_and_bad_rows(oracle):
    ctx, k = 640, 70
    pool, tables = build_pool(oracle, [ctx, ctx], 32, seed=17)
    rng = np.random.default_rng(3)
    rows = np.stack([np.sort(rng.choice(ctx, k, replace=False)) for _ in range(2)]).astype(np.uint32)
    got, bad = gpu_gather_rows(pool, tables, rows, n_rows=[k, 33])
    want = oracle.kv_gather_rows_paged(pool, tables, rows, W, PT, n_rows=[k, 33])
    assert bad == 0
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1, :33], want[1, :33])
    assert np.all(got[1, 33:] == 0x5A5A)            # rows past n_rows are not written
    rows_bad = rows.copy()
    rows_bad[0, 7] = 10 * PT + 5                    # block 10 == max_blocks: out of the table
    rows_bad[1, 2] = 0xFFFFFFFF
    got, bad = gpu_gather_rows(pool, tables, rows_bad)
    assert bad == 2 and np.all(got[0, 7] == 0x5A5A) and np.all(got[1, 2] == 0x5A5A)
    keep = np.ones((2, k), bool)
    keep[0, 7] = keep[1, 2] = False
    full = oracle.kv_gather_rows_paged(pool, tables, rows, W, PT)
    assert np.array_equal(got[keep], full[keep])


def test_sparse_rows_other_shapes(oracle):
    """The sparse gather's generic form: other widths and page sizes, unsorted lists."""
    for width, pt, ctx, k in ((512, 64, 300, 77), (128, 16, 100, 40), (1024, 32, 65, 65), (64, 4, 9, 5)):
        lens = [ctx, ctx]
        pool, tables = build_pool(oracle, lens, 64, seed=width + 3, width=width, pt=pt)
        rows = np.random.default_rng(width).integers(0, ctx, (2, k)).astype(np.uint32)
        got, bad = gpu_gather_rows(pool, tables, rows, width=width, pt=pt)
        want = oracle.kv_gather_rows_paged(pool, tables, rows, width, pt)
        assert bad == 0 and np.array_equal(got, want), (width, pt)
