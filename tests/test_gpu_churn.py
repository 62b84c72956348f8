"""benchmark configuration 5 on the device: 10k seeded steps of appends and whole-sequence frees with
LIFO page reuse and x200 outlier tokens; the device pool must equal the oracle's byte for byte
throughout, and every surviving sequence must gather identically."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.churn import N_PAGES, PT, W, churn_events
from tests.gpu_util import back, dev, dzeros

pytestmark = pytest.mark.gpu


def test_config5_churn_10k_steps(oracle):
    page_bytes = oracle.kv_page_bytes(PT, W)
    want = np.zeros(N_PAGES * page_bytes, np.uint8)
    pool, bad = dzeros(N_PAGES * page_bytes), dzeros(4)
    n_events, final, stats = 0, None, None
    for ev in churn_events(steps=10_000, seed=0x5EED0005):
        if ev[0] == "append":
            _, slots, rows = ev
            oracle.kv_append_paged(rows, slots, want, W, PT, N_PAGES)
            hip.launch_kv_append_paged(dev(rows), dev(slots), pool, slots.size, W, PT, N_PAGES, bad)
            n_events += 1
            if n_events % 2500 == 0:
                assert np.array_equal(back(pool), want), f"pool diverged by event {n_events}"
        elif ev[0] == "final":
            _, final, stats = ev
    assert int(back(bad, np.uint32)[0]) == 0
    assert np.array_equal(back(pool), want)
    assert stats["freed_seqs"] + stats["evictions"] > 300 and stats["appended"] > 300_000
    # saturation really happened: outlier tokens put 0x7e codes next to crushed small ones
    codes = want.reshape(N_PAGES, page_bytes)[:, : PT * W]
    assert np.count_nonzero((codes & 0x7F) == 0x7E) > 1000
    seqs = sorted(final)
    lens = np.array([final[s][1] for s in seqs], np.int32)
    max_blocks = max(len(final[s][0]) for s in seqs)
    tables = np.zeros((len(seqs), max_blocks), np.int32)
    for i, s in enumerate(seqs):
        tables[i, : len(final[s][0])] = final[s][0]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    out = dzeros(int(cu[-1]) * W * 2)
    hip.launch_kv_gather_paged(pool, dev(tables), dev(lens), dev(cu), out, len(seqs), max_blocks,
                               W, PT, N_PAGES)
    assert np.array_equal(back(out, np.uint16).reshape(-1, W),
                          oracle.kv_gather_paged(want, tables, lens, W, PT, n_threads=8))
