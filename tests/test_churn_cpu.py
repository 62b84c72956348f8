"""Config 5's event stream on the host only: the allocator never hands a live page out twice,
freed pages are reused, and the oracle's pool round-trips every live sequence."""
import numpy as np

from tests.churn import N_PAGES, PT, W, churn_events
from tests.util import bf16_to_f32


def test_churn_stream_keeps_pages_disjoint_and_roundtrips(oracle):
    page_bytes = oracle.kv_page_bytes(PT, W)
    pool = np.zeros(N_PAGES * page_bytes, np.uint8)
    last = np.zeros((N_PAGES * PT, W), np.uint16)   # the row most recently written per slot
    final = stats = None
    n_append = 0
    for ev in churn_events(steps=400, seed=0x5EED0005):
        if ev[0] == "append":
            _, slots, rows = ev
            assert len(set(slots.tolist())) == slots.size
            assert oracle.kv_append_paged(rows, slots, pool, W, PT, N_PAGES) == 0
            last[slots] = rows
            n_append += 1
        elif ev[0] == "final":
            _, final, stats = ev
    assert n_append > 100 and stats["freed_seqs"] > 10 and stats["max_len"] >= 16384
    # every live sequence's slots are distinct across sequences
    seen = set()
    for s, (table, ln) in final.items():
        pages = table.tolist()
        assert not (seen & set(pages))
        seen |= set(pages)
        out = oracle.kv_gather_paged(pool, table[None, :], np.array([ln], np.int32), W, PT)
        # spot check: the gathered row dequantises the LAST row written to that slot
        for t in (0, ln // 2, ln - 1):
            slot = pages[t // PT] * PT + t % PT
            src = bf16_to_f32(last[slot])
            got = bf16_to_f32(out[t])
            amax = np.abs(src).max()
            assert np.all(np.abs(got - src) <= np.abs(src) / 16 * 1.01 + amax / 448 * 2.0 ** -9 + 1e-30)
