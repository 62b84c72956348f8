"""Host allocator: LIFO reuse in the order of crates/core/src/arena.rs:132-149, checked
against a pure-Python model under seeded churn."""
import numpy as np
import pytest

from rivoli_amd.pagepool import PagePool, PoolExhausted


class ModelPool:
    """Independent restatement: free list = Python list used as a stack, frontier grows."""

    def __init__(self, n_pages, pt):
        self.n, self.pt, self.frontier, self.free, self.seqs = n_pages, pt, 0, [], {}

    def extend(self, sid, n):
        pages, ln = self.seqs.setdefault(sid, ([], 0))
        need = -(-(ln + n) // self.pt) - len(pages)
        if need > len(self.free) + self.n - self.frontier:
            raise PoolExhausted
        for _ in range(need):
            if self.free:
                pages.append(self.free.pop())
            else:
                pages.append(self.frontier)
                self.frontier += 1
        slots = [pages[t // self.pt] * self.pt + t % self.pt for t in range(ln, ln + n)]
        self.seqs[sid] = (pages, ln + n)
        return slots

    def free_seq(self, sid):
        pages, _ = self.seqs.pop(sid, ([], 0))
        self.free.extend(pages)
        return len(pages)


def test_lifo_reuse_and_frontier():
    p = PagePool(8, 4)
    a, b = p.seq_create(), p.seq_create()
    assert p.seq_extend(a, 5).tolist() == [0, 1, 2, 3, 4]       # pages 0,1
    assert p.seq_extend(b, 4).tolist() == [8, 9, 10, 11]        # page 2
    assert p.seq_extend(a, 3).tolist() == [5, 6, 7]             # fills page 1, no new page
    assert p.block_table(a).tolist() == [0, 1] and p.frontier == 3
    assert p.seq_free(a) == 2 and p.pages_free == 7
    c = p.seq_create()
    # pushed in block-table order [0, 1] -> popped last-freed first: 1, then 0, then frontier
    assert p.seq_extend(c, 12).tolist() == [4, 5, 6, 7, 0, 1, 2, 3, 12, 13, 14, 15]
    assert p.block_table(c).tolist() == [1, 0, 3] and p.frontier == 4


def test_exhaustion_is_all_or_nothing():
    p = PagePool(2, 4)
    a = p.seq_create()
    p.seq_extend(a, 6)
    before = (p.pages_free, p.seq_len(a), p.block_table(a).tolist())
    with pytest.raises(PoolExhausted):
        p.seq_extend(a, 3)
    assert (p.pages_free, p.seq_len(a), p.block_table(a).tolist()) == before
    assert p.seq_extend(a, 2).tolist() == [6, 7]
    with pytest.raises(ValueError):
        p.seq_extend(99, 1)
    with pytest.raises(ValueError):
        p.seq_free(a) and p.seq_free(a)


def test_seeded_churn_matches_model_and_never_double_owns():
    rng = np.random.default_rng(0xC0FFEE)
    n_pages, pt = 256, 64
    pool, model = PagePool(n_pages, pt), ModelPool(n_pages, pt)
    live = {}
    for step in range(4000):
        if live and (rng.random() < 0.15 or pool.pages_free < 4):
            sid = list(live)[rng.integers(len(live))]
            assert pool.seq_free(sid) == model.free_seq(live.pop(sid))
        else:
            if not live or rng.random() < 0.2:
                sid = pool.seq_create()
                live[sid] = step            # model key is unique per incarnation
            sid = list(live)[rng.integers(len(live))]
            n = int(rng.integers(1, 200))
            try:
                want = model.extend(live[sid], n)
            except PoolExhausted:
                with pytest.raises(PoolExhausted):
                    pool.seq_extend(sid, n)
                continue
            assert pool.seq_extend(sid, n).tolist() == want
        if step % 97 == 0:
            owned = np.concatenate([pool.block_table(s) for s in live] or [np.zeros(0, np.int32)])
            assert len(set(owned.tolist())) == owned.size == pool.pages_owned
            assert pool.pages_owned + pool.pages_free == n_pages
            assert owned.size == 0 or owned.max() < pool.frontier <= n_pages
